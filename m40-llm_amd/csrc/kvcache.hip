// KV cache objects for gfx950: dense f16 cache and the fp16-K / q4-V compressed cache
// (recent ring + exact old backing), appends with fused RoPE-K, bulk fill, readers.
//
// Reference: layout cuda/kernels.cu:5304-5312; create :5387-5543; append family :5793-6306;
// compressed append/evict :6108-6250 with kernels :2230-2311 and ring write :5786-5790;
// reset :6308-6358; debug readers :6360-6379, :6449-6677.
//
// Only the storage the fp16-K/q4-V direct path reads is allocated for compressed caches
// (ring, old K, q4 V, scales, seq_map); the block-summary and representative side tables of
// the reference's lossy modes are not.
#include "common.hpp"

#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <new>
#include <vector>

namespace {

constexpr int kThreads = 256;

// Dense append: cast (and optionally rotate K) one token into [seq][position].
// position = *position_dev if given, else `position`, else (use_seq_map) seq_map[seq].
template <bool ROPE>
__global__ __launch_bounds__(kThreads) void dense_append_kernel(
    const float* __restrict__ k_in, const float* __restrict__ v_in, uint16_t* __restrict__ k_base,
    uint16_t* __restrict__ v_base, uint32_t* __restrict__ seq_map, uint32_t seq_id, uint32_t max_seq_len,
    uint32_t num_heads, uint32_t head_dim, uint32_t position, const uint32_t* __restrict__ position_dev,
    float freq_base, float freq_scale, uint32_t layout, uint32_t rope_position, uint32_t use_rope_position) {
    if (position_dev) position = *position_dev;
    if (position >= max_seq_len) return;
    const size_t ept = (size_t)num_heads * head_dim;
    uint16_t* k_out = k_base + ((size_t)seq_id * max_seq_len + position) * ept;
    uint16_t* v_out = v_base + ((size_t)seq_id * max_seq_len + position) * ept;
    const size_t idx = (size_t)blockIdx.x * kThreads + threadIdx.x;
    if (ROPE) {
        const size_t pairs = ept / 2u;
        if (idx >= pairs) return;
        const uint32_t half_dim = head_dim / 2u;
        const uint32_t off = (uint32_t)(idx % half_dim), head = (uint32_t)(idx / half_dim);
        size_t i0, i1;
        m40_rope_pair(head, off, head_dim, layout, &i0, &i1);
        float y0, y1;
        m40_rope_rotate(use_rope_position ? rope_position : position, off, head_dim, freq_base, freq_scale,
                        k_in[i0], k_in[i1], &y0, &y1);
        k_out[i0] = m40_f2h(y0);
        k_out[i1] = m40_f2h(y1);
        v_out[i0] = m40_f2h(v_in[i0]);
        v_out[i1] = m40_f2h(v_in[i1]);
    } else {
        if (idx >= ept) return;
        k_out[idx] = m40_f2h(k_in[idx]);
        v_out[idx] = m40_f2h(v_in[idx]);
    }
    if (idx == 0) seq_map[seq_id] = position + 1u;
}

__global__ __launch_bounds__(kThreads) void dense_append_f16_kernel(
    const uint16_t* __restrict__ k_in, const uint16_t* __restrict__ v_in, uint16_t* __restrict__ k_base,
    uint16_t* __restrict__ v_base, uint32_t* __restrict__ seq_map, uint32_t seq_id, uint32_t max_seq_len,
    size_t ept, uint32_t position) {
    const size_t idx = (size_t)blockIdx.x * kThreads + threadIdx.x;
    if (idx >= ept) return;
    k_base[((size_t)seq_id * max_seq_len + position) * ept + idx] = k_in[idx];
    v_base[((size_t)seq_id * max_seq_len + position) * ept + idx] = v_in[idx];
    if (idx == 0) seq_map[seq_id] = position + 1u;
}

// Prefill: RoPE of Q and K (in place, f32, for the attention that follows) and the cast of the rotated K and of V
// into the dense cache, for every row of a packed batch in one launch.  One workgroup per row; the row's sequence
// is found in the by-value table (at most kPrefillSeqs sequences).  Same rotation function and the same inverse
// frequencies as the per-token appends and the standalone RoPE, so the bits agree with the per-token call sequence
// (reference: src/infer/forward.rs:2349-2396, three launches per token and layer).
constexpr int kPrefillSeqs = 64;
struct PrefillSeqTable {
    uint32_t n;
    uint32_t slot[kPrefillSeqs], q_off[kPrefillSeqs], len[kPrefillSeqs], start[kPrefillSeqs];
};

__global__ __launch_bounds__(kThreads) void prefill_rope_append_kernel(
    float* __restrict__ q, float* __restrict__ k, float* __restrict__ v, uint16_t* __restrict__ k_base,
    uint16_t* __restrict__ v_base, uint32_t* __restrict__ seq_map, PrefillSeqTable t, uint32_t q_heads,
    uint32_t kv_heads, uint32_t head_dim, uint32_t max_seq_len, const float* __restrict__ inv_freq_table,
    float freq_base, float freq_scale, uint32_t layout, const float* __restrict__ bq, const float* __restrict__ bk,
    const float* __restrict__ bv) {
    const uint32_t row = blockIdx.x;
    uint32_t s = 0;
    for (uint32_t i = 1; i < t.n; ++i)
        if (row >= t.q_off[i]) s = i;
    const uint32_t local = row - t.q_off[s];
    const uint32_t position = t.start[s] + local;
    const uint32_t slot = t.slot[s];
    const uint32_t half_dim = head_dim / 2u;
    const uint32_t q_pairs = q_heads * half_dim, kv_pairs = kv_heads * half_dim;
    float* q_row = q + (size_t)row * q_heads * head_dim;
    float* k_row = k + (size_t)row * kv_heads * head_dim;
    float* v_row = v + (size_t)row * kv_heads * head_dim;
    const size_t ept = (size_t)kv_heads * head_dim;
    uint16_t* k_out = k_base + ((size_t)slot * max_seq_len + position) * ept;
    uint16_t* v_out = v_base + ((size_t)slot * max_seq_len + position) * ept;
    for (uint32_t idx = threadIdx.x; idx < q_pairs + kv_pairs; idx += kThreads) {
        const bool is_q = idx < q_pairs;
        const uint32_t p = is_q ? idx : idx - q_pairs;
        const uint32_t off = p % half_dim, head = p / half_dim;
        size_t i0, i1;
        m40_rope_pair(head, off, head_dim, layout, &i0, &i1);
        const float f = inv_freq_table ? inv_freq_table[off] : m40_rope_inv_freq(off, head_dim, freq_base);
        const float2 cs = m40_rope_cos_sin_freq(position, f, freq_scale);
        float* x = is_q ? q_row : k_row;
        const float* bias = is_q ? bq : bk;
        float x0 = x[i0], x1 = x[i1];
        if (bias) {   // the bias add of the per-row sequence (forward.rs:149-160), before the rotation
            x0 = x0 + bias[i0];
            x1 = x1 + bias[i1];
        }
        float y0, y1;
        m40_rope_apply(cs, x0, x1, &y0, &y1);
        x[i0] = y0;
        x[i1] = y1;
        if (!is_q) {
            float v0 = v_row[i0], v1 = v_row[i1];
            if (bv) {
                v0 = v0 + bv[i0];
                v1 = v1 + bv[i1];
                v_row[i0] = v0;
                v_row[i1] = v1;
            }
            k_out[i0] = m40_f2h(y0);
            k_out[i1] = m40_f2h(y1);
            v_out[i0] = m40_f2h(v0);
            v_out[i1] = m40_f2h(v1);
        }
    }
    if (threadIdx.x == 0 && local + 1u == t.len[s]) seq_map[slot] = position + 1u;
}

// Compressed append: one wave per kv head.  Phase 1 reads the ring row that is about to be
// overwritten into registers and, when position >= W, evicts it to old index position-W
// (K copied, V quantised to 4 bits with one f32 scale per token-head).  Phase 2, after a
// barrier, writes the rotated K and the cast V into the ring.
template <int HD, bool G32>
__global__ __launch_bounds__(64) void compressed_append_kernel(
    const float* __restrict__ k_in, const float* __restrict__ v_in, uint16_t* __restrict__ recent_k,
    uint16_t* __restrict__ recent_v, uint16_t* __restrict__ old_k, uint8_t* __restrict__ q4_v,
    float* __restrict__ q4_scale, uint32_t* __restrict__ seq_map, uint32_t seq_id, uint32_t max_seq_len,
    uint32_t recent_window, uint32_t num_heads, uint32_t position, float freq_base, float freq_scale,
    uint32_t layout, uint32_t evict) {
    constexpr int PAIRS = HD / 2;
    const uint32_t head = blockIdx.x, lane = threadIdx.x;
    const size_t ept = (size_t)num_heads * HD;
    const uint32_t ring = position % recent_window;
    const size_t ring_base = ((size_t)seq_id * recent_window + ring) * ept + (size_t)head * HD;
    const bool active = lane < PAIRS;
    const uint32_t d0 = 2u * lane;

    if (evict && position >= recent_window) {
        const uint32_t old_pos = position - recent_window;
        // the old store is head-major, [sequence][kv head][token][...]: the tokens of a block are one contiguous run
        const size_t old_row = ((size_t)seq_id * num_heads + head) * max_seq_len + old_pos;
        const size_t old_base = old_row * HD;
        float v0 = 0.0f, v1 = 0.0f;
        if (active) {
            old_k[old_base + d0] = recent_k[ring_base + d0];
            old_k[old_base + d0 + 1] = recent_k[ring_base + d0 + 1];
            v0 = m40_h2f(recent_v[ring_base + d0]);
            v1 = m40_h2f(recent_v[ring_base + d0 + 1]);
        }
        if (G32) {
            // groups of 32 dimensions = 16 lanes; lanes past the head (head_dim 64) form groups of their own, unused
            uint32_t dm;
            const uint8_t byte = m40_pack_q4g32_pair(v0, v1, &dm);
            if (active && (lane & 15u) == 0u)
                reinterpret_cast<uint32_t*>(q4_scale)[old_row * (HD / 32) + lane / 16u] = dm;
            if (active) q4_v[old_row * PAIRS + lane] = byte;
        } else {
            const float max_v = m40_max64(fmaxf(fabsf(v0), fabsf(v1)));
            const float scale = max_v > 0.0f ? max_v / 7.0f : 1.0f / 7.0f;
            if (lane == 0) q4_scale[old_row] = scale;
            if (active) q4_v[old_row * PAIRS + lane] = m40_pack_q4_pair(v0, v1, scale);
        }
    }
    __syncthreads();
    if (active) {
        size_t i0, i1;
        m40_rope_pair(0, lane, HD, layout, &i0, &i1);
        const float* kh = k_in + (size_t)head * HD;
        float y0, y1;
        m40_rope_rotate(position, lane, HD, freq_base, freq_scale, kh[i0], kh[i1], &y0, &y1);
        recent_k[ring_base + i0] = m40_f2h(y0);
        recent_k[ring_base + i1] = m40_f2h(y1);
        recent_v[ring_base + d0] = m40_f2h(v_in[(size_t)head * HD + d0]);
        recent_v[ring_base + d0 + 1] = m40_f2h(v_in[(size_t)head * HD + d0 + 1]);
    }
    if (head == 0 && lane == 0) seq_map[seq_id] = position + 1u;
}

// Bulk fill of a compressed cache from f16 rows: grid (token, kv head), one wave each.
template <int HD, bool G32>
__global__ __launch_bounds__(64) void compressed_bulk_fill_kernel(
    const uint16_t* __restrict__ k_rows, const uint16_t* __restrict__ v_rows, uint16_t* __restrict__ recent_k,
    uint16_t* __restrict__ recent_v, uint16_t* __restrict__ old_k, uint8_t* __restrict__ q4_v,
    float* __restrict__ q4_scale, uint32_t* __restrict__ seq_map, uint32_t seq_id, uint32_t max_seq_len,
    uint32_t recent_window, uint32_t num_heads, uint32_t seq_len, uint32_t has_old) {
    constexpr int PAIRS = HD / 2;
    const uint32_t t = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
    const size_t ept = (size_t)num_heads * HD;
    const uint32_t old_len = seq_len > recent_window ? seq_len - recent_window : 0;
    const bool active = lane < PAIRS;
    const uint32_t d0 = 2u * lane;
    const size_t src = (size_t)t * ept + (size_t)head * HD;
    if (t < old_len) {
        if (!has_old) return;
        const size_t old_row = ((size_t)seq_id * num_heads + head) * max_seq_len + t;
        const size_t old_base = old_row * HD;
        float v0 = 0.0f, v1 = 0.0f;
        if (active) {
            old_k[old_base + d0] = k_rows[src + d0];
            old_k[old_base + d0 + 1] = k_rows[src + d0 + 1];
            v0 = m40_h2f(v_rows[src + d0]);
            v1 = m40_h2f(v_rows[src + d0 + 1]);
        }
        if (G32) {
            // groups of 32 dimensions = 16 lanes; lanes past the head (head_dim 64) form groups of their own, unused
            uint32_t dm;
            const uint8_t byte = m40_pack_q4g32_pair(v0, v1, &dm);
            if (active && (lane & 15u) == 0u)
                reinterpret_cast<uint32_t*>(q4_scale)[old_row * (HD / 32) + lane / 16u] = dm;
            if (active) q4_v[old_row * PAIRS + lane] = byte;
        } else {
            const float max_v = m40_max64(fmaxf(fabsf(v0), fabsf(v1)));
            const float scale = max_v > 0.0f ? max_v / 7.0f : 1.0f / 7.0f;
            if (lane == 0) q4_scale[old_row] = scale;
            if (active) q4_v[old_row * PAIRS + lane] = m40_pack_q4_pair(v0, v1, scale);
        }
    } else {
        const size_t ring_base = ((size_t)seq_id * recent_window + (t % recent_window)) * ept + (size_t)head * HD;
        if (active) {
            recent_k[ring_base + d0] = k_rows[src + d0];
            recent_k[ring_base + d0 + 1] = k_rows[src + d0 + 1];
            recent_v[ring_base + d0] = v_rows[src + d0];
            recent_v[ring_base + d0 + 1] = v_rows[src + d0 + 1];
        }
    }
    if (t == 0 && head == 0 && lane == 0) seq_map[seq_id] = seq_len;
}

__global__ void set_u32_kernel(uint32_t* p, uint32_t idx, uint32_t value) {
    if (threadIdx.x == 0 && blockIdx.x == 0) p[idx] = value;
}

size_t kv_elems(const M40llmKVCache* kv) {
    return (size_t)kv->max_seq_len * kv->max_batch_size * kv->num_heads * kv->head_dim;
}

float host_h2f(uint16_t h) {
    const uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu, mant = h & 0x3ffu, u;
    if (exp == 0) {
        if (mant == 0) u = sign;
        else {
            int e = -1;
            do { mant <<= 1; e++; } while (!(mant & 0x400u));
            mant &= 0x3ffu;
            u = sign | ((uint32_t)(127 - 15 - e) << 23) | (mant << 13);
        }
    } else if (exp == 31) u = sign | 0x7f800000u | (mant << 13);
    else u = sign | ((exp + 127 - 15) << 23) | (mant << 13);
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}

uint32_t selected_block_order_from_env() {
    const char* v = std::getenv("M40LLM_KV_SELECTED_BLOCK_ORDER");
    if (!v || !v[0]) return 0;
    if (std::strcmp(v, "chronological") == 0) return 1u;
    if (std::strcmp(v, "descending") == 0) return 2u;
    return 0u;
}

}  // namespace

extern "C" {

M40llmKVCache* m40llm_kvcache_create(M40llmCudaContext* ctx, uint32_t max_seq_len, uint32_t max_batch_size,
                                     uint32_t num_heads, uint32_t head_dim) {
    if (!ctx) return nullptr;
    if (m40_ensure_device(ctx) != 0) return nullptr;
    M40llmKVCache* kv = new (std::nothrow) M40llmKVCache();
    if (!kv) return nullptr;
    std::memset(kv, 0, sizeof(*kv));
    kv->max_seq_len = max_seq_len;
    kv->max_batch_size = max_batch_size;
    kv->num_heads = num_heads;
    kv->head_dim = head_dim;
    kv->device_id = ctx->device_id;
    const size_t bytes = kv_elems(kv) * sizeof(uint16_t);
    const size_t seq_map_size = (size_t)max_batch_size * sizeof(uint32_t);
    if (hipMalloc(reinterpret_cast<void**>(&kv->d_k), bytes ? bytes : 2) != hipSuccess ||
        hipMalloc(reinterpret_cast<void**>(&kv->d_v), bytes ? bytes : 2) != hipSuccess ||
        hipMalloc(reinterpret_cast<void**>(&kv->d_seq_map), seq_map_size ? seq_map_size : 4) != hipSuccess) {
        (void)hipGetLastError();
        m40llm_kvcache_destroy(kv);
        return nullptr;
    }
    (void)hipMemset(kv->d_k, 0, bytes);
    (void)hipMemset(kv->d_v, 0, bytes);
    (void)hipMemset(kv->d_seq_map, 0, seq_map_size);
    (void)hipDeviceSynchronize();
    return kv;
}

M40llmKVCache* m40llm_kvcache_create_compressed(M40llmCudaContext* ctx, uint32_t max_seq_len,
                                                uint32_t max_batch_size, uint32_t num_heads, uint32_t head_dim,
                                                uint32_t recent_window, uint32_t block_size, uint32_t top_blocks,
                                                uint32_t representatives, uint32_t representative_policy,
                                                uint32_t exact_old_backing) {
    if (!ctx || recent_window == 0 || block_size == 0) return nullptr;
    if (m40_ensure_device(ctx) != 0) return nullptr;
    if (exact_old_backing == 1u || exact_old_backing > 3u) return nullptr;  // q8 backing is not part of this build
    // backing 3 (no counterpart in the reference): backing 2 with old V in groups of 32 under an f16 scale and minimum
    const bool old_store = exact_old_backing == 2u || exact_old_backing == 3u;
    if (old_store && head_dim != 64 && head_dim != 128) return nullptr;  // kernels.cu:5371
    M40llmKVCache* kv = new (std::nothrow) M40llmKVCache();
    if (!kv) return nullptr;
    std::memset(kv, 0, sizeof(*kv));
    kv->max_seq_len = max_seq_len;
    kv->max_batch_size = max_batch_size;
    kv->num_heads = num_heads;
    kv->head_dim = head_dim;
    kv->compressed = 1;
    kv->recent_window = recent_window;
    kv->block_size = block_size;
    kv->top_blocks = top_blocks;
    kv->representatives = representatives;
    kv->representative_policy = representative_policy;
    kv->device_id = ctx->device_id;
    const uint32_t old_capacity = max_seq_len > recent_window ? max_seq_len - recent_window : 0;
    kv->max_blocks = old_capacity == 0 ? 1 : (old_capacity + block_size - 1) / block_size;

    const size_t ept = (size_t)num_heads * head_dim;
    const size_t recent_bytes = (size_t)max_batch_size * recent_window * ept * sizeof(uint16_t);
    const size_t seq_map_size = (size_t)max_batch_size * sizeof(uint32_t);
    bool ok = hipMalloc(reinterpret_cast<void**>(&kv->d_recent_k), recent_bytes ? recent_bytes : 2) == hipSuccess &&
              hipMalloc(reinterpret_cast<void**>(&kv->d_recent_v), recent_bytes ? recent_bytes : 2) == hipSuccess &&
              hipMalloc(reinterpret_cast<void**>(&kv->d_seq_map), seq_map_size ? seq_map_size : 4) == hipSuccess;
    if (ok) {
        (void)hipMemset(kv->d_recent_k, 0, recent_bytes);
        (void)hipMemset(kv->d_recent_v, 0, recent_bytes);
        (void)hipMemset(kv->d_seq_map, 0, seq_map_size);
    }
    if (ok && old_store) {
        // kM40OldStoreSlackRows zeroed rows behind each array (see M40llmKVCache)
        const size_t old_k_bytes = (kv_elems(kv) + (size_t)kM40OldStoreSlackRows * head_dim) * sizeof(uint16_t);
        const size_t q4_bytes = ((size_t)max_seq_len * max_batch_size * num_heads + kM40OldStoreSlackRows) * (head_dim / 2u);
        const size_t scale_bytes = ((size_t)max_seq_len * max_batch_size * num_heads + kM40OldStoreSlackRows) *
                                   (exact_old_backing == 3u ? (head_dim / 32u) * sizeof(uint32_t) : sizeof(float));
        ok = hipMalloc(reinterpret_cast<void**>(&kv->d_fp16_old_k), old_k_bytes ? old_k_bytes : 2) == hipSuccess &&
             hipMalloc(reinterpret_cast<void**>(&kv->d_q4_old_v), q4_bytes ? q4_bytes : 1) == hipSuccess &&
             hipMalloc(reinterpret_cast<void**>(&kv->d_q4_old_v_scale), scale_bytes ? scale_bytes : 4) == hipSuccess;
        if (ok) {
            (void)hipMemset(kv->d_fp16_old_k, 0, old_k_bytes);
            (void)hipMemset(kv->d_q4_old_v, 0, q4_bytes);
            (void)hipMemset(kv->d_q4_old_v_scale, 0, scale_bytes);
            kv->fp16_k_q4_v_old_backing = 1;
            kv->v_format = exact_old_backing == 3u ? 1u : 0u;
        }
    }
    if (!ok) {
        (void)hipGetLastError();
        m40llm_kvcache_destroy(kv);
        return nullptr;
    }
    (void)hipDeviceSynchronize();
    return kv;
}

void m40llm_kvcache_destroy(M40llmKVCache* kv) {
    if (!kv) return;
    (void)hipSetDevice(kv->device_id);
    void* ptrs[] = {kv->d_k, kv->d_v, kv->d_seq_map, kv->d_recent_k, kv->d_recent_v,
                    kv->d_fp16_old_k, kv->d_q4_old_v, kv->d_q4_old_v_scale};
    for (void* p : ptrs)
        if (p) (void)hipFree(p);
    delete kv;
}

int m40llm_kvcache_reset(M40llmCudaContext* ctx, M40llmKVCache* kv) {
    if (!ctx || !kv) return -1;
    if (m40_ensure_device(ctx) != 0) return -2;
    hipStream_t s = ctx->decode_stream;
    if (hipMemsetAsync(kv->d_seq_map, 0, (size_t)kv->max_batch_size * sizeof(uint32_t), s) != hipSuccess) return -3;
    if (kv->compressed) {
        const size_t ept = (size_t)kv->num_heads * kv->head_dim;
        const size_t recent_bytes = (size_t)kv->max_batch_size * kv->recent_window * ept * sizeof(uint16_t);
        (void)hipMemsetAsync(kv->d_recent_k, 0, recent_bytes, s);
        (void)hipMemsetAsync(kv->d_recent_v, 0, recent_bytes, s);
        if (kv->d_fp16_old_k) (void)hipMemsetAsync(kv->d_fp16_old_k, 0, kv_elems(kv) * sizeof(uint16_t), s);
        if (kv->d_q4_old_v)
            (void)hipMemsetAsync(kv->d_q4_old_v, 0,
                                 (size_t)kv->max_seq_len * kv->max_batch_size * kv->num_heads * (kv->head_dim / 2u), s);
        if (kv->d_q4_old_v_scale)
            (void)hipMemsetAsync(kv->d_q4_old_v_scale, 0,
                                 (size_t)kv->max_seq_len * kv->max_batch_size * kv->num_heads *
                                     (kv->v_format ? (kv->head_dim / 32u) * sizeof(uint32_t) : sizeof(float)), s);
    }
    return hipStreamSynchronize(s) == hipSuccess ? 0 : -4;
}

// Current length of a sequence as the device sees it after everything already enqueued on the
// decode stream (the reference reads seq_map with a blocking copy, kernels.cu:5846).
static int read_cur_len(M40llmCudaContext* ctx, M40llmKVCache* kv, uint32_t seq_id, uint32_t* out) {
    if (hipStreamSynchronize(ctx->decode_stream) != hipSuccess) return -1;
    if (hipMemcpy(out, kv->d_seq_map + seq_id, sizeof(uint32_t), hipMemcpyDeviceToHost) != hipSuccess) return -1;
    return 0;
}

int m40llm_kvcache_append_token(M40llmCudaContext* ctx, M40llmKVCache* kv, uint32_t seq_id,
                                const void* k_dev_f16, const void* v_dev_f16) {
    if (!ctx || !kv || !k_dev_f16 || !v_dev_f16) return -1;
    if (seq_id >= kv->max_batch_size) return -2;
    if (!kv->d_k || !kv->d_v) return -5;
    uint32_t cur_len = 0;
    if (read_cur_len(ctx, kv, seq_id, &cur_len) != 0) return -3;
    if (cur_len >= kv->max_seq_len) return -4;
    const size_t ept = (size_t)kv->num_heads * kv->head_dim;
    (void)hipGetLastError();
    dense_append_f16_kernel<<<(unsigned)((ept + kThreads - 1) / kThreads), kThreads, 0, ctx->decode_stream>>>(
        static_cast<const uint16_t*>(k_dev_f16), static_cast<const uint16_t*>(v_dev_f16), kv->d_k, kv->d_v,
        kv->d_seq_map, seq_id, kv->max_seq_len, ept, cur_len);
    if (hipGetLastError() != hipSuccess) return -5;
    return hipStreamSynchronize(ctx->decode_stream) == hipSuccess ? 0 : -7;
}

int m40llm_kvcache_append_token_f32_async(M40llmCudaContext* ctx, M40llmKVCache* kv, uint32_t seq_id,
                                          const void* k_dev_f32, const void* v_dev_f32) {
    if (!ctx || !kv || !k_dev_f32 || !v_dev_f32) return -1;
    if (seq_id >= kv->max_batch_size) return -2;
    if (!kv->d_k || !kv->d_v) return -5;
    uint32_t cur_len = 0;
    if (read_cur_len(ctx, kv, seq_id, &cur_len) != 0) return -3;
    if (cur_len >= kv->max_seq_len) return -4;
    const size_t ept = (size_t)kv->num_heads * kv->head_dim;
    if (ept == 0) return 0;
    (void)hipGetLastError();
    dense_append_kernel<false><<<(unsigned)((ept + kThreads - 1) / kThreads), kThreads, 0, ctx->decode_stream>>>(
        static_cast<const float*>(k_dev_f32), static_cast<const float*>(v_dev_f32), kv->d_k, kv->d_v,
        kv->d_seq_map, seq_id, kv->max_seq_len, kv->num_heads, kv->head_dim, cur_len, nullptr, 0.f, 0.f, 0, 0, 0);
    return hipGetLastError() == hipSuccess ? 0 : -5;
}

int m40llm_kvcache_append_token_f32(M40llmCudaContext* ctx, M40llmKVCache* kv, uint32_t seq_id,
                                    const void* k_dev_f32, const void* v_dev_f32) {
    int rc = m40llm_kvcache_append_token_f32_async(ctx, kv, seq_id, k_dev_f32, v_dev_f32);
    if (rc != 0) return rc;
    return hipStreamSynchronize(ctx->decode_stream) == hipSuccess ? 0 : -7;
}

int m40llm_kvcache_append_token_f32_rope_k_layout_async(M40llmCudaContext* ctx, M40llmKVCache* kv,
                                                        uint32_t seq_id, const void* k_dev_f32,
                                                        const void* v_dev_f32, uint32_t past_len,
                                                        float freq_base, float freq_scale, uint32_t rope_layout) {
    if (!ctx || !kv || !k_dev_f32 || !v_dev_f32) return -1;
    if (seq_id >= kv->max_batch_size) return -2;
    if (kv->head_dim == 0 || kv->num_heads == 0) return -3;
    if (kv->head_dim % 2 != 0) return -4;
    if (!kv->d_k || !kv->d_v) return -7;
    uint32_t cur_len = 0;
    if (read_cur_len(ctx, kv, seq_id, &cur_len) != 0) return -5;
    if (cur_len >= kv->max_seq_len) return -6;
    const size_t pairs = (size_t)kv->num_heads * kv->head_dim / 2u;
    (void)hipGetLastError();
    // stored at the cache's current length, rotated for position past_len (kernels.cu:5996-6017)
    dense_append_kernel<true><<<(unsigned)((pairs + kThreads - 1) / kThreads), kThreads, 0, ctx->decode_stream>>>(
        static_cast<const float*>(k_dev_f32), static_cast<const float*>(v_dev_f32), kv->d_k, kv->d_v,
        kv->d_seq_map, seq_id, kv->max_seq_len, kv->num_heads, kv->head_dim, cur_len, nullptr, freq_base,
        freq_scale, rope_layout, past_len, 1);
    return hipGetLastError() == hipSuccess ? 0 : -7;
}

int m40llm_kvcache_append_token_f32_rope_k_async(M40llmCudaContext* ctx, M40llmKVCache* kv, uint32_t seq_id,
                                                 const void* k_dev_f32, const void* v_dev_f32,
                                                 uint32_t past_len, float freq_base, float freq_scale) {
    return m40llm_kvcache_append_token_f32_rope_k_layout_async(ctx, kv, seq_id, k_dev_f32, v_dev_f32, past_len,
                                                               freq_base, freq_scale, M40LLM_ROPE_LAYOUT_ADJACENT);
}

int m40llm_kvcache_append_token_f32_rope_k(M40llmCudaContext* ctx, M40llmKVCache* kv, uint32_t seq_id,
                                           const void* k_dev_f32, const void* v_dev_f32, uint32_t past_len,
                                           float freq_base, float freq_scale) {
    int rc = m40llm_kvcache_append_token_f32_rope_k_async(ctx, kv, seq_id, k_dev_f32, v_dev_f32, past_len,
                                                          freq_base, freq_scale);
    if (rc != 0) return rc;
    return hipStreamSynchronize(ctx->decode_stream) == hipSuccess ? 0 : -7;
}

int m40llm_kvcache_append_token_f32_rope_k_compressed_at_layout_async(
    M40llmCudaContext* ctx, M40llmKVCache* kv, uint32_t seq_id, const void* k_dev_f32, const void* v_dev_f32,
    uint32_t position, float freq_base, float freq_scale, uint32_t rope_layout) {
    if (!ctx || !kv || !k_dev_f32 || !v_dev_f32) return -1;
    if (!kv->compressed) return -2;
    if (seq_id >= kv->max_batch_size) return -3;
    if ((kv->head_dim != 64 && kv->head_dim != 128) || kv->num_heads == 0 || kv->recent_window == 0 ||
        kv->block_size == 0)
        return -4;
    if (position >= kv->max_seq_len) return -5;
    (void)hipGetLastError();
    const uint32_t evict = kv->fp16_k_q4_v_old_backing ? 1u : 0u;
    auto launch = [&](auto kernel) {
        kernel<<<kv->num_heads, 64, 0, ctx->decode_stream>>>(
            static_cast<const float*>(k_dev_f32), static_cast<const float*>(v_dev_f32), kv->d_recent_k,
            kv->d_recent_v, kv->d_fp16_old_k, kv->d_q4_old_v, kv->d_q4_old_v_scale, kv->d_seq_map, seq_id,
            kv->max_seq_len, kv->recent_window, kv->num_heads, position, freq_base, freq_scale, rope_layout, evict);
    };
    if (kv->head_dim == 64) {
        if (kv->v_format) launch(compressed_append_kernel<64, true>); else launch(compressed_append_kernel<64, false>);
    } else {
        if (kv->v_format) launch(compressed_append_kernel<128, true>); else launch(compressed_append_kernel<128, false>);
    }
    return hipGetLastError() == hipSuccess ? 0 : -6;
}

int m40llm_kvcache_append_token_f32_rope_k_compressed_at_async(M40llmCudaContext* ctx, M40llmKVCache* kv,
                                                               uint32_t seq_id, const void* k_dev_f32,
                                                               const void* v_dev_f32, uint32_t position,
                                                               float freq_base, float freq_scale) {
    return m40llm_kvcache_append_token_f32_rope_k_compressed_at_layout_async(
        ctx, kv, seq_id, k_dev_f32, v_dev_f32, position, freq_base, freq_scale, M40LLM_ROPE_LAYOUT_ADJACENT);
}

int m40llm_kvcache_append_token_f32_rope_k_at_layout_async(M40llmCudaContext* ctx, M40llmKVCache* kv,
                                                           uint32_t seq_id, const void* k_dev_f32,
                                                           const void* v_dev_f32, uint32_t position,
                                                           uint32_t past_len, float freq_base, float freq_scale,
                                                           uint32_t rope_layout) {
    if (!ctx || !kv || !k_dev_f32 || !v_dev_f32) return -1;
    if (kv->compressed) {
        return m40llm_kvcache_append_token_f32_rope_k_compressed_at_layout_async(
            ctx, kv, seq_id, k_dev_f32, v_dev_f32, position, freq_base, freq_scale, rope_layout);
    }
    if (seq_id >= kv->max_batch_size) return -2;
    if (kv->head_dim == 0 || kv->num_heads == 0) return -3;
    if (kv->head_dim % 2 != 0) return -4;
    if (position >= kv->max_seq_len) return -5;
    (void)past_len;  // ignored by the reference as well (kernels.cu:6064)
    const size_t pairs = (size_t)kv->num_heads * kv->head_dim / 2u;
    (void)hipGetLastError();
    dense_append_kernel<true><<<(unsigned)((pairs + kThreads - 1) / kThreads), kThreads, 0, ctx->decode_stream>>>(
        static_cast<const float*>(k_dev_f32), static_cast<const float*>(v_dev_f32), kv->d_k, kv->d_v,
        kv->d_seq_map, seq_id, kv->max_seq_len, kv->num_heads, kv->head_dim, position, nullptr, freq_base,
        freq_scale, rope_layout, 0, 0);
    return hipGetLastError() == hipSuccess ? 0 : -6;
}

int m40llm_ext_prefill_rope_append_async(M40llmCudaContext* ctx, M40llmKVCache* kv, void* d_q_f32, void* d_k_f32,
                                         void* d_v_f32, uint32_t batch, const uint32_t* seq_slots_host,
                                         const uint32_t* q_lens_host, const uint32_t* start_pos_host, uint32_t q_heads,
                                         float freq_base, float freq_scale, uint32_t rope_layout, const void* d_bq_f32,
                                         const void* d_bk_f32, const void* d_bv_f32) {
    return m40llm_ext_prefill_rope_append_on_stream_async(ctx, kv, d_q_f32, d_k_f32, d_v_f32, batch, seq_slots_host, q_lens_host,
                                                          start_pos_host, q_heads, freq_base, freq_scale, rope_layout, d_bq_f32,
                                                          d_bk_f32, d_bv_f32, M40LLM_STREAM_DECODE);
}

int m40llm_ext_prefill_rope_append_on_stream_async(M40llmCudaContext* ctx, M40llmKVCache* kv, void* d_q_f32, void* d_k_f32,
                                                   void* d_v_f32, uint32_t batch, const uint32_t* seq_slots_host,
                                                   const uint32_t* q_lens_host, const uint32_t* start_pos_host,
                                                   uint32_t q_heads, float freq_base, float freq_scale, uint32_t rope_layout,
                                                   const void* d_bq_f32, const void* d_bk_f32, const void* d_bv_f32,
                                                   uint32_t stream_kind) {
    if (!ctx || !kv || !d_q_f32 || !d_k_f32 || !d_v_f32 || !seq_slots_host || !q_lens_host) return -1;
    if (stream_kind > 1u) return -2;
    const int n_bias = (d_bq_f32 != nullptr) + (d_bk_f32 != nullptr) + (d_bv_f32 != nullptr);
    if (n_bias != 0 && n_bias != 3) return -2;
    if (kv->compressed || !kv->d_k || !kv->d_v) return -9;
    if (batch == 0 || batch > (uint32_t)kPrefillSeqs || q_heads == 0) return -2;
    if (kv->head_dim == 0 || kv->num_heads == 0) return -3;
    if (kv->head_dim % 2 != 0) return -4;
    if (rope_layout > M40LLM_ROPE_LAYOUT_NEOX) return -2;
    PrefillSeqTable t{};
    t.n = batch;
    uint64_t rows = 0;
    for (uint32_t i = 0; i < batch; ++i) {
        const uint32_t start = start_pos_host ? start_pos_host[i] : 0u;
        if (seq_slots_host[i] >= kv->max_batch_size) return -2;
        if (q_lens_host[i] == 0) return -7;
        if ((uint64_t)start + q_lens_host[i] > kv->max_seq_len) return -5;
        for (uint32_t j = 0; j < i; ++j)
            if (seq_slots_host[j] == seq_slots_host[i]) return -8;   // two sequences of one call would race on a slot
        t.slot[i] = seq_slots_host[i];
        t.q_off[i] = (uint32_t)rows;
        t.len[i] = q_lens_host[i];
        t.start[i] = start;
        rows += q_lens_host[i];
        if (rows > 0x7fffffffull) return -2;
    }
    hipStream_t stream = stream_kind == M40LLM_STREAM_PREFILL ? ctx->prefill_stream : ctx->decode_stream;
    const float* table = m40_rope_inv_freq_table(ctx, stream_kind, stream, kv->head_dim, freq_base);
    (void)hipGetLastError();
    prefill_rope_append_kernel<<<(unsigned)rows, kThreads, 0, stream>>>(
        static_cast<float*>(d_q_f32), static_cast<float*>(d_k_f32), static_cast<float*>(d_v_f32), kv->d_k, kv->d_v,
        kv->d_seq_map, t, q_heads, kv->num_heads, kv->head_dim, kv->max_seq_len, table, freq_base, freq_scale, rope_layout,
        static_cast<const float*>(d_bq_f32), static_cast<const float*>(d_bk_f32), static_cast<const float*>(d_bv_f32));
    return hipGetLastError() == hipSuccess ? 0 : -6;
}

int m40llm_kvcache_append_token_f32_rope_k_at_async(M40llmCudaContext* ctx, M40llmKVCache* kv, uint32_t seq_id,
                                                    const void* k_dev_f32, const void* v_dev_f32,
                                                    uint32_t position, uint32_t past_len, float freq_base,
                                                    float freq_scale) {
    return m40llm_kvcache_append_token_f32_rope_k_at_layout_async(ctx, kv, seq_id, k_dev_f32, v_dev_f32, position,
                                                                  past_len, freq_base, freq_scale,
                                                                  M40LLM_ROPE_LAYOUT_ADJACENT);
}

int m40llm_kvcache_append_token_f32_rope_k_position_dev_layout_async(
    M40llmCudaContext* ctx, M40llmKVCache* kv, uint32_t seq_id, const void* k_dev_f32, const void* v_dev_f32,
    const uint32_t* position_dev, float freq_base, float freq_scale, uint32_t rope_layout) {
    if (!ctx || !kv || !k_dev_f32 || !v_dev_f32 || !position_dev) return -1;
    if (seq_id >= kv->max_batch_size) return -2;
    if (kv->head_dim == 0 || kv->num_heads == 0) return -3;
    if (kv->head_dim % 2 != 0) return -4;
    if (!kv->d_k || !kv->d_v) return -5;
    const size_t pairs = (size_t)kv->num_heads * kv->head_dim / 2u;
    (void)hipGetLastError();
    dense_append_kernel<true><<<(unsigned)((pairs + kThreads - 1) / kThreads), kThreads, 0, ctx->decode_stream>>>(
        static_cast<const float*>(k_dev_f32), static_cast<const float*>(v_dev_f32), kv->d_k, kv->d_v,
        kv->d_seq_map, seq_id, kv->max_seq_len, kv->num_heads, kv->head_dim, 0, position_dev, freq_base,
        freq_scale, rope_layout, 0, 0);
    return hipGetLastError() == hipSuccess ? 0 : -5;
}

int m40llm_kvcache_append_token_f32_rope_k_position_dev_async(M40llmCudaContext* ctx, M40llmKVCache* kv,
                                                              uint32_t seq_id, const void* k_dev_f32,
                                                              const void* v_dev_f32, const uint32_t* position_dev,
                                                              float freq_base, float freq_scale) {
    return m40llm_kvcache_append_token_f32_rope_k_position_dev_layout_async(
        ctx, kv, seq_id, k_dev_f32, v_dev_f32, position_dev, freq_base, freq_scale, M40LLM_ROPE_LAYOUT_ADJACENT);
}

int m40llm_kvcache_debug_read_token(M40llmCudaContext* ctx, M40llmKVCache* kv, uint32_t seq_id, uint32_t token,
                                    void* out_k_host, void* out_v_host) {
    (void)ctx;
    if (!kv || !out_k_host || !out_v_host) return -1;
    if (seq_id >= kv->max_batch_size) return -2;
    if (token >= kv->max_seq_len) return -3;
    if (!kv->d_k || !kv->d_v) return -4;
    const size_t ept = (size_t)kv->num_heads * kv->head_dim;
    const size_t off = ((size_t)seq_id * kv->max_seq_len + token) * ept;
    if (hipMemcpy(out_k_host, kv->d_k + off, ept * 2, hipMemcpyDeviceToHost) != hipSuccess) return -4;
    if (hipMemcpy(out_v_host, kv->d_v + off, ept * 2, hipMemcpyDeviceToHost) != hipSuccess) return -5;
    return 0;
}

int m40llm_ext_kvcache_debug_read_raw(M40llmCudaContext* ctx, const M40llmKVCache* kv, uint32_t which,
                                      size_t offset, size_t bytes, void* out_host) {
    if (!ctx || !kv || !out_host) return -1;
    const void* src = nullptr;
    size_t total = 0, item = 0;     // item: bytes of one (token, kv head) entry of a head-major array, else 0
    const size_t ept = (size_t)kv->num_heads * kv->head_dim;
    switch (which) {
        case 0: src = kv->d_fp16_old_k; total = kv_elems(kv) * 2; item = (size_t)kv->head_dim * 2; break;
        case 1: src = kv->d_q4_old_v; total = (size_t)kv->max_seq_len * kv->max_batch_size * kv->num_heads * (kv->head_dim / 2u); item = kv->head_dim / 2u; break;
        case 2:      // f32 scale per (token, kv head); with groups of 32: head_dim / 32 words of scale | min << 16
            item = kv->v_format ? (size_t)(kv->head_dim / 32u) * 4 : 4;
            src = kv->d_q4_old_v_scale; total = (size_t)kv->max_seq_len * kv->max_batch_size * kv->num_heads * item; break;
        case 3: src = kv->d_recent_k; total = (size_t)kv->max_batch_size * kv->recent_window * ept * 2; break;
        case 4: src = kv->d_recent_v; total = (size_t)kv->max_batch_size * kv->recent_window * ept * 2; break;
        case 5: src = kv->d_seq_map; total = (size_t)kv->max_batch_size * 4; break;
        default: return -2;
    }
    if (!src) return -3;
    if (offset > total || bytes > total - offset) return -4;
    if (hipStreamSynchronize(ctx->decode_stream) != hipSuccess) return -5;
    if (item == 0) {
        if (hipMemcpy(out_host, static_cast<const char*>(src) + offset, bytes, hipMemcpyDeviceToHost) != hipSuccess) return -5;
        return 0;
    }
    // The old store lives head-major on the device ([sequence][kv head][token][...]); the answer is given in the
    // reference's order, [sequence][token][kv head][...] (cuda/kernels.cu:5435-5543), whatever the device layout.
    // Only the (sequence, kv head) token runs that meet [offset, offset + bytes) are copied: one contiguous device
    // run per sequence and head into a staging buffer of at most one head's tokens, then item by item into place.
    if (bytes == 0) return 0;
    const size_t S = kv->max_seq_len, H = kv->num_heads;
    const size_t row0 = offset / item / H, row1 = (offset + bytes - 1) / item / H;      // token rows b * S + t
    char* out = static_cast<char*>(out_host);
    try {
        std::vector<char> run;
        for (size_t b = row0 / S; b <= row1 / S; ++b) {
            const size_t t_lo = b == row0 / S ? row0 % S : 0, t_hi = b == row1 / S ? row1 % S : S - 1;
            run.resize((t_hi - t_lo + 1) * item);
            for (size_t h = 0; h < H; ++h) {
                if (hipMemcpy(run.data(), static_cast<const char*>(src) + ((b * H + h) * S + t_lo) * item, run.size(),
                              hipMemcpyDeviceToHost) != hipSuccess)
                    return -5;
                for (size_t t = t_lo; t <= t_hi; ++t) {
                    const size_t at = ((b * S + t) * H + h) * item;                     // in the reference's order
                    const size_t lo = at > offset ? at : offset, hi = at + item < offset + bytes ? at + item : offset + bytes;
                    if (lo < hi) std::memcpy(out + (lo - offset), run.data() + (t - t_lo) * item + (lo - at), hi - lo);
                }
            }
        }
    } catch (const std::bad_alloc&) {
        return -6;
    }
    return 0;
}

int m40llm_ext_kvcache_bulk_fill_f16(M40llmCudaContext* ctx, M40llmKVCache* kv, uint32_t seq_id,
                                     const void* k_dev_f16, const void* v_dev_f16, uint32_t seq_len) {
    if (!ctx || !kv || !k_dev_f16 || !v_dev_f16) return -1;
    if (seq_id >= kv->max_batch_size) return -2;
    if (seq_len == 0 || seq_len > kv->max_seq_len) return -3;
    hipStream_t s = ctx->decode_stream;
    const size_t ept = (size_t)kv->num_heads * kv->head_dim;
    (void)hipGetLastError();
    if (!kv->compressed) {
        const size_t off = (size_t)seq_id * kv->max_seq_len * ept;
        if (hipMemcpyAsync(kv->d_k + off, k_dev_f16, (size_t)seq_len * ept * 2, hipMemcpyDeviceToDevice, s) != hipSuccess ||
            hipMemcpyAsync(kv->d_v + off, v_dev_f16, (size_t)seq_len * ept * 2, hipMemcpyDeviceToDevice, s) != hipSuccess)
            return -4;
        set_u32_kernel<<<1, 64, 0, s>>>(kv->d_seq_map, seq_id, seq_len);
    } else {
        if (kv->head_dim != 64 && kv->head_dim != 128) return -5;
        dim3 grid(seq_len, kv->num_heads);
        const uint32_t has_old = kv->fp16_k_q4_v_old_backing ? 1u : 0u;
        auto launch = [&](auto kernel) {
            kernel<<<grid, 64, 0, s>>>(
                static_cast<const uint16_t*>(k_dev_f16), static_cast<const uint16_t*>(v_dev_f16), kv->d_recent_k,
                kv->d_recent_v, kv->d_fp16_old_k, kv->d_q4_old_v, kv->d_q4_old_v_scale, kv->d_seq_map, seq_id,
                kv->max_seq_len, kv->recent_window, kv->num_heads, seq_len, has_old);
        };
        if (kv->head_dim == 64) {
            if (kv->v_format) launch(compressed_bulk_fill_kernel<64, true>); else launch(compressed_bulk_fill_kernel<64, false>);
        } else {
            if (kv->v_format) launch(compressed_bulk_fill_kernel<128, true>); else launch(compressed_bulk_fill_kernel<128, false>);
        }
    }
    if (hipGetLastError() != hipSuccess) return -6;
    return hipStreamSynchronize(s) == hipSuccess ? 0 : -7;
}

// Telemetry twin of the block ranking (host side, q-head 0 against kv-head 0 only, plain top-k
// policy).  Mirrors cuda/kernels.cu:6449-6677 for the fp16 old-K backing and the dense cache.
int m40llm_kvcache_debug_select_old_blocks(M40llmCudaContext* ctx, const M40llmKVCache* kv, uint32_t seq_id,
                                           const void* q_dev_f32, uint32_t q_heads, uint32_t seq_len,
                                           uint32_t recent_window, uint32_t block_size, uint32_t top_blocks,
                                           uint32_t* out_blocks_host, float* out_scores_host,
                                           uint32_t* out_start_host, uint32_t* out_end_host, uint32_t* out_count,
                                           uint32_t max_out, uint32_t* out_total_old_blocks) {
    if (!ctx || !kv || !q_dev_f32 || !out_blocks_host || !out_scores_host || !out_start_host || !out_end_host ||
        !out_count || !out_total_old_blocks)
        return -1;
    if (seq_id >= kv->max_batch_size) return -2;
    if (q_heads == 0 || kv->num_heads == 0 || kv->head_dim == 0) return -3;
    if (seq_len == 0 || seq_len > kv->max_seq_len || block_size == 0 || max_out == 0) return -4;
    const uint32_t eff_recent = kv->compressed ? kv->recent_window : recent_window;
    const uint32_t eff_block = kv->compressed ? kv->block_size : block_size;
    if (eff_recent == 0 || eff_block == 0) return -5;
    const uint32_t old_len = seq_len > eff_recent ? seq_len - eff_recent : 0;
    const uint32_t old_blocks = old_len == 0 ? 0 : (old_len + eff_block - 1) / eff_block;
    *out_total_old_blocks = old_blocks;
    *out_count = 0;
    if (old_blocks == 0) return 0;
    if (hipStreamSynchronize(ctx->decode_stream) != hipSuccess) return -6;

    const uint32_t hd = kv->head_dim;
    const float scale = hd == 64u ? 0.125f : 0.08838834764831845f;
    std::vector<float> q(hd);
    if (hipMemcpy(q.data(), q_dev_f32, hd * sizeof(float), hipMemcpyDeviceToHost) != hipSuccess) return -7;
    const size_t ept = (size_t)kv->num_heads * hd;
    const uint16_t* src = nullptr;
    const bool fp16_old = kv->compressed && kv->fp16_k_q4_v_old_backing && kv->d_fp16_old_k;
    if (fp16_old) src = kv->d_fp16_old_k;
    else if (!kv->compressed && kv->d_k) src = kv->d_k;
    else return -8;  // summary-backed ranking of the lossy modes is not part of this build
    // rows of kv head 0: the fp16 old store is head-major (one contiguous [token][hd] plane per head), the dense
    // cache token-major
    const size_t row = fp16_old ? (size_t)hd : ept;
    std::vector<uint16_t> kh((size_t)old_len * row);
    if (hipMemcpy(kh.data(), src + (size_t)seq_id * kv->max_seq_len * ept, kh.size() * 2,
                  hipMemcpyDeviceToHost) != hipSuccess)
        return -12;

    std::vector<std::pair<float, uint32_t>> scored;
    scored.reserve(old_blocks);
    for (uint32_t b = 0; b < old_blocks; ++b) {
        const uint32_t start = b * eff_block, end = std::min(start + eff_block, old_len);
        float score = 0.0f;
        if (fp16_old) {
            for (uint32_t pos = start; pos < end; ++pos)
                for (uint32_t d = 0; d < hd; ++d) score += q[d] * host_h2f(kh[(size_t)pos * row + d]);
            score /= (float)(end - start);
        } else {
            std::vector<float> mean_k(hd, 0.0f);
            for (uint32_t pos = start; pos < end; ++pos)
                for (uint32_t d = 0; d < hd; ++d) mean_k[d] += host_h2f(kh[(size_t)pos * ept + d]);
            const float inv_count = 1.0f / (float)(end - start);
            for (uint32_t d = 0; d < hd; ++d) score += q[d] * (mean_k[d] * inv_count);
        }
        scored.emplace_back(score * scale, b);
    }
    std::sort(scored.begin(), scored.end(), [](const auto& a, const auto& b) {
        if (a.first == b.first) return a.second < b.second;
        return a.first > b.first;
    });
    const uint32_t requested = top_blocks == 0 ? old_blocks : std::min(top_blocks, old_blocks);
    const uint32_t capacity = std::min(std::min(requested, max_out), 64u);
    std::vector<uint32_t> selected;
    for (uint32_t i = 0; i < std::min(requested, capacity); ++i) selected.push_back(scored[i].second);
    const uint32_t order = selected_block_order_from_env();
    if (order == 1u) std::sort(selected.begin(), selected.end());
    else if (order == 2u) std::sort(selected.begin(), selected.end(), std::greater<uint32_t>());
    for (uint32_t i = 0; i < selected.size(); ++i) {
        const uint32_t b = selected[i];
        float sc = -1e30f;
        for (const auto& e : scored)
            if (e.second == b) { sc = e.first; break; }
        out_blocks_host[i] = b;
        out_scores_host[i] = sc;
        out_start_host[i] = b * eff_block;
        out_end_host[i] = std::min(b * eff_block + eff_block, old_len);
    }
    *out_count = (uint32_t)selected.size();
    return 0;
}

}  // extern "C"
