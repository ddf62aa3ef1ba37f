// Packed variable-length causal prefill attention for gfx950, f32 in and out (the step before decode).
//
// Q and Out are [total_q][q_heads][hd], K and V [total_kv][kv_heads][hd]; sequence b owns q_lens[b] query tokens from
// q_offsets[b] and kv_lens[b] keys from kv_offsets[b]; query q_idx attends keys 0 .. kv_len - q_len + q_idx.
//
// The reference walks every key once per (query, head) with one workgroup each (cuda/kernels.cu:3749-3835).  Here a
// workgroup owns 64 consecutive queries of one q head (four waves x 16 queries) and streams the sequence's keys in
// tiles of 32 through LDS, so a key row is fetched once per 64 queries.  Both products run on v_mfma_f32_16x16x32_f16
// with every f32 operand split exactly into an f16 high and an f16 low part (x = hi + lo to 2^-22): a product is
// three instructions, hi hi + lo hi + hi lo (the lo lo term is below 2^-22 of the operands' magnitudes), which is
// five times the rate of the f32 matrix instruction for the same product at f32-level accuracy:
//   scores  S[query][key] = sum_d Q[query][d] K[key][d]   A = Q (two f16 parts, in registers for the whole kernel),
//           B = K tile (two f16 planes in LDS)
//   output  O[query][d]  += sum_key P[query][key] V[key][d]   A = softmax weights (two f16 planes through a small LDS
//           tile per wave, which turns the accumulator layout into the A-operand layout), B = V tile, stored
//           transposed [d][key] so that eight consecutive keys are one 16-byte read
// with a running maximum per query (the rows of a lane's accumulators are the same four queries in both products,
// so the rescaling needs no exchange).  The result is the same softmax as the reference's three passes
// (p = exp(s - max) / sum), within f32 rounding.  Operands beyond the f16 range (|x| > 65504) are not supported by the
// split (none occur after RMSNorm-scaled projections; the decode-side attention has no such limit).
//
// Reference: kernel cuda/kernels.cu:3749-3835; entry points, argument checks and their codes :4834-4977
// (lengths are read back to the host and validated before the launch, also in the _async form).
#include "common.hpp"

#include <vector>

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = 4;
constexpr int kQTile = 16 * kWaves;      // queries per workgroup
constexpr int kKTile = 32;               // keys per LDS tile = the K depth of one matrix instruction of the P . V product

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));

__device__ __forceinline__ m40_float4 mfma32(half8 a, half8 b, m40_float4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ float row_max16(float x) {     // over the 16 lanes of a row group
    x = fmaxf(x, m40_dpp_f<M40_DPP_XOR1>(x));
    x = fmaxf(x, m40_dpp_f<M40_DPP_XOR2>(x));
    x = fmaxf(x, m40_dpp_f<M40_DPP_HALF_MIRROR>(x));
    x = fmaxf(x, m40_dpp_f<M40_DPP_MIRROR>(x));
    return x;
}
// x = hi + lo with both parts f16: exact to about 2^-22 relative for values inside the f16 range
__device__ __forceinline__ void split(float x, _Float16* hi, _Float16* lo) {
    const _Float16 h = static_cast<_Float16>(x);
    *hi = h;
    *lo = static_cast<_Float16>(x - static_cast<float>(h));
}

struct PrefillArgs {
    const float* Q; const float* K; const float* V; float* Out;
    const uint32_t* q_offsets; const uint32_t* kv_offsets; const uint32_t* q_lens; const uint32_t* kv_lens;
    uint32_t q_heads, kv_heads;
};

template <int HD>
__global__ __launch_bounds__(kThreads) void prefill_attn_kernel(PrefillArgs p) {
    constexpr int KS = HD / 32;            // matrix-instruction k-steps of a score tile
    constexpr int DT = HD / 16;            // 16-column output tiles
    constexpr int KSTR = HD + 8;           // LDS halves per K row: 16-byte fragment reads of 16 keys hit 64 distinct banks
    constexpr int VSTR = kKTile + 8;       // LDS halves per row of the transposed V tile [column][key]
    constexpr int PSTR = kKTile + 8;       // LDS halves per row of a wave's weight tile
    constexpr int KLD = kKTile * HD / 4 / kThreads;        // float4 loads of K per thread and tile
    constexpr int VLD = kKTile / 2 * HD / 4 / kThreads;    // key pairs x float4 columns of V per thread and tile
    __shared__ __attribute__((aligned(16))) _Float16 k_lds[2][kKTile * KSTR];   // [hi, lo][key][d]
    __shared__ __attribute__((aligned(16))) _Float16 v_lds[2][HD * VSTR];       // [hi, lo][d][key]
    __shared__ __attribute__((aligned(16))) _Float16 p_lds[kWaves][2][16 * PSTR];

    const uint32_t b = blockIdx.z, h = blockIdx.y;
    const uint32_t q_len = p.q_lens[b], kv_len = p.kv_lens[b];
    const uint32_t q0 = (gridDim.x - 1u - blockIdx.x) * kQTile;   // late query tiles see the most keys: they start first
    if (q0 >= q_len || q_len > kv_len) return;
    const uint32_t kvh = h / (p.q_heads / p.kv_heads);
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int j = lane & 15, g = lane >> 4;
    const float inv_sqrt = HD == 64 ? 0.125f : 0.08838834764831845f;
    const uint32_t shift = kv_len - q_len;                        // query q attends keys 0 .. shift + q
    const uint32_t wg_last_q = q0 + kQTile - 1 < q_len - 1 ? q0 + kQTile - 1 : q_len - 1;
    const uint32_t n_tiles = (shift + wg_last_q) / kKTile + 1;    // key tiles this workgroup walks

    // ---- this wave's 16 queries: A operand of the score product, lane (query j, k group g) holds
    //      Q[j][32 s + 8 g .. + 7] as a high and a low f16 part
    const uint32_t wq0 = q0 + 16u * wave;                         // first query of the wave
    const bool wave_live = wq0 < q_len;
    const uint32_t my_q = wq0 + j < q_len ? wq0 + j : q_len - 1;  // a query past the end repeats the last one (not stored)
    half8 qh[KS], ql[KS];
    {
        const float* qp = p.Q + ((size_t)(p.q_offsets[b] + my_q) * p.q_heads + h) * HD + 8 * g;
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            const float4 x0 = *reinterpret_cast<const float4*>(qp + 32 * s), x1 = *reinterpret_cast<const float4*>(qp + 32 * s + 4);
            const float x[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                _Float16 a, c;
                split(x[i], &a, &c);
                qh[s][i] = a;
                ql[s][i] = c;
            }
        }
    }
    // queries of this lane's accumulator rows: 4 g + r; their last visible key
    uint32_t row_end[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const uint32_t q = wq0 + 4u * g + r;
        row_end[r] = shift + (q < q_len ? q : q_len - 1);
    }
    const uint32_t wave_end = shift + (wq0 + 15u < q_len ? wq0 + 15u : q_len - 1);    // last key any query of the wave sees

    // ---- K / V tile loads.  K: thread t moves float4 t, t + 256, ... of the tile's [32][HD] block.  V: a thread takes
    //      the same four columns of two adjacent keys, so that the transposed tile is written two keys (one 32-bit
    //      word) at a time.
    const float* Kb = p.K + ((size_t)p.kv_offsets[b] * p.kv_heads + kvh) * HD;
    const float* Vb = p.V + ((size_t)p.kv_offsets[b] * p.kv_heads + kvh) * HD;
    const size_t row_stride = (size_t)p.kv_heads * HD;
    float4 kreg[KLD], vreg[VLD][2];
    auto issue = [&](uint32_t tile) {
#pragma unroll
        for (int u = 0; u < KLD; ++u) {
            const int f = u * kThreads + tid;                     // float4 index inside the tile
            const uint32_t key_in = (uint32_t)(f / (HD / 4)), c4 = (uint32_t)(f % (HD / 4));
            uint32_t key = tile * kKTile + key_in;
            key = key < kv_len ? key : kv_len - 1;                // past the sequence: a valid row, masked later
            kreg[u] = *reinterpret_cast<const float4*>(Kb + (size_t)key * row_stride + 4 * c4);
        }
#pragma unroll
        for (int u = 0; u < VLD; ++u) {
            const int f = u * kThreads + tid;
            const uint32_t pair = (uint32_t)(f / (HD / 4)), c4 = (uint32_t)(f % (HD / 4));
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                uint32_t key = tile * kKTile + 2u * pair + (uint32_t)e;
                key = key < kv_len ? key : kv_len - 1;
                vreg[u][e] = *reinterpret_cast<const float4*>(Vb + (size_t)key * row_stride + 4 * c4);
            }
        }
    };
    auto to_lds = [&]() {
#pragma unroll
        for (int u = 0; u < KLD; ++u) {
            const int f = u * kThreads + tid;
            const int key_in = f / (HD / 4), c4 = f % (HD / 4);
            const float x[4] = {kreg[u].x, kreg[u].y, kreg[u].z, kreg[u].w};
            half4 hi, lo;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                _Float16 a, c;
                split(x[i], &a, &c);
                hi[i] = a;
                lo[i] = c;
            }
            *reinterpret_cast<half4*>(&k_lds[0][key_in * KSTR + 4 * c4]) = hi;
            *reinterpret_cast<half4*>(&k_lds[1][key_in * KSTR + 4 * c4]) = lo;
        }
#pragma unroll
        for (int u = 0; u < VLD; ++u) {
            const int f = u * kThreads + tid;
            const int pair = f / (HD / 4), c4 = f % (HD / 4);
            const float x0[4] = {vreg[u][0].x, vreg[u][0].y, vreg[u][0].z, vreg[u][0].w};
            const float x1[4] = {vreg[u][1].x, vreg[u][1].y, vreg[u][1].z, vreg[u][1].w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                half2v hi, lo;
                _Float16 a, c;
                split(x0[i], &a, &c);
                hi[0] = a; lo[0] = c;
                split(x1[i], &a, &c);
                hi[1] = a; lo[1] = c;
                *reinterpret_cast<half2v*>(&v_lds[0][(4 * c4 + i) * VSTR + 2 * pair]) = hi;
                *reinterpret_cast<half2v*>(&v_lds[1][(4 * c4 + i) * VSTR + 2 * pair]) = lo;
            }
        }
    };
    issue(0);

    float m_run[4], l_run[4];             // running maximum of the row (equal in its 16 lanes); this lane's share of the sum
    m40_float4 O[DT];
#pragma unroll
    for (int r = 0; r < 4; ++r) { m_run[r] = -INFINITY; l_run[r] = 0.0f; }
#pragma unroll
    for (int d = 0; d < DT; ++d) O[d] = m40_float4{0.f, 0.f, 0.f, 0.f};
    _Float16* my_ph = p_lds[wave][0];
    _Float16* my_pl = p_lds[wave][1];

    for (uint32_t tile = 0; tile < n_tiles; ++tile) {
        __syncthreads();                  // the previous tile has been read by every wave
        to_lds();
        __syncthreads();
        if (tile + 1 < n_tiles) issue(tile + 1);
        const uint32_t key0 = tile * kKTile;
        if (!wave_live || key0 > wave_end) continue;              // nothing of this tile is visible to the wave

        // scores of the two 16-key halves: lane (key j, g) gets rows 4 g + r.  q . k = qh kh + ql kh + qh kl
        // (the ql kl term is below 2^-22 of |q| |k|)
        m40_float4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            const int off = 32 * s + 8 * g;
            const half8 k0h = *reinterpret_cast<const half8*>(&k_lds[0][j * KSTR + off]);
            const half8 k0l = *reinterpret_cast<const half8*>(&k_lds[1][j * KSTR + off]);
            const half8 k1h = *reinterpret_cast<const half8*>(&k_lds[0][(16 + j) * KSTR + off]);
            const half8 k1l = *reinterpret_cast<const half8*>(&k_lds[1][(16 + j) * KSTR + off]);
            s0 = mfma32(qh[s], k0h, s0);
            s1 = mfma32(qh[s], k1h, s1);
            s0 = mfma32(ql[s], k0h, s0);
            s1 = mfma32(ql[s], k1h, s1);
            s0 = mfma32(qh[s], k0l, s0);
            s1 = mfma32(qh[s], k1l, s1);
        }
        float f[4];
        bool moved = false;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const bool a0 = key0 + (uint32_t)j <= row_end[r], a1 = key0 + 16u + (uint32_t)j <= row_end[r];
            const float x0 = a0 ? s0[r] * inv_sqrt : -INFINITY, x1 = a1 ? s1[r] * inv_sqrt : -INFINITY;
            const float n = fmaxf(m_run[r], row_max16(fmaxf(x0, x1)));
            // no maximum yet: the old state weighs nothing; a masked key weighs nothing
            f[r] = m_run[r] == -INFINITY ? 0.0f : __expf(m_run[r] - n);
            const float p0 = a0 ? __expf(x0 - n) : 0.0f;
            const float p1 = a1 ? __expf(x1 - n) : 0.0f;
            l_run[r] = fmaf(l_run[r], f[r], p0 + p1);
            moved = moved || m_run[r] != n;
            m_run[r] = n;
            _Float16 a, c;
            split(p0, &a, &c);
            my_ph[(4 * g + r) * PSTR + j] = a;
            my_pl[(4 * g + r) * PSTR + j] = c;
            split(p1, &a, &c);
            my_ph[(4 * g + r) * PSTR + 16 + j] = a;
            my_pl[(4 * g + r) * PSTR + 16 + j] = c;
        }
        if (__any(moved)) {               // the accumulators are only rescaled when some row's maximum rose
#pragma unroll
            for (int d = 0; d < DT; ++d)
#pragma unroll
                for (int r = 0; r < 4; ++r) O[d][r] *= f[r];
        }
        __builtin_amdgcn_wave_barrier();
        // O += P . V over the tile's 32 keys in one k-step: A = P[query j][key 8 g .. + 7], B = V^T[column 16 d + j][key 8 g .. + 7];
        // p v = ph vh + pl vh + ph vl
        const half8 ph = *reinterpret_cast<const half8*>(&my_ph[j * PSTR + 8 * g]);
        const half8 pl = *reinterpret_cast<const half8*>(&my_pl[j * PSTR + 8 * g]);
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int d = 0; d < DT; ++d) {
            const half8 vh = *reinterpret_cast<const half8*>(&v_lds[0][(16 * d + j) * VSTR + 8 * g]);
            const half8 vl = *reinterpret_cast<const half8*>(&v_lds[1][(16 * d + j) * VSTR + 8 * g]);
            O[d] = mfma32(ph, vh, O[d]);
            O[d] = mfma32(pl, vh, O[d]);
            O[d] = mfma32(ph, vl, O[d]);
        }
    }

    // ---- out = O / sum
    if (!wave_live) return;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const uint32_t q = wq0 + 4u * g + r;
        const float l = m40_sum16(l_run[r]);
        const float denom = l > 0.0f ? l : 1.0f;
        if (q < q_len) {
            float* op = p.Out + ((size_t)(p.q_offsets[b] + q) * p.q_heads + h) * HD + j;
#pragma unroll
            for (int d = 0; d < DT; ++d) op[16 * d] = O[d][r] / denom;
        }
    }
}

int prefill_impl(M40llmCudaContext* ctx, const void* q, const void* k, const void* v, const uint32_t* q_offsets,
                 const uint32_t* kv_offsets, const uint32_t* q_lens, const uint32_t* kv_lens, uint32_t batch,
                 uint32_t q_heads, uint32_t kv_heads, uint32_t head_dim, void* out, bool synchronize) {
    if (!ctx || !q || !k || !v || !q_offsets || !kv_offsets || !q_lens || !kv_lens || !out) return -1;
    if (batch == 0) return -2;
    if (q_heads == 0 || kv_heads == 0 || q_heads % kv_heads != 0) return -3;
    if (head_dim != 64 && head_dim != 128) return -9;
    // the lengths are validated on the host before the launch, as the reference does (also in the _async form)
    std::vector<uint32_t> host(2 * (size_t)batch);
    if (hipMemcpy(host.data(), q_lens, (size_t)batch * sizeof(uint32_t), hipMemcpyDeviceToHost) != hipSuccess) return -7;
    if (hipMemcpy(host.data() + batch, kv_lens, (size_t)batch * sizeof(uint32_t), hipMemcpyDeviceToHost) != hipSuccess) return -7;
    uint32_t max_q = 0, max_kv = 0;
    for (uint32_t i = 0; i < batch; ++i) {
        const uint32_t ql = host[i], kl = host[batch + i];
        if (ql == 0 || kl == 0 || ql > kl || kl > 8192) return -8;
        max_q = ql > max_q ? ql : max_q;
        max_kv = kl > max_kv ? kl : max_kv;
    }
    if (!m40_aligned16(q) || !m40_aligned16(k) || !m40_aligned16(v)) return -4;
    PrefillArgs a{};
    a.Q = static_cast<const float*>(q); a.K = static_cast<const float*>(k); a.V = static_cast<const float*>(v);
    a.Out = static_cast<float*>(out);
    a.q_offsets = q_offsets; a.kv_offsets = kv_offsets; a.q_lens = q_lens; a.kv_lens = kv_lens;
    a.q_heads = q_heads; a.kv_heads = kv_heads;
    (void)hipGetLastError();
    const dim3 grid((max_q + kQTile - 1) / kQTile, q_heads, batch);
    if (head_dim == 64) prefill_attn_kernel<64><<<grid, kThreads, 0, ctx->prefill_stream>>>(a);
    else prefill_attn_kernel<128><<<grid, kThreads, 0, ctx->prefill_stream>>>(a);
    if (hipGetLastError() != hipSuccess) return -4;
    if (synchronize && hipStreamSynchronize(ctx->prefill_stream) != hipSuccess) return -5;
    return 0;
}

}  // namespace

extern "C" {

int m40llm_attention_prefill_f32_gqa_varlen(M40llmCudaContext* ctx, const void* q_dev_f32, const void* k_dev_f32,
                                            const void* v_dev_f32, const uint32_t* q_offsets_dev,
                                            const uint32_t* kv_offsets_dev, const uint32_t* q_lens_dev,
                                            const uint32_t* kv_lens_dev, uint32_t batch_size, uint32_t q_heads,
                                            uint32_t kv_heads, uint32_t head_dim, void* out_dev_f32) {
    return prefill_impl(ctx, q_dev_f32, k_dev_f32, v_dev_f32, q_offsets_dev, kv_offsets_dev, q_lens_dev, kv_lens_dev,
                        batch_size, q_heads, kv_heads, head_dim, out_dev_f32, true);
}

int m40llm_attention_prefill_f32_gqa_varlen_async(M40llmCudaContext* ctx, const void* q_dev_f32, const void* k_dev_f32,
                                                  const void* v_dev_f32, const uint32_t* q_offsets_dev,
                                                  const uint32_t* kv_offsets_dev, const uint32_t* q_lens_dev,
                                                  const uint32_t* kv_lens_dev, uint32_t batch_size, uint32_t q_heads,
                                                  uint32_t kv_heads, uint32_t head_dim, void* out_dev_f32) {
    return prefill_impl(ctx, q_dev_f32, k_dev_f32, v_dev_f32, q_offsets_dev, kv_offsets_dev, q_lens_dev, kv_lens_dev,
                        batch_size, q_heads, kv_heads, head_dim, out_dev_f32, false);
}

}  // extern "C"
