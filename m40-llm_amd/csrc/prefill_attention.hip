// Packed variable-length causal prefill attention for gfx950, all f32 (the step before decode).
//
// Q and Out are [total_q][q_heads][hd], K and V [total_kv][kv_heads][hd]; sequence b owns q_lens[b] query tokens from
// q_offsets[b] and kv_lens[b] keys from kv_offsets[b]; query q_idx attends keys 0 .. kv_len - q_len + q_idx.
//
// The reference walks every key once per (query, head) with one workgroup each (cuda/kernels.cu:3749-3835).  Here a
// workgroup owns 64 consecutive queries of one q head (four waves x 16 queries) and streams the sequence's keys in
// tiles of 32 through LDS, so a key row is fetched once per 64 queries.  Both products run on the f32 matrix
// instruction v_mfma_f32_16x16x4_f32 (inputs stay f32: no split, no rounding of K or V):
//   scores  S[query][key] = sum_d Q[query][d] K[key][d]   A = Q (kept in registers for the whole kernel), B = K tile
//   output  O[query][d]  += sum_key P[query][key] V[key][d]   A = softmax weights (through a 2 KB LDS tile per wave,
//           which turns the accumulator layout into the A-operand layout), B = V tile
// with a running maximum per query (the rows of a lane's accumulators are the same four queries in both products,
// so the rescaling needs no exchange).  The result is the same softmax as the reference's three passes
// (p = exp(s - max) / sum), within f32 rounding.
//
// Reference: kernel cuda/kernels.cu:3749-3835; entry points, argument checks and their codes :4834-4977
// (lengths are read back to the host and validated before the launch, also in the _async form).
#include "common.hpp"

#include <vector>

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = 4;
constexpr int kQTile = 16 * kWaves;      // queries per workgroup
constexpr int kKTile = 32;               // keys per LDS tile

__device__ __forceinline__ m40_float4 mfma16x16x4(float a, float b, m40_float4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ float row_max16(float x) {     // over the 16 lanes of a row group
    x = fmaxf(x, m40_dpp_f<M40_DPP_XOR1>(x));
    x = fmaxf(x, m40_dpp_f<M40_DPP_XOR2>(x));
    x = fmaxf(x, m40_dpp_f<M40_DPP_HALF_MIRROR>(x));
    x = fmaxf(x, m40_dpp_f<M40_DPP_MIRROR>(x));
    return x;
}

struct PrefillArgs {
    const float* Q; const float* K; const float* V; float* Out;
    const uint32_t* q_offsets; const uint32_t* kv_offsets; const uint32_t* q_lens; const uint32_t* kv_lens;
    uint32_t q_heads, kv_heads;
};

template <int HD>
__global__ __launch_bounds__(kThreads) void prefill_attn_kernel(PrefillArgs p) {
    constexpr int KS = HD / 4;             // MFMA k-steps of a score tile
    constexpr int DT = HD / 16;            // 16-column output tiles
    constexpr int KSTR = HD + 4;           // LDS floats per K row: key j, group g -> bank 4 j + g
    constexpr int VSTR = HD + 16;          // LDS floats per V row: key group g, column j -> bank 16 g + j
    constexpr int PSTR = kKTile + 4;       // LDS floats per row of a wave's weight tile
    constexpr int LD4 = kKTile * HD / 4 / kThreads;      // float4 loads per thread and tile, for K and for V
    __shared__ __attribute__((aligned(16))) float k_lds[kKTile * KSTR];
    __shared__ __attribute__((aligned(16))) float v_lds[kKTile * VSTR];
    __shared__ float p_lds[kWaves][16 * PSTR];

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

    // ---- this wave's 16 queries: A operand of the score product, lane (query j, k group g) holds Q[j][4 s + g]
    const uint32_t wq0 = q0 + 16u * wave;                         // first query of the wave
    const bool wave_live = wq0 < q_len;
    const uint32_t my_q = wq0 + j < q_len ? wq0 + j : q_len - 1;  // a query past the end repeats the last one (not stored)
    float qa[KS];
    {
        const float* qp = p.Q + ((size_t)(p.q_offsets[b] + my_q) * p.q_heads + h) * HD + g;
#pragma unroll
        for (int s = 0; s < KS; ++s) qa[s] = qp[4 * s];
    }
    // queries of this lane's accumulator rows: 4 g + r; their last visible key
    uint32_t row_end[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const uint32_t q = wq0 + 4u * g + r;
        row_end[r] = shift + (q < q_len ? q : q_len - 1);
    }
    const uint32_t wave_end = shift + (wq0 + 15u < q_len ? wq0 + 15u : q_len - 1);    // last key any query of the wave sees

    // ---- K / V tile loads: thread t moves float4 t, t + 256, ... of the tile's [32][HD] block
    const float* Kb = p.K + ((size_t)p.kv_offsets[b] * p.kv_heads + kvh) * HD;
    const float* Vb = p.V + ((size_t)p.kv_offsets[b] * p.kv_heads + kvh) * HD;
    const size_t row_stride = (size_t)p.kv_heads * HD;
    float4 kreg[LD4], vreg[LD4];
    auto issue = [&](uint32_t tile) {
#pragma unroll
        for (int u = 0; u < LD4; ++u) {
            const int f = u * kThreads + tid;                     // float4 index inside the tile
            const uint32_t key_in = (uint32_t)(f / (HD / 4)), c4 = (uint32_t)(f % (HD / 4));
            uint32_t key = tile * kKTile + key_in;
            key = key < kv_len ? key : kv_len - 1;                // past the sequence: a valid row, masked later
            kreg[u] = *reinterpret_cast<const float4*>(Kb + (size_t)key * row_stride + 4 * c4);
            vreg[u] = *reinterpret_cast<const float4*>(Vb + (size_t)key * row_stride + 4 * c4);
        }
    };
    auto to_lds = [&]() {
#pragma unroll
        for (int u = 0; u < LD4; ++u) {
            const int f = u * kThreads + tid;
            const int key_in = f / (HD / 4), c4 = f % (HD / 4);
            float* kd = k_lds + key_in * KSTR + 4 * c4;
            kd[0] = kreg[u].x; kd[1] = kreg[u].y; kd[2] = kreg[u].z; kd[3] = kreg[u].w;
            float* vd = v_lds + key_in * VSTR + 4 * c4;
            vd[0] = vreg[u].x; vd[1] = vreg[u].y; vd[2] = vreg[u].z; vd[3] = vreg[u].w;
        }
    };
    issue(0);

    float m_run[4], l_run[4];             // running maximum of the row (equal in its 16 lanes); this lane's share of the sum
    m40_float4 O[DT];
#pragma unroll
    for (int r = 0; r < 4; ++r) { m_run[r] = -INFINITY; l_run[r] = 0.0f; }
#pragma unroll
    for (int d = 0; d < DT; ++d) O[d] = m40_float4{0.f, 0.f, 0.f, 0.f};
    float* my_p = p_lds[wave];

    for (uint32_t tile = 0; tile < n_tiles; ++tile) {
        __syncthreads();                  // the previous tile has been read by every wave
        to_lds();
        __syncthreads();
        if (tile + 1 < n_tiles) issue(tile + 1);
        const uint32_t key0 = tile * kKTile;
        if (!wave_live || key0 > wave_end) continue;              // nothing of this tile is visible to the wave

        // scores of the two 16-key halves: lane (key j, g) gets rows 4 g + r
        m40_float4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            s0 = mfma16x16x4(qa[s], k_lds[j * KSTR + 4 * s + g], s0);
            s1 = mfma16x16x4(qa[s], k_lds[(16 + j) * KSTR + 4 * s + g], s1);
        }
        float p0[4], p1[4], f[4];
        bool moved = false;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const bool a0 = key0 + (uint32_t)j <= row_end[r], a1 = key0 + 16u + (uint32_t)j <= row_end[r];
            const float x0 = a0 ? s0[r] * inv_sqrt : -INFINITY, x1 = a1 ? s1[r] * inv_sqrt : -INFINITY;
            const float n = fmaxf(m_run[r], row_max16(fmaxf(x0, x1)));
            // no maximum yet: the old state weighs nothing; a masked key weighs nothing
            f[r] = m_run[r] == -INFINITY ? 0.0f : __expf(m_run[r] - n);
            p0[r] = a0 ? __expf(x0 - n) : 0.0f;
            p1[r] = a1 ? __expf(x1 - n) : 0.0f;
            l_run[r] = fmaf(l_run[r], f[r], p0[r] + p1[r]);
            moved = moved || m_run[r] != n;
            m_run[r] = n;
            my_p[(4 * g + r) * PSTR + j] = p0[r];
            my_p[(4 * g + r) * PSTR + 16 + j] = p1[r];
        }
        if (__any(moved)) {               // the accumulators are only rescaled when some row's maximum rose
#pragma unroll
            for (int d = 0; d < DT; ++d)
#pragma unroll
                for (int r = 0; r < 4; ++r) O[d][r] *= f[r];
        }
        __builtin_amdgcn_wave_barrier();
        // O += P . V: A = P[query j][key 4 s + g], B = V[key 4 s + g][column 16 d + j]
        float pa[kKTile / 4];
#pragma unroll
        for (int s = 0; s < kKTile / 4; ++s) pa[s] = my_p[j * PSTR + 4 * s + g];
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int d = 0; d < DT; ++d) {
#pragma unroll
            for (int s = 0; s < kKTile / 4; ++s) O[d] = mfma16x16x4(pa[s], v_lds[(4 * s + g) * VSTR + 16 * d + j], O[d]);
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
