// Row-batched GEMV for the small projections of a batched decode step on gfx950: up to eight activation rows
// against f16 GGUF weights [N][K] with K <= 2048, on the vector ALUs.
//
// For the Q/K/V and O projections of a batch-8 step (N ~ 2048, K = 2048: 8-10 MB of weights) the matrix-core
// kernel has too few 16-column tiles to fill the chip without splitting K, and a split K costs a second launch that
// adds the slices.  Here a wave owns two output columns and all eight rows: the rows sit in LDS as f32 (64 KB per
// workgroup), every lane multiplies its 16-byte weight chunks with the matching eight activations of each row
// (16 accumulators), and the epilogue (bias, residual, RoPE, cache append) runs in the same kernel.  Arithmetic per
// output element is the batch-1 GEMV's: same lane -> k mapping, same FMA chain, same butterfly.  Everything a
// workgroup needs early (rows, norm weights, positions) is requested before the weight stream.
#include "common.hpp"
#include "gemv_core.hpp"

namespace {

constexpr int kThreads = 256;       // measured: 256 threads and two columns per wave beat 512 threads / four columns
constexpr int kWaves = kThreads / 64;
constexpr int kRows = 8;
constexpr int kCols = 2;            // columns per wave
constexpr int kMaxK = 2048;         // 8 rows x 2048 x 4 bytes = 64 KB of LDS
constexpr int kU = kMaxK / 4 / kThreads;   // 16-byte pieces of a row per thread

// Requests rows [0, rows) of x (and the norm weights when given) for this thread: 16-byte piece tid + kThreads * u of each row.
struct RowsRegs {
    float4 x[kRows][kU];
    uint4 w[kU];
};
__device__ __forceinline__ void rows_load(const float* __restrict__ x, const void* __restrict__ norm_w, uint32_t w_dtype,
                                          int rows, int K, RowsRegs& r) {
    const int n4 = K >> 2;
#pragma unroll
    for (int u = 0; u < kU; ++u) {
        const int i = u * kThreads + (int)threadIdx.x;
        const int ic = i < n4 ? i : 0;
#pragma unroll
        for (int row = 0; row < kRows; ++row)
            r.x[row][u] = reinterpret_cast<const float4*>(x + (size_t)(row < rows ? row : 0) * K)[ic];
        if (norm_w) {
            if (w_dtype == 0u) {
                const uint2 h = reinterpret_cast<const uint2*>(norm_w)[ic];
                r.w[u].x = h.x; r.w[u].y = h.y; r.w[u].z = 0u; r.w[u].w = 0u;
            } else {
                r.w[u] = reinterpret_cast<const uint4*>(norm_w)[ic];
            }
        }
    }
}

// LDS rows a[row][k] = x[row][k] (* rsqrt(mean(x[row]^2) + eps) * w[k] with norm weights); rows >= `rows` are zero.
// Reduction order per row identical to the batch-1 staging (thread-local chain, wave butterfly, waves in order).
__device__ __forceinline__ void rows_stage(const RowsRegs& r, bool normed, uint32_t w_dtype, float eps, int rows, int K,
                                           float* __restrict__ a_lds, float (*wave_sums)[kRows]) {
    const int tid = threadIdx.x, n4 = K >> 2;
    float scale[kRows];
    if (normed) {
        float ss[kRows];
#pragma unroll
        for (int row = 0; row < kRows; ++row) {
            ss[row] = 0.0f;
#pragma unroll
            for (int u = 0; u < kU; ++u) {
                if (u * kThreads + tid < n4) {
                    const float4 v = r.x[row][u];
                    ss[row] = fmaf(v.x, v.x, ss[row]); ss[row] = fmaf(v.y, v.y, ss[row]);
                    ss[row] = fmaf(v.z, v.z, ss[row]); ss[row] = fmaf(v.w, v.w, ss[row]);
                }
            }
            ss[row] = m40_sum64(ss[row]);
        }
        if ((tid & 63) == 0) {
#pragma unroll
            for (int row = 0; row < kRows; ++row) wave_sums[tid >> 6][row] = ss[row];
        }
        __syncthreads();
#pragma unroll
        for (int row = 0; row < kRows; ++row) {
            float total = 0.0f;
#pragma unroll
            for (int w = 0; w < kWaves; ++w) total += wave_sums[w][row];
            scale[row] = 1.0f / sqrtf(total / static_cast<float>(K) + eps);
        }
    }
#pragma unroll
    for (int u = 0; u < kU; ++u) {
        const int i = u * kThreads + tid;
        if (i < n4) {
            float4 wv = make_float4(1.0f, 1.0f, 1.0f, 1.0f);
            if (normed) {
                wv = make_float4(__uint_as_float(r.w[u].x), __uint_as_float(r.w[u].y), __uint_as_float(r.w[u].z),
                                 __uint_as_float(r.w[u].w));
                if (w_dtype == 0u)
                    wv = make_float4(m40_h2f((uint16_t)(r.w[u].x & 0xffffu)), m40_h2f((uint16_t)(r.w[u].x >> 16)),
                                     m40_h2f((uint16_t)(r.w[u].y & 0xffffu)), m40_h2f((uint16_t)(r.w[u].y >> 16)));
            }
#pragma unroll
            for (int row = 0; row < kRows; ++row) {
                float4 v = r.x[row][u];
                if (normed) v = make_float4(v.x * scale[row] * wv.x, v.y * scale[row] * wv.y, v.z * scale[row] * wv.z,
                                            v.w * scale[row] * wv.w);
                if (row >= rows) v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                reinterpret_cast<float4*>(a_lds + (size_t)row * K)[i] = v;
            }
        }
    }
    __syncthreads();
}

// acc[c][row] = sum over the wave's chunks, then over the lanes: valid in every lane.
__device__ __forceinline__ void rows_dot(const GemvRegs<kCols>& regs, const float* __restrict__ a_lds, int K, int lane,
                                         float (&acc)[kCols][kRows]) {
    const int nch = K >> 3;
#pragma unroll
    for (int c = 0; c < kCols; ++c)
#pragma unroll
        for (int row = 0; row < kRows; ++row) acc[c][row] = 0.0f;
#pragma unroll
    for (int i = 0; i < kGemvPrefetch; ++i) {
        const int kc = lane + 64 * i;
        if (kc < nch) {
#pragma unroll
            for (int row = 0; row < kRows; ++row) {
                const float4 a0 = *reinterpret_cast<const float4*>(a_lds + (size_t)row * K + 8 * kc);
                const float4 a1 = *reinterpret_cast<const float4*>(a_lds + (size_t)row * K + 8 * kc + 4);
#pragma unroll
                for (int c = 0; c < kCols; ++c) gemv_fma8(regs.w[i][c], a0, a1, acc[c][row]);
            }
        }
    }
#pragma unroll
    for (int c = 0; c < kCols; ++c)
#pragma unroll
        for (int row = 0; row < kRows; ++row) acc[c][row] = m40_sum64(acc[c][row]);
}

// value of acc[c][row] for a per-lane (c, row): a chain of selects, the indices are not compile-time constants
__device__ __forceinline__ float rows_pick(const float (&acc)[kCols][kRows], int c, int row) {
    float v = 0.0f;
#pragma unroll
    for (int cc = 0; cc < kCols; ++cc)
#pragma unroll
        for (int rr = 0; rr < kRows; ++rr) v = (cc == c && rr == row) ? acc[cc][rr] : v;
    return v;
}

// out[row][n] = residual[row][n] + W[n] . a[row]      (residual may be null or alias out)
__global__ __launch_bounds__(kThreads) void rows_gemv_residual_kernel(const float* __restrict__ a,
                                                                      const uint16_t* __restrict__ W,
                                                                      const float* residual, float* out, int rows, int N,
                                                                      int K) {
    extern __shared__ float a_lds[];
    __shared__ float wave_sums[kWaves][kRows];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int col0 = (blockIdx.x * kWaves + wave) * kCols;
    // lane (row, c) of the epilogue: kRows * kCols lanes write one element each
    const int e_row = (lane / kCols) & (kRows - 1), e_c = lane % kCols;
    const int e_col = col0 + e_c < N ? col0 + e_c : N - 1;
    RowsRegs xr;
    rows_load(a, nullptr, 0u, rows, K, xr);
    const float res = *(residual ? residual + (size_t)(e_row < rows ? e_row : 0) * N + e_col : a);
    const uint4* bp[kCols];
#pragma unroll
    for (int c = 0; c < kCols; ++c) bp[c] = reinterpret_cast<const uint4*>(W + (size_t)(col0 + c < N ? col0 + c : N - 1) * K);
    GemvRegs<kCols> regs;
    gemv_prefetch<kCols>(bp, 0, K >> 3, lane, regs);
    rows_stage(xr, false, 0u, 0.0f, rows, K, a_lds, wave_sums);
    float acc[kCols][kRows];
    rows_dot(regs, a_lds, K, lane, acc);
    if (lane < kRows * kCols && e_row < rows && col0 + e_c < N) {
        const float d = rows_pick(acc, e_c, e_row);
        out[(size_t)e_row * N + col0 + e_c] = residual ? res + d : d;
    }
}

struct RowsQkvArgs {
    const float* x;
    const void* norm_w;
    const uint16_t *wq, *wk, *wv;
    const float *bq, *bk, *bv;
    float* q_out;                 // [rows][q_heads * head_dim]
    uint16_t* k_cache; uint16_t* v_cache; uint32_t* seq_map;
    const uint32_t* ids_dev; const uint32_t* lens_dev;
    uint32_t rows, d_model, max_seq_len, max_batch, q_heads, kv_heads, head_dim, rope_layout, norm_dtype;
    float eps, rope_base, rope_scale;
    const float* rope_table;      // pair frequencies of (head_dim, rope_base), or null
};

// RMSNorm of every row, Q/K/V projections, bias, RoPE at each row's position, q out, K/V (f16) into the cache rows.
// A wave owns kCols / 2 rotation pairs.  Pair space: Q pairs, then K pairs, then V pairs.
__global__ __launch_bounds__(kThreads) void rows_norm_qkv_kernel(RowsQkvArgs p) {
    extern __shared__ float a_lds[];
    __shared__ float wave_sums[kWaves][kRows];
    const int K = (int)p.d_model;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const uint32_t half = p.head_dim / 2u;
    const uint32_t q_pairs = p.q_heads * half, kv_pairs = p.kv_heads * half;
    const uint32_t total = q_pairs + 2u * kv_pairs;
    constexpr int kPairs = kCols / 2;
    const uint32_t pair0 = (blockIdx.x * kWaves + wave) * (uint32_t)kPairs;
    const uint4* bp[kCols];
#pragma unroll
    for (int q = 0; q < kPairs; ++q) {
        uint32_t pair = pair0 + q;
        pair = pair < total ? pair : total - 1u;
        int which; uint32_t local;
        if (pair < q_pairs) { which = 0; local = pair; }
        else if (pair < q_pairs + kv_pairs) { which = 1; local = pair - q_pairs; }
        else { which = 2; local = pair - q_pairs - kv_pairs; }
        size_t i0, i1;
        m40_rope_pair(local / half, local % half, p.head_dim, which == 2 ? M40LLM_ROPE_LAYOUT_ADJACENT : p.rope_layout, &i0, &i1);
        const uint16_t* W = which == 0 ? p.wq : (which == 1 ? p.wk : p.wv);
        bp[2 * q] = reinterpret_cast<const uint4*>(W + i0 * (size_t)K);
        bp[2 * q + 1] = reinterpret_cast<const uint4*>(W + i1 * (size_t)K);
    }
    // epilogue lane (row, pair q): kRows * kPairs lanes rotate and write one pair each
    const int e_row = (lane / kPairs) & (kRows - 1), e_q = lane % kPairs;
    uint32_t e_pair = pair0 + (uint32_t)e_q;
    const bool e_live = lane < kPairs * kRows && e_row < (int)p.rows && e_pair < total;
    e_pair = e_pair < total ? e_pair : total - 1u;
    int e_which; uint32_t e_local;
    if (e_pair < q_pairs) { e_which = 0; e_local = e_pair; }
    else if (e_pair < q_pairs + kv_pairs) { e_which = 1; e_local = e_pair - q_pairs; }
    else { e_which = 2; e_local = e_pair - q_pairs - kv_pairs; }
    const uint32_t e_off = e_local % half;
    size_t e_i0, e_i1;
    m40_rope_pair(e_local / half, e_off, p.head_dim, e_which == 2 ? M40LLM_ROPE_LAYOUT_ADJACENT : p.rope_layout, &e_i0, &e_i1);
    const float* bias = e_which == 0 ? p.bq : (e_which == 1 ? p.bk : p.bv);

    RowsRegs xr;
    rows_load(p.x, p.norm_w, p.norm_dtype, (int)p.rows, K, xr);
    const uint32_t e_rowc = e_row < (int)p.rows ? (uint32_t)e_row : 0u;
    const uint32_t position = p.lens_dev[e_rowc];
    const uint32_t seq = p.ids_dev[e_rowc];
    const float b0 = *(bias ? bias + e_i0 : p.x), b1 = *(bias ? bias + e_i1 : p.x);
    float inv_freq = p.rope_table ? p.rope_table[e_off] : 0.0f;
    GemvRegs<kCols> regs;
    gemv_prefetch<kCols>(bp, 0, K >> 3, lane, regs);
    // the rotation angle does not depend on the projections: evaluated while the weights are in flight
    float2 cs = make_float2(1.0f, 0.0f);
    if (e_which != 2) {
        if (!p.rope_table) inv_freq = m40_rope_inv_freq(e_off, p.head_dim, p.rope_base);
        cs = m40_rope_cos_sin_freq(position, inv_freq, p.rope_scale);
    }
    rows_stage(xr, true, p.norm_dtype, p.eps, (int)p.rows, K, a_lds, wave_sums);
    float acc[kCols][kRows];
    rows_dot(regs, a_lds, K, lane, acc);
    if (!e_live || position >= p.max_seq_len || seq >= p.max_batch) return;
    float y0 = rows_pick(acc, 2 * e_q, e_row), y1 = rows_pick(acc, 2 * e_q + 1, e_row);
    if (bias) { y0 = y0 + b0; y1 = y1 + b1; }
    if (e_which != 2) m40_rope_apply(cs, y0, y1, &y0, &y1);
    if (e_which == 0) {
        float* q = p.q_out + (size_t)e_row * p.q_heads * p.head_dim;
        q[e_i0] = y0;
        q[e_i1] = y1;
    } else {
        const size_t ept = (size_t)p.kv_heads * p.head_dim;
        uint16_t* dst = (e_which == 1 ? p.k_cache : p.v_cache) + ((size_t)seq * p.max_seq_len + position) * ept;
        dst[e_i0] = m40_f2h(y0);
        dst[e_i1] = m40_f2h(y1);
        if (e_which == 1 && e_local == 0) p.seq_map[seq] = position + 1u;
    }
}

}  // namespace

bool m40_rows_gemv_supported(int rows, int K) {
    return rows >= 1 && rows <= kRows && K >= 8 && K <= kMaxK && K % 8 == 0;
}

int m40_rows_gemv_residual(hipStream_t stream, const float* a, const uint16_t* W, const float* residual, float* out,
                           int rows, int N, int K) {
    if (!m40_rows_gemv_supported(rows, K) || !m40_aligned16(a) || !m40_aligned16(W)) return -6;
    const int blocks = (N + kWaves * kCols - 1) / (kWaves * kCols);
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(rows_gemv_residual_kernel),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, kRows * kMaxK * 4);
    if (attr != hipSuccess) return -7;
    rows_gemv_residual_kernel<<<blocks, kThreads, (size_t)kRows * K * sizeof(float), stream>>>(a, W, residual, out, rows, N, K);
    return hipGetLastError() == hipSuccess ? 0 : -7;
}

int m40_rows_norm_qkv(M40llmCudaContext* ctx, hipStream_t stream, const M40llmKVCache* kv, const uint32_t* ids_dev, const uint32_t* lens_dev,
                      uint32_t rows, const float* x, const void* norm_w, uint32_t norm_dtype, float eps,
                      const uint16_t* wq, const uint16_t* wk, const uint16_t* wv, const float* bq, const float* bk,
                      const float* bv, uint32_t d_model, uint32_t q_heads, float rope_base, float rope_scale,
                      uint32_t rope_layout, float* q_out) {
    if (!m40_rows_gemv_supported((int)rows, (int)d_model) || !m40_aligned16(x) || !m40_aligned16(norm_w) ||
        !m40_aligned16(wq) || !m40_aligned16(wk) || !m40_aligned16(wv))
        return -6;
    RowsQkvArgs p{};
    p.x = x; p.norm_w = norm_w; p.wq = wq; p.wk = wk; p.wv = wv; p.bq = bq; p.bk = bk; p.bv = bv;
    p.q_out = q_out; p.k_cache = kv->d_k; p.v_cache = kv->d_v; p.seq_map = kv->d_seq_map;
    p.ids_dev = ids_dev; p.lens_dev = lens_dev;
    p.rows = rows; p.d_model = d_model; p.max_seq_len = kv->max_seq_len; p.max_batch = kv->max_batch_size;
    p.q_heads = q_heads; p.kv_heads = kv->num_heads; p.head_dim = kv->head_dim; p.rope_layout = rope_layout;
    p.norm_dtype = norm_dtype; p.eps = eps; p.rope_base = rope_base; p.rope_scale = rope_scale;
    p.rope_table = m40_rope_inv_freq_table(ctx, 1, stream, kv->head_dim, rope_base);
    const uint32_t pairs = (q_heads + 2u * kv->num_heads) * (kv->head_dim / 2u);
    const uint32_t blocks = (pairs + (kCols / 2) * kWaves - 1u) / ((kCols / 2) * kWaves);
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(rows_norm_qkv_kernel),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, kRows * kMaxK * 4);
    if (attr != hipSuccess) return -7;
    rows_norm_qkv_kernel<<<blocks, kThreads, (size_t)kRows * d_model * sizeof(float), stream>>>(p);
    return hipGetLastError() == hipSuccess ? 0 : -7;
}
