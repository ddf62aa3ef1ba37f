// RMSNorm, RoPE, SwiGLU, residual add, dtype casts, q8_0 dequant and argmax for gfx950.
// Reference semantics: cuda/kernels.cu:736-891 (kernels), :1036-1241 and :7370-7546 (entry points).
#include "common.hpp"

namespace {

constexpr int kThreads = 256;

// ---- RMSNorm: one workgroup per row ------------------------------------------------
// y = x * scale * w, scale = 1/sqrt(sum(x^2)/dim + eps)   (kernels.cu:764-766, :800-805)
template <bool WEIGHTED>
__global__ __launch_bounds__(kThreads) void rms_norm_kernel(const float* __restrict__ in,
                                                            const void* __restrict__ weight,
                                                            float* __restrict__ out, uint32_t rows,
                                                            uint32_t dim, float eps,
                                                            uint32_t weight_dtype) {
    __shared__ float wave_sums[kThreads / 64];
    const uint32_t row = blockIdx.x;
    if (row >= rows) return;
    const float* x = in + (size_t)row * dim;
    float* y = out + (size_t)row * dim;
    const uint32_t tid = threadIdx.x;
    const bool vec = (dim % 4u == 0u) && m40_aligned16(x) && m40_aligned16(y);

    float ss = 0.0f;
    if (vec) {
        const float4* x4 = reinterpret_cast<const float4*>(x);
        for (uint32_t i = tid; i < dim / 4u; i += kThreads) {
            const float4 v = x4[i];
            ss = fmaf(v.x, v.x, ss);
            ss = fmaf(v.y, v.y, ss);
            ss = fmaf(v.z, v.z, ss);
            ss = fmaf(v.w, v.w, ss);
        }
    } else {
        for (uint32_t i = tid; i < dim; i += kThreads) ss += x[i] * x[i];
    }
    ss = m40_sum64(ss);
    if ((tid & 63u) == 0u) wave_sums[tid >> 6] = ss;
    __syncthreads();
    float total = 0.0f;
#pragma unroll
    for (int w = 0; w < kThreads / 64; ++w) total += wave_sums[w];
    const float scale = 1.0f / sqrtf(total / static_cast<float>(dim) + eps);

    const uint16_t* w16 = reinterpret_cast<const uint16_t*>(weight);
    const float* w32 = reinterpret_cast<const float*>(weight);
    if (vec && (!WEIGHTED || (weight_dtype == 0u ? (reinterpret_cast<uintptr_t>(weight) & 7u) == 0 : m40_aligned16(weight)))) {
        // four elements per access (the same operations per element as the scalar form)
        const float4* x4 = reinterpret_cast<const float4*>(x);
        float4* y4 = reinterpret_cast<float4*>(y);
        for (uint32_t i = tid; i < dim / 4u; i += kThreads) {
            const float4 a = x4[i];
            float v[4] = {a.x * scale, a.y * scale, a.z * scale, a.w * scale};
            if (WEIGHTED) {
                if (weight_dtype == 0u) {
                    const uint2 h = reinterpret_cast<const uint2*>(w16)[i];
                    v[0] *= m40_h2f(static_cast<uint16_t>(h.x & 0xffffu)); v[1] *= m40_h2f(static_cast<uint16_t>(h.x >> 16));
                    v[2] *= m40_h2f(static_cast<uint16_t>(h.y & 0xffffu)); v[3] *= m40_h2f(static_cast<uint16_t>(h.y >> 16));
                } else {
                    const float4 w = reinterpret_cast<const float4*>(w32)[i];
                    v[0] *= w.x; v[1] *= w.y; v[2] *= w.z; v[3] *= w.w;
                }
            }
            y4[i] = make_float4(v[0], v[1], v[2], v[3]);
        }
        return;
    }
    for (uint32_t i = tid; i < dim; i += kThreads) {
        float v = x[i] * scale;
        if (WEIGHTED) v = v * (weight_dtype == 0u ? m40_h2f(w16[i]) : w32[i]);
        y[i] = v;
    }
}

// ---- RoPE ----------------------------------------------------------------------------
// One thread per rotated pair.  position = past_len (+ row), or *past_len_dev when given.
__global__ __launch_bounds__(kThreads) void rope_kernel(float* __restrict__ a, float* __restrict__ b,
                                                        uint32_t rows, uint32_t num_heads,
                                                        uint32_t head_dim, uint32_t past_len,
                                                        const uint32_t* __restrict__ past_len_dev,
                                                        float freq_base, float freq_scale,
                                                        uint32_t layout) {
    const uint32_t pairs_per_row = (num_heads * head_dim) / 2u;
    const uint32_t total = rows * pairs_per_row;
    const uint32_t idx = blockIdx.x * kThreads + threadIdx.x;
    if (idx >= total) return;
    if (past_len_dev) past_len = *past_len_dev;
    const uint32_t row = idx / pairs_per_row;
    const uint32_t pair = idx % pairs_per_row;
    const uint32_t head = pair / (head_dim / 2u);
    const uint32_t off = pair % (head_dim / 2u);
    size_t i0, i1;
    m40_rope_pair(head, off, head_dim, layout, &i0, &i1);
    const size_t base = (size_t)row * num_heads * head_dim;
    float y0, y1;
    m40_rope_rotate(past_len + row, off, head_dim, freq_base, freq_scale, a[base + i0], a[base + i1], &y0, &y1);
    a[base + i0] = y0;
    a[base + i1] = y1;
    if (b) {
        m40_rope_rotate(past_len + row, off, head_dim, freq_base, freq_scale, b[base + i0], b[base + i1], &y0, &y1);
        b[base + i0] = y0;
        b[base + i1] = y1;
    }
}

// Element-wise kernels over large arrays (the prefill's residual adds and SwiGLU: tens of MB per call): 16 bytes per lane
// and access, four accesses in flight per thread; `out` may be one of the inputs (same index read, then written).  The
// scalar form serves unaligned arrays and the last n % 4 elements.
__global__ __launch_bounds__(kThreads) void residual_add_kernel(const float* a, const float* b, float* out, size_t n) {
    const size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x;
    if (i < n) out[i] = a[i] + b[i];
}

__global__ __launch_bounds__(kThreads) void residual_add4_kernel(const float4* a, const float4* b, float4* out, size_t n4) {
    for (size_t base = (size_t)blockIdx.x * (4 * kThreads) + threadIdx.x; base < n4; base += (size_t)gridDim.x * (4 * kThreads)) {
        float4 x[4], y[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const size_t i = base + (size_t)u * kThreads;
            if (i < n4) { x[u] = a[i]; y[u] = b[i]; }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const size_t i = base + (size_t)u * kThreads;
            if (i < n4) out[i] = make_float4(x[u].x + y[u].x, x[u].y + y[u].y, x[u].z + y[u].z, x[u].w + y[u].w);
        }
    }
}

__device__ __forceinline__ float swiglu_one(float g, float u) {
    const float silu = g / (1.0f + expf(-g));
    return silu * u;
}

__global__ __launch_bounds__(kThreads) void swiglu_kernel(const float* gate, const float* up, float* out, size_t n) {
    const size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x;
    if (i < n) out[i] = swiglu_one(gate[i], up[i]);
}

__global__ __launch_bounds__(kThreads) void swiglu4_kernel(const float4* gate, const float4* up, float4* out, size_t n4) {
    for (size_t base = (size_t)blockIdx.x * (4 * kThreads) + threadIdx.x; base < n4; base += (size_t)gridDim.x * (4 * kThreads)) {
        float4 g[4], v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const size_t i = base + (size_t)u * kThreads;
            if (i < n4) { g[u] = gate[i]; v[u] = up[i]; }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const size_t i = base + (size_t)u * kThreads;
            if (i < n4)
                out[i] = make_float4(swiglu_one(g[u].x, v[u].x), swiglu_one(g[u].y, v[u].y), swiglu_one(g[u].z, v[u].z),
                                     swiglu_one(g[u].w, v[u].w));
        }
    }
}

__global__ __launch_bounds__(kThreads) void f16_to_f32_kernel(const uint16_t* __restrict__ in,
                                                              float* __restrict__ out, size_t n) {
    const size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x;
    if (i < n) out[i] = m40_h2f(in[i]);
}

// q8_0 block = { f16 d; int8 qs[32] }, 34 bytes   (kernels.cu:856-867)
__global__ __launch_bounds__(kThreads) void q80_to_f32_kernel(const uint8_t* __restrict__ in,
                                                              float* __restrict__ out, size_t n) {
    const size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x;
    if (i < n) {
        const size_t blk = i / 32, idx = i % 32;
        const uint8_t* base = in + blk * 34;
        const uint16_t dh = (uint16_t)base[0] | ((uint16_t)base[1] << 8);
        const int8_t q = static_cast<int8_t>(base[2 + idx]);
        out[i] = m40_h2f(dh) * static_cast<float>(q);
    }
}

// ---- argmax: first index of the row maximum, plus the top-1/top-2 gap -----------------
struct Top2 {
    float a;      // largest
    float b;      // second largest
    uint32_t ia;  // index of the first occurrence of a
};
__device__ __forceinline__ Top2 top2_merge(const Top2& x, const Top2& y) {
    Top2 r;
    if (x.a > y.a || (x.a == y.a && x.ia < y.ia)) {
        r.a = x.a; r.ia = x.ia;
        r.b = fmaxf(x.b, y.a);
    } else {
        r.a = y.a; r.ia = y.ia;
        r.b = fmaxf(y.b, x.a);
    }
    return r;
}

__global__ __launch_bounds__(1024) void argmax_kernel(const float* __restrict__ logits, size_t n,
                                                      uint32_t* __restrict__ out_idx,
                                                      float* __restrict__ out_gap) {
    __shared__ float sa[16], sb[16];
    __shared__ uint32_t si[16];
    const float* x = logits + (size_t)blockIdx.x * n;
    Top2 t{-INFINITY, -INFINITY, 0xffffffffu};
    for (size_t i = threadIdx.x; i < n; i += blockDim.x) {
        const float v = x[i];
        if (v > t.a) { t.b = t.a; t.a = v; t.ia = (uint32_t)i; }
        else if (v > t.b) t.b = v;
    }
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        Top2 u;
        u.a = __shfl_xor(t.a, o, 64);
        u.b = __shfl_xor(t.b, o, 64);
        u.ia = __shfl_xor(t.ia, o, 64);
        t = top2_merge(t, u);
    }
    const uint32_t wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63u) == 0u) { sa[wave] = t.a; sb[wave] = t.b; si[wave] = t.ia; }
    __syncthreads();
    if (threadIdx.x == 0) {
        Top2 r{sa[0], sb[0], si[0]};
        for (uint32_t w = 1; w < blockDim.x / 64u; ++w) r = top2_merge(r, Top2{sa[w], sb[w], si[w]});
        out_idx[blockIdx.x] = r.ia == 0xffffffffu ? 0u : r.ia;
        if (out_gap) out_gap[blockIdx.x] = r.a - r.b;
    }
}

// Reads n16 16-byte words and folds them into one word per workgroup: the plain HBM read stream of one launch, as a
// yardstick for the bandwidth-bound kernels (nothing else is computed).  A workgroup owns a contiguous range and
// walks it with four streaming loads per thread in flight, like a wave of the GEMV walks its columns.
__global__ __launch_bounds__(256) void read_probe_kernel(const uint4* __restrict__ src, size_t n16, uint32_t* __restrict__ out) {
    const size_t per = (n16 + gridDim.x - 1) / gridDim.x;
    const size_t begin = (size_t)blockIdx.x * per;
    const size_t end = begin + per < n16 ? begin + per : n16;
    uint32_t acc = 0u;
    for (size_t base = begin + threadIdx.x; base < end; base += 4u * 256u) {
        uint4 v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const size_t i = base + (size_t)u * 256u;
            v[u] = m40_load_stream(src + (i < end ? i : base));
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const uint32_t w = v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
            acc ^= base + (size_t)u * 256u < end ? w : 0u;         // a stand-in load past the end does not count
        }
    }
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) acc ^= (uint32_t)__shfl_xor((int)acc, o, 64);
    if ((threadIdx.x & 63u) == 0u) atomicXor(&out[blockIdx.x & 2047u], acc);
}

inline int blocks_for(size_t n) { return (int)((n + kThreads - 1) / kThreads); }
// workgroups of the 16-byte forms: one pass of four accesses per thread, at most 8192 workgroups (then they loop)
inline int wide_blocks_for(size_t n4) {
    const size_t groups = (n4 + 4 * kThreads - 1) / (4 * kThreads);
    return (int)(groups < 8192 ? groups : 8192);
}

}  // namespace

extern "C" {

int m40llm_rms_norm_f32_async(M40llmCudaContext* ctx, const void* d_in, void* d_out, uint32_t rows,
                              uint32_t dim, float eps) {
    if (!ctx || !d_in || !d_out || dim == 0) return -1;
    if (rows == 0) return 0;
    (void)hipGetLastError();
    rms_norm_kernel<false><<<rows, kThreads, 0, ctx->decode_stream>>>(
        static_cast<const float*>(d_in), nullptr, static_cast<float*>(d_out), rows, dim, eps, 1u);
    return hipGetLastError() == hipSuccess ? 0 : -2;
}

int m40llm_rms_norm_f32(M40llmCudaContext* ctx, const void* d_in, void* d_out, uint32_t rows,
                        uint32_t dim, float eps) {
    int rc = m40llm_rms_norm_f32_async(ctx, d_in, d_out, rows, dim, eps);
    if (rc != 0) return rc;
    return hipStreamSynchronize(ctx->decode_stream) == hipSuccess ? 0 : -3;
}

int m40llm_rms_norm_f32_weighted_async(M40llmCudaContext* ctx, const void* d_in, const void* d_weight,
                                       void* d_out, uint32_t rows, uint32_t dim, float eps,
                                       uint32_t weight_dtype) {
    if (!ctx || !d_in || !d_weight || !d_out || dim == 0) return -1;
    if (weight_dtype > 1) return -4;
    if (rows == 0) return 0;
    (void)hipGetLastError();
    rms_norm_kernel<true><<<rows, kThreads, 0, ctx->decode_stream>>>(
        static_cast<const float*>(d_in), d_weight, static_cast<float*>(d_out), rows, dim, eps, weight_dtype);
    return hipGetLastError() == hipSuccess ? 0 : -2;
}

int m40llm_rms_norm_f32_weighted(M40llmCudaContext* ctx, const void* d_in, const void* d_weight,
                                 void* d_out, uint32_t rows, uint32_t dim, float eps,
                                 uint32_t weight_dtype) {
    int rc = m40llm_rms_norm_f32_weighted_async(ctx, d_in, d_weight, d_out, rows, dim, eps, weight_dtype);
    if (rc != 0) return rc;
    return hipStreamSynchronize(ctx->decode_stream) == hipSuccess ? 0 : -3;
}

static int rope_launch(M40llmCudaContext* ctx, float* a, float* b, uint32_t rows, uint32_t num_heads,
                       uint32_t head_dim, uint32_t past_len, const uint32_t* past_len_dev,
                       float freq_base, float freq_scale, uint32_t layout) {
    const uint32_t total_pairs = rows * ((num_heads * head_dim) / 2u);
    if (total_pairs == 0) return 0;
    (void)hipGetLastError();
    rope_kernel<<<blocks_for(total_pairs), kThreads, 0, ctx->decode_stream>>>(
        a, b, rows, num_heads, head_dim, past_len, past_len_dev, freq_base, freq_scale, layout);
    return hipGetLastError() == hipSuccess ? 0 : -3;
}

int m40llm_rope_f32_layout_async(M40llmCudaContext* ctx, void* d_q, void* d_k, uint32_t rows,
                                 uint32_t num_heads, uint32_t head_dim, uint32_t past_len,
                                 float freq_base, float freq_scale, uint32_t rope_layout) {
    if (!ctx || !d_q || !d_k || head_dim == 0 || num_heads == 0) return -1;
    if (head_dim % 2 != 0) return -2;
    return rope_launch(ctx, static_cast<float*>(d_q), static_cast<float*>(d_k), rows, num_heads, head_dim,
                       past_len, nullptr, freq_base, freq_scale, rope_layout);
}

int m40llm_rope_f32_async(M40llmCudaContext* ctx, void* d_q, void* d_k, uint32_t rows,
                          uint32_t num_heads, uint32_t head_dim, uint32_t past_len, float freq_base,
                          float freq_scale) {
    return m40llm_rope_f32_layout_async(ctx, d_q, d_k, rows, num_heads, head_dim, past_len, freq_base,
                                        freq_scale, M40LLM_ROPE_LAYOUT_ADJACENT);
}

int m40llm_rope_f32(M40llmCudaContext* ctx, void* d_q, void* d_k, uint32_t rows, uint32_t num_heads,
                    uint32_t head_dim, uint32_t past_len, float freq_base, float freq_scale) {
    int rc = m40llm_rope_f32_async(ctx, d_q, d_k, rows, num_heads, head_dim, past_len, freq_base, freq_scale);
    if (rc != 0) return rc;
    return hipStreamSynchronize(ctx->decode_stream) == hipSuccess ? 0 : -4;
}

int m40llm_rope_f32_inplace_layout_async(M40llmCudaContext* ctx, void* d_x, uint32_t rows,
                                         uint32_t num_heads, uint32_t head_dim, uint32_t past_len,
                                         float freq_base, float freq_scale, uint32_t rope_layout) {
    if (!ctx || !d_x || head_dim == 0 || num_heads == 0) return -1;
    if (head_dim % 2 != 0) return -2;
    return rope_launch(ctx, static_cast<float*>(d_x), nullptr, rows, num_heads, head_dim, past_len, nullptr,
                       freq_base, freq_scale, rope_layout);
}

int m40llm_rope_f32_inplace_async(M40llmCudaContext* ctx, void* d_x, uint32_t rows,
                                  uint32_t num_heads, uint32_t head_dim, uint32_t past_len,
                                  float freq_base, float freq_scale) {
    return m40llm_rope_f32_inplace_layout_async(ctx, d_x, rows, num_heads, head_dim, past_len, freq_base,
                                                freq_scale, M40LLM_ROPE_LAYOUT_ADJACENT);
}

int m40llm_rope_f32_inplace(M40llmCudaContext* ctx, void* d_x, uint32_t rows, uint32_t num_heads,
                            uint32_t head_dim, uint32_t past_len, float freq_base, float freq_scale) {
    int rc = m40llm_rope_f32_inplace_async(ctx, d_x, rows, num_heads, head_dim, past_len, freq_base, freq_scale);
    if (rc != 0) return rc;
    return hipStreamSynchronize(ctx->decode_stream) == hipSuccess ? 0 : -4;
}

int m40llm_rope_f32_inplace_position_dev_layout_async(M40llmCudaContext* ctx, void* d_x, uint32_t rows,
                                                      uint32_t num_heads, uint32_t head_dim,
                                                      const uint32_t* past_len_dev, float freq_base,
                                                      float freq_scale, uint32_t rope_layout) {
    if (!ctx || !d_x || !past_len_dev || head_dim == 0 || num_heads == 0) return -1;
    if (head_dim % 2 != 0) return -2;
    return rope_launch(ctx, static_cast<float*>(d_x), nullptr, rows, num_heads, head_dim, 0, past_len_dev,
                       freq_base, freq_scale, rope_layout);
}

int m40llm_rope_f32_inplace_position_dev_async(M40llmCudaContext* ctx, void* d_x, uint32_t rows,
                                               uint32_t num_heads, uint32_t head_dim,
                                               const uint32_t* past_len_dev, float freq_base,
                                               float freq_scale) {
    return m40llm_rope_f32_inplace_position_dev_layout_async(ctx, d_x, rows, num_heads, head_dim,
                                                             past_len_dev, freq_base, freq_scale,
                                                             M40LLM_ROPE_LAYOUT_ADJACENT);
}

int m40llm_residual_add_f32_async(M40llmCudaContext* ctx, const void* d_a, const void* d_b, void* d_out,
                                  size_t n) {
    if (!ctx || !d_a || !d_b || !d_out) return -1;
    if (m40_ensure_device(ctx) != 0) return -2;
    if (n == 0) return 0;
    (void)hipGetLastError();
    const float* a = static_cast<const float*>(d_a);
    const float* b = static_cast<const float*>(d_b);
    float* out = static_cast<float*>(d_out);
    size_t done = 0;
    if (n >= 4096 && m40_aligned16(a) && m40_aligned16(b) && m40_aligned16(out)) {
        const size_t n4 = n / 4;
        residual_add4_kernel<<<wide_blocks_for(n4), kThreads, 0, ctx->decode_stream>>>(
            reinterpret_cast<const float4*>(a), reinterpret_cast<const float4*>(b), reinterpret_cast<float4*>(out), n4);
        done = 4 * n4;
    }
    if (done < n)
        residual_add_kernel<<<blocks_for(n - done), kThreads, 0, ctx->decode_stream>>>(a + done, b + done, out + done, n - done);
    return hipGetLastError() == hipSuccess ? 0 : -3;
}

int m40llm_residual_add_f32(M40llmCudaContext* ctx, const void* d_a, const void* d_b, void* d_out, size_t n) {
    int rc = m40llm_residual_add_f32_async(ctx, d_a, d_b, d_out, n);
    if (rc != 0) return rc;
    return hipStreamSynchronize(ctx->decode_stream) == hipSuccess ? 0 : -4;
}

int m40llm_swiglu_f32_async(M40llmCudaContext* ctx, const void* d_gate, const void* d_up, void* d_out,
                            size_t n) {
    if (!ctx || !d_gate || !d_up || !d_out) return -1;
    if (m40_ensure_device(ctx) != 0) return -2;
    if (n == 0) return 0;
    (void)hipGetLastError();
    const float* gate = static_cast<const float*>(d_gate);
    const float* up = static_cast<const float*>(d_up);
    float* out = static_cast<float*>(d_out);
    size_t done = 0;
    if (n >= 4096 && m40_aligned16(gate) && m40_aligned16(up) && m40_aligned16(out)) {
        const size_t n4 = n / 4;
        swiglu4_kernel<<<wide_blocks_for(n4), kThreads, 0, ctx->decode_stream>>>(
            reinterpret_cast<const float4*>(gate), reinterpret_cast<const float4*>(up), reinterpret_cast<float4*>(out), n4);
        done = 4 * n4;
    }
    if (done < n)
        swiglu_kernel<<<blocks_for(n - done), kThreads, 0, ctx->decode_stream>>>(gate + done, up + done, out + done, n - done);
    return hipGetLastError() == hipSuccess ? 0 : -3;
}

int m40llm_swiglu_f32(M40llmCudaContext* ctx, const void* d_gate, const void* d_up, void* d_out, size_t n) {
    int rc = m40llm_swiglu_f32_async(ctx, d_gate, d_up, d_out, n);
    if (rc != 0) return rc;
    return hipStreamSynchronize(ctx->decode_stream) == hipSuccess ? 0 : -4;
}

int m40llm_f16_to_f32(M40llmCudaContext* ctx, const void* d_in_f16, void* d_out_f32, size_t n) {
    if (!ctx || !d_in_f16 || !d_out_f32) return -1;
    if (m40_ensure_device(ctx) != 0) return -4;
    (void)hipGetLastError();
    hipPointerAttribute_t attr;
    if (hipPointerGetAttributes(&attr, d_in_f16) != hipSuccess) {
        (void)hipGetLastError();
        return -2;
    }
    if (reinterpret_cast<uintptr_t>(d_in_f16) % 2u != 0) return -3;
    if (n == 0) return 0;
    f16_to_f32_kernel<<<blocks_for(n), kThreads, 0, ctx->prefill_stream>>>(
        static_cast<const uint16_t*>(d_in_f16), static_cast<float*>(d_out_f32), n);
    if (hipGetLastError() != hipSuccess) return -2;
    return hipStreamSynchronize(ctx->prefill_stream) == hipSuccess ? 0 : -3;
}

int m40llm_q80_to_f32(M40llmCudaContext* ctx, const void* d_in_q80, void* d_out_f32, size_t n) {
    if (!ctx || !d_in_q80 || !d_out_f32) return -1;
    if (n == 0) return 0;
    (void)hipGetLastError();
    q80_to_f32_kernel<<<blocks_for(n), kThreads, 0, ctx->prefill_stream>>>(
        static_cast<const uint8_t*>(d_in_q80), static_cast<float*>(d_out_f32), n);
    if (hipGetLastError() != hipSuccess) return -2;
    return hipStreamSynchronize(ctx->prefill_stream) == hipSuccess ? 0 : -3;
}

int m40llm_ext_argmax_f32_async(M40llmCudaContext* ctx, const void* d_logits_f32, uint32_t rows, size_t n,
                                uint32_t* out_idx_dev, float* out_gap_dev) {
    if (!ctx || !d_logits_f32 || !out_idx_dev) return -1;
    if (rows == 0 || n == 0) return -2;
    (void)hipGetLastError();
    argmax_kernel<<<rows, 1024, 0, ctx->decode_stream>>>(static_cast<const float*>(d_logits_f32), n,
                                                         out_idx_dev, out_gap_dev);
    return hipGetLastError() == hipSuccess ? 0 : -3;
}

int m40llm_ext_read_probe_async(M40llmCudaContext* ctx, const void* d_src, size_t bytes, uint32_t workgroups,
                                uint32_t* d_out_u32) {
    if (!ctx || !d_src || !d_out_u32) return -1;
    if (bytes < 16 || workgroups == 0 || workgroups > 65536u || (reinterpret_cast<uintptr_t>(d_src) & 15u) != 0u) return -2;
    (void)hipGetLastError();
    read_probe_kernel<<<workgroups, 256, 0, ctx->decode_stream>>>(static_cast<const uint4*>(d_src), bytes / 16, d_out_u32);
    return hipGetLastError() == hipSuccess ? 0 : -3;
}

}  // extern "C"
