// Fused batch-1 decode-step kernels for gfx950 (no counterpart in the reference, which issues one
// launch per primitive op).  Each kernel streams f16 GGUF-layout weights exactly once with 128-bit
// loads, keeps the activation vector in LDS, and folds the neighbouring elementwise ops into the
// GEMV prologue / epilogue:
//
//   norm_qkv_rope_append : RMSNorm(x) -> Q,K,V projections (+bias) -> RoPE(Q) -> q_out,
//                          RoPE(K) -> f16 K append, f16 V append                      (steps 1-5)
//   gemv_residual        : out = residual + W . a                                     (steps 7-8, 12-13)
//   norm_gate_up_swiglu  : RMSNorm(x) -> gate, up projections -> silu(gate) * up      (steps 9-11)
//   norm_gemv            : RMSNorm(x) -> W . xn                                       (output norm + lm_head)
//   embed_token_dev / greedy_step : device-side token feedback so consecutive tokens need no host round trip
//
// The arithmetic of every output element follows the unfused kernels operation for operation
// (same reduction order for the norm, same lane->k mapping and FMA chain for the dot products, the
// shared RoPE rotation), so this path and the reference call sequence produce identical bits.
// Step numbers refer to the reference's per-layer call order, src/infer/forward.rs:304-662.
#include "common.hpp"
#include "gemv_core.hpp"

namespace {

constexpr int kThreads = 256;
constexpr int kWavesPerBlock = 4;

// x -> LDS as normalised activations: a[k] = x[k] * scale * w[k], scale = 1/sqrt(sum(x^2)/K + eps).
// Reduction order identical to rms_norm_kernel (elementwise.hip).
//
// In two halves so that the caller can request x and the norm weights first, then the GEMV weights, and only then
// wait: loads return in issue order, so x arrives ahead of the weight stream and the whole prologue (sum of squares,
// scaling, LDS, two barriers) runs while the weights are still in flight.  A batch is four 16-byte loads per thread
// and array (K <= 4096 in one batch); longer rows take further batches inside stage_finish.
constexpr int kStageBatch = 4;
struct StageRegs {
    float4 x[kStageBatch];
    uint4 w[kStageBatch];      // raw bits: four f32 norm weights, or four f16 in .x/.y
};

__device__ __forceinline__ void stage_load(const float* __restrict__ x, const void* __restrict__ w, uint32_t w_dtype,
                                           int K, int batch, StageRegs& r) {
    const int n4 = K >> 2;
    int idx[kStageBatch];
#pragma unroll
    for (int u = 0; u < kStageBatch; ++u) {
        const int i = (batch * kStageBatch + u) * kThreads + (int)threadIdx.x;
        idx[u] = i < n4 ? i : 0;                 // past the end: a valid address, ignored later (no load under a branch)
    }
#pragma unroll
    for (int u = 0; u < kStageBatch; ++u) r.x[u] = reinterpret_cast<const float4*>(x)[idx[u]];
    // One unconditional batch whatever the weights' type: a branch around loads makes the compiler wait for every
    // load in flight at its join (the rows above).  f32: 16 bytes per index as two halves; f16: 8 bytes, asked for twice.
    const char* wb = static_cast<const char*>(w);
    const int stride = w_dtype == 0u ? 8 : 16, hi_off = w_dtype == 0u ? 0 : 8;
#pragma unroll
    for (int u = 0; u < kStageBatch; ++u) {
        const uint2 lo = *reinterpret_cast<const uint2*>(wb + (size_t)idx[u] * stride);
        const uint2 hi = *reinterpret_cast<const uint2*>(wb + (size_t)idx[u] * stride + hi_off);
        r.w[u].x = lo.x; r.w[u].y = lo.y; r.w[u].z = hi.x; r.w[u].w = hi.y;
    }
}

__device__ __forceinline__ void stage_sumsq(const StageRegs& r, int K, int batch, float& ss) {
    const int n4 = K >> 2;
#pragma unroll
    for (int u = 0; u < kStageBatch; ++u) {
        const int i = (batch * kStageBatch + u) * kThreads + (int)threadIdx.x;
        if (i < n4) {
            ss = fmaf(r.x[u].x, r.x[u].x, ss);
            ss = fmaf(r.x[u].y, r.x[u].y, ss);
            ss = fmaf(r.x[u].z, r.x[u].z, ss);
            ss = fmaf(r.x[u].w, r.x[u].w, ss);
        }
    }
}

__device__ __forceinline__ void stage_store(const StageRegs& r, uint32_t w_dtype, int K, int batch, float scale,
                                            float* __restrict__ a_lds) {
    const int n4 = K >> 2;
#pragma unroll
    for (int u = 0; u < kStageBatch; ++u) {
        const int i = (batch * kStageBatch + u) * kThreads + (int)threadIdx.x;
        if (i < n4) {
            float4 wv = make_float4(__uint_as_float(r.w[u].x), __uint_as_float(r.w[u].y), __uint_as_float(r.w[u].z),
                                    __uint_as_float(r.w[u].w));
            if (w_dtype == 0u) {
                const uint32_t h0 = r.w[u].x, h1 = r.w[u].y;
                wv = make_float4(m40_h2f((uint16_t)(h0 & 0xffffu)), m40_h2f((uint16_t)(h0 >> 16)),
                                 m40_h2f((uint16_t)(h1 & 0xffffu)), m40_h2f((uint16_t)(h1 >> 16)));
            }
            reinterpret_cast<float4*>(a_lds)[i] = make_float4(r.x[u].x * scale * wv.x, r.x[u].y * scale * wv.y,
                                                              r.x[u].z * scale * wv.z, r.x[u].w * scale * wv.w);
        }
    }
}

// `first` holds batch 0, loaded by the caller before its weight prefetch.
__device__ __forceinline__ void stage_finish(const StageRegs& first, const float* __restrict__ x,
                                             const void* __restrict__ w, uint32_t w_dtype, float eps, int K,
                                             float* __restrict__ a_lds, float* __restrict__ wave_sums) {
    const int tid = threadIdx.x;
    const int nbatch = ((K >> 2) + kStageBatch * kThreads - 1) / (kStageBatch * kThreads);
    float ss = 0.0f;
    stage_sumsq(first, K, 0, ss);
    if (nbatch > 1) {       // rows longer than one batch: kept apart so that the usual case has no loop with loads in it
        for (int b = 1; b < nbatch; ++b) {
            StageRegs r;
            stage_load(x, w, w_dtype, K, b, r);
            stage_sumsq(r, K, b, ss);
        }
    }
    ss = m40_sum64(ss);
    if ((tid & 63) == 0) wave_sums[tid >> 6] = ss;
    __syncthreads();
    float total = 0.0f;
#pragma unroll
    for (int i = 0; i < kWavesPerBlock; ++i) total += wave_sums[i];
    const float scale = 1.0f / sqrtf(total / static_cast<float>(K) + eps);
    stage_store(first, w_dtype, K, 0, scale, a_lds);
    if (nbatch > 1) {
        for (int b = 1; b < nbatch; ++b) {
            StageRegs r;
            stage_load(x, w, w_dtype, K, b, r);
            stage_store(r, w_dtype, K, b, scale, a_lds);
        }
    }
    __syncthreads();
}

struct QkvArgs {
    const float* x;
    const void* norm_w;
    const uint16_t *wq, *wk, *wv;
    const float *bq, *bk, *bv;
    float* q_out;
    uint16_t* k_cache;   // base of this slot: [max_seq_len][kvh][hd]
    uint16_t* v_cache;
    uint32_t* seq_map_entry;
    const uint32_t* position_dev;
    const float* rope_table;   // pair frequencies of (head_dim, rope_base), or null: the kernel evaluates the power
    float4* rope_cs;           // with rope_table: {position bits, cos, sin, tag of (position, scale)} per pair, kept from launch to launch
    uint32_t position, max_seq_len;
    uint32_t d_model, q_heads, kv_heads, head_dim, rope_layout, norm_dtype;
    float eps, rope_base, rope_scale;
};

// One wave per PAIRS consecutive rotation pairs (two output columns each).  Pair space: Q pairs, then K pairs, then
// V pairs.
template <int PAIRS>
__global__ __launch_bounds__(kThreads) void norm_qkv_rope_append_kernel(QkvArgs p) {
    extern __shared__ float a_lds[];
    __shared__ float wave_sums[kWavesPerBlock];
    const int K = (int)p.d_model;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    // x and the norm weights are requested before anything else is computed, then (below) the position and the pair's
    // rotation entry, then the GEMV weights; the norm prologue runs while the weights stream in
    StageRegs xr;
    stage_load(p.x, p.norm_w, p.norm_dtype, K, 0, xr);
    __builtin_amdgcn_sched_barrier(0);
    const uint32_t half = p.head_dim / 2u;
    const uint32_t q_pairs = p.q_heads * half, kv_pairs = p.kv_heads * half;
    const uint32_t pair0 = (blockIdx.x * kWavesPerBlock + wave) * PAIRS;
    bool live[PAIRS];
    int which[PAIRS];       // 0 Q, 1 K, 2 V
    uint32_t local[PAIRS], off[PAIRS];
    size_t i0[PAIRS], i1[PAIRS];
    const uint4* bp[2 * PAIRS];
#pragma unroll
    for (int q = 0; q < PAIRS; ++q) {
        uint32_t pair = pair0 + q;
        live[q] = pair < q_pairs + 2u * kv_pairs;
        if (!live[q]) pair = 0;
        if (pair < q_pairs) { which[q] = 0; local[q] = pair; }
        else if (pair < q_pairs + kv_pairs) { which[q] = 1; local[q] = pair - q_pairs; }
        else { which[q] = 2; local[q] = pair - q_pairs - kv_pairs; }
        const uint32_t head = local[q] / half;
        off[q] = local[q] % half;
        m40_rope_pair(head, off[q], p.head_dim, which[q] == 2 ? M40LLM_ROPE_LAYOUT_ADJACENT : p.rope_layout, &i0[q], &i1[q]);
        const uint16_t* W = which[q] == 0 ? p.wq : (which[q] == 1 ? p.wk : p.wv);
        bp[2 * q] = reinterpret_cast<const uint4*>(W + i0[q] * (size_t)K);
        bp[2 * q + 1] = reinterpret_cast<const uint4*>(W + i1[q] * (size_t)K);
    }
    // position and pair frequencies are requested with x, ahead of the weights.  Unconditionally: a load under a branch
    // costs a wait for everything in flight at the branch's join, which here held the weight requests back until x, the
    // norm weights and the position had arrived.  An absent input reads the first bytes of Wq and is ignored.
    const uint32_t position_loaded = *(p.position_dev ? p.position_dev : reinterpret_cast<const uint32_t*>(p.wq));
    float inv_freq[PAIRS];
    float4 kept[PAIRS];        // the pair's rotation as left by an earlier launch (the step's first layer)
#pragma unroll
    for (int q = 0; q < PAIRS; ++q) {
        inv_freq[q] = *(p.rope_table ? p.rope_table + off[q] : reinterpret_cast<const float*>(p.wq));
        kept[q] = *(p.rope_cs ? p.rope_cs + off[q] : reinterpret_cast<const float4*>(p.wq));
    }
    const uint32_t position = p.position_dev ? position_loaded : p.position;
    __builtin_amdgcn_sched_barrier(0);
    GemvRegs<2 * PAIRS> regs;
    gemv_prefetch<2 * PAIRS>(bp, 0, K >> 3, lane, regs);
    __builtin_amdgcn_sched_barrier(0);
    // the rotation angle does not depend on the data: evaluated while the weights are in flight
    float2 cs[PAIRS];
#pragma unroll
    for (int q = 0; q < PAIRS; ++q) {
        cs[q] = make_float2(1.0f, 0.0f);
        if (which[q] != 2) {
            // The angle depends on the position only: all layers of a step share it.  An entry is 16 bytes, stored and
            // loaded whole; its first word is the position and its last word a tag of (position, scale), so a reader
            // takes cos / sin (the words between them) only when both ends are this step's -- also if a launch that
            // writes the entry (the step's first layer) overlaps its readers and the 16 bytes were not seen as one.
            const uint32_t tag = position ^ __float_as_uint(p.rope_scale) ^ 0x9e3779b9u;
            const bool hit = p.rope_cs && __float_as_uint(kept[q].x) == position && __float_as_uint(kept[q].w) == tag;
            if (hit) {
                cs[q] = make_float2(kept[q].y, kept[q].z);
            } else {
                if (!p.rope_table) inv_freq[q] = m40_rope_inv_freq(off[q], p.head_dim, p.rope_base);      // replaces the ignored bytes
                cs[q] = m40_rope_cos_sin_freq(position, inv_freq[q], p.rope_scale);
                if (p.rope_cs && which[q] == 0 && local[q] < half && lane == 0)      // the waves of q head 0 keep it
                    p.rope_cs[off[q]] = make_float4(__uint_as_float(position), cs[q].x, cs[q].y, __uint_as_float(tag));
            }
        }
    }
    stage_finish(xr, p.x, p.norm_w, p.norm_dtype, p.eps, K, a_lds, wave_sums);
    float d[2 * PAIRS];
    gemv_accumulate<2 * PAIRS>(bp, a_lds, 0, K >> 3, lane, regs, d);
    gemv_finish<2 * PAIRS, 1>(d, nullptr, wave, lane);
    if (lane != 0 || position >= p.max_seq_len) return;
#pragma unroll
    for (int q = 0; q < PAIRS; ++q) {
        if (!live[q]) continue;
        const float* bias = which[q] == 0 ? p.bq : (which[q] == 1 ? p.bk : p.bv);
        float y0 = d[2 * q], y1 = d[2 * q + 1];
        if (bias) { y0 = y0 + bias[i0[q]]; y1 = y1 + bias[i1[q]]; }
        if (which[q] != 2) m40_rope_apply(cs[q], y0, y1, &y0, &y1);
        if (which[q] == 0) {
            p.q_out[i0[q]] = y0;
            p.q_out[i1[q]] = y1;
        } else {
            uint16_t* dst = (which[q] == 1 ? p.k_cache : p.v_cache) + (size_t)position * p.kv_heads * p.head_dim;
            dst[i0[q]] = m40_f2h(y0);
            dst[i1[q]] = m40_f2h(y1);
            if (which[q] == 1 && local[q] == 0) *p.seq_map_entry = position + 1u;
        }
    }
}

// out[n] = residual[n] + W[n] . a      (residual may alias out)
template <int COLS, int KSPLIT>
__global__ __launch_bounds__(kThreads) void gemv_residual_kernel(const float* __restrict__ a,
                                                                 const uint16_t* __restrict__ W,
                                                                 const float* residual, float* out, int N, int K) {
    __shared__ float red[4 * COLS];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int col0 = KSPLIT == 1 ? (blockIdx.x * kWavesPerBlock + wave) * COLS : blockIdx.x * COLS;
    if (col0 >= N) return;
    const uint4* bp[COLS];
#pragma unroll
    for (int c = 0; c < COLS; ++c) bp[c] = reinterpret_cast<const uint4*>(W + (size_t)(col0 + c < N ? col0 + c : N - 1) * K);
    int c_begin, c_end;
    gemv_range<KSPLIT>(K, wave, &c_begin, &c_end);
    // activations and residual first (cache hits), then the weight stream: nothing is requested after the weights
    // (measured: with K split over the waves the early activation loads cost more than they save)
    constexpr bool ACTS = KSPLIT == 1;
    GemvActRegs acts;
    if (ACTS) gemv_prefetch_acts(a, c_begin, c_end, lane, acts);
    float res[COLS];
#pragma unroll
    for (int c = 0; c < COLS; ++c) res[c] = residual ? residual[col0 + c < N ? col0 + c : N - 1] : 0.0f;
    GemvRegs<COLS> regs;
    gemv_prefetch<COLS, KSPLIT != 1>(bp, c_begin, c_end, lane, regs);
    float d[COLS];
    if (ACTS) gemv_accumulate<COLS>(bp, a, c_begin, c_end, lane, regs, acts, d);
    else gemv_accumulate<COLS>(bp, a, c_begin, c_end, lane, regs, d);
    gemv_finish<COLS, KSPLIT>(d, red, wave, lane);
    if (lane == 0 && (KSPLIT == 1 || wave == 0)) {
#pragma unroll
        for (int c = 0; c < COLS; ++c)
            if (col0 + c < N) out[col0 + c] = residual ? res[c] + d[c] : d[c];
    }
}

// hid[j] = silu(Wg[j] . xn) * (Wu[j] . xn),  xn = RMSNorm(x) * w.  A wave owns PAIRS consecutive j (gate and up rows).
template <int PAIRS>
__global__ __launch_bounds__(kThreads) void norm_gate_up_swiglu_kernel(const float* __restrict__ x,
                                                                       const void* __restrict__ norm_w,
                                                                       uint32_t norm_dtype, float eps,
                                                                       const uint16_t* __restrict__ Wg,
                                                                       const uint16_t* __restrict__ Wu,
                                                                       float* __restrict__ hid, int F, int K) {
    extern __shared__ float a_lds[];
    __shared__ float wave_sums[kWavesPerBlock];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int j0 = (blockIdx.x * kWavesPerBlock + wave) * PAIRS;
    const uint4* bp[2 * PAIRS];
#pragma unroll
    for (int q = 0; q < PAIRS; ++q) {
        const int j = j0 + q < F ? j0 + q : F - 1;
        bp[2 * q] = reinterpret_cast<const uint4*>(Wg + (size_t)j * K);
        bp[2 * q + 1] = reinterpret_cast<const uint4*>(Wu + (size_t)j * K);
    }
    StageRegs xr;
    stage_load(x, norm_w, norm_dtype, K, 0, xr);
    GemvRegs<2 * PAIRS> regs;
    gemv_prefetch<2 * PAIRS>(bp, 0, K >> 3, lane, regs);
    stage_finish(xr, x, norm_w, norm_dtype, eps, K, a_lds, wave_sums);
    float d[2 * PAIRS];
    gemv_accumulate<2 * PAIRS>(bp, a_lds, 0, K >> 3, lane, regs, d);
    gemv_finish<2 * PAIRS, 1>(d, nullptr, wave, lane);
    if (lane == 0) {
#pragma unroll
        for (int q = 0; q < PAIRS; ++q) {
            if (j0 + q < F) {
                const float g = d[2 * q];
                const float silu = g / (1.0f + expf(-g));
                hid[j0 + q] = silu * d[2 * q + 1];
            }
        }
    }
}

// logits = W . RMSNorm(x); optionally the workgroup's top-2 (largest, second, first index of largest) goes
// to blk_top (a | b | idx planes of `top_cap` entries) for the device-side greedy pick.
template <int COLS>
__global__ __launch_bounds__(kThreads) void norm_gemv_kernel(const float* __restrict__ x,
                                                             const void* __restrict__ norm_w, uint32_t norm_dtype,
                                                             float eps, const uint16_t* __restrict__ W,
                                                             float* __restrict__ out, int N, int K,
                                                             float* __restrict__ blk_top, uint32_t top_cap) {
    extern __shared__ float a_lds[];
    __shared__ float wave_sums[kWavesPerBlock];
    __shared__ float top_a[kWavesPerBlock], top_b[kWavesPerBlock];
    __shared__ uint32_t top_i[kWavesPerBlock];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int col0 = (blockIdx.x * kWavesPerBlock + wave) * COLS;
    const bool live = col0 < N;
    const uint4* bp[COLS];
#pragma unroll
    for (int c = 0; c < COLS; ++c) {
        const int col = (live && col0 + c < N) ? col0 + c : N - 1;
        bp[c] = reinterpret_cast<const uint4*>(W + (size_t)col * K);
    }
    StageRegs xr;
    stage_load(x, norm_w, norm_dtype, K, 0, xr);
    GemvRegs<COLS> regs;
    gemv_prefetch<COLS>(bp, 0, K >> 3, lane, regs);
    stage_finish(xr, x, norm_w, norm_dtype, eps, K, a_lds, wave_sums);
    float d[COLS];
    gemv_accumulate<COLS>(bp, a_lds, 0, K >> 3, lane, regs, d);
    gemv_finish<COLS, 1>(d, nullptr, wave, lane);
    if (lane == 0) {
        float a = -INFINITY, b = -INFINITY;
        uint32_t ia = 0xffffffffu;
#pragma unroll
        for (int c = 0; c < COLS; ++c) {
            if (live && col0 + c < N) {
                out[col0 + c] = d[c];
                if (d[c] > a) { b = a; a = d[c]; ia = (uint32_t)(col0 + c); }
                else if (d[c] > b) b = d[c];
            }
        }
        top_a[wave] = a; top_b[wave] = b; top_i[wave] = ia;
    }
    if (blk_top == nullptr) return;
    __syncthreads();
    if (threadIdx.x == 0 && blockIdx.x < top_cap) {
        float a = top_a[0], b = top_b[0];
        uint32_t ia = top_i[0];
        for (int w = 1; w < kWavesPerBlock; ++w) {     // ascending columns: ties keep the lower index
            const float oa = top_a[w], ob = top_b[w];
            if (oa > a) { b = fmaxf(a, ob); a = oa; ia = top_i[w]; }
            else b = fmaxf(b, oa);
        }
        blk_top[blockIdx.x] = a;
        blk_top[top_cap + blockIdx.x] = b;
        reinterpret_cast<uint32_t*>(blk_top)[2 * (size_t)top_cap + blockIdx.x] = ia;
    }
}

__global__ __launch_bounds__(kThreads) void embed_token_dev_kernel(const uint16_t* __restrict__ table,
                                                                   const uint32_t* __restrict__ token_dev,
                                                                   uint32_t vocab, uint32_t d_model,
                                                                   float* __restrict__ out) {
    uint32_t tok = token_dev[blockIdx.y];
    if (tok >= vocab) tok = vocab - 1;
    const uint32_t i = blockIdx.x * kThreads + threadIdx.x;
    if (i < d_model) out[(size_t)blockIdx.y * d_model + i] = m40_h2f(table[(size_t)tok * d_model + i]);
}

// Device-side greedy bookkeeping.  state: [0] position, [1] step, [2] current token,
// [3] capacity, then ids[capacity], then gaps[capacity] (f32 bits).  Candidates come either from the
// per-workgroup top-2 planes written by norm_gemv_kernel (n_blocks entries) or from a scan of the logits.
// With a table, the embedding row of the picked token is converted to f32 into x_out as well.
__global__ __launch_bounds__(1024) void greedy_step_kernel(const float* __restrict__ logits, uint32_t n,
                                                           const float* __restrict__ blk_top, uint32_t top_cap,
                                                           uint32_t n_blocks, uint32_t* __restrict__ state,
                                                           const uint16_t* __restrict__ table, uint32_t d_model,
                                                           float* __restrict__ x_out) {
    __shared__ float sa[16], sb[16];
    __shared__ uint32_t si[16];
    __shared__ uint32_t s_tok;
    float a = -INFINITY, b = -INFINITY;
    uint32_t ia = 0xffffffffu;
    auto offer = [&](float oa, float ob, uint32_t oi) {
        if (oa > a || (oa == a && oi < ia)) { b = fmaxf(a, ob); a = oa; ia = oi; }
        else b = fmaxf(b, oa);
    };
    if (blk_top) {
        const uint32_t* idx = reinterpret_cast<const uint32_t*>(blk_top) + 2 * (size_t)top_cap;
        for (uint32_t i = threadIdx.x; i < n_blocks; i += blockDim.x) offer(blk_top[i], blk_top[top_cap + i], idx[i]);
    } else {
        for (uint32_t i = threadIdx.x; i < n; i += blockDim.x) offer(logits[i], -INFINITY, i);
    }
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const float oa = __shfl_xor(a, o, 64), ob = __shfl_xor(b, o, 64);
        const uint32_t oi = __shfl_xor(ia, o, 64);
        offer(oa, ob, oi);
    }
    const uint32_t wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63u) == 0u) { sa[wave] = a; sb[wave] = b; si[wave] = ia; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (uint32_t w = 1; w < blockDim.x / 64u; ++w) offer(sa[w], sb[w], si[w]);
        uint32_t tok = ia == 0xffffffffu ? 0u : ia;
        if (tok >= n) tok = n - 1;
        const uint32_t step = state[1], cap = state[3];
        if (step < cap) {
            state[4 + step] = tok;
            state[4 + cap + step] = __float_as_uint(a - b);
        }
        state[2] = tok;
        state[1] = step + 1u;
        state[0] = state[0] + 1u;
        s_tok = tok;
    }
    if (table == nullptr) return;
    __syncthreads();
    const uint32_t tok = s_tok;
    for (uint32_t i = threadIdx.x; i < d_model; i += blockDim.x) x_out[i] = m40_h2f(table[(size_t)tok * d_model + i]);
}

bool fast_ok(const void* a, const void* b, int K) { return K % 8 == 0 && m40_aligned16(a) && m40_aligned16(b); }

}  // namespace

extern "C" {

int m40llm_ext_fused_norm_qkv_rope_append_async(
    M40llmCudaContext* ctx, M40llmKVCache* kv, uint32_t seq_id, const void* d_x_f32, const void* d_norm_w,
    uint32_t norm_weight_dtype, float eps, const void* d_wq_f16, const void* d_wk_f16, const void* d_wv_f16,
    const void* d_bq_f32, const void* d_bk_f32, const void* d_bv_f32, uint32_t d_model, uint32_t q_heads,
    uint32_t position, const uint32_t* position_dev, float freq_base, float freq_scale, uint32_t rope_layout, void* d_q_out_f32) {
    if (!ctx || !kv || !d_x_f32 || !d_norm_w || !d_wq_f16 || !d_wk_f16 || !d_wv_f16 || !d_q_out_f32) return -1;
    if (kv->compressed || !kv->d_k || !kv->d_v) return -2;
    if (seq_id >= kv->max_batch_size) return -2;
    if (norm_weight_dtype > 1) return -4;
    if (kv->head_dim == 0 || kv->head_dim % 2 != 0 || kv->num_heads == 0 || q_heads == 0) return -3;
    if (!position_dev && position >= kv->max_seq_len) return -5;
    if (d_model == 0) return -3;
    const uint32_t D = d_model;
    if (!fast_ok(d_x_f32, d_wq_f16, (int)D) || !m40_aligned16(d_wk_f16) || !m40_aligned16(d_wv_f16) ||
        !m40_aligned16(d_norm_w) || (size_t)D * 4 > 60 * 1024)
        return -6;
    QkvArgs p{};
    p.x = static_cast<const float*>(d_x_f32);
    p.norm_w = d_norm_w;
    p.wq = static_cast<const uint16_t*>(d_wq_f16);
    p.wk = static_cast<const uint16_t*>(d_wk_f16);
    p.wv = static_cast<const uint16_t*>(d_wv_f16);
    p.bq = static_cast<const float*>(d_bq_f32);
    p.bk = static_cast<const float*>(d_bk_f32);
    p.bv = static_cast<const float*>(d_bv_f32);
    p.q_out = static_cast<float*>(d_q_out_f32);
    const size_t ept = (size_t)kv->num_heads * kv->head_dim;
    p.k_cache = kv->d_k + (size_t)seq_id * kv->max_seq_len * ept;
    p.v_cache = kv->d_v + (size_t)seq_id * kv->max_seq_len * ept;
    p.seq_map_entry = kv->d_seq_map + seq_id;
    p.position_dev = position_dev;
    p.position = position;
    p.max_seq_len = kv->max_seq_len;
    p.d_model = D; p.q_heads = q_heads; p.kv_heads = kv->num_heads; p.head_dim = kv->head_dim;
    p.rope_layout = rope_layout; p.norm_dtype = norm_weight_dtype;
    p.eps = eps; p.rope_base = freq_base; p.rope_scale = freq_scale;
    p.rope_table = m40_rope_inv_freq_table(ctx, 1, ctx->decode_stream, kv->head_dim, freq_base);
    p.rope_cs = m40_rope_cs_cache(ctx, p.rope_table);
    const uint32_t pairs = (q_heads + 2u * kv->num_heads) * (kv->head_dim / 2u);
    (void)hipGetLastError();
    // one pair per wave: two per wave measured 3 % slower on the whole token at 1280 pairs
    norm_qkv_rope_append_kernel<1><<<(pairs + kWavesPerBlock - 1) / kWavesPerBlock, kThreads, (size_t)D * 4, ctx->decode_stream>>>(p);
    return hipGetLastError() == hipSuccess ? 0 : -7;
}

int m40llm_ext_gemv_residual_f32xf16_async(M40llmCudaContext* ctx, const void* d_a_f32, const void* d_w_f16,
                                           const void* d_residual_f32, void* d_out_f32, int N, int K) {
    if (!ctx || !d_a_f32 || !d_w_f16 || !d_out_f32) return -1;
    if (N <= 0 || K <= 0) return -2;
    if (!fast_ok(d_a_f32, d_w_f16, K)) return -6;
    (void)hipGetLastError();
    const float* a = static_cast<const float*>(d_a_f32);
    const uint16_t* W = static_cast<const uint16_t*>(d_w_f16);
    const float* r = static_cast<const float*>(d_residual_f32);
    float* o = static_cast<float*>(d_out_f32);
    const GemvShape g = gemv_pick_shape(N, K);
    if (g.ksplit == 4) gemv_residual_kernel<2, 4><<<g.blocks, kThreads, 0, ctx->decode_stream>>>(a, W, r, o, N, K);
    else if (g.cols == 4) gemv_residual_kernel<4, 1><<<g.blocks, kThreads, 0, ctx->decode_stream>>>(a, W, r, o, N, K);
    else if (g.cols == 2) gemv_residual_kernel<2, 1><<<g.blocks, kThreads, 0, ctx->decode_stream>>>(a, W, r, o, N, K);
    else gemv_residual_kernel<1, 1><<<g.blocks, kThreads, 0, ctx->decode_stream>>>(a, W, r, o, N, K);
    return hipGetLastError() == hipSuccess ? 0 : -7;
}

int m40llm_ext_fused_norm_gate_up_swiglu_async(M40llmCudaContext* ctx, const void* d_x_f32, const void* d_norm_w,
                                               uint32_t norm_weight_dtype, float eps, const void* d_wgate_f16,
                                               const void* d_wup_f16, void* d_hid_f32, int ffn, int d_model) {
    if (!ctx || !d_x_f32 || !d_norm_w || !d_wgate_f16 || !d_wup_f16 || !d_hid_f32) return -1;
    if (ffn <= 0 || d_model <= 0) return -2;
    if (norm_weight_dtype > 1) return -4;
    if (!fast_ok(d_x_f32, d_wgate_f16, d_model) || !m40_aligned16(d_wup_f16) || !m40_aligned16(d_norm_w) ||
        (size_t)d_model * 4 > 60 * 1024)
        return -6;
    (void)hipGetLastError();
    // two (gate, up) row pairs per wave once there are enough rows to fill the chip that way (measured: 3 % faster
    // than one pair at FFN 5632; four pairs are slower)
    if (ffn >= 4096)
    norm_gate_up_swiglu_kernel<2><<<(ffn + 7) / 8, kThreads, (size_t)d_model * 4, ctx->decode_stream>>>(
        static_cast<const float*>(d_x_f32), d_norm_w, norm_weight_dtype, eps, static_cast<const uint16_t*>(d_wgate_f16),
        static_cast<const uint16_t*>(d_wup_f16), static_cast<float*>(d_hid_f32), ffn, d_model);
    else
    norm_gate_up_swiglu_kernel<1><<<(ffn + 3) / 4, kThreads, (size_t)d_model * 4, ctx->decode_stream>>>(
        static_cast<const float*>(d_x_f32), d_norm_w, norm_weight_dtype, eps, static_cast<const uint16_t*>(d_wgate_f16),
        static_cast<const uint16_t*>(d_wup_f16), static_cast<float*>(d_hid_f32), ffn, d_model);
    return hipGetLastError() == hipSuccess ? 0 : -7;
}

int m40llm_ext_fused_norm_gemv_f32xf16_async(M40llmCudaContext* ctx, const void* d_x_f32, const void* d_norm_w,
                                             uint32_t norm_weight_dtype, float eps, const void* d_w_f16,
                                             void* d_out_f32, int N, int K, void* d_block_top2,
                                             uint32_t top2_capacity, uint32_t* out_n_blocks) {
    if (!ctx || !d_x_f32 || !d_norm_w || !d_w_f16 || !d_out_f32) return -1;
    if (N <= 0 || K <= 0) return -2;
    if (norm_weight_dtype > 1) return -4;
    if (!fast_ok(d_x_f32, d_w_f16, K) || !m40_aligned16(d_norm_w) || (size_t)K * 4 > 60 * 1024) return -6;
    (void)hipGetLastError();
    const float* x = static_cast<const float*>(d_x_f32);
    const uint16_t* W = static_cast<const uint16_t*>(d_w_f16);
    float* o = static_cast<float*>(d_out_f32);
    float* top = static_cast<float*>(d_block_top2);
    const size_t lds = (size_t)K * 4;
    const int cols = N >= 16384 ? 4 : (N >= 6144 ? 2 : 1);
    const int blocks = (N + 4 * cols - 1) / (4 * cols);
    if (top && (uint32_t)blocks > top2_capacity) return -5;
    if (out_n_blocks) *out_n_blocks = (uint32_t)blocks;
    if (cols == 4) norm_gemv_kernel<4><<<blocks, kThreads, lds, ctx->decode_stream>>>(x, d_norm_w, norm_weight_dtype, eps, W, o, N, K, top, top2_capacity);
    else if (cols == 2) norm_gemv_kernel<2><<<blocks, kThreads, lds, ctx->decode_stream>>>(x, d_norm_w, norm_weight_dtype, eps, W, o, N, K, top, top2_capacity);
    else norm_gemv_kernel<1><<<blocks, kThreads, lds, ctx->decode_stream>>>(x, d_norm_w, norm_weight_dtype, eps, W, o, N, K, top, top2_capacity);
    return hipGetLastError() == hipSuccess ? 0 : -7;
}

int m40llm_ext_embed_token_dev_async(M40llmCudaContext* ctx, const void* d_table_f16, const uint32_t* token_dev,
                                     uint32_t vocab, uint32_t d_model, void* d_out_f32) {
    if (!ctx || !d_table_f16 || !token_dev || !d_out_f32) return -1;
    if (vocab == 0 || d_model == 0) return -2;
    (void)hipGetLastError();
    embed_token_dev_kernel<<<(d_model + kThreads - 1) / kThreads, kThreads, 0, ctx->decode_stream>>>(
        static_cast<const uint16_t*>(d_table_f16), token_dev, vocab, d_model, static_cast<float*>(d_out_f32));
    return hipGetLastError() == hipSuccess ? 0 : -3;
}

int m40llm_ext_embed_rows_async(M40llmCudaContext* ctx, const void* d_table_f16, const uint32_t* tokens_dev, uint32_t rows,
                                uint32_t vocab, uint32_t d_model, void* d_out_f32) {
    if (!ctx || !d_table_f16 || !tokens_dev || !d_out_f32) return -1;
    if (vocab == 0 || d_model == 0 || rows == 0 || rows > 65535u) return -2;
    (void)hipGetLastError();
    embed_token_dev_kernel<<<dim3((d_model + kThreads - 1) / kThreads, rows), kThreads, 0, ctx->decode_stream>>>(
        static_cast<const uint16_t*>(d_table_f16), tokens_dev, vocab, d_model, static_cast<float*>(d_out_f32));
    return hipGetLastError() == hipSuccess ? 0 : -3;
}

int m40llm_ext_greedy_step_async(M40llmCudaContext* ctx, const void* d_logits_f32, uint32_t n,
                                 const void* d_block_top2, uint32_t top2_capacity, uint32_t n_blocks,
                                 uint32_t* state_dev, const void* d_table_f16, uint32_t d_model, void* d_x_out_f32) {
    if (!ctx || !state_dev || (!d_logits_f32 && !d_block_top2)) return -1;
    if (n == 0) return -2;
    if (d_block_top2 && (n_blocks == 0 || n_blocks > top2_capacity)) return -2;
    if (d_table_f16 && (!d_x_out_f32 || d_model == 0)) return -1;
    (void)hipGetLastError();
    greedy_step_kernel<<<1, 1024, 0, ctx->decode_stream>>>(
        static_cast<const float*>(d_logits_f32), n, static_cast<const float*>(d_block_top2), top2_capacity, n_blocks,
        state_dev, static_cast<const uint16_t*>(d_table_f16), d_model, static_cast<float*>(d_x_out_f32));
    return hipGetLastError() == hipSuccess ? 0 : -3;
}

}  // extern "C"
