// Shared host/device definitions of the gfx950 implementation of the m40llm C ABI.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>

#include "../../include/m40llm.h"

// ---------------------------------------------------------------------------------
// Opaque handles.  Layout is private to this library (the reference declares them
// zero-sized on the Rust side, src/cuda.rs:30-45).
// ---------------------------------------------------------------------------------
struct M40llmCudaEvent {
    hipEvent_t event;
};

struct M40llmCudaGraphExec {
    hipGraph_t graph;
    hipGraphExec_t exec;
};

// Per-stream scratch owned by the context.  Two streams may run a GEMM or an
// attention call at the same time, so each stream kind has its own copy.
struct M40StreamScratch {
    void* gemm_pack;         // packed f16 hi/lo activation fragments for the MFMA GEMM
    size_t gemm_pack_bytes;
    void* attn_partial;      // split-KV partial results (m, l, acc[hd]) of the attention kernels
    size_t attn_partial_bytes;
    void* select;            // block scores / selected ids / counts of the block-select path
    size_t select_bytes;
    void* tiled_pack;        // f16 high / low planes of the activations of the many-row GEMM; grown on demand
    size_t tiled_pack_bytes;
    void* attn_planes;       // f16 high / low planes of K and V^T for the prefill attention; grown on demand
    size_t attn_planes_bytes;
};

struct M40llmCudaContext {
    int device_id;
    hipStream_t prefill_stream;
    hipStream_t decode_stream;
    hipEvent_t prefill_waits_decode_event;
    hipEvent_t decode_waits_prefill_event;
    M40StreamScratch scratch[2];   // [stream_kind]
    int num_cus;
    // RoPE pair frequencies base^(-2 i / head_dim), i < head_dim / 2, filled on the device on first use of a
    // (head_dim, base) on a stream: kM40RopeSlots tables of kM40RopeTableLen floats per stream
    float* rope_tables;
    // beside every frequency table: the rotation of each pair at the position last asked for, as {position bits, cos,
    // sin, scale bits} (16 bytes, written and read whole); a decode step computes the angles once, in its first layer
    float4* rope_cs;
    uint32_t* host_staging;        // pinned, kM40HostStagingWords words: device metadata read back for validation
    struct { float base; uint32_t head_dim; uint32_t ready; } rope_slots[2][4];
};
constexpr int kM40HostStagingWords = 2048;
constexpr uint32_t kM40OldStoreSlackRows = 64;
constexpr int kM40RopeSlots = 4;
constexpr int kM40RopeTableLen = 256;
// Table of a (head_dim, base) for kernels launched on `stream` (of kind stream_kind), or nullptr (head_dim too large,
// no free slot, or the stream is being captured and the table does not exist yet): callers then evaluate the power.
const float* m40_rope_inv_freq_table(M40llmCudaContext* ctx, uint32_t stream_kind, hipStream_t stream, uint32_t head_dim,
                                     float base);

struct M40llmKVCache {
    // dense storage, f16 [seq][token][kv_head][head_dim]
    uint16_t* d_k;
    uint16_t* d_v;
    uint32_t* d_seq_map;           // tokens appended per sequence
    // compressed storage
    uint16_t* d_recent_k;          // ring [seq][W][kvh][hd], slot = pos % W
    uint16_t* d_recent_v;
    // old store, head-major so that the tokens of a block are one contiguous run per kv head (the handle is
    // opaque; debug read-backs answer in the reference's [seq][token][kvh] order).  Each array is followed by
    // kM40OldStoreSlackRows zeroed rows: the attention reads whole passes of rows and ignores those past a block.
    uint16_t* d_fp16_old_k;        // [seq][kvh][max_seq_len][hd], token index = absolute position
    uint8_t* d_q4_old_v;           // [seq][kvh][max_seq_len][hd/2]
    float* d_q4_old_v_scale;       // [seq][kvh][max_seq_len]; with v_format 1: u32 [seq][kvh][max_seq_len][hd/32]
    uint32_t max_seq_len;
    uint32_t max_batch_size;
    uint32_t num_heads;            // kv heads
    uint32_t head_dim;
    uint32_t compressed;
    uint32_t recent_window;
    uint32_t block_size;
    uint32_t max_blocks;
    uint32_t top_blocks;
    uint32_t representatives;
    uint32_t representative_policy;
    uint32_t fp16_k_q4_v_old_backing;
    uint32_t v_format;             // old V: 0 the reference's q4 (f32 scale per token and head), 1 groups of 32 with f16 scale + f16 min
    int device_id;
};

// ---------------------------------------------------------------------------------
// Host helpers
// ---------------------------------------------------------------------------------
static inline int m40_ensure_device(M40llmCudaContext* ctx) {
    if (!ctx) return -1;
    return hipSetDevice(ctx->device_id) == hipSuccess ? 0 : -2;
}

static inline hipStream_t m40_select_stream(M40llmCudaContext* ctx, uint32_t stream_kind) {
    if (!ctx) return nullptr;
    if (stream_kind == 0) return ctx->prefill_stream;
    if (stream_kind == 1) return ctx->decode_stream;
    return nullptr;
}

#ifdef __HIPCC__
#define M40_HD __host__ __device__
#else
#define M40_HD
#endif
M40_HD static inline bool m40_aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Internal launch entry points shared between translation units ------------------
// GEMM family (gemm.hip)
int m40_launch_gemm_f32xf16_gguf(M40llmCudaContext* ctx, hipStream_t stream, uint32_t stream_kind,
                                 const float* A, const uint16_t* B, float* C, int M, int N, int K);
// skinny MFMA GEMM (skinny_mfma.hip): fmt 0 = f16 GGUF weights, 1 = q8_0 blocks.  `up` != null multiplies
// silu(A) by it while packing; W1/C1 give an optional second matrix of the same shape.
// Row-batched vector-ALU GEMV (rows_gemv.hip): up to eight rows, K <= 2048, epilogue in the same kernel.
bool m40_rows_gemv_supported(int rows, int K);
int m40_rows_gemv_residual(hipStream_t stream, const float* a, const uint16_t* W, const float* residual, float* out,
                           int rows, int N, int K);
int m40_rows_norm_qkv(M40llmCudaContext* ctx, hipStream_t stream, const M40llmKVCache* kv, const uint32_t* ids_dev, const uint32_t* lens_dev,
                      uint32_t rows, const float* x, const void* norm_w, uint32_t norm_dtype, float eps,
                      const uint16_t* wq, const uint16_t* wk, const uint16_t* wv, const float* bq, const float* bk,
                      const float* bv, uint32_t d_model, uint32_t q_heads, float rope_base, float rope_scale,
                      uint32_t rope_layout, float* q_out);
// rows_mfma.hip: persistent matrix-core kernel for up to eight rows and K = 2048, epilogue inside (one launch)
// the {position, cos, sin, scale} entries that belong to a table returned by m40_rope_inv_freq_table (or null)
float4* m40_rope_cs_cache(M40llmCudaContext* ctx, const float* table);
bool m40_rows_mfma_supported(int rows, int K);
int m40_rows_mfma_swiglu(M40llmCudaContext* ctx, hipStream_t stream, const float* x, const void* norm_w, uint32_t norm_dtype,
                         float eps, const uint16_t* wgate, const uint16_t* wup, float* out, int rows, int ffn, int K,
                         float* zero = nullptr, int zero_count = 0);
// rows_khalf_mfma.hip: up to eight rows against [N][K] with a long K in one launch: tiles x two halves of K, each
// workgroup adding its sums (the first half's with the residual) into a result that an earlier launch has cleared
bool m40_rows_khalf_supported(const M40llmCudaContext* ctx, int rows, int N, int K);
int m40_rows_khalf_residual(M40llmCudaContext* ctx, hipStream_t stream, const float* a, const uint16_t* W,
                            const float* residual, float* out_zeroed, int rows, int N, int K);
int m40_zero_f32(hipStream_t stream, float* dst, size_t n);
int m40_rows_mfma_plain(M40llmCudaContext* ctx, hipStream_t stream, const float* x, const void* norm_w, uint32_t norm_dtype,
                        float eps, const uint16_t* W, float* out, int rows, int N, int K);
bool m40_rows_mfma_qkv_supported(int rows, int K, uint32_t head_dim);
int m40_rows_mfma_qkv(M40llmCudaContext* ctx, hipStream_t stream, const M40llmKVCache* kv, const uint32_t* ids_dev,
                      const uint32_t* lens_dev, uint32_t rows, const float* x, const void* norm_w, uint32_t norm_dtype, float eps,
                      const uint16_t* wq, const uint16_t* wk, const uint16_t* wv, const float* bq, const float* bk,
                      const float* bv, uint32_t d_model, uint32_t q_heads, float rope_base, float rope_scale,
                      uint32_t rope_layout, float* q_out);
// many-row f32 x f16 GEMM on 128 x 128 tiles (gemm_tiled.hip): M > 32, K a multiple of 32, 16-byte aligned operands
bool m40_gemm_tiled_supported(const void* A, const void* B, int M, int N, int K);
int m40_launch_gemm_tiled(M40llmCudaContext* ctx, hipStream_t stream, uint32_t stream_kind, const float* A, const uint16_t* B,
                          float* C, int M, int N, int K);
// up to three weight matrices over the same activations in one launch; 1 = declined (no packing buffer), else 0 / -2
int m40_launch_gemm_tiled_multi(M40llmCudaContext* ctx, hipStream_t stream, uint32_t stream_kind, const float* A, int M, int K,
                                int n_mats, const uint16_t* const* B, const int* N, float* const* C);
// the same with the rows of A produced by the packing pass (source_kind 0: A as it is, 1: RMSNorm of A with norm_w, 2:
// SwiGLU of A (gate) and A2 (up)) and an optional residual per matrix added to the product (R[i] may be C[i])
int m40_launch_gemm_tiled_fused(M40llmCudaContext* ctx, hipStream_t stream, uint32_t stream_kind, int source_kind, const float* A,
                                const float* A2, const void* norm_w, uint32_t norm_dtype, float eps, int M, int K, int n_mats,
                                const uint16_t* const* B, const int* N, float* const* C, const float* const* R);
bool m40_skinny_supported(const M40llmCudaContext* ctx, uint32_t stream_kind, int M, int N, int K, int fmt);
int m40_launch_skinny(M40llmCudaContext* ctx, hipStream_t stream, uint32_t stream_kind, int fmt, const float* A,
                      const float* up, const void* W0, float* C0, const void* W1, float* C1, int M, int N, int K);
// q8_0 weights on the int8 matrix instruction (q80_i8.hip): 2 <= M <= 16 rows, K a multiple of 256; A and W 16-byte aligned
bool m40_q80_i8_supported(const M40llmCudaContext* ctx, uint32_t stream_kind, int M, int N, int K);
int m40_launch_q80_i8(M40llmCudaContext* ctx, hipStream_t stream, uint32_t stream_kind, const float* A, const uint8_t* W,
                      float* C, int M, int N, int K);
int m40_launch_q80_i8_ffn(M40llmCudaContext* ctx, hipStream_t stream, uint32_t stream_kind, const float* x,
                          const uint8_t* wg, const uint8_t* wu, const uint8_t* wd, float* out, int M, int d_model, int ffn);
// attention over an explicit dense range (attention.hip)
struct M40AttnArgs {
    const uint16_t* K;       // base of the cache (sequence 0)
    const uint16_t* V;
    uint32_t max_seq_len, kv_heads, head_dim, q_heads;
    const float* Q;          // [batch][q_heads][hd]
    float* Out;
    uint32_t batch;
    // one of: fixed (seq_id, seq_len) for batch==1, or device arrays
    uint32_t seq_id, seq_len;
    const uint32_t* seq_ids_dev;
    const uint32_t* seq_lens_dev;   // also used alone for the seq_len_dev variant (batch==1)
    uint32_t max_len_hint;          // upper bound of any row's length (sizes the grid)
    uint32_t window;                // 0 = whole sequence, else only the last `window` tokens
    uint32_t len_bias;              // added to lengths read from seq_lens_dev
    uint32_t max_batch;             // 0, or the bound that device-side sequence ids are checked against
    // chunk partials go here instead of into the context's per-stream arena (null = the arena); with an override
    // the chunking is the one the arena would get, and a call whose partials do not fit is refused with -9
    float* partial_override;
    size_t partial_override_bytes;
};
// attention.hip: resolves this device's copy of the fixed partial buffer of
// m40llm_ext_attention_last_token_f32_gqa_static_scratch_async (the device must be current); 0 or a negative code
int m40_attention_static_scratch_init(int device_id);
int m40_launch_dense_attention(M40llmCudaContext* ctx, hipStream_t stream, uint32_t stream_kind,
                               const M40AttnArgs& a);

// ---------------------------------------------------------------------------------
// Device helpers
// ---------------------------------------------------------------------------------
#ifdef __HIPCC__
#include <hip/hip_fp16.h>

typedef _Float16 m40_half;
typedef _Float16 m40_half8 __attribute__((ext_vector_type(8)));
typedef _Float16 m40_half4 __attribute__((ext_vector_type(4)));
typedef float m40_float4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float m40_h2f(uint16_t bits) {
    return static_cast<float>(__builtin_bit_cast(_Float16, bits));
}
// round-to-nearest-even f32 -> f16 (v_cvt_f16_f32 in the default rounding mode).  The empty asm pins the
// f32 value first: without it the compiler folds a preceding multiply(-add) and the conversion into one
// mixed-precision FMA that rounds once, to f16, where the reference rounds to f32 and then to f16 (the two
// differ whenever the f32 result sits exactly between two f16 values).
__device__ __forceinline__ uint16_t m40_f2h(float x) {
    asm volatile("" : "+v"(x));
    return __builtin_bit_cast(uint16_t, static_cast<_Float16>(x));
}

// Streaming (read-once) 128-bit load: keeps weights / old K out of the way of data that is reused.
typedef uint32_t m40_u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 m40_load_stream(const uint4* p) {
    const m40_u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const m40_u32x4*>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}

// 8 halves packed in a uint4 -> 8 floats
__device__ __forceinline__ void m40_unpack8(const uint4& w, float (&f)[8]) {
    const uint32_t u[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        f[2 * i] = m40_h2f(static_cast<uint16_t>(u[i] & 0xffffu));
        f[2 * i + 1] = m40_h2f(static_cast<uint16_t>(u[i] >> 16));
    }
}

// Cross-lane add through DPP (row = 16 lanes).  ctrl: quad_perm / row_* selector.
template <int CTRL>
__device__ __forceinline__ float m40_dpp_f(float x) {
    return __builtin_bit_cast(
        float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, true));
}
#define M40_DPP_XOR1 0xB1        // quad_perm [1,0,3,2]
#define M40_DPP_XOR2 0x4E        // quad_perm [2,3,0,1]
#define M40_DPP_HALF_MIRROR 0x141  // lane i <-> 7-i inside each group of 8
#define M40_DPP_MIRROR 0x140       // lane i <-> 15-i inside each row of 16

// Butterfly sums.  After the xor-1/xor-2 steps every lane of a quad holds the quad
// sum, so the mirrors act as xor-4 / xor-8 on those sums; additions are commutative,
// hence every lane ends with the bits of the halving tree
//   ((x0+x1)+(x2+x3)) + ((x4+x5)+(x6+x7)) ...
__device__ __forceinline__ float m40_sum8(float x) {   // over aligned groups of 8 lanes
    x += m40_dpp_f<M40_DPP_XOR1>(x);
    x += m40_dpp_f<M40_DPP_XOR2>(x);
    x += m40_dpp_f<M40_DPP_HALF_MIRROR>(x);
    return x;
}
__device__ __forceinline__ float m40_sum16(float x) {  // over rows of 16 lanes
    x = m40_sum8(x);
    x += m40_dpp_f<M40_DPP_MIRROR>(x);
    return x;
}
// The xor-16 and xor-32 steps on the vector ALU: v_permlane16_swap (v_permlane32_swap) exchanges the odd rows of 16 (32)
// lanes of its first operand with the even rows of its second; with both operands holding x, one register ends with
// the even rows' values in every lane and the other with the odd rows', and their sum or maximum is the butterfly
// step -- the same two numbers in either order as lane l joining lane l ^ 16 (l ^ 32), hence the same bits as the
// ds_bpermute form (__shfl_xor), which pays an LDS round trip per step (36 ns against 21 ns in a dependent chain).
// The s_nop covers the wait states between a vector write of an operand and the swap.  All 64 lanes must be active.
__device__ __forceinline__ void m40_swap_rows16(float& a, float& b) { asm("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a), "+v"(b)); }
__device__ __forceinline__ void m40_swap_rows32(float& a, float& b) { asm("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b)); }
__device__ __forceinline__ float m40_add_xor16(float x) { float a = x, b = x; m40_swap_rows16(a, b); return a + b; }
__device__ __forceinline__ float m40_add_xor32(float x) { float a = x, b = x; m40_swap_rows32(a, b); return a + b; }
__device__ __forceinline__ float m40_max_xor16(float x) { float a = x, b = x; m40_swap_rows16(a, b); return fmaxf(a, b); }
__device__ __forceinline__ float m40_max_xor32(float x) { float a = x, b = x; m40_swap_rows32(a, b); return fmaxf(a, b); }
// Butterfly sum over the lanes that differ in the bits FROM, 2 FROM, ... 32 (lanes equal in the bits below FROM keep
// separate sums): xor 8 is a rotation of the row of 16 by 8, xor 16 and 32 the swaps above -- the partner of every
// step and the order of the steps are those of  for (o = FROM; o < 64; o <<= 1) v += __shfl_xor(v, o).
#define M40_DPP_ROW_ROR8 0x128
template <int FROM>
__device__ __forceinline__ float m40_sum_lanes_from(float v) {
    static_assert(FROM == 8 || FROM == 16 || FROM == 32, "steps below 8 have no single-instruction form here");
    if (FROM <= 8) v += m40_dpp_f<M40_DPP_ROW_ROR8>(v);
    if (FROM <= 16) v = m40_add_xor16(v);
    return m40_add_xor32(v);
}
__device__ __forceinline__ float m40_sum64(float x) {  // whole wave
    x = m40_sum16(x);
    x = m40_add_xor16(x);
    x = m40_add_xor32(x);
    return x;
}
__device__ __forceinline__ float m40_max16(float x) {  // over rows of 16 lanes
    x = fmaxf(x, m40_dpp_f<M40_DPP_XOR1>(x));
    x = fmaxf(x, m40_dpp_f<M40_DPP_XOR2>(x));
    x = fmaxf(x, m40_dpp_f<M40_DPP_HALF_MIRROR>(x));      // quads hold their maximum: the mirrors join 4 + 4 and 8 + 8
    x = fmaxf(x, m40_dpp_f<M40_DPP_MIRROR>(x));
    return x;
}
__device__ __forceinline__ float m40_max64(float x) {
    x = m40_max16(x);
    x = m40_max_xor16(x);
    x = m40_max_xor32(x);
    return x;
}

__device__ __forceinline__ float m40_inv_sqrt_head_dim(uint32_t hd) {
    return hd == 64u ? 0.125f : (hd == 128u ? 0.08838834764831845f : 1.0f / sqrtf((float)hd));
}

// RoPE pair addressing and rotation shared by every kernel that rotates, so the
// fused append and the standalone RoPE produce identical bits.
__device__ __forceinline__ void m40_rope_pair(uint32_t head, uint32_t off, uint32_t head_dim,
                                              uint32_t layout, size_t* i0, size_t* i1) {
    const size_t hb = (size_t)head * head_dim;
    if (layout == M40LLM_ROPE_LAYOUT_NEOX) {
        *i0 = hb + off;
        *i1 = *i0 + head_dim / 2u;
    } else {
        *i0 = hb + 2u * off;
        *i1 = *i0 + 1u;
    }
}
// cos/sin of the rotation angle of pair `off` at `position`.  Deliberately not inlined: every kernel
// that rotates (standalone RoPE, the rotating KV appends, the fused QKV kernel) must produce the same
// bits for the same input, and the compiler's choices inside the inlined trigonometric code were seen
// to differ by an ulp between call sites.
__device__ __noinline__ static float m40_rope_inv_freq(uint32_t off, uint32_t head_dim, float base) {
    // The per-pair frequency is evaluated in double and rounded once: theta multiplies it by
    // the position, so a one-ulp difference in a float powf would grow to ~position * 2^-23
    // radians.  The rounded double result equals the host libm's powf for the bases and
    // exponents in use.
    const float exponent = -2.0f * static_cast<float>(off) / static_cast<float>(head_dim);
    return static_cast<float>(pow(static_cast<double>(base), static_cast<double>(exponent)));
}
// cos/sin at `position` for a pair whose frequency is already known (from m40_rope_inv_freq or from the context's
// table of the same values).
__device__ __noinline__ static float2 m40_rope_cos_sin_freq(uint32_t position, float inv_freq, float scale) {
    const float pos = static_cast<float>(position) * scale;
    const float theta = pos * inv_freq;
    return make_float2(cosf(theta), sinf(theta));
}
__device__ __forceinline__ float2 m40_rope_cos_sin(uint32_t position, uint32_t off, uint32_t head_dim, float base,
                                                   float scale) {
    return m40_rope_cos_sin_freq(position, m40_rope_inv_freq(off, head_dim, base), scale);
}
__device__ __forceinline__ void m40_rope_apply(float2 cs, float x0, float x1, float* y0, float* y1) {
    // explicit fused multiply-adds: the same rounding in every kernel that inlines this rotation
    *y0 = fmaf(x0, cs.x, -(x1 * cs.y));
    *y1 = fmaf(x0, cs.y, x1 * cs.x);
}
__device__ __forceinline__ void m40_rope_rotate(uint32_t position, uint32_t off, uint32_t head_dim,
                                                float base, float scale, float x0, float x1,
                                                float* y0, float* y1) {
    m40_rope_apply(m40_rope_cos_sin(position, off, head_dim, base, scale), x0, x1, y0, y1);
}

// q4 V pair, two's-complement nibbles, even dim in the low nibble
__device__ __forceinline__ uint8_t m40_pack_q4_pair(float a, float b, float scale) {
    int qa = (int)lrintf(a / scale);
    int qb = (int)lrintf(b / scale);
    qa = qa < -7 ? -7 : (qa > 7 ? 7 : qa);
    qb = qb < -7 ? -7 : (qb > 7 ? 7 : qb);
    return (uint8_t)((qa & 0x0f) | ((qb & 0x0f) << 4));
}

// 4-bit V in groups of 32 under an f16 scale and an f16 minimum (old-store format 1; no counterpart in the reference).
// The lane holds dimensions 2 lane, 2 lane + 1 of a head; a group is 16 consecutive lanes.  Returns the packed byte
// and, in *dm, the group's word: bits of d = f16((max - min) / 15) | bits of m = f16(min) << 16.
__device__ __forceinline__ uint8_t m40_pack_q4g32_pair(float a, float b, uint32_t* dm) {
    float mn = fminf(a, b), mx = fmaxf(a, b);
#pragma unroll
    for (int o = 1; o < 16; o <<= 1) {
        mn = fminf(mn, __shfl_xor(mn, o, 64));
        mx = fmaxf(mx, __shfl_xor(mx, o, 64));
    }
    const uint16_t db = m40_f2h((mx - mn) / 15.0f), mb = m40_f2h(mn);
    const float d = m40_h2f(db), m = m40_h2f(mb);
    *dm = (uint32_t)db | ((uint32_t)mb << 16);
    int qa = d > 0.0f ? (int)lrintf((a - m) / d) : 0;
    int qb = d > 0.0f ? (int)lrintf((b - m) / d) : 0;
    qa = qa < 0 ? 0 : (qa > 15 ? 15 : qa);
    qb = qb < 0 ? 0 : (qb > 15 ? 15 : qb);
    return (uint8_t)(qa | (qb << 4));
}
#endif  // __HIPCC__
