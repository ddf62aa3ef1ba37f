// GEMV / skinny GEMM family for gfx950: C[M,N] f32 = A[M,K] x B, f32 accumulation.
//
//   M == 1      : wave-per-column GEMV (gemv_core.hpp).  64 lanes stride the K dimension with 128-bit
//                 loads of the f16 weights (GGUF layout: K contiguous per output column), f32 FMA
//                 per lane, one DPP/shuffle butterfly per column; few columns x long K splits K over
//                 the four waves of a workgroup.  HBM-bound; bytes = 2*N*K.
//   2 <= M <= 16: MFMA (v_mfma_f32_16x16x32_f16).  The f32 activations are split exactly into
//                 f16 hi + f16 lo parts (after a per-row power-of-two scale), the f16 weights go
//                 from HBM to the B operand registers without passing LDS: lane (n, g) loads the
//                 32 contiguous bytes k = 64t+16g .. +15 of column n, which are the B fragments
//                 of two MFMAs.  Weights are read once for all rows.
//   otherwise   : a plain wave-per-output kernel (any shape, any alignment).
//
// Reference semantics: gemm_f32xf16_gguf_f32_kernel cuda/kernels.cu:5037-5052 and the entry
// points :5068-5302 (which run on the prefill stream and block until done).
#include "common.hpp"
#include "gemv_core.hpp"

namespace {

// ---------------------------------------------------------------------------------------
// M == 1
// ---------------------------------------------------------------------------------------
template <int COLS, int KSPLIT>
__global__ __launch_bounds__(256) void gemv_f32xf16_gguf_kernel(const float* __restrict__ A,
                                                                const uint16_t* __restrict__ B,
                                                                float* __restrict__ C, int N, int K) {
    __shared__ float red[4 * COLS];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int col0 = KSPLIT == 1 ? (blockIdx.x * 4 + wave) * COLS : blockIdx.x * COLS;
    if (col0 >= N) return;   // uniform per wave (KSPLIT 1) or per workgroup (KSPLIT 4)
    const uint4* bp[COLS];
#pragma unroll
    for (int c = 0; c < COLS; ++c) {
        const int col = col0 + c < N ? col0 + c : N - 1;
        bp[c] = reinterpret_cast<const uint4*>(B + (size_t)col * K);
    }
    int c_begin, c_end;
    gemv_range<KSPLIT>(K, wave, &c_begin, &c_end);
    constexpr bool ACTS = KSPLIT == 1;     // measured: with K split over the waves the early loads do not pay
    GemvActRegs acts;
    if (ACTS) gemv_prefetch_acts(A, c_begin, c_end, lane, acts);      // before the weights: they return first
    GemvRegs<COLS> regs;
    gemv_prefetch<COLS, KSPLIT != 1>(bp, c_begin, c_end, lane, regs);
    float acc[COLS];
    if (ACTS) gemv_accumulate<COLS>(bp, A, c_begin, c_end, lane, regs, acts, acc);
    else gemv_accumulate<COLS>(bp, A, c_begin, c_end, lane, regs, acc);
    gemv_finish<COLS, KSPLIT>(acc, red, wave, lane);
    if (lane == 0 && (KSPLIT == 1 || wave == 0)) {
#pragma unroll
        for (int c = 0; c < COLS; ++c)
            if (col0 + c < N) C[col0 + c] = acc[c];
    }
}

// ---------------------------------------------------------------------------------------
// 2 <= M <= 16: activation packing + MFMA
// ---------------------------------------------------------------------------------------
// Packed layout: for k-tile t (64 values of k) and half s in {0,1}, lane l of the wave finds
// its A fragment (8 halves = 16 bytes) at P[((t*2+s)*64 + l)]:
//     row = l % 16,  k = 64t + 16*(l/16) + 8s + 0..7
// which pairs with the B fragment "column n, same k" that the GEMM kernel loads.
// STACKED (M <= 8): rows 0..7 carry hi(A[row]), rows 8..15 carry lo(A[row-8]).
// Otherwise two fragment sets are written: hi at P, lo at P + K/64*2*64.
// One workgroup per (padded) row; row_scale[row] = 2^e receives the factor to undo.
__global__ __launch_bounds__(256) void pack_a_hilo_kernel(const float* __restrict__ A, int M, int K,
                                                          int stacked, uint4* __restrict__ P,
                                                          float* __restrict__ row_scale) {
    __shared__ float wave_max[4];
    const int row = blockIdx.x;  // 0..7 (stacked) or 0..15
    const int tid = threadIdx.x;
    const bool live = row < M;
    float inv_scale = 1.0f, scale = 1.0f;
    if (live) {
        float mx = 0.0f;
        for (int k = tid; k < K; k += 256) mx = fmaxf(mx, fabsf(A[(size_t)row * K + k]));
        mx = m40_max64(mx);
        if ((tid & 63) == 0) wave_max[tid >> 6] = mx;
        __syncthreads();
        mx = fmaxf(fmaxf(wave_max[0], wave_max[1]), fmaxf(wave_max[2], wave_max[3]));
        if (mx > 0.0f && mx < INFINITY) {
            int e;
            (void)frexpf(mx, &e);         // mx = f * 2^e, f in [0.5, 1)
            e -= 11;                      // scaled max in [2^10, 2^11)
            e = e < -100 ? -100 : (e > 100 ? 100 : e);
            scale = ldexpf(1.0f, e);
            inv_scale = ldexpf(1.0f, -e);
        }
    }
    if (tid == 0) row_scale[row] = scale;
    const int frags = (K >> 6) * 2;  // (t, s) pairs
    uint4* P_lo = P + (size_t)frags * 64;
    // each thread produces whole 8-half fragments of this row: one per (t, s, g)
    for (int f = tid; f < frags * 4; f += 256) {
        const int g = f & 3, ts = f >> 2;
        const int t = ts >> 1, s = ts & 1;
        const int k0 = 64 * t + 16 * g + 8 * s;
        uint32_t hi[4] = {0, 0, 0, 0}, lo[4] = {0, 0, 0, 0};
        if (live) {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float a = A[(size_t)row * K + k0 + j] * inv_scale;
                const _Float16 h = static_cast<_Float16>(a);
                const _Float16 l = static_cast<_Float16>(a - static_cast<float>(h));
                hi[j >> 1] |= (uint32_t)__builtin_bit_cast(uint16_t, h) << (16 * (j & 1));
                lo[j >> 1] |= (uint32_t)__builtin_bit_cast(uint16_t, l) << (16 * (j & 1));
            }
        }
        const size_t frag_base = (size_t)ts * 64 + (size_t)g * 16;
        if (stacked) {
            P[frag_base + row] = make_uint4(hi[0], hi[1], hi[2], hi[3]);
            P[frag_base + row + 8] = make_uint4(lo[0], lo[1], lo[2], lo[3]);
        } else {
            P[frag_base + row] = make_uint4(hi[0], hi[1], hi[2], hi[3]);
            P_lo[frag_base + row] = make_uint4(lo[0], lo[1], lo[2], lo[3]);
        }
    }
}

__device__ __forceinline__ m40_float4 mfma16x16x32(const uint4& a, const uint4& b, m40_float4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(m40_half8, a),
                                                  __builtin_bit_cast(m40_half8, b), c, 0, 0, 0);
}

// Grid: ceil(ntiles / T) workgroups of T*S waves.  Wave (t, s) owns output columns
// [16*ntile, 16*ntile+16) and k-tiles [s*KT/S, (s+1)*KT/S); slices are summed through LDS in
// ascending s, so the result does not depend on timing.
template <bool STACKED>
__global__ __launch_bounds__(1024) void gemm_mfma_f32xf16_gguf_kernel(
    const uint4* __restrict__ P, const float* __restrict__ row_scale, const uint16_t* __restrict__ B,
    float* __restrict__ C, int M, int N, int K, int T, int S) {
    extern __shared__ float red[];  // [S][T][16][16]
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int t_in = wave % T, s = wave / T;
    const int ntiles = (N + 15) >> 4;
    int ntile = blockIdx.x * T + t_in;
    const bool tile_live = ntile < ntiles;
    if (!tile_live) ntile = ntiles - 1;
    const int j = lane & 15, g = lane >> 4;
    const int col = ntile * 16 + j;
    const int col_c = col < N ? col : N - 1;
    const int KT = K >> 6;
    const int t_begin = (int)(((long long)s * KT) / S), t_end = (int)(((long long)(s + 1) * KT) / S);
    const uint16_t* bcol = B + (size_t)col_c * K + 16 * g;
    const uint4* P_lo = P + (size_t)KT * 2 * 64;

    m40_float4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
    for (int t = t_begin; t < t_end; ++t) {
        const uint4* bp = reinterpret_cast<const uint4*>(bcol + 64 * t);
        const uint4 b0 = m40_load_stream(bp);
        const uint4 b1 = m40_load_stream(bp + 1);
        const uint4 a0 = P[(size_t)(t * 2 + 0) * 64 + lane];
        const uint4 a1 = P[(size_t)(t * 2 + 1) * 64 + lane];
        acc = mfma16x16x32(a0, b0, acc);
        acc = mfma16x16x32(a1, b1, acc);
        if (!STACKED) {
            const uint4 l0 = P_lo[(size_t)(t * 2 + 0) * 64 + lane];
            const uint4 l1 = P_lo[(size_t)(t * 2 + 1) * 64 + lane];
            acc = mfma16x16x32(l0, b0, acc);
            acc = mfma16x16x32(l1, b1, acc);
        }
    }
    // lane (j, g) holds D[4g + r][j], r = 0..3
    if (STACKED) {
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[r] = m40_add_xor32(acc[r]);  // hi rows + lo rows
    }
    float* my = red + ((size_t)(s * T + t_in) * 256);
    if (!STACKED || g < 2) {
#pragma unroll
        for (int r = 0; r < 4; ++r) my[(4 * g + r) * 16 + j] = acc[r];
    }
    __syncthreads();
    if (s == 0 && tile_live && (!STACKED || g < 2)) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int row = 4 * g + r;
            float v = 0.0f;
            for (int ss = 0; ss < S; ++ss) v += red[((size_t)(ss * T + t_in) * 256) + row * 16 + j];
            if (row < M && col < N) C[(size_t)row * N + col] = v * row_scale[row];
        }
    }
}

// ---------------------------------------------------------------------------------------
// Any shape: one wave per output element, lanes stride k.
// ---------------------------------------------------------------------------------------
template <typename AT, bool GGUF>
__global__ __launch_bounds__(256) void gemm_generic_kernel(const AT* __restrict__ A,
                                                           const uint16_t* __restrict__ B,
                                                           float* __restrict__ C, int M, int N, int K) {
    const long long out = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (out >= (long long)M * N) return;
    const int row = (int)(out / N), col = (int)(out % N);
    const int lane = threadIdx.x & 63;
    float acc = 0.0f;
    for (int k = lane; k < K; k += 64) {
        float a;
        if constexpr (sizeof(AT) == 2) a = m40_h2f(A[(size_t)row * K + k]);
        else a = A[(size_t)row * K + k];
        const float b = m40_h2f(GGUF ? B[(size_t)col * K + k] : B[(size_t)k * N + col]);
        acc = fmaf(a, b, acc);
    }
    acc = m40_sum64(acc);
    if (lane == 0) C[(size_t)row * N + col] = acc;
}

// Row-major B[k*N + n]: a thread owns one output column for four rows, k ascending with one
// accumulator per output (the reference's own order, kernels.cu:4999-5032); lanes read
// consecutive n, so every B load is one contiguous 128-byte line per wave.
template <typename AT, typename CT, typename BT = uint16_t>
__global__ __launch_bounds__(256) void gemm_rowmajor_kernel(const AT* __restrict__ A,
                                                            const BT* __restrict__ B,
                                                            CT* __restrict__ C, int M, int N, int K) {
    const int col = blockIdx.x * 256 + threadIdx.x;
    const int row0 = blockIdx.y * 4;
    if (col >= N) return;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int k = 0; k < K; ++k) {
        float b;
        if constexpr (sizeof(BT) == 2) b = m40_h2f(B[(size_t)k * N + col]);
        else b = B[(size_t)k * N + col];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int row = row0 + r < M ? row0 + r : M - 1;
            float a;
            if constexpr (sizeof(AT) == 2) a = m40_h2f(A[(size_t)row * K + k]);
            else a = A[(size_t)row * K + k];
            acc[r] = fmaf(a, b, acc[r]);
        }
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        if (row0 + r < M) {
            if constexpr (sizeof(CT) == 2) C[(size_t)(row0 + r) * N + col] = m40_f2h(acc[r]);
            else C[(size_t)(row0 + r) * N + col] = acc[r];
        }
    }
}

// ---------------------------------------------------------------------------------------
// q8_0 weights, native GGUF blocks {f16 d; int8 qs[32]} (34 bytes) along K.
// One wave per output column; lane handles blocks lane, lane+64, ...; per block the partial
// sum of a*q is formed first and scaled by d once.
// ---------------------------------------------------------------------------------------
template <int ROWS>
__global__ __launch_bounds__(256) void gemm_f32xq80_kernel(const float* __restrict__ A,
                                                           const uint8_t* __restrict__ B,
                                                           float* __restrict__ C, int M, int N, int K,
                                                           int row0) {
    const int col = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (col >= N) return;
    const int lane = threadIdx.x & 63;
    const int nblk = K >> 5;
    const uint8_t* colp = B + (size_t)col * nblk * 34;
    float acc[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) acc[r] = 0.0f;
    for (int b = lane; b < nblk; b += 64) {
        const uint16_t* p16 = reinterpret_cast<const uint16_t*>(colp + (size_t)b * 34);  // 2-byte aligned
        const float d = m40_h2f(p16[0]);
        float part[ROWS];
#pragma unroll
        for (int r = 0; r < ROWS; ++r) part[r] = 0.0f;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const uint16_t two = p16[1 + i];
            const float q0 = (float)(int8_t)(two & 0xff), q1 = (float)(int8_t)(two >> 8);
#pragma unroll
            for (int r = 0; r < ROWS; ++r) {
                const int row = row0 + r < M ? row0 + r : M - 1;
                const float* a = A + (size_t)row * K + b * 32 + 2 * i;
                part[r] = fmaf(a[0], q0, part[r]);
                part[r] = fmaf(a[1], q1, part[r]);
            }
        }
#pragma unroll
        for (int r = 0; r < ROWS; ++r) acc[r] = fmaf(d, part[r], acc[r]);
    }
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        const float s = m40_sum64(acc[r]);
        if (lane == 0 && row0 + r < M) C[(size_t)(row0 + r) * N + col] = s;
    }
}

// ---------------------------------------------------------------------------------------
// q8_0 GEMV for one or two activation rows.  The activations never change between columns, so every
// lane keeps the 32-value slice of the one block position it owns in registers for the whole launch
// and streams only weights: kw waves (a team) split the blocks of a column into contiguous parts of an
// even number of blocks, and a team walks over several columns with the blocks of the next columns
// already in flight.  A block is 34 bytes at 2-byte alignment; with an even block count per column the
// block's offset modulo 4 is twice its parity, which equals the lane's parity, so each lane reads nine
// dwords from the dword-aligned address below its block and shifts by a per-lane constant.  The two
// bytes read beyond an even block belong to the odd block that always follows it in the column; the
// two bytes read before an odd block belong to the even block in front of it.  Quants go int8 -> f32
// exactly; per block the partial sum of a*q is formed first and scaled by d once, as in the kernel
// above.
// ---------------------------------------------------------------------------------------
constexpr int kQ80GemvThreads = 512;
constexpr int kQ80GemvWaves = kQ80GemvThreads / 64;
constexpr int kQ80GemvMaxCols = 32;   // columns per team of waves
constexpr int kQ80GemvDepth = 2;      // columns in flight per wave (N = 14336, K = 4096 at one row: 15.2 / 13.2 / 14.8 / 14.4 us with 1 / 2 / 3 / 4)
constexpr int kQ80GemvChunk = 128;    // blocks of activations staged through LDS at a time (two float4 per thread)
constexpr int kQ80GemvMaxChunks = 64 * kQ80GemvWaves / kQ80GemvChunk;
static_assert(kQ80GemvChunk * 8 == 2 * kQ80GemvThreads, "two float4 per thread and chunk");

struct Q80GemvArgs {
    const float* A;        // [M][K]
    const float* up;       // not null: the activations are silu(A) * up
    const uint8_t* W[2];   // columns [0, N0) come from W[0] into C[0], [N0, N) from W[1] into C[1]
    float* C[2];
    int N0, N, K;
    int kw;                // waves per column: 1, 2, 4 or 8
    int per;               // blocks per wave (even, at most 64)
};

typedef uint32_t q80_u32x4 __attribute__((ext_vector_type(4), aligned(4)));   // dword-aligned 16-byte load

__device__ __forceinline__ float q80_byte(uint32_t w, int n) {
    return static_cast<float>(static_cast<int8_t>(w >> (8 * n)));
}

template <int ROWS>
__global__ __launch_bounds__(kQ80GemvThreads) void q80_gemv_kernel(Q80GemvArgs p) {
    __shared__ float part_s[kQ80GemvWaves][kQ80GemvMaxCols][ROWS];
    __shared__ float act_s[ROWS][kQ80GemvChunk * 33];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int kw = p.kw, tpw = kQ80GemvWaves / kw;
    const int kpart = wave & (kw - 1), team_local = wave / kw;
    const int team = blockIdx.x * tpw + team_local, nteams = gridDim.x * tpw;
    const int nblk = p.K >> 5;
    const unsigned sh = (lane & 1) * 2;
    const int blk_own = kpart * p.per + lane;
    const bool have = lane < p.per && blk_own < nblk;
    // Lanes without a block read a block of their own parity with zero activations, and columns beyond
    // the last one re-read the last one: the loop below has no branch around a load, so the loads of
    // the next columns stay in flight while one column is summed.
    const int blk = have ? blk_own : (lane & 1);
    const size_t col_bytes = (size_t)nblk * 34;
    const size_t blk_off = (size_t)blk * 34 - sh;

    uint32_t w[kQ80GemvDepth][9];
    auto fetch = [&](uint32_t* dst, int col) {
        col = min(col, p.N - 1);
        const int m = col >= p.N0;
        const uint32_t* src = reinterpret_cast<const uint32_t*>(p.W[m] + (size_t)(col - (m ? p.N0 : 0)) * col_bytes + blk_off);
        const q80_u32x4 lo = *reinterpret_cast<const q80_u32x4*>(src);
        const q80_u32x4 hi = *reinterpret_cast<const q80_u32x4*>(src + 4);
        dst[0] = lo.x; dst[1] = lo.y; dst[2] = lo.z; dst[3] = lo.w;
        dst[4] = hi.x; dst[5] = hi.y; dst[6] = hi.z; dst[7] = hi.w;
        dst[8] = src[8];
    };
#pragma unroll
    for (int d = 0; d < kQ80GemvDepth; ++d) fetch(w[d], team + d * nteams);

    // Activations: the workgroup reads each row once, coalesced (SwiGLU applied here when asked for), and
    // passes it through LDS in chunks of 128 blocks, from which every lane picks the slice of its block.
    // Rows of a block sit 33 floats apart so that the per-lane reads spread over the banks.
    float a[ROWS][32];
#pragma unroll
    for (int r = 0; r < ROWS; ++r)
#pragma unroll
        for (int q = 0; q < 32; ++q) a[r][q] = 0.0f;
    {
        const int nchunks = (nblk + kQ80GemvChunk - 1) / kQ80GemvChunk;
        float4 g[ROWS][kQ80GemvMaxChunks][2];
#pragma unroll
        for (int c = 0; c < kQ80GemvMaxChunks; ++c) {
            if (c >= nchunks) break;
#pragma unroll
            for (int r = 0; r < ROWS; ++r)
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const int e = (c * kQ80GemvChunk * 8 + h * kQ80GemvThreads + threadIdx.x) * 4;
                    float4 v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                    if (e < p.K) {
                        v = *reinterpret_cast<const float4*>(p.A + (size_t)r * p.K + e);
                        if (p.up) {
                            const float4 u = *reinterpret_cast<const float4*>(p.up + (size_t)r * p.K + e);
                            v.x = v.x / (1.0f + expf(-v.x)) * u.x;
                            v.y = v.y / (1.0f + expf(-v.y)) * u.y;
                            v.z = v.z / (1.0f + expf(-v.z)) * u.z;
                            v.w = v.w / (1.0f + expf(-v.w)) * u.w;
                        }
                    }
                    g[r][c][h] = v;
                }
        }
#pragma unroll
        for (int c = 0; c < kQ80GemvMaxChunks; ++c) {
            if (c >= nchunks) break;
#pragma unroll
            for (int r = 0; r < ROWS; ++r)
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const int e = h * kQ80GemvThreads + threadIdx.x;     // float4 index inside the chunk
                    float* dst = &act_s[r][(e >> 3) * 33 + (e & 7) * 4];
                    dst[0] = g[r][c][h].x; dst[1] = g[r][c][h].y; dst[2] = g[r][c][h].z; dst[3] = g[r][c][h].w;
                }
            __syncthreads();
            if (have && blk_own / kQ80GemvChunk == c) {
#pragma unroll
                for (int r = 0; r < ROWS; ++r)
#pragma unroll
                    for (int q = 0; q < 32; ++q) a[r][q] = act_s[r][(blk_own % kQ80GemvChunk) * 33 + q];
            }
            __syncthreads();
        }
    }

    const int team_cols = team < p.N ? (p.N - team + nteams - 1) / nteams : 0;
    for (int i0 = 0; i0 < team_cols; i0 += kQ80GemvDepth) {
#pragma unroll
        for (int d = 0; d < kQ80GemvDepth; ++d) {
            const int col = team + (i0 + d) * nteams;
            float acc[ROWS];
#pragma unroll
            for (int r = 0; r < ROWS; ++r) acc[r] = 0.0f;
            uint32_t x[9];
#pragma unroll
            for (int i = 0; i < 8; ++i) x[i] = __builtin_amdgcn_alignbyte(w[d][i + 1], w[d][i], sh);
            x[8] = __builtin_amdgcn_alignbyte(0u, w[d][8], sh);
            fetch(w[d], col + kQ80GemvDepth * nteams);
            const float dscale = m40_h2f(static_cast<uint16_t>(x[0] & 0xffffu));
#pragma unroll
            for (int q = 0; q < 32; ++q) {
                const float f = q80_byte(x[(q + 2) >> 2], (q + 2) & 3);
#pragma unroll
                for (int r = 0; r < ROWS; ++r) acc[r] = fmaf(a[r][q], f, acc[r]);
            }
            const int m = col >= p.N0;
            const int c = col - (m ? p.N0 : 0), nm = m ? p.N - p.N0 : p.N0;
#pragma unroll
            for (int r = 0; r < ROWS; ++r) {
                const float s = m40_sum64(acc[r] * dscale);
                if (lane == 0 && col < p.N) {
                    if (kw == 1) p.C[m][(size_t)r * nm + c] = s;
                    else part_s[wave][i0 + d][r] = s;
                }
            }
        }
    }
    if (kw == 1) return;
    __syncthreads();
    // One thread per (team, column, row) adds the K-parts in a fixed order.
    for (int t = threadIdx.x; t < tpw * kQ80GemvMaxCols * ROWS; t += kQ80GemvThreads) {
        const int r = t % ROWS, i = (t / ROWS) % kQ80GemvMaxCols, tl = t / (ROWS * kQ80GemvMaxCols);
        const int col = blockIdx.x * tpw + tl + i * nteams;
        if (col >= p.N) continue;
        float s = 0.0f;
        for (int k = 0; k < kw; ++k) s += part_s[tl * kw + k][i][r];
        const int m = col >= p.N0;
        const int c = col - (m ? p.N0 : 0), nm = m ? p.N - p.N0 : p.N0;
        p.C[m][(size_t)r * nm + c] = s;
    }
}

bool q80_gemv_supported(int M, int N, int K) {
    // beyond two rows the f32 multiply-adds outweigh the weight stream and the matrix-core kernel is faster
    return M >= 1 && M <= 2 && N >= 1 && K % 64 == 0 && K <= 64 * 32 * kQ80GemvWaves;
}

// W1/C1 may be null (one matrix of N columns); otherwise both matrices have N columns.
int launch_q80_gemv(hipStream_t stream, const float* A, const float* up, const uint8_t* W0, float* C0,
                    const uint8_t* W1, float* C1, int M, int N, int K) {
    Q80GemvArgs p;
    p.A = A; p.up = up;
    p.W[0] = W0; p.C[0] = C0; p.W[1] = W1; p.C[1] = C1;
    p.N0 = N; p.N = W1 ? 2 * N : N; p.K = K;
    const int nblk = K / 32;
    p.kw = 1;
    while (p.kw * 64 < nblk) p.kw *= 2;
    p.per = (nblk + p.kw - 1) / p.kw;
    p.per += p.per & 1;
    const int tpw = kQ80GemvWaves / p.kw;
    const int cols_target = 16;   // columns per team: amortises the activation staging; measured best of 4..32
    int nteams = (p.N + cols_target - 1) / cols_target;
    int blocks = (nteams + tpw - 1) / tpw;
    if (blocks < 1) blocks = 1;
    if ((p.N + blocks * tpw - 1) / (blocks * tpw) > kQ80GemvMaxCols) return -2;
    if (M == 1) q80_gemv_kernel<1><<<blocks, kQ80GemvThreads, 0, stream>>>(p);
    else q80_gemv_kernel<2><<<blocks, kQ80GemvThreads, 0, stream>>>(p);
    return hipGetLastError() == hipSuccess ? 0 : -2;
}

// GGUF f16 weights [N][K] -> f32 [K][N] (the reference's "column-major NT" operand of its f32 x f32 route,
// kernels.cu:5054-5066): consecutive threads write consecutive n.
__global__ __launch_bounds__(256) void materialize_gguf_kernel(const uint16_t* __restrict__ B, float* __restrict__ Bt,
                                                               int N, int K) {
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (size_t)N * K) return;
    const size_t n = idx % (size_t)N, k = idx / (size_t)N;
    Bt[idx] = m40_h2f(B[n * (size_t)K + k]);
}

int pick_mfma_shape(int ntiles, int KT, int* T, int* S) {
    // Aim for a few thousand waves in flight and >= 512 workgroups where N allows it.
    int s = 1;
    while (s < 16 && (long long)ntiles * s < 4096 && KT / (s * 2) >= 2) s *= 2;
    int t = 1;
    while (t * s < 16 && t < 4 && ntiles / (t * 2) >= 1024) t *= 2;
    *T = t;
    *S = s;
    return 0;
}

}  // namespace

int m40_launch_gemm_f32xf16_gguf(M40llmCudaContext* ctx, hipStream_t stream, uint32_t stream_kind,
                                 const float* A, const uint16_t* B, float* C, int M, int N, int K) {
    if (M <= 0 || N <= 0 || K <= 0) return -2;
    (void)hipGetLastError();
    const bool fast = (K % 8 == 0) && m40_aligned16(A) && m40_aligned16(B);
    if (fast && M == 1) {
        const GemvShape g = gemv_pick_shape(N, K);
        if (g.ksplit == 4) gemv_f32xf16_gguf_kernel<2, 4><<<g.blocks, 256, 0, stream>>>(A, B, C, N, K);
        else if (g.cols == 4) gemv_f32xf16_gguf_kernel<4, 1><<<g.blocks, 256, 0, stream>>>(A, B, C, N, K);
        else if (g.cols == 2) gemv_f32xf16_gguf_kernel<2, 1><<<g.blocks, 256, 0, stream>>>(A, B, C, N, K);
        else gemv_f32xf16_gguf_kernel<1, 1><<<g.blocks, 256, 0, stream>>>(A, B, C, N, K);
    } else if (fast && m40_gemm_tiled_supported(A, B, M, N, K)) {
        // many rows (prefill): one pass over the weights for all rows; declined (1) only when its packing buffer
        // cannot be provided, then the skinny kernels take the rows 16 at a time
        const int rc = m40_launch_gemm_tiled(ctx, stream, stream_kind, A, B, C, M, N, K);
        if (rc != 1) return rc;
        return m40_launch_skinny(ctx, stream, stream_kind, 0, A, nullptr, B, C, nullptr, nullptr, M, N, K);
    } else if (fast && N <= 8192 && m40_rows_gemv_supported(M, K)) {
        // few columns: the vector-ALU row kernel needs no K split and no second launch
        return m40_rows_gemv_residual(stream, A, B, nullptr, C, M, N, K);
    } else if (fast && m40_skinny_supported(ctx, stream_kind, M, N, K, 0)) {
        return m40_launch_skinny(ctx, stream, stream_kind, 0, A, nullptr, B, C, nullptr, nullptr, M, N, K);
    } else if (fast && K % 64 == 0 && (size_t)K * 64 <= ctx->scratch[stream_kind].gemm_pack_bytes - 256) {
        M40StreamScratch& sc = ctx->scratch[stream_kind];
        const int KT = K >> 6;
        const int ntiles = (N + 15) >> 4;
        int T, S;
        pick_mfma_shape(ntiles, KT, &T, &S);
        // scratch: [row_scale: 16 floats (64 B, padded to 256)] [P hi (+lo)]
        float* row_scale = static_cast<float*>(sc.gemm_pack);
        uint4* P = reinterpret_cast<uint4*>(static_cast<char*>(sc.gemm_pack) + 256);
        for (int r0 = 0; r0 < M; r0 += 16) {
            const int m = M - r0 < 16 ? M - r0 : 16;
            const bool stacked = m <= 8;
            pack_a_hilo_kernel<<<stacked ? 8 : 16, 256, 0, stream>>>(A + (size_t)r0 * K, m, K, stacked ? 1 : 0,
                                                                     P, row_scale);
            const size_t lds = (size_t)S * T * 256 * sizeof(float);
            const int blocks = (ntiles + T - 1) / T;
            if (stacked) {
                gemm_mfma_f32xf16_gguf_kernel<true><<<blocks, T * S * 64, lds, stream>>>(
                    P, row_scale, B, C + (size_t)r0 * N, m, N, K, T, S);
            } else {
                gemm_mfma_f32xf16_gguf_kernel<false><<<blocks, T * S * 64, lds, stream>>>(
                    P, row_scale, B, C + (size_t)r0 * N, m, N, K, T, S);
            }
        }
    } else {
        const long long outs = (long long)M * N;
        gemm_generic_kernel<float, true><<<(unsigned)((outs + 3) / 4), 256, 0, stream>>>(A, B, C, M, N, K);
    }
    return hipGetLastError() == hipSuccess ? 0 : -2;
}

// Up to three f16 weight matrices applied to the same activations.  Many rows: one packing pass and one launch of
// the tiled kernel; otherwise (or when that declines) one GEMM per matrix.
static int launch_multi_f32xf16(M40llmCudaContext* ctx, hipStream_t stream, uint32_t stream_kind, const float* A, int M, int K,
                                int n_mats, const uint16_t* const* B, const int* N, float* const* C) {
    bool tiled = (K % 8 == 0);
    for (int i = 0; i < n_mats && tiled; ++i) tiled = m40_gemm_tiled_supported(A, B[i], M, N[i], K);
    if (tiled) {
        const int rc = m40_launch_gemm_tiled_multi(ctx, stream, stream_kind, A, M, K, n_mats, B, N, C);
        if (rc != 1) return rc;
    }
    for (int i = 0; i < n_mats; ++i) {
        const int rc = m40_launch_gemm_f32xf16_gguf(ctx, stream, stream_kind, A, B[i], C[i], M, N[i], K);
        if (rc != 0) return rc;
    }
    return 0;
}

static int launch_q80(M40llmCudaContext* ctx, hipStream_t stream, uint32_t stream_kind, const float* A, const uint8_t* B,
                      float* C, int M, int N, int K) {
    if (m40_aligned16(B) && m40_aligned16(A) && q80_gemv_supported(M, N, K))
        return launch_q80_gemv(stream, A, nullptr, B, C, nullptr, nullptr, M, N, K);
    if (m40_aligned16(B) && m40_aligned16(A) && m40_q80_i8_supported(ctx, stream_kind, M, N, K))
        return m40_launch_q80_i8(ctx, stream, stream_kind, A, B, C, M, N, K);
    if (m40_aligned16(B) && m40_aligned16(A) && m40_skinny_supported(ctx, stream_kind, M, N, K, 1))
        return m40_launch_skinny(ctx, stream, stream_kind, 1, A, nullptr, B, C, nullptr, nullptr, M, N, K);
    (void)hipGetLastError();
    for (int r0 = 0; r0 < M; r0 += 4) {
        const int m = M - r0;
        if (m >= 4) gemm_f32xq80_kernel<4><<<(N + 3) / 4, 256, 0, stream>>>(A, B, C, M, N, K, r0);
        else if (m == 3) gemm_f32xq80_kernel<3><<<(N + 3) / 4, 256, 0, stream>>>(A, B, C, M, N, K, r0);
        else if (m == 2) gemm_f32xq80_kernel<2><<<(N + 3) / 4, 256, 0, stream>>>(A, B, C, M, N, K, r0);
        else gemm_f32xq80_kernel<1><<<(N + 3) / 4, 256, 0, stream>>>(A, B, C, M, N, K, r0);
    }
    return hipGetLastError() == hipSuccess ? 0 : -2;
}

extern "C" {

int m40llm_gemm_f32xf16_gguf_f32(M40llmCudaContext* ctx, const void* d_A_f32, const void* d_B_f16,
                                 void* d_C_f32, int M, int N, int K) {
    if (!ctx || !d_A_f32 || !d_B_f16 || !d_C_f32) return -1;
    int rc = m40_launch_gemm_f32xf16_gguf(ctx, ctx->prefill_stream, 0, static_cast<const float*>(d_A_f32),
                                          static_cast<const uint16_t*>(d_B_f16), static_cast<float*>(d_C_f32),
                                          M, N, K);
    if (rc != 0) return rc;
    return hipStreamSynchronize(ctx->prefill_stream) == hipSuccess ? 0 : -3;
}

int m40llm_ext_gemm_f32xf16_gguf_f32_multi_async(M40llmCudaContext* ctx, const void* d_A_f32, int M, int K, int n_mats,
                                                 const void* d_B0_f16, int N0, void* d_C0_f32, const void* d_B1_f16, int N1,
                                                 void* d_C1_f32, const void* d_B2_f16, int N2, void* d_C2_f32,
                                                 uint32_t stream_kind) {
    if (!ctx || !d_A_f32) return -1;
    if (n_mats < 1 || n_mats > 3 || M <= 0 || K <= 0) return -2;
    const uint16_t* B[3] = {static_cast<const uint16_t*>(d_B0_f16), static_cast<const uint16_t*>(d_B1_f16),
                            static_cast<const uint16_t*>(d_B2_f16)};
    float* C[3] = {static_cast<float*>(d_C0_f32), static_cast<float*>(d_C1_f32), static_cast<float*>(d_C2_f32)};
    const int N[3] = {N0, N1, N2};
    for (int i = 0; i < n_mats; ++i) {
        if (!B[i] || !C[i]) return -1;
        if (N[i] <= 0) return -2;
    }
    if (m40_ensure_device(ctx) != 0) return -2;
    hipStream_t stream = m40_select_stream(ctx, stream_kind);
    if (!stream) return -3;
    return launch_multi_f32xf16(ctx, stream, stream_kind, static_cast<const float*>(d_A_f32), M, K, n_mats, B, N, C);
}

int m40llm_ext_prefill_gemm_fused_async(M40llmCudaContext* ctx, uint32_t source_kind, const void* d_a_f32, const void* d_a2_f32,
                                        const void* d_norm_weight, uint32_t norm_weight_dtype, float eps, int M, int K,
                                        int n_mats, const void* d_B0_f16, int N0, void* d_C0_f32, const void* d_R0_f32,
                                        const void* d_B1_f16, int N1, void* d_C1_f32, const void* d_B2_f16, int N2,
                                        void* d_C2_f32, uint32_t stream_kind) {
    if (!ctx || !d_a_f32) return -1;
    if (source_kind > 2u || n_mats < 1 || n_mats > 3 || M <= 0 || K <= 0) return -2;
    if (source_kind == 1u && (!d_norm_weight || norm_weight_dtype > 1u)) return -1;
    if (source_kind == 2u && !d_a2_f32) return -1;
    if (d_R0_f32 && n_mats != 1) return -2;
    const uint16_t* B[3] = {static_cast<const uint16_t*>(d_B0_f16), static_cast<const uint16_t*>(d_B1_f16),
                            static_cast<const uint16_t*>(d_B2_f16)};
    float* C[3] = {static_cast<float*>(d_C0_f32), static_cast<float*>(d_C1_f32), static_cast<float*>(d_C2_f32)};
    const float* R[3] = {static_cast<const float*>(d_R0_f32), nullptr, nullptr};
    const int N[3] = {N0, N1, N2};
    for (int i = 0; i < n_mats; ++i) {
        if (!B[i] || !C[i]) return -1;
        if (N[i] <= 0) return -2;
    }
    if (m40_ensure_device(ctx) != 0) return -2;
    hipStream_t stream = m40_select_stream(ctx, stream_kind);
    if (!stream) return -3;
    const float* A = static_cast<const float*>(d_a_f32);
    bool tiled = true;
    for (int i = 0; i < n_mats && tiled; ++i) tiled = m40_gemm_tiled_supported(A, B[i], M, N[i], K);
    if (source_kind == 1u) tiled = tiled && m40_aligned16(d_norm_weight);
    if (source_kind == 2u) tiled = tiled && m40_aligned16(d_a2_f32);
    if (!tiled) return 1;
    return m40_launch_gemm_tiled_fused(ctx, stream, stream_kind, (int)source_kind, A, static_cast<const float*>(d_a2_f32),
                                       d_norm_weight, norm_weight_dtype, eps, M, K, n_mats, B, N, C, R);
}

int m40llm_ext_gemm_f32xf16_gguf_f32_async(M40llmCudaContext* ctx, const void* d_A_f32, const void* d_B_f16,
                                           void* d_C_f32, int M, int N, int K, uint32_t stream_kind) {
    if (!ctx || !d_A_f32 || !d_B_f16 || !d_C_f32) return -1;
    hipStream_t stream = m40_select_stream(ctx, stream_kind);
    if (!stream) return -4;
    return m40_launch_gemm_f32xf16_gguf(ctx, stream, stream_kind, static_cast<const float*>(d_A_f32),
                                        static_cast<const uint16_t*>(d_B_f16), static_cast<float*>(d_C_f32),
                                        M, N, K);
}

int m40llm_gemm_f32xf16_f32(M40llmCudaContext* ctx, const void* d_A_f32, const void* d_B_f16, void* d_C_f32,
                            int M, int N, int K) {
    if (!ctx || !d_A_f32 || !d_B_f16 || !d_C_f32) return -1;
    if (M <= 0 || N <= 0 || K <= 0) return -2;
    (void)hipGetLastError();
    dim3 grid((N + 255) / 256, (M + 3) / 4);
    gemm_rowmajor_kernel<float, float><<<grid, 256, 0, ctx->prefill_stream>>>(
        static_cast<const float*>(d_A_f32), static_cast<const uint16_t*>(d_B_f16), static_cast<float*>(d_C_f32),
        M, N, K);
    if (hipGetLastError() != hipSuccess) return -2;
    return hipStreamSynchronize(ctx->prefill_stream) == hipSuccess ? 0 : -3;
}

int m40llm_materialize_gguf_f16_to_f32_colmajor_nt(M40llmCudaContext* ctx, const void* d_B_f16,
                                                   void* d_B_f32_colmajor_nt, int N, int K) {
    if (!ctx || !d_B_f16 || !d_B_f32_colmajor_nt) return -1;
    if (N <= 0 || K <= 0) return -2;
    (void)hipGetLastError();
    const size_t total = (size_t)N * K;
    materialize_gguf_kernel<<<(unsigned)((total + 255) / 256), 256, 0, ctx->prefill_stream>>>(
        static_cast<const uint16_t*>(d_B_f16), static_cast<float*>(d_B_f32_colmajor_nt), N, K);
    if (hipGetLastError() != hipSuccess) return -3;
    return hipStreamSynchronize(ctx->prefill_stream) == hipSuccess ? 0 : -4;
}

// The reference routes this through cublasSgemm (kernels.cu:5217-5242); same operands, plain f32 accumulation here.
int m40llm_gemm_f32xf32_f32_async(M40llmCudaContext* ctx, const void* d_A_f32, const void* d_B_f32_colmajor_nt,
                                  void* d_C_f32, int M, int N, int K) {
    if (!ctx || !d_A_f32 || !d_B_f32_colmajor_nt || !d_C_f32) return -1;
    if (M <= 0 || N <= 0 || K <= 0) return -2;
    (void)hipGetLastError();
    dim3 grid((N + 255) / 256, (M + 3) / 4);
    gemm_rowmajor_kernel<float, float, float><<<grid, 256, 0, ctx->prefill_stream>>>(
        static_cast<const float*>(d_A_f32), static_cast<const float*>(d_B_f32_colmajor_nt),
        static_cast<float*>(d_C_f32), M, N, K);
    return hipGetLastError() == hipSuccess ? 0 : -3;
}

int m40llm_gemm_f32xf32_f32(M40llmCudaContext* ctx, const void* d_A_f32, const void* d_B_f32_colmajor_nt,
                            void* d_C_f32, int M, int N, int K) {
    const int rc = m40llm_gemm_f32xf32_f32_async(ctx, d_A_f32, d_B_f32_colmajor_nt, d_C_f32, M, N, K);
    if (rc != 0) return rc;
    return hipStreamSynchronize(ctx->prefill_stream) == hipSuccess ? 0 : -4;
}

int m40llm_gemm_f16xf16_f32(M40llmCudaContext* ctx, const void* d_A_f16, const void* d_B_f16, void* d_C_f32,
                            int M, int N, int K) {
    if (!ctx || !d_A_f16 || !d_B_f16 || !d_C_f32) return -1;
    if (M <= 0 || N <= 0 || K <= 0) return -2;
    (void)hipGetLastError();
    dim3 grid((N + 255) / 256, (M + 3) / 4);
    gemm_rowmajor_kernel<uint16_t, float><<<grid, 256, 0, ctx->prefill_stream>>>(
        static_cast<const uint16_t*>(d_A_f16), static_cast<const uint16_t*>(d_B_f16),
        static_cast<float*>(d_C_f32), M, N, K);
    if (hipGetLastError() != hipSuccess) return -2;
    return hipStreamSynchronize(ctx->prefill_stream) == hipSuccess ? 0 : -3;
}

int m40llm_gemm_f16_storage_f32_compute(M40llmCudaContext* ctx, const void* d_A, const void* d_B, void* d_C,
                                        int M, int N, int K) {
    if (!ctx || !d_A || !d_B || !d_C) return -1;
    if (M <= 0 || N <= 0 || K <= 0) return -2;
    (void)hipGetLastError();
    dim3 grid((N + 255) / 256, (M + 3) / 4);
    gemm_rowmajor_kernel<uint16_t, uint16_t><<<grid, 256, 0, ctx->prefill_stream>>>(
        static_cast<const uint16_t*>(d_A), static_cast<const uint16_t*>(d_B), static_cast<uint16_t*>(d_C), M, N, K);
    if (hipGetLastError() != hipSuccess) return -2;
    return hipStreamSynchronize(ctx->prefill_stream) == hipSuccess ? 0 : -3;
}

int m40llm_ext_gemm_f32xq80_gguf_f32(M40llmCudaContext* ctx, const void* d_A_f32, const void* d_B_q80,
                                     void* d_C_f32, int M, int N, int K) {
    if (!ctx || !d_A_f32 || !d_B_q80 || !d_C_f32) return -1;
    if (M <= 0 || N <= 0 || K <= 0 || K % 32 != 0) return -2;
    int rc = launch_q80(ctx, ctx->prefill_stream, 0, static_cast<const float*>(d_A_f32),
                        static_cast<const uint8_t*>(d_B_q80), static_cast<float*>(d_C_f32), M, N, K);
    if (rc != 0) return rc;
    return hipStreamSynchronize(ctx->prefill_stream) == hipSuccess ? 0 : -3;
}

int m40llm_ext_gemm_f32xq80_gguf_f32_async(M40llmCudaContext* ctx, const void* d_A_f32, const void* d_B_q80,
                                           void* d_C_f32, int M, int N, int K, uint32_t stream_kind) {
    if (!ctx || !d_A_f32 || !d_B_q80 || !d_C_f32) return -1;
    if (M <= 0 || N <= 0 || K <= 0 || K % 32 != 0) return -2;
    hipStream_t stream = m40_select_stream(ctx, stream_kind);
    if (!stream) return -4;
    return launch_q80(ctx, stream, stream_kind, static_cast<const float*>(d_A_f32),
                      static_cast<const uint8_t*>(d_B_q80), static_cast<float*>(d_C_f32), M, N, K);
}

int m40llm_ext_ffn_swiglu_q80_f32_async(M40llmCudaContext* ctx, const void* d_x_f32, const void* d_w_gate_q80,
                                        const void* d_w_up_q80, const void* d_w_down_q80,
                                        void* d_scratch_f32, void* d_out_f32, int M, int d_model, int ffn) {
    if (!ctx || !d_x_f32 || !d_w_gate_q80 || !d_w_up_q80 || !d_w_down_q80 || !d_scratch_f32 || !d_out_f32)
        return -1;
    if (M <= 0 || d_model <= 0 || ffn <= 0 || d_model % 32 != 0 || ffn % 32 != 0) return -2;
    float* gate = static_cast<float*>(d_scratch_f32);
    float* up = gate + (size_t)M * ffn;
    const float* x = static_cast<const float*>(d_x_f32);
    const uint8_t* wg = static_cast<const uint8_t*>(d_w_gate_q80);
    const uint8_t* wu = static_cast<const uint8_t*>(d_w_up_q80);
    const uint8_t* wd = static_cast<const uint8_t*>(d_w_down_q80);
    float* out = static_cast<float*>(d_out_f32);
    const bool aligned = m40_aligned16(wg) && m40_aligned16(wu) && m40_aligned16(wd) && m40_aligned16(x) &&
                         m40_aligned16(gate) && m40_aligned16(up);
    // two rows of a large FFN: the int8 form's three launches (52.8 us at 4096 / 14336) beat the two GEMV launches (63.5 us)
    const bool two_rows_i8 = M == 2 && (size_t)ffn * d_model >= ((size_t)1 << 24) && aligned &&
                             m40_q80_i8_supported(ctx, 1, M, ffn, d_model) && m40_q80_i8_supported(ctx, 1, M, d_model, ffn);
    if (!two_rows_i8 && aligned && q80_gemv_supported(M, ffn, d_model) && q80_gemv_supported(M, d_model, ffn)) {
        // gate and up in one launch; SwiGLU is applied while each lane loads its slices for the down projection
        (void)hipGetLastError();
        int rc = launch_q80_gemv(ctx->decode_stream, x, nullptr, wg, gate, wu, up, M, ffn, d_model);
        if (rc != 0) return rc;
        return launch_q80_gemv(ctx->decode_stream, gate, up, wd, out, nullptr, nullptr, M, d_model, ffn);
    }
    if (aligned && m40_q80_i8_supported(ctx, 1, M, ffn, d_model) && m40_q80_i8_supported(ctx, 1, M, d_model, ffn)) {
        // digit planes of x, gate / up / SwiGLU / digit planes of the hidden row, down projection: three launches
        const int rc = m40_launch_q80_i8_ffn(ctx, ctx->decode_stream, 1, x, wg, wu, wd, out, M, d_model, ffn);
        if (rc == 0) return 0;
    }
    if (aligned &&
        m40_skinny_supported(ctx, 1, M, ffn, d_model, 1) &&
        m40_skinny_supported(ctx, 1, M, d_model, ffn, 1)) {
        // gate and up in one launch; SwiGLU is applied while the hidden row is packed for the down projection
        int rc = m40_launch_skinny(ctx, ctx->decode_stream, 1, 1, x, nullptr, wg, gate, wu, up, M, ffn, d_model);
        if (rc != 0) return rc;
        return m40_launch_skinny(ctx, ctx->decode_stream, 1, 1, gate, up, wd, out, nullptr, nullptr, M, d_model, ffn);
    }
    int rc = launch_q80(ctx, ctx->decode_stream, 1, x, wg, gate, M, ffn, d_model);
    if (rc != 0) return rc;
    rc = launch_q80(ctx, ctx->decode_stream, 1, x, wu, up, M, ffn, d_model);
    if (rc != 0) return rc;
    rc = m40llm_swiglu_f32_async(ctx, gate, up, gate, (size_t)M * ffn);
    if (rc != 0) return -3;
    return launch_q80(ctx, ctx->decode_stream, 1, gate, wd, out, M, d_model, ffn);
}

}  // extern "C"
