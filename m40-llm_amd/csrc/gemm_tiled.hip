// Many-row GEMM for prefill: C[M,N] f32 = A[M,K] f32 x B (f16, GGUF order [N][K]), f32 accumulation, on the
// matrix cores.  Same contract as the reference's gemm_f32xf16_gguf_f32 (cuda/kernels.cu:5037-5052); used when M is
// beyond what the skinny kernels serve in one pass, where they would stream the weights once per 16 rows.
//
// Tiling: a workgroup of 4 waves owns a 128 x 128 tile of C and walks K in steps of 32.  Per step the 128 x 32 block
// of A, split into an f16 high part and an f16 low part under a per-row power-of-two scale (a = scale (hi + lo) up to
// 2^-22 relative; the scale multiplies the row of C at the end), is written to
// LDS with the 128 x 32 block of B; each wave then computes its 64 x 64 quarter with
// v_mfma_f32_16x16x32_f16, once with the high and once with the low part, so the products carry the f32 activations'
// precision.  The global loads of the next three steps are in flight (three rotating register sets) while a step
// computes from one LDS buffer and the following step's data moves into the other: one barrier per step.
//
// Larger grids (from 9/16 of a 128 x 256 tile per CU) take a second kernel built the same way round a wider tile and the
// direct global-to-LDS loads of gfx950 (gemm_tiled_wide_kernel, below): what bounded the 128 x 128 kernel was not
// arithmetic but the issue of its memory instructions, all of them between the barrier and the first matrix instruction.
//
// The split is done once per call by a packing pass (A -> two f16 planes in a per-stream buffer that grows on
// demand), so the 128 x 128 tiles along N do not each repeat it.  When the buffer cannot be grown (the stream is being
// captured) the launch is declined and the caller falls back to the skinny kernels.  Several weight matrices that
// share A (Q/K/V, gate/up) can be served by one packing pass and one launch.
#include "common.hpp"

#include <type_traits>
#include <utility>

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kBM = 128, kBN = 128, kBK = 32;
constexpr int kStride = kBK;                     // halves per LDS row: 64 B, no padding; 16-byte chunks are swizzled (below)
constexpr int kTileHalves = kBM * kStride;       // one 128 x 32 operand block
constexpr int kBufHalves = 3 * kTileHalves;      // A high, A low, B
constexpr int kThreads = 256;
constexpr int kMaxMats = 3;

// Up to three weight matrices that share the activations (Q/K/V, gate/up): their column tiles are laid side by side.
struct TiledMats {
    int n;
    const uint16_t* B[kMaxMats];
    float* C[kMaxMats];
    const float* R[kMaxMats];       // not null: C = R + product (R may be C itself)
    int N[kMaxMats];
    int tile_start[kMaxMats + 1];   // first column tile of each matrix; [n] = total
};

// Where the rows of A come from: as they are, RMSNorm of the rows (what m40llm_rms_norm_f32_weighted writes: the same
// sums in the same order, cuda/kernels.cu:770-807), or SwiGLU of two arrays (kernels.cu:869-880).  The packing pass
// produces them on the fly, so the normalised / activated rows are never written out as f32 and read back.
struct PackSource {
    const float* a;
    const float* a2;           // SwiGLU: the up array (a is gate)
    const void* norm_w;        // RMSNorm weights
    uint32_t norm_dtype;       // 0 f16, 1 f32
    float eps;
};
enum { kPackPlain = 0, kPackNorm = 1, kPackSwiglu = 2 };

struct StepRegs {   // one K step of one thread: rows lrow and lrow + 64, 16 bytes (8 halves) of each
    uint4 ah[2], al[2], b[2];
};

// A [M][K] f32 -> hi, lo [M][K] f16 planes and one scale per row: a = scale * (hi + lo) up to 2^-22 relative.  The scale is
// the power of two that brings the row's largest magnitude into [2^10, 2^11) -- any finite f32 row fits the f16 planes,
// and small elements keep their low part out of the f16 subnormals.  The row stays in registers between the maximum and
// the split (up to K = 16384; beyond that it is read a second time).  A row that holds an
// infinity or a NaN is packed unscaled with those elements as they are (their low parts zero), so that its products come
// out non-finite as the f32 arithmetic of the reference would give them (cuda/kernels.cu:5037-5052), never as a finite
// value.
constexpr int kPackChunks = 8;       // 8-element chunks a thread keeps in registers

// SwiGLU of one element, the expression of swiglu_kernel (cuda/kernels.cu:869-880)
__device__ __forceinline__ float tiled_swiglu(float g, float u) {
    const float silu = g / (1.0f + expf(-g));
    return silu * u;
}

__device__ __forceinline__ float pack_abs_or_inf(float v) { return fabsf(v) <= 3.402823466e+38f ? fabsf(v) : INFINITY; }

__device__ __forceinline__ void pack_split8(const float4& x0, const float4& x1, float inv_scale, half8& h, half8& l) {
    const float x[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const bool finite = fabsf(x[j]) <= 3.402823466e+38f;
        // (a row with a non-finite element is not scaled: a finite neighbour beyond the f16 range then saturates, in a
        // row whose products are non-finite wherever that element meets a non-zero weight)
        const float xs = finite ? fminf(fmaxf(x[j] * inv_scale, -65504.0f), 65504.0f) : x[j];
        h[j] = static_cast<_Float16>(xs);
        l[j] = finite ? static_cast<_Float16>(xs - static_cast<float>(h[j])) : static_cast<_Float16>(0.0f);
    }
}

// ROW_THREADS = 64: a wave per row, four rows per workgroup, no barrier (K <= 4096 keeps the row in registers);
// 256: a workgroup per row (always for the RMSNorm source, whose sum of squares is formed with the thread layout and
// order of rms_norm_kernel so that the fused form gives the bits of the two-launch form).
template <int ROW_THREADS, int KIND>
__global__ __launch_bounds__(256) void pack_hilo_planes_kernel(PackSource src_args, _Float16* __restrict__ hi,
                                                               _Float16* __restrict__ lo, float* __restrict__ row_scale,
                                                               int M, int K) {
    static_assert(KIND != kPackNorm || ROW_THREADS == 256, "the norm's sums follow rms_norm_kernel's layout");
    __shared__ float wave_max[4];
    __shared__ float wave_sums[4];
    constexpr int kRowsPerGroup = 256 / ROW_THREADS;
    const int row = (int)blockIdx.x * kRowsPerGroup + (int)threadIdx.x / ROW_THREADS, tid = (int)threadIdx.x % ROW_THREADS;
    if (ROW_THREADS == 64 && row >= M) return;          // whole waves: no barrier in this form
    const float4* src = reinterpret_cast<const float4*>(src_args.a + (size_t)row * K);
    const float4* src2 = KIND == kPackSwiglu ? reinterpret_cast<const float4*>(src_args.a2 + (size_t)row * K) : nullptr;
    const int chunks = K >> 3;                     // K is a multiple of 32
    float norm_scale = 1.0f;
    if (KIND == kPackNorm) {
        float ss = 0.0f;
        for (int i = tid; i < K / 4; i += 256) {
            const float4 v = src[i];
            ss = fmaf(v.x, v.x, ss);
            ss = fmaf(v.y, v.y, ss);
            ss = fmaf(v.z, v.z, ss);
            ss = fmaf(v.w, v.w, ss);
        }
        ss = m40_sum64(ss);
        if ((tid & 63) == 0) wave_sums[tid >> 6] = ss;
        __syncthreads();
        float total = 0.0f;
#pragma unroll
        for (int w = 0; w < 4; ++w) total += wave_sums[w];
        norm_scale = 1.0f / sqrtf(total / static_cast<float>(K) + src_args.eps);
    }
    // the eight source values of chunk c
    auto load_chunk = [&](int c, float4& o0, float4& o1) {
        o0 = src[2 * c];
        o1 = src[2 * c + 1];
        if (KIND == kPackSwiglu) {
            const float4 u0 = src2[2 * c], u1 = src2[2 * c + 1];
            o0 = make_float4(tiled_swiglu(o0.x, u0.x), tiled_swiglu(o0.y, u0.y), tiled_swiglu(o0.z, u0.z), tiled_swiglu(o0.w, u0.w));
            o1 = make_float4(tiled_swiglu(o1.x, u1.x), tiled_swiglu(o1.y, u1.y), tiled_swiglu(o1.z, u1.z), tiled_swiglu(o1.w, u1.w));
        }
        if (KIND == kPackNorm) {
            float w[8];
            if (src_args.norm_dtype == 0u) {
                m40_unpack8(reinterpret_cast<const uint4*>(src_args.norm_w)[c], w);
            } else {
                const float4 w0 = reinterpret_cast<const float4*>(src_args.norm_w)[2 * c], w1 = reinterpret_cast<const float4*>(src_args.norm_w)[2 * c + 1];
                w[0] = w0.x; w[1] = w0.y; w[2] = w0.z; w[3] = w0.w; w[4] = w1.x; w[5] = w1.y; w[6] = w1.z; w[7] = w1.w;
            }
            // x * scale, then * weight: two roundings, as rms_norm_kernel has them
            o0 = make_float4(o0.x * norm_scale * w[0], o0.y * norm_scale * w[1], o0.z * norm_scale * w[2], o0.w * norm_scale * w[3]);
            o1 = make_float4(o1.x * norm_scale * w[4], o1.y * norm_scale * w[5], o1.z * norm_scale * w[6], o1.w * norm_scale * w[7]);
        }
    };
    const bool in_regs = chunks <= kPackChunks * ROW_THREADS;
    float4 x0[kPackChunks], x1[kPackChunks];
    float mx = 0.0f;
    if (in_regs) {
#pragma unroll
        for (int i = 0; i < kPackChunks; ++i) {
            const int c = tid + ROW_THREADS * i;
            if (c < chunks) load_chunk(c, x0[i], x1[i]);
        }
#pragma unroll
        for (int i = 0; i < kPackChunks; ++i) {
            if (tid + ROW_THREADS * i < chunks) {
                mx = fmaxf(mx, fmaxf(fmaxf(pack_abs_or_inf(x0[i].x), pack_abs_or_inf(x0[i].y)), fmaxf(pack_abs_or_inf(x0[i].z), pack_abs_or_inf(x0[i].w))));
                mx = fmaxf(mx, fmaxf(fmaxf(pack_abs_or_inf(x1[i].x), pack_abs_or_inf(x1[i].y)), fmaxf(pack_abs_or_inf(x1[i].z), pack_abs_or_inf(x1[i].w))));
            }
        }
    } else {
        for (int c = tid; c < chunks; c += ROW_THREADS) {
            float4 a, b;
            load_chunk(c, a, b);
            mx = fmaxf(mx, fmaxf(fmaxf(pack_abs_or_inf(a.x), pack_abs_or_inf(a.y)), fmaxf(pack_abs_or_inf(a.z), pack_abs_or_inf(a.w))));
            mx = fmaxf(mx, fmaxf(fmaxf(pack_abs_or_inf(b.x), pack_abs_or_inf(b.y)), fmaxf(pack_abs_or_inf(b.z), pack_abs_or_inf(b.w))));
        }
    }
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
    if (ROW_THREADS == 256) {
        if ((tid & 63) == 0) wave_max[tid >> 6] = mx;
        __syncthreads();
        mx = fmaxf(fmaxf(wave_max[0], wave_max[1]), fmaxf(wave_max[2], wave_max[3]));
    }
    float scale = 1.0f, inv_scale = 1.0f;
    if (mx > 0.0f && mx < INFINITY) {
        int ex;
        (void)frexpf(mx, &ex);        // mx = f * 2^ex, f in [0.5, 1)
        ex -= 11;
        ex = ex < -100 ? -100 : (ex > 100 ? 100 : ex);
        scale = ldexpf(1.0f, ex);
        inv_scale = ldexpf(1.0f, -ex);
    }
    if (tid == 0) row_scale[row] = scale;
    half8* hp = reinterpret_cast<half8*>(hi + (size_t)row * K);
    half8* lp = reinterpret_cast<half8*>(lo + (size_t)row * K);
    if (in_regs) {
#pragma unroll
        for (int i = 0; i < kPackChunks; ++i) {
            const int c = tid + ROW_THREADS * i;
            if (c < chunks) {
                half8 h, l;
                pack_split8(x0[i], x1[i], inv_scale, h, l);
                hp[c] = h;
                lp[c] = l;
            }
        }
    } else {
        for (int c = tid; c < chunks; c += ROW_THREADS) {
            float4 a, b;
            load_chunk(c, a, b);
            half8 h, l;
            pack_split8(a, b, inv_scale, h, l);
            hp[c] = h;
            lp[c] = l;
        }
    }
}

__global__ __launch_bounds__(kThreads, 2) void gemm_tiled_f32xf16_gguf_kernel(const _Float16* __restrict__ A_hi,
                                                                              const _Float16* __restrict__ A_lo,
                                                                              const float* __restrict__ row_scale,
                                                                              TiledMats mats, int M, int K, int k_splits) {
    extern __shared__ __align__(16) _Float16 lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int tiles_n = mats.tile_start[mats.n];
    // Workgroups are dealt to the eight dies in turn.  Renumbered so that each die owns a contiguous band of tile
    // rows: its L2 then holds one eighth of A (and streams B) instead of every die reading all of A.
    const int per_die = (int)gridDim.x / 8;
    int logical = (int)blockIdx.x < per_die * 8 ? ((int)blockIdx.x % 8) * per_die + (int)blockIdx.x / 8 : (int)blockIdx.x;
    // K split (few tiles, long K): split s of a tile walks its share of the K steps and writes its partial sums to
    // plane s of the output buffer (a reduction launch adds the planes in order)
    const int tiles_all = (int)gridDim.x / k_splits;
    const int split = logical / tiles_all;
    logical -= split * tiles_all;
    const int tile_m = logical / tiles_n;
    int tile_n = logical % tiles_n;
    int mat = 0;
#pragma unroll
    for (int i = 1; i < kMaxMats; ++i)
        if (i < mats.n && tile_n >= mats.tile_start[i]) mat = i;
    tile_n -= mats.tile_start[mat];
    const uint16_t* __restrict__ B = mats.B[mat];
    float* __restrict__ C = mats.C[mat];
    const int N = mats.N[mat];
    const int m0 = tile_m * kBM, n0 = tile_n * kBN;
    // loader role: four lanes cover the 64 bytes one row contributes to a step, so a wave's load instruction touches
    // 16 rows (16 cache lines) instead of 32; each thread serves rows lrow and lrow + 64
    const int lrow = tid >> 2, lchunk = tid & 3;
    size_t a_off[2], b_off[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int ar = m0 + lrow + 64 * i < M ? m0 + lrow + 64 * i : M - 1;   // clamped: computed, never stored
        const int bc = n0 + lrow + 64 * i < N ? n0 + lrow + 64 * i : N - 1;
        a_off[i] = (size_t)ar * K + lchunk * 8;
        b_off[i] = (size_t)bc * K + lchunk * 8;
    }
    const int steps_all = K / kBK, per_split = (steps_all + k_splits - 1) / k_splits;
    const int step0 = split * per_split;
    const int steps = step0 + per_split <= steps_all ? per_split : steps_all - step0;     // >= 1 by the host's choice of k_splits

    auto issue = [&](StepRegs& r, int step) {
        const size_t k = (size_t)(step0 + step) * kBK;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            r.ah[i] = *reinterpret_cast<const uint4*>(A_hi + a_off[i] + k);
            r.al[i] = *reinterpret_cast<const uint4*>(A_lo + a_off[i] + k);
            r.b[i] = *reinterpret_cast<const uint4*>(B + b_off[i] + k);
        }
    };
    // LDS rows are 64 bytes = four 16-byte chunks; chunk c of row r is stored at position c ^ ((r / 4) % 4), so that
    // the 16-byte fragment reads of rows r and r + 4 (same banks without the swizzle) fall into different banks, with
    // no padding: 48 KB per workgroup
    auto to_lds = [&](const StepRegs& r, int buf) {
        _Float16* base = lds + buf * kBufHalves + lrow * kStride + ((lchunk ^ ((lrow >> 2) & 3)) * 8);
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            _Float16* p = base + i * 64 * kStride;
            *reinterpret_cast<u32x4*>(p) = u32x4{r.ah[i].x, r.ah[i].y, r.ah[i].z, r.ah[i].w};
            *reinterpret_cast<u32x4*>(p + kTileHalves) = u32x4{r.al[i].x, r.al[i].y, r.al[i].z, r.al[i].w};
            *reinterpret_cast<u32x4*>(p + 2 * kTileHalves) = u32x4{r.b[i].x, r.b[i].y, r.b[i].z, r.b[i].w};
        }
    };

    floatx4 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

    const int wm = wave >> 1, wn = wave & 1;
    // the scales of the rows this lane will store, requested now: at the end they would be 16 dependent round trips
    // (a load behind a store to memory it might alias waits for the store)
    float sc_all[4][4];
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int row = m0 + wm * 64 + mt * 16 + (lane >> 4) * 4 + r;
            sc_all[mt][r] = row_scale[row < M ? row : M - 1];
        }
    const int frag_row = lane & 15, frag_k = ((lane >> 4) ^ ((frag_row >> 2) & 3)) * 8;   // swizzled chunk of this lane's k group
    auto compute = [&](int buf) {
        const _Float16* base = lds + buf * kBufHalves;
        const _Float16* ah = base + (wm * 64 + frag_row) * kStride + frag_k;
        const _Float16* bb = base + 2 * kTileHalves + (wn * 64 + frag_row) * kStride + frag_k;
        half8 bf[4];
#pragma unroll
        for (int nt = 0; nt < 4; ++nt) bf[nt] = *reinterpret_cast<const half8*>(bb + nt * 16 * kStride);
#pragma unroll
        for (int mt = 0; mt < 4; ++mt) {
            const half8 hi = *reinterpret_cast<const half8*>(ah + mt * 16 * kStride);
            const half8 lo = *reinterpret_cast<const half8*>(ah + kTileHalves + mt * 16 * kStride);
            // the four high-part products first, then the four low-part ones: two instructions on one accumulator are
            // four instructions apart instead of back to back
#pragma unroll
            for (int nt = 0; nt < 4; ++nt) acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(hi, bf[nt], acc[mt][nt], 0, 0, 0);
#pragma unroll
            for (int nt = 0; nt < 4; ++nt) acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(lo, bf[nt], acc[mt][nt], 0, 0, 0);
        }
    };

    // Three register sets keep the loads of the next three steps in flight (a step's arithmetic is several times
    // shorter than the memory latency); the sets rotate with the step, so the loop is unrolled by three.  (Two sets and
    // three workgroups per CU measured the same on large shapes and slower on small grids.)
    StepRegs r0, r1, r2;
    const int last = steps - 1;
    issue(r0, 0);
    issue(r1, 1 < last ? 1 : last);
    issue(r2, 2 < last ? 2 : last);
    to_lds(r0, 0);
    __syncthreads();
    // step s: reload the set that step s consumed with step s + 3 (clamped: no branch around loads), compute from the
    // current LDS buffer, move step s + 1 into the other buffer
    auto step = [&](StepRegs& reload, const StepRegs& next, int s) {
        issue(reload, s + 3 < last ? s + 3 : last);
        compute(s & 1);
        to_lds(next, (s + 1) & 1);
        __syncthreads();
    };
    int s = 0;
    for (; s + 3 <= steps; s += 3) {
        step(r0, r1, s);
        step(r1, r2, s + 1);
        step(r2, r0, s + 2);
    }
    if (s < steps) step(r0, r1, s);
    if (s + 1 < steps) step(r1, r2, s + 1);

    // D fragment: lane holds rows 4 * (lane / 16) + r, column lane % 16 of each 16 x 16 tile
    const int out_col = lane & 15, out_row = (lane >> 4) * 4;
    const float* R = k_splits == 1 ? mats.R[mat] : nullptr;      // a K split adds the residual when it adds the planes
    // Two forms of the last step, chosen once per workgroup.  With a residual: per group of 16 rows its values first --
    // unconditional loads from clamped addresses, no branch and no wait between them -- then the stores; a load that
    // follows a store to memory it might alias is not moved ahead of it, and a load under a per-lane branch is awaited at
    // the branch's end (measured with both mistakes in place: +10 us on a 65 us launch).
    auto store_tile = [&](auto with_residual) {
#pragma unroll
        for (int mt = 0; mt < 4; ++mt) {
            float res[4][4];
            if (decltype(with_residual)::value) {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int row = m0 + wm * 64 + mt * 16 + out_row + r;
                    const size_t row_off = (size_t)(row < M ? row : M - 1) * N;
#pragma unroll
                    for (int nt = 0; nt < 4; ++nt) {
                        const int col = n0 + wn * 64 + nt * 16 + out_col;
                        res[r][nt] = R[row_off + (col < N ? col : N - 1)];
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int row = m0 + wm * 64 + mt * 16 + out_row + r;
                if (row >= M) continue;
                const float sc = sc_all[mt][r];       // a power of two: exact, also on the partial sums of a K split
#pragma unroll
                for (int nt = 0; nt < 4; ++nt) {
                    const int col = n0 + wn * 64 + nt * 16 + out_col;
                    if (col < N) {
                        const float v = acc[mt][nt][r] * sc;
                        C[((size_t)split * M + row) * N + col] = decltype(with_residual)::value ? res[r][nt] + v : v;
                    }
                }
            }
        }
    };
    if (R) store_tile(std::true_type{});
    else store_tile(std::false_type{});
}

// ---- wide tile: 128 x 256 per workgroup of four waves (wave tile 64 x 128), one workgroup per CU ---------------------------
//
// Measured on the 128 x 128 kernel above with parts of it switched off (M 4096, N 2048, K 2048): arithmetic alone 46 us,
// loads + LDS traffic + barriers alone 45 us, everything 87 us -- the two did not overlap.  A wave issues in order, and a
// memory instruction holds the issue slot until its unit accepts it; with the four waves of a CU in step behind the
// barrier, sixteen fragment reads, eight LDS writes and eight global loads each queue for ~500 cycles before the first
// matrix instruction of the step can go.  Here:
//  * every memory instruction of a step is issued under the step's matrix instructions, one per two of them
//    (sched_group_barrier), so it waits for its unit while the matrix pipe works;
//  * the fragments of step s + 1 are read from LDS during the arithmetic of step s (two fragment sets in registers);
//  * global data goes straight into LDS (global_load_lds_dwordx4: no registers, no LDS write instruction, no wait
//    before one), five 32 KB buffers deep -- a lane fetches the 16-byte chunk that belongs at its place in the swizzled
//    row layout, so a wave's instruction fills one contiguous kilobyte; the workgroup waits only for the step after
//    next (vmcnt) ahead of the barrier that publishes it;
//  * the wave tile is 64 x 128: per matrix instruction two thirds of the fragment bytes of a 64 x 64 tile (the activation
//    rows, read twice -- high and low part -- are the short side).
// M 4096, N 2048, K 2048: 79 -> 60 us; N 11264: 479 -> 404 us; K 5632: 232 -> 173 us.  Under this load the part lowers
// its clock (1.4-1.9 GHz measured inside the kernel, against 2.0-2.2 GHz in short or memory-bound launches), and a form
// with fewer issue cycles (32 x 32 x 16 instructions: 1370 instead of 1500 cycles per step) ran at a lower clock
// still and took the same time: what is left is energy per product, of which the exact hi + lo split is half.
constexpr int kWideBN = 256;
constexpr int kWideWM = 64, kWideWN = 128;                   // wave tile, waves 2 x 2
constexpr int kWideMT = kWideWM / 16, kWideNT = kWideWN / 16;
constexpr int kWidePlane = kBM * 64;                          // bytes of a 128-row operand block (32 k)
constexpr int kWideBuf = 2 * kWidePlane + kWideBN * 64;      // A high, A low, B: 32 KB
constexpr int kWideBufs = 5;
constexpr int kWideLds = kWideBufs * kWideBuf;               // 160 KB: the whole LDS of a CU
constexpr int kWideAL = kBM / 64, kWideBL = kWideBN / 64;    // 16-byte loads per thread: rows lrow + 64 i of a plane
constexpr int kWideLoads = 2 * kWideAL + kWideBL;

struct WideFrags { half8 hi[kWideMT], lo[kWideMT], b[kWideNT]; };

template <int... I, class F>
__device__ __forceinline__ void tiled_unrolled(std::integer_sequence<int, I...>, F&& f) { (f(std::integral_constant<int, I>{}), ...); }

// s_waitcnt for vector-memory operations only: at most n of them may still be outstanding
__device__ __forceinline__ constexpr int vmcnt_only(int n) { return 0x0f70 | (n & 15) | ((n >> 4) << 14); }

__global__ __launch_bounds__(kThreads, 1) void gemm_tiled_wide_kernel(const _Float16* __restrict__ A_hi,
                                                                      const _Float16* __restrict__ A_lo,
                                                                      const float* __restrict__ row_scale, TiledMats mats,
                                                                      int M, int K) {
    typedef __attribute__((address_space(3))) void* lds_dst_t;
    typedef const __attribute__((address_space(1))) void* global_src_t;
    extern __shared__ __align__(16) uint8_t wide_lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int tiles_n = mats.tile_start[mats.n];
    // each die owns a contiguous band of tile rows, as above
    const int per_die = (int)gridDim.x / 8;
    const int logical = (int)blockIdx.x < per_die * 8 ? ((int)blockIdx.x % 8) * per_die + (int)blockIdx.x / 8 : (int)blockIdx.x;
    const int tile_m = logical / tiles_n;
    int tile_n = logical % tiles_n;
    int mat = 0;
#pragma unroll
    for (int i = 1; i < kMaxMats; ++i)
        if (i < mats.n && tile_n >= mats.tile_start[i]) mat = i;
    tile_n -= mats.tile_start[mat];
    const uint16_t* __restrict__ B = mats.B[mat];
    float* __restrict__ C = mats.C[mat];
    const int N = mats.N[mat];
    const int m0 = tile_m * kBM, n0 = tile_n * kWideBN;
    // loader: thread -> row lrow (+ 64 i) of a plane and the place tid % 4 in that row's 64 bytes, which holds chunk
    // (tid % 4) ^ ((lrow / 4) % 4) of the row; the host guarantees that M * K and N * K fit 31 bits
    const int lrow = tid >> 2, gchunk = (tid & 3) ^ ((lrow >> 2) & 3);
    uint32_t a_off[kWideAL], b_off[kWideBL];     // in halves
#pragma unroll
    for (int i = 0; i < kWideAL; ++i) {
        const int ar = m0 + lrow + 64 * i < M ? m0 + lrow + 64 * i : M - 1;     // clamped: computed, never stored
        a_off[i] = (uint32_t)ar * (uint32_t)K + gchunk * 8;
    }
#pragma unroll
    for (int i = 0; i < kWideBL; ++i) {
        const int bc = n0 + lrow + 64 * i < N ? n0 + lrow + 64 * i : N - 1;
        b_off[i] = (uint32_t)bc * (uint32_t)K + gchunk * 8;
    }
    const int steps = K / kBK, last = steps - 1;
    // one instruction of a wave fills rows 16 wave .. 16 wave + 15 (+ 64 i) of a plane: a contiguous kilobyte, lane by lane
    auto issue = [&](int buf, int step) {
        step = step < last ? step : last;          // past the end: the last step again (no branch around loads)
        const _Float16* ah = A_hi + (size_t)step * kBK;
        const _Float16* al = A_lo + (size_t)step * kBK;
        const uint16_t* bb = B + (size_t)step * kBK;
        uint8_t* dst = wide_lds + buf * kWideBuf + wave * 1024;
#pragma unroll
        for (int i = 0; i < kWideAL; ++i) {
            __builtin_amdgcn_global_load_lds((global_src_t)(ah + a_off[i]), (lds_dst_t)(dst + i * 4096), 16, 0, 0);
            __builtin_amdgcn_global_load_lds((global_src_t)(al + a_off[i]), (lds_dst_t)(dst + kWidePlane + i * 4096), 16, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < kWideBL; ++i)
            __builtin_amdgcn_global_load_lds((global_src_t)(bb + b_off[i]), (lds_dst_t)(dst + 2 * kWidePlane + i * 4096), 16, 0, 0);
    };
    const int wm = wave >> 1, wn = wave & 1;
    float sc_all[kWideMT][4];          // the scales of the rows this lane will store, requested ahead of everything else
#pragma unroll
    for (int mt = 0; mt < kWideMT; ++mt)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int row = m0 + wm * kWideWM + mt * 16 + (lane >> 4) * 4 + r;
            sc_all[mt][r] = row_scale[row < M ? row : M - 1];
        }
    const int frag_row = lane & 15;
    const int fr_off = frag_row * 64 + (((lane >> 4) ^ ((frag_row >> 2) & 3)) * 16);
    auto read_frags = [&](WideFrags& f, int buf) {
        const uint8_t* base = wide_lds + buf * kWideBuf + fr_off;
        const uint8_t* a = base + wm * kWideWM * 64;
        const uint8_t* b = base + 2 * kWidePlane + wn * kWideWN * 64;
#pragma unroll
        for (int mt = 0; mt < kWideMT; ++mt) {
            f.hi[mt] = *reinterpret_cast<const half8*>(a + mt * 16 * 64);
            f.lo[mt] = *reinterpret_cast<const half8*>(a + kWidePlane + mt * 16 * 64);
        }
#pragma unroll
        for (int nt = 0; nt < kWideNT; ++nt) f.b[nt] = *reinterpret_cast<const half8*>(b + nt * 16 * 64);
    };
    floatx4 acc[kWideMT][kWideNT];
#pragma unroll
    for (int i = 0; i < kWideMT; ++i)
#pragma unroll
        for (int j = 0; j < kWideNT; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};
    // per accumulator the same order as the 128 x 128 kernel (step by step, high part then low part): the same bits
    auto compute = [&](const WideFrags& f) {
#pragma unroll
        for (int mt = 0; mt < kWideMT; ++mt) {
#pragma unroll
            for (int nt = 0; nt < kWideNT; ++nt) acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(f.hi[mt], f.b[nt], acc[mt][nt], 0, 0, 0);
#pragma unroll
            for (int nt = 0; nt < kWideNT; ++nt) acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(f.lo[mt], f.b[nt], acc[mt][nt], 0, 0, 0);
        }
    };

    WideFrags f[2];
    // steps 0 .. 4 requested, one per buffer; steps 0 and 1 awaited.  The barriers are bare s_barrier instructions with
    // the vector-memory wait written out: __syncthreads() would wait for every outstanding load (its fence covers LDS).
#pragma unroll
    for (int i = 0; i < kWideBufs; ++i) issue(i, i);
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(vmcnt_only((kWideBufs - 2) * kWideLoads));
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    read_frags(f[0], 0);
    // Before step s: the fragments of step s are requested into f[s % 2]; buffer (s + 1) % 5 is complete and visible;
    // steps s + 2 .. s + 3 are in flight.  Step s refills the buffer of step s - 1 -- whose fragments every wave had in
    // registers before the last barrier -- with step s + 4, and waits for step s + 2 ahead of its barrier.  (Step 0
    // requests step 4 a second time: buffer 0 is still being read then.)
    constexpr int kPeriod = 2 * kWideBufs;
    auto step = [&](auto ph_c, int s) __attribute__((always_inline)) {
        constexpr int ph = decltype(ph_c)::value;
        read_frags(f[(ph + 1) & 1], (ph + 1) % kWideBufs);
        issue((ph + kWideBufs - 1) % kWideBufs, s - 1 + kWideBufs);
        compute(f[ph & 1]);
        // issue order: two matrix instructions, one LDS read (16 times), then two matrix instructions, one load (8 times)
#pragma unroll
        for (int i = 0; i < 2 * kWideMT + kWideNT; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
#pragma unroll
        for (int i = 0; i < kWideLoads; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
            __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(vmcnt_only((kWideBufs - 3) * kWideLoads));
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
    };
    int s = 0;
    for (; s + kPeriod <= steps; s += kPeriod)
        tiled_unrolled(std::make_integer_sequence<int, kPeriod>(),
                       [&](auto ph_c) __attribute__((always_inline)) { step(ph_c, s + decltype(ph_c)::value); });
    tiled_unrolled(std::make_integer_sequence<int, kPeriod - 1>(), [&](auto ph_c) __attribute__((always_inline)) {
        if (s + decltype(ph_c)::value < steps) step(ph_c, s + decltype(ph_c)::value);
    });
    __builtin_amdgcn_s_waitcnt(vmcnt_only(0));      // no write into LDS may be outstanding when the workgroup ends

    const int out_col = lane & 15, out_row = (lane >> 4) * 4;
    const float* R = mats.R[mat];
    auto store_tile = [&](auto with_residual) {          // two forms, as in the kernel above
#pragma unroll
        for (int mt = 0; mt < kWideMT; ++mt) {
            float res[4][kWideNT];
            if (decltype(with_residual)::value) {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int row = m0 + wm * kWideWM + mt * 16 + out_row + r;
                    const size_t row_off = (size_t)(row < M ? row : M - 1) * N;
#pragma unroll
                    for (int nt = 0; nt < kWideNT; ++nt) {
                        const int col = n0 + wn * kWideWN + nt * 16 + out_col;
                        res[r][nt] = R[row_off + (col < N ? col : N - 1)];
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int row = m0 + wm * kWideWM + mt * 16 + out_row + r;
                if (row >= M) continue;
                const float sc = sc_all[mt][r];
#pragma unroll
                for (int nt = 0; nt < kWideNT; ++nt) {
                    const int col = n0 + wn * kWideWN + nt * 16 + out_col;
                    if (col < N) {
                        const float v = acc[mt][nt][r] * sc;
                        C[(size_t)row * N + col] = decltype(with_residual)::value ? res[r][nt] + v : v;
                    }
                }
            }
        }
    };
    if (R) store_tile(std::true_type{});
    else store_tile(std::false_type{});
}

// out[i] = planes[0][i] + planes[1][i] + ... in that order (n4 float4 per plane), then residual[i] + that (residual may be
// out); blockIdx.y = matrix, so the up to three matrices of a launch are summed by one launch as well
struct KPlaneSet {
    const float4* planes[kMaxMats];
    const float4* residual[kMaxMats];
    float4* out[kMaxMats];
    size_t n4[kMaxMats];
};
__global__ __launch_bounds__(256) void add_k_planes_kernel(KPlaneSet set, int k_splits) {
    const int m = blockIdx.y;
    const size_t n4 = set.n4[m];
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n4) return;
    const float4* planes = set.planes[m];
    float4 a = planes[i];
    for (int s = 1; s < k_splits; ++s) {
        const float4 b = planes[(size_t)s * n4 + i];
        a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w;
    }
    if (set.residual[m]) {
        const float4 r = set.residual[m][i];
        a = make_float4(r.x + a.x, r.y + a.y, r.z + a.z, r.w + a.w);
    }
    set.out[m][i] = a;
}

}  // namespace

bool m40_gemm_tiled_supported(const void* A, const void* B, int M, int N, int K) {
    return M > 32 && N >= 16 && K >= kBK && K % kBK == 0 && m40_aligned16(A) && m40_aligned16(B) &&
           ((long long)((M + kBM - 1) / kBM) * ((N + kBN - 1) / kBN)) <= 0x3fffffffll;
}

// Returns 1 when the activations' packing buffer cannot be provided (the stream is being captured and the buffer is
// too small, or the allocation fails): the caller then uses another kernel.
int m40_launch_gemm_tiled_fused(M40llmCudaContext* ctx, hipStream_t stream, uint32_t stream_kind, int source_kind, const float* A,
                                const float* A2, const void* norm_w, uint32_t norm_dtype, float eps, int M, int K, int n_mats,
                                const uint16_t* const* B, const int* N, float* const* C, const float* const* R) {
    if (!ctx || stream_kind > 1u || n_mats < 1 || n_mats > kMaxMats || source_kind < kPackPlain || source_kind > kPackSwiglu) return -2;
    if (source_kind == kPackSwiglu && (!A2 || !m40_aligned16(A2))) return -2;
    if (source_kind == kPackNorm && (!norm_w || norm_dtype > 1u || !m40_aligned16(norm_w))) return -2;
    TiledMats mats{};
    mats.n = n_mats;
    long long tiles_n = 0;
    for (int i = 0; i < n_mats; ++i) {
        if (!m40_gemm_tiled_supported(A, B[i], M, N[i], K) || !C[i]) return -2;
        mats.B[i] = B[i];
        mats.C[i] = C[i];
        mats.R[i] = R ? R[i] : nullptr;
        mats.N[i] = N[i];
        mats.tile_start[i] = (int)tiles_n;
        tiles_n += (N[i] + kBN - 1) / kBN;
    }
    mats.tile_start[n_mats] = (int)tiles_n;
    const long long tiles_m = (M + kBM - 1) / kBM;
    if (tiles_m * tiles_n > 0x7fffffffll) return -2;
    constexpr size_t lds_bytes = 2 * kBufHalves * sizeof(_Float16);   // 49152
    // two f16 planes of A (and the partial sums of a K split) in the stream's packing buffer, grown on demand (never while
    // the stream is being captured)
    M40StreamScratch& sc = ctx->scratch[stream_kind];
    // Few tiles and many K steps (short prompts, the down projection): split K so that the chip is covered and a
    // workgroup's chain of dependent steps is shorter; partial sums go to planes behind the packed activations and are
    // added in a fixed order by a second launch (every N a multiple of 4 for its float4 accesses).
    const int steps = K / kBK;
    int k_splits = 1;
    const long long tiles = tiles_m * tiles_n;
    bool n4_ok = true;
    size_t out_floats = 0;
    for (int i = 0; i < n_mats; ++i) {
        n4_ok = n4_ok && N[i] % 4 == 0 && m40_aligned16(C[i]) && m40_aligned16(mats.R[i]);
        out_floats += (size_t)M * N[i];
    }
    if (n4_ok && tiles <= 128) {   // above that a split only adds a partial-sum pass (measured at 176 tiles)
        k_splits = (int)(512 / tiles);
        if (k_splits > 4) k_splits = 4;
        while (k_splits > 1 && (steps / k_splits < 16 || (steps + k_splits - 1) / k_splits * (k_splits - 1) >= steps)) --k_splits;
    }
    const size_t scale_bytes = ((size_t)M * 4 + 15) & ~(size_t)15;
    const size_t need = (size_t)M * K * 4 + scale_bytes + (k_splits > 1 ? (size_t)k_splits * out_floats * 4 : 0);
    if (sc.tiled_pack_bytes < need) {
        hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(stream, &status) != hipSuccess || status != hipStreamCaptureStatusNone) return 1;
        if (hipStreamSynchronize(stream) != hipSuccess) return -2;
        if (sc.tiled_pack) (void)hipFree(sc.tiled_pack);
        sc.tiled_pack = nullptr;
        sc.tiled_pack_bytes = 0;
        const size_t want = need + need / 4;
        if (hipMalloc(&sc.tiled_pack, want) != hipSuccess) {
            (void)hipGetLastError();
            return 1;
        }
        sc.tiled_pack_bytes = want;
    }
    (void)hipGetLastError();
    _Float16* hi = static_cast<_Float16*>(sc.tiled_pack);
    _Float16* lo = hi + (size_t)M * K;
    float* row_scale = reinterpret_cast<float*>(static_cast<char*>(sc.tiled_pack) + (size_t)M * K * 4);
    const PackSource source{A, A2, norm_w, norm_dtype, eps};
    const bool wave_rows = K <= kPackChunks * 64 * 8;
    if (source_kind == kPackNorm)
        pack_hilo_planes_kernel<256, kPackNorm><<<(unsigned)M, 256, 0, stream>>>(source, hi, lo, row_scale, M, K);
    else if (source_kind == kPackSwiglu && wave_rows)
        pack_hilo_planes_kernel<64, kPackSwiglu><<<(unsigned)((M + 3) / 4), 256, 0, stream>>>(source, hi, lo, row_scale, M, K);
    else if (source_kind == kPackSwiglu)
        pack_hilo_planes_kernel<256, kPackSwiglu><<<(unsigned)M, 256, 0, stream>>>(source, hi, lo, row_scale, M, K);
    else if (wave_rows)
        pack_hilo_planes_kernel<64, kPackPlain><<<(unsigned)((M + 3) / 4), 256, 0, stream>>>(source, hi, lo, row_scale, M, K);
    else
        pack_hilo_planes_kernel<256, kPackPlain><<<(unsigned)M, 256, 0, stream>>>(source, hi, lo, row_scale, M, K);
    float* partial = reinterpret_cast<float*>(static_cast<char*>(sc.tiled_pack) + (size_t)M * K * 4 + scale_bytes);
    TiledMats launch = mats;
    if (k_splits > 1) {
        size_t at = 0;
        for (int i = 0; i < n_mats; ++i) {
            launch.C[i] = partial + at;
            at += (size_t)k_splits * M * N[i];
        }
    }
    // the wide tile from 9/16 of a tile per CU on (measured at K 2048: 144 tiles 52 against 68 us for the 128 x 128 kernel, 180
    // tiles 54 against 72 us; 120 tiles 51 against 48 us, 96 tiles 49 against 46 us), element offsets fitting its 32-bit arithmetic
    long long wide_tiles_n = 0;
    TiledMats wide = mats;
    bool wide_ok = k_splits == 1 && (long long)M * K < 0x7fffffffll;
    for (int i = 0; i < n_mats; ++i) {
        wide.tile_start[i] = (int)wide_tiles_n;
        wide_tiles_n += (N[i] + kWideBN - 1) / kWideBN;
        wide_ok = wide_ok && (long long)N[i] * K < 0x7fffffffll;
    }
    wide.tile_start[n_mats] = (int)wide_tiles_n;
    if (wide_ok && 16 * tiles_m * wide_tiles_n >= 9ll * ctx->num_cus) {
        static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_tiled_wide_kernel),
                                                           hipFuncAttributeMaxDynamicSharedMemorySize, kWideLds);
        wide_ok = attr == hipSuccess;
    } else {
        wide_ok = false;
    }
    if (wide_ok)
        gemm_tiled_wide_kernel<<<(unsigned)(tiles_m * wide_tiles_n), kThreads, kWideLds, stream>>>(hi, lo, row_scale, wide, M, K);
    else
        gemm_tiled_f32xf16_gguf_kernel<<<(unsigned)(tiles * k_splits), kThreads, lds_bytes, stream>>>(hi, lo, row_scale, launch, M, K, k_splits);
    if (k_splits > 1) {
        KPlaneSet set{};
        size_t blocks = 0;
        for (int i = 0; i < n_mats; ++i) {
            set.planes[i] = reinterpret_cast<const float4*>(launch.C[i]);
            set.residual[i] = reinterpret_cast<const float4*>(mats.R[i]);
            set.out[i] = reinterpret_cast<float4*>(C[i]);
            set.n4[i] = (size_t)M * N[i] / 4;
            blocks = blocks > (set.n4[i] + 255) / 256 ? blocks : (set.n4[i] + 255) / 256;
        }
        add_k_planes_kernel<<<dim3((unsigned)blocks, (unsigned)n_mats), 256, 0, stream>>>(set, k_splits);
    }
    return hipGetLastError() == hipSuccess ? 0 : -2;
}

int m40_launch_gemm_tiled_multi(M40llmCudaContext* ctx, hipStream_t stream, uint32_t stream_kind, const float* A, int M, int K,
                                int n_mats, const uint16_t* const* B, const int* N, float* const* C) {
    return m40_launch_gemm_tiled_fused(ctx, stream, stream_kind, kPackPlain, A, nullptr, nullptr, 0u, 0.0f, M, K, n_mats, B, N, C, nullptr);
}

int m40_launch_gemm_tiled(M40llmCudaContext* ctx, hipStream_t stream, uint32_t stream_kind, const float* A, const uint16_t* B,
                          float* C, int M, int N, int K) {
    return m40_launch_gemm_tiled_multi(ctx, stream, stream_kind, A, M, K, 1, &B, &N, &C);
}
