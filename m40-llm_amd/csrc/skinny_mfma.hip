// Skinny GEMM for the batched decode step on gfx950: C[M,N] = A[M,K] (f32) x W[N,K]^T with 1 <= M <= 16 rows
// per pass and W either f16 (GGUF order, K contiguous per output column) or q8_0 (34-byte blocks along K).
//
// The activations are split once per call into f16 hi + f16 lo fragments with a per-row power-of-two scale
// (inside the kernel, step by step); the product runs on v_mfma_f32_16x16x32_f16 with f32 accumulation.  One MFMA covers
// 32 consecutive k, which is exactly one q8_0 block, so the block scale multiplies the MFMA result.
//
// A workgroup is four waves = four 16-column tiles that walk the same range of K in steps of 256.  The
// activation fragments of a step (8 KB, or 16 KB above eight rows) are converted once per workgroup into LDS
// and shared by the four waves; weights are read once, straight from their GGUF bytes:
//   f16  : lane (column j, group g) loads its 16 bytes of k = 32 i + 8 g .. +7 per MFMA;
//   q8_0 : the 16 columns x 272 bytes of a step are copied with full 16-byte loads into a wave-private LDS
//          tile; each lane then reads the 8 quants of its (column, block, group) and turns them into f16 with
//          the 1024 + (q xor 0x80) construction (exact).
// Weight loads run two steps ahead of the step being multiplied and activation loads one step ahead, in a
// fixed issue order with no load under a branch, so that each wait names exactly the loads it needs and the
// younger ones stay in flight.  K is split over grid.y; slices write partial sums that a second kernel adds in
// slice order, so results never depend on timing.
#include "common.hpp"

#include <type_traits>

namespace {

constexpr int kTileK = 256;                       // k per step
constexpr int kWavesPerGroup = 4;                 // 16-column tiles per workgroup
constexpr int kThreads = kWavesPerGroup * 64;
constexpr int kQ8ColStride = 276;                 // LDS bytes per column of a staged tile: 272 + 4, an odd number of
                                                  // dwords, so that the 16 columns start in different banks
constexpr int kQ8TileBytes = 16 * kQ8ColStride;   // 16 columns x (8 blocks x 34 bytes + pad)

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ m40_float4 mfma16x16x32(const uint4& a, const uint4& b, m40_float4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(m40_half8, a),
                                                  __builtin_bit_cast(m40_half8, b), c, 0, 0, 0);
}

// two int8 (already xor 0x80, in the low bytes of two 16-bit lanes) -> packed f16 pair, exact
__device__ __forceinline__ uint32_t q8_pair_to_f16(uint32_t spread) {
    const half2_t v = __builtin_bit_cast(half2_t, spread | 0x64006400u);     // 1024 + u
    const half2_t k = {(_Float16)1152.0f, (_Float16)1152.0f};                // 1024 + 128
    return __builtin_bit_cast(uint32_t, v - k);
}

struct SkinnyArgs {
    const float* A;            // activations [M][K], f32
    const float* up;           // not null: the operand is silu(A) * up (SwiGLU of an FFN)
    const void* norm_w;        // not null: the operand is A * rsqrt(mean(A^2) + eps) * norm_w (RMSNorm)
    uint32_t norm_dtype;       // 0 f16, 1 f32
    float eps;
    const void* W[3];          // up to three weight matrices with the same K (Q/K/V, gate/up)
    float* C[3];               // direct outputs [M][N z] (S == 1 and no epilogue kernel)
    int N[3];
    int tile_begin[4];         // first 16-column tile of each matrix in the launch-wide tile list
    size_t part_off[3];        // float offset of matrix z in `partial`; layout there [S][16][N z]
    float* partial;
    int nmat, M, K, S, direct;
    int rms_deferred;          // RMSNorm operand: the kernel multiplies by A * norm_w only, and the kernel that adds the
                               // slices scales each row by rsqrt(mean(A^2) + eps) (the product is linear in that factor)
};

// FMT 0: f16 weights, 1: q8_0 weights.
template <int FMT, bool STACKED>
__global__ __launch_bounds__(kThreads, 2) void skinny_mfma_kernel(SkinnyArgs p) {
    constexpr int kASets = STACKED ? 1 : 2;
    __shared__ __attribute__((aligned(16))) uint2 a_lds[2][kASets][8 * 64 * 2];                    // activation fragments of a step, two buffers
    __shared__ float tscale_s[2][16];                                   // factor that undoes each row's scaling of the step
    __shared__ __attribute__((aligned(16))) uint8_t b_lds[FMT == 1 ? kWavesPerGroup * kQ8TileBytes : 16];

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int j = lane & 15, g = lane >> 4;
    const int ntiles = p.tile_begin[p.nmat];
    int gtile = blockIdx.x * kWavesPerGroup + wave;
    const bool tile_live = gtile < ntiles;
    if (!tile_live) gtile = ntiles - 1;
    const int z = (p.nmat > 2 && gtile >= p.tile_begin[2]) ? 2 : ((p.nmat > 1 && gtile >= p.tile_begin[1]) ? 1 : 0);
    const int N = p.N[z];
    const int n0 = (gtile - p.tile_begin[z]) * 16;
    const int KT = p.K / kTileK;
    const int kt0 = (int)(((long long)blockIdx.y * KT) / p.S), kt1 = (int)(((long long)(blockIdx.y + 1) * KT) / p.S);

    // ---- weight addressing
    const int col = n0 + j < N ? n0 + j : N - 1;
    const uint16_t* w16 = nullptr;
    const uint8_t* q_base = nullptr;
    uint32_t q_src[5] = {0, 0, 0, 0, 0};      // byte offsets of this lane's tile pieces from q_base (step 0)
    int q_dst[5] = {0, 0, 0, 0, 0};
    uint8_t* my_b = b_lds + (FMT == 1 ? wave * kQ8TileBytes : 0);
    if (FMT == 0) {
        w16 = static_cast<const uint16_t*>(p.W[z]) + (size_t)col * p.K + 8 * g;
    } else {
        const size_t col_stride = (size_t)(p.K >> 5) * 34;
        q_base = static_cast<const uint8_t*>(p.W[z]) + (size_t)n0 * col_stride;
#pragma unroll
        for (int i = 0; i < 5; ++i) {
            int q = i * 64 + lane;                // 16-byte piece of the 16 x 272-byte tile
            if (q >= 272) q = lane;               // no such piece: repeat this lane's first one, so that no load sits
                                                  // under a branch (a skipped load would make every wait conservative)
            const int c = q / 17, piece = q % 17;
            const int cc = n0 + c < N ? c : N - 1 - n0;
            q_src[i] = (uint32_t)((size_t)cc * col_stride + 16 * piece);
            q_dst[i] = c * kQ8ColStride + 16 * piece;
        }
    }

    // ---- activation addressing: thread (arow, acol) owns EPT consecutive k of row arow in every step:
    // k = 256 kt + EPT acol .. ; eight consecutive k form entry (MFMA i = k / 32, group (k / 8) % 4) of the fragments.
    // Up to eight rows: 32 lanes per row (8 elements per lane); above: 16 lanes per row (16 elements per lane).
    constexpr int EPT = STACKED ? 8 : 16;
    constexpr int TPR = kTileK / EPT;
    static_assert(TPR * (STACKED ? 8 : 16) == kThreads, "one thread per EPT activations of a step");
    const int arow = tid / TPR, acol = tid % TPR;
    const bool a_live = arow < p.M;
    const float* a_ptr = p.A + (size_t)(a_live ? arow : 0) * p.K + EPT * acol;
    // SwiGLU partner or f32 norm weights; with neither, the activations themselves (loaded and ignored: the same
    // loads are issued whatever the operand is)
    const bool norm16 = p.norm_w && p.norm_dtype == 0u;
    const float* b_ptr = p.up ? p.up + (size_t)(a_live ? arow : 0) * p.K + EPT * acol
                              : (p.norm_w && !norm16 ? static_cast<const float*>(p.norm_w) + EPT * acol : a_ptr);
    const uint16_t* nw16 = norm16 ? static_cast<const uint16_t*>(p.norm_w) + EPT * acol : nullptr;
    auto load_f32 = [&](const float* src, float (&v)[EPT]) {
#pragma unroll
        for (int e = 0; e < EPT; e += 4) {
            const float4 x = *reinterpret_cast<const float4*>(src + e);
            v[e] = x.x; v[e + 1] = x.y; v[e + 2] = x.z; v[e + 3] = x.w;
        }
    };
    auto row_reduce_max = [&](float x) -> float {
#pragma unroll
        for (int o = 1; o < TPR; o <<= 1) x = fmaxf(x, __shfl_xor(x, o, 64));
        return x;
    };

    float fa[EPT];             // this thread's activations of a step
    uint4 fbraw[EPT / 4];      // and their SwiGLU partner or norm weights, as loaded: f32 values, or (f16 norm weights)
                               // the eight weights of elements 8j..8j+7 in entries 2j and 2j+1 alike
    constexpr int NW = FMT == 0 ? 8 : 5;
    uint4 rb[2][NW];           // weights of two steps in flight.  f16: eight 16-byte loads; q8_0: five tile pieces
    // One batch of 16-byte loads whatever the second operand is: a branch around loads makes the compiler wait for
    // every load in flight at its join -- here that was a full wait right behind each step's barrier, which drained the
    // weight requests of the next two steps.  f16 norm weights are 16 bytes per eight elements, requested twice.
    auto issue_a = [&](int kt) {
        load_f32(a_ptr + (size_t)kt * kTileK, fa);
        const char* src = norm16 ? reinterpret_cast<const char*>(nw16 + (size_t)kt * kTileK)
                                 : reinterpret_cast<const char*>(b_ptr + (size_t)kt * kTileK);
#pragma unroll
        for (int i = 0; i < EPT / 4; ++i)
            fbraw[i] = *reinterpret_cast<const uint4*>(src + (norm16 ? 16 * (i / 2) : 16 * i));
    };
    auto fb_word = [&](int i, int w) -> uint32_t {
        const uint4 v = fbraw[i];
        return w == 0 ? v.x : (w == 1 ? v.y : (w == 2 ? v.z : v.w));
    };
    auto fb_f32 = [&](int e) { return __uint_as_float(fb_word(e / 4, e % 4)); };
    auto fb_f16 = [&](int e) { return m40_h2f((uint16_t)((fb_word(2 * (e / 8), (e % 8) / 2) >> (16 * (e & 1))) & 0xffffu)); };
    // Plain loads, not streaming ones: a lane's 16 bytes are a quarter of a 64-byte run of its column, and the rest
    // of each 128-byte line is asked for by the next instruction -- with the streaming hint the line is fetched again
    // (measured: +4.7 % on the batch-8 step with plain loads).
    auto issue_w = [&](uint4 (&dst)[NW], int kt) {
        if (FMT == 0) {
#pragma unroll
            for (int i = 0; i < 8; ++i)
                dst[i] = *reinterpret_cast<const uint4*>(w16 + (size_t)kt * kTileK + 32 * i);
        } else {
#pragma unroll
            for (int i = 0; i < 5; ++i)
                dst[i] = *reinterpret_cast<const uint4*>(q_base + (size_t)kt * 272 + q_src[i]);
        }
    };

    const int nsteps = kt1 - kt0;
    m40_float4 acc = {0.f, 0.f, 0.f, 0.f};
    // Order of issue, kept through the loop: activations of step s+1, then weights of step s+2.  A wait for the
    // activations leaves the younger weight loads in flight; a wait for the weights of step s+1 leaves those of
    // step s+2 in flight.
    issue_a(kt0);
    issue_w(rb[0], kt0);
    issue_w(rb[1], nsteps > 1 ? kt0 + 1 : kt0);      // a one-step slice loads its step twice (rare: K of 256 only)

    // RMS over the whole row (RMSNorm operand whose scale is not left to the slice-adding kernel)
    float rms = 1.0f;
    if (p.norm_w && !p.rms_deferred && a_live) {
        float sq = 0.0f;
        for (int k = 0; k < p.K; k += 4 * kTileK) {
            float v[4][EPT];
#pragma unroll
            for (int u = 0; u < 4; ++u) load_f32(a_ptr + (k + u * kTileK < p.K ? k + u * kTileK : k), v[u]);
#pragma unroll
            for (int u = 0; u < 4; ++u)
                if (k + u * kTileK < p.K) {
#pragma unroll
                    for (int e = 0; e < EPT; ++e) sq = fmaf(v[u][e], v[u][e], sq);
                }
        }
#pragma unroll
        for (int o = 1; o < TPR; o <<= 1) sq += __shfl_xor(sq, o, 64);
        rms = rsqrtf(sq / (float)p.K + p.eps);
    }

    // f32 -> f16 hi + f16 lo of the operand held in fa/fb, scaled by a power of two taken from the largest value of
    // the row within this step, straight into the fragment entries of buffer `buf`
    auto convert = [&](int buf) {
        float x[EPT];
        float mx = 0.0f;
#pragma unroll
        for (int e = 0; e < EPT; ++e) {
            float v = fa[e];
            if (p.up) v = v / (1.0f + expf(-v)) * fb_f32(e);
            else if (norm16) v = v * rms * fb_f16(e);
            else if (p.norm_w) v = v * rms * fb_f32(e);
            if (!a_live) v = 0.0f;
            x[e] = v;
            mx = fmaxf(mx, fabsf(v));
        }
        mx = row_reduce_max(mx);
        float scale = 1.0f, inv_scale = 1.0f;
        if (mx > 0.0f && mx < INFINITY) {
            int ex;
            (void)frexpf(mx, &ex);        // mx = f * 2^ex, f in [0.5, 1)
            ex -= 11;                     // scaled maximum in [2^10, 2^11)
            ex = ex < -100 ? -100 : (ex > 100 ? 100 : ex);
            scale = ldexpf(1.0f, ex);
            inv_scale = ldexpf(1.0f, -ex);
        }
        uint32_t hi[EPT / 2], lo[EPT / 2];
#pragma unroll
        for (int e = 0; e < EPT; e += 2) {
            uint32_t h2 = 0, l2 = 0;
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                const float v = x[e + q] * inv_scale;
                const _Float16 h = static_cast<_Float16>(v);
                const _Float16 l = static_cast<_Float16>(v - static_cast<float>(h));
                h2 |= (uint32_t)__builtin_bit_cast(uint16_t, h) << (16 * q);
                l2 |= (uint32_t)__builtin_bit_cast(uint16_t, l) << (16 * q);
            }
            hi[e / 2] = h2; lo[e / 2] = l2;
        }
        uint4* frag_hi = reinterpret_cast<uint4*>(a_lds[buf][0]);
        uint4* frag_lo = reinterpret_cast<uint4*>(a_lds[buf][kASets - 1]);
#pragma unroll
        for (int c = 0; c < EPT / 8; ++c) {
            const int kk = EPT * acol + 8 * c;                       // first k of this eight within the step
            const int entry = (kk >> 5) * 64 + ((kk >> 3) & 3) * 16 + arow;
            frag_hi[entry] = make_uint4(hi[4 * c], hi[4 * c + 1], hi[4 * c + 2], hi[4 * c + 3]);
            frag_lo[STACKED ? entry + 8 : entry] = make_uint4(lo[4 * c], lo[4 * c + 1], lo[4 * c + 2], lo[4 * c + 3]);
        }
        if (acol == 0) {
            tscale_s[buf][arow] = scale;
            if (STACKED) tscale_s[buf][arow + 8] = scale;
        }
    };
    convert(0);

    // One step.  BUF: which of the two fragment / weight buffers holds it; PREFETCH: steps s+1 (activations) and
    // s+2 (weights) exist and are requested here; LAST: no step follows.
    auto step = [&](auto buf_c, auto prefetch_c, auto last_c, int kt) {
        constexpr int BUF = decltype(buf_c)::value;
        constexpr bool PREFETCH = decltype(prefetch_c)::value;
        constexpr bool LAST = decltype(last_c)::value;
        if (FMT == 1) {
#pragma unroll
            for (int i = 0; i < 5; ++i) {
                uint32_t* dst = reinterpret_cast<uint32_t*>(my_b + q_dst[i]);      // 4-byte aligned only
                dst[0] = rb[BUF][i].x; dst[1] = rb[BUF][i].y; dst[2] = rb[BUF][i].z; dst[3] = rb[BUF][i].w;
            }
        }
        __syncthreads();       // fragments of this step are complete; nobody still reads the other buffer
        if (!LAST) issue_a(kt + 1);
        if (FMT == 1 && PREFETCH) issue_w(rb[BUF], kt + 2);
        m40_float4 tacc = {0.f, 0.f, 0.f, 0.f};
        const uint4* a_hi_frag = reinterpret_cast<const uint4*>(a_lds[BUF][0]);
        const uint4* a_lo_frag = reinterpret_cast<const uint4*>(a_lds[BUF][kASets - 1]);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint4 a_hi = a_hi_frag[i * 64 + lane];
            if (FMT == 0) {
                tacc = mfma16x16x32(a_hi, rb[BUF][i], tacc);
                if (!STACKED) tacc = mfma16x16x32(a_lo_frag[i * 64 + lane], rb[BUF][i], tacc);
            } else {
                const uint8_t* blk = my_b + j * kQ8ColStride + 34 * i;
                const float d = m40_h2f(*reinterpret_cast<const uint16_t*>(blk));
                uint32_t s0, s1, s2, s3;   // byte pairs (0,1) (2,3) (4,5) (6,7) of the lane's eight quants, spread to 16-bit lanes
                if (i & 1) {               // quants 4-byte aligned
                    const uint32_t* w = reinterpret_cast<const uint32_t*>(blk + 2 + 8 * g);
                    const uint32_t x0 = w[0] ^ 0x80808080u, x1 = w[1] ^ 0x80808080u;
                    s0 = __builtin_amdgcn_perm(0u, x0, 0x0c010c00u);
                    s1 = __builtin_amdgcn_perm(0u, x0, 0x0c030c02u);
                    s2 = __builtin_amdgcn_perm(0u, x1, 0x0c010c00u);
                    s3 = __builtin_amdgcn_perm(0u, x1, 0x0c030c02u);
                } else {                   // quants start two bytes into an aligned word
                    const uint32_t* w = reinterpret_cast<const uint32_t*>(blk + 8 * g);
                    const uint32_t x0 = w[0] ^ 0x80808080u, x1 = w[1] ^ 0x80808080u, x2 = w[2] ^ 0x80808080u;
                    s0 = __builtin_amdgcn_perm(0u, x0, 0x0c030c02u);
                    s1 = __builtin_amdgcn_perm(0u, x1, 0x0c010c00u);
                    s2 = __builtin_amdgcn_perm(0u, x1, 0x0c030c02u);
                    s3 = __builtin_amdgcn_perm(0u, x2, 0x0c010c00u);
                }
                const uint4 bq = make_uint4(q8_pair_to_f16(s0), q8_pair_to_f16(s1), q8_pair_to_f16(s2), q8_pair_to_f16(s3));
                const m40_float4 zero = {0.f, 0.f, 0.f, 0.f};
                m40_float4 dblk = mfma16x16x32(a_hi, bq, zero);
                if (!STACKED) dblk = mfma16x16x32(a_lo_frag[i * 64 + lane], bq, dblk);
#pragma unroll
                for (int r = 0; r < 4; ++r) tacc[r] = fmaf(d, dblk[r], tacc[r]);
            }
        }
        if (FMT == 0 && PREFETCH) issue_w(rb[BUF], kt + 2);   // the matrix cores have read this buffer
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[r] = fmaf(tscale_s[BUF][4 * g + r], tacc[r], acc[r]);
        if (!LAST) convert(BUF ^ 1);     // next step's fragments, while the other waves finish this one
    };
    {
        using std::integral_constant;
        const integral_constant<int, 0> b0; const integral_constant<int, 1> b1;
        const integral_constant<bool, true> yes; const integral_constant<bool, false> no;
        int s = 0;
        for (; s + 3 < nsteps; s += 2) {          // both steps of a pair have a step two ahead
            step(b0, yes, no, kt0 + s);
            step(b1, yes, no, kt0 + s + 1);
        }
        const int rem = nsteps - s;               // 1, 2 or 3
        if (rem == 3) {
            step(b0, yes, no, kt0 + s);
            step(b1, no, no, kt0 + s + 1);
            step(b0, no, yes, kt0 + s + 2);
        } else if (rem == 2) {
            step(b0, no, no, kt0 + s);
            step(b1, no, yes, kt0 + s + 1);
        } else {
            step(b0, no, yes, kt0 + s);
        }
    }
    // lane (j, g) holds rows 4g + r of column j
    if (STACKED) {
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[r] = m40_add_xor32(acc[r]);  // hi rows + lo rows
    }
    if (!tile_live || n0 + j >= N) return;
    if (STACKED && g >= 2) return;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int row = 4 * g + r;
        if (p.direct) {
            if (row < p.M) p.C[z][(size_t)row * N + n0 + j] = acc[r];
        } else {
            p.partial[p.part_off[z] + ((size_t)blockIdx.y * 16 + row) * N + n0 + j] = acc[r];
        }
    }
}

// The K slices of one output element.  Loading and adding are separate so that a kernel can request everything it
// needs before it waits for anything; slices beyond S re-read slice 0 and are left out of the sum (no load sits under
// a branch).  The sum runs over the slices in ascending order.
__device__ __forceinline__ void skinny_load(const SkinnyArgs& p, int z, int row, int n, float (&part)[16]) {
    const float* src = p.partial + p.part_off[z] + (size_t)row * p.N[z] + n;
    const size_t slice_stride = (size_t)16 * p.N[z];
#pragma unroll
    for (int s = 0; s < 16; ++s) part[s] = src[(size_t)(s < p.S ? s : 0) * slice_stride];
}
__device__ __forceinline__ float skinny_add(const SkinnyArgs& p, const float (&part)[16]) {
    float v = 0.0f;
#pragma unroll
    for (int s = 0; s < 16; ++s) v += s < p.S ? part[s] : 0.0f;
    return v;
}

// Epilogue over the slice partials; grid (ceil(N/256), rows, matrices).
//   mode 0: out z[row][n] = sum (+ bias[n]) (+ residual[row][n])        (residual may alias out)
//   mode 1: out 0[row][n] = silu(sum of matrix 0) * (sum of matrix 1)   (SwiGLU of gate and up)
struct EpilogueArgs {
    SkinnyArgs g;
    float* out[3];
    const float* bias;
    const float* residual;
    int mode;
};

// rsqrt(mean(A[row]^2) + eps) by a 256-thread workgroup, the same value in every thread; fixed summation order.
__device__ __forceinline__ float skinny_row_rms(const SkinnyArgs& g, int row) {
    __shared__ float red_s[4];
    const float* a = g.A + (size_t)row * g.K;
    float sq = 0.0f;
    for (int k0 = 0; k0 < g.K; k0 += 4096) {          // four 16-byte loads in flight per thread
        float4 v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int k = k0 + u * 1024 + 4 * (int)threadIdx.x;
            v[u] = *reinterpret_cast<const float4*>(a + (k < g.K ? k : 0));
            if (k >= g.K) v[u] = make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            sq = fmaf(v[u].x, v[u].x, sq); sq = fmaf(v[u].y, v[u].y, sq);
            sq = fmaf(v[u].z, v[u].z, sq); sq = fmaf(v[u].w, v[u].w, sq);
        }
    }
    sq = m40_sum64(sq);
    if ((threadIdx.x & 63u) == 0u) red_s[threadIdx.x >> 6] = sq;
    __syncthreads();
    sq = (red_s[0] + red_s[1]) + (red_s[2] + red_s[3]);
    return rsqrtf(sq / (float)g.K + g.eps);
}

__global__ __launch_bounds__(256) void skinny_epilogue_kernel(EpilogueArgs e) {
    const int z = blockIdx.z, row = blockIdx.y;
    const int n = blockIdx.x * 256 + threadIdx.x;
    const int N = e.g.N[z];
    const int nc = n < N ? n : N - 1;
    // every load of the thread goes out before the first wait: slices of one matrix (mode 0) or of gate and up
    // (mode 1; mode 0 reads its own slices twice rather than branch), bias and residual (or a stand-in address)
    float pa[16], pb[16];
    skinny_load(e.g, e.mode == 1 ? 0 : z, row, nc, pa);
    skinny_load(e.g, e.mode == 1 ? 1 : z, row, nc, pb);
    const float bias = *(e.bias ? e.bias + nc : e.g.partial);
    const float res = *(e.residual ? e.residual + (size_t)row * N + nc : e.g.partial);
    const float rms = (e.g.norm_w && e.g.rms_deferred) ? skinny_row_rms(e.g, row) : 1.0f;
    if (n >= N) return;
    if (e.mode == 1) {
        const float gate = rms * skinny_add(e.g, pa), up = rms * skinny_add(e.g, pb);
        e.out[0][(size_t)row * N + n] = gate / (1.0f + expf(-gate)) * up;
        return;
    }
    float v = rms * skinny_add(e.g, pa);
    if (e.bias) v = v + bias;
    if (e.residual) v = res + v;
    e.out[z][(size_t)row * N + n] = v;
}

// Q/K/V epilogue of a batched decode step: bias, RoPE at each row's position, q to its buffer, K and V (f16) into
// the cache row of (sequence ids[row], position lens[row]).  One thread per rotation pair; pair space = Q pairs,
// K pairs, V pairs (V pairs are adjacent elements, not rotated).
struct QkvEpilogueArgs {
    SkinnyArgs g;
    const float* bq; const float* bk; const float* bv;
    float* q_out;                 // [rows][q_heads * head_dim]
    uint16_t* k_cache; uint16_t* v_cache; uint32_t* seq_map;
    const uint32_t* ids_dev; const uint32_t* lens_dev;
    uint32_t max_seq_len, max_batch, q_heads, kv_heads, head_dim, rope_layout;
    float rope_base, rope_scale;
};
__global__ __launch_bounds__(256) void skinny_qkv_epilogue_kernel(QkvEpilogueArgs e) {
    const uint32_t row = blockIdx.y;
    const uint32_t half = e.head_dim / 2u;
    const uint32_t q_pairs = e.q_heads * half, kv_pairs = e.kv_heads * half;
    const uint32_t total = q_pairs + 2u * kv_pairs;
    const uint32_t pair_raw = blockIdx.x * 256u + threadIdx.x;
    const uint32_t pair = pair_raw < total ? pair_raw : total - 1u;
    int which;
    uint32_t local;
    if (pair < q_pairs) { which = 0; local = pair; }
    else if (pair < q_pairs + kv_pairs) { which = 1; local = pair - q_pairs; }
    else { which = 2; local = pair - q_pairs - kv_pairs; }
    const uint32_t head = local / half, off = local % half;
    size_t i0, i1;
    m40_rope_pair(head, off, e.head_dim, which == 2 ? M40LLM_ROPE_LAYOUT_ADJACENT : e.rope_layout, &i0, &i1);
    const float* bias = which == 0 ? e.bq : (which == 1 ? e.bk : e.bv);
    // all loads first: slices of both elements, biases (or a stand-in address), the row's position and sequence id
    float p0[16], p1[16];
    skinny_load(e.g, which, (int)row, (int)i0, p0);
    skinny_load(e.g, which, (int)row, (int)i1, p1);
    const float b0 = *(bias ? bias + i0 : e.g.partial), b1 = *(bias ? bias + i1 : e.g.partial);
    const uint32_t position = e.lens_dev[row];
    const uint32_t seq = e.ids_dev[row];
    const float rms = (e.g.norm_w && e.g.rms_deferred) ? skinny_row_rms(e.g, (int)row) : 1.0f;
    if (pair_raw >= total) return;
    float y0 = rms * skinny_add(e.g, p0), y1 = rms * skinny_add(e.g, p1);
    if (bias) { y0 = y0 + b0; y1 = y1 + b1; }
    if (position >= e.max_seq_len || seq >= e.max_batch) return;
    if (which != 2) m40_rope_rotate(position, off, e.head_dim, e.rope_base, e.rope_scale, y0, y1, &y0, &y1);
    if (which == 0) {
        float* q = e.q_out + (size_t)row * e.q_heads * e.head_dim;
        q[i0] = y0;
        q[i1] = y1;
    } else {
        const size_t ept = (size_t)e.kv_heads * e.head_dim;
        uint16_t* dst = (which == 1 ? e.k_cache : e.v_cache) + ((size_t)seq * e.max_seq_len + position) * ept;
        dst[i0] = m40_f2h(y0);
        dst[i1] = m40_f2h(y1);
        if (which == 1 && local == 0) e.seq_map[seq] = position + 1u;
    }
}

// Batched greedy step: one workgroup per row.  First index of the row maximum of logits[rows][n] and the
// top-1/top-2 gap go to ids[row][step] / gaps[row][step]; lens[row] += 1; the embedding row of the pick becomes the
// row's next input.  state = {unused, capacity, step of row 0, step of row 1, ...}.
struct GreedyBatchArgs {
    const float* logits; uint32_t n;
    uint32_t* state;              // [1] capacity, [2 + row] step of the row
    uint32_t* lens; uint32_t* ids; float* gaps;
    const uint16_t* table; uint32_t d_model; float* x_out;
};
__global__ __launch_bounds__(1024) void greedy_batch_kernel(GreedyBatchArgs a) {
    __shared__ float sa[16], sb[16];
    __shared__ uint32_t si[16];
    __shared__ uint32_t s_tok;
    const uint32_t row = blockIdx.x;
    const float* lg = a.logits + (size_t)row * a.n;
    float va = -INFINITY, vb = -INFINITY;
    uint32_t ia = 0xffffffffu;
    auto offer = [&](float oa, float ob, uint32_t oi) {
        if (oa > va || (oa == va && oi < ia)) { vb = fmaxf(va, ob); va = oa; ia = oi; }
        else vb = fmaxf(vb, oa);
    };
    if ((a.n & 3u) == 0u && (reinterpret_cast<uintptr_t>(lg) & 15u) == 0u) {
        // eight 16-byte loads per thread and batch, all requested before the first comparison; indices ascend within a
        // thread, and ties between threads are settled by index in offer()
        const float4* lg4 = reinterpret_cast<const float4*>(lg);
        const uint32_t n4 = a.n >> 2;
        for (uint32_t base = 0; base < n4; base += 8u * 1024u) {
            float4 v[8];
#pragma unroll
            for (uint32_t u = 0; u < 8u; ++u) {
                const uint32_t i = base + u * 1024u + threadIdx.x;
                v[u] = lg4[i < n4 ? i : n4 - 1u];
            }
#pragma unroll
            for (uint32_t u = 0; u < 8u; ++u) {
                const uint32_t i = base + u * 1024u + threadIdx.x;
                if (i < n4) {
                    offer(v[u].x, -INFINITY, 4u * i); offer(v[u].y, -INFINITY, 4u * i + 1u);
                    offer(v[u].z, -INFINITY, 4u * i + 2u); offer(v[u].w, -INFINITY, 4u * i + 3u);
                }
            }
        }
    } else {
#pragma unroll 4
        for (uint32_t i = threadIdx.x; i < a.n; i += 1024u) offer(lg[i], -INFINITY, i);
    }
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const float oa = __shfl_xor(va, o, 64), ob = __shfl_xor(vb, o, 64);
        const uint32_t oi = __shfl_xor(ia, o, 64);
        offer(oa, ob, oi);
    }
    const uint32_t wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63u) == 0u) { sa[wave] = va; sb[wave] = vb; si[wave] = ia; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (uint32_t w = 1; w < 16u; ++w) offer(sa[w], sb[w], si[w]);
        uint32_t tok = ia == 0xffffffffu ? 0u : ia;
        if (tok >= a.n) tok = a.n - 1;
        const uint32_t step = a.state[2 + row], cap = a.state[1];
        if (step < cap) {
            a.ids[(size_t)row * cap + step] = tok;
            a.gaps[(size_t)row * cap + step] = va - vb;
        }
        a.state[2 + row] = step + 1u;
        a.lens[row] = a.lens[row] + 1u;
        s_tok = tok;
    }
    __syncthreads();
    const uint32_t tok = s_tok;
    for (uint32_t i = threadIdx.x; i < a.d_model; i += 1024u)
        a.x_out[(size_t)row * a.d_model + i] = m40_h2f(a.table[(size_t)tok * a.d_model + i]);
}

// The same step in two launches for wide rows: kGreedyParts workgroups per row each reduce a contiguous range of the
// logits to (maximum, runner-up, first index of the maximum); one workgroup per row then merges the parts -- ties go
// to the lower index in both stages, so the pick equals the one-launch kernel's -- and does the bookkeeping.
constexpr uint32_t kGreedyParts = 32;
__global__ __launch_bounds__(256) void greedy_batch_part_kernel(GreedyBatchArgs a, float* part) {
    __shared__ float sa[4], sb[4];
    __shared__ uint32_t si[4];
    const uint32_t row = blockIdx.y, pt = blockIdx.x;
    const float4* lg4 = reinterpret_cast<const float4*>(a.logits + (size_t)row * a.n);
    const uint32_t n4 = a.n >> 2;
    const uint32_t per = (n4 + kGreedyParts - 1) / kGreedyParts;
    const uint32_t beg = pt * per, end = beg + per < n4 ? beg + per : n4;
    float va = -INFINITY, vb = -INFINITY;
    uint32_t ia = 0xffffffffu;
    auto offer = [&](float oa, float ob, uint32_t oi) {
        if (oa > va || (oa == va && oi < ia)) { vb = fmaxf(va, ob); va = oa; ia = oi; }
        else vb = fmaxf(vb, oa);
    };
    for (uint32_t base = beg; base < end; base += 8u * 256u) {
        float4 v[8];
#pragma unroll
        for (uint32_t u = 0; u < 8u; ++u) {
            const uint32_t i = base + u * 256u + threadIdx.x;
            v[u] = lg4[i < n4 ? i : n4 - 1u];
        }
#pragma unroll
        for (uint32_t u = 0; u < 8u; ++u) {
            const uint32_t i = base + u * 256u + threadIdx.x;
            if (i < end) {
                offer(v[u].x, -INFINITY, 4u * i); offer(v[u].y, -INFINITY, 4u * i + 1u);
                offer(v[u].z, -INFINITY, 4u * i + 2u); offer(v[u].w, -INFINITY, 4u * i + 3u);
            }
        }
    }
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const float oa = __shfl_xor(va, o, 64), ob = __shfl_xor(vb, o, 64);
        const uint32_t oi = __shfl_xor(ia, o, 64);
        offer(oa, ob, oi);
    }
    const uint32_t wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63u) == 0u) { sa[wave] = va; sb[wave] = vb; si[wave] = ia; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (uint32_t w = 1; w < 4u; ++w) offer(sa[w], sb[w], si[w]);
        float* dst = part + ((size_t)row * kGreedyParts + pt) * 4;
        dst[0] = va; dst[1] = vb; dst[2] = __uint_as_float(ia);
    }
}
__global__ __launch_bounds__(256) void greedy_batch_merge_kernel(GreedyBatchArgs a, const float* part) {
    __shared__ uint32_t s_tok;
    const uint32_t row = blockIdx.x;
    if (threadIdx.x < 64u) {
        static_assert(kGreedyParts <= 64, "one lane per part");
        const float* src = part + ((size_t)row * kGreedyParts + (threadIdx.x < kGreedyParts ? threadIdx.x : 0u)) * 4;
        const float pa = src[0], pb = src[1];
        const uint32_t pi = __float_as_uint(src[2]);
        const uint32_t step = a.state[2 + row], cap = a.state[1], len = a.lens[row];
        const bool live = threadIdx.x < kGreedyParts;
        float va = live ? pa : -INFINITY, vb = live ? pb : -INFINITY;
        uint32_t ia = live ? pi : 0xffffffffu;
        auto offer = [&](float oa, float ob, uint32_t oi) {
            if (oa > va || (oa == va && oi < ia)) { vb = fmaxf(va, ob); va = oa; ia = oi; }
            else vb = fmaxf(vb, oa);
        };
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const float oa = __shfl_xor(va, o, 64), ob = __shfl_xor(vb, o, 64);
            const uint32_t oi = __shfl_xor(ia, o, 64);
            offer(oa, ob, oi);
        }
        if (threadIdx.x == 0) {
            uint32_t tok = ia == 0xffffffffu ? 0u : ia;
            if (tok >= a.n) tok = a.n - 1;
            if (step < cap) {
                a.ids[(size_t)row * cap + step] = tok;
                a.gaps[(size_t)row * cap + step] = va - vb;
            }
            a.state[2 + row] = step + 1u;
            a.lens[row] = len + 1u;
            s_tok = tok;
        }
    }
    __syncthreads();
    const uint32_t tok = s_tok;
    for (uint32_t i = threadIdx.x; i < a.d_model; i += 256u)
        a.x_out[(size_t)row * a.d_model + i] = m40_h2f(a.table[(size_t)tok * a.d_model + i]);
}

int pick_slices(int ntiles, int KT, int num_cus) {
    const long long groups = (ntiles + kWavesPerGroup - 1) / kWavesPerGroup;
    int s = 1;
    // Measured on the batched decode step: about 1.5 workgroups per CU and at least two steps per slice.
    while (s < 16 && groups * s * 2 < 3LL * num_cus && KT / (s * 2) >= 2) s *= 2;
    return s > KT ? KT : s;
}

struct PackSpec {
    const float* A;
    const float* up;          // SwiGLU partner, or null
    const void* norm_w;       // RMSNorm weights, or null
    uint32_t norm_dtype;
    float eps;
};

// Launches the MFMA kernel for `m` (<= 16) rows over nmat matrices.  Returns the filled args (for an
// epilogue kernel) through *out; direct != 0 writes scaled results to C when the K range is not split.
int launch_core(M40llmCudaContext* ctx, hipStream_t stream, uint32_t stream_kind, int fmt, const PackSpec& pk, int m, int K,
                int nmat, const void* const* W, const int* N, float* const* C, bool want_direct, SkinnyArgs* out) {
    M40StreamScratch& sc = ctx->scratch[stream_kind];
    if (!m40_aligned16(pk.A) || (pk.up && !m40_aligned16(pk.up)) || (pk.norm_w && !m40_aligned16(pk.norm_w))) return -2;
    SkinnyArgs a{};
    a.A = pk.A; a.up = pk.up; a.norm_w = pk.norm_w; a.norm_dtype = pk.norm_dtype; a.eps = pk.eps;
    a.partial = static_cast<float*>(sc.attn_partial);
    a.nmat = nmat; a.M = m; a.K = K;
    int tiles = 0;
    size_t n_total = 0;
    for (int z = 0; z < nmat; ++z) {
        a.W[z] = W[z]; a.N[z] = N[z]; a.C[z] = C ? C[z] : nullptr;
        a.tile_begin[z] = tiles;
        tiles += (N[z] + 15) >> 4;
        n_total += (size_t)N[z];
    }
    a.tile_begin[nmat] = tiles;
    const int KT = K / kTileK;
    int S = pick_slices(tiles, KT, ctx->num_cus);
    while (S > 1 && (size_t)S * 16 * n_total * sizeof(float) > sc.attn_partial_bytes) S >>= 1;
    if ((size_t)S * 16 * n_total * sizeof(float) > sc.attn_partial_bytes && !(want_direct && S == 1)) return -2;
    a.S = S;
    a.direct = (want_direct && S == 1) ? 1 : 0;
    a.rms_deferred = (pk.norm_w && !a.direct) ? 1 : 0;
    size_t off = 0;
    for (int z = 0; z < nmat; ++z) {
        a.part_off[z] = off;
        off += (size_t)S * 16 * N[z];
    }
    const bool stacked = m <= 8;
    dim3 grid((tiles + kWavesPerGroup - 1) / kWavesPerGroup, S);
    if (fmt == 0) {
        if (stacked) skinny_mfma_kernel<0, true><<<grid, kThreads, 0, stream>>>(a);
        else skinny_mfma_kernel<0, false><<<grid, kThreads, 0, stream>>>(a);
    } else {
        if (stacked) skinny_mfma_kernel<1, true><<<grid, kThreads, 0, stream>>>(a);
        else skinny_mfma_kernel<1, false><<<grid, kThreads, 0, stream>>>(a);
    }
    *out = a;
    return 0;
}

void launch_plain_epilogue(hipStream_t stream, const SkinnyArgs& a, int nmat, float* const* out, const float* bias,
                           const float* residual, int mode) {
    EpilogueArgs e{};
    e.g = a;
    int nmax = 0;
    for (int z = 0; z < nmat; ++z) {
        e.out[z] = out[z];
        nmax = a.N[z] > nmax ? a.N[z] : nmax;
    }
    e.bias = bias; e.residual = residual; e.mode = mode;
    dim3 grid((nmax + 255) / 256, a.M, mode == 1 ? 1 : nmat);
    skinny_epilogue_kernel<<<grid, 256, 0, stream>>>(e);
}

bool rows_ok(const M40llmCudaContext* ctx, int rows, int K) {
    (void)ctx;
    return rows >= 1 && rows <= 16 && K > 0 && K % kTileK == 0;
}

}  // namespace

bool m40_skinny_supported(const M40llmCudaContext* ctx, uint32_t stream_kind, int M, int N, int K, int fmt) {
    (void)M;
    if (K % kTileK != 0 || N <= 0) return false;
    if (fmt != 0 && fmt != 1) return false;
    (void)ctx; (void)stream_kind;
    return true;
}

// up != nullptr: the activations are silu(A) * up.  W1/C1 may be null (one matrix).
int m40_launch_skinny(M40llmCudaContext* ctx, hipStream_t stream, uint32_t stream_kind, int fmt, const float* A,
                      const float* up, const void* W0, float* C0, const void* W1, float* C1, int M, int N, int K) {
    if (M <= 0 || N <= 0 || K <= 0) return -2;
    if (!m40_skinny_supported(ctx, stream_kind, M, N, K, fmt)) return -2;
    const int nmat = W1 ? 2 : 1;
    (void)hipGetLastError();
    for (int r0 = 0; r0 < M; r0 += 16) {
        const int m = M - r0 < 16 ? M - r0 : 16;
        PackSpec pk{A + (size_t)r0 * K, up ? up + (size_t)r0 * K : nullptr, nullptr, 0, 0.0f};
        const void* W[2] = {W0, W1};
        const int Ns[2] = {N, N};
        float* C[2] = {C0 + (size_t)r0 * N, C1 ? C1 + (size_t)r0 * N : nullptr};
        SkinnyArgs a{};
        const int rc = launch_core(ctx, stream, stream_kind, fmt, pk, m, K, nmat, W, Ns, C, true, &a);
        if (rc != 0) return rc;
        if (!a.direct) launch_plain_epilogue(stream, a, nmat, C, nullptr, nullptr, 0);
    }
    return hipGetLastError() == hipSuccess ? 0 : -2;
}

// ---- batched decode step entry points (rows <= 16, decode stream) -------------------------------------------
extern "C" {

int m40llm_ext_batched_norm_qkv_rope_append_async(
    M40llmCudaContext* ctx, M40llmKVCache* kv, const uint32_t* seq_ids_dev, const uint32_t* seq_lens_dev, uint32_t rows,
    const void* d_x_f32, const void* d_norm_w, uint32_t norm_weight_dtype, float eps, const void* d_wq_f16,
    const void* d_wk_f16, const void* d_wv_f16, const void* d_bq_f32, const void* d_bk_f32, const void* d_bv_f32,
    uint32_t d_model, uint32_t q_heads, float freq_base, float freq_scale, uint32_t rope_layout, void* d_q_out_f32) {
    if (!ctx || !kv || !seq_ids_dev || !seq_lens_dev || !d_x_f32 || !d_norm_w || !d_wq_f16 || !d_wk_f16 || !d_wv_f16 ||
        !d_q_out_f32)
        return -1;
    if (kv->compressed || !kv->d_k || !kv->d_v) return -2;
    if (norm_weight_dtype > 1) return -4;
    if (kv->head_dim == 0 || kv->head_dim % 2 != 0 || kv->num_heads == 0 || q_heads == 0) return -3;
    if (!rows_ok(ctx, (int)rows, (int)d_model)) return -6;
    if (!m40_aligned16(d_wq_f16) || !m40_aligned16(d_wk_f16) || !m40_aligned16(d_wv_f16)) return -6;
    (void)hipGetLastError();
    // up to eight rows and K = 2048: persistent matrix-core kernel with the whole epilogue inside
    if (m40_rows_mfma_qkv_supported((int)rows, (int)d_model, kv->head_dim) && m40_aligned16(d_x_f32) && m40_aligned16(d_norm_w) &&
        (int)((q_heads + 2u * kv->num_heads) * kv->head_dim / 16u) <= ctx->num_cus)
        return m40_rows_mfma_qkv(ctx, ctx->decode_stream, kv, seq_ids_dev, seq_lens_dev, rows, static_cast<const float*>(d_x_f32),
                                 d_norm_w, norm_weight_dtype, eps, static_cast<const uint16_t*>(d_wq_f16),
                                 static_cast<const uint16_t*>(d_wk_f16), static_cast<const uint16_t*>(d_wv_f16),
                                 static_cast<const float*>(d_bq_f32), static_cast<const float*>(d_bk_f32),
                                 static_cast<const float*>(d_bv_f32), d_model, q_heads, freq_base, freq_scale, rope_layout,
                                 static_cast<float*>(d_q_out_f32));
    // up to eight rows and K <= 2048: vector-ALU kernel with the whole epilogue inside (one launch instead of two)
    if (m40_rows_gemv_supported((int)rows, (int)d_model) && m40_aligned16(d_x_f32) && m40_aligned16(d_norm_w))
        return m40_rows_norm_qkv(ctx, ctx->decode_stream, kv, seq_ids_dev, seq_lens_dev, rows, static_cast<const float*>(d_x_f32),
                                 d_norm_w, norm_weight_dtype, eps, static_cast<const uint16_t*>(d_wq_f16),
                                 static_cast<const uint16_t*>(d_wk_f16), static_cast<const uint16_t*>(d_wv_f16),
                                 static_cast<const float*>(d_bq_f32), static_cast<const float*>(d_bk_f32),
                                 static_cast<const float*>(d_bv_f32), d_model, q_heads, freq_base, freq_scale, rope_layout,
                                 static_cast<float*>(d_q_out_f32));
    const int QN = (int)(q_heads * kv->head_dim), KN = (int)(kv->num_heads * kv->head_dim);
    PackSpec pk{static_cast<const float*>(d_x_f32), nullptr, d_norm_w, norm_weight_dtype, eps};
    const void* W[3] = {d_wq_f16, d_wk_f16, d_wv_f16};
    const int Ns[3] = {QN, KN, KN};
    SkinnyArgs a{};
    int rc = launch_core(ctx, ctx->decode_stream, 1, 0, pk, (int)rows, (int)d_model, 3, W, Ns, nullptr, false, &a);
    if (rc != 0) return -6;
    QkvEpilogueArgs e{};
    e.g = a;
    e.bq = static_cast<const float*>(d_bq_f32); e.bk = static_cast<const float*>(d_bk_f32);
    e.bv = static_cast<const float*>(d_bv_f32);
    e.q_out = static_cast<float*>(d_q_out_f32);
    e.k_cache = kv->d_k; e.v_cache = kv->d_v; e.seq_map = kv->d_seq_map;
    e.ids_dev = seq_ids_dev; e.lens_dev = seq_lens_dev;
    e.max_seq_len = kv->max_seq_len; e.max_batch = kv->max_batch_size; e.q_heads = q_heads; e.kv_heads = kv->num_heads;
    e.head_dim = kv->head_dim; e.rope_layout = rope_layout; e.rope_base = freq_base; e.rope_scale = freq_scale;
    const uint32_t pairs = (q_heads + 2u * kv->num_heads) * (kv->head_dim / 2u);
    skinny_qkv_epilogue_kernel<<<dim3((pairs + 255u) / 256u, rows), 256, 0, ctx->decode_stream>>>(e);
    return hipGetLastError() == hipSuccess ? 0 : -7;
}

int m40llm_ext_batched_gemm_residual_f32xf16_async(M40llmCudaContext* ctx, const void* d_a_f32, const void* d_w_f16,
                                                   const void* d_residual_f32, void* d_out_f32, uint32_t rows, int N, int K) {
    if (!ctx || !d_a_f32 || !d_w_f16 || !d_out_f32) return -1;
    if (N <= 0 || K <= 0) return -2;
    if (!rows_ok(ctx, (int)rows, K) || !m40_aligned16(d_w_f16)) return -6;
    (void)hipGetLastError();
    if (N <= 8192 && m40_rows_gemv_supported((int)rows, K) && m40_aligned16(d_a_f32))
        return m40_rows_gemv_residual(ctx->decode_stream, static_cast<const float*>(d_a_f32),
                                      static_cast<const uint16_t*>(d_w_f16), static_cast<const float*>(d_residual_f32),
                                      static_cast<float*>(d_out_f32), (int)rows, N, K);
    PackSpec pk{static_cast<const float*>(d_a_f32), nullptr, nullptr, 0, 0.0f};
    const void* W[1] = {d_w_f16};
    const int Ns[1] = {N};
    float* out[1] = {static_cast<float*>(d_out_f32)};
    SkinnyArgs a{};
    if (launch_core(ctx, ctx->decode_stream, 1, 0, pk, (int)rows, K, 1, W, Ns, nullptr, false, &a) != 0) return -6;
    launch_plain_epilogue(ctx->decode_stream, a, 1, out, nullptr, static_cast<const float*>(d_residual_f32), 0);
    return hipGetLastError() == hipSuccess ? 0 : -7;
}

int m40llm_ext_batched_gemm_residual_onto_zero_f32xf16_async(M40llmCudaContext* ctx, const void* d_a_f32, const void* d_w_f16,
                                                             const void* d_residual_f32, void* d_out_f32, uint32_t rows, int N,
                                                             int K) {
    if (!ctx || !d_a_f32 || !d_w_f16 || !d_out_f32) return -1;
    if (N <= 0 || K <= 0) return -2;
    const char* o = static_cast<const char*>(d_out_f32);
    auto apart = [&](const void* q, size_t bytes) {
        const char* c = static_cast<const char*>(q);
        return !c || c + bytes <= o || o + (size_t)rows * N * 4 <= c;
    };
    if (m40_rows_khalf_supported(ctx, (int)rows, N, K) && m40_aligned16(d_a_f32) && m40_aligned16(d_w_f16) &&
        apart(d_a_f32, (size_t)rows * K * 4) && apart(d_residual_f32, (size_t)rows * N * 4)) {
        (void)hipGetLastError();
        return m40_rows_khalf_residual(ctx, ctx->decode_stream, static_cast<const float*>(d_a_f32),
                                       static_cast<const uint16_t*>(d_w_f16), static_cast<const float*>(d_residual_f32),
                                       static_cast<float*>(d_out_f32), (int)rows, N, K);
    }
    // any other shape: the form that overwrites its result
    return m40llm_ext_batched_gemm_residual_f32xf16_async(ctx, d_a_f32, d_w_f16, d_residual_f32, d_out_f32, rows, N, K);
}

int m40llm_ext_batched_norm_gate_up_swiglu_async(M40llmCudaContext* ctx, const void* d_x_f32, const void* d_norm_w,
                                                 uint32_t norm_weight_dtype, float eps, const void* d_wgate_f16,
                                                 const void* d_wup_f16, void* d_hid_f32, uint32_t rows, int ffn, int d_model) {
    return m40llm_ext_batched_norm_gate_up_swiglu_clear_async(ctx, d_x_f32, d_norm_w, norm_weight_dtype, eps, d_wgate_f16,
                                                              d_wup_f16, d_hid_f32, rows, ffn, d_model, nullptr, 0);
}

int m40llm_ext_batched_norm_gate_up_swiglu_clear_async(M40llmCudaContext* ctx, const void* d_x_f32, const void* d_norm_w,
                                                       uint32_t norm_weight_dtype, float eps, const void* d_wgate_f16,
                                                       const void* d_wup_f16, void* d_hid_f32, uint32_t rows, int ffn,
                                                       int d_model, void* d_clear_f32, uint32_t clear_floats) {
    if (!ctx || !d_x_f32 || !d_norm_w || !d_wgate_f16 || !d_wup_f16 || !d_hid_f32) return -1;
    if (!d_clear_f32) clear_floats = 0;
    if (clear_floats > (1u << 30)) return -2;
    if (ffn <= 0 || d_model <= 0) return -2;
    if (norm_weight_dtype > 1) return -4;
    if (!rows_ok(ctx, (int)rows, d_model) || !m40_aligned16(d_wgate_f16) || !m40_aligned16(d_wup_f16)) return -6;
    (void)hipGetLastError();
    // up to eight rows and K = 2048: persistent kernel with the SwiGLU inside (one launch instead of two)
    if (m40_rows_mfma_supported((int)rows, d_model) && m40_aligned16(d_x_f32) && m40_aligned16(d_norm_w))
        return m40_rows_mfma_swiglu(ctx, ctx->decode_stream, static_cast<const float*>(d_x_f32), d_norm_w, norm_weight_dtype,
                                    eps, static_cast<const uint16_t*>(d_wgate_f16), static_cast<const uint16_t*>(d_wup_f16),
                                    static_cast<float*>(d_hid_f32), (int)rows, ffn, d_model,
                                    clear_floats ? static_cast<float*>(d_clear_f32) : nullptr, (int)clear_floats);
    if (clear_floats && m40_zero_f32(ctx->decode_stream, static_cast<float*>(d_clear_f32), clear_floats) != 0) return -7;
    PackSpec pk{static_cast<const float*>(d_x_f32), nullptr, d_norm_w, norm_weight_dtype, eps};
    const void* W[2] = {d_wgate_f16, d_wup_f16};
    const int Ns[2] = {ffn, ffn};
    float* out[2] = {static_cast<float*>(d_hid_f32), nullptr};
    SkinnyArgs a{};
    if (launch_core(ctx, ctx->decode_stream, 1, 0, pk, (int)rows, d_model, 2, W, Ns, nullptr, false, &a) != 0) return -6;
    launch_plain_epilogue(ctx->decode_stream, a, 2, out, nullptr, nullptr, 1);
    return hipGetLastError() == hipSuccess ? 0 : -7;
}

int m40llm_ext_batched_norm_gemm_f32xf16_async(M40llmCudaContext* ctx, const void* d_x_f32, const void* d_norm_w,
                                               uint32_t norm_weight_dtype, float eps, const void* d_w_f16, void* d_out_f32,
                                               uint32_t rows, int N, int K) {
    if (!ctx || !d_x_f32 || !d_norm_w || !d_w_f16 || !d_out_f32) return -1;
    if (N <= 0 || K <= 0) return -2;
    if (norm_weight_dtype > 1) return -4;
    if (!rows_ok(ctx, (int)rows, K) || !m40_aligned16(d_w_f16)) return -6;
    (void)hipGetLastError();
    if (m40_rows_mfma_supported((int)rows, K) && m40_aligned16(d_x_f32) && m40_aligned16(d_norm_w))
        return m40_rows_mfma_plain(ctx, ctx->decode_stream, static_cast<const float*>(d_x_f32), d_norm_w, norm_weight_dtype, eps,
                                   static_cast<const uint16_t*>(d_w_f16), static_cast<float*>(d_out_f32), (int)rows, N, K);
    PackSpec pk{static_cast<const float*>(d_x_f32), nullptr, d_norm_w, norm_weight_dtype, eps};
    const void* W[1] = {d_w_f16};
    const int Ns[1] = {N};
    float* out[1] = {static_cast<float*>(d_out_f32)};
    SkinnyArgs a{};
    if (launch_core(ctx, ctx->decode_stream, 1, 0, pk, (int)rows, K, 1, W, Ns, out, true, &a) != 0) return -6;
    if (!a.direct) launch_plain_epilogue(ctx->decode_stream, a, 1, out, nullptr, nullptr, 0);
    return hipGetLastError() == hipSuccess ? 0 : -7;
}

int m40llm_ext_batched_greedy_step_async(M40llmCudaContext* ctx, const void* d_logits_f32, uint32_t rows, uint32_t n,
                                         uint32_t* state_dev, uint32_t* seq_lens_dev, uint32_t* ids_dev, float* gaps_dev,
                                         const void* d_table_f16, uint32_t d_model, void* d_x_out_f32) {
    if (!ctx || !d_logits_f32 || !state_dev || !seq_lens_dev || !ids_dev || !gaps_dev || !d_table_f16 || !d_x_out_f32) return -1;
    if (rows == 0 || n == 0 || d_model == 0) return -2;
    (void)hipGetLastError();
    GreedyBatchArgs a{};
    a.logits = static_cast<const float*>(d_logits_f32); a.n = n; a.state = state_dev; a.lens = seq_lens_dev;
    a.ids = ids_dev; a.gaps = gaps_dev; a.table = static_cast<const uint16_t*>(d_table_f16); a.d_model = d_model;
    a.x_out = static_cast<float*>(d_x_out_f32);
    // Wide rows: parts in the block-select scratch of the decode stream (work on a stream is ordered, and the merge
    // launch consumes them before anything else on the stream can write there).
    M40StreamScratch& scr = ctx->scratch[1];
    const size_t part_bytes = (size_t)rows * kGreedyParts * 4 * sizeof(float);
    if (n >= 16384u && (n & 3u) == 0u && (reinterpret_cast<uintptr_t>(d_logits_f32) & 15u) == 0u && scr.select &&
        part_bytes <= scr.select_bytes) {
        float* part = static_cast<float*>(scr.select);
        greedy_batch_part_kernel<<<dim3(kGreedyParts, rows), 256, 0, ctx->decode_stream>>>(a, part);
        greedy_batch_merge_kernel<<<rows, 256, 0, ctx->decode_stream>>>(a, part);
    } else {
        greedy_batch_kernel<<<rows, 1024, 0, ctx->decode_stream>>>(a);
    }
    return hipGetLastError() == hipSuccess ? 0 : -3;
}

}  // extern "C"
