// q8_0 skinny GEMM and SwiGLU FFN for 3 <= M <= 16 rows on the int8 matrix instruction of gfx950.
//
// C[M,N] = A[M,K] (f32) x W[N,K]^T, W in q8_0: per output column K/32 blocks of {f16 scale d, 32 int8 quants}
// (reference dequantisation w = d * q: cuda/kernels.cu:856-867; f32 x q8_0 product: kernels.cu:5037-5052).
//
// The quants go into v_mfma_i32_16x16x32_i8 exactly as they are stored: one instruction covers one 32-k block of 16
// columns, and a lane's B operand is the 8 consecutive quants of its (column, block, k group).  What has to be made
// integer are the activations: every row is cut, block by block, into three signed 8-bit digits
// under a power-of-two block scale,
//     a = 2^E * (d1 + d2 / 128 + d3 / 16384),   |d1| <= 64, |d2|, |d3| <= 64,   error <= 2^-20 of the block's largest,
// each digit plane is one matrix instruction, the three exact i32 results are recombined once per block, and the
// block's factor 2^E * d_w multiplies them in f32.  No weight is converted and no product is rounded before that.
//
// Launches: a small pack kernel turns the f32 rows into digit planes (laid out in the order the A operand is
// loaded), then the product kernel; the FFN form packs its SwiGLU output itself (a workgroup's four waves produce
// exactly one 32-column block of the hidden row), so gate / up / down take three launches in all.
#include "common.hpp"

#include <type_traits>

namespace {

typedef int i32x4 __attribute__((ext_vector_type(4)));

// Packed activations.
//   MP = 8 or 16 (rows rounded up; rows above MP are zero and not stored), per 32-k block: three digit planes
//   [digit][k / 8][row < MP][8 bytes], then the 16 rows' block scales 2^(E-20) as f32.
//   MP = 0, "stacked", for at most four rows: ONE plane whose row 4 d + m holds digit d of row m (rows 12-15 zero), so
//   that a single matrix instruction multiplies all three digits.  Stored per step of eight blocks (256 k) as four
//   planes of 1 KB, [block pair][lane = 16 (k / 8) + row][block of the pair][8 bytes] -- a load instruction of a wave
//   reads one plane, 16 bytes per lane, one contiguous kilobyte -- then the step's 8 x 4 block scales.
__host__ __device__ constexpr int q80i8_block_bytes(int MP) { return MP == 0 ? 512 + 16 : 3 * 4 * MP * 8 + 64; }
constexpr int kStackStepBlocks = 8;
constexpr int kStackStepBytes = 64 * 64 + kStackStepBlocks * 4 * 4;      // 4224

// Digits of two neighbouring elements of one row of one block.  The 16 threads of a row (lanes pair = 0..15 of an
// aligned group of 16) hold the row's 32 values; digits go to dst in A-operand order, the exponent to dst's tail.
__device__ __forceinline__ void q80i8_pack_pair(float v0, float v1, int m, int pair, int MP, uint8_t* pack, int blk) {
    float mx = fmaxf(fabsf(v0), fabsf(v1));
#pragma unroll
    for (int o = 1; o < 16; o <<= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
    int ex = 0;
    if (mx > 0.0f && mx < INFINITY) (void)frexpf(mx, &ex);        // mx = f * 2^ex, f in [0.5, 1)
    ex = ex < -100 ? -100 : (ex > 100 ? 100 : ex);
    const float inv = ldexpf(1.0f, 6 - ex);                        // |a| * inv < 64
    const float v[2] = {v0, v1};
    int d[3][2];
#pragma unroll
    for (int e = 0; e < 2; ++e) {
        float s = (mx < INFINITY ? v[e] : 0.0f) * inv;
        s = fminf(fmaxf(s, -64.0f), 64.0f);
        const float d1 = rintf(s);
        const float r1 = (s - d1) * 128.0f;                        // exact: |s - d1| <= 0.5
        const float d2 = rintf(r1);
        const float r2 = (r1 - d2) * 128.0f;
        const float d3 = rintf(r2);
        d[0][e] = (int)d1; d[1][e] = (int)d2; d[2][e] = (int)d3;
    }
    const int k = 2 * pair, kg = k >> 3, kb = k & 7;
    // value = 2^(ex - 20) * ((d1 * 128 + d2) * 128 + d3)
    if (MP == 0) {
        uint8_t* step = pack + (size_t)(blk / kStackStepBlocks) * kStackStepBytes;
        const int b = blk % kStackStepBlocks;
        if (m < 4) {
#pragma unroll
            for (int dg = 0; dg < 3; ++dg) {
                const uint16_t two = (uint16_t)((d[dg][0] & 0xff) | ((d[dg][1] & 0xff) << 8));
                *reinterpret_cast<uint16_t*>(step + (b >> 1) * 1024 + (kg * 16 + dg * 4 + m) * 16 + (b & 1) * 8 + kb) = two;
            }
            if (pair == 0) reinterpret_cast<float*>(step + 64 * 64)[b * 4 + m] = ldexpf(1.0f, ex - 20);
        } else if (m >= 12) {
            *reinterpret_cast<uint16_t*>(step + (b >> 1) * 1024 + (kg * 16 + m) * 16 + (b & 1) * 8 + kb) = 0;
        }
        return;
    }
    uint8_t* dst = pack + (size_t)blk * q80i8_block_bytes(MP);
    if (m >= MP) return;
#pragma unroll
    for (int dg = 0; dg < 3; ++dg) {
        const uint16_t two = (uint16_t)((d[dg][0] & 0xff) | ((d[dg][1] & 0xff) << 8));
        *reinterpret_cast<uint16_t*>(dst + ((dg * 4 + kg) * MP + m) * 8 + kb) = two;
    }
    if (pair == 0) reinterpret_cast<float*>(dst + 3 * 4 * MP * 8)[m] = ldexpf(1.0f, ex - 20);
}

// grid = K / 32 blocks, 256 threads: thread (row tid / 16, pair tid % 16)
__global__ __launch_bounds__(256) void q80i8_pack_kernel(const float* __restrict__ A, int M, int MP, int K, uint8_t* pack) {
    const int blk = blockIdx.x, m = threadIdx.x >> 4, pair = threadIdx.x & 15;
    float2 v = make_float2(0.0f, 0.0f);
    if (m < M) v = *reinterpret_cast<const float2*>(A + (size_t)m * K + 32 * blk + 2 * pair);
    if (MP != 0 && threadIdx.x < 16)       // scales of rows >= MP
        reinterpret_cast<float*>(pack + (size_t)blk * q80i8_block_bytes(MP) + 3 * 4 * MP * 8)[threadIdx.x] = 0.0f;
    __syncthreads();
    q80i8_pack_pair(v.x, v.y, m, pair, MP, pack, blk);
}

struct Q80I8Args {
    const uint8_t* pack;       // packed activations
    const uint8_t* W0;         // MODE 0: the matrix; MODE 1: gate
    const uint8_t* W1;         // MODE 1: up
    float* C;                  // MODE 0: [M][N]
    uint8_t* out_pack;         // MODE 1: packed SwiGLU output (the A operand of the down projection)
    int M, MP, N, K;
};

// A step is 4 q8_0 blocks (128 k; 136 bytes per column = 17 pieces of 8 bytes) in the three-plane form and 8 blocks
// (256 k; 272 bytes = 17 pieces of 16 bytes, columns 16-byte aligned) in the stacked form: twice the bytes per load
// instruction, and a wave's outstanding loads are what is counted (63 at most), not its outstanding bytes.
template <bool STACK>
struct Q80I8Shape {
    static constexpr int kStepBlocks = STACK ? 8 : 4;
    static constexpr int kPiece = STACK ? 16 : 8;              // bytes per weight load and lane
    static constexpr int kColStride = 34 * kStepBlocks + 4;    // LDS bytes per column of a staged step: an odd number of
                                                               // dwords, so that the 16 columns start in different banks
    static constexpr int kTileBytes = 16 * kColStride;
};

// Activation operand of one step as loaded.  Three-plane form: per block three digit planes (this lane's row and k
// group) and the block scales of the lane's four output rows.  Stacked form: the lane's 64 bytes (8 blocks).
template <bool STACK>
struct Q80I8Acts {
    uint2 a[STACK ? 1 : 4][3];
    float4 e[STACK ? 1 : 4];
    uint4 s8[STACK ? 4 : 1];
};

// MODE 0: a wave owns 16 columns.  KSPLIT 1: the whole K; KSPLIT 4: the four waves of a workgroup share the 16
//         columns and each walks a quarter of the steps, partial tiles added in wave order through LDS.
// MODE 1: a wave owns 8 columns of gate and the same 8 of up (B columns 0-7 / 8-15), the whole K; the four waves of a
//         workgroup are 32 consecutive columns = one q8_0-sized block of the hidden row, which is SwiGLU'd and packed.
// A wave never waits for another inside the K loop.  Weights: the 16 columns of a step (136 bytes each as 8-byte
// pieces, or 272 bytes as 16-byte pieces in the stacked form) are requested D steps ahead, pass through a wave-private
// LDS tile, and are read back as the 8 quants of (column, block, k group) plus the block's scale.  Activations:
// requested with the same lead, always BEFORE the weight request of the same step, so that a wait for them never waits
// for younger weight loads (loads return in issue order); the first requests before the loop go out in the loop's own
// order, pinned, so that every wait inside the loop names exactly the loads it needs and three steps stay in flight.
// STACK: at most four rows, stacked pack: one matrix instruction per block; lane (j, g) then holds digit g of rows
// 0-3, every digit is summed over K on its own, and the three sums meet once at the end.
template <int MODE, int KSPLIT, bool STACK>
__global__ __launch_bounds__(256, 2) void q80i8_gemm_kernel(Q80I8Args p) {
    constexpr int kWaves = 4;      // (eight waves splitting K, 512 threads, was measured for the down projection: 21.4 against 20.5 us)
    using SH = Q80I8Shape<STACK>;
    constexpr int kStepBlocks = SH::kStepBlocks, kPiece = SH::kPiece, kColStride = SH::kColStride, kTileBytes = SH::kTileBytes;
    using WPiece = typename std::conditional<STACK, uint4, uint2>::type;
    __shared__ __attribute__((aligned(16))) uint8_t w_lds[kWaves][kTileBytes];
    __shared__ float s_tile[kWaves][16][17];
    // (Handing a step's activation planes round the four waves through LDS, one barrier per step, instead of every wave
    // fetching them for itself: measured, gate + up 31 -> 46 us -- the barrier makes every step wait for the slowest
    // wave's loads.  The planes are half of the bytes a CU requests: a kernel that only reads, with this kernel's
    // addressing, takes 25.7 us for the 125 MB of gate + up alone and 30.2 us with the planes.)
    const int tid = threadIdx.x, lane = tid & 63;
    // the wave index as a scalar: everything derived from it (tile, step range, base addresses) then lives in scalar
    // registers and the loads take their base from there
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int j = lane & 15, g = lane >> 4;
    const int nsteps_all = p.K / (32 * kStepBlocks);
    const size_t col_stride = (size_t)(p.K >> 5) * 34;
    int n0, s0, s1;
    if (MODE == 0) {
        n0 = (KSPLIT == 1 ? blockIdx.x * 4 + wave : blockIdx.x) * 16;
        if (n0 >= p.N) n0 = (p.N - 1) / 16 * 16;              // surplus waves repeat the last tile (no early exit: barriers)
        s0 = KSPLIT == 1 ? 0 : (int)(((long long)wave * nsteps_all) / KSPLIT);
        s1 = KSPLIT == 1 ? nsteps_all : (int)(((long long)(wave + 1) * nsteps_all) / KSPLIT);
    } else {
        n0 = (blockIdx.x * 4 + wave) * 8;
        s0 = 0; s1 = nsteps_all;
    }
    // ---- weight pieces of this lane: piece q of the 16-column step tile (17 pieces per column), q = lane + 64 i
    // (MODE 1: the up matrix is addressed from the gate matrix's base; both lie in one address space)
    const uint8_t* w_base = p.W0 + (size_t)n0 * col_stride;
    const ptrdiff_t up_delta = MODE == 1 ? p.W1 - p.W0 : 0;
    ptrdiff_t w_off[5];
    int w_dst[5];
#pragma unroll
    for (int i = 0; i < 5; ++i) {
        int q = i * 64 + lane;
        if (q >= 272) q = lane;               // no such piece: repeat this lane's first one, so that no load sits under a branch
        const int c = q / 17, piece = q % 17;
        if (MODE == 0) {
            const int cc = n0 + c < p.N ? c : p.N - 1 - n0;
            w_off[i] = (ptrdiff_t)cc * (ptrdiff_t)col_stride + kPiece * piece;
        } else {
            w_off[i] = (ptrdiff_t)(c & 7) * (ptrdiff_t)col_stride + kPiece * piece + (c < 8 ? 0 : up_delta);
        }
        w_dst[i] = c * kColStride + kPiece * piece;
    }
    uint8_t* my_w = w_lds[wave];
    // ---- activation addressing: A-operand row j (rows at or above MP are zero), k group g
    const int blk_bytes = q80i8_block_bytes(STACK ? 0 : p.MP);
    const bool row_live = STACK || j < p.MP;
    const uint32_t a_off = STACK ? (uint32_t)(lane * 16) : (uint32_t)((g * p.MP + (row_live ? j : 0)) * 8);
    const int plane = STACK ? 0 : 4 * p.MP * 8;
    const uint32_t e_off = (uint32_t)(3 * plane + 16 * g);
    // STACK: the 32 block scales of a step (8 blocks x 4 rows), one per lane 0-31, fetched with one load per step
    const uint32_t sv_off = (uint32_t)(64 * 64 + (lane & 31) * 4);
    constexpr int D = STACK ? 4 : 2;          // steps in flight (the three-plane form has no registers for more)

    WPiece wr[D][5];
    Q80I8Acts<STACK> acts[D];
    float sv[D];
    auto issue_w = [&](WPiece (&dst)[5], int step) {
        step = step < s1 ? step : s1 - 1;
        const uint8_t* base = w_base + (size_t)step * (34 * kStepBlocks);
#pragma unroll
        for (int i = 0; i < 5; ++i) dst[i] = *reinterpret_cast<const WPiece*>(base + w_off[i]);
    };
    // three-plane form: block b of a step; stacked form: the whole step (called with b == 0 only)
    auto issue_a_block = [&](Q80I8Acts<STACK>& act, float& sv_set, int b, int step) {
        step = step < s1 ? step : s1 - 1;
        if constexpr (STACK) {
            const uint8_t* base = p.pack + (size_t)step * kStackStepBytes;                    // uniform
#pragma unroll
            for (int i = 0; i < 4; ++i) act.s8[i] = *reinterpret_cast<const uint4*>(base + a_off + 1024 * i);
            sv_set = *reinterpret_cast<const float*>(base + sv_off);
        } else {
            const uint8_t* base = p.pack + (size_t)(step * kStepBlocks + b) * blk_bytes;      // uniform
#pragma unroll
            for (int d = 0; d < 3; ++d) act.a[b][d] = *reinterpret_cast<const uint2*>(base + d * plane + a_off);
            act.e[b] = *reinterpret_cast<const float4*>(base + e_off);
        }
    };
    float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    auto compute_block = [&](const Q80I8Acts<STACK>& act, float sv_cur, int b) {
        const uint8_t* blk = my_w + j * kColStride + 34 * b;
        const float dw = m40_h2f(*reinterpret_cast<const uint16_t*>(blk));
        uint2 bq;
        if (b & 1) {                       // quants 4-byte aligned
            const uint32_t* w = reinterpret_cast<const uint32_t*>(blk + 2 + 8 * g);
            bq = make_uint2(w[0], w[1]);
        } else {                           // quants start two bytes into an aligned word
            const uint32_t* w = reinterpret_cast<const uint32_t*>(blk + 8 * g);
            bq = make_uint2(__builtin_amdgcn_alignbyte(w[1], w[0], 2), __builtin_amdgcn_alignbyte(w[2], w[1], 2));
        }
        const long B = __builtin_bit_cast(long, bq);
        const i32x4 z = {0, 0, 0, 0};
        if constexpr (STACK) {
            const uint4 two = act.s8[b >> 1];
            const uint2 a8 = (b & 1) ? make_uint2(two.z, two.w) : make_uint2(two.x, two.y);
            const i32x4 rr = __builtin_amdgcn_mfma_i32_16x16x32_i8(__builtin_bit_cast(long, a8), B, z, 0, 0, 0);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float sa = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, sv_cur), 4 * b + r));
                acc[r] = fmaf(sa * dw, (float)rr[r], acc[r]);
            }
            return;
        } else {
        uint2 a0 = act.a[b][0], a1 = act.a[b][1], a2 = act.a[b][2];
        if (!row_live) { a0 = make_uint2(0, 0); a1 = a0; a2 = a0; }
        const i32x4 r1 = __builtin_amdgcn_mfma_i32_16x16x32_i8(__builtin_bit_cast(long, a0), B, z, 0, 0, 0);
        const i32x4 r2 = __builtin_amdgcn_mfma_i32_16x16x32_i8(__builtin_bit_cast(long, a1), B, z, 0, 0, 0);
        const i32x4 r3 = __builtin_amdgcn_mfma_i32_16x16x32_i8(__builtin_bit_cast(long, a2), B, z, 0, 0, 0);
        const float sa[4] = {act.e[b].x, act.e[b].y, act.e[b].z, act.e[b].w};
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float t = fmaf((float)(r1[r] * 128 + r2[r]), 128.0f, (float)r3[r]);
            acc[r] = fmaf(sa[r] * dw, t, acc[r]);
        }
        }
    };

    if (s0 < s1) {
        // Issue order, kept through the loop: A(s), W(s) for the D steps in flight, oldest first; a step consumes its
        // register set and refills it with step s + D, activations before weights.
#pragma unroll
        for (int i = 0; i < D; ++i) {
#pragma unroll
            for (int b = 0; b < (STACK ? 1 : kStepBlocks); ++b) issue_a_block(acts[i], sv[i], b, s0 + i);
            // the order of these first requests must be the loop's own (waits count outstanding loads in issue order:
            // were the compiler free to interleave them, the loop's waits would have to assume the worst of both orders)
            __builtin_amdgcn_sched_barrier(0);
            issue_w(wr[i], s0 + i);
            __builtin_amdgcn_sched_barrier(0);
        }
        auto step = [&](auto set_c, int s) {
            constexpr int SET = decltype(set_c)::value;
            // weights of this step -> the wave's LDS tile (waits for them and for everything older: this step's
            // activations; the younger steps stay in flight)
#pragma unroll
            for (int i = 0; i < 5; ++i) {
                uint32_t* dst = reinterpret_cast<uint32_t*>(my_w + w_dst[i]);      // 4-byte aligned only
                dst[0] = wr[SET][i].x; dst[1] = wr[SET][i].y;
                if constexpr (STACK) { dst[2] = wr[SET][i].z; dst[3] = wr[SET][i].w; }
            }
            const float sv_cur = sv[SET];
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int b = 0; b < kStepBlocks; ++b) {
                compute_block(acts[SET], sv_cur, b);
                if (!STACK) issue_a_block(acts[SET], sv[SET], b, s + D);     // the block's registers are free again
                __builtin_amdgcn_sched_barrier(0);
            }
            if (STACK) issue_a_block(acts[SET], sv[SET], 0, s + D);
            issue_w(wr[SET], s + D);
            __builtin_amdgcn_sched_barrier(0);
        };
        using std::integral_constant;
        int s = s0;
        for (; s + D <= s1; s += D) {
            step(integral_constant<int, 0>(), s);
            step(integral_constant<int, 1>(), s + 1);
            if (D == 4) {
                step(integral_constant<int, D - 2>(), s + 2);
                step(integral_constant<int, D - 1>(), s + 3);
            }
        }
        if (s < s1) step(integral_constant<int, 0>(), s);
        if (D == 4 && s + 1 < s1) step(integral_constant<int, 1>(), s + 1);
        if (D == 4 && s + 2 < s1) step(integral_constant<int, D - 2>(), s + 2);
    }

    if (STACK) {
        // lane (j, g) holds digit g of rows r: the three sums meet in the lanes g = 0
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float d2 = __shfl(acc[r], j + 16, 64), d3 = __shfl(acc[r], j + 32, 64);
            acc[r] = g == 0 ? fmaf(acc[r], 16384.0f, fmaf(d2, 128.0f, d3)) : 0.0f;
        }
    }
    // lane (j, g) holds rows 4g + r of column j
    if (MODE == 0) {
        if (KSPLIT > 1) {
#pragma unroll
            for (int r = 0; r < 4; ++r) s_tile[wave][4 * g + r][j] = acc[r];
            __syncthreads();
            const int m = tid >> 4, c = tid & 15;
            float v = s_tile[0][m][c];
#pragma unroll
            for (int w = 1; w < KSPLIT; ++w) v += s_tile[w][m][c];
            if (m < p.M && n0 + c < p.N) p.C[(size_t)m * p.N + n0 + c] = v;
        } else {
            const bool tile_live = (blockIdx.x * 4 + wave) * 16 < p.N;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int m = 4 * g + r;
                if (tile_live && m < p.M && n0 + j < p.N) p.C[(size_t)m * p.N + n0 + j] = acc[r];
            }
        }
    } else {
        // SwiGLU of gate (lanes j < 8) and up (j >= 8, eight lanes on), then the block's digit pack
        float* hbuf = &s_tile[0][0][0];          // [16 rows][32 columns], stride 33
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float up = __shfl_xor(acc[r], 8, 64);
            const float gt = acc[r];
            const float h = gt / (1.0f + expf(-gt)) * up;
            if (j < 8) hbuf[(4 * g + r) * 33 + wave * 8 + j] = h;
        }
        // 32 hidden columns = block blockIdx.x of the down projection's K
        if (!STACK && tid < 16) reinterpret_cast<float*>(p.out_pack + (size_t)blockIdx.x * blk_bytes + 3 * plane)[tid] = 0.0f;
        __syncthreads();
        const int m = tid >> 4, pair = tid & 15;
        q80i8_pack_pair(hbuf[m * 33 + 2 * pair], hbuf[m * 33 + 2 * pair + 1], m, pair, STACK ? 0 : p.MP, p.out_pack, (int)blockIdx.x);
    }
}

size_t pack_bytes(int K) { return (size_t)(K >> 5) * q80i8_block_bytes(16); }

}  // namespace

// 3 <= M <= 16, K a multiple of 128 -- of 256 up to four rows -- (whole steps), the context's packing buffer large
// enough.  The stacked form also needs the matrix 16-byte aligned (its columns then are: 272 bytes per 256 k).
bool m40_q80_i8_supported(const M40llmCudaContext* ctx, uint32_t stream_kind, int M, int N, int K) {
    if (!ctx || stream_kind > 1) return false;
    if (M < 3 || M > 16 || N < 1 || K < 128 || K % 128 != 0) return false;
    if (M <= 4 && K % 256 != 0) return false;
    return pack_bytes(K) <= ctx->scratch[stream_kind].gemm_pack_bytes;
}

static int rows_padded(int M) { return M <= 4 ? 0 : (M <= 8 ? 8 : 16); }   // 0: the stacked form

static void launch_gemm0(hipStream_t stream, const Q80I8Args& a) {
    const int tiles = (a.N + 15) / 16;
    // few tiles: one tile per workgroup with K split over its waves, so that the grid still covers the CUs
    const bool whole_k = tiles >= 1024 || a.K / (32 * (a.MP == 0 ? 8 : 4)) < 4;
    if (a.MP == 0) {
        if (whole_k) q80i8_gemm_kernel<0, 1, true><<<(tiles + 3) / 4, 256, 0, stream>>>(a);
        else q80i8_gemm_kernel<0, 4, true><<<tiles, 256, 0, stream>>>(a);
    } else {
        if (whole_k) q80i8_gemm_kernel<0, 1, false><<<(tiles + 3) / 4, 256, 0, stream>>>(a);
        else q80i8_gemm_kernel<0, 4, false><<<tiles, 256, 0, stream>>>(a);
    }
}

int m40_launch_q80_i8(M40llmCudaContext* ctx, hipStream_t stream, uint32_t stream_kind, const float* A, const uint8_t* W,
                      float* C, int M, int N, int K) {
    if (!m40_q80_i8_supported(ctx, stream_kind, M, N, K)) return -2;
    if (M <= 4 && !m40_aligned16(W)) return -2;
    (void)hipGetLastError();
    uint8_t* pack = static_cast<uint8_t*>(ctx->scratch[stream_kind].gemm_pack);
    const int MP = rows_padded(M);
    q80i8_pack_kernel<<<K >> 5, 256, 0, stream>>>(A, M, MP, K, pack);
    Q80I8Args a{};
    a.pack = pack; a.W0 = W; a.C = C; a.M = M; a.MP = MP; a.N = N; a.K = K;
    launch_gemm0(stream, a);
    return hipGetLastError() == hipSuccess ? 0 : -2;
}

// out[M][d_model] = (silu(x Wg^T) * (x Wu^T)) Wd^T
int m40_launch_q80_i8_ffn(M40llmCudaContext* ctx, hipStream_t stream, uint32_t stream_kind, const float* x,
                          const uint8_t* wg, const uint8_t* wu, const uint8_t* wd, float* out, int M, int d_model, int ffn) {
    if (!m40_q80_i8_supported(ctx, stream_kind, M, ffn, d_model) || !m40_q80_i8_supported(ctx, stream_kind, M, d_model, ffn))
        return -2;
    const size_t x_bytes = (pack_bytes(d_model) + 255) & ~(size_t)255;
    if (x_bytes + pack_bytes(ffn) > ctx->scratch[stream_kind].gemm_pack_bytes) return -2;
    if (M <= 4 && !(m40_aligned16(wg) && m40_aligned16(wu) && m40_aligned16(wd))) return -2;
    (void)hipGetLastError();
    uint8_t* xp = static_cast<uint8_t*>(ctx->scratch[stream_kind].gemm_pack);
    uint8_t* hp = xp + x_bytes;
    const int MP = rows_padded(M);
    q80i8_pack_kernel<<<d_model >> 5, 256, 0, stream>>>(x, M, MP, d_model, xp);
    Q80I8Args a{};
    a.pack = xp; a.W0 = wg; a.W1 = wu; a.out_pack = hp; a.M = M; a.MP = MP; a.N = ffn; a.K = d_model;
    if (MP == 0) q80i8_gemm_kernel<1, 1, true><<<ffn / 32, 256, 0, stream>>>(a);
    else q80i8_gemm_kernel<1, 1, false><<<ffn / 32, 256, 0, stream>>>(a);
    Q80I8Args b{};
    b.pack = hp; b.W0 = wd; b.C = out; b.M = M; b.MP = MP; b.N = d_model; b.K = ffn;
    launch_gemm0(stream, b);
    return hipGetLastError() == hipSuccess ? 0 : -2;
}
