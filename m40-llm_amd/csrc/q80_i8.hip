// q8_0 skinny GEMM and SwiGLU FFN for 2 <= M <= 16 rows on the int8 matrix instruction of gfx950.
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
// Up to four rows the three planes of all rows are stacked into the 16 operand rows: one instruction per block.  Five to
// eight rows take two operands per block -- digits 1 and 2 of the eight rows fill the sixteen rows of the first, digit 3
// the low half of the second -- two instructions and two thirds of the plane bytes.
//
// Launches: a small pack kernel turns the f32 rows into digit planes (laid out in the order the A operand is
// loaded), then the product kernel; the FFN form packs its SwiGLU output itself (a workgroup produces whole
// 32-column blocks of the hidden row), so gate / up / down take three launches in all -- two in the stacked form up
// to K = 4096, whose gate + up workgroups also pack the input rows themselves.  Where a product has few columns and a
// long K (the down projection), two workgroups share a column group, each adds its half of K into the result, and the
// launch before (pack, or gate + up) has cleared it: two terms onto zero, the same bits in either order.
#include "common.hpp"

#include <type_traits>

namespace {

typedef int i32x4 __attribute__((ext_vector_type(4)));

// Packed activations, stored per step of eight blocks (256 k) as planes of 1 KB -- a load instruction of a wave reads
// one plane, 16 bytes per lane, one contiguous kilobyte -- followed by the step's block scales 2^(E-20) as f32.
//   MP = 16, "three planes", 5 to 16 rows (rows at and above M are zero): twelve planes [block pair][digit]
//   [lane = 16 (k / 8) + row][block of the pair][8 bytes], then the scales [block][row].
//   MP = 0, "stacked", for at most four rows: the operand row 4 d + m holds digit d of row m (rows 12-15 zero), so
//   that a single matrix instruction multiplies all three digits: four planes [block pair][lane = 16 (k / 8) + operand
//   row][block of the pair][8 bytes], then the scales [block][row < 4].
//   MP = 8, "two operands", 5 to 8 rows: eight planes [block pair][operand][lane = 16 (k / 8) + operand row][block of
//   the pair][8 bytes]; operand 0 holds digit 1 of row m in operand row m and digit 2 in operand row 8 + m, operand 1
//   digit 3 in operand row m and zeros in rows 8-15: two matrix instructions per block instead of three, two thirds of
//   the plane bytes.  Then the scales [block][operand row], rows 8-15 repeating rows 0-7.
constexpr int kStepBlocks = 8;
constexpr int kStackStepBytes = 4 * 1024 + kStepBlocks * 4 * 4;        // 4224
constexpr int kPlaneStepBytes = 12 * 1024 + kStepBlocks * 16 * 4;      // 12800
constexpr int kTwoStepBytes = 8 * 1024 + kStepBlocks * 16 * 4;         // 8704
__host__ __device__ constexpr int q80i8_step_bytes(int MP) { return MP == 0 ? kStackStepBytes : (MP == 8 ? kTwoStepBytes : kPlaneStepBytes); }

// Digits of one element under its block's scale: n = rint(v * 2^(20 - ex)), |n| <= 2^20, cut into balanced base-128
// digits n = (d1 * 128 + d2) * 128 + d3 with d2, d3 in [-64, 63] and |d1| <= 64 (exact integer arithmetic, one rounding).
__device__ __forceinline__ void q80i8_digits(float v, float inv, int& d1, int& d2, int& d3) {
    const float s = fminf(fmaxf(v * inv, -1048576.0f), 1048576.0f);
    const int n = (int)rintf(s);
    d3 = (n << 25) >> 25;
    const int n1 = (n - d3) >> 7;
    d2 = (n1 << 25) >> 25;
    d1 = (n1 - d2) >> 7;
}
// |v|, or +inf for a NaN: a block that holds a non-finite element gets a NaN block scale, so that every output fed by it
// is NaN (the f32 product of the reference, kernels.cu:5037-5052, would give +-inf or NaN there; never a finite value)
__device__ __forceinline__ float q80i8_abs_or_inf(float v) { return fabsf(v) <= 3.402823466e+38f ? fabsf(v) : INFINITY; }
// the low bytes of four values as one word
__device__ __forceinline__ uint32_t q80i8_bytes4(int a, int b, int c, int d) {
    const uint32_t ab = __builtin_amdgcn_perm((uint32_t)b, (uint32_t)a, 0x0c0c0400u);
    const uint32_t cd = __builtin_amdgcn_perm((uint32_t)d, (uint32_t)c, 0x0c0c0400u);
    return __builtin_amdgcn_perm(cd, ab, 0x05040100u);
}

// Digits of two neighbouring elements of one row of one block.  The 16 threads of a row (lanes pair = 0..15 of an
// aligned group of 16) hold the row's 32 values; digits go to dst in A-operand order, the exponent to dst's tail.
__device__ __forceinline__ void q80i8_pack_pair(float v0, float v1, int m, int pair, int MP, uint8_t* pack, int blk) {
    float mx = fmaxf(q80i8_abs_or_inf(v0), q80i8_abs_or_inf(v1));
#pragma unroll
    for (int o = 1; o < 16; o <<= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
    const float block_scale_bad = __builtin_nanf("");
    int ex = 0;
    if (mx > 0.0f && mx < INFINITY) (void)frexpf(mx, &ex);        // mx = f * 2^ex, f in [0.5, 1)
    ex = ex < -100 ? -100 : (ex > 100 ? 100 : ex);
    const float inv = ldexpf(1.0f, 20 - ex);                       // |a| * inv < 2^20
    const float v[2] = {v0, v1};
    int d[3][2];
#pragma unroll
    for (int e = 0; e < 2; ++e) q80i8_digits(mx < INFINITY ? v[e] : 0.0f, inv, d[0][e], d[1][e], d[2][e]);
    const int k = 2 * pair, kg = k >> 3, kb = k & 7;
    // value = 2^(ex - 20) * ((d1 * 128 + d2) * 128 + d3)
    const int b = blk % kStepBlocks;
    if (MP == 0) {
        uint8_t* step = pack + (size_t)(blk / kStepBlocks) * kStackStepBytes;
        if (m < 4) {
#pragma unroll
            for (int dg = 0; dg < 3; ++dg) {
                const uint16_t two = (uint16_t)((d[dg][0] & 0xff) | ((d[dg][1] & 0xff) << 8));
                *reinterpret_cast<uint16_t*>(step + (b >> 1) * 1024 + (kg * 16 + dg * 4 + m) * 16 + (b & 1) * 8 + kb) = two;
            }
            if (pair == 0) reinterpret_cast<float*>(step + 64 * 64)[b * 4 + m] = mx < INFINITY ? ldexpf(1.0f, ex - 20) : block_scale_bad;
        } else if (m >= 12) {
            *reinterpret_cast<uint16_t*>(step + (b >> 1) * 1024 + (kg * 16 + m) * 16 + (b & 1) * 8 + kb) = 0;
        }
        return;
    }
    if (MP == 8) {
        uint8_t* step = pack + (size_t)(blk / kStepBlocks) * kTwoStepBytes;
        if (m < 8) {
            // (operand, operand row): digit 1 -> (0, m), digit 2 -> (0, 8 + m), digit 3 -> (1, m), zeros -> (1, 8 + m)
            const uint16_t two[4] = {(uint16_t)((d[0][0] & 0xff) | ((d[0][1] & 0xff) << 8)), (uint16_t)((d[1][0] & 0xff) | ((d[1][1] & 0xff) << 8)),
                                     (uint16_t)((d[2][0] & 0xff) | ((d[2][1] & 0xff) << 8)), (uint16_t)0};
#pragma unroll
            for (int o = 0; o < 4; ++o)
                *reinterpret_cast<uint16_t*>(step + ((b >> 1) * 2 + (o >> 1)) * 1024 + (kg * 16 + (o & 1) * 8 + m) * 16 + (b & 1) * 8 + kb) = two[o];
            if (pair == 0) {
                const float sc = mx < INFINITY ? ldexpf(1.0f, ex - 20) : block_scale_bad;
                reinterpret_cast<float*>(step + 8 * 1024)[b * 16 + m] = sc;
                reinterpret_cast<float*>(step + 8 * 1024)[b * 16 + 8 + m] = sc;
            }
        }
        return;
    }
    uint8_t* step = pack + (size_t)(blk / kStepBlocks) * kPlaneStepBytes;
#pragma unroll
    for (int dg = 0; dg < 3; ++dg) {
        const uint16_t two = (uint16_t)((d[dg][0] & 0xff) | ((d[dg][1] & 0xff) << 8));
        *reinterpret_cast<uint16_t*>(step + ((b >> 1) * 3 + dg) * 1024 + (kg * 16 + m) * 16 + (b & 1) * 8 + kb) = two;
    }
    if (pair == 0) reinterpret_cast<float*>(step + 12 * 1024)[b * 16 + m] = mx < INFINITY ? ldexpf(1.0f, ex - 20) : block_scale_bad;
}

// grid = K / 32 blocks, 256 threads: thread (row tid / 16, pair tid % 16).  zero (may be null): zero_count floats the
// launch clears on the side (the result of a product whose two K halves are added into it).
__global__ __launch_bounds__(256) void q80i8_pack_kernel(const float* __restrict__ A, int M, int MP, int K, uint8_t* pack,
                                                         float* zero, int zero_count) {
    const int blk = blockIdx.x, m = threadIdx.x >> 4, pair = threadIdx.x & 15;
    float2 v = make_float2(0.0f, 0.0f);
    if (m < M) v = *reinterpret_cast<const float2*>(A + (size_t)m * K + 32 * blk + 2 * pair);
    if (zero)
        for (int i = blk * 256 + (int)threadIdx.x; i < zero_count; i += (int)gridDim.x * 256) zero[i] = 0.0f;
    q80i8_pack_pair(v.x, v.y, m, pair, MP, pack, blk);
}

// Stacked digits of eight consecutive elements (k group kg of block blk) of row m < 4, written into the step planes
// at `planes` (LDS).  The four threads of a (block, row) are four neighbouring lanes; the arithmetic of q80i8_pack_pair.
__device__ __forceinline__ void q80i8_pack8_stacked(const float4& lo, const float4& hi, int m, int kg, int blk, bool store,
                                                    uint8_t* planes) {
    const float v[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    float mx = 0.0f;
#pragma unroll
    for (int e = 0; e < 8; ++e) mx = fmaxf(mx, q80i8_abs_or_inf(v[e]));
    mx = fmaxf(mx, __shfl_xor(mx, 1, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 2, 64));
    int ex = 0;
    if (mx > 0.0f && mx < INFINITY) (void)frexpf(mx, &ex);
    ex = ex < -100 ? -100 : (ex > 100 ? 100 : ex);
    const float inv = mx < INFINITY ? ldexpf(1.0f, 20 - ex) : 0.0f;
    int d[3][8];
#pragma unroll
    for (int e = 0; e < 8; ++e) q80i8_digits(mx < INFINITY ? v[e] : 0.0f, inv, d[0][e], d[1][e], d[2][e]);
    if (!store) return;
    uint8_t* step = planes + (size_t)(blk / kStepBlocks) * kStackStepBytes;
    const int b = blk % kStepBlocks;
#pragma unroll
    for (int dg = 0; dg < 3; ++dg)
        *reinterpret_cast<uint2*>(step + (b >> 1) * 1024 + (kg * 16 + dg * 4 + m) * 16 + (b & 1) * 8) =
            make_uint2(q80i8_bytes4(d[dg][0], d[dg][1], d[dg][2], d[dg][3]), q80i8_bytes4(d[dg][4], d[dg][5], d[dg][6], d[dg][7]));
    if (kg == 0) reinterpret_cast<float*>(step + 4 * 1024)[b * 4 + m] = mx < INFINITY ? ldexpf(1.0f, ex - 20) : __builtin_nanf("");
}

struct Q80I8Args {
    const uint8_t* pack;       // packed activations
    const uint8_t* W0;         // MODE 0: the matrix; MODE 1: gate
    const uint8_t* W1;         // MODE 1: up
    float* C;                  // MODE 0: [M][N]
    uint8_t* out_pack;         // MODE 1: packed SwiGLU output (the A operand of the down projection)
    const float* x;            // SELF: the f32 rows [M][K], packed by every workgroup for itself
    float* zero;               // MODE 1: cleared by the launch (zero_count floats), or null: the result of a down projection
    int zero_count;            //         whose two K halves are added into it
    int M, MP, N, K;
};

// A step is 8 q8_0 blocks (256 k): 272 bytes per column = 17 pieces of 16 bytes (columns 16-byte aligned).  What a
// wave may have outstanding is counted in load instructions (63 at most), not in bytes, and the launch time follows
// the number of load instructions a CU issues per weight byte: hence 16 bytes per lane and load throughout.
constexpr int kPiece = 16;                            // bytes per weight load and lane
constexpr int kColStride = 34 * kStepBlocks + 4;      // LDS bytes per column of a staged step: an odd number of dwords,
                                                      // so that the 16 columns start in different banks
constexpr int kTileBytes = 16 * kColStride;

// Activation operand of one step as loaded: the lane's 16 bytes of every plane, and its block scales.  Three-plane
// form: e[h] = the scales of block 4 h + (lane & 3) for the lane's four output rows -- the four lanes of a quad hold the
// four blocks, and the arithmetic fetches block b's from quad lane b & 3.  Stacked form: one scale per lane 0-31.
template <bool STACK, bool TWO = false>
struct Q80I8Acts {
    uint4 pl[STACK ? 4 : (TWO ? 8 : 12)];
    float4 e[STACK ? 1 : 2];
    float sv;
};

template <int... I, class F>
__device__ __forceinline__ void q80i8_unrolled(std::integer_sequence<int, I...>, F&& f) {
    (f(std::integral_constant<int, I>()), ...);
}

// MODE 0: a wave owns 16 columns.  KSPLIT 1: the whole K; KSPLIT 4: the four waves of a workgroup share the 16
//         columns and each walks a quarter of the steps, partial tiles added in wave order through LDS.
// MODE 1: a wave owns 8 columns of gate and the same 8 of up (B columns 0-7 / 8-15), the whole K; the four waves of a
//         workgroup are 32 consecutive columns = one q8_0-sized block of the hidden row, which is SwiGLU'd and packed.
// A wave never waits for another inside the K loop.  Weights: the 16 columns of a step (272 bytes each as 16-byte
// pieces) are requested D steps ahead, pass through a wave-private
// LDS tile, and are read back as the 8 quants of (column, block, k group) plus the block's scale.  Activations:
// requested with the same lead, always BEFORE the weight request of the same step, so that a wait for them never waits
// for younger weight loads (loads return in issue order); the first requests before the loop go out in the loop's own
// order, pinned, so that every wait inside the loop names exactly the loads it needs and three steps stay in flight.
// STACK: at most four rows, stacked pack: one matrix instruction per block; lane (j, g) then holds digit g of rows
// 0-3, every digit is summed over K on its own, and the three sums meet once at the end.
// T (three-plane form only): column tiles per wave.  With T = 2 a wave owns 32 columns and multiplies every
// activation plane it fetches with two weight tiles: the planes of 16 rows are three times the bytes of a 16-column
// weight tile, and fetching them once per 32 columns instead of once per 16 halves the loads a CU issues beside its
// weights (FFN at 16 rows: 91 -> 75 us with that alone).
// WAVES / KSPLIT column groups per workgroup, wave = group * KSPLIT + K part.
// KHALVES = 2 (MODE 0): two workgroups share a column group, each walks half of K and ADDS its sums into C, which the
// launch before has cleared: 0 + a + b is the same f32 in either order, so the result does not depend on timing.  A
// workgroup then needs only half of the activation planes, and twice as many workgroups can own two tiles each.
// SELF (stacked gate + up only, K <= 4096): no pack launch -- every workgroup turns the f32 rows into the digit planes of
// all steps itself, in LDS (4224 bytes per step, dynamic), behind its first weight requests, and the K loop reads its
// activation operands from there.
// DEPTH: steps in flight per wave, 0 = the form's default.  What pays is about 70 KB of weight requests outstanding per
// CU, not more (measured: 104 KB and 139 KB are slower, 35 KB too): a launch that puts two workgroups on a CU runs
// with half the depth of one that puts one there.
// TWO (not STACK): the two-operand form of 5 to 8 rows (digits 1 and 2 of the eight rows in one operand, digit 3 in the low
// half of a second): two matrix instructions per block and tile.
template <int MODE, int KSPLIT, bool STACK, int T = 1, int WAVES = 4, int KHALVES = 1, bool SELF = false, int DEPTH = 0,
          bool TWO = false>
__global__ __launch_bounds__(64 * WAVES, 2) void q80i8_gemm_kernel(Q80I8Args p) {
    static_assert(!TWO || !STACK, "two operands: a form of the unstacked kernel");
    static_assert(!SELF || (STACK && MODE == 1 && KSPLIT == 1 && WAVES == 4), "self-packing: the stacked gate + up launch");
    extern __shared__ __attribute__((aligned(16))) uint8_t q80i8_planes[];    // SELF: [step][4224]
    static_assert(KHALVES == 1 || (KHALVES == 2 && MODE == 0), "halves of K are added into a cleared result");
    static_assert(T == 1 || T == 2, "one or two column tiles per wave");
    constexpr int kWaves = WAVES;  // (stacked form, eight waves splitting K, measured for the down projection: 21.4 against 20.5 us)
    constexpr int kThreads = 64 * kWaves;
    constexpr int kGroups = kWaves / KSPLIT;
    static_assert(kGroups * KSPLIT == kWaves, "whole column groups");
    static_assert(MODE == 0 || (kGroups * 8 * T) % 32 == 0, "a workgroup's hidden columns are whole q8_0-sized blocks");
    using WPiece = uint4;
    constexpr int kCols = 16 * T;                      // columns of a wave
    constexpr int kPieces = kCols * 17;                // weight pieces of a step tile
    constexpr int kWLoads = (kPieces + 63) / 64;       // per lane
    __shared__ __attribute__((aligned(16))) uint8_t w_lds[kWaves][T * kTileBytes];
    __shared__ float s_tile[kWaves][16][kCols + 1];
    // (Handing a step's activation planes round the four waves through LDS, one barrier per step, instead of every wave
    // fetching them for itself: measured, gate + up 31 -> 46 us -- the barrier makes every step wait for the slowest
    // wave's loads.  The planes are half of the bytes a CU requests: a kernel that only reads, with this kernel's
    // addressing, takes 25.7 us for the 125 MB of gate + up alone and 30.2 us with the planes.)
    const int tid = threadIdx.x, lane = tid & 63;
    // the wave index as a scalar: everything derived from it (tile, step range, base addresses) then lives in scalar
    // registers and the loads take their base from there
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int j = lane & 15, g = lane >> 4;
    const int group = wave / KSPLIT, kpart = wave % KSPLIT;
    const int nsteps_all = p.K / (32 * kStepBlocks);
    const size_t col_stride = (size_t)(p.K >> 5) * 34;
    int n0, s0, s1;
    if (MODE == 0) {
        n0 = ((blockIdx.x / KHALVES) * kGroups + group) * kCols;
        if (n0 >= p.N) n0 = (p.N - 1) / kCols * kCols;        // surplus waves repeat the last tile (no early exit: barriers)
    } else {
        n0 = (blockIdx.x * kGroups + group) * 8 * T;
    }
    {
        // the workgroup's share of K (a half, or all of it), split over the K parts of a column group
        const int kparts = KSPLIT * KHALVES, part = (int)(blockIdx.x % KHALVES) * KSPLIT + kpart;
        s0 = (int)(((long long)part * nsteps_all) / kparts);
        s1 = (int)(((long long)(part + 1) * nsteps_all) / kparts);
    }
    // ---- weight pieces of this lane: piece q of the step tile (17 pieces per column), q = lane + 64 i
    // (MODE 1: B columns 16 t + 0..7 are gate columns n0 + 8 t + 0..7, 16 t + 8..15 the same columns of up; the up
    // matrix is addressed from the gate matrix's base: both lie in one address space)
    const uint8_t* w_base = p.W0 + (size_t)n0 * col_stride;
    const ptrdiff_t up_delta = MODE == 1 ? p.W1 - p.W0 : 0;
    ptrdiff_t w_off[kWLoads];
    int w_dst[kWLoads];
#pragma unroll
    for (int i = 0; i < kWLoads; ++i) {
        int q = i * 64 + lane;
        if (q >= kPieces) q = lane;           // no such piece: repeat this lane's first one, so that no load sits under a branch
        const int c = q / 17, piece = q % 17;
        if (MODE == 0) {
            const int cc = n0 + c < p.N ? c : p.N - 1 - n0;
            w_off[i] = (ptrdiff_t)cc * (ptrdiff_t)col_stride + kPiece * piece;
        } else {
            w_off[i] = (ptrdiff_t)(8 * (c >> 4) + (c & 7)) * (ptrdiff_t)col_stride + kPiece * piece + ((c & 8) ? up_delta : 0);
        }
        w_dst[i] = c * kColStride + kPiece * piece;
    }
    uint8_t* my_w = w_lds[wave];
    // ---- activation addressing: the lane's 16 bytes of every plane
    const uint32_t a_off = (uint32_t)(lane * 16);
    // STACK: the 32 block scales of a step (8 blocks x 4 rows), one per lane 0-31, fetched with one load per step;
    // three planes: [block][row] f32, the lane takes rows 4 g .. 4 g + 3 of blocks (lane & 3) and 4 + (lane & 3)
    const uint32_t sv_off = (uint32_t)(4 * 1024 + (lane & 31) * 4);
    const uint32_t e_off = (uint32_t)((TWO ? 8 : 12) * 1024 + (lane & 3) * 64 + g * 16);
    constexpr int kStepBytes = STACK ? kStackStepBytes : (TWO ? kTwoStepBytes : kPlaneStepBytes);
    constexpr int kPlanes = STACK ? 4 : (TWO ? 8 : 12);
    constexpr int D = DEPTH ? DEPTH : (STACK ? (T == 1 ? 4 : 2) : 2);   // steps in flight (two 32-column steps are as many bytes as four of 16
                                                 // columns; the three-plane form has no registers for more)

    // SELF: the rows' elements of this thread, requested before the weights (loads return in issue order).  Thread ->
    // (block 16 pass + tid / 16, row (tid / 4) % 4, k group tid % 4), eight passes for K <= 4096
    constexpr int kSelfPasses = SELF ? 8 : 1;
    float4 xr[kSelfPasses][2];
    if constexpr (SELF) {
        const int nblk = p.K >> 5, m = (tid >> 2) & 3, kg = tid & 3;
#pragma unroll
        for (int ps = 0; ps < kSelfPasses; ++ps) {
            const int blk = ps * 16 + (tid >> 4);
            const float* src = p.x + (size_t)(m < p.M ? m : 0) * p.K + 32 * (blk < nblk ? blk : 0) + 8 * kg;
            xr[ps][0] = reinterpret_cast<const float4*>(src)[0];
            xr[ps][1] = reinterpret_cast<const float4*>(src)[1];
        }
        __builtin_amdgcn_sched_barrier(0);
    }
    WPiece wr[D][kWLoads];
    Q80I8Acts<STACK, TWO> acts[D];
    auto issue_w = [&](WPiece (&dst)[kWLoads], int step) {
        step = step < s1 ? step : s1 - 1;
        const uint8_t* base = w_base + (size_t)step * (34 * kStepBlocks);
#pragma unroll
        for (int i = 0; i < kWLoads; ++i) dst[i] = *reinterpret_cast<const WPiece*>(base + w_off[i]);
    };
    auto issue_a = [&](Q80I8Acts<STACK, TWO>& act, int step) {
        step = step < s1 ? step : s1 - 1;
        const uint8_t* base = p.pack + (size_t)step * kStepBytes;                    // uniform
#pragma unroll
        for (int i = 0; i < kPlanes; ++i) act.pl[i] = *reinterpret_cast<const uint4*>(base + a_off + 1024 * i);
        if constexpr (STACK) {
            act.sv = *reinterpret_cast<const float*>(base + sv_off);
        } else {
            act.e[0] = *reinterpret_cast<const float4*>(base + e_off);
            act.e[1] = *reinterpret_cast<const float4*>(base + e_off + 256);
        }
    };
    // the planes of block pair `pair` (and, with it, the scales of the four blocks that pair completes)
    // (measured, 8 / 16 rows: gate + up and the two-halves products 3-4 % faster spread, FFN 55.3 -> 53.8 / 61.3 -> 59.2 us;
    // the K-split single GEMM of many columns 2 % slower, so it keeps its requests at the end of the step)
    constexpr bool kSpread = !STACK && (MODE == 1 || KHALVES == 2);
    auto issue_a_part = [&](Q80I8Acts<STACK, TWO>& act, int step, int pair) {
        step = step < s1 ? step : s1 - 1;
        const uint8_t* base = p.pack + (size_t)step * kStepBytes;
        constexpr int kPerPair = kPlanes / 4;
#pragma unroll
        for (int i = 0; i < kPerPair; ++i) act.pl[pair * kPerPair + i] = *reinterpret_cast<const uint4*>(base + a_off + 1024 * (pair * kPerPair + i));
        if constexpr (!STACK) {
            if (pair == 1) act.e[0] = *reinterpret_cast<const float4*>(base + e_off);
            if (pair == 3) act.e[1] = *reinterpret_cast<const float4*>(base + e_off + 256);
        }
    };
    float acc[T][4];
#pragma unroll
    for (int t = 0; t < T; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[t][r] = 0.0f;
    // B operand (the 8 quants of column 16 t + j, block b, k group g) and the block's scale, from the wave's tile:
    // read as whole words one block ahead of their use, put together when used
    struct WRaw { uint32_t w0, w1, w2; uint16_t d; };
    struct WOperand { long B; float dw; };
    auto weight_read = [&](int t, int b) -> WRaw {
        const uint8_t* blk = my_w + (16 * t + j) * kColStride + 34 * b;
        WRaw r;
        r.d = *reinterpret_cast<const uint16_t*>(blk);
        if (b & 1) {                       // quants 4-byte aligned
            const uint32_t* w = reinterpret_cast<const uint32_t*>(blk + 2 + 8 * g);
            r.w0 = w[0]; r.w1 = w[1]; r.w2 = 0;
        } else {                           // quants start two bytes into an aligned word
            const uint32_t* w = reinterpret_cast<const uint32_t*>(blk + 8 * g);
            r.w0 = w[0]; r.w1 = w[1]; r.w2 = w[2];
        }
        return r;
    };
    auto weight_operand = [&](const WRaw& r, int b) -> WOperand {
        const uint2 bq = (b & 1) ? make_uint2(r.w0, r.w1)
                                 : make_uint2(__builtin_amdgcn_alignbyte(r.w1, r.w0, 2), __builtin_amdgcn_alignbyte(r.w2, r.w1, 2));
        return WOperand{__builtin_bit_cast(long, bq), m40_h2f(r.d)};
    };
    auto compute_block = [&](const Q80I8Acts<STACK, TWO>& act, auto b_c, const WOperand (&w)[T]) {
        constexpr int b = decltype(b_c)::value;
        const i32x4 z = {0, 0, 0, 0};
        auto half = [](const uint4& two) { return __builtin_bit_cast(long, (b & 1) ? make_uint2(two.z, two.w) : make_uint2(two.x, two.y)); };
        if constexpr (STACK) {
            float sa[4];
#pragma unroll
            for (int r = 0; r < 4; ++r)
                sa[r] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, act.sv), 4 * b + r));
#pragma unroll
            for (int t = 0; t < T; ++t) {
                const float dw = w[t].dw;
                const i32x4 rr = __builtin_amdgcn_mfma_i32_16x16x32_i8(half(act.pl[b >> 1]), w[t].B, z, 0, 0, 0);
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[t][r] = fmaf(sa[r] * dw, (float)rr[r], acc[t][r]);
            }
        } else if constexpr (TWO) {
            const long a0 = half(act.pl[(b >> 1) * 2]), a1 = half(act.pl[(b >> 1) * 2 + 1]);
            constexpr int kQuad = (b & 3) * 0x55;
            const float4 eh = act.e[b >> 2];
#define M40_FROM_QUAD(v) __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), kQuad, 0xf, 0xf, true))
            const float sa[4] = {M40_FROM_QUAD(eh.x), M40_FROM_QUAD(eh.y), M40_FROM_QUAD(eh.z), M40_FROM_QUAD(eh.w)};
#undef M40_FROM_QUAD
            // operand rows 0-7 (lanes g < 2): digit 1 in the first product, digit 3 in the second; rows 8-15: digit 2, zero
            const float wgt = g < 2 ? 16384.0f : 128.0f;
#pragma unroll
            for (int t = 0; t < T; ++t) {
                const long B = w[t].B;
                const float dw = w[t].dw;
                const i32x4 r1 = __builtin_amdgcn_mfma_i32_16x16x32_i8(a0, B, z, 0, 0, 0);
                const i32x4 r2 = __builtin_amdgcn_mfma_i32_16x16x32_i8(a1, B, z, 0, 0, 0);
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[t][r] = fmaf(sa[r] * dw, fmaf((float)r1[r], wgt, (float)r2[r]), acc[t][r]);
            }
#pragma unroll
            for (int t = 0; t < T; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r) asm volatile("" : "+v"(acc[t][r]));
        } else {
            const long a0 = half(act.pl[(b >> 1) * 3]), a1 = half(act.pl[(b >> 1) * 3 + 1]), a2 = half(act.pl[(b >> 1) * 3 + 2]);
            // the block's scales sit in quad lane b & 3
            constexpr int kQuad = (b & 3) * 0x55;
            const float4 eh = act.e[b >> 2];
#define M40_FROM_QUAD(v) __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), kQuad, 0xf, 0xf, true))
            const float sa[4] = {M40_FROM_QUAD(eh.x), M40_FROM_QUAD(eh.y), M40_FROM_QUAD(eh.z), M40_FROM_QUAD(eh.w)};
#undef M40_FROM_QUAD
#pragma unroll
            for (int t = 0; t < T; ++t) {
                const long B = w[t].B;
                const float dw = w[t].dw;
                const i32x4 r1 = __builtin_amdgcn_mfma_i32_16x16x32_i8(a0, B, z, 0, 0, 0);
                const i32x4 r2 = __builtin_amdgcn_mfma_i32_16x16x32_i8(a1, B, z, 0, 0, 0);
                const i32x4 r3 = __builtin_amdgcn_mfma_i32_16x16x32_i8(a2, B, z, 0, 0, 0);
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    // |r1|, |r2|, |r3| <= 32 * 64 * 128 = 2^18 each.  The whole sum (r1 * 128 + r2) * 128 + r3 reaches 2^32 (a
                    // block of like-signed activations against like-signed large quants) and would wrap in 32 bits: the
                    // two low digits are joined as an integer (< 2^26), the leading one (exact as f32) is added by one
                    // fused multiply-add -- two roundings of <= 2^-24 of the block sum in place of none
                    const float sum = fmaf((float)r1[r], 16384.0f, (float)(r2[r] * 128 + r3[r]));
                    acc[t][r] = fmaf(sa[r] * dw, sum, acc[t][r]);
                }
            }
            // the sums are folded here, not wherever the compiler would sink them to: twelve result registers per
            // block and tile would otherwise stay live to the end of the step
#pragma unroll
            for (int t = 0; t < T; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r) asm volatile("" : "+v"(acc[t][r]));
        }
    };

    if (s0 < s1) {
        // Issue order, kept through the loop: A(s), W(s) for the D steps in flight, oldest first; a step consumes its
        // register set and refills it with step s + D, activations before weights.
#pragma unroll
        for (int i = 0; i < D; ++i) {
            if constexpr (!SELF) issue_a(acts[i], s0 + i);
            // the order of these first requests must be the loop's own (waits count outstanding loads in issue order:
            // were the compiler free to interleave them, the loop's waits would have to assume the worst of both orders)
            __builtin_amdgcn_sched_barrier(0);
            issue_w(wr[i], s0 + i);
            __builtin_amdgcn_sched_barrier(0);
        }
        if constexpr (SELF) {
            // operand rows 12-15 of every plane are zero
            for (int i = tid; i < nsteps_all * 4 * 4 * 4; i += kThreads) {
                const int st = i >> 6, pl = (i >> 4) & 3, kgz = (i >> 2) & 3, row = 12 + (i & 3);
                *reinterpret_cast<uint4*>(q80i8_planes + st * kStackStepBytes + pl * 1024 + (kgz * 16 + row) * 16) = make_uint4(0, 0, 0, 0);
            }
            const int nblk = p.K >> 5, m = (tid >> 2) & 3, kg = tid & 3;
#pragma unroll
            for (int ps = 0; ps < kSelfPasses; ++ps) {
                const int blk = ps * 16 + (tid >> 4);
                const bool row_live = m < p.M;
                const float4 z4 = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                q80i8_pack8_stacked(row_live ? xr[ps][0] : z4, row_live ? xr[ps][1] : z4, m, kg, blk, blk < nblk, q80i8_planes);
            }
            __syncthreads();
        }
        // SELF: the planes of a step are read from LDS one step ahead of their use
        Q80I8Acts<STACK, TWO> lds_next;
        auto read_planes = [&](int s) {
            const uint8_t* base = q80i8_planes + (s < s1 ? s : s1 - 1) * kStackStepBytes;
#pragma unroll
            for (int i = 0; i < kPlanes; ++i) lds_next.pl[i] = *reinterpret_cast<const uint4*>(base + a_off + 1024 * i);
            lds_next.sv = *reinterpret_cast<const float*>(base + sv_off);
        };
        if constexpr (SELF) read_planes(s0);
        auto step = [&](auto set_c, int s) __attribute__((always_inline)) {
            constexpr int SET = decltype(set_c)::value;
            Q80I8Acts<STACK, TWO> from_lds;
            if constexpr (SELF) {
                from_lds = lds_next;
                read_planes(s + 1);
            }
            const Q80I8Acts<STACK, TWO>& act_now = SELF ? from_lds : acts[SET];
            // weights of this step -> the wave's LDS tile (waits for them and for everything older: this step's
            // activations; the younger steps stay in flight)
#pragma unroll
            for (int i = 0; i < kWLoads; ++i) {
                uint32_t* dst = reinterpret_cast<uint32_t*>(my_w + w_dst[i]);      // 4-byte aligned only
                dst[0] = wr[SET][i].x; dst[1] = wr[SET][i].y; dst[2] = wr[SET][i].z; dst[3] = wr[SET][i].w;
            }
            __builtin_amdgcn_sched_barrier(0);
            // the weight operands of block b + 1 are read from LDS ahead of block b's arithmetic
            WRaw cur[T], nxt[T];
#pragma unroll
            for (int t = 0; t < T; ++t) cur[t] = weight_read(t, 0);
            // unstacked forms: the step's requests are spread over the step instead of queueing at its end (a memory
            // instruction holds the wave's issue slot until its unit takes it) -- the weights of step s + D as soon as
            // this step's have left their registers, the planes of a block pair once its two blocks are done
            q80i8_unrolled(std::make_integer_sequence<int, kStepBlocks>(), [&](auto b_c) {
                constexpr int b = decltype(b_c)::value;
                if (b + 1 < kStepBlocks) {
#pragma unroll
                    for (int t = 0; t < T; ++t) nxt[t] = weight_read(t, b + 1);
                }
                WOperand w[T];
#pragma unroll
                for (int t = 0; t < T; ++t) w[t] = weight_operand(cur[t], b);
                compute_block(act_now, b_c, w);
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (kSpread) {
                    if (b & 1) issue_a_part(acts[SET], s + D, b >> 1);
                    __builtin_amdgcn_sched_barrier(0);
                }
#pragma unroll
                for (int t = 0; t < T; ++t) cur[t] = nxt[t];
            });
            if constexpr (!kSpread && !SELF) issue_a(acts[SET], s + D);
            issue_w(wr[SET], s + D);
            __builtin_amdgcn_sched_barrier(0);
        };
        // whole turns of the ring, then the steps that are left (each in its own register set)
        int s = s0;
        for (; s + D <= s1; s += D)
            q80i8_unrolled(std::make_integer_sequence<int, D>(),
                           [&](auto set_c) __attribute__((always_inline)) { step(set_c, s + decltype(set_c)::value); });
        q80i8_unrolled(std::make_integer_sequence<int, D - 1>(), [&](auto set_c) __attribute__((always_inline)) {
            if (s + decltype(set_c)::value < s1) step(set_c, s + decltype(set_c)::value);
        });
    }

    if (TWO) {
        // lanes g and g + 2 hold the (digit 1, digit 3) and the digit 2 part of rows 4 (g & 1) + r: both get the sum
#pragma unroll
        for (int t = 0; t < T; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[t][r] = m40_add_xor32(acc[t][r]);
    }
    if (STACK) {
        // lane (j, g) holds digit g of rows r: the three sums meet in the lanes g = 0
#pragma unroll
        for (int t = 0; t < T; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float d2 = __shfl(acc[t][r], j + 16, 64), d3 = __shfl(acc[t][r], j + 32, 64);
                acc[t][r] = g == 0 ? fmaf(acc[t][r], 16384.0f, fmaf(d2, 128.0f, d3)) : 0.0f;
            }
    }
    // lane (j, g) holds rows 4g + r of columns 16 t + j
    if (KSPLIT > 1) {
        // the K parts of a column group meet in part 0, added in part order
        if (kpart != 0) {
#pragma unroll
            for (int t = 0; t < T; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r) s_tile[wave][4 * g + r][16 * t + j] = acc[t][r];
        }
        __syncthreads();
        if (kpart == 0) {
#pragma unroll
            for (int w = 1; w < KSPLIT; ++w)
#pragma unroll
                for (int t = 0; t < T; ++t)
#pragma unroll
                    for (int r = 0; r < 4; ++r) acc[t][r] += s_tile[wave + w][4 * g + r][16 * t + j];
        }
    }
    if constexpr (MODE == 0) {
        const bool tile_live = kpart == 0 && ((blockIdx.x / KHALVES) * kGroups + group) * kCols < p.N;
#pragma unroll
        for (int t = 0; t < T; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int m = 4 * g + r, n = n0 + 16 * t + j;
                if (tile_live && m < p.M && n < p.N) {
                    if (KHALVES == 1) p.C[(size_t)m * p.N + n] = acc[t][r];
                    else atomicAdd(&p.C[(size_t)m * p.N + n], acc[t][r]);
                }
            }
    } else {
        if (p.zero)
            for (int i = (int)blockIdx.x * kThreads + tid; i < p.zero_count; i += (int)gridDim.x * kThreads) p.zero[i] = 0.0f;
        // SwiGLU of gate (lanes j < 8) and up (j >= 8, eight lanes on), then the digit pack of the workgroup's blocks
        constexpr int kHidden = kGroups * 8 * T, kHStride = kHidden + 1;
        __shared__ float hbuf[16 * kHStride];          // [16 rows][hidden columns of the workgroup]
#pragma unroll
        for (int t = 0; t < T; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float up = __shfl_xor(acc[t][r], 8, 64);
                const float gt = acc[t][r];
                const float h = gt / (1.0f + expf(-gt)) * up;
                if (kpart == 0 && j < 8) hbuf[(4 * g + r) * kHStride + group * 8 * T + 8 * t + j] = h;
            }
        __syncthreads();
        // the workgroup's hidden columns = blocks (kHidden / 32) blockIdx.x ... of the down projection's K
        for (int i = tid; i < 256 * (kHidden / 32); i += kThreads) {
            const int t = i >> 8, m = (i >> 4) & 15, pair = i & 15;
            q80i8_pack_pair(hbuf[m * kHStride + 32 * t + 2 * pair], hbuf[m * kHStride + 32 * t + 2 * pair + 1], m, pair,
                            STACK ? 0 : p.MP, p.out_pack, (int)blockIdx.x * (kHidden / 32) + t);
        }
    }
}

size_t pack_bytes(int K) { return (size_t)(K / (32 * kStepBlocks)) * kPlaneStepBytes; }

}  // namespace

// 2 <= M <= 16, K a multiple of 256 (whole steps), the context's packing buffer large enough; the matrix 16-byte
// aligned (its columns then are: 272 bytes per 256 k).
bool m40_q80_i8_supported(const M40llmCudaContext* ctx, uint32_t stream_kind, int M, int N, int K) {
    if (!ctx || stream_kind > 1) return false;
    if (M < 2 || M > 16 || N < 1 || K < 256 || K % 256 != 0) return false;
    return pack_bytes(K) <= ctx->scratch[stream_kind].gemm_pack_bytes;
}

static int rows_padded(int M) { return M <= 4 ? 0 : (M <= 8 ? 8 : 16); }   // 0: the stacked form, 8: two operands, 16: three planes

// the unstacked kernel in its three-plane (MP 16) or two-operand (MP 8) form
#define M40_Q80_UNSTACKED(MP, GRID, THREADS, ARGS, ...)                                                             \
    do {                                                                                                            \
        if ((MP) == 8) q80i8_gemm_kernel<__VA_ARGS__, true><<<(GRID), (THREADS), 0, stream>>>(ARGS);                \
        else q80i8_gemm_kernel<__VA_ARGS__, false><<<(GRID), (THREADS), 0, stream>>>(ARGS);                         \
    } while (0)

static void launch_gemm0(hipStream_t stream, const Q80I8Args& a) {
    const int tiles = (a.N + 15) / 16;
    const int nsteps = a.K / (32 * kStepBlocks);
    // few tiles: one tile per workgroup with K split over its waves, so that the grid still covers the CUs
    // (stacked form, N = 14336, K = 4096: 224 workgroups walking the whole K 16.6 us, 896 splitting it 23.7 us)
    const bool whole_k = tiles >= (a.MP == 0 ? 768 : 1024) || nsteps < 4;
    if (a.MP == 0) {
        // (N = 14336 as 448 workgroups of two tiles splitting K: 17.5 us against 16.7 us for the 224 walking the whole K)
        if (whole_k) q80i8_gemm_kernel<0, 1, true><<<(tiles + 3) / 4, 256, 0, stream>>>(a);
        else q80i8_gemm_kernel<0, 4, true><<<tiles, 256, 0, stream>>>(a);
        return;
    }
    // three-plane form: two column tiles per wave where the grid still covers the chip with them (measured at 16
    // rows: N = 14336, K = 4096 34.4 -> 22.8 us); else, with K long enough, eight waves share a tile's K (N = 4096,
    // K = 14336: 24.4 -> 23.5 us; two tiles per wave there would leave 128 workgroups: 31.5 us)
    const int pairs = (tiles + 1) / 2;
    if (whole_k) {
        if ((pairs + 3) / 4 >= 192) M40_Q80_UNSTACKED(a.MP, (pairs + 3) / 4, 256, a, 0, 1, false, 2, 4, 1, false, 0);
        else M40_Q80_UNSTACKED(a.MP, (tiles + 3) / 4, 256, a, 0, 1, false, 1, 4, 1, false, 0);
    } else {
        if (pairs > 256) M40_Q80_UNSTACKED(a.MP, pairs, 256, a, 0, 4, false, 2, 4, 1, false, 1);   // two workgroups per CU
        else if (pairs >= 192) M40_Q80_UNSTACKED(a.MP, pairs, 256, a, 0, 4, false, 2, 4, 1, false, 0);
        else if (nsteps >= 16) M40_Q80_UNSTACKED(a.MP, tiles, 512, a, 0, 8, false, 1, 8, 1, false, 0);
        else M40_Q80_UNSTACKED(a.MP, tiles, 256, a, 0, 4, false, 1, 4, 1, false, 0);
    }
}

int m40_launch_q80_i8(M40llmCudaContext* ctx, hipStream_t stream, uint32_t stream_kind, const float* A, const uint8_t* W,
                      float* C, int M, int N, int K) {
    if (!m40_q80_i8_supported(ctx, stream_kind, M, N, K)) return -2;
    if (!m40_aligned16(W)) return -2;
    (void)hipGetLastError();
    uint8_t* pack = static_cast<uint8_t*>(ctx->scratch[stream_kind].gemm_pack);
    const int MP = rows_padded(M);
    Q80I8Args a{};
    a.pack = pack; a.W0 = W; a.C = C; a.M = M; a.MP = MP; a.N = N; a.K = K;
    // few column tiles and a long K: tile pairs x two halves of K, added into a result the pack launch clears
    // (N = 4096, K = 14336: 17.5 -> 15.5 us at four rows, 23.7 -> 21.0 us at sixteen, pack launch aside)
    const char *c0 = reinterpret_cast<const char*>(C), *a0 = reinterpret_cast<const char*>(A);
    const bool apart = c0 + (size_t)M * N * 4 <= a0 || a0 + (size_t)M * K * 4 <= c0;
    const int pairs = (N + 31) / 32;
    if (apart && 2 * pairs >= 192 && 2 * pairs <= 1024 && K / (32 * kStepBlocks) >= 32) {
        q80i8_pack_kernel<<<K >> 5, 256, 0, stream>>>(A, M, MP, K, pack, C, M * N);
        if (MP == 0) q80i8_gemm_kernel<0, 4, true, 2, 4, 2><<<2 * pairs, 256, 0, stream>>>(a);
        else M40_Q80_UNSTACKED(MP, 2 * pairs, 256, a, 0, 4, false, 2, 4, 2, false, 0);
        return hipGetLastError() == hipSuccess ? 0 : -2;
    }
    q80i8_pack_kernel<<<K >> 5, 256, 0, stream>>>(A, M, MP, K, pack, nullptr, 0);
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
    if (!(m40_aligned16(wg) && m40_aligned16(wu) && m40_aligned16(wd))) return -2;
    (void)hipGetLastError();
    uint8_t* xp = static_cast<uint8_t*>(ctx->scratch[stream_kind].gemm_pack);
    uint8_t* hp = xp + x_bytes;
    const int MP = rows_padded(M);
    Q80I8Args a{};
    a.pack = xp; a.W0 = wg; a.W1 = wu; a.out_pack = hp; a.x = x; a.M = M; a.MP = MP; a.N = ffn; a.K = d_model;
    const bool two_tiles = ffn % 64 == 0 && ffn / 64 >= 192;
    // stacked form, K <= 4096: no pack launch, the gate + up workgroups pack the rows themselves into LDS (FFN 14336 at
    // four rows: 47.8 -> 46.9 us; with the earlier, twice as long digit arithmetic the launch lost what the pack launch cost)
    const bool self_pack = MP == 0 && two_tiles && d_model <= 16 * 32 * kStepBlocks && m40_aligned16(x);
    if (!self_pack) q80i8_pack_kernel<<<d_model >> 5, 256, 0, stream>>>(x, M, MP, d_model, xp, nullptr, 0);
    // down projection as column-tile pairs x two halves of K, added into a result the gate + up launch clears
    const bool out_apart = reinterpret_cast<const char*>(out) + (size_t)M * d_model * 4 <= reinterpret_cast<const char*>(x) ||
                           reinterpret_cast<const char*>(x) + (size_t)M * d_model * 4 <= reinterpret_cast<const char*>(out);
    // (FFN 14336 -> 4096: 49.6 -> 48.1 us at four rows, 64.2 -> 61.0 us at sixteen; with eight waves per workgroup 63.1 us)
    const int down_pairs = (d_model + 31) / 32;
    const bool halves = out_apart && 2 * down_pairs >= 192 && 2 * down_pairs <= 1024 && ffn / (32 * kStepBlocks) >= 32;
    if (halves) { a.zero = out; a.zero_count = M * d_model; }
    // two column tiles per wave where 192 workgroups and more remain: every activation plane fetched is used twice
    // (stacked form, FFN 14336: 52.9 -> 49.2 us; with three 32-column steps in flight instead of two 50.1 us)
    if (self_pack) {
        auto* kern = q80i8_gemm_kernel<1, 1, true, 2, 4, 1, true>;
        static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                                           hipFuncAttributeMaxDynamicSharedMemorySize, 16 * kStackStepBytes);
        if (attr != hipSuccess) return -2;
        kern<<<ffn / 64, 256, (size_t)(d_model / (32 * kStepBlocks)) * kStackStepBytes, stream>>>(a);
    } else if (MP == 0 && two_tiles) q80i8_gemm_kernel<1, 1, true, 2><<<ffn / 64, 256, 0, stream>>>(a);
    else if (MP == 0) q80i8_gemm_kernel<1, 1, true><<<ffn / 32, 256, 0, stream>>>(a);
    // (a workgroup of two column groups x two K halves, two waves per SIMD instead of one: measured, 64.5 -> 66 us)
    else if (ffn % 64 == 0 && ffn / 64 >= 192) M40_Q80_UNSTACKED(MP, ffn / 64, 256, a, 1, 1, false, 2, 4, 1, false, 0);
    else M40_Q80_UNSTACKED(MP, ffn / 32, 256, a, 1, 1, false, 1, 4, 1, false, 0);
    Q80I8Args b{};
    b.pack = hp; b.W0 = wd; b.C = out; b.M = M; b.MP = MP; b.N = d_model; b.K = ffn;
    if (halves) {
        const int pairs = (d_model + 31) / 32;
        if (MP == 0) q80i8_gemm_kernel<0, 4, true, 2, 4, 2><<<2 * pairs, 256, 0, stream>>>(b);
        else M40_Q80_UNSTACKED(MP, 2 * pairs, 256, b, 0, 4, false, 2, 4, 2, false, 0);
    } else {
        launch_gemm0(stream, b);
    }
    return hipGetLastError() == hipSuccess ? 0 : -2;
}
