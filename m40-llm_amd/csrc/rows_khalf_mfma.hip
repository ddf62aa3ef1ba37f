// Row-batched projection with a long K and few output columns -- the down projection of a batched decode step -- in
// one launch: out[rows][N] += residual + a[rows][K] . W^T for up to eight activation rows, f16 GGUF weights [N][K].
//
// A workgroup owns one 16-column tile and one half of K; its eight waves split that half into contiguous runs of
// MFMA k-steps (32 k each), add their sums in wave order through LDS, and the workgroup ADDS its 16 x rows values
// into `out`, which an earlier launch on the stream has cleared.  Two terms onto zero -- (residual + first half) and
// (second half) -- are the same f32 in either order of arrival, so the result does not depend on timing, and no
// second launch is needed to put K slices together.
//
// Nothing is shared between the waves inside the K loop, so nothing waits for a barrier there.  A wave converts
// its own activations: lane (k group kg, operand row r16) loads four f32 of row r16 & 7 -- the first or second half
// of the 8-k chunk kg of a k-step, by r16 >> 3 -- splits them into f16 hi + lo under a power-of-two scale taken from
// the row's largest value of the batch, and trades two registers with its partner lane (r16 ^ 8) so that operand
// rows 0-7 hold the hi parts and rows 8-15 the lo parts of all eight k: one matrix instruction per k-step covers
// both.  The weights of a batch of four k-steps come as whole runs (an instruction of a wave reads 256 contiguous
// bytes of each of four columns), pass through a wave-private LDS tile and are read back in B-operand order.
//
// What the launch time follows, measured with timestamps inside the kernel (2048 columns, K = 11008, eight rows):
//  * Requests in flight: two batches per wave = 64 KB of weights and 64 KB of activations per CU.  More is slower
//    (weights alone: 10.4 us with 64 KB per CU in flight, 12.1 us with 128 KB, 19.8 us with everything requested up
//    front): the first data then reaches some waves only after 10 us, and the launch ends with the unluckiest wave.
//  * No register may spill: a reload is a vector memory operation and returns in issue order behind every weight
//    request in flight.  Addresses are a uniform base (scalar registers) plus one per-lane 32-bit offset per batch.
//  * The activations are as many bytes per workgroup as the weights (each workgroup needs its half of all rows) and
//    come from L2 / the memory-side cache: they add 2-3 us to the weights' 10-11 us; they are requested ahead of the
//    weights of the same batch (loads return in issue order), never under a branch.
//
// Reference semantics: f32 x f16 GGUF product cuda/kernels.cu:5037-5052; the residual add of the batched layer
// src/infer/forward.rs:2095-2136.
#include "common.hpp"

#include <type_traits>

namespace {

constexpr int kWaves = 8;
constexpr int kThreads = 64 * kWaves;
constexpr int kBatchSteps = 4;                        // k-steps (32 k) per batch: 256 bytes of every column
constexpr int kRunLanes = kBatchSteps * 4;             // lanes that cover a column's 64 bytes x steps of a batch
constexpr int kColsPerLoad = 64 / kRunLanes;
constexpr int kWLoads = 16 / kColsPerLoad;
constexpr int kStageRow = kBatchSteps * 64 + 16;      // LDS bytes per column of a batch: +16 spreads the columns over the banks
constexpr int kStageBytes = 16 * kStageRow;
constexpr int kRedBytes = kWaves * 4 * 64 * 4;
constexpr int kDynamicLds = kWaves * kStageBytes + kRedBytes;

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

struct KHalfArgs {
    const float* A;            // [rows][K]
    const uint16_t* W;         // [N][K] f16
    const float* residual;     // [rows][N] or null
    float* out;                // [rows][N], holds zeros when the launch starts
    int rows, N, K;
};

// value of the partner lane (lane ^ 8) within a row of 16 lanes
__device__ __forceinline__ uint32_t from_partner8(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x128 /* row_ror:8 */, 0xf, 0xf, false);
}

__global__ __launch_bounds__(kThreads, 1) void rows_khalf_kernel(KHalfArgs p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t khalf_lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    uint8_t* stage = khalf_lds + wave * kStageBytes;
    float* red = reinterpret_cast<float*>(khalf_lds + kWaves * kStageBytes);      // [wave][r][lane]
    const int j = lane & 15, g = lane >> 4;
    const int tile = (int)blockIdx.x >> 1, half = (int)blockIdx.x & 1;
    const int n0 = tile * 16;
    // The element this thread adds into `out` at the end (threads below 128: row tid / 16, column tid % 16), and its
    // residual value, requested ahead of everything else: one unconditional load from a clamped address -- at the end it
    // would be a round trip to memory with the whole workgroup waiting.
    const int e_row = (tid >> 4) & 7, e_j = tid & 15;
    const size_t e_off = (size_t)(e_row < p.rows ? e_row : 0) * p.N + (n0 + e_j < p.N ? n0 + e_j : p.N - 1);
    const float e_res = *(p.residual ? p.residual + e_off : p.A);
    __builtin_amdgcn_sched_barrier(0);

    // this wave's k-steps [ws0, ws1)
    const int KS = p.K >> 5;
    const int hs0 = (int)((long long)KS * half / 2), hs1 = (int)((long long)KS * (half + 1) / 2);
    const int ws0 = hs0 + (int)((long long)(hs1 - hs0) * wave / kWaves);
    const int ws1 = hs0 + (int)((long long)(hs1 - hs0) * (wave + 1) / kWaves);
    const int nb = (ws1 - ws0 + kBatchSteps - 1) / kBatchSteps;

    // activations: lane (kg = g, r16 = j) -> row j & 7, elements 8 kg + 4 (j >> 3) .. + 3 of a k-step
    const int row = j & 7, part = j >> 3;
    const bool row_live = row < p.rows;
    const uint32_t a_voff = (uint32_t)(((size_t)(row_live ? row : 0) * p.K + 8 * g + 4 * part) * 4);   // bytes from a k-step's start in row 0
    // weights: instruction li of a batch covers kColsPerLoad columns, lane -> (column, 16-byte piece of its run)
    const int w_col = lane / kRunLanes, w_piece = lane % kRunLanes;
    const int w_step = w_piece >> 2;                                  // k-step of the piece inside its batch
    uint8_t* w_dst = stage + w_col * kStageRow + 16 * w_piece;       // + kColsPerLoad li columns
    uint4 ar[2][kBatchSteps];                              // activations of a batch: as loaded (four f32), then as A operands
    uint4 wr[2][kWLoads];
    // k-steps past the wave's run repeat its last one (no load under a branch); their activations count as zero
    auto issue_a = [&](uint4 (&a)[kBatchSteps], int s0) {
#pragma unroll
        for (int i = 0; i < kBatchSteps; ++i) {
            const int s = s0 + i < ws1 ? s0 + i : ws1 - 1;
            a[i] = *reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(p.A + (size_t)s * 32) + a_voff);
        }
        __builtin_amdgcn_sched_barrier(0);
    };
    auto issue_w = [&](uint4 (&w)[kWLoads], int s0) {
        const int live = ws1 - s0;
        const int st = w_step < live ? w_step : (live > 0 ? live - 1 : 0);
        const uint32_t voff = (uint32_t)(((size_t)w_col * p.K + 32 * st + 8 * (lane & 3)) * 2);
        const int sb = s0 < ws1 ? s0 : ws1 - 1;
#pragma unroll
        for (int li = 0; li < kWLoads; ++li) {
            w[li] = *reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(p.W + (size_t)(n0 + kColsPerLoad * li) * p.K + (size_t)sb * 32) + voff);
        }
        __builtin_amdgcn_sched_barrier(0);
    };
    m40_float4 acc = {0.f, 0.f, 0.f, 0.f};
    auto batch = [&](uint4 (&aop)[kBatchSteps], uint4 (&w)[kWLoads], auto prefetch_c, int b) {
        const int s0 = ws0 + kBatchSteps * b;
        const int live_steps = ws1 - s0;
        float mx = 0.0f;
#pragma unroll
        for (int i = 0; i < kBatchSteps; ++i) {
            const float4 a = __builtin_bit_cast(float4, aop[i]);
            mx = fmaxf(mx, fmaxf(fmaxf(fabsf(a.x), fabsf(a.y)), fmaxf(fabsf(a.z), fabsf(a.w))));
        }
        mx = fmaxf(mx, __builtin_bit_cast(float, from_partner8(__builtin_bit_cast(uint32_t, mx))));
        mx = m40_max_xor16(mx);
        mx = m40_max_xor32(mx);
        float scale = 1.0f, inv_scale = 1.0f;
        if (mx > 0.0f && mx < INFINITY) {
            int ex;
            (void)frexpf(mx, &ex);        // mx = f * 2^ex, f in [0.5, 1)
            ex -= 11;                     // scaled maximum in [2^10, 2^11)
            ex = ex < -100 ? -100 : (ex > 100 ? 100 : ex);
            scale = ldexpf(1.0f, ex);
            inv_scale = ldexpf(1.0f, -ex);
        }
        if (!row_live) inv_scale = 0.0f;
#pragma unroll
        for (int i = 0; i < kBatchSteps; ++i) {
            const float4 a = __builtin_bit_cast(float4, aop[i]);
            const float inv = i < live_steps ? inv_scale : 0.0f;
            const f32x2 s01 = {a.x * inv, a.y * inv}, s23 = {a.z * inv, a.w * inv};
            const f16x2 h01 = __builtin_convertvector(s01, f16x2), h23 = __builtin_convertvector(s23, f16x2);
            const f16x2 l01 = __builtin_convertvector(s01 - __builtin_convertvector(h01, f32x2), f16x2);
            const f16x2 l23 = __builtin_convertvector(s23 - __builtin_convertvector(h23, f32x2), f16x2);
            const uint32_t h0 = __builtin_bit_cast(uint32_t, h01), h1 = __builtin_bit_cast(uint32_t, h23);
            const uint32_t l0 = __builtin_bit_cast(uint32_t, l01), l1 = __builtin_bit_cast(uint32_t, l23);
            const uint32_t r0 = from_partner8(part ? h0 : l0), r1 = from_partner8(part ? h1 : l1);
            aop[i] = part ? make_uint4(r0, r1, l0, l1) : make_uint4(h0, h1, r0, r1);
        }
#pragma unroll
        for (int li = 0; li < kWLoads; ++li)
            *reinterpret_cast<u32x4*>(w_dst + kColsPerLoad * li * kStageRow) = u32x4{w[li].x, w[li].y, w[li].z, w[li].w};
        __builtin_amdgcn_wave_barrier();
        m40_float4 tacc = {0.f, 0.f, 0.f, 0.f};
        uint4 bw[kBatchSteps];
#pragma unroll
        for (int i = 0; i < kBatchSteps; ++i) bw[i] = *reinterpret_cast<const uint4*>(stage + j * kStageRow + 64 * i + 16 * g);
#pragma unroll
        for (int i = 0; i < kBatchSteps; ++i)
            tacc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(m40_half8, aop[i]), __builtin_bit_cast(m40_half8, bw[i]), tacc, 0, 0, 0);
        __builtin_amdgcn_wave_barrier();
        if (decltype(prefetch_c)::value) { issue_a(aop, s0 + 2 * kBatchSteps); issue_w(w, s0 + 2 * kBatchSteps); }
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[r] = fmaf(__shfl(scale, 4 * (g & 1) + r, 64), tacc[r], acc[r]);
    };
    if (nb > 0) {
        const std::integral_constant<bool, true> yes;
        const std::integral_constant<bool, false> no;
        issue_a(ar[0], ws0); issue_w(wr[0], ws0);
        issue_a(ar[1], ws0 + kBatchSteps); issue_w(wr[1], ws0 + kBatchSteps);
        int b = 0;
        for (; b + 3 < nb; b += 2) {                  // both batches of a pair have a batch two ahead
            batch(ar[0], wr[0], yes, b);
            batch(ar[1], wr[1], yes, b + 1);
        }
        const int rem = nb - b;                       // 1, 2 or 3
        if (rem == 3) {
            batch(ar[0], wr[0], yes, b);
            batch(ar[1], wr[1], no, b + 1);
            batch(ar[0], wr[0], no, b + 2);
        } else if (rem == 2) {
            batch(ar[0], wr[0], no, b);
            batch(ar[1], wr[1], no, b + 1);
        } else {
            batch(ar[0], wr[0], no, b);
        }
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        acc[r] = m40_add_xor32(acc[r]);          // hi rows (g 0, 1) + lo rows (g 2, 3)
        red[(wave * 4 + r) * 64 + lane] = acc[r];
    }
    __syncthreads();
    // thread t < 128: element (row t / 16, column t % 16), the waves' sums in wave order
    if (tid < 128) {
        const int e_lane = 16 * (e_row >> 2) + e_j, e_r = e_row & 3;
        float v = red[e_r * 64 + e_lane];
#pragma unroll
        for (int w = 1; w < kWaves; ++w) v += red[(w * 4 + e_r) * 64 + e_lane];
        const int col = n0 + e_j;
        if (e_row < p.rows && col < p.N) {
            if (half == 0 && p.residual) v = e_res + v;
            atomicAdd(p.out + (size_t)e_row * p.N + col, v);
        }
    }
}

__global__ __launch_bounds__(256) void zero_f32_kernel(float* dst, size_t n) {
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) dst[i] = 0.0f;
}

}  // namespace

// Where the one-launch form pays: enough tiles x halves to cover the CUs with workgroups of eight waves, and a K long
// enough that every wave has at least one full batch
bool m40_rows_khalf_supported(const M40llmCudaContext* ctx, int rows, int N, int K) {
    if (rows < 1 || rows > 8 || N < 16 || N % 16 != 0 || K < 32 || K % 32 != 0) return false;
    const int tiles = (N + 15) / 16;
    return 2 * tiles >= ctx->num_cus / 2 && 2 * tiles <= 4 * ctx->num_cus && K / 32 >= 2 * kWaves * 8;
}

int m40_rows_khalf_residual(M40llmCudaContext* ctx, hipStream_t stream, const float* a, const uint16_t* W,
                            const float* residual, float* out_zeroed, int rows, int N, int K) {
    if (!m40_rows_khalf_supported(ctx, rows, N, K) || !m40_aligned16(a) || !m40_aligned16(W)) return -6;
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(rows_khalf_kernel),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, kDynamicLds);
    if (attr != hipSuccess) return -7;
    KHalfArgs p{a, W, residual, out_zeroed, rows, N, K};
    rows_khalf_kernel<<<2 * ((N + 15) / 16), kThreads, kDynamicLds, stream>>>(p);
    return hipGetLastError() == hipSuccess ? 0 : -7;
}

int m40_zero_f32(hipStream_t stream, float* dst, size_t n) {
    if (n == 0) return 0;
    const size_t groups = (n + 255) / 256;
    zero_f32_kernel<<<(unsigned)(groups < 1024 ? groups : 1024), 256, 0, stream>>>(dst, n);
    return hipGetLastError() == hipSuccess ? 0 : -7;
}
