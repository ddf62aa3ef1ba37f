// Many-row GEMM for prefill: C[M,N] f32 = A[M,K] f32 x B (f16, GGUF order [N][K]), f32 accumulation, on the
// matrix cores.  Same contract as the reference's gemm_f32xf16_gguf_f32 (cuda/kernels.cu:5037-5052); used when M is
// beyond what the skinny kernels serve in one pass, where they would stream the weights once per 16 rows.
//
// Tiling: a workgroup of 4 waves owns a 128 x 128 tile of C and walks K in steps of 32.  Per step the 128 x 32 block
// of A is read as f32, split exactly into an f16 high part and an f16 low part (a = hi + lo up to 2^-22 relative),
// and written to LDS with the 128 x 32 block of B; each wave then computes its 64 x 64 quarter with
// v_mfma_f32_16x16x32_f16, once with the high and once with the low part, so the products carry the f32 activations'
// precision.  Global loads for step k+1 are issued before the arithmetic of step k and land in the other LDS buffer
// after it: one barrier per step.
#include "common.hpp"

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef _Float16 half4v __attribute__((ext_vector_type(4)));

constexpr int kBM = 128, kBN = 128, kBK = 32;
constexpr int kStride = kBK + 8;                 // halves per LDS row: 80 B, conflict-free 16-byte fragment reads
constexpr int kTileHalves = kBM * kStride;       // one 128 x 32 operand block
constexpr int kBufHalves = 3 * kTileHalves;      // A high, A low, B
constexpr int kThreads = 256;

struct StepRegs {
    float4 a[4];   // 16 consecutive f32 of one A row
    uint4 b[2];    // 16 consecutive f16 of one B column
};

__device__ __forceinline__ void split16(const float4 (&a)[4], half8 (&hi)[2], half8 (&lo)[2]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float x[4] = {a[i].x, a[i].y, a[i].z, a[i].w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            // clamped to the f16 range: a value beyond +-65504 keeps its sign and loses precision instead of becoming
            // an infinity (and its low part a NaN)
            const float xc = fminf(fmaxf(x[j], -65504.0f), 65504.0f);
            const _Float16 h = static_cast<_Float16>(xc);
            const _Float16 l = static_cast<_Float16>(fminf(fmaxf(x[j] - static_cast<float>(h), -65504.0f), 65504.0f));
            hi[i >> 1][(i & 1) * 4 + j] = h;
            lo[i >> 1][(i & 1) * 4 + j] = l;
        }
    }
}

__global__ __launch_bounds__(kThreads, 2) void gemm_tiled_f32xf16_gguf_kernel(const float* __restrict__ A,
                                                                              const uint16_t* __restrict__ B,
                                                                              float* __restrict__ C, int M, int N, int K,
                                                                              int tiles_n) {
    extern __shared__ __align__(16) _Float16 lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int tile_m = blockIdx.x / tiles_n, tile_n = blockIdx.x % tiles_n;
    const int m0 = tile_m * kBM, n0 = tile_n * kBN;
    // loader role: row (or column) tid / 2, k half tid % 2
    const int lrow = tid >> 1, lhalf = tid & 1;
    const int a_row = m0 + lrow < M ? m0 + lrow : M - 1;     // clamped: rows beyond M are computed and never stored
    const int b_col = n0 + lrow < N ? n0 + lrow : N - 1;
    const float* a_src = A + (size_t)a_row * K + lhalf * 16;
    const uint16_t* b_src = B + (size_t)b_col * K + lhalf * 16;
    const int steps = K / kBK;

    auto issue = [&](StepRegs& r, int step) {
        const float4* ap = reinterpret_cast<const float4*>(a_src + (size_t)step * kBK);
        const uint4* bp = reinterpret_cast<const uint4*>(b_src + (size_t)step * kBK);
#pragma unroll
        for (int i = 0; i < 4; ++i) r.a[i] = ap[i];
        r.b[0] = bp[0];
        r.b[1] = bp[1];
    };
    auto to_lds = [&](const StepRegs& r, int buf) {
        _Float16* base = lds + buf * kBufHalves;
        half8 hi[2], lo[2];
        split16(r.a, hi, lo);
        _Float16* ah = base + lrow * kStride + lhalf * 16;
        _Float16* al = ah + kTileHalves;
        _Float16* bb = ah + 2 * kTileHalves;
        *reinterpret_cast<half8*>(ah) = hi[0];
        *reinterpret_cast<half8*>(ah + 8) = hi[1];
        *reinterpret_cast<half8*>(al) = lo[0];
        *reinterpret_cast<half8*>(al + 8) = lo[1];
        typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
        *reinterpret_cast<u32x4*>(bb) = u32x4{r.b[0].x, r.b[0].y, r.b[0].z, r.b[0].w};
        *reinterpret_cast<u32x4*>(bb + 8) = u32x4{r.b[1].x, r.b[1].y, r.b[1].z, r.b[1].w};
    };

    floatx4 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

    const int wm = wave >> 1, wn = wave & 1;
    const int frag_row = lane & 15, frag_k = (lane >> 4) * 8;
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
#pragma unroll
            for (int nt = 0; nt < 4; ++nt) {
                acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(hi, bf[nt], acc[mt][nt], 0, 0, 0);
                acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(lo, bf[nt], acc[mt][nt], 0, 0, 0);
            }
        }
    };

    StepRegs regs;
    issue(regs, 0);
    to_lds(regs, 0);
    __syncthreads();
    for (int s = 0; s < steps; ++s) {
        const int next = s + 1 < steps ? s + 1 : s;     // the last step reloads its own block: no branch around loads
        issue(regs, next);
        compute(s & 1);
        to_lds(regs, (s + 1) & 1);
        __syncthreads();
    }

    // D fragment: lane holds rows 4 * (lane / 16) + r, column lane % 16 of each 16 x 16 tile
    const int out_col = lane & 15, out_row = (lane >> 4) * 4;
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int row = m0 + wm * 64 + mt * 16 + out_row + r;
            if (row >= M) continue;
#pragma unroll
            for (int nt = 0; nt < 4; ++nt) {
                const int col = n0 + wn * 64 + nt * 16 + out_col;
                if (col < N) C[(size_t)row * N + col] = acc[mt][nt][r];
            }
        }
    }
}

}  // namespace

bool m40_gemm_tiled_supported(const void* A, const void* B, int M, int N, int K) {
    return M > 32 && N >= 16 && K >= kBK && K % kBK == 0 && m40_aligned16(A) && m40_aligned16(B) &&
           ((long long)((M + kBM - 1) / kBM) * ((N + kBN - 1) / kBN)) <= 0x7fffffffll;
}

int m40_launch_gemm_tiled(hipStream_t stream, const float* A, const uint16_t* B, float* C, int M, int N, int K) {
    if (!m40_gemm_tiled_supported(A, B, M, N, K)) return -2;
    static bool attr_set = false;
    constexpr size_t lds_bytes = 2 * kBufHalves * sizeof(_Float16);   // 61440
    if (!attr_set) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_tiled_f32xf16_gguf_kernel),
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes) != hipSuccess)
            return -2;
        attr_set = true;
    }
    const int tiles_m = (M + kBM - 1) / kBM, tiles_n = (N + kBN - 1) / kBN;
    (void)hipGetLastError();
    gemm_tiled_f32xf16_gguf_kernel<<<tiles_m * tiles_n, kThreads, lds_bytes, stream>>>(A, B, C, M, N, K, tiles_n);
    return hipGetLastError() == hipSuccess ? 0 : -2;
}
