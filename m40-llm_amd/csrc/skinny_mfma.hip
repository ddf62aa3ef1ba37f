// Skinny GEMM for the batched decode step on gfx950: C[M,N] = A[M,K] (f32) x W[N,K]^T with 1 <= M <= 16 rows
// per pass and W either f16 (GGUF order, K contiguous per output column) or q8_0 (34-byte blocks along K).
//
// The activations are split once per call into f16 hi + f16 lo fragments with a per-row power-of-two scale
// (pack kernel below); the product runs on v_mfma_f32_16x16x32_f16 with f32 accumulation.  One MFMA covers
// 32 consecutive k, which is exactly one q8_0 block, so the block scale multiplies the MFMA result.
//
// A workgroup is eight waves = eight 16-column tiles that walk the same range of K in steps of 256.  The
// activation fragments of a step (8 KB, or 16 KB above eight rows) are loaded once per workgroup into LDS and
// shared by the eight waves; weights are read once, straight from their GGUF bytes:
//   f16  : lane (column j, group g) loads its 16 bytes of k = 32 i + 8 g .. +7 per MFMA;
//   q8_0 : the 16 columns x 272 bytes of a step are copied with full 16-byte loads into a wave-private LDS
//          tile; each lane then reads the 8 quants of its (column, block, group) and turns them into f16 with
//          the 1024 + (q xor 0x80) construction (exact).
// Loads of step t+1 are in flight while step t is multiplied.  K is split over grid.y; slices write partial
// sums that a second kernel adds in slice order, so results never depend on timing.
#include "common.hpp"

namespace {

constexpr int kTileK = 256;                       // k per step
constexpr int kWavesPerGroup = 8;                 // 16-column tiles per workgroup
constexpr int kThreads = kWavesPerGroup * 64;
constexpr int kQ8TileBytes = 16 * 272;            // 16 columns x 8 blocks x 34 bytes

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));

// ---- activation packing -----------------------------------------------------------------------------------
// Fragment i (k = 32 i .. 32 i + 31) is 64 x 16 bytes: entry g*16 + row holds the eight halves k = 32 i + 8 g + 0..7
// of that row.  STACKED (M <= 8): rows 0-7 hold hi, rows 8-15 lo.  Otherwise two fragment sets: hi, then lo at
// +K/32*64 entries.  With `up`, the packed value is silu(A) * up (the SwiGLU of an FFN) instead of A.
__global__ __launch_bounds__(256) void pack_a_blocked_kernel(const float* __restrict__ A, const float* __restrict__ up,
                                                             int M, int K, int stacked, uint4* __restrict__ P,
                                                             float* __restrict__ row_scale) {
    __shared__ float wave_max[4];
    const int row = blockIdx.x;  // 0..7 (stacked) or 0..15
    const int tid = threadIdx.x;
    const bool live = row < M;
    auto value = [&](int k) -> float {
        const float a = A[(size_t)row * K + k];
        if (!up) return a;
        return a / (1.0f + expf(-a)) * up[(size_t)row * K + k];
    };
    float inv_scale = 1.0f, scale = 1.0f;
    if (live) {
        float mx = 0.0f;
        for (int k = tid; k < K; k += 256) mx = fmaxf(mx, fabsf(value(k)));
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
    const int frags = K >> 5;
    uint4* P_lo = P + (size_t)frags * 64;
    for (int f = tid; f < frags * 4; f += 256) {
        const int g = f & 3, i = f >> 2;
        const int k0 = 32 * i + 8 * g;
        uint32_t hi[4] = {0, 0, 0, 0}, lo[4] = {0, 0, 0, 0};
        if (live) {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float a = value(k0 + j) * inv_scale;
                const _Float16 h = static_cast<_Float16>(a);
                const _Float16 l = static_cast<_Float16>(a - static_cast<float>(h));
                hi[j >> 1] |= (uint32_t)__builtin_bit_cast(uint16_t, h) << (16 * (j & 1));
                lo[j >> 1] |= (uint32_t)__builtin_bit_cast(uint16_t, l) << (16 * (j & 1));
            }
        }
        const size_t base = (size_t)i * 64 + (size_t)g * 16;
        P[base + row] = make_uint4(hi[0], hi[1], hi[2], hi[3]);
        if (stacked) P[base + row + 8] = make_uint4(lo[0], lo[1], lo[2], lo[3]);
        else P_lo[base + row] = make_uint4(lo[0], lo[1], lo[2], lo[3]);
    }
}

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
    const uint4* P;            // packed activations
    const float* row_scale;
    const void* W[2];          // up to two weight matrices of the same shape (grid.z)
    float* C[2];               // their outputs [M][N]
    float* partial;            // [grid.z][S][16][N] when S > 1
    int M, N, K, S;
};

// FMT 0: f16 weights, 1: q8_0 weights.
template <int FMT, bool STACKED>
__global__ __launch_bounds__(kThreads) void skinny_mfma_kernel(SkinnyArgs p) {
    constexpr int kASets = STACKED ? 1 : 2;
    constexpr int kABufs = STACKED ? 2 : 1;                             // LDS budget: two sets are single-buffered
    __shared__ uint4 a_lds[kABufs][kASets][8 * 64];                     // activation fragments of a step
    __shared__ __attribute__((aligned(16))) uint8_t b_lds[FMT == 1 ? kWavesPerGroup * kQ8TileBytes : 16];

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int j = lane & 15, g = lane >> 4;
    const int ntiles = (p.N + 15) >> 4;
    int ntile = blockIdx.x * kWavesPerGroup + wave;
    const bool tile_live = ntile < ntiles;
    if (!tile_live) ntile = ntiles - 1;
    const int n0 = ntile * 16;
    const int KT = p.K / kTileK;
    const int kt0 = (int)(((long long)blockIdx.y * KT) / p.S), kt1 = (int)(((long long)(blockIdx.y + 1) * KT) / p.S);
    const int frags_total = p.K >> 5;
    const uint4* P_lo = p.P + (size_t)frags_total * 64;

    // ---- weight addressing
    const int col = n0 + j < p.N ? n0 + j : p.N - 1;
    const uint16_t* w16 = nullptr;
    const uint8_t* q_src[5] = {nullptr, nullptr, nullptr, nullptr, nullptr};
    int q_dst[5] = {0, 0, 0, 0, 0};
    uint8_t* my_b = b_lds + (FMT == 1 ? wave * kQ8TileBytes : 0);
    if (FMT == 0) {
        w16 = static_cast<const uint16_t*>(p.W[blockIdx.z]) + (size_t)col * p.K + 8 * g;
    } else {
        const size_t col_stride = (size_t)(p.K >> 5) * 34;
        const uint8_t* base = static_cast<const uint8_t*>(p.W[blockIdx.z]);
#pragma unroll
        for (int i = 0; i < 5; ++i) {
            const int q = i * 64 + lane;          // 16-byte piece of the 16 x 272-byte tile
            if (q < 272) {
                const int c = q / 17, piece = q % 17;
                const int cc = n0 + c < p.N ? n0 + c : p.N - 1;
                q_src[i] = base + (size_t)cc * col_stride + 16 * piece;
                q_dst[i] = c * 272 + 16 * piece;
            }
        }
    }

    uint4 ra[kASets];          // this thread's share of the activation fragments of a step
    uint4 rb[8];               // f16: the eight 16-byte weight loads of a step; q8_0: five tile pieces
    auto issue_loads = [&](int kt) {
        const size_t f0 = (size_t)kt * 8 * 64;
        ra[0] = p.P[f0 + tid];
        if (!STACKED) ra[1] = P_lo[f0 + tid];
        if (FMT == 0) {
#pragma unroll
            for (int i = 0; i < 8; ++i)
                rb[i] = m40_load_stream(reinterpret_cast<const uint4*>(w16 + (size_t)kt * kTileK + 32 * i));
        } else {
#pragma unroll
            for (int i = 0; i < 5; ++i)
                if (q_src[i]) rb[i] = m40_load_stream(reinterpret_cast<const uint4*>(q_src[i] + (size_t)kt * 272));
        }
    };

    m40_float4 acc = {0.f, 0.f, 0.f, 0.f};
    if (kt0 < kt1) issue_loads(kt0);
    for (int kt = kt0; kt < kt1; ++kt) {
        const int buf = kABufs == 2 ? ((kt - kt0) & 1) : 0;
        a_lds[buf][0][tid] = ra[0];
        if (!STACKED) a_lds[buf][1][tid] = ra[1];
        uint4 wb[8];
        if (FMT == 0) {
#pragma unroll
            for (int i = 0; i < 8; ++i) wb[i] = rb[i];
        } else {
#pragma unroll
            for (int i = 0; i < 5; ++i)
                if (q_src[i]) *reinterpret_cast<uint4*>(my_b + q_dst[i]) = rb[i];
        }
        __syncthreads();
        if (kt + 1 < kt1) issue_loads(kt + 1);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint4 a_hi = a_lds[buf][0][i * 64 + lane];
            if (FMT == 0) {
                acc = mfma16x16x32(a_hi, wb[i], acc);
                if (!STACKED) acc = mfma16x16x32(a_lds[buf][1][i * 64 + lane], wb[i], acc);
            } else {
                const uint8_t* blk = my_b + j * 272 + 34 * i;
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
                if (!STACKED) dblk = mfma16x16x32(a_lds[buf][1][i * 64 + lane], bq, dblk);
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[r] = fmaf(d, dblk[r], acc[r]);
            }
        }
        if (kABufs == 1) __syncthreads();   // the single buffer is rewritten by the next step
    }
    // lane (j, g) holds rows 4g + r of column j
    if (STACKED) {
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[r] += __shfl_xor(acc[r], 32, 64);  // hi rows + lo rows
    }
    if (!tile_live || n0 + j >= p.N) return;
    if (STACKED && g >= 2) return;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int row = 4 * g + r;
        if (p.S == 1) {
            if (row < p.M) p.C[blockIdx.z][(size_t)row * p.N + n0 + j] = acc[r] * p.row_scale[row];
        } else {
            p.partial[(((size_t)blockIdx.z * p.S + blockIdx.y) * 16 + row) * p.N + n0 + j] = acc[r];
        }
    }
}

// C[row][n] = row_scale[row] * sum over slices (ascending) of partial[z][slice][row][n]
__global__ __launch_bounds__(256) void skinny_reduce_kernel(SkinnyArgs p, int rows) {
    const int n = blockIdx.x * 256 + threadIdx.x;
    if (n >= p.N) return;
    const int z = blockIdx.z;
    for (int row = blockIdx.y; row < rows; row += gridDim.y) {
        float v = 0.0f;
        for (int s = 0; s < p.S; ++s) v += p.partial[(((size_t)z * p.S + s) * 16 + row) * p.N + n];
        p.C[z][(size_t)row * p.N + n] = v * p.row_scale[row];
    }
}

int pick_slices(int ntiles, int KT, int nmat, int num_cus) {
    const long long groups = (long long)((ntiles + kWavesPerGroup - 1) / kWavesPerGroup) * nmat;
    int s = 1;
    while (s < 16 && groups * s < 2LL * num_cus && KT / (s * 2) >= 1) s *= 2;
    return s > KT ? KT : s;
}

}  // namespace

bool m40_skinny_supported(const M40llmCudaContext* ctx, uint32_t stream_kind, int M, int N, int K, int fmt) {
    (void)M;
    if (K % kTileK != 0 || N <= 0) return false;
    if (fmt != 0 && fmt != 1) return false;
    const M40StreamScratch& sc = ctx->scratch[stream_kind];
    return (size_t)K * 64 + 256 <= sc.gemm_pack_bytes;
}

// up != nullptr: the activations are silu(A) * up.  W1/C1 may be null (one matrix).
int m40_launch_skinny(M40llmCudaContext* ctx, hipStream_t stream, uint32_t stream_kind, int fmt, const float* A,
                      const float* up, const void* W0, float* C0, const void* W1, float* C1, int M, int N, int K) {
    if (M <= 0 || N <= 0 || K <= 0) return -2;
    if (!m40_skinny_supported(ctx, stream_kind, M, N, K, fmt)) return -2;
    M40StreamScratch& sc = ctx->scratch[stream_kind];
    float* row_scale = static_cast<float*>(sc.gemm_pack);
    uint4* P = reinterpret_cast<uint4*>(static_cast<char*>(sc.gemm_pack) + 256);
    const int nmat = W1 ? 2 : 1;
    const int ntiles = (N + 15) >> 4;
    const int KT = K / kTileK;
    int S = pick_slices(ntiles, KT, nmat, ctx->num_cus);
    while (S > 1 && (size_t)nmat * S * 16 * N * sizeof(float) > sc.attn_partial_bytes) S >>= 1;
    (void)hipGetLastError();
    for (int r0 = 0; r0 < M; r0 += 16) {
        const int m = M - r0 < 16 ? M - r0 : 16;
        const bool stacked = m <= 8;
        pack_a_blocked_kernel<<<stacked ? 8 : 16, 256, 0, stream>>>(A + (size_t)r0 * K, up ? up + (size_t)r0 * K : nullptr,
                                                                    m, K, stacked ? 1 : 0, P, row_scale);
        SkinnyArgs a{};
        a.P = P; a.row_scale = row_scale;
        a.W[0] = W0; a.W[1] = W1;
        a.C[0] = C0 + (size_t)r0 * N; a.C[1] = C1 ? C1 + (size_t)r0 * N : nullptr;
        a.partial = static_cast<float*>(sc.attn_partial);
        a.M = m; a.N = N; a.K = K; a.S = S;
        dim3 grid((ntiles + kWavesPerGroup - 1) / kWavesPerGroup, S, nmat);
        if (fmt == 0) {
            if (stacked) skinny_mfma_kernel<0, true><<<grid, kThreads, 0, stream>>>(a);
            else skinny_mfma_kernel<0, false><<<grid, kThreads, 0, stream>>>(a);
        } else {
            if (stacked) skinny_mfma_kernel<1, true><<<grid, kThreads, 0, stream>>>(a);
            else skinny_mfma_kernel<1, false><<<grid, kThreads, 0, stream>>>(a);
        }
        if (S > 1) {
            dim3 rgrid((N + 255) / 256, m < 4 ? m : 4, nmat);
            skinny_reduce_kernel<<<rgrid, 256, 0, stream>>>(a, m);
        }
    }
    return hipGetLastError() == hipSuccess ? 0 : -2;
}
