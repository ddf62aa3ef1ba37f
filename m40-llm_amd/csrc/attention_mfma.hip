// Last-token GQA attention over long dense f16 KV ranges on the matrix cores (gfx950).
//
// At long contexts the per-token arithmetic of the vector-ALU kernel (one FMA per K element and q head, plus
// cross-lane sums) costs more issue slots than the HBM stream leaves room for.  Here both products run on
// v_mfma_f32_16x16x32_f16:
//   scores  S[h][t] = sum_d q[h][d] K[t][d]:  A = q (16 rows = up to 8 q heads x {hi, lo} f16 split), B = K rows read
//           straight from the cache (a lane's 16 bytes are 8 consecutive d of its token);
//   output  O[h][d] = sum_t P[h][t] V[t][d]:  A = softmax weights (hi/lo split, re-laid out through a 1 KB LDS tile),
//           B = V, staged row-major in LDS by 16-byte global loads and read back one token column at a time.
// A workgroup is four waves on one kv head and one chunk of tokens; a wave walks 32-token tiles with a running
// maximum (the rows of one head live in one 16-lane row, so the softmax state never leaves that row), the four
// waves are merged through LDS, and chunks are merged by the same second kernel as the vector-ALU path.
//
// Reference semantics: cuda/kernels.cu:1367-1655 (three-pass softmax per q head, kv head = qh / group, scale
// literals 0.125f / 0.08838834764831845f); the running-maximum form is algebraically the same softmax.
#include "attention_params.hpp"

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = 4;
constexpr int kTile = 32;                 // tokens per wave step

__device__ __forceinline__ m40_float4 mfma16x16x32(const uint4& a, const uint4& b, m40_float4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(m40_half8, a),
                                                  __builtin_bit_cast(m40_half8, b), c, 0, 0, 0);
}
__device__ __forceinline__ float max16(float x) {   // over rows of 16 lanes
    x = fmaxf(x, m40_dpp_f<M40_DPP_XOR1>(x));
    x = fmaxf(x, m40_dpp_f<M40_DPP_XOR2>(x));
    x = fmaxf(x, m40_dpp_f<M40_DPP_HALF_MIRROR>(x));
    x = fmaxf(x, m40_dpp_f<M40_DPP_MIRROR>(x));
    return x;
}
__device__ __forceinline__ uint16_t f16_bits(float x) { return __builtin_bit_cast(uint16_t, static_cast<_Float16>(x)); }

template <int HD>
__global__ __launch_bounds__(kThreads, 2) void attn_mfma_kernel(AttnParams p) {
    constexpr int KS = HD / 32;            // MFMA k-steps of a score tile
    constexpr int DT = HD / 16;            // 16-column output tiles
    constexpr int RS = HD * 2 + 8;         // LDS bytes per V row (8-byte aligned, spreads the row groups over the banks)
    constexpr int PIECES = HD / 8;         // 16-byte pieces per row
    __shared__ __attribute__((aligned(16))) uint8_t v_lds[kWaves][kTile * RS];
    __shared__ __attribute__((aligned(16))) uint16_t p_lds[kWaves][16][40];      // rows of 80 bytes
    __shared__ float m_s[kWaves][8], l_s[kWaves][8];
    __shared__ float o_s[kWaves][8][HD];

    const uint32_t b = blockIdx.z;
    const uint32_t seq_id = p.seq_ids_dev ? p.seq_ids_dev[b] : p.seq_id;
    const uint32_t len = p.seq_lens_dev ? p.seq_lens_dev[b] + p.len_bias : p.seq_len;
    if (len == 0 || len > p.max_seq_len) return;
    if (p.max_batch != 0 && seq_id >= p.max_batch) return;
    const uint32_t t0 = (p.window != 0 && len > p.window) ? len - p.window : 0;
    if (len - t0 > p.span_limit) return;      // longer than the launch was sized for: the row is skipped
    const uint32_t cbeg = t0 + blockIdx.y * p.chunk;
    if (cbeg >= len) return;
    const uint32_t cend = cbeg + p.chunk < len ? cbeg + p.chunk : len;
    const uint32_t ntok = cend - cbeg;

    const uint32_t kvh = blockIdx.x / p.subgroups, sub = blockIdx.x % p.subgroups;
    const uint32_t group = p.q_heads / p.kv_heads;
    const uint32_t qh0 = kvh * group + sub * 8u;
    const uint32_t gcount = (sub * 8u + 8u <= group) ? 8u : group - sub * 8u;

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int c16 = lane & 15, g = lane >> 4;
    const size_t row_stride = (size_t)p.kv_heads * HD;
    const uint16_t* Kb = p.K + ((size_t)seq_id * p.max_seq_len) * row_stride + (size_t)kvh * HD;
    const uint16_t* Vb = p.V + ((size_t)seq_id * p.max_seq_len) * row_stride + (size_t)kvh * HD;
    const float* Qb = p.Q + ((size_t)b * p.q_heads + qh0) * HD;      // gcount heads, contiguous

    // ---- weight loads of the first tile go out before anything else ------------------------------------
    uint4 kreg[2][KS], vreg[DT];
    const int my_tiles_begin = wave;
    const int ntiles = (int)((ntok + kTile - 1) / kTile);
    auto issue = [&](int tile) {
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
            uint32_t t = cbeg + (uint32_t)(tile * kTile + 16 * hf + c16);
            t = t < cend ? t : cend - 1u;
#pragma unroll
            for (int i = 0; i < KS; ++i)
                kreg[hf][i] = *reinterpret_cast<const uint4*>(Kb + (size_t)t * row_stride + 32 * i + 8 * g);
        }
#pragma unroll
        for (int k = 0; k < DT; ++k) {
            const int q = k * 64 + lane;
            uint32_t t = cbeg + (uint32_t)(tile * kTile + q / PIECES);
            t = t < cend ? t : cend - 1u;
            vreg[k] = *reinterpret_cast<const uint4*>(Vb + (size_t)t * row_stride + 8 * (q % PIECES));
        }
    };
    if (my_tiles_begin < ntiles) issue(my_tiles_begin);

    // ---- q fragments: power-of-two scaled, split into f16 hi + lo -----------------------------------------
    // A-operand row rho = c16: head 2*(rho/4) + (rho%4)/2, part rho&1 (0 hi, 1 lo).  Every wave holds each q value
    // of the group (twice: hi and lo lanes), so the largest magnitude needs no exchange between waves.  All loads
    // go out together, behind the first tile's.
    const uint32_t qhead = 2u * (uint32_t)(c16 >> 2) + (uint32_t)((c16 & 3) >> 1);
    const bool q_live = qhead < gcount;
    float qv[KS][8];
    {
        const float* qp = Qb + (size_t)(q_live ? qhead : 0u) * HD + 8 * g;
#pragma unroll
        for (int i = 0; i < KS; ++i) {
            const float4 x = *reinterpret_cast<const float4*>(qp + 32 * i);
            const float4 y = *reinterpret_cast<const float4*>(qp + 32 * i + 4);
            qv[i][0] = x.x; qv[i][1] = x.y; qv[i][2] = x.z; qv[i][3] = x.w;
            qv[i][4] = y.x; qv[i][5] = y.y; qv[i][6] = y.z; qv[i][7] = y.w;
        }
    }
    float qmax = 0.0f;
#pragma unroll
    for (int i = 0; i < KS; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) qmax = fmaxf(qmax, q_live ? fabsf(qv[i][j]) : 0.0f);
    qmax = m40_max64(qmax);
    float q_inv = 1.0f, q_scale = 1.0f;
    if (qmax > 0.0f && qmax < INFINITY) {
        int e;
        (void)frexpf(qmax, &e);
        e -= 11;
        e = e < -100 ? -100 : (e > 100 ? 100 : e);
        q_scale = ldexpf(1.0f, e);
        q_inv = ldexpf(1.0f, -e);
    }
    const float score_scale = (HD == 64 ? 0.125f : 0.08838834764831845f) * q_scale;
    uint4 qf[KS];
    {
        const bool lo_part = (c16 & 1) != 0;
#pragma unroll
        for (int i = 0; i < KS; ++i) {
            uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float a = qv[i][j] * q_inv;
                const _Float16 hi = static_cast<_Float16>(a);
                const _Float16 v = lo_part ? static_cast<_Float16>(a - static_cast<float>(hi)) : hi;
                w[j >> 1] |= (uint32_t)__builtin_bit_cast(uint16_t, v) << (16 * (j & 1));
            }
            qf[i] = q_live ? make_uint4(w[0], w[1], w[2], w[3]) : make_uint4(0, 0, 0, 0);
        }
    }

    // ---- token tiles ------------------------------------------------------------------------------------------------
    float m0 = -INFINITY, m1 = -INFINITY;      // running maxima of heads 2g, 2g+1 (equal across the 16-lane row)
    float l0 = 0.0f, l1 = 0.0f;                // this lane's share of the running sums
    m40_float4 O[DT];
#pragma unroll
    for (int d = 0; d < DT; ++d) O[d] = m40_float4{0.f, 0.f, 0.f, 0.f};
    uint8_t* my_v = v_lds[wave];

    for (int tile = my_tiles_begin; tile < ntiles; tile += kWaves) {
        // V tile -> LDS (row-major, two 8-byte stores per piece)
#pragma unroll
        for (int k = 0; k < DT; ++k) {
            const int q = k * 64 + lane;
            uint2* dst = reinterpret_cast<uint2*>(my_v + (q / PIECES) * RS + 16 * (q % PIECES));
            dst[0] = make_uint2(vreg[k].x, vreg[k].y);
            dst[1] = make_uint2(vreg[k].z, vreg[k].w);
        }
        // scores of the two 16-token halves
        m40_float4 sA = {0.f, 0.f, 0.f, 0.f}, sB = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < KS; ++i) {
            sA = mfma16x16x32(qf[i], kreg[0][i], sA);
            sB = mfma16x16x32(qf[i], kreg[1][i], sB);
        }
        if (tile + kWaves < ntiles) issue(tile + kWaves);      // in flight during the rest of this tile
        const bool vA = (uint32_t)(tile * kTile + c16) < ntok, vB = (uint32_t)(tile * kTile + 16 + c16) < ntok;
        const float a0 = vA ? (sA[0] + sA[1]) * score_scale : -INFINITY;
        const float a1 = vA ? (sA[2] + sA[3]) * score_scale : -INFINITY;
        const float b0 = vB ? (sB[0] + sB[1]) * score_scale : -INFINITY;
        const float b1 = vB ? (sB[2] + sB[3]) * score_scale : -INFINITY;
        const float n0 = fmaxf(m0, max16(fmaxf(a0, b0)));
        const float n1 = fmaxf(m1, max16(fmaxf(a1, b1)));
        const float f0 = __expf(m0 - n0), f1 = __expf(m1 - n1);       // first tile: exp(-inf) = 0
        const float pA0 = __expf(a0 - n0), pB0 = __expf(b0 - n0);
        const float pA1 = __expf(a1 - n1), pB1 = __expf(b1 - n1);
        l0 = fmaf(l0, f0, pA0 + pB0);
        l1 = fmaf(l1, f1, pA1 + pB1);
        const bool moved = (m0 != n0) || (m1 != n1);
        m0 = n0; m1 = n1;
        if (__any(moved)) {
#pragma unroll
            for (int d = 0; d < DT; ++d) {
                O[d][0] *= f0; O[d][1] *= f0; O[d][2] *= f1; O[d][3] *= f1;
            }
        }
        // softmax weights -> LDS in A-operand order: row 4g + {0: hi head 2g, 1: lo, 2: hi head 2g+1, 3: lo}
        {
            uint16_t (*pl)[40] = p_lds[wave];
            const _Float16 hA0 = static_cast<_Float16>(pA0), hB0 = static_cast<_Float16>(pB0);
            const _Float16 hA1 = static_cast<_Float16>(pA1), hB1 = static_cast<_Float16>(pB1);
            pl[4 * g + 0][c16] = __builtin_bit_cast(uint16_t, hA0);
            pl[4 * g + 1][c16] = f16_bits(pA0 - static_cast<float>(hA0));
            pl[4 * g + 2][c16] = __builtin_bit_cast(uint16_t, hA1);
            pl[4 * g + 3][c16] = f16_bits(pA1 - static_cast<float>(hA1));
            pl[4 * g + 0][16 + c16] = __builtin_bit_cast(uint16_t, hB0);
            pl[4 * g + 1][16 + c16] = f16_bits(pB0 - static_cast<float>(hB0));
            pl[4 * g + 2][16 + c16] = __builtin_bit_cast(uint16_t, hB1);
            pl[4 * g + 3][16 + c16] = f16_bits(pB1 - static_cast<float>(hB1));
        }
        const uint4 pa = *reinterpret_cast<const uint4*>(&p_lds[wave][c16][8 * g]);
        // O += P . V, one 16-column tile at a time: lane (column c16, group g) gathers tokens 8g .. 8g+7
#pragma unroll
        for (int d = 0; d < DT; ++d) {
            const uint8_t* col = my_v + (8 * g) * RS + 2 * (16 * d + c16);
            uint32_t w[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t lo = *reinterpret_cast<const uint16_t*>(col + (2 * j) * RS);
                const uint32_t hi = *reinterpret_cast<const uint16_t*>(col + (2 * j + 1) * RS);
                w[j] = lo | (hi << 16);
            }
            O[d] = mfma16x16x32(pa, make_uint4(w[0], w[1], w[2], w[3]), O[d]);
        }
    }

    // ---- merge the four waves --------------------------------------------------------------------------------------
    l0 = m40_sum16(l0);
    l1 = m40_sum16(l1);
    if (c16 == 0) {
        m_s[wave][2 * g] = m0; m_s[wave][2 * g + 1] = m1;
        l_s[wave][2 * g] = l0; l_s[wave][2 * g + 1] = l1;
    }
#pragma unroll
    for (int d = 0; d < DT; ++d) {
        o_s[wave][2 * g][16 * d + c16] = O[d][0] + O[d][1];
        o_s[wave][2 * g + 1][16 * d + c16] = O[d][2] + O[d][3];
    }
    __syncthreads();
    const bool final_out = p.nchunks == 1;
    for (uint32_t e = tid; e < gcount * HD; e += kThreads) {
        const uint32_t h = e / HD, d = e % HD;
        float M = m_s[0][h];
#pragma unroll
        for (int w = 1; w < kWaves; ++w) M = fmaxf(M, m_s[w][h]);
        float num = 0.0f, den = 0.0f;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) {
            const float f = __expf(m_s[w][h] - M);       // a wave without tiles holds -inf -> 0
            num = fmaf(o_s[w][h][d], f, num);
            den = fmaf(l_s[w][h], f, den);
        }
        const uint32_t qh = qh0 + h;
        if (final_out) {
            p.Out[((size_t)b * p.q_heads + qh) * HD + d] = num / (den > 0.0f ? den : 1.0f);
        } else {
            float* w = p.ws + (((size_t)b * p.q_heads + qh) * p.nchunks + blockIdx.y) * (HD + 2);
            w[2 + d] = num;
            if (d == 0) {
                w[0] = M;
                w[1] = den;
            }
        }
    }
}

}  // namespace

void m40_launch_attn_mfma(hipStream_t stream, const AttnParams& p, uint32_t head_dim, uint32_t batch) {
    dim3 grid(p.kv_heads * p.subgroups, p.nchunks, batch);
    if (head_dim == 64) attn_mfma_kernel<64><<<grid, kThreads, 0, stream>>>(p);
    else attn_mfma_kernel<128><<<grid, kThreads, 0, stream>>>(p);
}
