// Block-select "exact old" attention for gfx950: exact recent window + top-k old blocks chosen
// by mean-K block scores, over (a) the fp16-K / q4-V compressed cache and (b) a dense cache.
//
//   1. score  : a group of lanes per (old block, kv head) streams the block's K rows once (128-bit loads) and keeps,
//               per dimension and q head of the GQA group, the running sum q[d] * K[t][d] over the block's tokens in
//               token order (one fused multiply-add per element), so old K is read once per kv head, not once per q
//               head.  The per-dimension sums are then added by the halving tree over 128 slots that the reference's
//               128-thread kernel uses (cuda/kernels.cu:2893-2912): scores carry the reference kernel's bits.
//               score = (tree sum / len) * inv_sqrt.
//   2. rank   : per q head, blocks ordered by (score descending, block id ascending): the order the reference's
//               strict-'>' insertion into a list initialised to -1e30 produces (cuda/kernels.cu:2913-2927); the
//               first min(top_blocks, old_blocks) valid ones are kept.  A block's rank is the number of blocks above
//               it, counted 64 blocks at a time with one compare and a wave-wide ballot.
//   3. attend : per q head, softmax attention over [tokens of the selected blocks] ++ [recent window], one block per
//               wave.  Old V is unpacked from 4 bits in registers (value = nibble * scale, rounded through f16 as
//               the reference does).
//   4. combine: chunk partials merged in ascending order.
//
// The compressed cache keeps its old store head-major ([kv head][token][...]), so a selected block is one contiguous
// run of K rows, of packed V and of scales; the dense cache is token-major ([token][kv head][head_dim]).
//
// Reference: kernel cuda/kernels.cu:2832-3096 (compressed) and :1825-1983 (dense), entry points
// :4504-4577 and :4025-4070.  Only the plain top-k policy and score-rank block order are built.
#include "common.hpp"

#include <cstdlib>
#include <cstring>

namespace {

struct BsParams {
    // token t of kv head h of the old part: old_k + h * old_head_stride + t * old_tok_stride (elements)
    const uint16_t* old_k;     // compressed: [kvh][max_seq_len][hd] of this sequence; dense: K of this sequence
    const uint16_t* new_k;     // ring [W][kvh][hd] of this sequence, or dense K of this sequence
    const uint16_t* dense_v;   // ring V (compressed) or dense V of this sequence
    const uint8_t* q4_v;       // [kvh][max_seq_len][hd/2] of this sequence (compressed only)
    const float* q4_scale;     // [kvh][max_seq_len]; v_format 1: u32 [kvh][max_seq_len][hd/32], scale | min << 16
    uint32_t v_format;
    const float* Q;            // [q_heads][hd]
    float* Out;
    float* scores;             // [q_heads][nblk]
    uint32_t* sel;             // [q_heads][64]   block ids in rank order
    float* sel_scores;         // [q_heads][64]
    uint32_t* counts;          // [q_heads] selected blocks
    float* partial;            // [q_heads][nchunks][hd+2]
    size_t old_head_stride;
    uint32_t old_tok_stride;
    uint32_t max_seq_len;
    uint32_t kv_heads, q_heads, seq_len, recent_window, block_size, top_n;
    uint32_t old_len, nblk, compressed;
    uint32_t old_chunks, nchunks;   // chunks of the selected-block list, and those plus the chunks of the recent window
};

constexpr int kBsMaxSlots = 8;
// Several independent slots (sequences) per launch: blockIdx.z picks the slot.
struct BsMulti {
    BsParams slot[kBsMaxSlots];
};

// ---- 1. block scores ------------------------------------------------------------------------
// Two waves per workgroup; a lane holds DPL consecutive dimensions (DPL = 4: 8-byte loads, 32 lanes per row at
// head_dim 128), so a wave owns 64 / (HD / DPL) blocks at once: lane (block bg, chunk c) walks the tokens of its block
// in order with 32 rows in flight.  Four dimensions per lane give twice the waves of eight (two per SIMD on one
// 32 K-token sequence), which is what hides the latency of the row stream.
template <int DPL> struct BsLoadWord;
template <> struct BsLoadWord<8> { typedef uint4 type; };
template <> struct BsLoadWord<4> { typedef uint2 type; };
__device__ __forceinline__ uint4 bs_load_row(const uint4* p) { return m40_load_stream(p); }
__device__ __forceinline__ uint2 bs_load_row(const uint2* p) {
    typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
    const u32x2 v = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(p));
    return make_uint2(v.x, v.y);
}
__device__ __forceinline__ void bs_unpack(const uint4& w, float (&f)[8]) { m40_unpack8(w, f); }
__device__ __forceinline__ void bs_unpack(const uint2& w, float (&f)[4]) {
    f[0] = m40_h2f((uint16_t)(w.x & 0xffffu)); f[1] = m40_h2f((uint16_t)(w.x >> 16));
    f[2] = m40_h2f((uint16_t)(w.y & 0xffffu)); f[3] = m40_h2f((uint16_t)(w.y >> 16));
}

template <int HD, int G, int DPL, bool PRED>
__device__ __forceinline__ void bs_score_block(const uint16_t* kb, uint32_t tok_stride, uint32_t start, uint32_t end,
                                               uint32_t block_size, const float (&q)[G][DPL], float (&acc)[G][DPL]) {
    constexpr int U = 16;      // rows in flight per lane (32: 36.0 / 88.9 us for one / four slots at 32 K, 16: 35.8 / 87.0, 8: 35.4 / 87.5)
    typedef typename BsLoadWord<DPL>::type Word;
    Word buf[U];
    auto load = [&](int u, uint32_t off) {
        uint32_t t = start + off + (uint32_t)u;
        t = t < end ? t : end - 1u;               // rows past the block re-read its last row and are not used
        buf[u] = bs_load_row(reinterpret_cast<const Word*>(kb + (size_t)t * tok_stride));
    };
    auto consume = [&](int u, uint32_t off) {
        float kf[DPL];
        bs_unpack(buf[u], kf);
        const bool valid = !PRED || (start + off + (uint32_t)u < end);
#pragma unroll
        for (int h = 0; h < G; ++h)
#pragma unroll
            for (int j = 0; j < DPL; ++j) {
                const float v = fmaf(q[h][j], kf[j], acc[h][j]);
                acc[h][j] = valid ? v : acc[h][j];
            }
    };
    // A rolling window: row u of the next batch is requested as soon as row u of this one has been used, so U rows
    // stay in flight.  The scheduler must not sink a load below later arithmetic (it would, to save registers, and
    // every load would then be waited for on its own): nothing moves across the barriers.
#pragma unroll
    for (int u = 0; u < U; ++u) load(u, 0);
    __builtin_amdgcn_sched_barrier(0);
    uint32_t off = 0;
    while (off + U < block_size) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            consume(u, off);
            load(u, off + U);
            __builtin_amdgcn_sched_barrier(0);
        }
        off += U;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) consume(u, off);
}

template <int HD, int G, int DPL>
__global__ __launch_bounds__(128) void bs_score_kernel(BsMulti multi) {
    const BsParams& p = multi.slot[blockIdx.z];
    constexpr int C = HD / DPL;   // lanes per K row
    constexpr int BPW = 64 / C;   // blocks per wave
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int bg = lane / C, c = lane % C;
    const uint32_t first = (blockIdx.x * 2u + (uint32_t)wave) * BPW;
    if (first >= p.nblk) return;                       // the whole wave is past the last block
    const bool live = first + (uint32_t)bg < p.nblk;
    const uint32_t blk = live ? first + (uint32_t)bg : p.nblk - 1u;
    const uint32_t kvh = blockIdx.y;
    const uint32_t start = blk * p.block_size;
    const uint32_t end = start + p.block_size < p.old_len ? start + p.block_size : p.old_len;
    const uint16_t* kb = p.old_k + (size_t)kvh * p.old_head_stride + DPL * c;
    const uint32_t group = p.q_heads / p.kv_heads;
    const float inv_sqrt = HD == 64 ? 0.125f : 0.08838834764831845f;
    const float len = (float)(end - start);
    // every block of the wave is whole and the unrolled batches divide it: no per-row validity test
    const bool whole = __all((end - start == p.block_size) ? 1 : 0) && (p.block_size % 32u == 0u);

    for (uint32_t h0 = 0; h0 < group; h0 += G) {
        float q[G][DPL], acc[G][DPL];
#pragma unroll
        for (int h = 0; h < G; ++h) {
            const uint32_t hh = h0 + h < group ? h0 + h : group - 1u;
            const float* qp = p.Q + ((size_t)kvh * group + hh) * HD + DPL * c;
#pragma unroll
            for (int j = 0; j < DPL; j += 4) {
                const float4 qq = *reinterpret_cast<const float4*>(qp + j);
                q[h][j] = qq.x; q[h][j + 1] = qq.y; q[h][j + 2] = qq.z; q[h][j + 3] = qq.w;
            }
#pragma unroll
            for (int j = 0; j < DPL; ++j) acc[h][j] = 0.0f;
        }
        if (whole) bs_score_block<HD, G, DPL, false>(kb, p.old_tok_stride, start, end, p.block_size, q, acc);
        else bs_score_block<HD, G, DPL, true>(kb, p.old_tok_stride, start, end, p.block_size, q, acc);
        // The reference's tree over 128 slots, slot = dimension d = DPL c + j: slot d += slot d + 64, then + 32, ...
        // down to + DPL (lane c takes lane c + 64 / DPL, ..., c + 1 of its block), then the rest inside the lane.
        // With head_dim 64 the upper 64 slots hold 0.
#pragma unroll
        for (int h = 0; h < G; ++h) {
            float v[DPL];
#pragma unroll
            for (int j = 0; j < DPL; ++j) {
                float x = acc[h][j];
                if (HD == 128) x += __shfl_xor(x, 64 / DPL, 64);
                else x += 0.0f;
#pragma unroll
                for (int o = 32 / DPL; o >= 1; o >>= 1) x += __shfl_xor(x, o, 64);
                v[j] = x;
            }
            float r;
            if (DPL == 8) {
                const float s0 = v[0] + v[4 % DPL], s1 = v[1] + v[5 % DPL], s2 = v[2] + v[6 % DPL], s3 = v[3] + v[7 % DPL];
                r = (s0 + s2) + (s1 + s3);
            } else {
                r = (v[0] + v[2]) + (v[1] + v[3]);
            }
            if (c == 0 && live && h0 + h < group)
                p.scores[((size_t)kvh * group + h0 + h) * p.nblk + blk] = (r / len) * inv_sqrt;
        }
    }
}

// ---- 2. ranking ---------------------------------------------------------------------------------------------------
// Block b is at rank #{o : score[o] > score[b] or (== and o < b)}: the order the reference's strict-'>' insertion
// into a list initialised to -1e30 produces (cuda/kernels.cu:2913-2927); scores that are NaN or not above -1e30 never
// enter the list.  Grid (q head, 16 candidate blocks, slot), four waves of 4 candidates each.  A wave holds the order
// keys of all blocks 64 at a time, one per lane, and counts the blocks above a candidate with one compare and a
// wave-wide ballot per 64 blocks.  sel[rank] = block for rank < top_n; the first workgroup of a head also writes the
// list length and the unused tail of the list.
__device__ __forceinline__ uint32_t bs_order_key(float s) {
    const uint32_t u = __float_as_uint(s);
    const uint32_t k = (u & 0x80000000u) ? ~u : (u | 0x80000000u);      // monotone in s
    return (s > -1e30f) ? k : 0u;                                       // invalid (and NaN): below every valid key
}
constexpr int kBsRankThreads = 256, kBsRankCand = 16;
__global__ __launch_bounds__(kBsRankThreads) void bs_rank_kernel(BsMulti multi) {
    const BsParams& p = multi.slot[blockIdx.z];
    extern __shared__ uint32_t s_keys[];            // order keys of the head's blocks, padded with zeros to 64 words
    __shared__ uint32_t s_valid[kBsRankThreads / 64];
    const uint32_t qh = blockIdx.x, y = blockIdx.y;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    if (p.nblk == 0) {
        if (y == 0) {
            if (tid < 64) { p.sel[qh * 64 + tid] = 0xffffffffu; p.sel_scores[qh * 64 + tid] = -1e30f; }
            if (tid == 0) p.counts[qh] = 0;
        }
        return;
    }
    if (y * kBsRankCand >= p.nblk) return;
    const uint32_t n64 = (p.nblk + 63u) / 64u;
    const float* scores = p.scores + (size_t)qh * p.nblk;
    uint32_t valid = 0;
    for (uint32_t b = tid; b < n64 * 64u; b += kBsRankThreads) {
        const uint32_t k = b < p.nblk ? bs_order_key(scores[b]) : 0u;
        s_keys[b] = k;
        valid += k != 0u ? 1u : 0u;
    }
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) valid += __shfl_xor(valid, o, 64);
    if (lane == 0) s_valid[wave] = valid;
    __syncthreads();
    constexpr int CPW = kBsRankCand / (kBsRankThreads / 64);     // candidates per wave
    const uint32_t cand0 = y * kBsRankCand + (uint32_t)wave * CPW;
    uint32_t kb[CPW], above[CPW];
#pragma unroll
    for (int i = 0; i < CPW; ++i) {
        const uint32_t b = cand0 + i;
        kb[i] = b < p.nblk ? s_keys[b] : 0u;      // wave-uniform
        above[i] = 0;
    }
    for (uint32_t ch = 0; ch < n64; ++ch) {
        const uint32_t o = ch * 64u + (uint32_t)lane;
        const uint32_t ko = s_keys[o];
#pragma unroll
        for (int i = 0; i < CPW; ++i) {
            // blocks before the candidate count when they score at least as high, blocks after it when higher
            const uint32_t thr = kb[i] + (o >= cand0 + i ? 1u : 0u);
            above[i] += (uint32_t)__popcll(__ballot(ko >= thr));
        }
    }
    if (lane == 0) {
#pragma unroll
        for (int i = 0; i < CPW; ++i) {
            if (kb[i] != 0u && above[i] < p.top_n) {
                p.sel[qh * 64 + above[i]] = cand0 + i;
                p.sel_scores[qh * 64 + above[i]] = scores[cand0 + i];
            }
        }
    }
    if (y == 0 && tid < 64) {
        uint32_t total = 0;
        for (int w = 0; w < kBsRankThreads / 64; ++w) total += s_valid[w];
        const uint32_t count = total < p.top_n ? total : p.top_n;
        if ((uint32_t)tid >= count) { p.sel[qh * 64 + tid] = 0xffffffffu; p.sel_scores[qh * 64 + tid] = -1e30f; }
        if (tid == 0) p.counts[qh] = count;
    }
}

// ---- 3. attention over the selected old blocks and the recent window ---------------------------------------------
// Grid (q head, chunk, slot), four waves per workgroup.  Chunks [0, old_chunks) cover the ranked list, one block per
// wave; the other chunks cover the recent window, kBsNewChunk tokens each.  A wave attends 64 (q4 store) or 32 (f16
// rows) tokens per pass: every lane issues the loads of all of its token rows before any arithmetic, scores stay in
// registers, and passes are joined with a running maximum.
constexpr int kBsThreads = 256, kBsWaves = 4;
constexpr int kBsNewChunk = 128;    // recent tokens per workgroup
constexpr int kBsPassQuant = 64;    // tokens per wave pass over the q4 old store
constexpr int kBsPassF16 = 32;      // tokens per wave pass over f16 K / V rows (twice the bytes per token)

struct BsWaveState {
    float m;          // running maximum (wave-uniform)
    float l;          // this lane's share of the sum of weights
    float acc[8];     // this lane's share of the weighted V sum, dimensions 8c .. 8c+7
};

// Token rows of one pass of a wave (at most kPass tokens) as they arrive from memory.
// VF (with QUANT): old V format, 0 the reference's q4 with one f32 scale per token and head, 1 groups of 32 with an f16
// scale and an f16 minimum.
template <int HD, bool QUANT, int VF = 0>
struct BsRows {
    static constexpr int kPass = QUANT ? kBsPassQuant : kBsPassF16;
    static constexpr int S = kPass / (64 / (HD / 8));
    uint4 kw[S];
    uint4 vw[QUANT ? 1 : S];
    uint32_t qw[QUANT ? S : 1];
    float qs[QUANT ? S : 1];         // VF 1: the bits of the group's scale | min << 16
    uint32_t t_begin, t_end;
};

// Requests tokens [t_begin, t_end) of kv head kvh.  Every load is issued, in a fixed order, before anything that
// follows the call, and none sits under a branch.
//   QUANT: old tokens of the compressed cache (K f16 head-major, V 4-bit).  The rows of a pass are consecutive in all
//   three arrays, so a lane needs one 32-bit offset per array and the rest are instruction immediates; rows past
//   t_end are read as they lie (the next tokens, the next head, or the zeroed slack rows the cache allocates behind
//   its old store) and carry no weight.
//   Otherwise: f16 K and V rows of the ring or of a dense cache; rows past the end repeat the last one.
template <int HD, bool QUANT, int VF>
__device__ __forceinline__ void bs_issue(const BsParams& p, uint32_t kvh, uint32_t t_begin, uint32_t t_end,
                                         BsRows<HD, QUANT, VF>& r) {
    constexpr int LPT = HD / 8, TPW = 64 / LPT, S = BsRows<HD, QUANT, VF>::S;
    const int lane = threadIdx.x & 63;
    const int c = lane % LPT, tg = lane / LPT;
    r.t_begin = t_begin; r.t_end = t_end;
    if (QUANT) {
        const char* kbase = reinterpret_cast<const char*>(p.old_k + (size_t)kvh * p.old_head_stride);
        const char* vbase = reinterpret_cast<const char*>(p.q4_v + (size_t)kvh * p.max_seq_len * (HD / 2));
        // bytes of scale data per row: one f32, or one word per group of 32 dimensions (a lane's eight dimensions 8c..8c+7
        // lie in group c / 4)
        constexpr int SB = VF == 1 ? (HD / 32) * 4 : 4;
        const char* sbase = reinterpret_cast<const char*>(p.q4_scale) + (size_t)kvh * p.max_seq_len * SB;
        const uint32_t row = t_begin + (uint32_t)tg;
        const uint32_t koff = row * (HD * 2) + 16 * c, voff = row * (HD / 2) + 4 * c;
        const uint32_t soff = row * SB + (VF == 1 ? 4 * (c / 4) : 0);
#pragma unroll
        for (int s = 0; s < S; ++s) {
            r.kw[s] = *reinterpret_cast<const uint4*>(kbase + koff + s * (TPW * HD * 2));
            r.qw[s] = *reinterpret_cast<const uint32_t*>(vbase + voff + s * (TPW * HD / 2));
            r.qs[s] = *reinterpret_cast<const float*>(sbase + soff + s * (TPW * SB));
        }
    } else {
        const uint32_t row_bytes = p.kv_heads * HD * 2;
        const char* kbase = reinterpret_cast<const char*>(p.new_k + (size_t)kvh * HD);
        const char* vbase = reinterpret_cast<const char*>(p.dense_v + (size_t)kvh * HD);
        // ring row of the first token (one division per pass, wave-uniform); the rows after it wrap at most once
        const uint32_t wrap = p.compressed ? p.recent_window : 0xffffffffu;
        const uint32_t r0 = p.compressed ? t_begin % p.recent_window : t_begin;
#pragma unroll
        for (int s = 0; s < S; ++s) {
            uint32_t i = (uint32_t)(s * TPW + tg);
            i = t_begin + i < t_end ? i : t_end - 1u - t_begin;
            uint32_t rr = r0 + i;
            rr = rr >= wrap ? rr - wrap : rr;
            const size_t off = (size_t)rr * row_bytes + 16 * c;
            r.kw[s] = *reinterpret_cast<const uint4*>(kbase + off);
            r.vw[s] = *reinterpret_cast<const uint4*>(vbase + off);
        }
    }
    // the scheduler may not move these loads below later arithmetic (it would, to save registers, and each pass would
    // then cost another memory round trip), nor later loads above them
    __builtin_amdgcn_sched_barrier(0);
}

// two f32 -> two f16, round to nearest even; the values are pinned first so that a preceding multiply-add is not
// folded into a single-rounding mixed-precision instruction (the reference rounds to f32, then to f16)
__device__ __forceinline__ uint32_t bs_f2h_pair(float a, float b) {
    asm volatile("" : "+v"(a), "+v"(b));
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
    const f32x2 x = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(x, f16x2));
}

// Softmax terms of the rows of one pass, joined to the wave's running state.
template <int HD, bool QUANT, int VF>
__device__ __forceinline__ void bs_consume(const float (&q)[8], const BsRows<HD, QUANT, VF>& r, BsWaveState& st) {
    constexpr int LPT = HD / 8, TPW = 64 / LPT, S = BsRows<HD, QUANT, VF>::S;
    const int lane = threadIdx.x & 63;
    const int c = lane % LPT, tg = lane / LPT;
    const float inv_sqrt = HD == 64 ? 0.125f : 0.08838834764831845f;
    float sc[S];
    float pmax = -INFINITY;
#pragma unroll
    for (int s = 0; s < S; ++s) {
        float kf[8];
        m40_unpack8(r.kw[s], kf);
        float d = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) d = fmaf(q[j], kf[j], d);
        d = LPT == 8 ? m40_sum8(d) : m40_sum16(d);
        const bool valid = r.t_begin + (uint32_t)(s * TPW + tg) < r.t_end;
        sc[s] = valid ? d * inv_sqrt : -INFINITY;
        pmax = fmaxf(pmax, sc[s]);
    }
    pmax = m40_max64(pmax);
    const float m_new = fmaxf(st.m, pmax);
    const float f_old = st.m == -INFINITY ? 0.0f : __expf(st.m - m_new);
    st.l *= f_old;
#pragma unroll
    for (int j = 0; j < 8; ++j) st.acc[j] *= f_old;
    st.m = m_new;
#pragma unroll
    for (int s = 0; s < S; ++s) {
        const float e = __expf(sc[s] - m_new);        // rows past the end: exp(-inf) = 0
        if (c == 0) st.l += e;
        if (QUANT && VF == 1) {
            // value = fmaf(nibble, scale, min), scale and min f16 (one rounding; no pass through f16)
            const uint32_t dm = __float_as_uint(r.qs[s]);
            const float d = m40_h2f((uint16_t)(dm & 0xffffu)), mn = m40_h2f((uint16_t)(dm >> 16));
            const uint32_t even = r.qw[s] & 0x0f0f0f0fu, odd = (r.qw[s] >> 4) & 0x0f0f0f0fu;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                st.acc[2 * k] = fmaf(e, fmaf((float)((even >> (8 * k)) & 0xffu), d, mn), st.acc[2 * k]);
                st.acc[2 * k + 1] = fmaf(e, fmaf((float)((odd >> (8 * k)) & 0xffu), d, mn), st.acc[2 * k + 1]);
            }
        } else if (QUANT) {
            // value = nibble * scale rounded to f32, then through f16 (cuda/kernels.cu:3078-3084).  The eight nibbles
            // become bytes biased by 8 (two's complement n -> (n ^ 8) - 8), a byte converts in one instruction, and
            // byte * scale - 8 * scale in one fused operation is the product nibble * scale rounded once.
            const uint32_t even = (r.qw[s] & 0x0f0f0f0fu) ^ 0x08080808u;            // dimensions 0, 2, 4, 6
            const uint32_t odd = ((r.qw[s] >> 4) & 0x0f0f0f0fu) ^ 0x08080808u;      // dimensions 1, 3, 5, 7
            const float scale = r.qs[s], bias = -8.0f * scale;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const float v0 = fmaf((float)((even >> (8 * k)) & 0xffu), scale, bias);
                const float v1 = fmaf((float)((odd >> (8 * k)) & 0xffu), scale, bias);
                const uint32_t h = bs_f2h_pair(v0, v1);
                st.acc[2 * k] = fmaf(e, m40_h2f((uint16_t)(h & 0xffffu)), st.acc[2 * k]);
                st.acc[2 * k + 1] = fmaf(e, m40_h2f((uint16_t)(h >> 16)), st.acc[2 * k + 1]);
            }
        } else {
            float vf[8];
            m40_unpack8(r.vw[s], vf);
#pragma unroll
            for (int j = 0; j < 8; ++j) st.acc[j] = fmaf(e, vf[j], st.acc[j]);
        }
    }
}

// Tokens [t_begin, t_end) for one wave, kPass tokens per pass (one pass for a block of at most 64 old tokens, and
// for a wave's share of a chunk of the recent window).
template <int HD, bool QUANT, int VF = 0>
__device__ __forceinline__ void bs_wave_attend(const BsParams& p, uint32_t kvh, const float (&q)[8], uint32_t t_begin,
                                               uint32_t t_end, BsWaveState& st) {
    constexpr uint32_t kPass = BsRows<HD, QUANT, VF>::kPass;
    for (uint32_t t0 = t_begin; t0 < t_end; t0 += kPass) {
        BsRows<HD, QUANT, VF> rows;
        bs_issue<HD, QUANT, VF>(p, kvh, t0, t0 + kPass < t_end ? t0 + kPass : t_end, rows);
        bs_consume<HD, QUANT, VF>(q, rows, st);
    }
}

template <int HD>
__global__ __launch_bounds__(kBsThreads, 3) void bs_attend_kernel(BsMulti multi) {
    const BsParams& p = multi.slot[blockIdx.z];
    constexpr int LPT = HD / 8;
    __shared__ float red[kBsWaves][HD];
    __shared__ float wmax[kBsWaves], wsum[kBsWaves];
    const uint32_t qh = blockIdx.x, y = blockIdx.y;
    if (y >= p.nchunks) return;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int c = lane % LPT;
    // the division runs on the vector unit; the result is the same in every lane, and as a scalar it lets the row
    // loads take their base address from scalar registers
    const uint32_t kvh = (uint32_t)__builtin_amdgcn_readfirstlane((int)(qh / (p.q_heads / p.kv_heads)));

    float q[8];
    {
        const float4 q0 = *reinterpret_cast<const float4*>(p.Q + (size_t)qh * HD + 8 * c);
        const float4 q1 = *reinterpret_cast<const float4*>(p.Q + (size_t)qh * HD + 8 * c + 4);
        q[0] = q0.x; q[1] = q0.y; q[2] = q0.z; q[3] = q0.w; q[4] = q1.x; q[5] = q1.y; q[6] = q1.z; q[7] = q1.w;
    }
    BsWaveState st;
    st.m = -INFINITY; st.l = 0.0f;
#pragma unroll
    for (int j = 0; j < 8; ++j) st.acc[j] = 0.0f;

    if (y >= p.old_chunks) {
        // recent window: tokens old_len .. seq_len - 1, the chunk's tokens split evenly over the waves
        const uint32_t cbeg = p.old_len + (y - p.old_chunks) * kBsNewChunk;
        const uint32_t cend = cbeg + kBsNewChunk < p.seq_len ? cbeg + kBsNewChunk : p.seq_len;
        constexpr uint32_t per_wave = kBsNewChunk / kBsWaves;
        uint32_t b0 = cbeg + (uint32_t)wave * per_wave;
        b0 = b0 < cend ? b0 : cend;
        const uint32_t b1 = b0 + per_wave < cend ? b0 + per_wave : cend;
        bs_wave_attend<HD, false>(p, kvh, q, b0, b1, st);
    } else {
        // old part: wave w of chunk y attends the block of rank 4 y + w, if the list is that long
        const uint32_t rank = y * kBsWaves + (uint32_t)wave;
        const uint32_t count = p.counts[qh];
        const uint32_t blk = p.sel[qh * 64 + (rank < 64u ? rank : 63u)];
        uint32_t b0 = 0, b1 = 0;
        if (rank < count) {
            b0 = blk * p.block_size;
            b1 = b0 + p.block_size < p.old_len ? b0 + p.block_size : p.old_len;
        }
        if (p.compressed && p.v_format) bs_wave_attend<HD, true, 1>(p, kvh, q, b0, b1, st);
        else if (p.compressed) bs_wave_attend<HD, true, 0>(p, kvh, q, b0, b1, st);
        else bs_wave_attend<HD, false>(p, kvh, q, b0, b1, st);
    }

    // ---- join the lanes of a wave, then the waves ------------------------------------------------------------------
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        st.acc[j] = m40_sum_lanes_from<LPT>(st.acc[j]);
    }
    const float lsum = m40_sum64(st.l);
    if (lane == 0) { wmax[wave] = st.m; wsum[wave] = lsum; }
    if (lane < LPT) {
#pragma unroll
        for (int j = 0; j < 8; ++j) red[wave][8 * c + j] = st.acc[j];
    }
    __syncthreads();
    if (tid < HD) {
        float M = wmax[0];
#pragma unroll
        for (int w = 1; w < kBsWaves; ++w) M = fmaxf(M, wmax[w]);
        float v = 0.0f, l = 0.0f;
#pragma unroll
        for (int w = 0; w < kBsWaves; ++w) {
            const float f = wmax[w] == -INFINITY ? 0.0f : __expf(wmax[w] - M);
            v = fmaf(red[w][tid], f, v);
            l = fmaf(wsum[w], f, l);
        }
        if (p.nchunks == 1) {
            p.Out[(size_t)qh * HD + tid] = v / (l > 0.0f ? l : 1.0f);
        } else {
            float* w = p.partial + ((size_t)qh * p.nchunks + y) * (HD + 2);
            w[2 + tid] = v;                 // an empty chunk leaves M = -inf, which the merge skips
            if (tid == 0) { w[0] = M; w[1] = l; }
        }
    }
}

// Merge the chunk partials of one q head: 1024 threads = 1024/HD chunk lanes x HD dims, each lane folds chunks
// lane, lane + n_lanes, ... with a running maximum; the lanes are then folded in order.  Empty partials (maximum
// -inf) are skipped.
template <int HD>
__global__ __launch_bounds__(1024) void bs_combine_kernel(BsMulti multi) {
    const BsParams& p = multi.slot[blockIdx.z];
    if (p.nchunks <= 1) return;      // the attend kernel wrote the output itself
    constexpr int NCG = 1024 / HD;
    __shared__ float s_m[NCG], s_den[NCG];
    __shared__ float s_num[NCG][HD];
    const uint32_t qh = blockIdx.x, d = threadIdx.x % HD, cg = threadIdx.x / HD;
    const uint32_t n = p.nchunks;
    const float* w = p.partial + (size_t)qh * p.nchunks * (HD + 2);
    float m = -INFINITY, num = 0.0f, den = 0.0f;
    for (uint32_t ch = cg; ch < n; ch += NCG) {
        const float* wc = w + (size_t)ch * (HD + 2);
        const float mc = wc[0], lc = wc[1], vc = wc[2 + d];
        if (mc == -INFINITY) continue;
        const float nm = fmaxf(m, mc);
        const float fa = m == -INFINITY ? 0.0f : expf(m - nm);
        const float fb = expf(mc - nm);
        num = fmaf(num, fa, vc * fb);
        den = fmaf(den, fa, lc * fb);
        m = nm;
    }
    s_num[cg][d] = num;
    if (d == 0) { s_m[cg] = m; s_den[cg] = den; }
    __syncthreads();
    if (cg == 0) {
#pragma unroll
        for (int g = 1; g < NCG; ++g) {
            const float mc = s_m[g];
            if (mc == -INFINITY) continue;
            const float nm = fmaxf(m, mc);
            const float fa = m == -INFINITY ? 0.0f : expf(m - nm);
            const float fb = expf(mc - nm);
            num = fmaf(num, fa, s_num[g][d] * fb);
            den = fmaf(den, fa, s_den[g] * fb);
            m = nm;
        }
        p.Out[(size_t)qh * HD + d] = num / (den > 0.0f ? den : 1.0f);
    }
}

uint32_t policy_from_env() {
    const char* v = std::getenv("M40LLM_KV_BLOCK_SELECT_POLICY");
    if (!v || !v[0] || std::strcmp(v, "topk") == 0) return 0u;
    return 1u;  // any other policy name
}
uint32_t order_from_env() {
    const char* v = std::getenv("M40LLM_KV_SELECTED_BLOCK_ORDER");
    if (!v || !v[0]) return 0u;
    if (std::strcmp(v, "chronological") == 0 || std::strcmp(v, "descending") == 0) return 1u;
    return 0u;
}

// Fills the parameter block and checks scratch capacity.  Returns 0 or a negative code.
int prepare(M40llmCudaContext* ctx, const M40llmKVCache* kv, uint32_t seq_id, const void* q, uint32_t q_heads,
            uint32_t seq_len, uint32_t W, uint32_t bs, uint32_t top, void* out, bool compressed, BsParams* p,
            size_t* select_used = nullptr, size_t* partial_used = nullptr) {
    const size_t select_off = select_used ? *select_used : 0, partial_off = partial_used ? *partial_used : 0;
    std::memset(p, 0, sizeof(*p));
    const uint32_t hd = kv->head_dim, kvh = kv->num_heads;
    const size_t ept = (size_t)kvh * hd;
    const uint32_t old_len = seq_len > W ? seq_len - W : 0;
    const uint32_t nblk = old_len == 0 ? 0 : (old_len + bs - 1) / bs;
    const uint32_t sel_old = top < nblk ? top : nblk;
    const uint32_t recent_count = seq_len < W ? seq_len : W;
    uint32_t old_cap = sel_old * bs;
    if (old_cap > old_len) old_cap = old_len;
    const uint32_t capacity = recent_count + old_cap;
    if (capacity == 0 || capacity > seq_len) return -7;
    p->kv_heads = kvh; p->q_heads = q_heads; p->seq_len = seq_len; p->recent_window = W; p->block_size = bs;
    p->top_n = sel_old; p->old_len = old_len; p->nblk = nblk; p->compressed = compressed ? 1u : 0u;
    p->max_seq_len = kv->max_seq_len;
    p->Q = static_cast<const float*>(q);
    p->Out = static_cast<float*>(out);
    if (compressed) {
        if (((uint64_t)kv->max_seq_len + kM40OldStoreSlackRows) * hd * 2 > 0xffffffffull) return -7;   // 32-bit row offsets
        p->old_k = kv->d_fp16_old_k + (size_t)seq_id * kv->max_seq_len * ept;
        p->old_tok_stride = hd;
        p->old_head_stride = (size_t)kv->max_seq_len * hd;
        p->new_k = kv->d_recent_k + (size_t)seq_id * kv->recent_window * ept;
        p->dense_v = kv->d_recent_v + (size_t)seq_id * kv->recent_window * ept;
        p->q4_v = kv->d_q4_old_v + (size_t)seq_id * kv->max_seq_len * kvh * (hd / 2u);
        p->q4_scale = kv->d_q4_old_v_scale + (size_t)seq_id * kv->max_seq_len * kvh * (kv->v_format ? hd / 32u : 1u);
        p->v_format = kv->v_format;
    } else {
        p->old_k = kv->d_k + (size_t)seq_id * kv->max_seq_len * ept;
        p->old_tok_stride = (uint32_t)ept;
        p->old_head_stride = hd;
        p->new_k = p->old_k;
        p->dense_v = kv->d_v + (size_t)seq_id * kv->max_seq_len * ept;
    }
    M40StreamScratch& sc = ctx->scratch[1];
    // select scratch: scores | sel | sel_scores | counts
    const size_t scores_bytes = ((size_t)q_heads * (nblk ? nblk : 1) * 4 + 255) & ~(size_t)255;
    const size_t fixed = (size_t)q_heads * (64 * 4 + 64 * 4 + 4 + 4) + 1024;
    const size_t select_need = (scores_bytes + fixed + 255) & ~(size_t)255;
    if (select_off + select_need > sc.select_bytes) return -7;
    char* base = static_cast<char*>(sc.select) + select_off;
    p->scores = reinterpret_cast<float*>(base);
    p->sel = reinterpret_cast<uint32_t*>(base + scores_bytes);
    p->sel_scores = reinterpret_cast<float*>(p->sel + (size_t)q_heads * 64);
    p->counts = reinterpret_cast<uint32_t*>(p->sel_scores + (size_t)q_heads * 64);
    p->old_chunks = (sel_old + kBsWaves - 1) / kBsWaves;
    p->nchunks = p->old_chunks + (recent_count + kBsNewChunk - 1) / kBsNewChunk;
    const size_t partial_need = (((size_t)q_heads * p->nchunks * (hd + 2) * 4) + 255) & ~(size_t)255;
    if (partial_off + partial_need > sc.attn_partial_bytes) return -7;
    p->partial = reinterpret_cast<float*>(static_cast<char*>(sc.attn_partial) + partial_off);
    if (select_used) *select_used = select_off + select_need;
    if (partial_used) *partial_used = partial_off + partial_need;
    if ((size_t)((nblk + 63u) / 64u) * 256 > 60 * 1024) return -7;  // the order keys of one q head live in LDS
    return 0;
}

template <int HD>
int launch_multi(hipStream_t s, const BsMulti& m, uint32_t n, bool selection_only) {
    (void)hipGetLastError();
    const BsParams& p0 = m.slot[0];
    const uint32_t group = p0.q_heads / p0.kv_heads;
    uint32_t max_nblk = 0, max_chunks = 0;
    for (uint32_t i = 0; i < n; ++i) {
        max_nblk = m.slot[i].nblk > max_nblk ? m.slot[i].nblk : max_nblk;
        max_chunks = m.slot[i].nchunks > max_chunks ? m.slot[i].nchunks : max_chunks;
    }
    if (max_nblk > 0) {
        constexpr uint32_t DPL = 4;
        constexpr uint32_t per_wg = 2u * (64u / (HD / DPL));      // blocks per workgroup of two waves
        dim3 grid((max_nblk + per_wg - 1) / per_wg, p0.kv_heads, n);
        if (group >= 8) bs_score_kernel<HD, 8, DPL><<<grid, 128, 0, s>>>(m);
        else if (group >= 4) bs_score_kernel<HD, 4, DPL><<<grid, 128, 0, s>>>(m);
        else if (group >= 2) bs_score_kernel<HD, 2, DPL><<<grid, 128, 0, s>>>(m);
        else bs_score_kernel<HD, 1, DPL><<<grid, 128, 0, s>>>(m);
    }
    const size_t keys_lds = (size_t)((max_nblk + 63u) / 64u) * 256 + 16;
    bs_rank_kernel<<<dim3(p0.q_heads, max_nblk ? (max_nblk + kBsRankCand - 1) / kBsRankCand : 1, n), kBsRankThreads, keys_lds, s>>>(m);
    if (!selection_only) {
        bs_attend_kernel<HD><<<dim3(p0.q_heads, max_chunks, n), kBsThreads, 0, s>>>(m);
        if (max_chunks > 1) bs_combine_kernel<HD><<<dim3(p0.q_heads, 1, n), 1024, 0, s>>>(m);
    }
    return hipGetLastError() == hipSuccess ? 0 : -8;
}

template <int HD>
int launch_all(hipStream_t s, const BsParams& p, bool selection_only) {
    BsMulti m;
    std::memset(&m, 0, sizeof(m));
    m.slot[0] = p;
    return launch_multi<HD>(s, m, 1, selection_only);
}

int common_checks(M40llmCudaContext* ctx, const M40llmKVCache* kv, uint32_t seq_id, const void* q, uint32_t q_heads,
                  uint32_t seq_len, uint32_t W, uint32_t bs, uint32_t top, const void* out, bool compressed) {
    if (!ctx || !kv || !q || !out) return -1;
    if (compressed) {
        if (!kv->fp16_k_q4_v_old_backing || !kv->d_fp16_old_k || !kv->d_q4_old_v || !kv->d_q4_old_v_scale ||
            !kv->d_recent_k || !kv->d_recent_v)
            return -16;
    } else if (!kv->d_k || !kv->d_v) {
        return -16;
    }
    if (seq_id >= kv->max_batch_size) return -2;
    if (seq_len == 0 || seq_len > kv->max_seq_len) return -3;
    if (q_heads == 0 || kv->num_heads == 0 || q_heads % kv->num_heads != 0) return -4;
    if (kv->head_dim != 64 && kv->head_dim != 128) return -5;
    if (W == 0 || bs == 0 || top == 0 || top > 64) return -6;
    // The ring was written at position % (the cache's own window): a call with another window would read other
    // tokens' rows (the reference indexes the ring with the caller's value and returns whatever lies there).
    if (compressed && W != kv->recent_window) return -6;
    // Only the plain top-k policy in score-rank order is built; refuse the environment knobs of
    // the reference's experimental policies instead of silently computing something else.
    if (policy_from_env() != 0u || order_from_env() != 0u) return -17;
    return 0;
}

}  // namespace

extern "C" {

int m40llm_attention_last_token_f32_gqa_block_select_exact_fp16_k_q4_v_old_direct_async(
    M40llmCudaContext* ctx, const M40llmKVCache* kv, uint32_t seq_id, const void* q_dev_f32, uint32_t q_heads,
    uint32_t seq_len, uint32_t recent_window, uint32_t block_size, uint32_t top_blocks, void* out_dev_f32) {
    int rc = common_checks(ctx, kv, seq_id, q_dev_f32, q_heads, seq_len, recent_window, block_size, top_blocks,
                           out_dev_f32, true);
    if (rc != 0) return rc;
    BsParams p;
    rc = prepare(ctx, kv, seq_id, q_dev_f32, q_heads, seq_len, recent_window, block_size, top_blocks, out_dev_f32,
                 true, &p);
    if (rc != 0) return rc;
    return kv->head_dim == 64 ? launch_all<64>(ctx->decode_stream, p, false)
                              : launch_all<128>(ctx->decode_stream, p, false);
}

int m40llm_attention_last_token_f32_gqa_block_select_exact_async(
    M40llmCudaContext* ctx, const M40llmKVCache* kv, uint32_t seq_id, const void* q_dev_f32, uint32_t q_heads,
    uint32_t seq_len, uint32_t recent_window, uint32_t block_size, uint32_t top_blocks, void* out_dev_f32) {
    if (kv && kv->compressed) return -16;
    int rc = common_checks(ctx, kv, seq_id, q_dev_f32, q_heads, seq_len, recent_window, block_size, top_blocks,
                           out_dev_f32, false);
    if (rc != 0) return rc;
    BsParams p;
    rc = prepare(ctx, kv, seq_id, q_dev_f32, q_heads, seq_len, recent_window, block_size, top_blocks, out_dev_f32,
                 false, &p);
    if (rc != 0) return rc;
    return kv->head_dim == 64 ? launch_all<64>(ctx->decode_stream, p, false)
                              : launch_all<128>(ctx->decode_stream, p, false);
}

int m40llm_ext_attention_block_select_fp16_k_q4_v_multi_async(
    M40llmCudaContext* ctx, const M40llmKVCache* kv, uint32_t n_slots, const uint32_t* seq_ids_host,
    const uint32_t* seq_lens_host, const void* q_dev_f32, uint32_t q_heads, uint32_t recent_window, uint32_t block_size,
    uint32_t top_blocks, void* out_dev_f32) {
    if (!seq_ids_host || !seq_lens_host) return -1;
    if (n_slots == 0 || n_slots > (uint32_t)kBsMaxSlots) return -2;
    if (!kv) return -1;
    const size_t row = (size_t)q_heads * kv->head_dim;
    BsMulti m;
    std::memset(&m, 0, sizeof(m));
    size_t select_used = 0, partial_used = 0;
    for (uint32_t i = 0; i < n_slots; ++i) {
        const float* q = static_cast<const float*>(q_dev_f32) + i * row;
        float* out = static_cast<float*>(out_dev_f32) + i * row;
        int rc = common_checks(ctx, kv, seq_ids_host[i], q_dev_f32 ? q : nullptr, q_heads, seq_lens_host[i], recent_window,
                               block_size, top_blocks, out_dev_f32 ? out : nullptr, true);
        if (rc != 0) return rc;
        for (uint32_t k = 0; k < i; ++k)
            if (seq_ids_host[k] == seq_ids_host[i]) return -2;      // a slot at most once per call
        rc = prepare(ctx, kv, seq_ids_host[i], q, q_heads, seq_lens_host[i], recent_window, block_size, top_blocks, out, true,
                     &m.slot[i], &select_used, &partial_used);
        if (rc != 0) return rc;
    }
    return kv->head_dim == 64 ? launch_multi<64>(ctx->decode_stream, m, n_slots, false)
                              : launch_multi<128>(ctx->decode_stream, m, n_slots, false);
}

int m40llm_ext_block_select_read_selection(M40llmCudaContext* ctx, const M40llmKVCache* kv, uint32_t seq_id,
                                           const void* q_dev_f32, uint32_t q_heads, uint32_t seq_len,
                                           uint32_t recent_window, uint32_t block_size, uint32_t top_blocks,
                                           uint32_t* out_blocks_host, uint32_t* out_counts_host,
                                           float* out_scores_host) {
    if (!out_blocks_host || !out_counts_host) return -1;
    const bool compressed = kv && kv->compressed;
    int rc = common_checks(ctx, kv, seq_id, q_dev_f32, q_heads, seq_len, recent_window, block_size, top_blocks,
                           out_blocks_host, compressed);
    if (rc != 0) return rc;
    BsParams p;
    rc = prepare(ctx, kv, seq_id, q_dev_f32, q_heads, seq_len, recent_window, block_size, top_blocks,
                 nullptr, compressed, &p);
    if (rc != 0) return rc;
    rc = kv->head_dim == 64 ? launch_all<64>(ctx->decode_stream, p, true)
                            : launch_all<128>(ctx->decode_stream, p, true);
    if (rc != 0) return rc;
    if (hipStreamSynchronize(ctx->decode_stream) != hipSuccess) return -9;
    if (hipMemcpy(out_blocks_host, p.sel, (size_t)q_heads * 64 * 4, hipMemcpyDeviceToHost) != hipSuccess) return -9;
    if (hipMemcpy(out_counts_host, p.counts, (size_t)q_heads * 4, hipMemcpyDeviceToHost) != hipSuccess) return -9;
    if (out_scores_host &&
        hipMemcpy(out_scores_host, p.sel_scores, (size_t)q_heads * 64 * 4, hipMemcpyDeviceToHost) != hipSuccess)
        return -9;
    return 0;
}

}  // extern "C"
