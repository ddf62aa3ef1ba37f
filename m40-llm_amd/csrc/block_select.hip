// Block-select "exact old" attention for gfx950: exact recent window + top-k old blocks chosen
// by mean-K block scores, over (a) the fp16-K / q4-V compressed cache and (b) a dense cache.
//
//   1. score  : one wave per (old block, kv head) streams the block's K rows once (128-bit
//               loads), sums them per dimension in f32, and takes the dot of that sum with every
//               q head of the GQA group, so old K is read once per kv head, not once per q head.
//               score = (q . sum_t K[t]) / len * inv_sqrt.
//   2. select : per q head, rank blocks by (score desc, block id asc) and keep the first
//               min(top_blocks, old_blocks) whose score exceeds -1e30: the result of the
//               reference's strict-'>' insertion into a list initialised to -1e30.
//   3. attend : per q head, softmax attention over [tokens of the selected blocks in rank
//               order] ++ [recent window], split into chunks; old V is unpacked from 4 bits in
//               registers (value = nibble * scale, rounded through f16 as the reference does).
//   4. combine: chunk partials merged in ascending order.
//
// Reference: kernel cuda/kernels.cu:2832-3096 (compressed) and :1825-1983 (dense), entry points
// :4504-4577 and :4025-4070.  Only the plain top-k policy and score-rank block order are built.
#include "common.hpp"

#include <cstdlib>
#include <cstring>

namespace {

struct BsParams {
    // K sources: tokens < old_len come from old_k_base (indexed by absolute position); tokens
    // >= old_len from the ring (ring != 0) or from the same dense array.
    const uint16_t* old_k;     // [max_seq_len][kvh][hd] of this sequence
    const uint16_t* new_k;     // ring [W][kvh][hd] of this sequence, or dense K of this sequence
    const uint16_t* dense_v;   // dense V of this sequence (dense backing) or ring V (compressed)
    const uint8_t* q4_v;       // [max_seq_len][kvh][hd/2] of this sequence (compressed only)
    const float* q4_scale;     // [max_seq_len][kvh]
    const float* Q;            // [q_heads][hd]
    float* Out;
    float* scores;             // [q_heads][nblk]
    uint32_t* sel;             // [q_heads][64]
    float* sel_scores;         // [q_heads][64]
    uint32_t* counts;          // [q_heads] selected blocks
    uint32_t* ntok;            // [q_heads] attended tokens
    float* partial;            // [q_heads][nchunks][hd+2]
    uint32_t kv_heads, q_heads, seq_len, recent_window, block_size, top_n;
    uint32_t old_len, nblk, chunk, nchunks, compressed;
};

constexpr int kBsMaxSlots = 8;
// Several independent slots (sequences) per launch: blockIdx.z picks the slot.
struct BsMulti {
    BsParams slot[kBsMaxSlots];
};

// ---- 1. block scores ------------------------------------------------------------------------
template <int HD, int G>
__global__ __launch_bounds__(256) void bs_score_kernel(BsMulti multi) {
    const BsParams& p = multi.slot[blockIdx.z];
    constexpr int C = HD / 8;   // 16-byte chunks per K row
    constexpr int R = 64 / C;   // rows per wave step
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const uint32_t blk = blockIdx.x * 4 + wave;
    if (blk >= p.nblk) return;
    const uint32_t kvh = blockIdx.y;
    const int g = lane / C, c = lane % C;
    const uint32_t start = blk * p.block_size;
    const uint32_t end = start + p.block_size < p.old_len ? start + p.block_size : p.old_len;
    const size_t row_stride = (size_t)p.kv_heads * HD;
    const uint16_t* kb = p.old_k + (size_t)kvh * HD + 8 * c;

    float sum[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) sum[j] = 0.0f;
#pragma unroll 4
    for (uint32_t t = start + g; t < end; t += R) {
        const uint4 kw = m40_load_stream(reinterpret_cast<const uint4*>(kb + (size_t)t * row_stride));
        float kf[8];
        m40_unpack8(kw, kf);
#pragma unroll
        for (int j = 0; j < 8; ++j) sum[j] += kf[j];
    }
    // join the R row groups: lanes with equal c, strides R/2*C ... C
#pragma unroll
    for (int stride = (R / 2) * C; stride >= C; stride >>= 1) {
#pragma unroll
        for (int j = 0; j < 8; ++j) sum[j] += __shfl_xor(sum[j], stride, 64);
    }
    const uint32_t group = p.q_heads / p.kv_heads;
    const float inv_sqrt = HD == 64 ? 0.125f : 0.08838834764831845f;
    const float len = (float)(end - start);
    for (uint32_t h0 = 0; h0 < group; h0 += G) {
#pragma unroll
        for (int h = 0; h < G; ++h) {
            if (h0 + h < group) {
                const uint32_t qh = kvh * group + h0 + h;
                const float* qp = p.Q + (size_t)qh * HD + 8 * c;
                float part = 0.0f;
#pragma unroll
                for (int j = 0; j < 8; ++j) part = fmaf(qp[j], sum[j], part);
                part = C == 8 ? m40_sum8(part) : m40_sum16(part);
                if (lane == 0) p.scores[(size_t)qh * p.nblk + blk] = (part / len) * inv_sqrt;
            }
        }
    }
}

// ---- 2. top-k selection per q head -----------------------------------------------------------
// Rank by counting: block b is at rank #{o : score[o] > score[b] or (== and o < b)}, which is the order the
// reference's strict-'>' insertion produces (cuda/kernels.cu:2980-3022).  Grid (q head, 128 candidates); eight lanes
// share the count of one candidate.  The workgroup that owns the last block also writes the list length, the
// attended-token count and the unused tail of the list.
__global__ __launch_bounds__(1024) void bs_select_kernel(BsMulti multi) {
    const BsParams& p = multi.slot[blockIdx.z];
    extern __shared__ float s_sc[];  // [nblk]
    __shared__ uint32_t s_valid[16];
    __shared__ uint32_t s_last_rank;
    const uint32_t qh = blockIdx.x;
    if (p.nblk == 0) {
        // no old blocks: empty list, the q head attends the recent tokens only
        if (blockIdx.y == 0) {
            for (uint32_t i = threadIdx.x; i < 64u; i += 1024u) {
                p.sel[qh * 64 + i] = 0xffffffffu;
                p.sel_scores[qh * 64 + i] = -1e30f;
            }
            if (threadIdx.x == 0) {
                p.counts[qh] = 0;
                p.ntok[qh] = p.seq_len - p.old_len;
            }
        }
        return;
    }
    const uint32_t parts = (p.nblk + 127u) / 128u;
    if (blockIdx.y >= parts) return;
    const float* sc = p.scores + (size_t)qh * p.nblk;
    uint32_t valid = 0;
    for (uint32_t b = threadIdx.x; b < p.nblk; b += 1024u) {
        const float v = sc[b];
        s_sc[b] = v;
        valid += (v > -1e30f) ? 1u : 0u;       // NaN and anything <= -1e30 never enter the list
    }
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) valid += __shfl_xor(valid, o, 64);
    if ((threadIdx.x & 63u) == 0u) s_valid[threadIdx.x >> 6] = valid;
    if (threadIdx.x == 0) s_last_rank = 0xffffffffu;
    __syncthreads();
    const uint32_t b = blockIdx.y * 128u + (threadIdx.x >> 3), part = threadIdx.x & 7u;
    uint32_t rank = 0;
    float s = 0.0f;
    const bool cand = b < p.nblk;
    if (cand) {
        s = s_sc[b];
        const uint32_t o_begin = (uint32_t)(((uint64_t)part * p.nblk) / 8u), o_end = (uint32_t)(((uint64_t)(part + 1u) * p.nblk) / 8u);
        for (uint32_t o = o_begin; o < o_end; ++o) {
            const float so = s_sc[o];
            rank += (so > s || (so == s && o < b)) ? 1u : 0u;
        }
    }
    rank += __shfl_xor(rank, 1, 64);
    rank += __shfl_xor(rank, 2, 64);
    rank += __shfl_xor(rank, 4, 64);
    const bool listed = cand && part == 0u && (s > -1e30f) && rank < p.top_n;
    if (listed) {
        p.sel[qh * 64 + rank] = b;
        p.sel_scores[qh * 64 + rank] = s;
    }
    if (cand && part == 0u && b + 1u == p.nblk) s_last_rank = listed ? rank : 0xffffffffu;
    __syncthreads();
    if (blockIdx.y == parts - 1u) {
        uint32_t total_valid = 0;
        for (int w = 0; w < 16; ++w) total_valid += s_valid[w];
        const uint32_t count = total_valid < p.top_n ? total_valid : p.top_n;
        for (uint32_t i = count + threadIdx.x; i < 64u; i += 1024u) {
            p.sel[qh * 64 + i] = 0xffffffffu;
            p.sel_scores[qh * 64 + i] = -1e30f;
        }
        if (threadIdx.x == 0) {
            uint32_t tokens = count * p.block_size;
            if (s_last_rank != 0xffffffffu) tokens -= p.nblk * p.block_size - p.old_len;   // the last block may be partial
            p.counts[qh] = count;
            p.ntok[qh] = tokens + (p.seq_len - p.old_len);
        }
    }
}

// ---- 3. attention over the token list ---------------------------------------------------------
// Grid (q head, chunk of 128 list positions).  Eight waves; every lane issues the K and V loads of all of its token
// rows before any arithmetic (one memory round trip per workgroup), scores stay in registers.
constexpr int kBsChunk = 128;
template <int HD>
__global__ __launch_bounds__(512) void bs_attend_kernel(BsMulti multi) {
    const BsParams& p = multi.slot[blockIdx.z];
    constexpr int LPT = HD / 8, TPW = 64 / LPT, kWaves = 8;
    constexpr int S = kBsChunk / (kWaves * TPW);
    __shared__ uint32_t pre[65], sel_s[64];
    __shared__ float red[kWaves][HD];
    __shared__ float wmax[kWaves], wsum[kWaves];

    const uint32_t qh = blockIdx.x;
    const uint32_t n = p.ntok[qh];
    const uint32_t cbeg = blockIdx.y * kBsChunk;
    if (cbeg >= n) return;
    const uint32_t cend = cbeg + kBsChunk < n ? cbeg + kBsChunk : n;
    const uint32_t count = p.counts[qh];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;

    // pre[r] = first list position of the r-th selected block (exclusive prefix of the block lengths); sel_s[r] = its id
    if (wave == 0) {
        uint32_t len = 0, b = 0;
        if ((uint32_t)lane < count) {
            b = p.sel[qh * 64 + lane];
            const uint32_t start = b * p.block_size;
            const uint32_t end = start + p.block_size < p.old_len ? start + p.block_size : p.old_len;
            len = end - start;
        }
        uint32_t incl = len;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const uint32_t up = __shfl_up(incl, o, 64);
            if (lane >= o) incl += up;
        }
        pre[lane] = incl - len;
        sel_s[lane] = b;
        if (lane == 63) pre[64] = incl;
    }
    __syncthreads();
    const uint32_t old_tokens = pre[64];

    const uint32_t kvh = qh / (p.q_heads / p.kv_heads);
    const int c = lane % LPT, tg = lane / LPT;
    const size_t row_stride = (size_t)p.kv_heads * HD;
    const float inv_sqrt = HD == 64 ? 0.125f : 0.08838834764831845f;

    // Every list position of the chunk is turned into a token first (no memory access: the block table is in LDS),
    // then all K / V / q4 / scale loads of the thread go out together with no branch around any of them: positions
    // past the end repeat the last one, and the load that a token does not need reads a valid dummy address.
    uint4 kw[S], vw[S];
    uint32_t qw[S];
    float qs[S];
    bool valid[S], quant[S];
    uint32_t tok[S], ring[S];
    const uint32_t ring_mod = p.compressed ? p.recent_window : 0xffffffffu;     // t % 0xffffffff = t: dense cache rows
#pragma unroll
    for (int s = 0; s < S; ++s) {
        uint32_t pos = cbeg + (uint32_t)((s * kWaves + wave) * TPW + tg);
        valid[s] = pos < cend;
        pos = valid[s] ? pos : cend - 1u;
        uint32_t lo = 0;                              // largest r < count with pre[r] <= pos (pre[0] = 0)
#pragma unroll
        for (uint32_t step = 32; step >= 1u; step >>= 1) {
            const uint32_t mid = lo + step;
            const uint32_t pm = pre[mid < 64u ? mid : 63u];
            const bool take = (mid < count) & (pm <= pos);
            lo = take ? mid : lo;
        }
        const uint32_t t_old = sel_s[lo] * p.block_size + (pos - pre[lo]);
        tok[s] = pos >= old_tokens ? p.old_len + (pos - old_tokens) : t_old;
        ring[s] = tok[s] % ring_mod;
    }
#pragma unroll
    for (int s = 0; s < S; ++s) {
        const uint32_t t = tok[s];
        const bool old = t < p.old_len;
        const size_t ring_off = (size_t)ring[s] * row_stride;
        const uint16_t* kp = (old ? p.old_k + (size_t)t * row_stride : p.new_k + ring_off) + (size_t)kvh * HD + 8 * c;
        quant[s] = p.compressed && old;
        const uint16_t* vp = quant[s] ? kp : p.dense_v + ring_off + (size_t)kvh * HD + 8 * c;
        const uint32_t* q4p = quant[s]
            ? reinterpret_cast<const uint32_t*>(p.q4_v + ((size_t)t * p.kv_heads + kvh) * (HD / 2) + 4 * c)
            : reinterpret_cast<const uint32_t*>(kp);
        const float* scp = quant[s] ? p.q4_scale + (size_t)t * p.kv_heads + kvh : reinterpret_cast<const float*>(kp);
        kw[s] = *reinterpret_cast<const uint4*>(kp);
        vw[s] = *reinterpret_cast<const uint4*>(vp);
        qw[s] = *q4p;
        qs[s] = *scp;
    }
    float q[8];
    {
        const float4 q0 = *reinterpret_cast<const float4*>(p.Q + (size_t)qh * HD + 8 * c);
        const float4 q1 = *reinterpret_cast<const float4*>(p.Q + (size_t)qh * HD + 8 * c + 4);
        q[0] = q0.x; q[1] = q0.y; q[2] = q0.z; q[3] = q0.w; q[4] = q1.x; q[5] = q1.y; q[6] = q1.z; q[7] = q1.w;
    }
    float sc[S];
    float lmax = -INFINITY;
#pragma unroll
    for (int s = 0; s < S; ++s) {
        float kf[8];
        m40_unpack8(kw[s], kf);
        float d = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) d = fmaf(q[j], kf[j], d);
        d = LPT == 8 ? m40_sum8(d) : m40_sum16(d);
        sc[s] = valid[s] ? d * inv_sqrt : -INFINITY;
        lmax = fmaxf(lmax, sc[s]);
    }
    lmax = m40_max64(lmax);
    if (lane == 0) wmax[wave] = lmax;
    __syncthreads();
    float m = wmax[0];
#pragma unroll
    for (int w = 1; w < kWaves; ++w) m = fmaxf(m, wmax[w]);

    float lsum = 0.0f;
    float acc[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = 0.0f;
#pragma unroll
    for (int s = 0; s < S; ++s) {
        const float e = valid[s] ? expf(sc[s] - m) : 0.0f;
        if (c == 0) lsum += e;
        float vf[8];
        if (quant[s]) {
            const uint32_t packed = qw[s];
            const float scale = qs[s];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int nib = (int)((packed >> (4 * j)) & 0xfu);
                const int sv = nib >= 8 ? nib - 16 : nib;
                vf[j] = m40_h2f(m40_f2h((float)sv * scale));       // the reference rounds the product through f16
            }
        } else {
            m40_unpack8(vw[s], vf);
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[j] = fmaf(e, vf[j], acc[j]);
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        float v = acc[j];
#pragma unroll
        for (int o = LPT; o < 64; o <<= 1) v += __shfl_xor(v, o, 64);
        acc[j] = v;
    }
    lsum = m40_sum64(lsum);
    if (lane == 0) wsum[wave] = lsum;
    if (tg == 0) {
#pragma unroll
        for (int j = 0; j < 8; ++j) red[wave][8 * c + j] = acc[j];
    }
    __syncthreads();
    if (tid < HD) {
        float v = 0.0f, l = 0.0f;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) {
            v += red[w][tid];
            l += wsum[w];
        }
        if (p.nchunks == 1) {
            p.Out[(size_t)qh * HD + tid] = v / (l > 0.0f ? l : 1.0f);
        } else {
            float* w = p.partial + ((size_t)qh * p.nchunks + blockIdx.y) * (HD + 2);
            w[2 + tid] = v;
            if (tid == 0) { w[0] = m; w[1] = l; }
        }
    }
}

// Merge the chunk partials of one q head: 1024 threads = 1024/HD chunk lanes x HD dims, each lane folds chunks
// lane, lane + n_lanes, ... with a running maximum; the lanes are then folded in order.
template <int HD>
__global__ __launch_bounds__(1024) void bs_combine_kernel(BsMulti multi) {
    const BsParams& p = multi.slot[blockIdx.z];
    if (p.nchunks <= 1) return;      // the attend kernel wrote the output itself
    constexpr int NCG = 1024 / HD;
    __shared__ float s_m[NCG], s_den[NCG];
    __shared__ float s_num[NCG][HD];
    const uint32_t qh = blockIdx.x, d = threadIdx.x % HD, cg = threadIdx.x / HD;
    const uint32_t n = (p.ntok[qh] + kBsChunk - 1) / kBsChunk;
    if (n == 0) return;
    const float* w = p.partial + (size_t)qh * p.nchunks * (HD + 2);
    float m = -INFINITY, num = 0.0f, den = 0.0f;
    for (uint32_t ch = cg; ch < n; ch += NCG) {
        const float* wc = w + (size_t)ch * (HD + 2);
        const float mc = wc[0], lc = wc[1], vc = wc[2 + d];
        const float nm = fmaxf(m, mc);
        const float fa = m == -INFINITY ? 0.0f : expf(m - nm);
        const float fb = mc == -INFINITY ? 0.0f : expf(mc - nm);
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
            const float nm = fmaxf(m, mc);
            const float fa = m == -INFINITY ? 0.0f : expf(m - nm);
            const float fb = mc == -INFINITY ? 0.0f : expf(mc - nm);
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
    p->Q = static_cast<const float*>(q);
    p->Out = static_cast<float*>(out);
    if (compressed) {
        p->old_k = kv->d_fp16_old_k + (size_t)seq_id * kv->max_seq_len * ept;
        p->new_k = kv->d_recent_k + (size_t)seq_id * kv->recent_window * ept;
        p->dense_v = kv->d_recent_v + (size_t)seq_id * kv->recent_window * ept;
        p->q4_v = kv->d_q4_old_v + (size_t)seq_id * kv->max_seq_len * kvh * (hd / 2u);
        p->q4_scale = kv->d_q4_old_v_scale + (size_t)seq_id * kv->max_seq_len * kvh;
    } else {
        p->old_k = kv->d_k + (size_t)seq_id * kv->max_seq_len * ept;
        p->new_k = p->old_k;
        p->dense_v = kv->d_v + (size_t)seq_id * kv->max_seq_len * ept;
    }
    M40StreamScratch& sc = ctx->scratch[1];
    // select scratch: scores | sel | sel_scores | counts | ntok
    const size_t scores_bytes = ((size_t)q_heads * (nblk ? nblk : 1) * 4 + 255) & ~(size_t)255;
    const size_t fixed = (size_t)q_heads * (64 * 4 + 64 * 4 + 4 + 4) + 1024;
    const size_t select_need = (scores_bytes + fixed + 255) & ~(size_t)255;
    if (select_off + select_need > sc.select_bytes) return -7;
    char* base = static_cast<char*>(sc.select) + select_off;
    p->scores = reinterpret_cast<float*>(base);
    p->sel = reinterpret_cast<uint32_t*>(base + scores_bytes);
    p->sel_scores = reinterpret_cast<float*>(p->sel + (size_t)q_heads * 64);
    p->counts = reinterpret_cast<uint32_t*>(p->sel_scores + (size_t)q_heads * 64);
    p->ntok = p->counts + q_heads;
    const uint32_t chunk = kBsChunk;
    p->chunk = chunk;
    p->nchunks = (capacity + chunk - 1) / chunk;
    const size_t partial_need = (((size_t)q_heads * p->nchunks * (hd + 2) * 4) + 255) & ~(size_t)255;
    if (partial_off + partial_need > sc.attn_partial_bytes) return -7;
    p->partial = reinterpret_cast<float*>(static_cast<char*>(sc.attn_partial) + partial_off);
    if (select_used) *select_used = select_off + select_need;
    if (partial_used) *partial_used = partial_off + partial_need;
    if ((size_t)nblk * 4 > 60 * 1024) return -7;  // block scores of one q head live in LDS
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
        dim3 grid((max_nblk + 3) / 4, p0.kv_heads, n);
        if (group >= 4) bs_score_kernel<HD, 4><<<grid, 256, 0, s>>>(m);
        else if (group >= 2) bs_score_kernel<HD, 2><<<grid, 256, 0, s>>>(m);
        else bs_score_kernel<HD, 1><<<grid, 256, 0, s>>>(m);
    }
    bs_select_kernel<<<dim3(p0.q_heads, max_nblk ? (max_nblk + 127) / 128 : 1, n), 1024, (size_t)(max_nblk ? max_nblk : 1) * 4, s>>>(m);
    if (!selection_only) {
        bs_attend_kernel<HD><<<dim3(p0.q_heads, max_chunks, n), 512, 0, s>>>(m);
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
