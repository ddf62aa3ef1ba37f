// Packed variable-length causal prefill attention for gfx950, f32 in and out (the step before decode).
//
// Q and Out are [total_q][q_heads][hd], K and V [total_kv][kv_heads][hd]; sequence b owns q_lens[b] query tokens from
// q_offsets[b] and kv_lens[b] keys from kv_offsets[b]; query q_idx attends keys 0 .. kv_len - q_len + q_idx.
//
// The reference walks every key once per (query, head) with one workgroup each (cuda/kernels.cu:3749-3835).  Here a
// workgroup owns 64 or 128 consecutive queries of one q head (four waves x one or two blocks of 16 queries) and streams
// the sequence's keys in tiles of 32 or 64 through LDS, so a key row is fetched once per 64 / 128 queries.  Both products run on v_mfma_f32_16x16x32_f16
// with every f32 operand split exactly into an f16 high and an f16 low part (x = hi + lo to 2^-22): a product is
// three instructions, hi hi + lo hi + hi lo (the lo lo term is below 2^-22 of the operands' magnitudes), which is
// five times the rate of the f32 matrix instruction for the same product at f32-level accuracy:
//   scores  S[query][key] = sum_d Q[query][d] K[key][d]   A = Q (two f16 parts, in registers for the whole kernel),
//           B = K tile (two f16 planes in LDS)
//   output  O[query][d]  += sum_key P[query][key] V[key][d]
// Both are formed transposed (S^T = K Q^T, O^T = V^T P^T) with the tile's keys ordered along the second product's k
// dimension the way the first product's accumulators hold them, so the softmax weights go from one matrix instruction
// into the next inside the lane (no LDS round trip), and maximum, sum and rescaling factor are one value per lane.
// V is stored transposed [d][key slot] so that a lane's eight key slots are one 16-byte read.
// The softmax is online, with a reference point per query in place of the running maximum: weights are
// exp2(x - n) with n within 8 (log2 units) of the largest score so far, moved only when a tile holds a larger one
// (the rows of a lane's accumulators are the same four queries in both products, so the rescaling needs no exchange).
// The result is the same softmax as the reference's three passes (p = exp(s - max) / sum), within f32 rounding.
// Two waves share a SIMD; a wave raises its priority for its matrix-instruction phases, so that the matrix pipe is
// fed first and the other wave's vector work (exponentials, splits) fills the issue slots in between
// (0.283 -> 0.252 ms for one 4096-token sequence at head_dim 64).  Operands beyond the f16 range (|x| > 65504) are not supported by the
// split (none occur after RMSNorm-scaled projections; the decode-side attention has no such limit).
//
// Reference: kernel cuda/kernels.cu:3749-3835; entry points, argument checks and their codes :4834-4977
// (lengths are read back to the host and validated before the launch, also in the _async form).
#include "common.hpp"

#include <vector>

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = 4;
// 16-query blocks per wave: a K / V fragment read from LDS serves every block of the wave.  Two blocks where long
// sequences alone fill the chip four workgroups deep, one otherwise -- two blocks halve the workgroup count and double
// the masked share of a short sequence's diagonal tiles.  One against two blocks, head_dim 128 at 16 / 32 q heads:
// 1 x 4096 tokens 0.30 / 0.33 and 0.63 / 0.53 ms, 4 x 4096 1.17 / 1.02 and 2.13 / 1.85 ms, 16 x 300 0.069 / 0.077 and
// 0.099 / 0.112 ms; head_dim 64 at 32 q heads: 1 x 1024 48 / 52 us, 1 x 2048 94 / 102 us, 16 x 300 59 / 69 us,
// 1 x 4096 0.260 / 0.240 ms, 2 x 4096 0.58 / 0.51 ms.
constexpr float kRefSlack = 8.0f;          // log2 units: weights stay below 256
constexpr uint32_t kTwoBlockMinQueries = 2048;      // a sequence counts as long from here
constexpr int kTwoBlockMinGroupsPerCu = 4;
// keys per LDS tile (KT below): one or two k-steps of the P . V product; 64 where two planes of K and V^T fit the
// static LDS limit (head_dim 64), 32 otherwise
constexpr int key_tile_of(int hd) { return hd == 64 ? 64 : 32; }

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ m40_float4 mfma32(half8 a, half8 b, m40_float4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}
// Issue order of a phase of STEPS steps, each two 16-byte LDS fragment reads and PER matrix instructions that use them:
// the reads run AHEAD steps in front of their instructions (left to itself the compiler reuses one register pair and
// waits for every read right after issuing it).
template <int STEPS, int PER, int AHEAD = 1>
__device__ __forceinline__ void fragment_pipeline() {
    __builtin_amdgcn_sched_group_barrier(0x100, 2 * (AHEAD < STEPS ? AHEAD : STEPS), 0);
#pragma unroll
    for (int i = 0; i < STEPS; ++i) {
        if (i + AHEAD < STEPS) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, PER, 0);
    }
}
// x = hi + lo with both parts f16: exact to about 2^-22 relative for values inside the f16 range
__device__ __forceinline__ void split(float x, _Float16* hi, _Float16* lo) {
    const _Float16 h = static_cast<_Float16>(x);
    *hi = h;
    *lo = static_cast<_Float16>(x - static_cast<float>(h));
}

struct PrefillArgs {
    const float* Q; const float* K; const float* V; float* Out;
    const _Float16* planes;     // per padded 32-key tile and kv head: K hi [32][HD], K lo, V^T hi [HD][32], V^T lo
    uint32_t plane_tiles;       // padded tiles in total (sequence b starts at tile kv_offsets[b] / 32 + b ... see pack)
    const uint32_t* q_offsets; const uint32_t* kv_offsets; const uint32_t* q_lens; const uint32_t* kv_lens;
    uint32_t q_heads, kv_heads;
};

// Order of a tile's 32 keys along the k dimension of the P . V product: k-slot 8 g + i holds key 4 g + i (i < 4) or
// key 16 + 4 g + (i - 4): exactly the eight keys whose scores lane group g holds after the two score products, so the
// weights go from the score accumulators into the next product's operand without leaving the lane.
__device__ __forceinline__ int key_of_slot(int slot) {
    const int base = slot & ~31, g = (slot & 31) >> 3, i = slot & 7;      // every 32 slots: one k-step over 32 keys
    return base + (i < 4 ? 4 * g + i : 16 + 4 * g + (i - 4));
}

// First padded tile of sequence b in the packed planes: every sequence starts on a tile boundary of its own, so a
// sequence gets one tile of slack (rows_before / 32 rounded down, plus b).
__device__ __forceinline__ uint32_t first_tile_of(uint32_t kv_offset, uint32_t b, uint32_t key_tile) { return kv_offset / key_tile + b; }

// K and V of one 32-key tile and kv head -> two f16 planes each, V transposed, in the order the attention kernel copies
// them to LDS.  Done once per call so that the 64-query workgroups (and the q heads of a group) do not each repeat the
// split.  Keys past the sequence end are written as zeros (they are masked anyway).
template <int HD>
__global__ __launch_bounds__(kThreads) void prefill_pack_kv_kernel(PrefillArgs p) {
    constexpr int kKTile = key_tile_of(HD);
    __shared__ float vt[kKTile][HD + 1];
    const uint32_t b = blockIdx.z, kvh = blockIdx.y, tile = blockIdx.x;
    const uint32_t kv_len = p.kv_lens[b];
    if (tile * kKTile >= kv_len) return;
    const float* Kb = p.K + ((size_t)p.kv_offsets[b] * p.kv_heads + kvh) * HD;
    const float* Vb = p.V + ((size_t)p.kv_offsets[b] * p.kv_heads + kvh) * HD;
    const size_t row_stride = (size_t)p.kv_heads * HD;
    _Float16* out = const_cast<_Float16*>(p.planes) + ((size_t)(first_tile_of(p.kv_offsets[b], b, kKTile) + tile) * p.kv_heads + kvh) * (4 * kKTile * HD);
    _Float16* kh = out, *kl = out + kKTile * HD, *vh = out + 2 * kKTile * HD, *vl = out + 3 * kKTile * HD;
    for (int e = threadIdx.x; e < kKTile * HD; e += kThreads) {
        const int key_in = e / HD, d = e % HD;
        const uint32_t key = tile * kKTile + key_in;
        const bool live = key < kv_len;
        const float kx = live ? Kb[(size_t)key * row_stride + d] : 0.0f;
        vt[key_in][d] = live ? Vb[(size_t)key * row_stride + d] : 0.0f;
        _Float16 a, c;
        split(kx, &a, &c);
        kh[e] = a;
        kl[e] = c;
    }
    __syncthreads();
    for (int e = threadIdx.x; e < kKTile * HD; e += kThreads) {
        const int d = e / kKTile, slot = e % kKTile;
        _Float16 a, c;
        split(vt[key_of_slot(slot)][d], &a, &c);
        vh[e] = a;
        vl[e] = c;
    }
}

// QB: 16-query blocks per wave.  With two, every K and V fragment a wave reads from LDS serves 32 queries instead of 16:
// the kernel's LDS traffic (each wave reads the whole K and V tile) was what it spent most of its time on.
template <int HD, int QB>
__global__ __launch_bounds__(kThreads) void prefill_attn_kernel(PrefillArgs p) {
    constexpr int kKTile = key_tile_of(HD);
    constexpr int KB = kKTile / 16;        // 16-key score blocks of a tile
    constexpr int KS = HD / 32;            // matrix-instruction k-steps of a score tile
    constexpr int DT = HD / 16;            // 16-column output tiles
    constexpr int KSTR = HD + 8;           // LDS halves per K row: 16-byte fragment reads of 16 keys hit 64 distinct banks
    constexpr int VSTR = kKTile + 8;       // LDS halves per row of the transposed V tile [column][key]
    constexpr int kQWave = 16 * QB;        // queries of a wave
    constexpr int kQGroup = kQWave * kWaves;
    // Two forms of the tile body, by measurement (one 4096-token sequence at 32 heads / eight sequences at 16 heads):
    // head_dim 64 skips a first block that a tile lies wholly behind (branches around its matrix instructions) and
    // leaves the order of fragment reads and matrix instructions to the compiler; head_dim 128 computes such a block
    // masked and orders reads one step ahead of their instructions.  The other way round costs 5-6 % at either size.
    constexpr bool kSkip = QB > 1 && HD == 64, kPipe = HD == 128;
    __shared__ __attribute__((aligned(16))) _Float16 k_lds[2][kKTile * KSTR];   // [hi, lo][key][d]
    __shared__ __attribute__((aligned(16))) _Float16 v_lds[2][HD * VSTR];       // [hi, lo][d][key]

    // Workgroups are dispatched in index order, x fastest: x = q head, y = query tile from the end of the sequence,
    // z = sequence (ordering the tiles of all sequences together by key count measured slower: the sequences' keys
    // then compete for the caches).
    // The tiles with the most keys (the longest workgroups) of every head start first and the short ones fill the
    // tail; with the head as the slow index the last heads' long tiles started near the end of the kernel and the
    // chip ran at a third of its occupancy.  Neighbouring workgroups are the q heads of one kv group on the same keys.
    const uint32_t b = blockIdx.z, h = blockIdx.x;
    const uint32_t q_len = p.q_lens[b], kv_len = p.kv_lens[b];
    const uint32_t q0 = (gridDim.y - 1u - blockIdx.y) * kQGroup;
    if (q0 >= q_len || q_len > kv_len) return;
    const uint32_t kvh = h / (p.q_heads / p.kv_heads);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);       // as a scalar: tests on it branch without masks
    const int j = lane & 15, g = lane >> 4;
    const float inv_sqrt = HD == 64 ? 0.125f : 0.08838834764831845f;
    const uint32_t shift = kv_len - q_len;                        // query q attends keys 0 .. shift + q
    const uint32_t wg_last_q = q0 + kQGroup - 1 < q_len - 1 ? q0 + kQGroup - 1 : q_len - 1;
    const uint32_t n_tiles = (shift + wg_last_q) / kKTile + 1;    // key tiles this workgroup walks

    // ---- this wave's query blocks: A operand of the score product, lane (query j, k group g) of block qb holds
    //      Q[j][32 s + 8 g .. + 7] as a high and a low f16 part
    const uint32_t wq0 = q0 + (uint32_t)kQWave * wave;            // first query of the wave
    const bool wave_live = wq0 < q_len;
    uint32_t row_end[QB];                                         // last key this lane's query of the block sees
    uint32_t blk_end[QB];                                         // last key any query of the block sees
    half8 qh[QB][KS], ql[QB][KS];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
        const uint32_t bq0 = wq0 + 16u * qb;
        const uint32_t my_q = bq0 + j < q_len ? bq0 + j : q_len - 1;      // a query past the end repeats the last one (not stored)
        row_end[qb] = shift + my_q;
        blk_end[qb] = shift + (bq0 + 15u < q_len ? bq0 + 15u : q_len - 1);
        const float* qp = p.Q + ((size_t)(p.q_offsets[b] + my_q) * p.q_heads + h) * HD + 8 * g;
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            const float4 x0 = *reinterpret_cast<const float4*>(qp + 32 * s), x1 = *reinterpret_cast<const float4*>(qp + 32 * s + 4);
            const float x[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                _Float16 a, c;
                split(x[i], &a, &c);
                qh[qb][s][i] = a;
                ql[qb][s][i] = c;
            }
        }
    }
    const uint32_t wave_first_end = shift + (wq0 < q_len ? wq0 : q_len - 1);          // last key the wave's first query sees
    const uint32_t wave_end = blk_end[QB - 1];                                        // last key any query of the wave sees

    // ---- K / V tile loads: 16-byte pieces of the packed f16 planes (prefill_pack_kv_kernel), straight into LDS
    constexpr int PIECES = kKTile * HD / 8 / kThreads;           // per plane and thread: 1 (HD 64) or 2 (HD 128)
    const _Float16* tile_base = p.planes + ((size_t)first_tile_of(p.kv_offsets[b], b, kKTile) * p.kv_heads + kvh) * (4 * kKTile * HD);
    const size_t tile_stride = (size_t)p.kv_heads * (4 * kKTile * HD);
    uint4 kreg[2][PIECES], vreg[2][PIECES];
    auto issue = [&](uint32_t tile) {
        const _Float16* t = tile_base + (size_t)tile * tile_stride;
#pragma unroll
        for (int u = 0; u < PIECES; ++u) {
            const int c = u * kThreads + tid;
#pragma unroll
            for (int pl = 0; pl < 2; ++pl) {
                kreg[pl][u] = *reinterpret_cast<const uint4*>(t + pl * kKTile * HD + 8 * c);
                vreg[pl][u] = *reinterpret_cast<const uint4*>(t + (2 + pl) * kKTile * HD + 8 * c);
            }
        }
    };
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    auto to_lds = [&]() {
#pragma unroll
        for (int u = 0; u < PIECES; ++u) {
            const int c = u * kThreads + tid;
            const int key_in = c / (HD / 8), kpart = c % (HD / 8);     // K plane [key][HD]
            const int d = c / (kKTile / 8), vpart = c % (kKTile / 8);  // V^T plane [d][32 keys]
#pragma unroll
            for (int pl = 0; pl < 2; ++pl) {
                *reinterpret_cast<u32x4*>(&k_lds[pl][key_in * KSTR + 8 * kpart]) = u32x4{kreg[pl][u].x, kreg[pl][u].y, kreg[pl][u].z, kreg[pl][u].w};
                *reinterpret_cast<u32x4*>(&v_lds[pl][d * VSTR + 8 * vpart]) = u32x4{vreg[pl][u].x, vreg[pl][u].y, vreg[pl][u].z, vreg[pl][u].w};
            }
        }
    };
    issue(0);

    // Products are formed transposed, S^T = K Q^T and O^T = V^T P^T, so that a lane (query j, group g) ends up with the
    // scores of ONE query for keys 4 g .. 4 g + 3 of both 16-key blocks, which are the k-slots 8 g .. 8 g + 7 of the
    // second product (key_of_slot): the weights never pass through LDS, and the running maximum, the sum and the
    // rescaling factor are one value per lane and query block.
    float m_run[QB], l_run[QB];              // maximum over the query's keys so far (equal in its four lanes); this lane's share of the sum
    m40_float4 O[QB][DT];                    // O^T[16 d + 4 g + r][query j] of the block
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
        m_run[qb] = -INFINITY;
        l_run[qb] = 0.0f;
#pragma unroll
        for (int d = 0; d < DT; ++d) O[qb][d] = m40_float4{0.f, 0.f, 0.f, 0.f};
    }
    const float scale_log2 = inv_sqrt * 1.4426950408889634f;     // scores in units of log2: weights are exp2(x - max)

    for (uint32_t tile = 0; tile < n_tiles; ++tile) {
        __syncthreads();                  // the previous tile has been read by every wave
        to_lds();
        __syncthreads();
        if (tile + 1 < n_tiles) issue(tile + 1);
        const uint32_t key0 = tile * kKTile;
        if (!wave_live || key0 > wave_end) continue;              // nothing of this tile is visible to the wave
        // a block whose queries all end before this tile (only the first can: later queries see more, and at most one
        // tile per wave).  Computing it all the same changes nothing: every score is masked, and the weights are
        // exp2(-inf - m) = 0 with the finite reference point that tile 0 has left (key 0 is visible to every query).
        bool blk_on[QB];
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) blk_on[qb] = !kSkip || key0 <= blk_end[qb];
        // S^T of the tile's 16-key blocks: lane (query j, g) gets keys 16 kb + 4 g + r.  k . q = kh qh + kh ql + kl qh
        // (the kl ql term is below 2^-22 of |q| |k|); a K fragment read serves every query block of the wave
        m40_float4 sc[QB][KB];
#pragma unroll
        for (int qb = 0; qb < QB; ++qb)
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) sc[qb][kb] = m40_float4{0.f, 0.f, 0.f, 0.f};
        __builtin_amdgcn_s_setprio(1);
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            const int off = 32 * s + 8 * g;
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) {
                const half8 kh = *reinterpret_cast<const half8*>(&k_lds[0][(16 * kb + j) * KSTR + off]);
                const half8 kl = *reinterpret_cast<const half8*>(&k_lds[1][(16 * kb + j) * KSTR + off]);
#pragma unroll
                for (int qb = 0; qb < QB; ++qb) {
                    if (kSkip && !blk_on[qb]) continue;
                    sc[qb][kb] = mfma32(kh, qh[qb][s], sc[qb][kb]);
                    sc[qb][kb] = mfma32(kh, ql[qb][s], sc[qb][kb]);
                    sc[qb][kb] = mfma32(kl, qh[qb][s], sc[qb][kb]);
                }
            }
        }
        if (kPipe) fragment_pipeline<KS * KB, 3 * QB>();
        __builtin_amdgcn_s_setprio(0);
        const bool whole = key0 + (uint32_t)kKTile - 1u <= wave_first_end;      // every key of the tile visible to every query
        half8 ph[QB][KB / 2], pl[QB][KB / 2];       // k-step t: slots 8 g + i = blocks 2 t (i < 4) and 2 t + 1 (i >= 4)
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) {
            if (kSkip && !blk_on[qb]) continue;
            float x[4 * KB];
            float mx = -INFINITY;
            if (whole) {                      // the usual tile (a uniform branch): no per-key comparison
#pragma unroll
                for (int kb = 0; kb < KB; ++kb)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        x[4 * kb + r] = sc[qb][kb][r] * scale_log2;
                        mx = fmaxf(mx, x[4 * kb + r]);
                    }
            } else {
#pragma unroll
                for (int kb = 0; kb < KB; ++kb)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const bool visible = key0 + 16u * kb + 4u * g + r <= row_end[qb];
                        x[4 * kb + r] = visible ? sc[qb][kb][r] * scale_log2 : -INFINITY;
                        mx = fmaxf(mx, x[4 * kb + r]);
                    }
            }
            // The weights are exp2(x - n) for a reference point n per query that need not be the maximum: any n within
            // kRefSlack of it keeps the weights below 2^kRefSlack, far inside the range of the f16 split, and the softmax
            // is the same.  The reference point moves (cross-lane maximum, rescaling of the sum and the accumulators)
            // only when some lane of the wave sees a score more than kRefSlack above its query's: after the first tiles
            // of a sequence that is rare, and the usual tile has no cross-lane exchange between its two products.
            float n = m_run[qb];
            if (__any(mx > n + kRefSlack)) {
                mx = fmaxf(mx, __shfl_xor(mx, 16));
                mx = fmaxf(mx, __shfl_xor(mx, 32));
                n = fmaxf(n, mx);
                // no reference point yet: the old state weighs nothing
                const float f = m_run[qb] == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(m_run[qb] - n);
                l_run[qb] *= f;
#pragma unroll
                for (int d = 0; d < DT; ++d)
#pragma unroll
                    for (int r = 0; r < 4; ++r) O[qb][d][r] *= f;
                m_run[qb] = n;
            }
            float psum = 0.0f;
#pragma unroll
            for (int i = 0; i < 4 * KB; i += 2) {
                // two weights at a time: the packed f32 -> f16 conversion of gfx950 halves the conversion instructions
                const f32x2 pv = {__builtin_amdgcn_exp2f(x[i] - n), __builtin_amdgcn_exp2f(x[i + 1] - n)};   // a masked key: exp2(-inf) = 0
                psum += pv.x + pv.y;
                const half2v a = __builtin_convertvector(pv, half2v);
                const half2v c = __builtin_convertvector(pv - __builtin_convertvector(a, f32x2), half2v);
                ph[qb][i >> 3][i & 7] = a.x; ph[qb][i >> 3][(i & 7) + 1] = a.y;
                pl[qb][i >> 3][i & 7] = c.x; pl[qb][i >> 3][(i & 7) + 1] = c.y;
            }
            l_run[qb] += psum;
        }
        // O^T += V^T . P^T, 32 keys per k-step: A = V^T[column 16 d + j][k-slots 32 t + 8 g .. + 7], B = this lane's
        // eight weights of the step;  v p = vh ph + vh pl + vl ph; a V fragment read serves every query block
        __builtin_amdgcn_s_setprio(1);
#pragma unroll
        for (int d = 0; d < DT; ++d) {
#pragma unroll
            for (int t = 0; t < KB / 2; ++t) {
                const half8 vh = *reinterpret_cast<const half8*>(&v_lds[0][(16 * d + j) * VSTR + 32 * t + 8 * g]);
                const half8 vl = *reinterpret_cast<const half8*>(&v_lds[1][(16 * d + j) * VSTR + 32 * t + 8 * g]);
#pragma unroll
                for (int qb = 0; qb < QB; ++qb) {
                    if (kSkip && !blk_on[qb]) continue;
                    O[qb][d] = mfma32(vh, ph[qb][t], O[qb][d]);
                    O[qb][d] = mfma32(vh, pl[qb][t], O[qb][d]);
                    O[qb][d] = mfma32(vl, ph[qb][t], O[qb][d]);
                }
            }
        }
        if (kPipe) fragment_pipeline<DT * (KB / 2), 3 * QB>();
        __builtin_amdgcn_s_setprio(0);
    }

    // ---- out = O / sum: this lane holds columns 16 d + 4 g .. + 3 of its query
    if (!wave_live) return;
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
        float l = l_run[qb] + __shfl_xor(l_run[qb], 16);
        l += __shfl_xor(l, 32);
        const float denom = l > 0.0f ? l : 1.0f;
        const uint32_t q = wq0 + 16u * qb + (uint32_t)j;
        if (q < q_len) {
            float* op = p.Out + ((size_t)(p.q_offsets[b] + q) * p.q_heads + h) * HD + 4 * g;
#pragma unroll
            for (int d = 0; d < DT; ++d)
                *reinterpret_cast<float4*>(op + 16 * d) =
                    make_float4(O[qb][d][0] / denom, O[qb][d][1] / denom, O[qb][d][2] / denom, O[qb][d][3] / denom);
        }
    }
}

int prefill_impl(M40llmCudaContext* ctx, const void* q, const void* k, const void* v, const uint32_t* q_offsets,
                 const uint32_t* kv_offsets, const uint32_t* q_lens, const uint32_t* kv_lens, uint32_t batch,
                 uint32_t q_heads, uint32_t kv_heads, uint32_t head_dim, void* out, bool synchronize,
                 const uint32_t* kv_offsets_host = nullptr, const uint32_t* q_lens_host = nullptr,
                 const uint32_t* kv_lens_host = nullptr) {
    if (!ctx || !q || !k || !v || !q_offsets || !kv_offsets || !q_lens || !kv_lens || !out) return -1;
    if (batch == 0) return -2;
    if (q_heads == 0 || kv_heads == 0 || q_heads % kv_heads != 0) return -3;
    if (head_dim != 64 && head_dim != 128) return -9;
    // the lengths are validated on the host before the launch, as the reference does (also in the _async form); a caller
    // that holds the tables on the host passes them and spares the three blocking read-backs (each one drains the device)
    const bool host_tables = kv_offsets_host && q_lens_host && kv_lens_host;
    std::vector<uint32_t> host(2 * (size_t)batch);
    if (host_tables) {
        for (uint32_t i = 0; i < batch; ++i) { host[i] = q_lens_host[i]; host[batch + i] = kv_lens_host[i]; }
    } else {
        if (hipMemcpy(host.data(), q_lens, (size_t)batch * sizeof(uint32_t), hipMemcpyDeviceToHost) != hipSuccess) return -7;
        if (hipMemcpy(host.data() + batch, kv_lens, (size_t)batch * sizeof(uint32_t), hipMemcpyDeviceToHost) != hipSuccess) return -7;
    }
    uint32_t max_q = 0, max_kv = 0;
    for (uint32_t i = 0; i < batch; ++i) {
        const uint32_t ql = host[i], kl = host[batch + i];
        if (ql == 0 || kl == 0 || ql > kl || kl > 8192) return -8;
        max_q = ql > max_q ? ql : max_q;
        max_kv = kl > max_kv ? kl : max_kv;
    }
    if (!m40_aligned16(q) || !m40_aligned16(k) || !m40_aligned16(v) || !m40_aligned16(out)) return -4;
    PrefillArgs a{};
    a.Q = static_cast<const float*>(q); a.K = static_cast<const float*>(k); a.V = static_cast<const float*>(v);
    a.Out = static_cast<float*>(out);
    a.q_offsets = q_offsets; a.kv_offsets = kv_offsets; a.q_lens = q_lens; a.kv_lens = kv_lens;
    a.q_heads = q_heads; a.kv_heads = kv_heads;
    // f16 planes of K and V (prefill_pack_kv_kernel) in the prefill stream's buffer, grown on demand.  The packed
    // layout needs the sequences' key ranges to lie one after the other (offsets non-decreasing with the batch index,
    // no overlap), which is how packed batches are built; anything else is refused.
    std::vector<uint32_t> offs(batch);
    if (host_tables) offs.assign(kv_offsets_host, kv_offsets_host + batch);
    else if (hipMemcpy(offs.data(), kv_offsets, (size_t)batch * sizeof(uint32_t), hipMemcpyDeviceToHost) != hipSuccess) return -7;
    uint64_t end_prev = 0;
    for (uint32_t i = 0; i < batch; ++i) {
        if (offs[i] < end_prev) return -8;
        end_prev = (uint64_t)offs[i] + host[batch + i];
    }
    const uint32_t kKTile = (uint32_t)key_tile_of((int)head_dim);
    const uint64_t plane_tiles = (offs[batch - 1] / kKTile + (batch - 1)) + (host[2 * (size_t)batch - 1] + kKTile - 1) / kKTile;
    const size_t need = (size_t)plane_tiles * kv_heads * 4 * kKTile * head_dim * sizeof(_Float16);
    M40StreamScratch& sc = ctx->scratch[0];
    if (sc.attn_planes_bytes < need) {
        if (hipStreamSynchronize(ctx->prefill_stream) != hipSuccess) return -5;
        if (sc.attn_planes) (void)hipFree(sc.attn_planes);
        sc.attn_planes = nullptr;
        sc.attn_planes_bytes = 0;
        if (hipMalloc(&sc.attn_planes, need + need / 4) != hipSuccess) {
            (void)hipGetLastError();
            return -4;
        }
        sc.attn_planes_bytes = need + need / 4;
    }
    a.planes = static_cast<const _Float16*>(sc.attn_planes);
    a.plane_tiles = (uint32_t)plane_tiles;
    (void)hipGetLastError();
    const dim3 pack_grid((max_kv + kKTile - 1) / kKTile, kv_heads, batch);
    uint64_t long_groups = 0;           // two-block workgroups that the long sequences make
    for (uint32_t i = 0; i < batch; ++i)
        if (host[i] >= kTwoBlockMinQueries) long_groups += (uint64_t)((host[i] + 32u * kWaves - 1) / (32u * kWaves)) * q_heads;
    const uint32_t blocks = long_groups >= (uint64_t)kTwoBlockMinGroupsPerCu * (uint64_t)ctx->num_cus ? 2u : 1u;
    const uint32_t q_group = 16u * kWaves * blocks;     // queries per workgroup
    const dim3 grid(q_heads, (max_q + q_group - 1) / q_group, batch);
    if (head_dim == 64) {
        prefill_pack_kv_kernel<64><<<pack_grid, kThreads, 0, ctx->prefill_stream>>>(a);
        if (blocks == 2) prefill_attn_kernel<64, 2><<<grid, kThreads, 0, ctx->prefill_stream>>>(a);
        else prefill_attn_kernel<64, 1><<<grid, kThreads, 0, ctx->prefill_stream>>>(a);
    } else {
        prefill_pack_kv_kernel<128><<<pack_grid, kThreads, 0, ctx->prefill_stream>>>(a);
        if (blocks == 2) prefill_attn_kernel<128, 2><<<grid, kThreads, 0, ctx->prefill_stream>>>(a);
        else prefill_attn_kernel<128, 1><<<grid, kThreads, 0, ctx->prefill_stream>>>(a);
    }
    if (hipGetLastError() != hipSuccess) return -4;
    if (synchronize && hipStreamSynchronize(ctx->prefill_stream) != hipSuccess) return -5;
    return 0;
}

}  // namespace

extern "C" {

int m40llm_attention_prefill_f32_gqa_varlen(M40llmCudaContext* ctx, const void* q_dev_f32, const void* k_dev_f32,
                                            const void* v_dev_f32, const uint32_t* q_offsets_dev,
                                            const uint32_t* kv_offsets_dev, const uint32_t* q_lens_dev,
                                            const uint32_t* kv_lens_dev, uint32_t batch_size, uint32_t q_heads,
                                            uint32_t kv_heads, uint32_t head_dim, void* out_dev_f32) {
    return prefill_impl(ctx, q_dev_f32, k_dev_f32, v_dev_f32, q_offsets_dev, kv_offsets_dev, q_lens_dev, kv_lens_dev,
                        batch_size, q_heads, kv_heads, head_dim, out_dev_f32, true);
}

int m40llm_attention_prefill_f32_gqa_varlen_async(M40llmCudaContext* ctx, const void* q_dev_f32, const void* k_dev_f32,
                                                  const void* v_dev_f32, const uint32_t* q_offsets_dev,
                                                  const uint32_t* kv_offsets_dev, const uint32_t* q_lens_dev,
                                                  const uint32_t* kv_lens_dev, uint32_t batch_size, uint32_t q_heads,
                                                  uint32_t kv_heads, uint32_t head_dim, void* out_dev_f32) {
    return prefill_impl(ctx, q_dev_f32, k_dev_f32, v_dev_f32, q_offsets_dev, kv_offsets_dev, q_lens_dev, kv_lens_dev,
                        batch_size, q_heads, kv_heads, head_dim, out_dev_f32, false);
}

int m40llm_ext_attention_prefill_f32_gqa_varlen_host_tables_async(M40llmCudaContext* ctx, const void* q_dev_f32,
                                                                  const void* k_dev_f32, const void* v_dev_f32,
                                                                  const uint32_t* q_offsets_dev, const uint32_t* kv_offsets_dev,
                                                                  const uint32_t* q_lens_dev, const uint32_t* kv_lens_dev,
                                                                  const uint32_t* kv_offsets_host, const uint32_t* q_lens_host,
                                                                  const uint32_t* kv_lens_host, uint32_t batch_size,
                                                                  uint32_t q_heads, uint32_t kv_heads, uint32_t head_dim,
                                                                  void* out_dev_f32) {
    if (!kv_offsets_host || !q_lens_host || !kv_lens_host) return -1;
    return prefill_impl(ctx, q_dev_f32, k_dev_f32, v_dev_f32, q_offsets_dev, kv_offsets_dev, q_lens_dev, kv_lens_dev,
                        batch_size, q_heads, kv_heads, head_dim, out_dev_f32, false, kv_offsets_host, q_lens_host, kv_lens_host);
}

}  // extern "C"
