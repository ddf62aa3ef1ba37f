// Row-batched projections (up to eight activation rows, K = 2048) against f16 GGUF weights [N][K] on the matrix
// cores, one launch per projection, for the wide matrices of a batched decode step (gate/up, lm_head).
//
// The split-K kernel of skinny_mfma.hip converts a step of activations per barrier and needs a second launch to add
// its slices.  Here the workgroups are persistent: each converts the eight rows once into f16 hi + lo MFMA fragments
// for the whole of K (64 KB of LDS, per-row power-of-two scale, RMSNorm weights folded in), then walks its share of
// the column tiles.  A tile's K range is split over the eight waves (8 MFMA steps each), so a wave requests its whole
// share of a tile in eight 16-byte loads per lane, with at most one tile in flight (more outstanding requests per CU
// make the launch slower, not faster: the first data then reaches some CUs late); the waves' partial sums
// meet in LDS in wave order and every result element is written once (residual, bias or SwiGLU applied), so nothing
// is left for a second launch and no result depends on timing.
//
// Start-up, measured with timestamps inside the kernel on the batch-8 step: the activation rows and norm weights are
// requested before any index arithmetic and ahead of the weight tiles (loads return in issue order; behind 64 KB of
// weights per CU the rows arrived 3 us later), one batch of loads whatever the norm weights' type (a branch around
// loads costs a full wait at its join), and the fragment layout in LDS is swizzled so that the conversion pass, whose
// lanes hold one row at consecutive chunks, does not pile onto four banks.  What remains is the memory system: a CU
// holds about one tile of outstanding requests, the first tile arrives about 4 us after it is requested with all 256
// CUs asking at once, and from there tiles arrive at the HBM rate (2.3-2.7 us per 64 KB and CU = 6.2-7.3 TB/s).
//
// SwiGLU form: a tile is eight gate columns and the eight up columns of the same index, so that gate and up of an
// output element come out of one MFMA accumulator tile, eight lanes apart.
//
// Reference semantics: RMSNorm cuda/kernels.cu:770-807, f32 x f16 GGUF product :5037-5052, SwiGLU :869-880; call
// order of the batched layer src/infer/forward.rs:1831-2136.
#include "common.hpp"

#include <type_traits>

namespace {

constexpr int kRows = 8;
constexpr int kK = 2048;                      // the one K this kernel is built for
constexpr int kFragBytes = (kK / 32) * 64 * 16;   // 64 KB: [k-step][lane] 16-byte A-operand entries

// Per wave count (4 or 8 waves share a tile's K range):
template <int WAVES>
struct Shape {
    static constexpr int kThreads = 64 * WAVES;
    static constexpr int kSteps = kK / 32 / WAVES;          // MFMA k-steps per wave and tile
    static constexpr int kRunLanes = kK / WAVES * 2 / 16;   // lanes that cover a column's share of K with 16 bytes each
    static constexpr int kColsPerLoad = 64 / kRunLanes;     // columns one load instruction of a wave covers
    static constexpr int kLoads = 16 / kColsPerLoad;        // load instructions per wave and tile
    static constexpr int kStageRow = kK / WAVES * 2 + 16;   // LDS bytes per column of a wave's share: +16 spreads the columns over the banks
    static constexpr int kStageBytes = 16 * kStageRow;      // per wave
    static constexpr int kDynamicLds = kFragBytes + WAVES * kStageBytes;
    static constexpr int kRowThreads = kThreads / kRows;    // threads that convert one activation row
    static constexpr int kChunks = kK / 8 / kRowThreads;    // 8-element chunks per thread
    static_assert(kRunLanes <= 64 && kRowThreads <= 64, "a column run and an activation row stay inside a wave");
};

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ m40_float4 mfma16x16x32(const uint4& a, const uint4& b, m40_float4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(m40_half8, a),
                                                  __builtin_bit_cast(m40_half8, b), c, 0, 0, 0);
}

// Where entry e of the A-operand fragments ([k-step][lane], 16 bytes each) lives in LDS.  The row index (low four bits)
// is xor-ed with the four bits above it: a k-step's 64 entries stay one contiguous, merely permuted kilobyte for the
// operand reads, while the conversion pass -- whose lanes hold the same row at consecutive chunks, entries 16 and 64
// apart -- spreads over all banks instead of hitting four of them.
__device__ __forceinline__ int frag_slot(int e) { return e ^ ((e >> 4) & 15); }

struct RowsMfmaArgs {
    const float* x;            // [rows][K]
    const void* norm_w;        // RMSNorm weights, or null
    uint32_t norm_dtype;       // 0 f16, 1 f32
    float eps;
    const uint16_t* W0;        // [N][K]
    const uint16_t* W1;        // SwiGLU: the up matrix
    float* out;                // [rows][N]
    int rows, N, units;        // units: 16-column tiles (plain) or 8-column gate/up tiles (SwiGLU)
    float* zero;               // not null: zero_count floats the launch clears on the side (the result of a following
    int zero_count;            // product whose two K halves are added into it)
    // Q/K/V form: W0 / W1 / W2 are the three matrices; a tile is 16 columns of one head that hold eight whole rotation
    // pairs (split-half layout: eight columns and their partners half a head further on)
    const uint16_t* W2;
    const float *bq, *bk, *bv;
    float* q_out;                 // [rows][q_heads * head_dim]
    uint16_t* k_cache; uint16_t* v_cache; uint32_t* seq_map;
    const uint32_t* ids_dev; const uint32_t* lens_dev;
    const float* rope_table;      // pair frequencies of (head_dim, rope_base), or null
    uint32_t max_seq_len, max_batch, q_heads, kv_heads, head_dim, rope_layout;
    float rope_base, rope_scale;
};

// Column i (0..15) of Q/K/V tile `unit`: which matrix, and the column inside it.
struct QkvTile {
    int which, head, tt;          // tt: tile inside the head
    bool split;                   // split-half pairs: columns 8 tt + i and head_dim / 2 + 8 tt + i
};
__device__ __forceinline__ QkvTile qkv_tile(const RowsMfmaArgs& p, int unit) {
    const int tph = (int)p.head_dim / 16;
    const int qt = (int)p.q_heads * tph, kt = (int)p.kv_heads * tph;
    QkvTile t;
    t.which = unit < qt ? 0 : (unit < qt + kt ? 1 : 2);
    const int local = unit - (t.which == 0 ? 0 : (t.which == 1 ? qt : qt + kt));
    t.head = local / tph;
    t.tt = local % tph;
    t.split = t.which != 2 && p.rope_layout == M40LLM_ROPE_LAYOUT_NEOX;
    return t;
}
__device__ __forceinline__ int qkv_col(const RowsMfmaArgs& p, const QkvTile& t, int i) {
    const int hd = (int)p.head_dim;
    return t.split ? t.head * hd + (i & 8 ? hd / 2 : 0) + 8 * t.tt + (i & 7) : t.head * hd + 16 * t.tt + i;
}

// MODE 0: out = x W^T; 1: SwiGLU of gate and up; 2: Q/K/V with bias, RoPE and cache append
template <int MODE, int WAVES>
__global__ __launch_bounds__(64 * WAVES, 1) void rows_mfma_kernel(RowsMfmaArgs p) {
    using S = Shape<WAVES>;
    constexpr int kWaves = WAVES, kSteps = S::kSteps, kLoads = S::kLoads, kStageRow = S::kStageRow,
                  kStageBytes = S::kStageBytes, kRunLanes = S::kRunLanes, kColsPerLoad = S::kColsPerLoad,
                  kRowThreads = S::kRowThreads, kChunks = S::kChunks;
    constexpr bool SWIGLU = MODE == 1;
    constexpr bool QKV = MODE == 2;
    extern __shared__ __attribute__((aligned(16))) uint8_t frag_bytes[];
    uint4* a_frag = reinterpret_cast<uint4*>(frag_bytes);
    uint8_t* stage = frag_bytes + kFragBytes + (threadIdx.x >> 6) * kStageBytes;     // this wave's share of the weight tile
    __shared__ float red_s[2][kWaves][4][64];      // the waves' tile sums, two tiles deep
    __shared__ float row_scale_s[kRows];           // undoes the row's power-of-two scale, times the RMSNorm factor

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int j = lane & 15, g = lane >> 4;
    // The activation rows and the norm weights are requested before anything else is computed: they head the longest
    // dependent chain of the kernel (rows -> scale -> fragments -> first matrix instruction).
    const int row = tid / kRowThreads, l = tid % kRowThreads;
    const bool live = row < p.rows;
    const float* xr = p.x + (size_t)(live ? row : 0) * kK;
    float v[kChunks][8];
    float sq = 0.0f;            // sum of squares of the raw row (RMSNorm only)
#pragma unroll
    for (int c = 0; c < kChunks; ++c) {
        const float4 a = reinterpret_cast<const float4*>(xr)[2 * (l + kRowThreads * c)];
        const float4 b = reinterpret_cast<const float4*>(xr)[2 * (l + kRowThreads * c) + 1];
        v[c][0] = a.x; v[c][1] = a.y; v[c][2] = a.z; v[c][3] = a.w;
        v[c][4] = b.x; v[c][5] = b.y; v[c][6] = b.z; v[c][7] = b.w;
    }
    // Everything the prologue needs goes out first, the weight tiles behind it: loads return in issue order, so the
    // rows and the norm weights (cache hits or a short fetch) are not kept waiting behind 64 KB of weights per
    // workgroup, and both tiles are on their way while the rows are converted.
    const bool norm16 = p.norm_w && p.norm_dtype == 0u;
    uint4 wraw[2 * kChunks];
    {
        // one unconditional batch of loads whatever the weights are (a branch around loads costs a full wait at
        // its join): f32 weights are 32 bytes per chunk; f16 weights 16 bytes, requested twice; without a norm the
        // row itself is read again and ignored
        const uint4* wp = p.norm_w ? static_cast<const uint4*>(p.norm_w) : reinterpret_cast<const uint4*>(xr);
        const int mul = norm16 ? 1 : 2, second = norm16 ? 0 : 1;
#pragma unroll
        for (int c = 0; c < kChunks; ++c) {
            wraw[2 * c] = wp[mul * (l + kRowThreads * c)];
            wraw[2 * c + 1] = wp[mul * (l + kRowThreads * c) + second];
        }
    }
    __builtin_amdgcn_sched_barrier(0);
    // consecutive, nearly equal runs of tiles (a finer split of the last tile was measured and gains nothing: the
    // launch is bound by the memory system, and the workgroups still running share what the finished ones leave)
    const int u_begin = (int)((uint32_t)blockIdx.x * (uint32_t)p.units / gridDim.x);          // units < 2^20, workgroups <= 2^10
    const int n_units = (int)(((uint32_t)blockIdx.x + 1u) * (uint32_t)p.units / gridDim.x) - u_begin;

    // Weight loads are whole runs: an instruction of a wave reads the wave's share of K of one column (four waves) or
    // two columns (eight) of the tile, 16 bytes per lane.  (Reading the MFMA operand layout straight from memory -- 16 columns x 64 bytes per
    // instruction, 4 KB apart -- streams a third slower: measured 26.5 us against 18.2 us for these 90 MB.)  The
    // operand layout is produced by a pass through the wave's own LDS tile.
    // No load under a branch: a tile past the workgroup's range re-reads the first 16 bytes of its first tile.
    uint4 b0[kLoads];
    constexpr int kEarlyLoads = kLoads * 5 / 8;       // (B=8 step at the Qwen2.5-3B shape, early part 0 / 2 / 3 / 4 / 5 / 6 / 8 of 8 loads:
                                                      // 2.49 / 2.38 / 2.34 / 2.33 / 2.32 / 2.33 / 2.35 ms; two whole tiles in flight: 2.39 ms)
    const int run_lane = lane % kRunLanes, run_col = lane / kRunLanes;
    auto issue = [&](uint4 (&b)[kLoads], int local, int l_begin = 0, int l_end = 64) {
        const bool live = local < n_units;
        const int unit = u_begin + (live ? local : 0);
        const int lane_off = live ? 8 * run_lane : 0;
#pragma unroll
        for (int li = 0; li < kLoads; ++li) {
            if (li < l_begin || li >= l_end) continue;
            const int i = li * kColsPerLoad + run_col;      // column of the tile (i & 8 is the same for the whole instruction)
            int col;
            const uint16_t* W = p.W0;
            if (SWIGLU) {
                col = 8 * unit + (i & 7);
                if (li * kColsPerLoad & 8) W = p.W1;
                col = col < p.N ? col : p.N - 1;
            } else if (QKV) {
                const QkvTile t = qkv_tile(p, unit);
                col = qkv_col(p, t, i);
                W = t.which == 0 ? p.W0 : (t.which == 1 ? p.W1 : p.W2);
            } else {
                col = 16 * unit + i;
                col = col < p.N ? col : p.N - 1;
            }
            b[li] = *reinterpret_cast<const uint4*>(W + (size_t)col * kK + wave * (kK / kWaves) + lane_off);
        }
    };
    issue(b0, 0);
    __builtin_amdgcn_sched_barrier(0);
    // the tile element this thread writes (see `finish`)
    constexpr int kTileCols = SWIGLU ? 8 : 16;      // output columns of a tile
    const int n_out = kTileCols * p.rows;
    const int e_out = tid % n_out, e_row = e_out / kTileCols, e_j = e_out % kTileCols;
    const int e_lane = 16 * (e_row >> 2) + e_j, e_r = e_row & 3;

    // Q/K/V form: what the thread's element needs besides the product -- its column and its partner's, biases, the
    // row's position and sequence, the pair's frequency.  Requested for the first tile before anything else, so that
    // the rotation is ready when the product is.
    struct QkvOperands {
        int which, col, partner_j;
        bool second;
        uint32_t position, seq;
        float bias_own, bias_other, inv_freq;
    };
    auto qkv_operands = [&](int unit) {
        QkvOperands o;
        const QkvTile t = qkv_tile(p, unit);
        o.which = t.which;
        o.col = qkv_col(p, t, e_j);
        o.partner_j = t.split ? e_j ^ 8 : e_j ^ 1;
        o.second = t.split ? (e_j & 8) != 0 : (e_j & 1) != 0;
        const uint32_t off = t.split ? (uint32_t)(8 * t.tt + (e_j & 7)) : (uint32_t)((16 * t.tt + e_j) >> 1);
        const float* bias = t.which == 0 ? p.bq : (t.which == 1 ? p.bk : p.bv);
        o.position = p.lens_dev[e_row];
        o.seq = p.ids_dev[e_row];
        o.bias_own = bias ? bias[o.col] : 0.0f;
        o.bias_other = bias ? bias[qkv_col(p, t, o.partner_j)] : 0.0f;
        o.inv_freq = p.rope_table ? p.rope_table[off] : m40_rope_inv_freq(off, p.head_dim, p.rope_base);
        return o;
    };
    QkvOperands first_ops{};
    float2 first_cs = make_float2(1.0f, 0.0f);
    if (QKV) first_ops = qkv_operands(u_begin);

    // ---- the eight rows -> f16 hi + lo fragments, once -------------------------------------------------------
    // Thread (row = tid / kRowThreads, l = tid % kRowThreads) owns the 8-element chunks l, l + kRowThreads, ... of its
    // row, so a row lives in one wave (or half-wave) and its maximum and sum of squares need no LDS.
    {
        if (norm16) {
            float sq0 = 0.0f;
#pragma unroll
            for (int c = 0; c < kChunks; ++c) {
                float w[8];
                m40_unpack8(wraw[2 * c], w);
#pragma unroll
                for (int e = 0; e < 8; ++e) { sq0 = fmaf(v[c][e], v[c][e], sq0); v[c][e] *= w[e]; }
            }
            sq = sq0;
        } else if (p.norm_w) {
            float sq0 = 0.0f;
#pragma unroll
            for (int c = 0; c < kChunks; ++c) {
                const uint4 a = wraw[2 * c], b = wraw[2 * c + 1];
                const float w[8] = {__uint_as_float(a.x), __uint_as_float(a.y), __uint_as_float(a.z), __uint_as_float(a.w),
                                    __uint_as_float(b.x), __uint_as_float(b.y), __uint_as_float(b.z), __uint_as_float(b.w)};
#pragma unroll
                for (int e = 0; e < 8; ++e) { sq0 = fmaf(v[c][e], v[c][e], sq0); v[c][e] *= w[e]; }
            }
            sq = sq0;
        }
        float mx = 0.0f;
#pragma unroll
        for (int c = 0; c < kChunks; ++c)
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                if (!live) v[c][e] = 0.0f;
                mx = fmaxf(mx, fabsf(v[c][e]));
            }
        // over the row's lanes (an aligned group of 16, 32 or 64): the bits of the xor butterfly 1, 2, ..., on the vector ALU
        static_assert(kRowThreads == 16 || kRowThreads == 32 || kRowThreads == 64, "a row is 16, 32 or 64 lanes");
        sq = m40_sum16(sq);
        mx = m40_max16(mx);
        if (kRowThreads >= 32) { sq = m40_add_xor16(sq); mx = m40_max_xor16(mx); }
        if (kRowThreads >= 64) { sq = m40_add_xor32(sq); mx = m40_max_xor32(mx); }
        float scale = 1.0f, inv_scale = 1.0f;
        if (mx > 0.0f && mx < INFINITY) {
            int ex;
            (void)frexpf(mx, &ex);        // mx = f * 2^ex, f in [0.5, 1)
            ex -= 11;                     // scaled maximum in [2^10, 2^11)
            ex = ex < -100 ? -100 : (ex > 100 ? 100 : ex);
            scale = ldexpf(1.0f, ex);
            inv_scale = ldexpf(1.0f, -ex);
        }
#pragma unroll
        for (int c = 0; c < kChunks; ++c) {
            uint32_t hi[4], lo[4];
#pragma unroll
            for (int e = 0; e < 8; e += 2) {
                const f32x2 s2 = {v[c][e] * inv_scale, v[c][e + 1] * inv_scale};
                const f16x2 h2 = __builtin_convertvector(s2, f16x2);                       // one packed conversion
                const f16x2 l2 = __builtin_convertvector(s2 - __builtin_convertvector(h2, f32x2), f16x2);
                hi[e / 2] = __builtin_bit_cast(uint32_t, h2);
                lo[e / 2] = __builtin_bit_cast(uint32_t, l2);
            }
            const int chunk = l + kRowThreads * c;                              // k = 8 chunk .. +7
            const int entry = (chunk >> 2) * 64 + (chunk & 3) * 16 + row;   // A operand: lane = 16 (k / 8 % 4) + row
            a_frag[frag_slot(entry)] = make_uint4(hi[0], hi[1], hi[2], hi[3]);          // rows 0..7: hi parts
            a_frag[frag_slot(entry + 8)] = make_uint4(lo[0], lo[1], lo[2], lo[3]);      // rows 8..15: lo parts
        }
        if (l == 0) row_scale_s[row] = scale * (p.norm_w ? rsqrtf(sq / (float)kK + p.eps) : 1.0f);
    }
    if (QKV && first_ops.which != 2) first_cs = m40_rope_cos_sin_freq(first_ops.position, first_ops.inv_freq, p.rope_scale);
    __syncthreads();

    // ---- tiles -------------------------------------------------------------------------------------------------
    // tile quarter: registers -> LDS (column-major as loaded) -> MFMA B operand (lane (j, g): 16 bytes of column j)
    auto to_lds = [&](const uint4 (&b)[kLoads]) {
#pragma unroll
        for (int li = 0; li < kLoads; ++li)      // built from the elements: a whole-struct copy would keep the array in scratch memory
            *reinterpret_cast<u32x4*>(stage + (li * kColsPerLoad + run_col) * kStageRow + 16 * run_lane) =
                u32x4{b[li].x, b[li].y, b[li].z, b[li].w};
        __builtin_amdgcn_wave_barrier();
    };
    auto compute = [&](int parity) {
        m40_float4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < kSteps; ++i) {
            const uint4 bw = *reinterpret_cast<const uint4*>(stage + j * kStageRow + 64 * i + 16 * g);
            acc = mfma16x16x32(a_frag[frag_slot((kSteps * wave + i) * 64 + lane)], bw, acc);
        }
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            acc[r] = m40_add_xor32(acc[r]);       // hi rows (g 0, 1) + lo rows (g 2, 3)
            red_s[parity][wave][r][lane] = acc[r];
        }
    };
    // After the barrier every thread can form any element of the tile from red_s.  Thread t writes element t modulo
    // the tile's live elements, so every thread stores exactly once (some twice the same value to the same address):
    // no store sits under a branch, and the waits of the loop stay exact.
    auto tile_sum = [&](int parity, int ln) {
        float t = red_s[parity][0][e_r][ln];
#pragma unroll
        for (int w = 1; w < kWaves; ++w) t += red_s[parity][w][e_r][ln];
        return t;
    };
    auto finish = [&](int local, int parity) {
        const int unit = u_begin + local;
        const float s = row_scale_s[e_row];
        if (QKV) {
            const QkvOperands& o = first_ops;          // one tile per workgroup in this form (checked by the host)
            float own = tile_sum(parity, e_lane) * s + o.bias_own;
            const float other = tile_sum(parity, (e_lane & ~15) + o.partner_j) * s + o.bias_other;
            if (o.position >= p.max_seq_len || o.seq >= p.max_batch) return;
            if (o.which != 2) {
                const float2 cs = first_cs;
                float r0, r1;
                m40_rope_apply(cs, o.second ? other : own, o.second ? own : other, &r0, &r1);
                own = o.second ? r1 : r0;
            }
            if (o.which == 0) {
                p.q_out[(size_t)e_row * p.q_heads * p.head_dim + o.col] = own;
            } else {
                const size_t ept = (size_t)p.kv_heads * p.head_dim;
                uint16_t* dst = (o.which == 1 ? p.k_cache : p.v_cache) + ((size_t)o.seq * p.max_seq_len + o.position) * ept;
                dst[o.col] = m40_f2h(own);
                if (o.which == 1 && o.col == 0) p.seq_map[o.seq] = o.position + 1u;
            }
            return;
        }
        int col = kTileCols * unit + e_j;
        col = col < p.N ? col : p.N - 1;          // a column past the end was computed from the last column's weights
        float v = tile_sum(parity, e_lane) * s;
        if (SWIGLU) {
            const float up = tile_sum(parity, e_lane + 8) * s;
            v = v / (1.0f + expf(-v)) * up;
        }
        p.out[(size_t)e_row * p.N + col] = v;
    };
    // One tile from register set b; PREFETCH: tile local + 1 exists and is requested into the same set.
    auto tile = [&](uint4 (&b)[kLoads], auto prefetch_c, int local, int parity) {
        to_lds(b);
        // the next tile's requests go out in two parts, around this tile's arithmetic: at most one tile (64 KB per
        // CU) is ever in flight, and for the length of the arithmetic only kEarlyLoads / kLoads of it
        if (decltype(prefetch_c)::value) issue(b, local + 1, 0, kEarlyLoads);
        compute(parity);
        __syncthreads();
        finish(local, parity);
        if (decltype(prefetch_c)::value) issue(b, local + 1, kEarlyLoads, kLoads);
    };
    if (QKV) {
        tile(b0, std::integral_constant<bool, false>{}, 0, 0);
    } else {
        const std::integral_constant<bool, true> yes;
        const std::integral_constant<bool, false> no;
        int local = 0;
        for (; local + 1 < n_units; ++local) tile(b0, yes, local, local & 1);
        tile(b0, no, local, local & 1);
    }
    // behind everything else: nothing in this launch waits for these stores
    if (p.zero)
        for (int i = (int)blockIdx.x * S::kThreads + tid; i < p.zero_count; i += (int)gridDim.x * S::kThreads) p.zero[i] = 0.0f;
}

template <int MODE, int WAVES>
int launch_w(M40llmCudaContext* ctx, hipStream_t stream, const RowsMfmaArgs& a) {
    using S = Shape<WAVES>;
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(rows_mfma_kernel<MODE, WAVES>),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, S::kDynamicLds);
    if (attr != hipSuccess) return -7;
    int grid = ctx->num_cus;           // one workgroup per CU: most of its LDS
    if (grid > a.units) grid = a.units;
    rows_mfma_kernel<MODE, WAVES><<<grid, S::kThreads, S::kDynamicLds, stream>>>(a);
    return hipGetLastError() == hipSuccess ? 0 : -7;
}
template <int MODE>
int launch(M40llmCudaContext* ctx, hipStream_t stream, const RowsMfmaArgs& a) {
    // eight waves: the conversion pass is spread over twice the lanes and twice as many requests are in flight per CU
    // as with four (batch-8 step at the Qwen2.5-3B shape: 2.58 -> 2.55 ms)
    return launch_w<MODE, 8>(ctx, stream, a);
}

}  // namespace

bool m40_rows_mfma_supported(int rows, int K) { return rows >= 1 && rows <= kRows && K == kK; }

int m40_rows_mfma_swiglu(M40llmCudaContext* ctx, hipStream_t stream, const float* x, const void* norm_w, uint32_t norm_dtype,
                         float eps, const uint16_t* wgate, const uint16_t* wup, float* out, int rows, int ffn, int K,
                         float* zero, int zero_count) {
    if (!m40_rows_mfma_supported(rows, K) || ffn <= 0) return -6;
    if (!m40_aligned16(x) || !m40_aligned16(wgate) || !m40_aligned16(wup) || (norm_w && !m40_aligned16(norm_w))) return -6;
    RowsMfmaArgs a{};
    a.x = x; a.norm_w = norm_w; a.norm_dtype = norm_dtype; a.eps = eps; a.W0 = wgate; a.W1 = wup; a.out = out;
    a.rows = rows; a.N = ffn; a.units = (ffn + 7) / 8;
    a.zero = zero; a.zero_count = zero_count;
    return launch<1>(ctx, stream, a);
}

int m40_rows_mfma_plain(M40llmCudaContext* ctx, hipStream_t stream, const float* x, const void* norm_w, uint32_t norm_dtype,
                        float eps, const uint16_t* W, float* out, int rows, int N, int K) {
    if (!m40_rows_mfma_supported(rows, K) || N <= 0) return -6;
    if (!m40_aligned16(x) || !m40_aligned16(W) || (norm_w && !m40_aligned16(norm_w))) return -6;
    RowsMfmaArgs a{};
    a.x = x; a.norm_w = norm_w; a.norm_dtype = norm_dtype; a.eps = eps; a.W0 = W; a.out = out; a.rows = rows; a.N = N; a.units = (N + 15) / 16;
    return launch<0>(ctx, stream, a);
}

bool m40_rows_mfma_qkv_supported(int rows, int K, uint32_t head_dim) {
    return m40_rows_mfma_supported(rows, K) && head_dim >= 16 && head_dim % 16 == 0;
}

int m40_rows_mfma_qkv(M40llmCudaContext* ctx, hipStream_t stream, const M40llmKVCache* kv, const uint32_t* ids_dev,
                      const uint32_t* lens_dev, uint32_t rows, const float* x, const void* norm_w, uint32_t norm_dtype, float eps,
                      const uint16_t* wq, const uint16_t* wk, const uint16_t* wv, const float* bq, const float* bk,
                      const float* bv, uint32_t d_model, uint32_t q_heads, float rope_base, float rope_scale,
                      uint32_t rope_layout, float* q_out) {
    if (!m40_rows_mfma_qkv_supported((int)rows, (int)d_model, kv->head_dim)) return -6;
    // one tile per workgroup: the rotation angle of a thread's element is computed once, ahead of the product
    if ((int)((q_heads + 2u * kv->num_heads) * kv->head_dim / 16u) > ctx->num_cus) return -6;
    if (!m40_aligned16(x) || !m40_aligned16(norm_w) || !m40_aligned16(wq) || !m40_aligned16(wk) || !m40_aligned16(wv)) return -6;
    RowsMfmaArgs a{};
    a.x = x; a.norm_w = norm_w; a.norm_dtype = norm_dtype; a.eps = eps; a.W0 = wq; a.W1 = wk; a.W2 = wv;
    a.bq = bq; a.bk = bk; a.bv = bv; a.q_out = q_out; a.k_cache = kv->d_k; a.v_cache = kv->d_v; a.seq_map = kv->d_seq_map;
    a.ids_dev = ids_dev; a.lens_dev = lens_dev;
    a.rope_table = m40_rope_inv_freq_table(ctx, 1, stream, kv->head_dim, rope_base);
    a.max_seq_len = kv->max_seq_len; a.max_batch = kv->max_batch_size; a.q_heads = q_heads; a.kv_heads = kv->num_heads;
    a.head_dim = kv->head_dim; a.rope_layout = rope_layout; a.rope_base = rope_base; a.rope_scale = rope_scale;
    a.rows = (int)rows; a.N = (int)((q_heads + 2u * kv->num_heads) * kv->head_dim);
    a.units = a.N / 16;
    return launch<2>(ctx, stream, a);
}
