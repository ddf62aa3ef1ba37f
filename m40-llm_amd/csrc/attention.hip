// Last-token GQA attention over the dense f16 KV cache for gfx950 (single sequence, device
// length, recent-window and variable-length batched forms share one kernel).
//
// Work split: grid = (kv_head x q-head subgroup, token chunk, batch row).  A workgroup of eight waves
// owns a chunk of 8 * TPW * S token rows (TPW = rows per 64-lane load: 8 at head_dim 64, 4 at 128).
// Every lane issues all of its S K-row and S V-row 128-bit loads before any arithmetic, so a chunk
// costs one memory round trip; the rows serve all G q heads of the subgroup.  Scores stay in
// registers.  With one chunk the kernel writes the output; otherwise it writes the softmax partial
// (max, sum, weighted V) and a second kernel merges the chunks in ascending order.
//
// Reference semantics: three-pass softmax per q head, kv head = qh / (q_heads / kv_heads),
// scale literals for head_dim 64 / 128: cuda/kernels.cu:1367-1655, entry points :3837-4023,
// batched :1740-1823 and :4694-4832.
#include "attention_params.hpp"

#include <atomic>
#include <mutex>

// Fixed chunk-partial buffer of m40llm_ext_attention_last_token_f32_gqa_static_scratch_async: device memory that
// exists from the moment the code object is loaded, so that entry point never allocates.  Every GPU the library
// runs on holds its own copy (at its own address) until the process ends.  In host code the array's name is a
// stand-in, not a device address: host code only ever uses the pointers that hipGetSymbolAddress returned
// (g_static_scratch_ptr), one per device.
constexpr size_t kStaticScratchBytes = 2u << 20;   // 2 MiB
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kStaticScratchMaxDevices = 64;
static std::atomic<float*> g_static_scratch_ptr[kStaticScratchMaxDevices];
static std::mutex g_static_scratch_mutex;
// Who used a device's array last, and an event behind that call's last launch: a call from another context while
// that work is still outstanding is refused (-10) instead of racing.  The event is made with the pointer, at set-up.
struct StaticScratchUse {
    const M40llmCudaContext* owner;
    hipEvent_t done;
    bool have_event, recorded;
};
static StaticScratchUse g_static_scratch_use[kStaticScratchMaxDevices];

int m40_attention_static_scratch_init(int device_id) {
    if (device_id < 0 || device_id >= kStaticScratchMaxDevices) return -2;
    std::lock_guard<std::mutex> lock(g_static_scratch_mutex);
    if (g_static_scratch_ptr[device_id].load(std::memory_order_acquire)) return 0;
    void* ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) {
        (void)hipGetLastError();
        return -4;
    }
    StaticScratchUse& use = g_static_scratch_use[device_id];
    if (!use.have_event) {
        if (hipEventCreateWithFlags(&use.done, hipEventDisableTiming) == hipSuccess) use.have_event = true;
        else (void)hipGetLastError();
    }
    g_static_scratch_ptr[device_id].store(static_cast<float*>(ptr), std::memory_order_release);
    return 0;
}

namespace {

constexpr int kAttnThreads = 512;
constexpr int kWaves = kAttnThreads / 64;


// HD in {64, 128}; G = q heads per workgroup (<= 4); S = token rows per lane group
template <int HD, int G, int S>
__global__ __launch_bounds__(kAttnThreads, 2) void attn_partial_kernel(AttnParams p) {
    constexpr int LPT = HD / 8;      // lanes per token row
    constexpr int TPW = 64 / LPT;    // token rows per wave load
    __shared__ float red[kWaves][G][HD];
    __shared__ float wmax[kWaves][G];
    __shared__ float wsum[kWaves][G];

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

    const uint32_t kvh = blockIdx.x / p.subgroups;
    const uint32_t sub = blockIdx.x % p.subgroups;
    const uint32_t group = p.q_heads / p.kv_heads;
    const uint32_t qh0 = kvh * group + sub * G;          // first q head of this workgroup
    const uint32_t gcount = (sub * G + G <= group) ? G : group - sub * G;

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int c = lane % LPT, tg = lane / LPT;
    const size_t row_stride = (size_t)p.kv_heads * HD;
    const size_t base = ((size_t)seq_id * p.max_seq_len) * row_stride + (size_t)kvh * HD + 8 * c;
    const uint16_t* Kb = p.K + base;
    const uint16_t* Vb = p.V + base;
    const float inv_sqrt = HD == 64 ? 0.125f : 0.08838834764831845f;

    // every load of this lane, issued before anything waits on memory
    uint4 kw[S], vw[S];
    bool valid[S];
#pragma unroll
    for (int s = 0; s < S; ++s) {
        const uint32_t t = cbeg + (uint32_t)((s * kWaves + wave) * TPW + tg);
        valid[s] = t < cend;
        kw[s] = make_uint4(0, 0, 0, 0);
        vw[s] = make_uint4(0, 0, 0, 0);
        if (valid[s]) {
            kw[s] = *reinterpret_cast<const uint4*>(Kb + (size_t)t * row_stride);
            vw[s] = *reinterpret_cast<const uint4*>(Vb + (size_t)t * row_stride);
        }
    }
    float q[G][8];
#pragma unroll
    for (int h = 0; h < G; ++h) {
        const uint32_t qh = qh0 + (h < (int)gcount ? h : 0);
        const float* qp = p.Q + ((size_t)b * p.q_heads + qh) * HD + 8 * c;
        const float4 q0 = *reinterpret_cast<const float4*>(qp);
        const float4 q1 = *reinterpret_cast<const float4*>(qp + 4);
        q[h][0] = q0.x; q[h][1] = q0.y; q[h][2] = q0.z; q[h][3] = q0.w;
        q[h][4] = q1.x; q[h][5] = q1.y; q[h][6] = q1.z; q[h][7] = q1.w;
    }

    // ---- scores (every lane of a row group ends up with the row's score) -----------------------
    float sc[S][G];
    float lmax[G];
#pragma unroll
    for (int h = 0; h < G; ++h) lmax[h] = -INFINITY;
#pragma unroll
    for (int s = 0; s < S; ++s) {
        float kf[8];
        m40_unpack8(kw[s], kf);
#pragma unroll
        for (int h = 0; h < G; ++h) {
            float d = 0.0f;
#pragma unroll
            for (int j = 0; j < 8; ++j) d = fmaf(q[h][j], kf[j], d);
            d = LPT == 8 ? m40_sum8(d) : m40_sum16(d);
            sc[s][h] = valid[s] ? d * inv_sqrt : -INFINITY;
            lmax[h] = fmaxf(lmax[h], sc[s][h]);
        }
    }
#pragma unroll
    for (int h = 0; h < G; ++h) {
        const float m = m40_max64(lmax[h]);
        if (lane == 0) wmax[wave][h] = m;
    }
    __syncthreads();
    float mh[G];
#pragma unroll
    for (int h = 0; h < G; ++h) {
        float m = wmax[0][h];
#pragma unroll
        for (int w = 1; w < kWaves; ++w) m = fmaxf(m, wmax[w][h]);
        mh[h] = m;
    }

    // ---- exp, row sums, weighted V -----------------------------------------------------------
    float lsum[G];
    float acc[G][8];
#pragma unroll
    for (int h = 0; h < G; ++h) {
        lsum[h] = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[h][j] = 0.0f;
    }
#pragma unroll
    for (int s = 0; s < S; ++s) {
        float vf[8];
        m40_unpack8(vw[s], vf);
#pragma unroll
        for (int h = 0; h < G; ++h) {
            const float e = valid[s] ? expf(sc[s][h] - mh[h]) : 0.0f;
            if (c == 0) lsum[h] += e;
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[h][j] = fmaf(e, vf[j], acc[h][j]);
        }
    }
    // join the TPW token rows of the wave (lanes with equal c), then the waves
#pragma unroll
    for (int h = 0; h < G; ++h) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            acc[h][j] = m40_sum_lanes_from<LPT>(acc[h][j]);
        }
        const float ssum = m40_sum64(lsum[h]);
        if (lane == 0) wsum[wave][h] = ssum;
    }
    if (tg == 0) {
#pragma unroll
        for (int h = 0; h < G; ++h)
#pragma unroll
            for (int j = 0; j < 8; ++j) red[wave][h][8 * c + j] = acc[h][j];
    }
    __syncthreads();

    const bool final_out = p.nchunks == 1;
    for (uint32_t e = tid; e < gcount * HD; e += kAttnThreads) {
        const uint32_t h = e / HD, d = e % HD;
        float v = 0.0f, l = 0.0f;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) {
            v += red[w][h][d];
            l += wsum[w][h];
        }
        const uint32_t qh = qh0 + h;
        if (final_out) {
            const float denom = l > 0.0f ? l : 1.0f;
            p.Out[((size_t)b * p.q_heads + qh) * HD + d] = v / denom;
        } else {
            float* w = p.ws + (((size_t)b * p.q_heads + qh) * p.nchunks + blockIdx.y) * (HD + 2);
            w[2 + d] = v;
            if (d == 0) {
                w[0] = mh[h];
                w[1] = l;
            }
        }
    }
}

// Merge chunk partials: grid (q_heads, batch), 256 threads = 256/HD chunk lanes x HD dims.  Each chunk lane
// folds chunks lane, lane + n_lanes, ... with a running maximum; the chunk lanes are then folded in order.
template <int HD>
__global__ __launch_bounds__(256) void attn_combine_kernel(AttnParams p) {
    constexpr int NCG = 256 / HD;
    __shared__ float s_m[NCG], s_den[NCG];
    __shared__ float s_num[NCG][HD];
    const uint32_t qh = blockIdx.x, b = blockIdx.y;
    const uint32_t d = threadIdx.x % HD, cg = threadIdx.x / HD;
    // The lane's first kPre chunk partials are requested together with the row's length and id, before either is
    // known (one memory round trip instead of a chain of three); partials of chunks past the row's end are stale
    // values inside the buffer and are never used.  The chunks are folded in the same ascending order either way.
    constexpr uint32_t kPre = 8;
    const float* w = p.ws + (((size_t)b * p.q_heads + qh) * p.nchunks) * (HD + 2);
    float pm[kPre], pl[kPre], pv[kPre];
#pragma unroll
    for (uint32_t u = 0; u < kPre; ++u) {
        const uint32_t ch = cg + u * NCG;
        const float* wc = w + (size_t)(ch < p.nchunks ? ch : 0u) * (HD + 2);
        pm[u] = wc[0]; pl[u] = wc[1]; pv[u] = wc[2 + d];
    }
    const uint32_t len = p.seq_lens_dev ? p.seq_lens_dev[b] + p.len_bias : p.seq_len;
    const uint32_t sid = (p.max_batch != 0 && p.seq_ids_dev) ? p.seq_ids_dev[b] : 0u;
    if (len == 0 || len > p.max_seq_len) return;
    if (p.max_batch != 0 && p.seq_ids_dev && sid >= p.max_batch) return;
    const uint32_t t0 = (p.window != 0 && len > p.window) ? len - p.window : 0;
    if (len - t0 > p.span_limit) return;      // longer than the launch was sized for: the row is skipped
    const uint32_t n = (len - t0 + p.chunk - 1) / p.chunk;
    float m = -INFINITY, num = 0.0f, den = 0.0f;
    auto fold = [&](float mc, float lc, float vc) {
        const float nm = fmaxf(m, mc);
        const float fa = m == -INFINITY ? 0.0f : expf(m - nm);
        const float fb = mc == -INFINITY ? 0.0f : expf(mc - nm);
        num = fmaf(num, fa, vc * fb);
        den = fmaf(den, fa, lc * fb);
        m = nm;
    };
#pragma unroll
    for (uint32_t u = 0; u < kPre; ++u)
        if (cg + u * NCG < n) fold(pm[u], pl[u], pv[u]);
#pragma unroll 4
    for (uint32_t ch = cg + kPre * NCG; ch < n; ch += NCG) {
        const float* wc = w + (size_t)ch * (HD + 2);
        fold(wc[0], wc[1], wc[2 + d]);
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
        den = den > 0.0f ? den : 1.0f;
        p.Out[((size_t)b * p.q_heads + qh) * HD + d] = num / den;
    }
}

// Any head_dim: one thread per output element, the reference's three passes verbatim
// (cuda/kernels.cu:1367-1426).  Used for head_dim other than 64 / 128 only.
__global__ __launch_bounds__(64) void attn_generic_kernel(AttnParams p, uint32_t head_dim) {
    const uint32_t b = blockIdx.z, qh = blockIdx.y;
    const uint32_t d = blockIdx.x * 64 + threadIdx.x;
    if (d >= head_dim) return;
    const uint32_t seq_id = p.seq_ids_dev ? p.seq_ids_dev[b] : p.seq_id;
    const uint32_t len = p.seq_lens_dev ? p.seq_lens_dev[b] + p.len_bias : p.seq_len;
    if (len == 0 || len > p.max_seq_len) return;
    const uint32_t t0 = (p.window != 0 && len > p.window) ? len - p.window : 0;
    if (len - t0 > p.span_limit) return;      // longer than the launch was sized for: the row is skipped
    const uint32_t kvh = qh / (p.q_heads / p.kv_heads);
    const size_t ept = (size_t)p.kv_heads * head_dim;
    const float inv_sqrt = m40_inv_sqrt_head_dim(head_dim);
    const float* q = p.Q + ((size_t)b * p.q_heads + qh) * head_dim;
    const uint16_t* Kb = p.K + ((size_t)seq_id * p.max_seq_len) * ept + (size_t)kvh * head_dim;
    const uint16_t* Vb = p.V + ((size_t)seq_id * p.max_seq_len) * ept + (size_t)kvh * head_dim;
    float mx = -1e30f;
    for (uint32_t t = t0; t < len; ++t) {
        float dot = 0.0f;
        for (uint32_t k = 0; k < head_dim; ++k) dot += q[k] * m40_h2f(Kb[(size_t)t * ept + k]);
        mx = fmaxf(mx, dot * inv_sqrt);
    }
    float den = 0.0f, acc = 0.0f;
    for (uint32_t t = t0; t < len; ++t) {
        float dot = 0.0f;
        for (uint32_t k = 0; k < head_dim; ++k) dot += q[k] * m40_h2f(Kb[(size_t)t * ept + k]);
        const float e = expf(dot * inv_sqrt - mx);
        den += e;
        acc += e * m40_h2f(Vb[(size_t)t * ept + d]);
    }
    den = den > 0.0f ? den : 1.0f;
    p.Out[((size_t)b * p.q_heads + qh) * head_dim + d] = acc / den;
}

template <int HD, int G, int S>
void launch_partial(hipStream_t stream, const AttnParams& p, uint32_t batch) {
    dim3 grid(p.kv_heads * p.subgroups, p.nchunks, batch);
    attn_partial_kernel<HD, G, S><<<grid, kAttnThreads, 0, stream>>>(p);
}

template <int HD, int G>
void launch_g(hipStream_t stream, const AttnParams& p, uint32_t batch, int S) {
    switch (S) {
        case 8: launch_partial<HD, G, 8>(stream, p, batch); break;
        case 4: launch_partial<HD, G, 4>(stream, p, batch); break;
        case 2: launch_partial<HD, G, 2>(stream, p, batch); break;
        default: launch_partial<HD, G, 1>(stream, p, batch); break;
    }
}

// Chooses rows per lane group (S), q heads per workgroup (G) and the chunking for a span of `span` tokens.
template <int HD>
int launch_hd(M40llmCudaContext* ctx, hipStream_t stream, float* partial, size_t partial_bytes, bool fixed_chunking,
              AttnParams& p, uint32_t batch, uint32_t group, uint32_t span) {
    constexpr uint32_t kRowsPerStep = kWaves * (64 / (HD / 8));   // token rows one workgroup covers per S
    if (span > 512 && m40_aligned16(p.Q)) {
        // long rows: matrix-core kernel (it reads q with 16-byte loads).  Chunks are a multiple of 128 tokens (one
        // 32-token tile per wave and pass) sized for about one workgroup per CU -- measured best at 32 K tokens (256
        // workgroups of 1024 tokens: 32 us against 36 us with twice as many half-sized ones) and on the batch-8 step
        // -- rounded to the nearest multiple, and up while more than two workgroups would land on a CU.
        p.subgroups = (group + 7) / 8;
        const uint64_t groups = (uint64_t)batch * p.kv_heads * p.subgroups;
        uint64_t chunk = (((uint64_t)span * groups / ctx->num_cus) + 64) / 128 * 128;
        if (chunk < 128) chunk = 128;
        while (groups * ((span + chunk - 1) / chunk) > 2ull * ctx->num_cus) chunk += 128;
        if (chunk > 2048) chunk = 2048;
        for (;;) {
            p.chunk = (uint32_t)chunk;
            p.nchunks = (span + p.chunk - 1) / p.chunk;
            if (p.nchunks == 1 || (size_t)batch * p.q_heads * p.nchunks * (HD + 2) * sizeof(float) <= partial_bytes) break;
            if (fixed_chunking) return -9;   // the caller wants this chunking or none (fixed-size partial buffer)
            chunk *= 2;
        }
        p.ws = partial;
        m40_launch_attn_mfma(stream, p, HD, batch);
        if (p.nchunks > 1) {
            dim3 grid(p.q_heads, batch);
            attn_combine_kernel<HD><<<grid, 256, 0, stream>>>(p);
        }
        return 0;
    }
    int G = group >= 4 ? 4 : (group >= 2 ? 2 : 1);
    const uint64_t rows = (uint64_t)batch * p.kv_heads;
    // Short rows are latency-bound, not bandwidth-bound: spread the q heads over more workgroups, down to one head
    // each (K/V of a short row stay in L2, so re-reading them per head costs nothing; measured +3 % on the whole
    // batch-1 token against two heads per workgroup).
    while (span <= 1024 && G > 1 && rows * ((group + G - 1) / G) < 128) G >>= 1;
    p.subgroups = (group + G - 1) / G;
    int S = 8;
    if (span <= kRowsPerStep * 8) {
        // one chunk, no merge launch: the smallest S that covers the span
        S = 1;
        while ((uint32_t)S * kRowsPerStep < span) S <<= 1;
    } else {
        // split until the grid covers the CUs about twice
        while (S > 2 && rows * p.subgroups * ((span + kRowsPerStep * S - 1) / (kRowsPerStep * S)) < 2u * (uint32_t)ctx->num_cus)
            S >>= 1;
    }
    p.chunk = kRowsPerStep * (uint32_t)S;
    p.nchunks = (span + p.chunk - 1) / p.chunk;
    if (p.nchunks > 1) {
        const size_t need = (size_t)batch * p.q_heads * p.nchunks * (HD + 2) * sizeof(float);
        if (need > partial_bytes) {
            if (fixed_chunking) return -9;
            if (S == 8) return -7;
            S = 8;
            p.chunk = kRowsPerStep * 8u;
            p.nchunks = (span + p.chunk - 1) / p.chunk;
            if ((size_t)batch * p.q_heads * p.nchunks * (HD + 2) * sizeof(float) > partial_bytes) return -7;
        }
    }
    p.ws = partial;
    switch (G) {
        case 4: launch_g<HD, 4>(stream, p, batch, S); break;
        case 2: launch_g<HD, 2>(stream, p, batch, S); break;
        default: launch_g<HD, 1>(stream, p, batch, S); break;
    }
    if (p.nchunks > 1) {
        dim3 grid(p.q_heads, batch);
        attn_combine_kernel<HD><<<grid, 256, 0, stream>>>(p);
    }
    return 0;
}

}  // namespace

int m40_launch_dense_attention(M40llmCudaContext* ctx, hipStream_t stream, uint32_t stream_kind,
                               const M40AttnArgs& a) {
    AttnParams p{};
    p.K = a.K; p.V = a.V; p.Q = a.Q; p.Out = a.Out;
    p.seq_ids_dev = a.seq_ids_dev; p.seq_lens_dev = a.seq_lens_dev;
    p.seq_id = a.seq_id; p.seq_len = a.seq_len;
    p.max_seq_len = a.max_seq_len; p.kv_heads = a.kv_heads; p.q_heads = a.q_heads; p.window = a.window;
    p.subgroups = 1;
    p.len_bias = a.len_bias;
    p.max_batch = a.max_batch;
    (void)hipGetLastError();
    const uint32_t group = a.q_heads / a.kv_heads;
    uint32_t span = a.max_len_hint;
    if (a.window != 0 && span > a.window) span = a.window;
    if (span == 0) span = 1;
    p.span_limit = span;

    if ((a.head_dim == 64 || a.head_dim == 128) && m40_aligned16(a.Q) && m40_aligned16(a.K) && m40_aligned16(a.V)) {
        M40StreamScratch& scr = ctx->scratch[stream_kind];
        float* partial = a.partial_override ? a.partial_override : static_cast<float*>(scr.attn_partial);
        const size_t partial_bytes = a.partial_override ? a.partial_override_bytes : scr.attn_partial_bytes;
        const bool fixed = a.partial_override != nullptr;
        const int rc = a.head_dim == 64 ? launch_hd<64>(ctx, stream, partial, partial_bytes, fixed, p, a.batch, group, span)
                                        : launch_hd<128>(ctx, stream, partial, partial_bytes, fixed, p, a.batch, group, span);
        if (rc != 0) return rc;
    } else {
        p.chunk = span; p.nchunks = 1;
        dim3 grid((a.head_dim + 63) / 64, a.q_heads, a.batch);
        attn_generic_kernel<<<grid, 64, 0, stream>>>(p, a.head_dim);
    }
    return hipGetLastError() == hipSuccess ? 0 : -4;
}

// Reads the (ids, lens) pair of a batched call back to the host for validation, as the reference
// does before launching (cuda/kernels.cu:4721-4754); returns the largest length.
// The reference copies both metadata arrays to the host and validates them before it launches (kernels.cu:4723-4754).
// Here the copies are ordered on the decode stream (they see whatever earlier decode-stream work wrote) and land in
// the context's pinned staging words: two asynchronous copies and one wait.
static int validate_batch(M40llmCudaContext* ctx, const M40llmKVCache* kv, const uint32_t* ids_dev,
                          const uint32_t* lens_dev, uint32_t batch, uint32_t* max_len) {
    uint32_t *ids, *lens;
    const bool staged = ctx->host_staging && 2u * batch <= (uint32_t)kM40HostStagingWords;
    if (staged) {
        ids = ctx->host_staging;
        lens = ctx->host_staging + batch;
    } else {
        ids = new uint32_t[batch];
        lens = new uint32_t[batch];
    }
    int rc = 0;
    if (hipMemcpyAsync(lens, lens_dev, (size_t)batch * 4, hipMemcpyDeviceToHost, ctx->decode_stream) != hipSuccess ||
        hipMemcpyAsync(ids, ids_dev, (size_t)batch * 4, hipMemcpyDeviceToHost, ctx->decode_stream) != hipSuccess ||
        hipStreamSynchronize(ctx->decode_stream) != hipSuccess) {
        (void)hipGetLastError();
        rc = -7;
    }
    uint32_t mx = 0;
    for (uint32_t i = 0; rc == 0 && i < batch; ++i) {
        if (ids[i] >= kv->max_batch_size) rc = -8;
        else if (lens[i] == 0 || lens[i] > kv->max_seq_len) rc = -8;
        else if (lens[i] > mx) mx = lens[i];
    }
    if (!staged) { delete[] ids; delete[] lens; }
    *max_len = mx;
    return rc;
}

extern "C" {

int m40llm_attention_last_token_f32_gqa_async(M40llmCudaContext* ctx, const M40llmKVCache* kv, uint32_t seq_id,
                                              const void* q_dev_f32, uint32_t q_heads, uint32_t seq_len,
                                              void* out_dev_f32) {
    if (!ctx || !kv || !q_dev_f32 || !out_dev_f32) return -1;
    if (seq_id >= kv->max_batch_size) return -2;
    if (seq_len == 0 || seq_len > kv->max_seq_len) return -3;
    if (q_heads == 0 || kv->num_heads == 0 || q_heads % kv->num_heads != 0) return -6;
    if (!kv->d_k || !kv->d_v) return -4;
    M40AttnArgs a{};
    a.K = kv->d_k; a.V = kv->d_v; a.max_seq_len = kv->max_seq_len; a.kv_heads = kv->num_heads;
    a.head_dim = kv->head_dim; a.q_heads = q_heads; a.Q = static_cast<const float*>(q_dev_f32);
    a.Out = static_cast<float*>(out_dev_f32); a.batch = 1; a.seq_id = seq_id; a.seq_len = seq_len;
    a.max_len_hint = seq_len;
    return m40_launch_dense_attention(ctx, ctx->decode_stream, 1, a);
}

// m40llm_attention_last_token_f32_gqa_async for callers that cannot allocate (HIP graph capture, serving loops and
// harnesses that forbid hipMalloc): same checks, kernels, chunking and results, but the chunk partials of a long
// row go into this device's copy of the fixed 2 MiB array above instead of the context's arena.  Calls nothing that
// allocates.  -9: the partials of this (q_heads, head_dim, seq_len) do not fit the fixed buffer.  All calls on one
// GPU share that buffer (every partial a call reads it has written itself, so nothing needs clearing between
// calls).  Calls of one context are ordered on its decode stream; a call from another context while the last user's
// work is still outstanding returns -10 (busy) instead of racing.  Under stream capture no event can be queried, so
// captured calls are not guarded: replays that overlap on one GPU race.
int m40llm_ext_attention_last_token_f32_gqa_static_scratch_async(M40llmCudaContext* ctx, const M40llmKVCache* kv,
                                                                 uint32_t seq_id, const void* q_dev_f32,
                                                                 uint32_t q_heads, uint32_t seq_len,
                                                                 void* out_dev_f32) {
    if (!ctx || !kv || !q_dev_f32 || !out_dev_f32) return -1;
    if (seq_id >= kv->max_batch_size) return -2;
    if (seq_len == 0 || seq_len > kv->max_seq_len) return -3;
    if (q_heads == 0 || kv->num_heads == 0 || q_heads % kv->num_heads != 0) return -6;
    if (!kv->d_k || !kv->d_v) return -4;
    if (ctx->device_id < 0 || ctx->device_id >= kStaticScratchMaxDevices) return -4;
    float* ptr = g_static_scratch_ptr[ctx->device_id].load(std::memory_order_acquire);
    if (!ptr) {
        // a context made before this translation unit could resolve the symbol: resolve it now, on the context's device
        if (m40_ensure_device(ctx) != 0 || m40_attention_static_scratch_init(ctx->device_id) != 0) return -4;
        ptr = g_static_scratch_ptr[ctx->device_id].load(std::memory_order_acquire);
    }
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(ctx->decode_stream, &capture) != hipSuccess) { (void)hipGetLastError(); capture = hipStreamCaptureStatusNone; }
    const bool guarded = capture == hipStreamCaptureStatusNone;
    std::unique_lock<std::mutex> lock(g_static_scratch_mutex, std::defer_lock);
    StaticScratchUse& use = g_static_scratch_use[ctx->device_id];
    if (guarded) {
        lock.lock();
        if (use.owner && use.owner != ctx && use.have_event && use.recorded) {
            const hipError_t q = hipEventQuery(use.done);
            if (q == hipErrorNotReady) return -10;
            if (q != hipSuccess) (void)hipGetLastError();
        }
    }
    M40AttnArgs a{};
    a.K = kv->d_k; a.V = kv->d_v; a.max_seq_len = kv->max_seq_len; a.kv_heads = kv->num_heads;
    a.head_dim = kv->head_dim; a.q_heads = q_heads; a.Q = static_cast<const float*>(q_dev_f32);
    a.Out = static_cast<float*>(out_dev_f32); a.batch = 1; a.seq_id = seq_id; a.seq_len = seq_len;
    a.max_len_hint = seq_len;
    a.partial_override = ptr;
    a.partial_override_bytes = kStaticScratchBytes;
    const int rc = m40_launch_dense_attention(ctx, ctx->decode_stream, 1, a);
    if (guarded && rc == 0 && use.have_event) {
        use.owner = ctx;
        use.recorded = hipEventRecord(use.done, ctx->decode_stream) == hipSuccess;
        if (!use.recorded) (void)hipGetLastError();
    }
    return rc;
}

int m40llm_attention_last_token_f32_gqa(M40llmCudaContext* ctx, const M40llmKVCache* kv, uint32_t seq_id,
                                        const void* q_dev_f32, uint32_t q_heads, uint32_t seq_len,
                                        void* out_dev_f32) {
    int rc = m40llm_attention_last_token_f32_gqa_async(ctx, kv, seq_id, q_dev_f32, q_heads, seq_len, out_dev_f32);
    if (rc != 0) return rc;
    return hipStreamSynchronize(ctx->decode_stream) == hipSuccess ? 0 : -5;
}

// MHA form: q heads == kv heads (cuda/kernels.cu:3837-3861), synchronous.
int m40llm_attention_last_token_f32(M40llmCudaContext* ctx, const M40llmKVCache* kv, uint32_t seq_id,
                                    const void* q_dev_f32, uint32_t seq_len, void* out_dev_f32) {
    if (!ctx || !kv || !q_dev_f32 || !out_dev_f32) return -1;
    if (seq_id >= kv->max_batch_size) return -2;
    if (seq_len == 0 || seq_len > kv->max_seq_len) return -3;
    if (!kv->d_k || !kv->d_v || kv->num_heads == 0) return -4;
    M40AttnArgs a{};
    a.K = kv->d_k; a.V = kv->d_v; a.max_seq_len = kv->max_seq_len; a.kv_heads = kv->num_heads;
    a.head_dim = kv->head_dim; a.q_heads = kv->num_heads; a.Q = static_cast<const float*>(q_dev_f32);
    a.Out = static_cast<float*>(out_dev_f32); a.batch = 1; a.seq_id = seq_id; a.seq_len = seq_len;
    a.max_len_hint = seq_len;
    int rc = m40_launch_dense_attention(ctx, ctx->decode_stream, 1, a);
    if (rc != 0) return -4;
    return hipStreamSynchronize(ctx->decode_stream) == hipSuccess ? 0 : -5;
}

int m40llm_attention_last_token_f32_gqa_seq_len_dev_async(M40llmCudaContext* ctx, const M40llmKVCache* kv,
                                                          uint32_t seq_id, const void* q_dev_f32,
                                                          uint32_t q_heads, const uint32_t* seq_len_dev,
                                                          void* out_dev_f32) {
    if (!ctx || !kv || !q_dev_f32 || !seq_len_dev || !out_dev_f32) return -1;
    if (seq_id >= kv->max_batch_size) return -2;
    if (q_heads == 0 || kv->num_heads == 0 || q_heads % kv->num_heads != 0) return -3;
    if (!kv->d_k || !kv->d_v) return -4;
    M40AttnArgs a{};
    a.K = kv->d_k; a.V = kv->d_v; a.max_seq_len = kv->max_seq_len; a.kv_heads = kv->num_heads;
    a.head_dim = kv->head_dim; a.q_heads = q_heads; a.Q = static_cast<const float*>(q_dev_f32);
    a.Out = static_cast<float*>(out_dev_f32); a.batch = 1; a.seq_id = seq_id; a.seq_len = 0;
    a.seq_lens_dev = seq_len_dev;            // row 0 of a one-row batch
    a.max_len_hint = kv->max_seq_len;        // the length is unknown on the host: size for the maximum
    return m40_launch_dense_attention(ctx, ctx->decode_stream, 1, a);
}

// Extension: the sequence length is (*position_dev + 1); max_len_hint bounds it and sizes the grid.
int m40llm_ext_attention_last_token_f32_gqa_position_dev_async(M40llmCudaContext* ctx, const M40llmKVCache* kv,
                                                               uint32_t seq_id, const void* q_dev_f32,
                                                               uint32_t q_heads, const uint32_t* position_dev,
                                                               uint32_t max_len_hint, void* out_dev_f32) {
    if (!ctx || !kv || !q_dev_f32 || !position_dev || !out_dev_f32) return -1;
    if (seq_id >= kv->max_batch_size) return -2;
    if (max_len_hint == 0 || max_len_hint > kv->max_seq_len) return -3;
    if (q_heads == 0 || kv->num_heads == 0 || q_heads % kv->num_heads != 0) return -6;
    if (!kv->d_k || !kv->d_v) return -4;
    M40AttnArgs a{};
    a.K = kv->d_k; a.V = kv->d_v; a.max_seq_len = kv->max_seq_len; a.kv_heads = kv->num_heads;
    a.head_dim = kv->head_dim; a.q_heads = q_heads; a.Q = static_cast<const float*>(q_dev_f32);
    a.Out = static_cast<float*>(out_dev_f32); a.batch = 1; a.seq_id = seq_id; a.seq_len = 0;
    a.seq_lens_dev = position_dev; a.len_bias = 1; a.max_len_hint = max_len_hint;
    return m40_launch_dense_attention(ctx, ctx->decode_stream, 1, a);
}

int m40llm_attention_last_token_f32_gqa_dense_recent_async(M40llmCudaContext* ctx, const M40llmKVCache* kv,
                                                           uint32_t seq_id, const void* q_dev_f32,
                                                           uint32_t q_heads, uint32_t seq_len,
                                                           uint32_t recent_window, void* out_dev_f32) {
    if (!ctx || !kv || !q_dev_f32 || !out_dev_f32) return -1;
    if (seq_id >= kv->max_batch_size) return -2;
    if (seq_len == 0 || seq_len > kv->max_seq_len) return -3;
    if (q_heads == 0 || kv->num_heads == 0 || q_heads % kv->num_heads != 0) return -4;
    if (kv->head_dim != 64 && kv->head_dim != 128) return -5;
    if (recent_window == 0) return -6;
    if (!kv->d_k || !kv->d_v) return -7;
    M40AttnArgs a{};
    a.K = kv->d_k; a.V = kv->d_v; a.max_seq_len = kv->max_seq_len; a.kv_heads = kv->num_heads;
    a.head_dim = kv->head_dim; a.q_heads = q_heads; a.Q = static_cast<const float*>(q_dev_f32);
    a.Out = static_cast<float*>(out_dev_f32); a.batch = 1; a.seq_id = seq_id; a.seq_len = seq_len;
    a.max_len_hint = seq_len; a.window = recent_window;
    return m40_launch_dense_attention(ctx, ctx->decode_stream, 1, a) == 0 ? 0 : -7;
}

static int batched_impl(M40llmCudaContext* ctx, const M40llmKVCache* kv, const uint32_t* seq_ids_dev,
                        const uint32_t* seq_lens_dev, uint32_t batch_size, const void* q_dev_f32,
                        uint32_t q_heads, void* out_dev_f32, bool synchronize) {
    if (!ctx || !kv || !seq_ids_dev || !seq_lens_dev || !q_dev_f32 || !out_dev_f32) return -1;
    if (batch_size == 0) return -2;
    if (q_heads == 0 || kv->num_heads == 0 || q_heads % kv->num_heads != 0) return -3;
    if (kv->head_dim != 64 && kv->head_dim != 128) return -6;
    if (!kv->d_k || !kv->d_v) return -6;
    uint32_t max_len = 0;
    int rc = validate_batch(ctx, kv, seq_ids_dev, seq_lens_dev, batch_size, &max_len);
    if (rc != 0) return rc;
    if (max_len == 0) return -8;
    M40AttnArgs a{};
    a.K = kv->d_k; a.V = kv->d_v; a.max_seq_len = kv->max_seq_len; a.kv_heads = kv->num_heads;
    a.head_dim = kv->head_dim; a.q_heads = q_heads; a.Q = static_cast<const float*>(q_dev_f32);
    a.Out = static_cast<float*>(out_dev_f32); a.batch = batch_size;
    a.seq_ids_dev = seq_ids_dev; a.seq_lens_dev = seq_lens_dev; a.max_len_hint = max_len;
    rc = m40_launch_dense_attention(ctx, ctx->decode_stream, 1, a);
    if (rc != 0) return -4;
    if (synchronize && hipStreamSynchronize(ctx->decode_stream) != hipSuccess) return -5;
    return 0;
}

// Row-batched attention whose ids / lengths stay on the device: nothing is copied back for validation; rows whose
// id or length (+ len_bias) is out of range are skipped by the kernel.  max_len_hint bounds every row's length.
int m40llm_ext_attention_last_token_f32_gqa_batched_lens_dev_async(M40llmCudaContext* ctx, const M40llmKVCache* kv,
                                                                   const uint32_t* seq_ids_dev,
                                                                   const uint32_t* seq_lens_dev, uint32_t len_bias,
                                                                   uint32_t batch_size, uint32_t max_len_hint,
                                                                   const void* q_dev_f32, uint32_t q_heads,
                                                                   void* out_dev_f32) {
    if (!ctx || !kv || !seq_ids_dev || !seq_lens_dev || !q_dev_f32 || !out_dev_f32) return -1;
    if (batch_size == 0) return -2;
    if (q_heads == 0 || kv->num_heads == 0 || q_heads % kv->num_heads != 0) return -3;
    if (kv->head_dim != 64 && kv->head_dim != 128) return -6;
    if (!kv->d_k || !kv->d_v) return -6;
    if (max_len_hint == 0 || max_len_hint > kv->max_seq_len) return -8;
    M40AttnArgs a{};
    a.K = kv->d_k; a.V = kv->d_v; a.max_seq_len = kv->max_seq_len; a.kv_heads = kv->num_heads;
    a.head_dim = kv->head_dim; a.q_heads = q_heads; a.Q = static_cast<const float*>(q_dev_f32);
    a.Out = static_cast<float*>(out_dev_f32); a.batch = batch_size;
    a.seq_ids_dev = seq_ids_dev; a.seq_lens_dev = seq_lens_dev; a.len_bias = len_bias; a.max_len_hint = max_len_hint;
    a.max_batch = kv->max_batch_size;
    return m40_launch_dense_attention(ctx, ctx->decode_stream, 1, a) == 0 ? 0 : -4;
}

int m40llm_attention_last_token_f32_gqa_batched(M40llmCudaContext* ctx, const M40llmKVCache* kv,
                                                const uint32_t* seq_ids_dev, const uint32_t* seq_lens_dev,
                                                uint32_t batch_size, const void* q_dev_f32, uint32_t q_heads,
                                                void* out_dev_f32) {
    return batched_impl(ctx, kv, seq_ids_dev, seq_lens_dev, batch_size, q_dev_f32, q_heads, out_dev_f32, true);
}

int m40llm_attention_last_token_f32_gqa_batched_async(M40llmCudaContext* ctx, const M40llmKVCache* kv,
                                                      const uint32_t* seq_ids_dev, const uint32_t* seq_lens_dev,
                                                      uint32_t batch_size, const void* q_dev_f32,
                                                      uint32_t q_heads, void* out_dev_f32) {
    return batched_impl(ctx, kv, seq_ids_dev, seq_lens_dev, batch_size, q_dev_f32, q_heads, out_dev_f32, false);
}

}  // extern "C"
