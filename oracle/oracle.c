/*
 * CPU oracle for the m40-llm decode-step hot path.  TEST INFRASTRUCTURE ONLY:
 * the checker the HIP path is compared against, never the thing shipped.
 *
 * Each function cites the reference source it restates (paths are relative to
 * the reference checkout).  Build with -ffp-contract=off so every C operator is
 * one IEEE binary32 rounding; fused multiply-adds appear only where fmaf() is
 * written out.
 *
 * Pinning status (what independent evidence each part is checked against lives
 * in tests/test_oracle_*.py):
 *   f16 conversion ........ numpy float16 (independent RNE), all 65536 codes
 *   KV layout ............. reference literal index(1,2,2,4)=104
 *   attention ............. float64 softmax, L=1 / equal-K invariants, closed-form fixtures
 *   prefill attention ..... float64 softmax on the reference's fixture; one-key, one-token and per-sequence invariants
 *   q4 V .................. brute-force quantiser, byte-accounting literals 8192/2048/128
 *   block selection ....... brute-force sort on tiny inputs, "all blocks selected == dense"
 *   GEMM .................. reference known answers [19,22;43,50], [40,46]; float64 matmul
 *   q8_0 .................. reference fixture formula; float64 dequant
 *   RMSNorm / RoPE adjacent float64 closed forms on the reference fixtures
 *   RoPE NeoX ............. no reference test exists; pinned by the permutation
 *                           identity NeoX == adjacent after 2i->i, 2i+1->i+hd/2,
 *                           norm preservation and position 0 = identity
 *   greedy ................ reference literals ([0.1,-0.2,5,1]->2, [0,5,1]->1, NaN case)
 *   layer / model ......... float64 numpy restatement on a toy model; L=1 => context=V
 *   packed prefill forward  float64 restatement without the f16 round trip of K / V (fits to 2e-5, the one with the
 *                           round trip does not); batch == each prompt alone; layer-0 cache == the token path's
 */
#include "oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

static int g_threads = 1;

void orc_set_threads(int n) {
    g_threads = n < 1 ? 1 : n;
#ifdef _OPENMP
    omp_set_num_threads(g_threads);
#endif
}
int orc_get_threads(void) { return g_threads; }

/* ------------------------------------------------------------------------ */
/* f32 <-> f16, round to nearest even.                                       */
/* Reference: half::f16::from_f32 / to_f32 as used by append_token_host      */
/* (src/cuda.rs:3605-3631) and __float2half_rn (cuda/kernels.cu:5545-5552).  */
/* ------------------------------------------------------------------------ */
uint16_t orc_f32_to_f16(float x) {
    uint32_t u;
    memcpy(&u, &x, 4);
    const uint32_t sign = (u >> 16) & 0x8000u;
    const uint32_t absu = u & 0x7fffffffu;
    if (absu >= 0x7f800000u) { /* inf / nan */
        if (absu > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((absu >> 13) & 0x3ffu));
        return (uint16_t)(sign | 0x7c00u);
    }
    if (absu >= 0x477ff000u) { /* rounds to >= 65520 -> inf */
        return (uint16_t)(sign | 0x7c00u);
    }
    if (absu < 0x38800000u) { /* subnormal half or zero: value < 2^-14 */
        if (absu < 0x33000000u) return (uint16_t)sign; /* < 2^-25 -> 0 */
        const uint32_t exp = absu >> 23;                /* 102..112 */
        const uint32_t mant = (absu & 0x7fffffu) | 0x800000u;
        const uint32_t shift = 126u - exp;              /* 14..24 */
        uint32_t half_mant = mant >> shift;
        const uint32_t rem = mant & ((1u << shift) - 1u);
        const uint32_t halfway = 1u << (shift - 1u);
        if (rem > halfway || (rem == halfway && (half_mant & 1u))) half_mant++;
        return (uint16_t)(sign | half_mant);
    }
    /* normal */
    uint32_t half = ((absu - 0x38000000u) >> 13);
    const uint32_t rem = absu & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (half & 1u))) half++;
    return (uint16_t)(sign | half);
}

static float f16_to_f32_bits(uint16_t h) {
    const uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t mant = h & 0x3ffu;
    uint32_t u;
    if (exp == 0) {
        if (mant == 0) {
            u = sign;
        } else {
            int e = -1;
            do { mant <<= 1; e++; } while (!(mant & 0x400u));
            mant &= 0x3ffu;
            u = sign | ((uint32_t)(127 - 15 - e) << 23) | (mant << 13);
        }
    } else if (exp == 31) {
        u = sign | 0x7f800000u | (mant << 13);
    } else {
        u = sign | ((exp + 127 - 15) << 23) | (mant << 13);
    }
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* Every f16 value's f32 image, filled from the routine above when the library is loaded: the conversions inside
 * the GEMM and attention loops are one table read each (same bits, a few times faster than the branches). */
static float f16_table[65536];
__attribute__((constructor)) static void fill_f16_table(void) {
    for (uint32_t h = 0; h < 65536u; ++h) f16_table[h] = f16_to_f32_bits((uint16_t)h);
}
static inline float h2f(uint16_t h) { return f16_table[h]; }
float orc_f16_to_f32(uint16_t h) { return h2f(h); }

void orc_f32_to_f16_n(const float* in, uint16_t* out, size_t n) {
    for (size_t i = 0; i < n; ++i) out[i] = orc_f32_to_f16(in[i]);
}
void orc_f16_to_f32_n(const uint16_t* in, float* out, size_t n) {
    for (size_t i = 0; i < n; ++i) out[i] = h2f(in[i]);
}

/* ------------------------------------------------------------------------ */
/* KV layout [seq][token][head][dim].  Reference: cuda/kernels.cu:5304-5312, */
/* tests/kv_layout.rs (index(1,2,2,4) == 104 for max_seq 4, heads 3, hd 5).  */
/* ------------------------------------------------------------------------ */
size_t orc_kv_elems_per_token(uint32_t kv_heads, uint32_t head_dim) {
    return (size_t)kv_heads * (size_t)head_dim;
}
size_t orc_kv_base(uint32_t max_seq_len, uint32_t kv_heads, uint32_t head_dim,
                   uint32_t seq, uint32_t token) {
    return ((size_t)seq * (size_t)max_seq_len + (size_t)token) *
           orc_kv_elems_per_token(kv_heads, head_dim);
}
size_t orc_kv_index(uint32_t max_seq_len, uint32_t kv_heads, uint32_t head_dim,
                    uint32_t seq, uint32_t token, uint32_t head, uint32_t dim) {
    return orc_kv_base(max_seq_len, kv_heads, head_dim, seq, token) +
           (size_t)head * (size_t)head_dim + (size_t)dim;
}

/* ------------------------------------------------------------------------ */
/* RMSNorm.  Reference: cuda/kernels.cu:736-807 (y = x*scale*w, scale =       */
/* rsqrtf(sum(x^2)/dim + eps)), CPU form tests/rmsnorm_rope.rs:9-40           */
/* (sequential sum of squares).                                               */
/* ------------------------------------------------------------------------ */
void orc_rms_norm(const float* in, float* out, uint32_t rows, uint32_t dim, float eps) {
    for (uint32_t r = 0; r < rows; ++r) {
        const float* x = in + (size_t)r * dim;
        float ss = 0.0f;
        for (uint32_t i = 0; i < dim; ++i) ss += x[i] * x[i];
        const float scale = 1.0f / sqrtf(ss / (float)dim + eps);
        for (uint32_t i = 0; i < dim; ++i) out[(size_t)r * dim + i] = x[i] * scale;
    }
}

int orc_rms_norm_weighted(const float* in, const void* weight, float* out,
                          uint32_t rows, uint32_t dim, float eps, uint32_t weight_dtype) {
    if (weight_dtype > 1) return -4; /* cuda/kernels.cu:1096 */
    const uint16_t* w16 = (const uint16_t*)weight;
    const float* w32 = (const float*)weight;
    for (uint32_t r = 0; r < rows; ++r) {
        const float* x = in + (size_t)r * dim;
        float ss = 0.0f;
        for (uint32_t i = 0; i < dim; ++i) ss += x[i] * x[i];
        const float scale = 1.0f / sqrtf(ss / (float)dim + eps);
        for (uint32_t i = 0; i < dim; ++i) {
            const float w = weight_dtype == 0 ? h2f(w16[i]) : w32[i];
            out[(size_t)r * dim + i] = x[i] * scale * w; /* order x*scale*w, kernels.cu:805 */
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------ */
/* RoPE.  Reference: rope_pair_indices cuda/kernels.cu:5570-5585,             */
/* rope_f32_inplace_kernel :7300-7332; CPU adjacent tests/rmsnorm_rope.rs:43. */
/* Position is cast to float before the multiply by freq_scale.               */
/* ------------------------------------------------------------------------ */
static void rope_pair(uint32_t head, uint32_t off, uint32_t head_dim, uint32_t layout,
                      size_t* i0, size_t* i1) {
    const size_t hb = (size_t)head * head_dim;
    if (layout == 1u) {
        *i0 = hb + off;
        *i1 = *i0 + head_dim / 2u;
    } else {
        *i0 = hb + 2u * off;
        *i1 = *i0 + 1u;
    }
}

static void rope_cs(uint32_t position, uint32_t off, uint32_t head_dim, float base, float scale,
                    float* c, float* s) {
    const float pos = (float)position * scale;
    const float theta = pos * powf(base, -2.0f * (float)off / (float)head_dim);
    *c = cosf(theta);
    *s = sinf(theta);
}

void orc_rope_inplace(float* x, uint32_t rows, uint32_t num_heads, uint32_t head_dim,
                      uint32_t past_len, float freq_base, float freq_scale, uint32_t layout) {
    const uint32_t half = head_dim / 2u;
    for (uint32_t r = 0; r < rows; ++r) {
        float* row = x + (size_t)r * num_heads * head_dim;
        for (uint32_t h = 0; h < num_heads; ++h) {
            for (uint32_t i = 0; i < half; ++i) {
                size_t i0, i1;
                float c, s;
                rope_pair(h, i, head_dim, layout, &i0, &i1);
                rope_cs(past_len + r, i, head_dim, freq_base, freq_scale, &c, &s);
                const float x0 = row[i0], x1 = row[i1];
                row[i0] = x0 * c - x1 * s;
                row[i1] = x0 * s + x1 * c;
            }
        }
    }
}

/* Reference: cuda/kernels.cu:869-891 */
void orc_residual_add(const float* a, const float* b, float* out, size_t n) {
    for (size_t i = 0; i < n; ++i) out[i] = a[i] + b[i];
}
void orc_swiglu(const float* gate, const float* up, float* out, size_t n) {
    for (size_t i = 0; i < n; ++i) {
        const float g = gate[i];
        const float silu = g / (1.0f + expf(-g));
        out[i] = silu * up[i];
    }
}

/* q8_0: 34-byte blocks {f16 d; int8 qs[32]}.  Reference: cuda/kernels.cu:856-867,
 * src/infer/embeddings.rs:93-112, src/gguf.rs:312-313. */
void orc_q80_to_f32(const uint8_t* in, float* out, size_t n) {
    for (size_t i = 0; i < n; ++i) {
        const size_t blk = i / 32, idx = i % 32;
        const uint8_t* base = in + blk * 34;
        uint16_t dh;
        memcpy(&dh, base, 2);
        const float d = h2f(dh);
        const int8_t q = (int8_t)base[2 + idx];
        out[i] = d * (float)q;
    }
}

/* ------------------------------------------------------------------------ */
/* GEMM family.  Reference kernels cuda/kernels.cu:4999-5052: one accumulator */
/* per output, k ascending, acc += a*b.  Column loops are spread over threads */
/* and interleaved four at a time; each output's own order is unchanged.      */
/* ------------------------------------------------------------------------ */
void orc_gemm_f32xf16_gguf(const float* A, const uint16_t* B, float* C, int M, int N, int K) {
    for (int i = 0; i < M; ++i) {
        const float* a = A + (size_t)i * K;
#pragma omp parallel for schedule(static) if (N >= 64)
        for (int j0 = 0; j0 < N; j0 += 4) {
            const int nj = N - j0 < 4 ? N - j0 : 4;
            float acc[4] = {0.f, 0.f, 0.f, 0.f};
            const uint16_t* b[4];
            for (int c = 0; c < 4; ++c) b[c] = B + (size_t)(j0 + (c < nj ? c : 0)) * K;
            for (int kk = 0; kk < K; ++kk) {
                const float av = a[kk];
                acc[0] += av * h2f(b[0][kk]);
                acc[1] += av * h2f(b[1][kk]);
                acc[2] += av * h2f(b[2][kk]);
                acc[3] += av * h2f(b[3][kk]);
            }
            for (int c = 0; c < nj; ++c) C[(size_t)i * N + j0 + c] = acc[c];
        }
    }
}

void orc_gemm_f32xf16_rowmajor(const float* A, const uint16_t* B, float* C, int M, int N, int K) {
    for (int i = 0; i < M; ++i)
        for (int j = 0; j < N; ++j) {
            float acc = 0.0f;
            for (int kk = 0; kk < K; ++kk)
                acc += A[(size_t)i * K + kk] * h2f(B[(size_t)kk * N + j]);
            C[(size_t)i * N + j] = acc;
        }
}

void orc_gemm_f16xf16_rowmajor(const uint16_t* A, const uint16_t* B, float* C, int M, int N, int K) {
    for (int i = 0; i < M; ++i)
        for (int j = 0; j < N; ++j) {
            float acc = 0.0f;
            for (int kk = 0; kk < K; ++kk)
                acc += h2f(A[(size_t)i * K + kk]) * h2f(B[(size_t)kk * N + j]);
            C[(size_t)i * N + j] = acc;
        }
}

/* q8_0 GEMM: no such kernel exists in the reference; semantics = its q8_0
 * dequant (x = d*q, cuda/kernels.cu:856-867) followed by its GGUF-layout f32
 * GEMM loop (cuda/kernels.cu:5037-5052). */
void orc_gemm_f32xq80_gguf(const float* A, const uint8_t* B, float* C, int M, int N, int K) {
    const size_t col_bytes = (size_t)(K / 32) * 34;
    for (int i = 0; i < M; ++i) {
        const float* a = A + (size_t)i * K;
#pragma omp parallel for schedule(static) if (N >= 64)
        for (int j = 0; j < N; ++j) {
            const uint8_t* col = B + (size_t)j * col_bytes;
            float acc = 0.0f;
            for (int blk = 0; blk < K / 32; ++blk) {
                const uint8_t* base = col + (size_t)blk * 34;
                uint16_t dh;
                memcpy(&dh, base, 2);
                const float d = h2f(dh);
                const int8_t* qs = (const int8_t*)(base + 2);
                for (int t = 0; t < 32; ++t) {
                    const float x = d * (float)qs[t];
                    acc += a[blk * 32 + t] * x;
                }
            }
            C[(size_t)i * N + j] = acc;
        }
    }
}

void orc_ffn_swiglu_q80(const float* x, const uint8_t* w_gate, const uint8_t* w_up,
                        const uint8_t* w_down, float* scratch_gate, float* scratch_up,
                        float* out, int M, int d_model, int ffn) {
    /* op order of the reference MLP: gate, up GEMMs -> swiglu -> down GEMM
     * (src/infer/forward.rs:557-625) */
    orc_gemm_f32xq80_gguf(x, w_gate, scratch_gate, M, ffn, d_model);
    orc_gemm_f32xq80_gguf(x, w_up, scratch_up, M, ffn, d_model);
    orc_swiglu(scratch_gate, scratch_up, scratch_gate, (size_t)M * ffn);
    orc_gemm_f32xq80_gguf(scratch_gate, w_down, out, M, d_model, ffn);
}

/* ------------------------------------------------------------------------ */
/* Dense KV append.  Reference: append_token_host src/cuda.rs:3605-3631,      */
/* fused RoPE-K append cuda/kernels.cu:5624-5676 (V is cast only).            */
/* ------------------------------------------------------------------------ */
void orc_kv_append_f32(uint16_t* K, uint16_t* V, uint32_t max_seq_len, uint32_t kv_heads,
                       uint32_t head_dim, uint32_t seq, uint32_t token,
                       const float* k_f32, const float* v_f32) {
    const size_t base = orc_kv_base(max_seq_len, kv_heads, head_dim, seq, token);
    const size_t n = orc_kv_elems_per_token(kv_heads, head_dim);
    for (size_t i = 0; i < n; ++i) {
        K[base + i] = orc_f32_to_f16(k_f32[i]);
        V[base + i] = orc_f32_to_f16(v_f32[i]);
    }
}

static void rope_k_to_f16(const float* k_f32, uint16_t* k_out, uint32_t kv_heads, uint32_t head_dim,
                          uint32_t position, float freq_base, float freq_scale, uint32_t layout) {
    const uint32_t half = head_dim / 2u;
    for (uint32_t h = 0; h < kv_heads; ++h)
        for (uint32_t i = 0; i < half; ++i) {
            size_t i0, i1;
            float c, s;
            rope_pair(h, i, head_dim, layout, &i0, &i1);
            rope_cs(position, i, head_dim, freq_base, freq_scale, &c, &s);
            const float k0 = k_f32[i0], k1 = k_f32[i1];
            k_out[i0] = orc_f32_to_f16(k0 * c - k1 * s);
            k_out[i1] = orc_f32_to_f16(k0 * s + k1 * c);
        }
}

void orc_kv_append_f32_rope_k(uint16_t* K, uint16_t* V, uint32_t max_seq_len, uint32_t kv_heads,
                              uint32_t head_dim, uint32_t seq, uint32_t position,
                              const float* k_f32, const float* v_f32,
                              float freq_base, float freq_scale, uint32_t layout) {
    const size_t base = orc_kv_base(max_seq_len, kv_heads, head_dim, seq, position);
    const size_t n = orc_kv_elems_per_token(kv_heads, head_dim);
    rope_k_to_f16(k_f32, K + base, kv_heads, head_dim, position, freq_base, freq_scale, layout);
    for (size_t i = 0; i < n; ++i) V[base + i] = orc_f32_to_f16(v_f32[i]);
}

/* inv_sqrt: literal constants in the head_dim 64 / 128 kernels
 * (cuda/kernels.cu:1515, :1597), 1/sqrtf(hd) otherwise (:1384, src/cuda.rs:4574) */
float orc_inv_sqrt_head_dim(uint32_t head_dim) {
    if (head_dim == 64u) return 0.125f;
    if (head_dim == 128u) return 0.08838834764831845f;
    return 1.0f / sqrtf((float)head_dim);
}

/* ------------------------------------------------------------------------ */
/* Last-token attention, three passes.  Reference: CPU body                  */
/* src/cuda.rs:4561-4628, GQA head mapping                                    */
/* tests/attention_parity_cuda_grid.rs:1415-1469 (kv = qh / (q_heads/kvh)).   */
/* ------------------------------------------------------------------------ */
void orc_attention_last_token_gqa(const uint16_t* K, const uint16_t* V, uint32_t max_seq_len,
                                  uint32_t kv_heads, uint32_t head_dim, uint32_t seq,
                                  const float* q, uint32_t q_heads, uint32_t seq_len, float* out) {
    const uint32_t group = q_heads / kv_heads;
    const float inv_sqrt = orc_inv_sqrt_head_dim(head_dim);
    /* Heads are independent and spread over threads (when this call is not itself inside a parallel loop).  The weight
     * of a key, expf(score - max) / denom, is the same number for every output column: it is computed once per key, and
     * the weighted sum walks the keys in the outer loop with one accumulator per column -- every column's own sum still
     * adds its keys in ascending order, so the results are the reference's bit for bit. */
#pragma omp parallel for schedule(dynamic) if ((size_t)seq_len * q_heads >= 4096)
    for (uint32_t h = 0; h < q_heads; ++h) {
        float* scores = (float*)malloc(sizeof(float) * ((size_t)(seq_len ? seq_len : 1) + head_dim));
        float* acc = scores + (seq_len ? seq_len : 1);
        const uint32_t kvh = h / group;
        const float* qh = q + (size_t)h * head_dim;
        float max_score = -INFINITY;
        for (uint32_t t = 0; t < seq_len; ++t) {
            const size_t base = orc_kv_index(max_seq_len, kv_heads, head_dim, seq, t, kvh, 0);
            float dot = 0.0f;
            for (uint32_t d = 0; d < head_dim; ++d) dot += qh[d] * h2f(K[base + d]);
            const float s = dot * inv_sqrt;
            scores[t] = s;
            if (s > max_score) max_score = s;
        }
        float denom = 0.0f;
        for (uint32_t t = 0; t < seq_len; ++t) denom += expf(scores[t] - max_score);
        if (!(denom > 0.0f)) denom = 1.0f;
        for (uint32_t d = 0; d < head_dim; ++d) acc[d] = 0.0f;
        for (uint32_t t = 0; t < seq_len; ++t) {
            const size_t base = orc_kv_index(max_seq_len, kv_heads, head_dim, seq, t, kvh, 0);
            const float p = expf(scores[t] - max_score) / denom;
            for (uint32_t d = 0; d < head_dim; ++d) acc[d] += p * h2f(V[base + d]);
        }
        float* oh = out + (size_t)h * head_dim;
        for (uint32_t d = 0; d < head_dim; ++d) oh[d] = acc[d];
        free(scores);
    }
}

/* Reference: cuda/kernels.cu:1740-1823 (one row per batch entry, rows with
 * seq_len 0 skipped), checked against per-sequence calls in
 * tests/attention_batched_varlen.rs:200-221. */
void orc_attention_last_token_gqa_batched(const uint16_t* K, const uint16_t* V,
                                          uint32_t max_seq_len, uint32_t kv_heads,
                                          uint32_t head_dim, const uint32_t* seq_ids,
                                          const uint32_t* seq_lens, uint32_t batch,
                                          const float* q, uint32_t q_heads, float* out) {
    const size_t row = (size_t)q_heads * head_dim;
#pragma omp parallel for schedule(dynamic) if (batch > 1)
    for (uint32_t b = 0; b < batch; ++b) {
        if (seq_lens[b] == 0) continue;
        orc_attention_last_token_gqa(K, V, max_seq_len, kv_heads, head_dim, seq_ids[b],
                                     q + b * row, q_heads, seq_lens[b], out + b * row);
    }
}

/* ------------------------------------------------------------------------ */
/* Packed variable-length causal prefill attention, all f32.                   */
/* Reference: cuda/kernels.cu:3749-3835 (kernel: query q_idx of sequence b      */
/* attends keys 0 .. kv_len - q_len + q_idx; three passes; p = exp / denom      */
/* before the weighted sum), argument checks and their codes :4834-4895, CPU    */
/* restatement tests/attention_prefill_varlen.rs:27-76.  Q and Out are          */
/* [total_q][q_heads][hd], K and V [total_kv][kv_heads][hd]; offsets in tokens. */
/* ------------------------------------------------------------------------ */
int orc_attention_prefill_gqa_varlen(const float* q, const float* k, const float* v,
                                     const uint32_t* q_offsets, const uint32_t* kv_offsets,
                                     const uint32_t* q_lens, const uint32_t* kv_lens, uint32_t batch,
                                     uint32_t q_heads, uint32_t kv_heads, uint32_t head_dim, float* out) {
    if (!q || !k || !v || !q_offsets || !kv_offsets || !q_lens || !kv_lens || !out) return -1;
    if (batch == 0) return -2;
    if (q_heads == 0 || kv_heads == 0 || q_heads % kv_heads != 0) return -3;
    if (head_dim != 64 && head_dim != 128) return -9;
    for (uint32_t b = 0; b < batch; ++b)
        if (q_lens[b] == 0 || kv_lens[b] == 0 || q_lens[b] > kv_lens[b] || kv_lens[b] > 8192) return -8;
    const uint32_t group = q_heads / kv_heads;
    const float inv_sqrt = orc_inv_sqrt_head_dim(head_dim);
    /* queries are independent and spread over threads; a key's weight is computed once and the weighted sum keeps one
     * accumulator per column with the keys in the outer loop (each column's sum in ascending key order, as in the
     * reference: the same bits) */
    for (uint32_t b = 0; b < batch; ++b) {
#pragma omp parallel for schedule(dynamic, 4)
        for (uint32_t qi = 0; qi < q_lens[b]; ++qi) {
            float* scores = (float*)malloc(sizeof(float) * ((size_t)kv_lens[b] + head_dim));
            float* acc = scores + kv_lens[b];
            const uint32_t causal_end = kv_lens[b] - q_lens[b] + qi;
            for (uint32_t h = 0; h < q_heads; ++h) {
                const uint32_t kvh = h / group;
                const float* qh = q + ((size_t)(q_offsets[b] + qi) * q_heads + h) * head_dim;
                float max_score = -1e30f;
                for (uint32_t t = 0; t <= causal_end; ++t) {
                    const float* kh = k + ((size_t)(kv_offsets[b] + t) * kv_heads + kvh) * head_dim;
                    float dot = 0.0f;
                    for (uint32_t d = 0; d < head_dim; ++d) dot += qh[d] * kh[d];
                    const float s = dot * inv_sqrt;
                    scores[t] = s;
                    if (s > max_score) max_score = s;
                }
                float denom = 0.0f;
                for (uint32_t t = 0; t <= causal_end; ++t) denom += expf(scores[t] - max_score);
                if (!(denom > 0.0f)) denom = 1.0f;
                for (uint32_t d = 0; d < head_dim; ++d) acc[d] = 0.0f;
                for (uint32_t t = 0; t <= causal_end; ++t) {
                    const float* vh = v + ((size_t)(kv_offsets[b] + t) * kv_heads + kvh) * head_dim;
                    const float p = expf(scores[t] - max_score) / denom;
                    for (uint32_t d = 0; d < head_dim; ++d) acc[d] += p * vh[d];
                }
                float* oh = out + ((size_t)(q_offsets[b] + qi) * q_heads + h) * head_dim;
                for (uint32_t d = 0; d < head_dim; ++d) oh[d] = acc[d];
            }
            free(scores);
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------ */
/* fp16-K / q4-V compressed cache.                                           */
/* Layout: cuda/kernels.cu:5357-5385, :5435-5543; append/evict :6108-6250     */
/* with kernels :2230-2311, ring write :5786-5790.                            */
/* ------------------------------------------------------------------------ */
orc_ckv* orc_ckv_create(uint32_t max_seq_len, uint32_t max_batch, uint32_t kv_heads,
                        uint32_t head_dim, uint32_t recent_window, uint32_t block_size) {
    return orc_ckv_create_fmt(max_seq_len, max_batch, kv_heads, head_dim, recent_window, block_size, 0u);
}
orc_ckv* orc_ckv_create_fmt(uint32_t max_seq_len, uint32_t max_batch, uint32_t kv_heads,
                            uint32_t head_dim, uint32_t recent_window, uint32_t block_size, uint32_t v_format) {
    if (recent_window == 0 || block_size == 0 || v_format > 1u) return NULL;
    if (head_dim != 64 && head_dim != 128) return NULL;
    orc_ckv* c = (orc_ckv*)calloc(1, sizeof(orc_ckv));
    c->max_seq_len = max_seq_len;
    c->max_batch = max_batch;
    c->kv_heads = kv_heads;
    c->head_dim = head_dim;
    c->recent_window = recent_window;
    c->block_size = block_size;
    const size_t ept = (size_t)kv_heads * head_dim;
    c->recent_k = (uint16_t*)calloc((size_t)max_batch * recent_window * ept, 2);
    c->recent_v = (uint16_t*)calloc((size_t)max_batch * recent_window * ept, 2);
    c->old_k = (uint16_t*)calloc((size_t)max_batch * max_seq_len * ept, 2);
    c->q4_v = (uint8_t*)calloc((size_t)max_batch * max_seq_len * kv_heads * (head_dim / 2), 1);
    c->q4_scale = (float*)calloc((size_t)max_batch * max_seq_len * kv_heads, 4);
    c->v_format = v_format;
    c->q4_dm = v_format ? (uint32_t*)calloc((size_t)max_batch * max_seq_len * kv_heads * (head_dim / 32), 4) : NULL;
    c->seq_map = (uint32_t*)calloc(max_batch, 4);
    return c;
}
void orc_ckv_destroy(orc_ckv* c) {
    if (!c) return;
    free(c->recent_k); free(c->recent_v); free(c->old_k);
    free(c->q4_v); free(c->q4_scale); free(c->q4_dm); free(c->seq_map);
    free(c);
}
size_t orc_ckv_bytes_old_k(const orc_ckv* c) {
    return (size_t)c->max_batch * c->max_seq_len * c->kv_heads * c->head_dim * 2;
}
size_t orc_ckv_bytes_q4_v(const orc_ckv* c) {
    return (size_t)c->max_batch * c->max_seq_len * c->kv_heads * (c->head_dim / 2);
}
size_t orc_ckv_bytes_q4_scale(const orc_ckv* c) {
    if (c->v_format) return (size_t)c->max_batch * c->max_seq_len * c->kv_heads * (c->head_dim / 32) * 4;
    return (size_t)c->max_batch * c->max_seq_len * c->kv_heads * 4;
}

/* pack_q4_pair / quantize_evicted_recent_v_to_q4_old_kernel,
 * cuda/kernels.cu:2254-2311 (CPU twin tests/attention_parity_cuda_grid.rs:1471-1505):
 * scale = max|v|/7 (1/7 when all zero), q = clamp(lrintf(v/scale), -7, 7),
 * byte = (q_even & 15) | ((q_odd & 15) << 4). */
void orc_q4_quantize_row(const uint16_t* v_f16, uint32_t head_dim, uint8_t* packed, float* scale) {
    float max_v = 0.0f;
    for (uint32_t d = 0; d < head_dim; ++d) max_v = fmaxf(max_v, fabsf(h2f(v_f16[d])));
    const float sc = max_v > 0.0f ? max_v / 7.0f : 1.0f / 7.0f;
    *scale = sc;
    for (uint32_t pair = 0; pair < head_dim / 2u; ++pair) {
        const float a = h2f(v_f16[2 * pair]);
        const float b = h2f(v_f16[2 * pair + 1]);
        long qa = lrintf(a / sc), qb = lrintf(b / sc);
        if (qa < -7) qa = -7; if (qa > 7) qa = 7;
        if (qb < -7) qb = -7; if (qb > 7) qb = 7;
        packed[pair] = (uint8_t)(((int)qa & 0x0f) | (((int)qb & 0x0f) << 4));
    }
}

/* unpack_q4, cuda/kernels.cu:2260-2264 */
float orc_q4_unpack(uint8_t packed, uint32_t lane, float scale) {
    const uint8_t nib = lane == 0u ? (packed & 0x0f) : ((packed >> 4) & 0x0f);
    const int sv = nib >= 8u ? (int)nib - 16 : (int)nib;
    return (float)sv * scale;
}

/* 4-bit V in groups of 32 with an f16 scale and an f16 minimum (the V format the compressed-attention benchmark
 * configuration names; the reference has no such format, so this definition is the contract):
 *   per group: mn, mx = smallest and largest value; d = f16((mx - mn) / 15), m = f16(mn), both then read back as f32;
 *   q = d > 0 ? clamp(lrintf((v - m) / d), 0, 15) : 0;  byte = q_even | q_odd << 4;  word = bits(d) | bits(m) << 16;
 *   value = fmaf((float)q, d, m)  (one rounding, no pass through f16). */
void orc_q4g32_quantize_row(const uint16_t* v_f16, uint32_t head_dim, uint8_t* packed, uint32_t* dm) {
    for (uint32_t g = 0; g < head_dim / 32u; ++g) {
        float mn = h2f(v_f16[32 * g]), mx = mn;
        for (uint32_t i = 1; i < 32u; ++i) {
            const float v = h2f(v_f16[32 * g + i]);
            mn = fminf(mn, v); mx = fmaxf(mx, v);
        }
        const uint16_t db = orc_f32_to_f16((mx - mn) / 15.0f), mb = orc_f32_to_f16(mn);
        const float d = h2f(db), m = h2f(mb);
        dm[g] = (uint32_t)db | ((uint32_t)mb << 16);
        for (uint32_t pair = 0; pair < 16u; ++pair) {
            long q[2];
            for (int e = 0; e < 2; ++e) {
                const float v = h2f(v_f16[32 * g + 2 * pair + e]);
                q[e] = d > 0.0f ? lrintf((v - m) / d) : 0;
                if (q[e] < 0) q[e] = 0;
                if (q[e] > 15) q[e] = 15;
            }
            packed[16 * g + pair] = (uint8_t)((int)q[0] | ((int)q[1] << 4));
        }
    }
}
float orc_q4g32_unpack(uint8_t packed, uint32_t lane, uint32_t dm) {
    const uint8_t nib = lane == 0u ? (packed & 0x0f) : ((packed >> 4) & 0x0f);
    return fmaf((float)nib, h2f((uint16_t)(dm & 0xffffu)), h2f((uint16_t)(dm >> 16)));
}

/* m40llm_kvcache_append_token_f32_rope_k_compressed_at_layout_async,
 * cuda/kernels.cu:6108-6250: evict ring slot pos%W to old index pos-W first,
 * then overwrite the ring slot; seq_map[seq] = pos+1.  Error codes as there. */
int orc_ckv_append_rope_k_at(orc_ckv* c, uint32_t seq, uint32_t position,
                             const float* k_f32, const float* v_f32,
                             float freq_base, float freq_scale, uint32_t layout) {
    if (!c || !k_f32 || !v_f32) return -1;
    if (seq >= c->max_batch) return -3;
    if (position >= c->max_seq_len) return -5;
    const uint32_t W = c->recent_window, kvh = c->kv_heads, hd = c->head_dim;
    const size_t ept = (size_t)kvh * hd;
    const uint32_t ring = position % W;
    uint16_t* rk = c->recent_k + ((size_t)seq * W + ring) * ept;
    uint16_t* rv = c->recent_v + ((size_t)seq * W + ring) * ept;
    if (position >= W) {
        const uint32_t old_pos = position - W;
        uint16_t* ok = c->old_k + ((size_t)seq * c->max_seq_len + old_pos) * ept;
        memcpy(ok, rk, ept * 2);
        for (uint32_t h = 0; h < kvh; ++h) {
            uint8_t* qv = c->q4_v + ((size_t)seq * c->max_seq_len + old_pos) * kvh * (hd / 2) +
                          (size_t)h * (hd / 2);
            float* sc = c->q4_scale + ((size_t)seq * c->max_seq_len + old_pos) * kvh + h;
            if (c->v_format)
                orc_q4g32_quantize_row(rv + (size_t)h * hd, hd, qv,
                                       c->q4_dm + (((size_t)seq * c->max_seq_len + old_pos) * kvh + h) * (hd / 32));
            else
                orc_q4_quantize_row(rv + (size_t)h * hd, hd, qv, sc);
        }
    }
    rope_k_to_f16(k_f32, rk, kvh, hd, position, freq_base, freq_scale, layout);
    for (size_t i = 0; i < ept; ++i) rv[i] = orc_f32_to_f16(v_f32[i]);
    c->seq_map[seq] = position + 1u;
    return 0;
}

/* Block scores over old K for one q head.  kbase points at token 0 of this
 * sequence ([max_seq_len][kvh][hd] f16).  Reference: device kernel
 * cuda/kernels.cu:2893-2912 (order 0), host twins :6526-6568. */
static uint32_t block_scores_impl(const uint16_t* kbase, uint32_t kv_heads, uint32_t head_dim,
                                  const float* qh, uint32_t kvh, uint32_t old_len,
                                  uint32_t block_size, int order,
                                  float* out_scores, double* out_f64) {
    const uint32_t nblk = old_len == 0 ? 0 : (old_len + block_size - 1) / block_size;
    const size_t ept = (size_t)kv_heads * head_dim;
    const float inv_sqrt = orc_inv_sqrt_head_dim(head_dim);
    for (uint32_t b = 0; b < nblk; ++b) {
        const uint32_t start = b * block_size;
        const uint32_t end = start + block_size < old_len ? start + block_size : old_len;
        const float len = (float)(end - start);
        if (order == 1) {
            double acc = 0.0;
            for (uint32_t t = start; t < end; ++t) {
                const uint16_t* k = kbase + (size_t)t * ept + (size_t)kvh * head_dim;
                for (uint32_t d = 0; d < head_dim; ++d)
                    acc += (double)qh[d] * (double)h2f(k[d]);
            }
            const double sc = acc / (double)(end - start) * (double)inv_sqrt;
            if (out_f64) out_f64[b] = sc;
            if (out_scores) out_scores[b] = (float)sc;
        } else if (order == 0) {
            float red[128];
            for (uint32_t tid = 0; tid < 128; ++tid) {
                float part = 0.0f;
                for (uint32_t t = start; t < end; ++t) {
                    const uint16_t* k = kbase + (size_t)t * ept + (size_t)kvh * head_dim;
                    for (uint32_t d = tid; d < head_dim; d += 128)
                        part = fmaf(qh[d], h2f(k[d]), part); /* nvcc contracts a*b+c */
                }
                red[tid] = part;
            }
            for (uint32_t stride = 64; stride > 0; stride >>= 1)
                for (uint32_t tid = 0; tid < stride; ++tid) red[tid] += red[tid + stride];
            out_scores[b] = (red[0] / len) * inv_sqrt;
        } else {
            /* order 2: 64 lanes, lane = g*C + c, C = head_dim/8 chunks, R = 64/C row groups */
            const uint32_t C = head_dim / 8u, R = 64u / C;
            float sum[64][8];
            for (uint32_t lane = 0; lane < 64; ++lane) {
                const uint32_t g = lane / C, c = lane % C;
                for (int j = 0; j < 8; ++j) sum[lane][j] = 0.0f;
                for (uint32_t t = start + g; t < end; t += R) {
                    const uint16_t* k = kbase + (size_t)t * ept + (size_t)kvh * head_dim + 8u * c;
                    for (int j = 0; j < 8; ++j) sum[lane][j] += h2f(k[j]);
                }
            }
            for (uint32_t stride = R / 2u; stride > 0; stride >>= 1) { /* butterfly over g */
                float nxt[64][8];
                for (uint32_t lane = 0; lane < 64; ++lane) {
                    const uint32_t other = lane ^ (stride * C);
                    for (int j = 0; j < 8; ++j) nxt[lane][j] = sum[lane][j] + sum[other][j];
                }
                memcpy(sum, nxt, sizeof(sum));
            }
            float part[64];
            for (uint32_t lane = 0; lane < 64; ++lane) {
                const uint32_t c = lane % C;
                float p = 0.0f;
                for (int j = 0; j < 8; ++j) p = fmaf(qh[8u * c + j], sum[lane][j], p);
                part[lane] = p;
            }
            for (uint32_t stride = 1; stride < C; stride <<= 1) { /* butterfly over c */
                float nxt[64];
                for (uint32_t lane = 0; lane < 64; ++lane) nxt[lane] = part[lane] + part[lane ^ stride];
                memcpy(part, nxt, sizeof(part));
            }
            out_scores[b] = (part[0] / len) * inv_sqrt;
        }
    }
    return nblk;
}

uint32_t orc_ckv_block_scores(const orc_ckv* c, uint32_t seq, const float* q_head, uint32_t kv_head,
                              uint32_t seq_len, uint32_t recent_window, uint32_t block_size,
                              int order, float* out_scores, double* out_scores_f64) {
    const uint32_t old_len = seq_len > recent_window ? seq_len - recent_window : 0;
    const uint16_t* kbase = c->old_k + (size_t)seq * c->max_seq_len * c->kv_heads * c->head_dim;
    return block_scores_impl(kbase, c->kv_heads, c->head_dim, q_head, kv_head, old_len,
                             block_size, order, out_scores, out_scores_f64);
}

/* Insertion with strict '>' into a descending list of length top_n initialised
 * to -1e30 / 0xffffffff: cuda/kernels.cu:2884-2927. */
uint32_t orc_select_top_blocks(const float* scores, uint32_t n_blocks, uint32_t top_blocks,
                               uint32_t* out_blocks, float* out_scores) {
    float sel_s[64];
    uint32_t sel_b[64];
    const uint32_t top_n = top_blocks < n_blocks ? top_blocks : n_blocks;
    for (uint32_t i = 0; i < 64; ++i) { sel_s[i] = -1e30f; sel_b[i] = 0xffffffffu; }
    for (uint32_t b = 0; b < n_blocks; ++b) {
        const float s = scores[b];
        uint32_t insert = top_n;
        for (uint32_t i = 0; i < top_n; ++i)
            if (s > sel_s[i]) { insert = i; break; }
        if (insert < top_n) {
            for (uint32_t j = top_n - 1; j > insert; --j) { sel_s[j] = sel_s[j - 1]; sel_b[j] = sel_b[j - 1]; }
            sel_s[insert] = s;
            sel_b[insert] = b;
        }
    }
    uint32_t count = 0;
    for (uint32_t i = 0; i < top_n; ++i) {
        if (sel_b[i] == 0xffffffffu) continue; /* append_unique_block skips empty slots, :263-271 */
        out_blocks[count] = sel_b[i];
        if (out_scores) out_scores[count] = sel_s[i];
        count++;
    }
    return count;
}

/* Softmax attention for one q head over an explicit token list; K/V fetched by
 * callbacks.  Three passes with the token-list order kept, as
 * cuda/kernels.cu:3024-3095. */
typedef struct {
    const orc_ckv* c;                 /* compressed backing, or NULL */
    const uint16_t* K; const uint16_t* V; /* dense backing */
    uint32_t max_seq_len, kv_heads, head_dim, seq, recent_start, recent_window;
} kv_src;

static const uint16_t* src_k_row(const kv_src* s, uint32_t t, uint32_t kvh) {
    if (s->c) {
        const size_t ept = (size_t)s->kv_heads * s->head_dim;
        if (t < s->recent_start)
            return s->c->old_k + ((size_t)s->seq * s->max_seq_len + t) * ept + (size_t)kvh * s->head_dim;
        return s->c->recent_k + ((size_t)s->seq * s->recent_window + (t % s->recent_window)) * ept +
               (size_t)kvh * s->head_dim;
    }
    return s->K + orc_kv_index(s->max_seq_len, s->kv_heads, s->head_dim, s->seq, t, kvh, 0);
}

static float src_v(const kv_src* s, uint32_t t, uint32_t kvh, uint32_t d) {
    if (s->c) {
        if (t < s->recent_start) {
            const size_t q4_base = ((size_t)s->seq * s->max_seq_len + t) * s->kv_heads * (s->head_dim / 2) +
                                   (size_t)kvh * (s->head_dim / 2);
            const size_t sc_idx = ((size_t)s->seq * s->max_seq_len + t) * s->kv_heads + kvh;
            if (s->c->v_format)
                return orc_q4g32_unpack(s->c->q4_v[q4_base + d / 2u], d & 1u,
                                        s->c->q4_dm[sc_idx * (s->head_dim / 32) + d / 32u]);
            const float v = orc_q4_unpack(s->c->q4_v[q4_base + d / 2u], d & 1u, s->c->q4_scale[sc_idx]);
            return h2f(orc_f32_to_f16(v)); /* rounded through f16, kernels.cu:3085-3086 */
        }
        const size_t ept = (size_t)s->kv_heads * s->head_dim;
        return h2f(s->c->recent_v[((size_t)s->seq * s->recent_window + (t % s->recent_window)) * ept +
                                             (size_t)kvh * s->head_dim + d]);
    }
    return h2f(s->V[orc_kv_index(s->max_seq_len, s->kv_heads, s->head_dim, s->seq, t, kvh, d)]);
}

static void attend_token_list(const kv_src* s, const float* qh, uint32_t kvh, const uint32_t* tokens,
                              uint32_t n, float* scores, float* out_h) {
    const float inv_sqrt = orc_inv_sqrt_head_dim(s->head_dim);
    float max_score = -1e30f;
    for (uint32_t i = 0; i < n; ++i) {
        const uint16_t* k = src_k_row(s, tokens[i], kvh);
        float dot = 0.0f;
        for (uint32_t d = 0; d < s->head_dim; ++d) dot += qh[d] * h2f(k[d]);
        scores[i] = dot * inv_sqrt;
        if (scores[i] > max_score) max_score = scores[i];
    }
    float denom = 0.0f;
    for (uint32_t i = 0; i < n; ++i) denom += expf(scores[i] - max_score);
    if (!(denom > 0.0f)) denom = 1.0f;
    for (uint32_t d = 0; d < s->head_dim; ++d) {
        float acc = 0.0f;
        for (uint32_t i = 0; i < n; ++i) {
            const float p = expf(scores[i] - max_score) / denom;
            acc += p * src_v(s, tokens[i], kvh, d);
        }
        out_h[d] = acc;
    }
}

static int block_select_attention(const kv_src* s, const uint16_t* kbase_scores, const float* q,
                                  uint32_t q_heads, uint32_t seq_len, uint32_t recent_window,
                                  uint32_t block_size, uint32_t top_blocks, int score_order,
                                  float* out, uint32_t* sel_blocks, uint32_t* sel_counts) {
    const uint32_t kv_heads = s->kv_heads, hd = s->head_dim;
    const uint32_t old_len = seq_len > recent_window ? seq_len - recent_window : 0;
    const uint32_t old_blocks = old_len == 0 ? 0 : (old_len + block_size - 1) / block_size;
    const uint32_t sel_old = top_blocks < old_blocks ? top_blocks : old_blocks;
    const uint32_t recent_count = seq_len < recent_window ? seq_len : recent_window;
    uint32_t old_cap = sel_old * block_size;
    if (old_cap > old_len) old_cap = old_len;
    const uint32_t capacity = recent_count + old_cap; /* cuda/kernels.cu:125-133 */
    if (capacity == 0 || capacity > seq_len) return -7;
    const uint32_t group = q_heads / kv_heads;
    int rc = 0;
#pragma omp parallel for schedule(dynamic)
    for (uint32_t h = 0; h < q_heads; ++h) {
        const uint32_t kvh = h / group;
        const float* qh = q + (size_t)h * hd;
        float* bs = (float*)malloc(sizeof(float) * (old_blocks ? old_blocks : 1));
        uint32_t* tokens = (uint32_t*)malloc(sizeof(uint32_t) * capacity);
        float* scores = (float*)malloc(sizeof(float) * capacity);
        uint32_t blocks[64];
        block_scores_impl(kbase_scores, kv_heads, hd, qh, kvh, old_len, block_size, score_order, bs, NULL);
        const uint32_t nsel = orc_select_top_blocks(bs, old_blocks, top_blocks, blocks, NULL);
        uint32_t n = 0;
        for (uint32_t i = 0; i < nsel; ++i) {
            const uint32_t start = blocks[i] * block_size;
            const uint32_t end = start + block_size < old_len ? start + block_size : old_len;
            for (uint32_t t = start; t < end; ++t) tokens[n++] = t;
        }
        for (uint32_t t = old_len; t < seq_len; ++t) tokens[n++] = t;
        if (sel_blocks) {
            for (uint32_t i = 0; i < 64; ++i) sel_blocks[(size_t)h * 64 + i] = i < nsel ? blocks[i] : 0xffffffffu;
        }
        if (sel_counts) sel_counts[h] = nsel;
        if (n > 0 && n <= capacity) attend_token_list(s, qh, kvh, tokens, n, scores, out + (size_t)h * hd);
        free(bs); free(tokens); free(scores);
    }
    return rc;
}

/* m40llm_attention_last_token_f32_gqa_block_select_exact_fp16_k_q4_v_old_direct_async,
 * cuda/kernels.cu:4504-4577 (argument checks and their codes) + kernel :2832-3096,
 * plain top-k policy, selected blocks kept in score-rank order. */
int orc_ckv_attention_block_select(const orc_ckv* c, uint32_t seq, const float* q, uint32_t q_heads,
                                   uint32_t seq_len, uint32_t recent_window, uint32_t block_size,
                                   uint32_t top_blocks, int score_order, float* out,
                                   uint32_t* sel_blocks, uint32_t* sel_counts) {
    if (!c || !q || !out) return -1;
    if (seq >= c->max_batch) return -2;
    if (seq_len == 0 || seq_len > c->max_seq_len) return -3;
    if (q_heads == 0 || c->kv_heads == 0 || q_heads % c->kv_heads != 0) return -4;
    if (c->head_dim != 64 && c->head_dim != 128) return -5;
    if (recent_window == 0 || block_size == 0 || top_blocks == 0 || top_blocks > 64) return -6;
    kv_src s;
    memset(&s, 0, sizeof(s));
    s.c = c; s.max_seq_len = c->max_seq_len; s.kv_heads = c->kv_heads; s.head_dim = c->head_dim;
    s.seq = seq; s.recent_window = recent_window;
    s.recent_start = seq_len > recent_window ? seq_len - recent_window : 0;
    const uint16_t* kbase = c->old_k + (size_t)seq * c->max_seq_len * c->kv_heads * c->head_dim;
    return block_select_attention(&s, kbase, q, q_heads, seq_len, recent_window, block_size,
                                  top_blocks, score_order, out, sel_blocks, sel_counts);
}

/* m40llm_attention_last_token_f32_gqa_block_select_exact_async,
 * cuda/kernels.cu:4025-4070 + kernel :1825-1983 (dense backing; the reference
 * accepts head_dim 64 only and returns -5 otherwise). */
int orc_dense_attention_block_select(const uint16_t* K, const uint16_t* V, uint32_t max_seq_len,
                                     uint32_t kv_heads, uint32_t head_dim, uint32_t seq,
                                     const float* q, uint32_t q_heads, uint32_t seq_len,
                                     uint32_t recent_window, uint32_t block_size,
                                     uint32_t top_blocks, int score_order, float* out,
                                     uint32_t* sel_blocks, uint32_t* sel_counts) {
    if (!K || !V || !q || !out) return -1;
    if (seq_len == 0 || seq_len > max_seq_len) return -3;
    if (q_heads == 0 || kv_heads == 0 || q_heads % kv_heads != 0) return -4;
    if (head_dim != 64 && head_dim != 128) return -5;
    if (recent_window == 0 || block_size == 0 || top_blocks == 0 || top_blocks > 64) return -6;
    kv_src s;
    memset(&s, 0, sizeof(s));
    s.K = K; s.V = V; s.max_seq_len = max_seq_len; s.kv_heads = kv_heads; s.head_dim = head_dim;
    s.seq = seq; s.recent_window = recent_window;
    s.recent_start = seq_len > recent_window ? seq_len - recent_window : 0;
    const uint16_t* kbase = K + (size_t)seq * max_seq_len * kv_heads * head_dim;
    return block_select_attention(&s, kbase, q, q_heads, seq_len, recent_window, block_size,
                                  top_blocks, score_order, out, sel_blocks, sel_counts);
}

/* m40llm_kvcache_debug_select_old_blocks over the fp16 old-K backing,
 * cuda/kernels.cu:6449-6677, plain top-k policy: q-head 0 against kv-head 0
 * (base has no head offset, :6533), sequential sum, score/len * scale, sort by
 * (score desc, block asc), window/block size taken from the cache. */
int orc_ckv_debug_select_old_blocks(const orc_ckv* c, uint32_t seq, const float* q_head0,
                                    uint32_t seq_len, uint32_t top_blocks,
                                    uint32_t* out_blocks, float* out_scores,
                                    uint32_t* out_start, uint32_t* out_end,
                                    uint32_t* out_count, uint32_t max_out,
                                    uint32_t* out_total_old_blocks) {
    if (!c || !q_head0 || !out_blocks || !out_scores || !out_start || !out_end || !out_count ||
        !out_total_old_blocks) return -1;
    if (seq >= c->max_batch) return -2;
    if (seq_len == 0 || seq_len > c->max_seq_len || max_out == 0) return -4;
    const uint32_t W = c->recent_window, bs = c->block_size, hd = c->head_dim;
    const uint32_t old_len = seq_len > W ? seq_len - W : 0;
    const uint32_t old_blocks = old_len == 0 ? 0 : (old_len + bs - 1) / bs;
    *out_total_old_blocks = old_blocks;
    *out_count = 0;
    if (old_blocks == 0) return 0;
    const float scale = hd == 64u ? 0.125f : 0.08838834764831845f;
    const size_t ept = (size_t)c->kv_heads * hd;
    const uint16_t* kbase = c->old_k + (size_t)seq * c->max_seq_len * ept;
    float* sc = (float*)malloc(sizeof(float) * old_blocks);
    uint32_t* idx = (uint32_t*)malloc(sizeof(uint32_t) * old_blocks);
    for (uint32_t b = 0; b < old_blocks; ++b) {
        const uint32_t start = b * bs, end = start + bs < old_len ? start + bs : old_len;
        float score = 0.0f;
        for (uint32_t pos = start; pos < end; ++pos)
            for (uint32_t d = 0; d < hd; ++d)
                score += q_head0[d] * h2f(kbase[(size_t)pos * ept + d]);
        score /= (float)(end - start);
        sc[b] = score * scale;
        idx[b] = b;
    }
    /* insertion sort by (score desc, block asc): same order as the std::sort comparator */
    for (uint32_t i = 1; i < old_blocks; ++i) {
        const uint32_t bi = idx[i];
        uint32_t j = i;
        while (j > 0 && (sc[idx[j - 1]] < sc[bi] || (sc[idx[j - 1]] == sc[bi] && idx[j - 1] > bi))) {
            idx[j] = idx[j - 1];
            --j;
        }
        idx[j] = bi;
    }
    uint32_t requested = top_blocks == 0 ? old_blocks : (top_blocks < old_blocks ? top_blocks : old_blocks);
    uint32_t capacity = requested < max_out ? requested : max_out;
    if (capacity > 64u) capacity = 64u;
    const uint32_t n = requested < capacity ? requested : capacity;
    for (uint32_t i = 0; i < n; ++i) {
        const uint32_t b = idx[i];
        out_blocks[i] = b;
        out_scores[i] = sc[b];
        out_start[i] = b * bs;
        out_end[i] = b * bs + bs < old_len ? b * bs + bs : old_len;
    }
    *out_count = n;
    free(sc); free(idx);
    return 0;
}

/* ------------------------------------------------------------------------ */
/* Sampling.  Reference: Sampler::sample with top_k = Some(1)                */
/* (src/sampling.rs:40-97 + softmax_temp :114-140), sample_greedy :99-112.   */
/* ------------------------------------------------------------------------ */
uint32_t orc_sample_greedy(const float* logits, size_t n) {
    size_t max_i = 0;
    float max_v = -INFINITY;
    for (size_t i = 0; i < n; ++i)
        if (logits[i] > max_v) { max_v = logits[i]; max_i = i; }
    return (uint32_t)max_i;
}

static int total_cmp_gt(float a, float b) { /* f32::total_cmp(a,b) == Greater */
    int32_t ia, ib;
    memcpy(&ia, &a, 4);
    memcpy(&ib, &b, 4);
    ia ^= (int32_t)(((uint32_t)(ia >> 31)) >> 1);
    ib ^= (int32_t)(((uint32_t)(ib >> 31)) >> 1);
    return ia > ib;
}

uint32_t orc_greedy_topk1(const float* logits, size_t n) {
    /* softmax_temp with temperature 1.0 */
    float max_logit = -INFINITY;
    for (size_t i = 0; i < n; ++i) {
        const float v = logits[i] * 1.0f;
        /* f32::max ignores NaN operands */
        if (v > max_logit || max_logit != max_logit) max_logit = v;
    }
    float* probs = (float*)malloc(sizeof(float) * n);
    float sum = 0.0f;
    for (size_t i = 0; i < n; ++i) {
        float x = expf(logits[i] * 1.0f - max_logit);
        if (!(isfinite(x) && x > 0.0f)) x = 0.0f;
        probs[i] = x;
        sum += x;
    }
    int all_zero = 0;
    if (sum <= 0.0f || !isfinite(sum)) {
        all_zero = 1;
    } else {
        for (size_t i = 0; i < n; ++i) {
            float p = probs[i] / sum;
            if (!isfinite(p) || p < 0.0f) p = 0.0f;
            probs[i] = p;
        }
    }
    uint32_t result;
    if (all_zero) {
        result = orc_sample_greedy(logits, n);
    } else if (n == 1) {
        result = 0;
    } else {
        /* stable descending sort by total_cmp, truncate to 1: first index of the maximum */
        size_t best = 0;
        for (size_t i = 1; i < n; ++i)
            if (total_cmp_gt(probs[i], probs[best])) best = i;
        if (!(probs[best] > 0.0f)) result = orc_sample_greedy(logits, n);
        else result = (uint32_t)best;
    }
    free(probs);
    return result;
}

float orc_top2_gap(const float* logits, size_t n) {
    float a = -INFINITY, b = -INFINITY;
    for (size_t i = 0; i < n; ++i) {
        const float v = logits[i];
        if (v > a) { b = a; a = v; }
        else if (v > b) b = v;
    }
    return a - b;
}

/* ------------------------------------------------------------------------ */
/* Whole-model decode.  Op order of one layer:                               */
/* forward_one_token_minimal_with_norms src/infer/forward.rs:304-662; slot =  */
/* seq*layers + layer src/infer/kv.rs:109-112; pos = seq_len-1; logits        */
/* src/infer/logits.rs:57-116; embedding row f16->f32                         */
/* src/infer/embeddings.rs:64-79.                                             */
/* ------------------------------------------------------------------------ */
orc_model_kv* orc_model_kv_create(const orc_model* m, uint32_t max_seq_len, uint32_t max_sequences) {
    orc_model_kv* kv = (orc_model_kv*)calloc(1, sizeof(orc_model_kv));
    kv->max_seq_len = max_seq_len;
    kv->max_sequences = max_sequences;
    const size_t elems = (size_t)max_sequences * m->n_layers * max_seq_len * m->kv_heads * m->head_dim;
    kv->K = (uint16_t*)calloc(elems, 2);
    kv->V = (uint16_t*)calloc(elems, 2);
    if (!kv->K || !kv->V) { free(kv->K); free(kv->V); free(kv); return NULL; }
    return kv;
}
void orc_model_kv_destroy(orc_model_kv* kv) {
    if (!kv) return;
    free(kv->K); free(kv->V); free(kv);
}

void orc_layer_forward(const orc_model* m, orc_model_kv* kv, uint32_t layer, uint32_t seq,
                       uint32_t pos, const float* x, float* out) {
    const uint32_t D = m->d_model, kv_dim = m->kv_heads * m->head_dim, F = m->ffn;
    float* xn = (float*)malloc(sizeof(float) * D);
    float* q = (float*)malloc(sizeof(float) * D);
    float* k = (float*)malloc(sizeof(float) * kv_dim);
    float* v = (float*)malloc(sizeof(float) * kv_dim);
    float* ctx = (float*)malloc(sizeof(float) * D);
    float* y = (float*)malloc(sizeof(float) * D);
    float* x1 = (float*)malloc(sizeof(float) * D);
    float* gate = (float*)malloc(sizeof(float) * F);
    float* up = (float*)malloc(sizeof(float) * F);
    const uint32_t slot = seq * m->n_layers + layer;

    orc_rms_norm_weighted(x, m->attn_norm[layer], xn, 1, D, m->rms_eps, 1);
    orc_gemm_f32xf16_gguf(xn, m->wq[layer], q, 1, (int)D, (int)D);
    orc_gemm_f32xf16_gguf(xn, m->wk[layer], k, 1, (int)kv_dim, (int)D);
    orc_gemm_f32xf16_gguf(xn, m->wv[layer], v, 1, (int)kv_dim, (int)D);
    if (m->has_qkv_bias) {
        orc_residual_add(q, m->bq[layer], q, D);
        orc_residual_add(k, m->bk[layer], k, kv_dim);
        orc_residual_add(v, m->bv[layer], v, kv_dim);
    }
    orc_rope_inplace(q, 1, m->q_heads, m->head_dim, pos, m->rope_base, m->rope_scale, m->rope_layout);
    orc_kv_append_f32_rope_k(kv->K, kv->V, kv->max_seq_len, m->kv_heads, m->head_dim, slot, pos,
                             k, v, m->rope_base, m->rope_scale, m->rope_layout);
    orc_attention_last_token_gqa(kv->K, kv->V, kv->max_seq_len, m->kv_heads, m->head_dim, slot,
                                 q, m->q_heads, pos + 1, ctx);
    orc_gemm_f32xf16_gguf(ctx, m->wo[layer], y, 1, (int)D, (int)D);
    orc_residual_add(x, y, x1, D);
    orc_rms_norm_weighted(x1, m->ffn_norm[layer], xn, 1, D, m->rms_eps, 1);
    orc_gemm_f32xf16_gguf(xn, m->wgate[layer], gate, 1, (int)F, (int)D);
    orc_gemm_f32xf16_gguf(xn, m->wup[layer], up, 1, (int)F, (int)D);
    orc_swiglu(gate, up, gate, F);
    orc_gemm_f32xf16_gguf(gate, m->wdown[layer], y, 1, (int)D, (int)F);
    orc_residual_add(x1, y, out, D);

    free(xn); free(q); free(k); free(v); free(ctx); free(y); free(x1); free(gate); free(up);
}

void orc_token_forward(const orc_model* m, orc_model_kv* kv, uint32_t seq, uint32_t pos,
                       uint32_t token_id, float* hidden_out) {
    const uint32_t D = m->d_model;
    float* a = (float*)malloc(sizeof(float) * D);
    float* b = (float*)malloc(sizeof(float) * D);
    orc_f16_to_f32_n(m->tok_emb + (size_t)token_id * D, a, D);
    for (uint32_t l = 0; l < m->n_layers; ++l) {
        orc_layer_forward(m, kv, l, seq, pos, a, b);
        float* t = a; a = b; b = t;
    }
    memcpy(hidden_out, a, sizeof(float) * D);
    free(a); free(b);
}

/* Packed prefill of several prompts: all tokens of all prompts as rows of one batch, layer by layer
 * (src/infer/forward.rs:2153-2600).  Per layer: RMSNorm of every row, Q / K / V projections (+ bias), then per prompt
 * and token the append of the rotated K and of V to the f16 cache at the token's position and the rotation of the f32
 * Q and K rows in place (forward.rs:2349-2396); the packed causal attention runs on the f32 Q, K, V rows -- NOT on the
 * f16 cache, which is where this path differs from the token-by-token one (forward.rs:2404-2415) -- then O projection +
 * residual, RMSNorm, gate / up, SwiGLU, down + residual.  Every prompt starts at position 0.  hidden_out receives the
 * rows [total][d_model] of the last layer.  Returns 0, or the attention's argument-check code. */
int orc_prefill_forward(const orc_model* m, orc_model_kv* kv, const uint32_t* seq_ids, const uint32_t* lens,
                        const uint32_t* tokens, uint32_t batch, float* hidden_out) {
    const uint32_t D = m->d_model, kv_dim = m->kv_heads * m->head_dim, F = m->ffn;
    size_t rows = 0;
    uint32_t* offsets = (uint32_t*)malloc(sizeof(uint32_t) * (batch ? batch : 1));
    for (uint32_t i = 0; i < batch; ++i) { offsets[i] = (uint32_t)rows; rows += lens[i]; }
    float* a = (float*)malloc(sizeof(float) * rows * D);
    float* b = (float*)malloc(sizeof(float) * rows * D);
    float* xn = (float*)malloc(sizeof(float) * rows * D);
    float* q = (float*)malloc(sizeof(float) * rows * D);
    float* k = (float*)malloc(sizeof(float) * rows * kv_dim);
    float* v = (float*)malloc(sizeof(float) * rows * kv_dim);
    float* att = (float*)malloc(sizeof(float) * rows * D);
    float* y = (float*)malloc(sizeof(float) * rows * D);
    float* x1 = (float*)malloc(sizeof(float) * rows * D);
    float* gate = (float*)malloc(sizeof(float) * rows * F);
    float* up = (float*)malloc(sizeof(float) * rows * F);
    int rc = 0;
    for (size_t r = 0; r < rows; ++r) orc_f16_to_f32_n(m->tok_emb + (size_t)tokens[r] * D, a + r * D, D);
    for (uint32_t l = 0; l < m->n_layers && rc == 0; ++l) {
        orc_rms_norm_weighted(a, m->attn_norm[l], xn, (uint32_t)rows, D, m->rms_eps, 1);
        orc_gemm_f32xf16_gguf(xn, m->wq[l], q, (int)rows, (int)D, (int)D);
        orc_gemm_f32xf16_gguf(xn, m->wk[l], k, (int)rows, (int)kv_dim, (int)D);
        orc_gemm_f32xf16_gguf(xn, m->wv[l], v, (int)rows, (int)kv_dim, (int)D);
        if (m->has_qkv_bias)
            for (size_t r = 0; r < rows; ++r) {
                orc_residual_add(q + r * D, m->bq[l], q + r * D, D);
                orc_residual_add(k + r * kv_dim, m->bk[l], k + r * kv_dim, kv_dim);
                orc_residual_add(v + r * kv_dim, m->bv[l], v + r * kv_dim, kv_dim);
            }
        for (uint32_t i = 0; i < batch; ++i) {
            const uint32_t slot = seq_ids[i] * m->n_layers + l;
            for (uint32_t t = 0; t < lens[i]; ++t) {
                const size_t r = (size_t)offsets[i] + t;
                orc_kv_append_f32_rope_k(kv->K, kv->V, kv->max_seq_len, m->kv_heads, m->head_dim, slot, t, k + r * kv_dim,
                                         v + r * kv_dim, m->rope_base, m->rope_scale, m->rope_layout);
                orc_rope_inplace(q + r * D, 1, m->q_heads, m->head_dim, t, m->rope_base, m->rope_scale, m->rope_layout);
                orc_rope_inplace(k + r * kv_dim, 1, m->kv_heads, m->head_dim, t, m->rope_base, m->rope_scale, m->rope_layout);
            }
        }
        rc = orc_attention_prefill_gqa_varlen(q, k, v, offsets, offsets, lens, lens, batch, m->q_heads, m->kv_heads,
                                              m->head_dim, att);
        if (rc != 0) break;
        orc_gemm_f32xf16_gguf(att, m->wo[l], y, (int)rows, (int)D, (int)D);
        orc_residual_add(a, y, x1, rows * D);
        orc_rms_norm_weighted(x1, m->ffn_norm[l], xn, (uint32_t)rows, D, m->rms_eps, 1);
        orc_gemm_f32xf16_gguf(xn, m->wgate[l], gate, (int)rows, (int)F, (int)D);
        orc_gemm_f32xf16_gguf(xn, m->wup[l], up, (int)rows, (int)F, (int)D);
        orc_swiglu(gate, up, gate, rows * F);
        orc_gemm_f32xf16_gguf(gate, m->wdown[l], y, (int)rows, (int)D, (int)F);
        orc_residual_add(x1, y, b, rows * D);
        float* t = a; a = b; b = t;
    }
    if (rc == 0) memcpy(hidden_out, a, sizeof(float) * rows * D);
    free(offsets); free(a); free(b); free(xn); free(q); free(k); free(v); free(att); free(y); free(x1); free(gate); free(up);
    return rc;
}

void orc_logits(const orc_model* m, const float* hidden, float* logits) {
    float* xn = (float*)malloc(sizeof(float) * m->d_model);
    orc_rms_norm_weighted(hidden, m->out_norm, xn, 1, m->d_model, m->rms_eps, 1);
    orc_gemm_f32xf16_gguf(xn, m->lm_head, logits, 1, (int)m->vocab, (int)m->d_model);
    free(xn);
}

void orc_decode_greedy(const orc_model* m, orc_model_kv* kv, uint32_t seq,
                       const uint32_t* prompt, uint32_t n_prompt, uint32_t n_gen,
                       uint32_t start_pos, uint32_t* ids_out, float* gaps_out) {
    float* hidden = (float*)malloc(sizeof(float) * m->d_model);
    float* logits = (float*)malloc(sizeof(float) * m->vocab);
    uint32_t pos = start_pos;
    for (uint32_t i = 0; i < n_prompt; ++i) {
        ids_out[i] = prompt[i];
        orc_token_forward(m, kv, seq, pos++, prompt[i], hidden);
    }
    for (uint32_t g = 0; g < n_gen; ++g) {
        orc_logits(m, hidden, logits);
        const uint32_t next = orc_greedy_topk1(logits, m->vocab);
        if (gaps_out) gaps_out[g] = orc_top2_gap(logits, m->vocab);
        ids_out[n_prompt + g] = next;
        if (g + 1 < n_gen) orc_token_forward(m, kv, seq, pos++, next, hidden);
    }
    free(hidden); free(logits);
}
