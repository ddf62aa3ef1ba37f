/*
 * CPU oracle for the m40-llm decode-step hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  This library is the checker that the HIP path is
 * compared against; nothing shipped may call it.  Every function restates, in
 * plain scalar C, what the reference computes; the reference file:line it
 * follows is cited at each definition in oracle.c.
 *
 * Floating point: all arithmetic is IEEE binary32 with one rounding per
 * operation (built with -ffp-contract=off), sums run in the sequential order
 * of the reference's scalar loops.  Storage conversions f32<->f16 are
 * round-to-nearest-even, done in software here (no compiler half type).
 */
#ifndef M40_ORACLE_H
#define M40_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- scalar conversions ------------------------------------------------ */
uint16_t orc_f32_to_f16(float x);
float    orc_f16_to_f32(uint16_t h);
void     orc_f32_to_f16_n(const float* in, uint16_t* out, size_t n);
void     orc_f16_to_f32_n(const uint16_t* in, float* out, size_t n);

/* ---- KV layout ----------------------------------------------------------- */
size_t orc_kv_elems_per_token(uint32_t kv_heads, uint32_t head_dim);
size_t orc_kv_base(uint32_t max_seq_len, uint32_t kv_heads, uint32_t head_dim,
                   uint32_t seq, uint32_t token);
size_t orc_kv_index(uint32_t max_seq_len, uint32_t kv_heads, uint32_t head_dim,
                    uint32_t seq, uint32_t token, uint32_t head, uint32_t dim);

/* ---- elementwise --------------------------------------------------------- */
void orc_rms_norm(const float* in, float* out, uint32_t rows, uint32_t dim, float eps);
/* weight_dtype 0 = f16, 1 = f32; returns -4 for anything else */
int  orc_rms_norm_weighted(const float* in, const void* weight, float* out,
                           uint32_t rows, uint32_t dim, float eps, uint32_t weight_dtype);
/* layout 0 = adjacent pairs (2i,2i+1), 1 = NeoX split half (i, i+hd/2) */
void orc_rope_inplace(float* x, uint32_t rows, uint32_t num_heads, uint32_t head_dim,
                      uint32_t past_len, float freq_base, float freq_scale, uint32_t layout);
void orc_residual_add(const float* a, const float* b, float* out, size_t n);
void orc_swiglu(const float* gate, const float* up, float* out, size_t n);
void orc_q80_to_f32(const uint8_t* in_q80, float* out, size_t n);

/* ---- GEMM family (C[M,N] f32 row-major, f32 accumulate, k ascending) ----- */
void orc_gemm_f32xf16_gguf(const float* A, const uint16_t* B, float* C, int M, int N, int K);
void orc_gemm_f32xf16_rowmajor(const float* A, const uint16_t* B, float* C, int M, int N, int K);
void orc_gemm_f16xf16_rowmajor(const uint16_t* A, const uint16_t* B, float* C, int M, int N, int K);
/* B in q8_0 blocks along K for every output column (column stride = K/32*34 bytes) */
void orc_gemm_f32xq80_gguf(const float* A, const uint8_t* B_q80, float* C, int M, int N, int K);
/* out[M,d_model] = down( swiglu(gate(x), up(x)) ), all three matrices q8_0 */
void orc_ffn_swiglu_q80(const float* x, const uint8_t* w_gate, const uint8_t* w_up,
                        const uint8_t* w_down, float* scratch_gate, float* scratch_up,
                        float* out, int M, int d_model, int ffn);

/* ---- dense KV cache + attention ------------------------------------------ */
/* K,V: f16 [max_batch][max_seq_len][kv_heads][head_dim] */
void orc_kv_append_f32(uint16_t* K, uint16_t* V, uint32_t max_seq_len, uint32_t kv_heads,
                       uint32_t head_dim, uint32_t seq, uint32_t token,
                       const float* k_f32, const float* v_f32);
void orc_kv_append_f32_rope_k(uint16_t* K, uint16_t* V, uint32_t max_seq_len, uint32_t kv_heads,
                              uint32_t head_dim, uint32_t seq, uint32_t position,
                              const float* k_f32, const float* v_f32,
                              float freq_base, float freq_scale, uint32_t layout);
void orc_attention_last_token_gqa(const uint16_t* K, const uint16_t* V, uint32_t max_seq_len,
                                  uint32_t kv_heads, uint32_t head_dim, uint32_t seq,
                                  const float* q, uint32_t q_heads, uint32_t seq_len, float* out);
void orc_attention_last_token_gqa_batched(const uint16_t* K, const uint16_t* V,
                                          uint32_t max_seq_len, uint32_t kv_heads,
                                          uint32_t head_dim, const uint32_t* seq_ids,
                                          const uint32_t* seq_lens, uint32_t batch,
                                          const float* q, uint32_t q_heads, float* out);
/* packed variable-length causal prefill attention, all f32 (cuda/kernels.cu:3749-3835, :4834-4895); returns the
 * reference's argument-check codes (-1, -2, -3, -9, -8) or 0 */
int orc_attention_prefill_gqa_varlen(const float* q, const float* k, const float* v,
                                     const uint32_t* q_offsets, const uint32_t* kv_offsets,
                                     const uint32_t* q_lens, const uint32_t* kv_lens, uint32_t batch,
                                     uint32_t q_heads, uint32_t kv_heads, uint32_t head_dim, float* out);
float orc_inv_sqrt_head_dim(uint32_t head_dim);

/* ---- fp16-K / q4-V compressed cache --------------------------------------- */
typedef struct orc_ckv {
    uint32_t max_seq_len, max_batch, kv_heads, head_dim, recent_window, block_size;
    uint16_t* recent_k;   /* [batch][W][kvh][hd] f16, slot = pos % W          */
    uint16_t* recent_v;
    uint16_t* old_k;      /* [batch][max_seq_len][kvh][hd] f16, index = pos-W  */
    uint8_t*  q4_v;       /* [batch][max_seq_len][kvh][hd/2]                    */
    float*    q4_scale;   /* [batch][max_seq_len][kvh]                          */
    uint32_t* seq_map;    /* [batch]                                             */
    uint32_t  v_format;   /* 0: reference q4 (one f32 scale per token and head); 1: groups of 32 with f16 scale + f16 min */
    uint32_t* q4_dm;      /* v_format 1: [batch][max_seq_len][kvh][hd/32], scale bits | min bits << 16 */
} orc_ckv;

orc_ckv* orc_ckv_create(uint32_t max_seq_len, uint32_t max_batch, uint32_t kv_heads,
                        uint32_t head_dim, uint32_t recent_window, uint32_t block_size);
/* the same cache with old V held 4-bit in groups of 32 under an f16 scale and an f16 minimum (no counterpart in the
 * reference: the benchmark configuration's V format, defined by orc_q4g32_quantize_row / orc_q4g32_unpack) */
orc_ckv* orc_ckv_create_fmt(uint32_t max_seq_len, uint32_t max_batch, uint32_t kv_heads,
                            uint32_t head_dim, uint32_t recent_window, uint32_t block_size, uint32_t v_format);
void     orc_q4g32_quantize_row(const uint16_t* v_f16, uint32_t head_dim, uint8_t* packed, uint32_t* dm);
float    orc_q4g32_unpack(uint8_t packed, uint32_t lane, uint32_t dm);
void     orc_ckv_destroy(orc_ckv* c);
size_t   orc_ckv_bytes_old_k(const orc_ckv* c);
size_t   orc_ckv_bytes_q4_v(const orc_ckv* c);
size_t   orc_ckv_bytes_q4_scale(const orc_ckv* c);
void     orc_q4_quantize_row(const uint16_t* v_f16, uint32_t head_dim, uint8_t* packed, float* scale);
float    orc_q4_unpack(uint8_t packed, uint32_t lane, float scale);
int      orc_ckv_append_rope_k_at(orc_ckv* c, uint32_t seq, uint32_t position,
                                  const float* k_f32, const float* v_f32,
                                  float freq_base, float freq_scale, uint32_t layout);
/* Block scores for one q head (ascending block id).  The reference holds three
 * summation orders for this one quantity (device kernel, host twin over the
 * fp16 backing, host twin over the dense backing: mean K first, then the dot).
 * order 0 = device-kernel order: per-dimension partial sums over the block's
 *           tokens, then a halving tree over 128 partials;
 * order 1 = double precision (gap reporting only);
 * order 2 = mean-K-first order, stated for 64 lanes: lane (g,c) sums rows
 *           t = start+g, start+g+R, ... of dims 8c..8c+7 (R = 512/head_dim),
 *           a halving butterfly joins the R row groups, each lane takes the
 *           fused-multiply-add dot of its 8 dims with q, and a butterfly over
 *           c (xor 1,2,4[,8]) joins the chunks.  This is the order the HIP
 *           kernel uses, so block ids can be compared exactly. */
uint32_t orc_ckv_block_scores(const orc_ckv* c, uint32_t seq, const float* q_head, uint32_t kv_head,
                              uint32_t seq_len, uint32_t recent_window, uint32_t block_size,
                              int order, float* out_scores, double* out_scores_f64);
/* Plain top-k with strict '>' insertion (ties keep the lower block id).
 * Returns the number selected; blocks in score-rank order. */
uint32_t orc_select_top_blocks(const float* scores, uint32_t n_blocks, uint32_t top_blocks,
                               uint32_t* out_blocks, float* out_scores);
/* Full per-call path.  sel_blocks/sel_counts may be NULL; sel_blocks is
 * [q_heads][64], filled with 0xffffffff beyond the count. */
int orc_ckv_attention_block_select(const orc_ckv* c, uint32_t seq, const float* q, uint32_t q_heads,
                                   uint32_t seq_len, uint32_t recent_window, uint32_t block_size,
                                   uint32_t top_blocks, int score_order, float* out,
                                   uint32_t* sel_blocks, uint32_t* sel_counts);
/* Same selection algorithm over a dense f16 cache (reference: head_dim 64 only) */
int orc_dense_attention_block_select(const uint16_t* K, const uint16_t* V, uint32_t max_seq_len,
                                     uint32_t kv_heads, uint32_t head_dim, uint32_t seq,
                                     const float* q, uint32_t q_heads, uint32_t seq_len,
                                     uint32_t recent_window, uint32_t block_size,
                                     uint32_t top_blocks, int score_order, float* out,
                                     uint32_t* sel_blocks, uint32_t* sel_counts);
/* Host twin used for telemetry: q-head 0 / kv-head 0 only, sequential sums,
 * sort by (score desc, block asc). */
int orc_ckv_debug_select_old_blocks(const orc_ckv* c, uint32_t seq, const float* q_head0,
                                    uint32_t seq_len, uint32_t top_blocks,
                                    uint32_t* out_blocks, float* out_scores,
                                    uint32_t* out_start, uint32_t* out_end,
                                    uint32_t* out_count, uint32_t max_out,
                                    uint32_t* out_total_old_blocks);

/* ---- sampling -------------------------------------------------------------- */
/* Sampler with top_k = 1: argmax of the temperature-1 softmax, stable
 * descending order (lowest index wins ties). */
uint32_t orc_greedy_topk1(const float* logits, size_t n);
/* first strict maximum of the raw logits */
uint32_t orc_sample_greedy(const float* logits, size_t n);
/* top-1 minus top-2 logit (for gap reporting) */
float    orc_top2_gap(const float* logits, size_t n);

/* ---- whole-model decode ---------------------------------------------------- */
typedef struct orc_model {
    uint32_t n_layers, d_model, q_heads, kv_heads, head_dim, ffn, vocab;
    float    rms_eps, rope_base, rope_scale;
    uint32_t rope_layout, has_qkv_bias;
    const uint16_t* const* wq;     /* [layers] -> f16 [d_model cols][d_model K]     */
    const uint16_t* const* wk;     /* [layers] -> f16 [kv_dim cols][d_model K]      */
    const uint16_t* const* wv;
    const uint16_t* const* wo;     /* [d_model cols][d_model K]                      */
    const uint16_t* const* wgate;  /* [ffn cols][d_model K]                          */
    const uint16_t* const* wup;
    const uint16_t* const* wdown;  /* [d_model cols][ffn K]                          */
    const float* const* bq;        /* [layers] or NULL entries                       */
    const float* const* bk;
    const float* const* bv;
    const float* const* attn_norm; /* f32 [d_model]                                  */
    const float* const* ffn_norm;
    const float*    out_norm;      /* f32 [d_model]                                  */
    const uint16_t* lm_head;       /* f16 [vocab cols][d_model K]                    */
    const uint16_t* tok_emb;       /* f16 [vocab][d_model]                           */
} orc_model;

/* Dense KV for the model: slot = sequence * n_layers + layer */
typedef struct orc_model_kv {
    uint32_t max_seq_len, max_sequences;
    uint16_t* K;
    uint16_t* V;
} orc_model_kv;

orc_model_kv* orc_model_kv_create(const orc_model* m, uint32_t max_seq_len, uint32_t max_sequences);
void          orc_model_kv_destroy(orc_model_kv* kv);
/* one decoder layer for one token at position pos (seq_len = pos+1) */
void orc_layer_forward(const orc_model* m, orc_model_kv* kv, uint32_t layer, uint32_t seq,
                       uint32_t pos, const float* x, float* out);
void orc_token_forward(const orc_model* m, orc_model_kv* kv, uint32_t seq, uint32_t pos,
                       uint32_t token_id, float* hidden_out);
/* packed prefill of several prompts as one batch of rows (src/infer/forward.rs:2153-2600): the attention runs on the
 * f32 K / V rows, the f16 cache is written on the side; hidden_out = [sum of lens][d_model] */
int  orc_prefill_forward(const orc_model* m, orc_model_kv* kv, const uint32_t* seq_ids, const uint32_t* lens,
                         const uint32_t* tokens, uint32_t batch, float* hidden_out);
void orc_logits(const orc_model* m, const float* hidden, float* logits);
/* prompt then n_gen greedy tokens; ids_out holds n_prompt+n_gen ids; gaps_out
 * (may be NULL) holds the top-1/top-2 logit gap of each generated token */
void orc_decode_greedy(const orc_model* m, orc_model_kv* kv, uint32_t seq,
                       const uint32_t* prompt, uint32_t n_prompt, uint32_t n_gen,
                       uint32_t start_pos, uint32_t* ids_out, float* gaps_out);

void orc_set_threads(int n);
int  orc_get_threads(void);

#ifdef __cplusplus
}
#endif
#endif
