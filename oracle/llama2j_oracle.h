/*
 * TEST INFRASTRUCTURE - NOT PART OF THE PRODUCT.
 *
 * CPU restatement of llama2j's per-token forward pass (its CPU mode), its
 * sampler (java.util.Random included), the group-int8 codec and the
 * checkpoint / quant-cache formats.  Only tests,
 * the smoke check and the cpu_baseline leg of the benchmark may link or
 * load this; the HIP library never does.
 *
 * Every function cites the reference file:line it restates.  Paths are
 * relative to the reference root; J/ = src/main/java/com/lastbot/llama2j/,
 * K/ = J/kernel/.
 *
 * The reference holds no golden vectors; each function is pinned by the
 * known answers, closed forms and brute-force checks in tests/test_oracle_*.py
 * (the reference was read, never executed: no JVM exists in this image).
 */
#ifndef LLAMA2J_ORACLE_H
#define LLAMA2J_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ORC_GROUP_SIZE 256          /* J/Run.java:27 */
#define ORC_GROUP_BYTES 264         /* J/Quant.java:35-37 : 256*8/8 + 8 */

/* ---- codec: J/Quant.java --------------------------------------------- */
int64_t orc_quant_nbytes(int64_t n_floats);                       /* :39-48  */
void orc_quant_encode(const float *in, int64_t n, uint8_t *out);  /* :156-193 */
void orc_quant_decode(const uint8_t *enc, int64_t float_index, int64_t size,
                      float *out);                                /* :79-108 */

/* ---- ops: the static CPU calls of the classes under K/ ------------------ */
void orc_rms(float *sum, const float *x, int size);                /* K/RootMeanSquare.java:25-35 */
void orc_wns_i8(float *out, const float *x, const uint8_t *enc, int64_t weight_index,
                const float *sum_of_squares, int size);            /* K/WeightNormalizeAndScale.java:32-77 */
void orc_matmul_i8(float *xout, const float *x, const uint8_t *enc, int64_t weight_index,
                   int n, int d);                                  /* K/MatMul.java:77-85 */
void orc_matmul_i8_aligned(float *xout, const float *x, const uint8_t *enc,
                           int64_t weight_index, int n, int d);    /* K/MatMul.java:97-151 */
void orc_matmul_i8_unaligned(float *xout, const float *x, const uint8_t *enc,
                             int64_t weight_index, int n, int d);  /* K/MatMul.java:153-212 */
void orc_matmul_f32(float *xout, const float *x, const float *w, int64_t weight_index,
                    int n, int d);                                 /* K/MatMul.java:29-60 */
void orc_rope_table(float *cos_t, float *sin_t, int dim, int head_size, int seq_len); /* K/ApplyRope.java:34-59 */
void orc_rope(float *q, float *k, const float *cos_t, const float *sin_t, int pos,
              int dim, int kv_dim);                                /* K/ApplyRope.java:61-92 */
void orc_attention_loop(const float *q, const float *key_cache, float *att, float *max,
                        int max_index, int64_t att_index, int64_t keybase, int kv_dim,
                        int query_index, int pos, int head_size); /* K/AttentionLoop.java:29-54 */
void orc_exp_sum_normalize(float *x, const float *max_value, int max_index, int64_t index,
                           int size);                              /* K/ExpSumNormalize.java:25-38 */
void orc_accum_weighted_value(float *xb, const float *att, const float *value_cache, int pos,
                              int xb_index, int64_t value_base, int head_size, int kv_dim,
                              int64_t att_index);                  /* K/AccumWeightedValue.java:31-88 */
void orc_accum(float *a, const float *b, int size);                /* K/Accum.java:26-30 */
void orc_silu_table(float *table);                                 /* K/Silu.java:47-57 : 8192 floats */
float orc_silu_lookup(const float *table, float val);              /* K/Silu.java:59-70 */
void orc_silu(float *hb, const float *hb2, const float *table, int hidden_dim); /* K/Silu.java:72-78 */
int orc_argmax(const float *logits, int n);                        /* J/Sampler.java:46-57 */

/* ---- model: J/Config, J/TransformerWeights, J/RunState, J/Run ----------- */
typedef struct {
    int32_t dim, hidden_dim, n_layers, n_heads, n_kv_heads, vocab_size, seq_len; /* J/Config.java:6-14 */
    int32_t shared_weights;                                                      /* J/Run.java:572 */
} orc_config;

enum { ORC_T_RMS_ATT = 0, ORC_T_WQ, ORC_T_WK, ORC_T_WV, ORC_T_WO, ORC_T_RMS_FFN,
       ORC_T_W1, ORC_T_W2, ORC_T_W3, ORC_T_RMS_FINAL, ORC_T_COUNT };  /* file order, J/TransformerWeights.java:54-111 */

typedef struct orc_model orc_model;

orc_model *orc_model_new(const orc_config *cfg);
void orc_model_free(orc_model *m);
int64_t orc_tensor_floats(const orc_config *cfg, int tensor);  /* float counts, J/TransformerWeights.java:54-111 */
const char *orc_tensor_name(int tensor);                       /* cache-file stems, same lines */
/* The model borrows nothing: bytes are copied in. */
int orc_model_set_quant(orc_model *m, int tensor, const uint8_t *bytes, int64_t nbytes);
int orc_model_set_emb(orc_model *m, const float *emb, int64_t nfloats);
int orc_model_set_wcls(orc_model *m, const float *wcls, int64_t nfloats);
uint8_t *orc_model_quant_ptr(orc_model *m, int tensor);        /* direct access for in-place generation */
float *orc_model_emb_ptr(orc_model *m);
float *orc_model_wcls_ptr(orc_model *m);                       /* == emb when shared */
/* activation taps (names follow J/RunState.java:20-34) */
enum { ORC_B_X = 0, ORC_B_XB, ORC_B_XB2, ORC_B_HB, ORC_B_HB2, ORC_B_Q, ORC_B_K, ORC_B_V,
       ORC_B_ATT, ORC_B_LOGITS, ORC_B_KCACHE, ORC_B_VCACHE, ORC_B_TMP1 };
float *orc_model_buffer(orc_model *m, int which);
void orc_model_reset(orc_model *m);                            /* zero KV cache and tmp1 (fresh RunState) */

/* per-layer taps, copied during forward once enabled: q,k (after RoPE), v, attention output,
 * x after the attention residual, SwiGLU output, x after the FFN residual */
enum { ORC_TAP_Q = 0, ORC_TAP_K, ORC_TAP_V, ORC_TAP_ATT_OUT, ORC_TAP_X_ATT, ORC_TAP_HB, ORC_TAP_X_FFN, ORC_TAP_COUNT };
int orc_model_enable_taps(orc_model *m);
float *orc_model_tap(orc_model *m, int which, int layer);

void orc_forward(orc_model *m, int token, int pos);            /* J/Run.java:62-169 */
/* Like orc_forward but stops after `n_layers_run` layers and skips the head; for op-level taps. */
void orc_forward_layers(orc_model *m, int token, int pos, int n_layers_run);
/* J/Run.java:611-685 with temperature 0.  out_tokens gets `next` of every iteration
 * executed (forced prompt ids included, a terminating 1 included); returns the final pos.
 * If logits_out != NULL it receives vocab floats per executed iteration.
 * seconds (may be NULL) = wall time from after the first iteration to the end (J/Run.java:682-684). */
int orc_generate_greedy(orc_model *m, const int32_t *prompt, int n_prompt, int steps,
                        int32_t *out_tokens, float *logits_out, double *seconds);

/* ---- sampling: J/Sampler.java, K/FindMax.java, J/Run.java:643-665 ---------- */
void orc_find_max(float *max, int max_index, const float *x, int64_t index, int size); /* K/FindMax.java:40-48 */
/* java.util.Random (the 48-bit linear congruential generator of the Java SE specification, which
 * J/Sampler.java:17-25 uses through nextFloat): seed scrambled with 0x5DEECE66D, next(bits) =
 * top bits of seed*0x5DEECE66D+0xB mod 2^48, nextFloat = next(24) / 2^24. */
typedef struct orc_sampler orc_sampler;
orc_sampler *orc_sampler_new(int64_t rng_seed, int vocab_size);     /* J/Sampler.java:24-31 */
void orc_sampler_free(orc_sampler *s);
int32_t orc_sampler_next_bits(orc_sampler *s, int bits);            /* java.util.Random.next */
float orc_sampler_next_float(orc_sampler *s);                       /* J/Sampler.java:20-22 */
int orc_sample(orc_sampler *s, const float *probs, int n);          /* J/Sampler.java:33-44 */
/* J/Sampler.java:76-120, including its whole-array sort: entries beyond the candidates of this call
 * keep what earlier calls left there and take part in the sort.  Returns -1 for a NaN and -2 when no probability
 * reaches the cutoff (the reference throws in both cases). */
int orc_sample_topp(orc_sampler *s, const float *probs, int n, float topp);
/* The same two with the random draw given by the caller instead of taken from the generator. */
int orc_sample_coin(const float *probs, int n, float coin);
int orc_sample_topp_coin(orc_sampler *s, const float *probs, int n, float topp, float coin);
/* J/Run.java:643-665: argmax at temperature 0, else divide, FindMax, ExpSumNormalize (logits become
 * probabilities in place) and sample / sample_topp (topp > 0.999 selects plain sampling). */
int orc_sample_step(orc_sampler *s, float *logits, int n, float temperature, float topp);
/* J/Run.java:611-685 with a sampler; as orc_generate_greedy otherwise. */
int orc_generate(orc_model *m, const int32_t *prompt, int n_prompt, int steps, float temperature,
                 float topp, int64_t rng_seed, int32_t *out_tokens, double *seconds);

/* ---- files: J/BinFileReader, J/BinFileWriter, J/TransformerWeights ------- */
int orc_write_quant_file(const char *path, const uint8_t *bytes, int64_t nbytes); /* J/BinFileWriter.java:20-34 */
int64_t orc_read_quant_file(const char *path, uint8_t *dst, int64_t cap);         /* J/TransformerWeights.java:219-221 */
/* Loads `<dir>/<base>.bin`; for each quant tensor uses `<dir>/<base>_<name>_256_8.quant`
 * when present, else encodes and writes it (J/TransformerWeights.java:191-232). */
orc_model *orc_load_checkpoint(const char *bin_path, int write_caches, char *err, int errlen);

/* ---- seeded synthetic tensors (benchmark inputs; not from the reference) -- */
/* value(seed, stream, i) = ((sum of four 16-bit fields of splitmix64(key)) - 131070) * scale,
 * key = seed*0x9E3779B97F4A7C15 + stream*0xD1B54A32D192ED03 + i; scale = sigma / 37837.2265625 */
void orc_synth_fill(uint64_t seed, uint32_t stream, int64_t first, int64_t n, float sigma,
                    float *out);
/* Fill the whole model: stream ids 0 = embedding, 1..10 = quant tensors in file order,
 * 11 = classifier (unshared only).  Quant tensors are encoded 256-group-wise as they are made. */
void orc_model_fill_synth(orc_model *m, uint64_t seed, float sigma);
void orc_synth_prompt(uint64_t seed, int n, int vocab, int32_t *out);  /* ids uniform in [3, vocab) */

int orc_num_threads(void);

#ifdef __cplusplus
}
#endif
#endif
