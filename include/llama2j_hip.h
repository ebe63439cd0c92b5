/*
 * libllama2j_hip.so - C ABI of the MI355X (gfx950) mode of llama2j's per-token forward pass.
 *
 * The library owns every device buffer (weights, activations, KV cache), takes llama2j's own
 * weight formats, and runs the whole token, argmax and token-loop step included, as one hand-written
 * gfx950 kernel, captured in a hipGraph and replayed on one GPU.  It is the
 * seam a `Mode.HIP` plugs into beside the reference's CPU and CUDA modes: each entry point
 * names the reference interface it replaces (paths relative to the reference root,
 * J/ = src/main/java/com/lastbot/llama2j/, K/ = J/kernel/).
 *
 * Conventions: plain C, no exceptions cross the boundary, 0 = success and negative = error (the text is
 * kept per context, l2j_ctx_last_error, and per calling thread, l2j_last_error).  Entry points that run the forward pass are
 * not re-entrant per context, and forwards of different contexts of one process take turns (the
 * whole-token kernel occupies every compute unit); uploads are thread safe (the reference uploads from
 * ten threads, J/TransformerWeights.java:52,204).  There is no CPU fallback: without a GPU l2j_create fails.
 */
#ifndef LLAMA2J_HIP_H
#define LLAMA2J_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct l2j_ctx l2j_ctx;

enum {
    L2J_OK = 0,
    L2J_E_ARG = -1,    /* bad argument (null, out of range token/pos, unsupported shape) */
    L2J_E_SIZE = -2,   /* byte/float count does not match the tensor (J/TransformerWeights.java:228-232) */
    L2J_E_STATE = -3,  /* call not legal in this state (forward before finalize, upload after) */
    L2J_E_HIP = -4,    /* a HIP runtime call failed (J/ContextCUDA.java:296-304) */
    L2J_E_OOM = -5,    /* device or host allocation failed (J/ContextCPU.java:20-26) */
    L2J_E_IO = -6      /* file missing, short or malformed */
};

/* J/Config.java:6-14 plus the two facts J/Run.java:550,572 derives; the first seven fields are
 * the 7-int header of the checkpoint (J/Run.java:563-569). */
typedef struct {
    int32_t dim, hidden_dim, n_layers, n_heads, n_kv_heads, vocab_size, seq_len;
    int32_t shared_weights; /* classifier == embedding (J/Run.java:572) */
    int32_t group_size;     /* 256 only (J/Run.java:27) */
    int32_t bits;           /* 8 only   (J/Run.java:28) */
    int32_t device;         /* HIP device ordinal */
    uint32_t flags;         /* L2J_F_* */
} l2j_config;

#define L2J_F_EXACT_SILU 1u /* use exact sigmoid instead of the reference's lookup table (K/Silu.java:30) */

/* Tensors in checkpoint file order (J/TransformerWeights.java:50-122). */
enum l2j_tensor {
    L2J_TOK_EMB = 0, L2J_RMS_ATT, L2J_WQ, L2J_WK, L2J_WV, L2J_WO, L2J_RMS_FFN,
    L2J_W1, L2J_W2, L2J_W3, L2J_RMS_FINAL, L2J_WCLS, L2J_TENSOR_COUNT
};

/* Read-back taps, named after J/RunState.java:20-34.  L2J_B_K / L2J_B_V are the rows written to the
 * cache at the current position.  Per-layer taps (layer >= 0) are filled by l2j_forward_taps. */
enum l2j_buffer {
    L2J_B_X = 0,      /* residual stream; per-layer: after the FFN residual (J/Run.java:158) */
    L2J_B_XB,         /* per-layer: attention output before Wo (J/Run.java:129) */
    L2J_B_XB2,        /* per-layer: residual stream after the attention residual (J/Run.java:136) */
    L2J_B_HB,         /* per-layer: SwiGLU output (J/Run.java:152) */
    L2J_B_Q,          /* per-layer: q after RoPE (J/Run.java:88) */
    L2J_B_K,          /* per-layer: k after RoPE */
    L2J_B_V,          /* per-layer: v */
    L2J_B_LOGITS,     /* J/Run.java:168 */
    L2J_B_KCACHE,     /* (layer, seq_len, kv_dim) fp32, J/RunState.java:101 ; `off` counts from the layer base */
    L2J_B_VCACHE,
    L2J_B_COUNT
};

/* = new ContextCUDA + RunState device half (J/Context.java:16-23, J/RunState.java:107-166). */
int l2j_create(const l2j_config *cfg, l2j_ctx **out);
/* = Context.close / RunState.close (J/Run.java:697-701, J/ContextCUDA.java:311-323). */
void l2j_destroy(l2j_ctx *ctx);
/* Text of the calling thread's last failed call (also for calls that have no context, l2j_create included). */
const char *l2j_last_error(void);
/* Text of the last failed call on this context, whatever thread made it, copied into buf (NUL-terminated, at most
 * cap - 1 bytes); returns the length.  For callers whose threads move between two downcalls: the reference uploads
 * from ten virtual threads (J/TransformerWeights.java:52,204) and turns a device error into
 * RuntimeException(message) (J/ContextCUDA.java:296-304). */
int l2j_ctx_last_error(l2j_ctx *ctx, char *buf, int32_t cap);
int l2j_device_count(void);
/* Launch shapes and algorithm switches of one context, the counterpart of the constants the reference compiles into
 * its kernels' launch code (the block sizes in the K/ classes, J/Run.java:27-28).  A context starts from the process
 * defaults (environment variable L2J_<NAME>, read once by l2j_create; unset: the built-in value), this call overrides
 * one of them, and the library never reads the environment afterwards.  Before l2j_finalize: "threads" (workgroup size of the weight-streaming kernels; -1, the default: by the longest row), "grid",
 * "attn_threads", "attn_rows", "attn_nsplit", "fused_attn_rows", "fused_attn_splits", "barrier_spins", "fuse" (1 whole-token
 * kernel, 0 one launch per phase, -1 by model size), "layers_per_launch", "by_value", "self_contained", "fast_steps",
 * "token_special", "graph" (0: launch kernel by kernel instead of replaying captured hipGraphs), "graph_tokens" (tokens per
 * replay in the decode loops).  At any time: "sampler_scan", "sampler_exp_wgs", "fallback" (1: when a bounded wait of the
 * whole-token kernel runs out, because something else holds compute units of the GPU, the context switches to one launch
 * per phase for good and repeats the call; 0: the call returns L2J_E_HIP), "batch_fuse" (l2j_decode_greedy_batch: 1 runs the
 * layers of a step in one resident kernel with grid barriers instead of eight launches per layer; the same results,
 * slower as measured, 0 by default; a bounded wait of that kernel that runs out is L2J_E_HIP), "sampler_wide" (1, the default: a
 * sampling step of a vocabulary of at most 36864 is one launch of a workgroup per 256 probabilities with grid barriers; a
 * bounded wait of it that runs out is L2J_E_HIP, and the context sets the option to 0 itself: seed the sampler again and go on;
 * 0: one launch per stage, as larger vocabularies always take), "prefill" (0, the default: the decode loops take the prompt
 * positions one by one, as the reference does; 1: the first whole steps of 32 prompt positions go through l2j_prefill, the
 * loop goes on behind them: the same tokens but where two logits lie within rounding of each other; shapes l2j_prefill
 * does not take run as with 0), "prefill_flash" (the attention of l2j_prefill's steps: 1, the default: 16 positions at a time on
 * the fp32 matrix cores from position 64 on, where that is the faster form, every position for itself below; 2: always;
 * 0: never), "prefill_split" (workgroups that share the keys of a head and 16 positions there: 1 to 4; 0, the default:
 * one below position 192, then as many of up to four as the GPU has compute units for).  l2j_get_option reads the value in force
 * ("fuse" reads 0 after such a switch; "wall_clock_khz", read-only: the rate of the device clock that l2j_decode_greedy
 * times itself with, 0 when the device does not tell it). */
int l2j_set_option(l2j_ctx *ctx, const char *name, int32_t value);
int l2j_get_option(l2j_ctx *ctx, const char *name, int32_t *value);

/* = allocateQuantAndCopyToDevice (J/ContextCUDA.java:138-158, J/TransformerWeights.java:238-257).
 * `ref_bytes` is the exact payload of a .quant cache: ceil(n/256) groups of 264 bytes
 * (big-endian fp32 min, max, then 256 unsigned codes; J/Quant.java:156-193).  The memory is
 * borrowed for the call only.  nbytes must equal ceil(n/256)*264. */
int l2j_upload_quant(l2j_ctx *ctx, int tensor, const uint8_t *ref_bytes, uint64_t nbytes);
/* One layer of a per-layer tensor, so no caller needs a buffer above 2^31 bytes (the reference's
 * own int offsets overflow at 13B, J/TransformerWeights.java:89).  Legal only when a layer's float
 * count is a multiple of 256. */
int l2j_upload_quant_layer(l2j_ctx *ctx, int tensor, int layer, const uint8_t *ref_bytes, uint64_t nbytes);
/* = allocateAndCopyToDevice for the fp32 tensors (J/TransformerWeights.java:125-141):
 * L2J_TOK_EMB and L2J_WCLS (ignored when shared). */
int l2j_upload_f32(l2j_ctx *ctx, int tensor, const float *data, uint64_t nfloats);
/* = Quant.encode (J/Quant.java:156-193) run on the GPU straight into the device layout:
 * a quant tensor given as fp32, `first` = float offset inside the tensor (multiple of 256 unless
 * it is the only call).  Bit-identical codes and min/max to the reference's encoder. */
int l2j_upload_f32_quantize(l2j_ctx *ctx, int tensor, uint64_t first, const float *data, uint64_t nfloats);
/* Serialises a device tensor back to .quant payload bytes (groups [group0, group0+ngroups)). */
int l2j_read_quant(l2j_ctx *ctx, int tensor, uint64_t group0, uint64_t ngroups, uint8_t *ref_bytes_out);
/* Ends the load phase: tables (RoPE K/ApplyRope.java:34-59, SiLU K/Silu.java:47-57) are built,
 * the KV cache is zeroed and the per-token graph is captured. */
int l2j_finalize(l2j_ctx *ctx);
/* Zeroes the KV cache (a fresh RunState, J/RunState.java:141-151). */
int l2j_reset(l2j_ctx *ctx);

/* = Run.transformer + the logits copy (J/Run.java:44-51, 625-632).  logits may be NULL. */
int l2j_forward(l2j_ctx *ctx, int32_t token, int32_t pos, float *logits_or_null);
/* = Run.transformer + Sampler.argmax (J/Sampler.java:46-57) with a 4-byte read-back. */
int l2j_forward_argmax(l2j_ctx *ctx, int32_t token, int32_t pos, int32_t *next);
/* Same result as l2j_forward but launched kernel by kernel, copying every per-layer tap
 * (the pattern of Mode.TEST, J/Run.java:186-303). */
int l2j_forward_taps(l2j_ctx *ctx, int32_t token, int32_t pos, float *logits_or_null);
/* = the token loop of Run.main with temperature 0 (J/Run.java:599-603, 611-685): BOS first,
 * prompt ids forced as outputs, first-max argmax afterwards, stop after emitting token 1.
 * out_tokens (capacity min(steps, seq_len), or seq_len when steps <= 0) receives `next` of every
 * executed iteration, *n_out the final pos.  *seconds (may be NULL) = GPU time from the end of
 * the first iteration to the end of the last one (J/Run.java:682-684, 703-706): the last workgroup of every token
 * stores the device's wall clock (s_memrealtime, rate = hipDeviceAttributeWallClockRate, which
 * l2j_get_option("wall_clock_khz") reports) in its loop step, and *seconds is the difference of the two stamps;
 * 0 when the device does not tell the clock's rate. */
int l2j_decode_greedy(l2j_ctx *ctx, const int32_t *prompt, int32_t n_prompt, int32_t steps,
                      int32_t *out_tokens, int32_t *n_out, double *seconds);

/* Sixteen or thirty-two sequences at once (n_seq), every weight read once per step for all of them (the reference has
 * no counterpart: "parallel processing of multiple queries" is on its wish-list, README.md:347).  Every sequence runs
 * the token loop of l2j_decode_greedy (BOS first, its own prompt ids forced, first-maximum argmax afterwards) for
 * exactly `steps` positions; a sequence that emits token 1 keeps running and the caller cuts it there.  prompts: n_seq
 * rows of prompt_stride ids, n_prompt[b] of them used; out_tokens: n_seq rows of `steps` ids.  The products of the
 * quantized matrices run on the bf16 matrix cores with the arithmetic of K/MatMul.java:117-151 kept: a code is a bf16
 * exactly, an fp32 activation is cut exactly into three bf16, the products are exact and the sums fp32 (the fp32
 * classifier runs on the fp32 matrix cores); sums are formed in another order than in the single-sequence path, so
 * logits agree to rounding, not bit for bit.  The first call makes a second copy of the quantized matrices on the
 * device, in the order this path reads them (as large as the matrices themselves: 6.9 GB at the 7B shape), its
 * activation buffers, a KV cache of n_seq x steps rows per layer and the captured graph of a step; the context keeps
 * them until l2j_destroy, so later calls allocate and capture nothing unless they ask for another n_seq, more steps or
 * longer prompts (then the set is replaced).  The context's own cache is not touched.  L2J_E_OOM when the device
 * memory does not suffice (n_seq x n_layers x steps x kv_dim x 8 bytes of cache).
 * Needs dim and hidden_dim in whole groups of 256 and head_size 64, 128 or 256.
 * *seconds (may be NULL): GPU time from the end of the first step to the end of the last. */
int l2j_decode_greedy_batch(l2j_ctx *ctx, const int32_t *prompts, const int32_t *n_prompt, int32_t n_seq,
                            int32_t prompt_stride, int32_t steps, int32_t *out_tokens, double *seconds);
/* Gives back what the calls for several sequences at once keep on the device (l2j_decode_greedy_batch,
 * l2j_decode_sample_batch, l2j_prefill): the second copy of the quantized matrices, the activation buffers, the KV cache
 * of the sequences, their samplers and the captured graph.  The next such call makes them again (and pays for it: the
 * copy of the matrices is one pass over them).  The single-sequence path and its cache are not touched.  No counterpart
 * in the reference. */
int l2j_release_batch(l2j_ctx *ctx);

/* ---- sampling on the device: J/Sampler.java and the sampling branch of J/Run.java:643-665 ----
 * The context holds one sampler = the reference's Sampler object: a java.util.Random and the ProbIndex
 * array that sample_topp sorts whole, so that entries of earlier calls take part in later ones
 * (J/Sampler.java:17-18, 92-97).  Any vocab_size >= 2: up to 36864 probabilities are kept in LDS, larger vocabularies are
 * sampled where they lie in device memory (same results, slower). */
/* = new Sampler(rngSeed, vocab_size) (J/Sampler.java:24-31, J/Run.java:620). */
int l2j_sampler_seed(l2j_ctx *ctx, int64_t rng_seed);
/* One sampling step (J/Run.java:643-665): temperature 0 = Sampler.argmax; else logits /= temperature,
 * FindMax (K/FindMax.java:40-48), ExpSumNormalize (K/ExpSumNormalize.java:25-38), then Sampler.sample
 * (J/Sampler.java:33-44) when topp > 0.999, else Sampler.sample_topp (J/Sampler.java:76-120).
 * logits_or_null: vocab_size floats of the caller to sample from (Sampler's methods take the array), or NULL for
 * the logits of the last forward; either way they are probabilities afterwards (L2J_B_LOGITS), as in the reference.
 * coin: the caller's Random.nextFloat() in [0, 1), or negative to draw from the context's generator (one draw per
 * call, none at temperature 0).  A NaN among the probabilities is an error, as sample_topp throws. */
int l2j_sample(l2j_ctx *ctx, const float *logits_or_null, float temperature, float topp, float coin, int32_t *next);
/* = the token loop of Run.main with a sampler (J/Run.java:599-603, 611-685): as l2j_decode_greedy, but every
 * unforced token is sampled as in l2j_sample from a sampler seeded with rng_seed; the logits never leave the device. */
int l2j_decode_sample(l2j_ctx *ctx, const int32_t *prompt, int32_t n_prompt, int32_t steps, float temperature,
                      float topp, int64_t rng_seed, int32_t *out_tokens, int32_t *n_out, double *seconds);
/* l2j_decode_greedy_batch with a sampler per sequence: sequence s owns a new Sampler(rng_seeds[s], vocab_size) and every
 * unforced token of it is sampled as in l2j_sample (temperature 0: the argmax, no sampler is made), i.e. n_seq runs of the
 * loop of l2j_decode_sample side by side; the reference has neither ("parallel processing of multiple queries" is on its
 * wish-list, README.md:347).  After a step's forward pass the sampling step of all sequences runs as one launch per stage
 * (exponentials, probabilities and candidates, the sort's three stages, the pick), the sequences side by side in each;
 * it keeps a sequence's probabilities in LDS (vocab_size <= 36864, option "sampler_scan"
 * on: else L2J_E_STATE).  The context's own sampler is not touched.  logits (may be NULL): as in
 * l2j_decode_greedy_batch_logits, the logits of every step before sampling, (steps, n_seq, vocab_size) floats. */
int l2j_decode_sample_batch(l2j_ctx *ctx, const int32_t *prompts, const int32_t *n_prompt, int32_t n_seq,
                            int32_t prompt_stride, int32_t steps, float temperature, float topp, const int64_t *rng_seeds,
                            int32_t *out_tokens, double *seconds, float *logits);

/* ---- tokenizer: J/Tokenizer.java (host only) ----
 * Strings cross the boundary as NUL-terminated UTF-8; inside, comparisons are on UTF-16 code units as in Java. */
typedef struct l2j_tokenizer l2j_tokenizer;
/* = new Tokenizer(path, vocabSize) (J/Tokenizer.java:61-90): LE int32 max_token_length (ignored), then per token
 * LE fp32 score, LE int32 length, UTF-8 bytes. */
int l2j_tokenizer_open(const char *path, int32_t vocab_size, l2j_tokenizer **out);
void l2j_tokenizer_close(l2j_tokenizer *tok);
/* = bpe_encode (J/Tokenizer.java:102-163): dummy-prefix blank, per-character lookup with byte fallback, then the best
 * scoring merge until none applies.  *n gets the token count (also when cap is too small: L2J_E_SIZE).  Where the
 * reference throws ArrayIndexOutOfBoundsException (its byte fallback gives negative ids for bytes above 0x7f), this
 * returns L2J_E_ARG. */
int l2j_bpe_encode(l2j_tokenizer *tok, const char *prompt_utf8, int32_t *tokens, int32_t cap, int32_t *n);
/* = bpe_decode(token, next) (J/Tokenizer.java:189-208): the blank after BOS stripped, raw byte tokens "<0xNN>" as one
 * Latin-1 character or nothing for control codes.  *len = bytes written before the NUL, or -1 where the reference
 * returns null. */
int l2j_bpe_decode(l2j_tokenizer *tok, int32_t token, int32_t next, char *out_utf8, int32_t cap, int32_t *len);

/* Activation / cache taps.  layer < 0 reads the live buffer, layer >= 0 the per-layer tap.
 * `off` and `n` are in floats. */
int l2j_read(l2j_ctx *ctx, int which, int layer, uint64_t off, float *dst, uint64_t n);
/* Seeds or restores rows [pos0, pos0+npos) of one layer's KV cache (kv_dim floats per row). */
int l2j_write_kv(l2j_ctx *ctx, int layer, int32_t pos0, int32_t npos, const float *k, const float *v);
int l2j_sync(l2j_ctx *ctx);

/* ---- host side of the load path (no GPU needed) ---------------------------------------- */
/* = Quant.numberOfBytesByFloatSize / Quant.encode / Quant.decode (J/Quant.java:39-48,156-193,79-108). */
uint64_t l2j_quant_nbytes(uint64_t nfloats);
int l2j_quant_encode(const float *in, uint64_t nfloats, uint8_t *out);
int l2j_quant_decode(const uint8_t *enc, uint64_t float_index, uint64_t size, float *out);
/* = BinFileWriter.write / the cache read in readAsQuant (J/BinFileWriter.java:20-34,
 * J/TransformerWeights.java:219-221): little-endian int32 byte count, then the bytes. */
int l2j_write_quant_file(const char *path, const uint8_t *bytes, uint64_t nbytes);
int64_t l2j_read_quant_file(const char *path, uint8_t *dst, uint64_t cap);
/* Cache file name rule `<dir>/<base>_<tensor>_256_8.quant` (J/TransformerWeights.java:194,
 * J/Quant.java:195-197).  Returns the length written to `out` or a negative error. */
int l2j_quant_cache_path(const char *bin_path, int tensor, char *out, int cap);
/* Reads the 7-int header (J/Run.java:563-573) into cfg (group 256, bits 8, device 0, flags 0). */
int l2j_read_checkpoint_header(const char *bin_path, l2j_config *cfg);
/* = the TransformerWeights constructor (J/TransformerWeights.java:43-144,191-356) + Context +
 * RunState: reads the llama2.c v0 checkpoint, takes each `.quant` cache when present, otherwise
 * quantizes (on the GPU) and, when write_caches != 0, writes the cache; uploads; finalizes. */
int l2j_load_checkpoint(const char *bin_path, int device, uint32_t flags, int write_caches, l2j_ctx **out);
int l2j_get_config(l2j_ctx *ctx, l2j_config *cfg);

/* The forward passes of n consecutive positions pos0 .. pos0 + n - 1 of one sequence, tokens[i] being the input token of
 * position pos0 + i: what n calls of l2j_forward(tokens[i], pos0 + i) leave in the KV cache and return for the last of
 * them, i.e. the prompt positions of the token loop (J/Run.java:623-640: the reference runs them one by one through
 * Run.transformer), 32 positions per step through the batched products on the matrix cores (every weight read once per
 * 32 positions).  logits (null: not wanted): the vocab_size logits of the last position; they are also what l2j_sample
 * samples from next.  seconds (null: not wanted): device time of the steps.  The sums are formed in another order than
 * l2j_forward's, so cache rows and logits agree with its to rounding (1e-6 of the largest), not bit for bit.  Shapes as for
 * l2j_decode_greedy_batch (else L2J_E_SIZE: take l2j_forward); its buffers and its copy of the matrices are shared. */
int l2j_prefill(l2j_ctx *ctx, const int32_t *tokens, int32_t n, int32_t pos0, float *logits, double *seconds);

/* ======================================================================================================
 * Measurement and test entry points.  Not part of what a Mode.HIP binds: bench.py and the test-suite use them.
 * ====================================================================================================== */
/* Benchmark input: fills every tensor on the device with seeded values
 * ((sum of the four 16-bit fields of splitmix64(seed*0x9E3779B97F4A7C15 + stream*0xD1B54A32D192ED03 + i))
 *  - 131070) * (sigma / 37837.2265625f), stream 0 = embedding, 1..10 = quant tensors in file
 * order, 11 = classifier, and quantizes the ten quant tensors with the reference's encoder. */
int l2j_fill_synthetic(l2j_ctx *ctx, uint64_t seed, float sigma);
/* Measurement and test: the running float32 sums of n <= 16777216 non-negative terms in element order, as the reference's
 * loops form them one addition after the other (sum += x, K/ExpSumNormalize.java:31-33; cdf += probabilities[i],
 * J/Sampler.java:37-40, 100-117), computed by the routine the device sampler uses.  sums[i] = terms[0] + ... + terms[i]. */
int l2j_running_sums(l2j_ctx *ctx, const float *terms, int32_t n, float *sums);
/* Measurement and test: the same sums as the one-launch sampling step forms them (option "sampler_wide"; many workgroups,
 * 256 terms each), asked the questions the sampler asks (J/Sampler.java:37-40, 100-117): *total = the sum of the
 * n <= 36864 non-negative terms added in element order; for every limit, index[q] = the first i whose running sum
 * exceeds limits[q] (-1: none does) and sum[q] = that running sum.  n_limits <= 4096. */
int l2j_sum_probe(l2j_ctx *ctx, const float *terms, int32_t n, const float *limits, int32_t n_limits, int32_t *index, float *sum,
                  float *total);
/* l2j_running_sums for callers that cannot allocate device memory (tight serving loops, harnesses that forbid
 * hipMalloc, code that runs while another thread captures a graph); it has no counterpart in the reference.  Same
 * results, but the terms and sums pass through a fixed 144 KB device array of the library (one per GPU, held until the
 * process ends) instead of a buffer allocated per call: n <= 36864, else L2J_E_SIZE.  No hipMalloc / hipFree is made;
 * the call does copy from and to the caller's host memory and synchronizes the context's stream, so it is not itself
 * something to record into a capture.  Every call on a GPU shares that GPU's array, so calls that overlapped would race:
 * the library runs them one after the other.  The array keeps the last call's contents; a call reads none of them (it
 * only reads the n terms it has just copied in). */
int l2j_running_sums_noalloc(l2j_ctx *ctx, const float *terms, int32_t n, float *sums);
/* Test: l2j_decode_greedy_batch that also returns the logits of every step, (steps, n_seq, vocab_size) floats, so that
 * the batched path's arithmetic can be compared with the single-sequence path's and the CPU's step by step (they pass
 * through a device buffer of that size, allocated for the call). */
int l2j_decode_greedy_batch_logits(l2j_ctx *ctx, const int32_t *prompts, const int32_t *n_prompt, int32_t n_seq,
                                   int32_t prompt_stride, int32_t steps, int32_t *out_tokens, float *logits);
/* Measurement and test of the matrix-core kernel for several sequences at once (the reference has none: "parallel
 * processing of multiple queries" is on its wish-list, README.md:347): y[b][r] = sum_k dequant(W[r][k]) * x[b][k] for
 * sixteen activation vectors x (16 x K floats) against one layer's matrix of a quantized matrix tensor (L2J_WQ..L2J_W3;
 * K a multiple of 256), in the arithmetic of K/MatMul.java:117-151 (exact products, fp32 sums, group scale and offset;
 * see l2j_decode_greedy_batch).  y: 16 x rows floats.  groups_per_slice is ignored (a slice of K is four groups of 256
 * codes since the kernel keeps the activations in its waves' registers; the argument remains for callers built against
 * the earlier kernel).  The call makes the tile-ordered copy of the tensor if the context has none yet.  *mean_us (may be
 * NULL): mean time of `rounds` launches of the product kernel. */
int l2j_batch_matmul(l2j_ctx *ctx, int tensor, int layer, const float *x, float *y, int32_t groups_per_slice,
                     int32_t rounds, double *mean_us);
/* Measurement: launches one kernel class `rounds` times at position `pos`, back to back on the context's stream,
 * and returns the mean kernel time from the start/stop events of each launch.  L2J_K_TOKEN is the kernel the forward pass runs: every phase of
 * every layer and the classifier in one launch.  The other classes launch one phase of it as a kernel of its
 * own, once per layer (cold weights, as inside a token). */
enum l2j_kernel_class { L2J_K_QKV = 0, L2J_K_ATTENTION, L2J_K_WO, L2J_K_W13, L2J_K_W2, L2J_K_CLASSIFIER, L2J_K_TOKEN, L2J_K_COUNT };
int l2j_time_kernel(l2j_ctx *ctx, int kernel_class, int32_t pos, int32_t rounds, double *mean_us,
                    uint64_t *algorithmic_bytes);
/* Measurement: runs k_copy16 (reads nbytes, writes nbytes) `rounds` times; hardware byte counters of the
 * other kernels are scaled by what the same counters report for this kernel of known size. */
int l2j_calibration_copy(l2j_ctx *ctx, uint64_t nbytes, int32_t rounds);
/* Algorithmic bytes one token streams at position pos: weights in the reference's storage format
 * (264 bytes per 256 weights, fp32 classifier and embedding row) plus KV cache read and write. */
uint64_t l2j_bytes_per_token(const l2j_config *cfg, int32_t pos);

#ifdef __cplusplus
}
#endif
#endif
