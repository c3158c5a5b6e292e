/*
 * moonhip.h -- C ABI of the MI355X (gfx950) FP16 matrix-product / attention path for
 * moondream-zig.  Plain pointers and sizes only; f16 values travel as raw IEEE
 * binary16 bit patterns (uint16_t), row-major, exactly as Zig's []f16 lays them out.
 *
 * Every entry point names the reference interface it replaces (file:line in the
 * reference tree).  All functions return MOON_OK (0) or a negative-free error code
 * below; moon_last_error() gives the text.  A moon_ctx owns one HIP stream, its
 * device workspaces and the resident-weight registry.  Calls on one ctx are
 * serialised by an internal mutex (the reference calls these ops from one thread,
 * text_model.zig:139-180).  Host-pointer ops are synchronous: on return the result
 * is in the caller's host buffer.  Device-pointer ops (moon_dev_*) are asynchronous
 * on the ctx stream; moon_sync() waits for them.
 *
 * There is no CPU fallback: without a usable GPU moon_ctx_create() fails and no op
 * can be called.
 */
#ifndef MOONHIP_H
#define MOONHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef uint16_t moon_f16;
typedef struct moon_ctx moon_ctx;
typedef struct moon_text_model moon_text_model;
typedef struct moon_vision_model moon_vision_model;

/* Error codes; the Zig shim maps them back to the reference's error names. */
enum {
    MOON_OK = 0,
    MOON_EINVAL_DIM = 1,    /* error.InvalidTensorDimension   hgemm.zig:369-372, hgemm_trans.zig:408-411 */
    MOON_ESHAPE = 2,        /* error.IncompatibleTensorShapes hgemm.zig:378-381, hgemm_trans.zig:417-420 */
    MOON_ESEQ_TOO_LONG = 3, /* error.SequenceTooLong          attention.zig:769, text_model.zig:113,478 */
    MOON_ENOMEM = 4,        /* error.OutOfMemory */
    MOON_EHIP = 5,          /* a HIP runtime call failed; see moon_last_error() */
    MOON_EINVAL = 6,        /* null pointer / unsupported argument */
    MOON_EROT_DIM = 7,      /* error.InvalidRotationDimension rope.zig:141-143 */
    MOON_ETOKEN = 8,        /* error.TokenIdOutOfBounds       text_model.zig:125-128 */
    MOON_EEPS = 9,          /* error.InvalidEpsilon           ops.zig:1174-1176 */
    MOON_ENODEVICE = 10,    /* no HIP device: the library has no CPU path */
    MOON_EFORMAT = 11,      /* moondream.bin: error.InvalidMagicNumber / InvalidVersion / InvalidHeader / InvalidNameLength /
                             * InvalidShapeLength / InvalidRead / UnknownTensorName (weights.zig:74-196, 317), or a missing tensor */
    MOON_ETEMPERATURE = 12  /* error.InvalidTemperature       sampling.zig:343-345 */
};

/* sampling.SamplingMethod (sampling.zig:240-245) */
enum {
    MOON_SAMPLE_GREEDY = 0,      /* argmax; the temperature is not applied (sampling.zig:370-372) */
    MOON_SAMPLE_MULTINOMIAL = 1, /* softmax, draw from all of it        (sampling.zig:373-377, 276-297) */
    MOON_SAMPLE_TOP_K = 2,       /* softmax, draw from the k most probable (sampling.zig:378-383, 300-339) */
    MOON_SAMPLE_MIN_P = 3        /* draw from probabilities >= min_p * the largest (sampling.zig:384-387, 114-219) */
};

/* sampling.SamplingConfig (sampling.zig:248-254).  top_k and min_p are optionals in the reference; here a top_k of 0
 * stands for the missing value and is refused.  min_tokens_to_keep is not read by any of the reference's methods. */
typedef struct moon_sampling_config {
    int method;        /* a MOON_SAMPLE_* value */
    float temperature; /* logits are divided by it unless it is exactly 1; <= 0 -> MOON_ETEMPERATURE */
    size_t top_k;      /* MOON_SAMPLE_TOP_K only; min(top_k, n) may be at most 1024 */
    float min_p;       /* MOON_SAMPLE_MIN_P only */
} moon_sampling_config;

/* epilogues fused into a matrix product */
enum {
    MOON_EPI_NONE = 0,      /* C = f16(acc)                                  hgemm.zig:138 */
    MOON_EPI_BIAS = 1,      /* C = f16(f16(acc) + bias)      + ops.broadcast_add_simd, ops.zig:1859-1913 */
    MOON_EPI_BIAS_GELU = 2  /* C = gelu(f16(f16(acc)+bias))  + ops.gelu, ops.zig:1635-1774 */
};

/* layout of the B operand */
enum {
    MOON_B_KN = 0, /* B[K,N] row-major: hgemm.matmul (vision weights, weights.zig:459-474) */
    MOON_B_NK = 1  /* B[N,K] row-major: hgemm_trans.matmul (text weights, weights.zig:439-454) */
};

/* ------------------------------------------------------------------ context */
int moon_ctx_create(int device, moon_ctx **out);
void moon_ctx_destroy(moon_ctx *ctx);
/* Text of the last error on this ctx (or of the last failed moon_ctx_create when ctx is NULL). */
const char *moon_last_error(const moon_ctx *ctx);
/* Measurement and test knob without a counterpart in the reference: names the matrix-product kernel that moon_hgemm,
 * moon_hgemm_trans, moon_linear and the sessions of this context take wherever the shape allows it ("regs", "dma",
 * "dma256", "w114", "w212", "w221"; "" or NULL: chosen by shape, the default).  Every kernel computes the same product to
 * the same rounding points; only the time changes.  The context starts with the value of MOON_GEMM_KERNEL. */
int moon_set_gemm_kernel(moon_ctx *ctx, const char *name);
/* Measurement aid without a counterpart in the reference: the name (with its grid and k split) of the kernel that the latest
 * matrix product, matrix-vector product or attention call on this context dispatched; "" before the first.  The text lives in
 * the context and changes with the next such call. */
const char *moon_last_kernel(const moon_ctx *ctx);
int moon_sync(moon_ctx *ctx);
/* Releases workspaces. Replaces attention.cleanupThreadPool() (attention.zig:814-818): the
 * reference frees its persistent worker pool there; here it drops cached device buffers. */
void moon_cleanup(moon_ctx *ctx);

/* ------------------------------------------------------------------ drop-in ops, host pointers */

/* hgemm.matmul(a[M,K], b[K,N]) -> c[M,N]   (hgemm.zig:362-426).
 * a_rows x a_cols and b_rows x b_cols are the two 2-D shapes; b_rows != a_cols -> MOON_ESHAPE. */
int moon_hgemm(moon_ctx *ctx, const moon_f16 *a, size_t a_rows, size_t a_cols,
               const moon_f16 *b, size_t b_rows, size_t b_cols, moon_f16 *c);

/* hgemm_trans.matmul(a[M,K], b_t[N,K]) -> c[M,N]   (hgemm_trans.zig:400-488; M==1 takes the
 * bandwidth-bound GEMV kernel like the reference's fast path :430-455). bt_cols != a_cols -> MOON_ESHAPE. */
int moon_hgemm_trans(moon_ctx *ctx, const moon_f16 *a, size_t a_rows, size_t a_cols,
                     const moon_f16 *b_t, size_t bt_rows, size_t bt_cols, moon_f16 *c);

/* Fused forms of "matmul then broadcast_add_simd (then gelu)" as the models call them
 * (text_model.zig:193-196, 310-315; vision_model.zig:279-282, 351-356). b_layout is MOON_B_KN / MOON_B_NK,
 * epilogue a MOON_EPI_* value; bias[N] may be NULL only for MOON_EPI_NONE. */
int moon_linear(moon_ctx *ctx, const moon_f16 *a, size_t M, size_t K, const moon_f16 *b, size_t N,
                int b_layout, const moon_f16 *bias, int epilogue, moon_f16 *c);

/* Keep a B operand (weight) resident on the device, keyed by its host address, so later
 * moon_hgemm / moon_hgemm_trans / moon_linear calls that pass the same pointer and size skip the upload.
 * The reference's per-layer weight tensors keep stable host addresses for the life of the model
 * (preslice_text.zig:53-79); the vision out_proj slice does not (vision_model.zig:332-335) and is
 * simply uploaded per call.  The caller must unregister before freeing or modifying the host buffer. */
int moon_weight_register(moon_ctx *ctx, const moon_f16 *host, size_t n_elems);
int moon_weight_unregister(moon_ctx *ctx, const moon_f16 *host);

/* attention.multiMasklessSDPA(n_heads, head_dim, q, k, v) (attention.zig:125-234).
 * q[n_heads,q_len,head_dim], k,v[n_heads,kv_len,head_dim] -> out[n_heads,q_len,head_dim]. */
int moon_sdpa_maskless(moon_ctx *ctx, const moon_f16 *q, const moon_f16 *k, const moon_f16 *v, moon_f16 *out,
                       size_t n_heads, size_t q_len, size_t kv_len, size_t head_dim);

/* attention.multiMaskedSDPA(q, k, v, mask, n_heads, head_dim) (attention.zig:416-541).
 * mask is Zig's Tensor(bool) data (one byte per element) of shape [1, q_len, mask_stride]. */
int moon_sdpa_masked(moon_ctx *ctx, const moon_f16 *q, const moon_f16 *k, const moon_f16 *v,
                     const uint8_t *mask, size_t mask_stride, moon_f16 *out,
                     size_t n_heads, size_t q_len, size_t kv_len, size_t head_dim);

/* attention.singleMaskedSDPA(q, k, v, mask) (attention.zig:759-811): q[32,1,64], k,v[32,kv_len,64],
 * mask[1,1,kv_len] -> out[32,1,64]; kv_len > 2048 -> MOON_ESEQ_TOO_LONG.  n_heads/head_dim are
 * arguments here (the reference hard-wires 32 x 64, attention.zig:248-249). */
int moon_sdpa_single(moon_ctx *ctx, const moon_f16 *q, const moon_f16 *k, const moon_f16 *v,
                     const uint8_t *mask, moon_f16 *out, size_t n_heads, size_t kv_len, size_t head_dim);

/* rope.applyRotEmb(x, n_heads, head_dim, freqs_cis, position_ids, rot_dim) (rope.zig:130-272).
 * x,out[n_heads,seq_len,head_dim]; freqs_cis is the caller's f32 table [table_rows, rot_dim/2, 2]
 * (rope.precomputeFreqsCis, rope.zig:32-128); position_ids[seq_len] are usize.
 * freq_pairs*2 != rot_dim -> MOON_EROT_DIM (rope.zig:141). */
int moon_rope_apply(moon_ctx *ctx, const moon_f16 *x, moon_f16 *out, size_t n_heads, size_t seq_len,
                    size_t head_dim, const float *freqs_cis, size_t table_rows, size_t freq_pairs,
                    const size_t *position_ids, size_t rot_dim);

/* ops.layerNorm(f16, x, weight, bias, eps) (ops.zig:1063-1419). eps <= 0 -> MOON_EEPS. */
int moon_layernorm(moon_ctx *ctx, const moon_f16 *x, const moon_f16 *gamma, const moon_f16 *beta,
                   moon_f16 *y, size_t rows, size_t dim, float eps);
/* ops.gelu(f16, &x) in place (ops.zig:1635-1774). */
int moon_gelu(moon_ctx *ctx, moon_f16 *x, size_t n);
/* ops.broadcast_add_simd(&a, b) for a[rows,cols] + b[cols] (ops.zig:1859-1913). */
int moon_bias_add(moon_ctx *ctx, moon_f16 *a, const moon_f16 *b, size_t rows, size_t cols);
/* ops.add(f16, &a, b) (ops.zig:312-323). */
int moon_add(moon_ctx *ctx, moon_f16 *a, const moon_f16 *b, size_t n);
/* sampling.argmax on f32(logits): first maximum wins (sampling.zig:257-273, moondream.zig:335-337). */
int moon_argmax(moon_ctx *ctx, const moon_f16 *logits, size_t n, size_t *index);
/* What createPatches and encode_image do between stbir_resize and the encoder (vision_model.zig:129-184) plus
 * rearrangeBCHWtoBTC (reshape_handler.zig:5-65): image[height, width, channels] u8 -> f16, taken twice (both crops hold the
 * same pixels), BHWC -> BCHW, / 255, (x - 0.5) / 0.5 (normalizePatch with mean = std = 0.5, reshape_handler.zig:67-96),
 * "b c (h p) (w q) -> b (h w) (c p q)": patches[2, (height/p)*(width/p), channels*p*p].  height or width not a multiple
 * of patch_size -> MOON_EINVAL_DIM (error.InvalidPatchSize).  Decoding the file and resizing it stay with stb on the host. */
int moon_image_patches(moon_ctx *ctx, const uint8_t *image, size_t height, size_t width, size_t channels, size_t patch_size,
                       moon_f16 *patches);
/* SamplingConfig's defaults (temperature 0.5, top_k 3, min_p 0.05; sampling.zig:250-252) with method greedy. */
void moon_sampling_config_default(moon_sampling_config *cfg);
/* sampling.sample(&f32(logits), config, rng, allocator) (sampling.zig:353-389, called at moondream.zig:335-337 and
 * moonchat.zig:597) on one row of n logits.  The reference draws one number per call from its PRNG,
 * rng.float(f32) in [0,1): pass it as u (unused by greedy); the generator stays with the caller.  The reference's sums
 * over the vocabulary are sequential f32 loops, and the candidate a draw lands on depends on their rounding: the device
 * answers from fast sums only where the answer provably does not depend on the rounding, and otherwise evaluates those
 * loops bit for bit (a few hundred microseconds; always for multinomial / min_p over thousands of near-equal
 * candidates, a few draws in 10^5 for top_k 3), so for the same exps the index is the reference's for every u.  (exp itself is the
 * classic two-part-reduction expf, error below one ulp, spelled out in csrc/sample.hip; a libm whose expf rounds some
 * argument differently can move a boundary by that last bit.)  top_k sorts at most 1024 candidates on the device: a
 * larger min(top_k, n) is refused with MOON_EINVAL, a deliberate limit (the reference's CLI default is 3). */
int moon_sample(moon_ctx *ctx, const moon_f16 *logits, size_t n, const moon_sampling_config *cfg, float u, size_t *index);
/* The same on the f32 row the reference's signature takes (sample(tensor: *Tensor(f32), ...), sampling.zig:353-358; at its
 * call sites the row is the f16 LM-head output cast to f32, moondream.zig:335): any f32 values are accepted. */
int moon_sample_f32(moon_ctx *ctx, const float *logits, size_t n, const moon_sampling_config *cfg, float u, size_t *index);
/* sampling.argmax(f32, tensor) (sampling.zig:257-273): first maximum wins. */
int moon_argmax_f32(moon_ctx *ctx, const float *logits, size_t n, size_t *index);

/* ------------------------------------------------------------------ device memory + device-pointer ops
 * The same kernels, on buffers that already live in HBM (what the benchmark times and what the
 * model sessions below are built from). */
int moon_dev_alloc(moon_ctx *ctx, size_t bytes, void **dptr);
int moon_dev_free(moon_ctx *ctx, void *dptr);
int moon_dev_upload(moon_ctx *ctx, void *dptr, const void *host, size_t bytes);
int moon_dev_download(moon_ctx *ctx, void *host, const void *dptr, size_t bytes);
/* Device-to-device copy by a plain kernel (bytes and both pointers multiples of 16); asynchronous on the context's
 * stream.  Its traffic is exactly `bytes` read + `bytes` written, which makes it the yardstick for counter readings. */
int moon_dev_copy(moon_ctx *ctx, void *dst, const void *src, size_t bytes);
/* Plain read of `bytes` (a multiple of 16, like the pointer) by a kernel that does nothing else; sink may be NULL or
 * point to 4 device bytes (never written for ordinary data).  No counterpart in the reference: it is the yardstick for
 * what one launch that streams this many bytes from HBM can reach on the device at hand. */
int moon_dev_read(moon_ctx *ctx, const void *src, size_t bytes, void *sink);
/* Deterministic synthetic data, bit-identical to the test generator on the host:
 * f16 ~N(0,std) (Irwin-Hall over splitmix64 counters) and uniform u32 in [0,modulo). */
int moon_dev_fill_normal_f16(moon_ctx *ctx, void *dptr, size_t n, uint64_t seed, uint64_t stream, float std_dev);
int moon_dev_fill_const_f16(moon_ctx *ctx, void *dptr, size_t n, float value);
int moon_dev_fill_uniform_u32(moon_ctx *ctx, void *dptr, size_t n, uint64_t seed, uint64_t stream, uint32_t modulo);

/* C[M,N] = epilogue(A[M,K] x B), B in b_layout.  M==1 with MOON_B_NK runs the GEMV kernel. */
int moon_dev_linear(moon_ctx *ctx, const void *a, size_t M, size_t K, const void *b, size_t N, int b_layout,
                    const void *bias, int epilogue, void *c);
/* causal_pos >= 0: row i may see keys j <= causal_pos + i (createAttentionMask(pos, seq_len),
 * attention.zig:256-281); causal_pos < 0: no mask.  mask (device, bytes, row stride mask_stride) may be
 * given instead for an arbitrary pattern. */
int moon_dev_sdpa(moon_ctx *ctx, const void *q, const void *k, const void *v, void *out, size_t n_heads,
                  size_t q_len, size_t kv_len, size_t head_dim, long causal_pos, const void *mask,
                  size_t mask_stride);
/* One decode-attention step on a KV cache in the reference layout [n_heads][max_seq][head_dim]
 * (text_model.zig:392-396): rotate q and the new k (first rot_dim dims, table on the device), append k', v at
 * position pos (updateCache, text_model.zig:476-515), attend over pos+1 keys.  qkv is [3*n_heads*head_dim]
 * (q | k | v, text_model.zig:198-226); out is [n_heads*head_dim] (already head-merged, :293-294). */
int moon_dev_decode_attention(moon_ctx *ctx, const void *qkv, void *cache_k, void *cache_v, const void *freqs_cis,
                              void *out, size_t n_heads, size_t head_dim, size_t rot_dim, size_t max_seq, size_t pos);
/* moon_dev_decode_attention for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments, same kernels and the same
 * result bits; the split-KV partials live in a static device array of the library (270,336 bytes per device, held until
 * the process ends) instead of a workspace grown on demand, so the call performs no hipMalloc / hipFree.  n_heads above
 * 128 -> MOON_EINVAL_DIM.  All calls on one device share that array: calls that overlap on one device (two contexts, two
 * threads) race; calls on one context are serialised as always.  Asynchronous on the context's stream. */
int moon_dev_decode_attention_noalloc(moon_ctx *ctx, const void *qkv, void *cache_k, void *cache_v, const void *freqs_cis,
                                      void *out, size_t n_heads, size_t head_dim, size_t rot_dim, size_t max_seq, size_t pos);
/* rope.precomputeFreqsCis(f32, dim, end, theta) (rope.zig:32-128) on the device: table[end, rot_dim/2, 2] f32 of
 * (cos, sin)(p * theta^(-2i/rot_dim)), the table the text session builds for itself (text_model.zig:88) and
 * moon_dev_decode_attention reads.  rot_dim odd or zero -> MOON_EROT_DIM. */
int moon_dev_rope_table(moon_ctx *ctx, void *table, size_t rot_dim, size_t end, float theta);
int moon_dev_layernorm(moon_ctx *ctx, const void *x, const void *gamma, const void *beta, void *y,
                       size_t rows, size_t dim, float eps);
/* moon_sample on logits that already sit in HBM; the index comes back to the host. */
int moon_dev_sample(moon_ctx *ctx, const void *logits, size_t n, const moon_sampling_config *cfg, float u, size_t *index);

/* HIP-event timer on the ctx stream (what the benchmark uses for kernel-level timing). */
int moon_timer_start(moon_ctx *ctx);
int moon_timer_stop(moon_ctx *ctx, float *elapsed_ms);

/* ------------------------------------------------------------------ text decoder session
 * Device-resident TextModel + KVCache (text_model.zig:39-345, 349-539).  Weights are given in the
 * moondream.bin text layout (weights.zig:439-454): per-layer matrices [L, out, in]. Host pointers;
 * they are uploaded once and may be freed afterwards. */
typedef struct moon_text_config {
    size_t vocab, dim, hidden_dim, n_layers, n_heads, head_dim, rot_dim, max_seq;
    float rope_theta, ln_eps;
} moon_text_config;

typedef struct moon_text_weights {
    const moon_f16 *word_token_embedding;      /* [vocab, dim] */
    const moon_f16 *t_ln_w, *t_ln_b;           /* [L, dim] */
    const moon_f16 *t_Wqkv_w, *t_Wqkv_b;       /* [L, 3*dim, dim], [L, 3*dim] */
    const moon_f16 *t_out_proj_w, *t_out_proj_b; /* [L, dim, dim], [L, dim] */
    const moon_f16 *t_fc1_w, *t_fc1_b;         /* [L, hidden, dim], [L, hidden] */
    const moon_f16 *t_fc2_w, *t_fc2_b;         /* [L, dim, hidden], [L, dim] */
    const moon_f16 *t_linear_w, *t_linear_b;   /* [vocab, dim], [vocab] */
    const moon_f16 *t_ln_out_w, *t_ln_out_b;   /* [dim] */
} moon_text_weights;

void moon_text_config_default(moon_text_config *cfg); /* config.zig:3-14 */
int moon_text_model_create(moon_ctx *ctx, const moon_text_config *cfg, const moon_text_weights *w,
                           moon_text_model **out);
/* Random-init decoder generated on the device: matrices, biases and the embedding ~N(0,std) from
 * (seed, stream = declaration order above), LayerNorm gamma = 1, beta = 0. */
int moon_text_model_create_synthetic(moon_ctx *ctx, const moon_text_config *cfg, uint64_t seed, float std_dev,
                                     moon_text_model **out);
void moon_text_model_destroy(moon_text_model *m);
/* KVCache.reset (text_model.zig:526-530). */
int moon_text_reset(moon_text_model *m);
/* text_encoder + text_decoder over n_ids tokens appended at the current cache length
 * (text_model.zig:106-180); n_ids == 1 runs the decode kernels. */
int moon_text_forward(moon_text_model *m, const uint32_t *ids, size_t n_ids);
/* TextModel.text_decoder as the reference's host calls it (text_model.zig:139-180; moondream.zig:296-327): the input is
 * rows of embeddings [n_rows, dim] in host memory (the image features and the prompt's embeddings side by side, later one
 * row per token), appended at the session's position.  moon_text_hidden then gives `output`. */
int moon_text_forward_embeds(moon_text_model *m, const moon_f16 *embeds, size_t n_rows);
/* TextModel.text_encoder (text_model.zig:106-137): embeds[n_ids, dim] = rows ids[i] of the embedding table, to host
 * memory.  Does not touch the session's position or cache.  error.TokenIdOutOfBounds -> MOON_ETOKEN. */
int moon_text_embed(moon_text_model *m, const uint32_t *ids, size_t n_ids, moon_f16 *embeds);
/* lm_head of the last position of the previous forward (text_model.zig:325-345) -> logits[vocab]. */
int moon_text_logits(moon_text_model *m, moon_f16 *logits);
/* n_steps of: lm_head -> argmax -> text_encoder([id]) -> text_decoder (moondream.zig:323-368),
 * entirely on the device; out_ids[n_steps]. */
int moon_text_greedy(moon_text_model *m, size_t n_steps, uint32_t *out_ids);
/* The same loop with sampling.sample in place of argmax (moondream.zig:323-368 with a sampling_config other than
 * greedy, moonchat.zig:597): n_steps of lm_head -> sample -> text_encoder([id]) -> text_decoder on the device,
 * logits never leave HBM.  u[n_steps] holds the numbers the reference would draw from its PRNG, one per step
 * (ignored, and may be NULL, for MOON_SAMPLE_GREEDY, which runs moon_text_greedy).  With top_k <= 3 the LM-head launch
 * itself decides the token wherever the four largest logits prove the reference's choice; every other draw, method and
 * top_k goes through the full evaluation of the row (the kernel behind moon_sample).  The ids are the same either way. */
int moon_text_sample(moon_text_model *m, const moon_sampling_config *cfg, const float *u, size_t n_steps, uint32_t *out_ids);
/* The generation loop of moondream.zig:323-368 (moonchat.zig:597-603) on the device: up to max_tokens steps of
 * {lm_head, sampling.sample (cfg == NULL or MOON_SAMPLE_GREEDY: arg-max), text_encoder of the new token, text_decoder},
 * ended early by the end-of-sequence token (moondream.zig:341: that token is not part of the output) or by the last cache
 * position (moondream.zig:324).  out_ids[max_tokens] receives the tokens, *n_out their number.  The host looks at the
 * device's state every 8 steps, so at most 8 steps are queued behind the stop; after a stop by the end-of-sequence token
 * the session needs a moon_text_forward before the next loop (the queued steps have overwritten its hidden state).
 * u[max_tokens]: as in moon_text_sample. */
int moon_text_generate(moon_text_model *m, const moon_sampling_config *cfg, const float *u, size_t max_tokens, uint32_t eos_token,
                       uint32_t *out_ids, size_t *n_out);
/* One step of that loop for a host that keeps the loop itself, as the reference does (moondream.zig:333-337:
 * text_model.lm_head + sampling.sample on the last position of the latest moon_text_forward): the token comes back, the
 * logits stay on the device.  The host then feeds it with moon_text_forward(m, &token, 1).  u: the reference's one draw
 * from its PRNG (ignored for the arg-max). */
int moon_text_next_token(moon_text_model *m, const moon_sampling_config *cfg, float u, uint32_t *token);
/* moon_text_greedy (decode modes 0, 2, 3) with a HIP event pair (on the library's stream) around every kernel launch:
 * avg_us[6] / launches[6] = average event interval and launch count of {LayerNorm+qkv+fc1 (in mode 0 the whole layer,
 * in mode 3 including the attention), rope+append+attention (mode 2 only), out_proj+fc2+residual (modes 2, 3), final
 * LayerNorm+LM head, arg-max, position bump}.  Where the LM-head launch also takes the arg-max and moves the position
 * on (the fused decode kernels), the last two kinds report no launches.  An interval holds the kernel plus the
 * command processor's work for the two events, a few microseconds more than the kernel alone.  Tokens and state
 * advance exactly as in moon_text_greedy; the host waits for the device after every step, so this call is for
 * measuring kernels, not throughput.
 * No counterpart in the reference (its bench.zig times whole ops on the host). */
int moon_text_greedy_profile(moon_text_model *m, size_t n_steps, uint32_t *out_ids, float *avg_us, size_t *launches);
/* How moon_text_greedy runs a decoder layer: 0 (default) = one kernel per layer (its workgroups hand qkv, fc1 and the
 * attention output to each other through counters, with bounded waits) where the device can hold enough of that
 * kernel's workgroups at once, else as mode 3 or 2; 2 = three kernels per layer and no waits inside kernels;
 * 3 = two kernels per layer (LayerNorm + qkv + fc1 + attention; out_proj + fc2 + residual).  All modes produce the same
 * bits.  A wait that expires makes the call return MOON_EHIP.  No counterpart in the reference. */
int moon_text_set_decode_mode(moon_text_model *m, int mode);
/* After a MOON_EHIP from moon_text_greedy / moon_text_sample caused by an expired wait inside a fused decode kernel the
 * session refuses further forward / greedy / sample calls until moon_text_reset: workgroups that gave up may have skipped
 * the cache append of their position.  moon_text_reset then also restarts the kernels' counters.
 * moon_text_debug_raise_wait_error sets the error word those waits look at, as an expired wait does (a test hook for
 * that path; no counterpart in the reference, whose ops cannot fail this way). */
int moon_text_debug_raise_wait_error(moon_text_model *m);
/* current KV length */
size_t moon_text_position(const moon_text_model *m);
/* Copy of the last forward's hidden states [n, dim] (n = tokens of that forward). */
int moon_text_hidden(moon_text_model *m, moon_f16 *hidden, size_t n_rows);
/* bytes of weights read per decoded token (layers + final LN + LM head) */
size_t moon_text_weight_bytes_per_token(const moon_text_model *m);

/* ------------------------------------------------------------------ vision encoder session
 * VisionModel.vision_encoder block loop (vision_model.zig:231-271) on a patch-embedding output
 * x[tokens, dim]; weights in the moondream.bin vision layout [L, in, out] (weights.zig:459-474). */
typedef struct moon_vision_config {
    size_t dim, hidden_dim, n_layers, n_heads, head_dim;
    float ln_eps;
} moon_vision_config;

typedef struct moon_vision_weights {
    const moon_f16 *v_Wqkv_w, *v_Wqkv_b;         /* [L, dim, 3*dim], [L, 3*dim] */
    const moon_f16 *v_out_proj_w, *v_out_proj_b; /* [L, dim, dim], [L, dim] */
    const moon_f16 *v_fc1_w, *v_fc1_b;           /* [L, dim, hidden], [L, hidden] */
    const moon_f16 *v_fc2_w, *v_fc2_b;           /* [L, hidden, dim], [L, dim] */
    const moon_f16 *v_norm1_w, *v_norm1_b, *v_norm2_w, *v_norm2_b; /* [L, dim] */
    const moon_f16 *v_norm_out_w, *v_norm_out_b; /* [dim] */
} moon_vision_weights;

void moon_vision_config_default(moon_vision_config *cfg); /* config.zig:16-26 */
int moon_vision_model_create(moon_ctx *ctx, const moon_vision_config *cfg, const moon_vision_weights *w,
                             moon_vision_model **out);
int moon_vision_model_create_synthetic(moon_ctx *ctx, const moon_vision_config *cfg, uint64_t seed, float std_dev,
                                       moon_vision_model **out);
void moon_vision_model_destroy(moon_vision_model *m);
/* x[tokens, dim] (host) -> out[tokens, dim] (host): n_layers blocks + final LayerNorm. */
int moon_vision_encode(moon_vision_model *m, const moon_f16 *x, size_t tokens, moon_f16 *out);
/* same with x/out already on the device (timed by the benchmark) */
int moon_vision_encode_dev(moon_vision_model *m, const void *x, size_t tokens, void *out);

/* The rest of VisionModel.encode_image around the encoder blocks (vision_model.zig:186-229, 366-387): the patch-embedding
 * product with its bias and the positional embedding in front (212-229), and behind the encoder the concatenation of the
 * two crops' features along the feature axis (189-196) and the projection MLP encode_mlp (366-387).  Attached to an encoder
 * session; matrices are given in the moondream.bin layout [in, out] (weights.zig:456-458, 476-479). */
typedef struct moon_vision_io_config {
    size_t patch_dim;   /* patch_size^2 * img_channels = 588 */
    size_t tokens;      /* num_patches = 729 per crop */
    size_t proj_hidden; /* 8192 */
    size_t out_dim;     /* 2048 */
} moon_vision_io_config;
typedef struct moon_vision_io_weights {
    const moon_f16 *v_patch_embedding_linear_w, *v_patch_embedding_linear_b; /* [patch_dim, dim], [dim] */
    const moon_f16 *v_pos_embedding;                                        /* [1, tokens, dim] */
    const moon_f16 *v_proj_fc1_w, *v_proj_fc1_b;                            /* [2 * dim, proj_hidden], [proj_hidden] */
    const moon_f16 *v_proj_fc2_w, *v_proj_fc2_b;                            /* [proj_hidden, out_dim], [out_dim] */
} moon_vision_io_weights;
void moon_vision_io_config_default(moon_vision_io_config *cfg); /* config.zig:16-26, 3-14 */
int moon_vision_io_attach(moon_vision_model *m, const moon_vision_io_config *cfg, const moon_vision_io_weights *w);
int moon_vision_io_attach_synthetic(moon_vision_model *m, const moon_vision_io_config *cfg, uint64_t seed, float std_dev);
/* patches[2 * tokens, patch_dim] (the two crops as rearrangeBCHWtoBTC leaves them, vision_model.zig:212-217; the reference
 * accepts exactly two, :204-208) -> out[tokens, out_dim].  The encoder runs on all 2 * tokens rows as one sequence, as the
 * reference does (attention_block takes q_len = B * M, :273-329).  MOON_EINVAL if nothing is attached. */
int moon_vision_encode_image(moon_vision_model *m, const moon_f16 *patches, moon_f16 *out);
int moon_vision_encode_image_dev(moon_vision_model *m, const void *patches, void *out);
/* VisionModel.vision_encoder (vision_model.zig:204-271) behind its rearrangeBCHWtoBTC: patches[2 * tokens, patch_dim] ->
 * out[2 * tokens, dim] = patch embedding + bias + positional embedding, the encoder blocks on all rows as one sequence, the
 * final LayerNorm (what encode_image then splits, concatenates and projects). */
int moon_vision_encoder(moon_vision_model *m, const moon_f16 *patches, moon_f16 *out);
/* VisionModel.encode_image from the resized image on (vision_model.zig:129-229): image[side, side, 3] as stbir left it
 * (side = sqrt(tokens) * sqrt(patch_dim / 3), 378 for the default configuration), normalised and cut into patches on the
 * device as moon_image_patches does, then moon_vision_encode_image's path. */
int moon_vision_encode_image_u8(moon_vision_model *m, const uint8_t *image, moon_f16 *out);

/* ------------------------------------------------------------------ moondream.bin (host side, no device call)
 * Weights.init (weights.zig:62-204): u32 magic 0x4D4F4F4E, u32 version 2, then per tensor {u32 name length, u32 number of
 * dims, u32 element count}, name, dims as u64, elements as little-endian binary16.  The file is memory-mapped; the
 * pointers handed out stay valid until moon_bin_close.  Errors come back as a status plus text in err[err_len]
 * (these calls take no context). */
typedef struct moon_bin moon_bin;
int moon_bin_open(const char *path, moon_bin **out, char *err, size_t err_len);
void moon_bin_close(moon_bin *bin);
size_t moon_bin_tensor_count(const moon_bin *bin);
/* tensor by position in the file / by name (MOON_EFORMAT if absent); any output pointer may be NULL.  A record's element
 * count must agree with its dimensions and fit the file (MOON_EFORMAT otherwise).  The data pointer addresses the bytes
 * where they lie in the file, after a name of any length: it may be odd, so copy from it (memcpy, moon_dev_upload, the
 * weight structs' consumers do) rather than dereference it as moon_f16. */
int moon_bin_tensor(const moon_bin *bin, size_t index, const char **name, size_t *ndim, size_t dims[4], const moon_f16 **data);
int moon_bin_find(const moon_bin *bin, const char *name, size_t *ndim, size_t dims[4], const moon_f16 **data);
/* Fill the weight structs of the sessions above from the file, checking every shape against the configuration exactly as
 * calculateShapes does (weights.zig:439-474): a mismatch is MOON_ESHAPE (error.ShapeMismatch), a missing tensor MOON_EFORMAT.
 * Then: moon_text_model_create(ctx, cfg, &w, &model) uploads straight from the mapping. */
int moon_bin_text_weights(const moon_bin *bin, const moon_text_config *cfg, moon_text_weights *w, char *err, size_t err_len);
int moon_bin_vision_weights(const moon_bin *bin, const moon_vision_config *cfg, moon_vision_weights *w, char *err, size_t err_len);
int moon_bin_vision_io_weights(const moon_bin *bin, const moon_vision_config *cfg, const moon_vision_io_config *io,
                               moon_vision_io_weights *w, char *err, size_t err_len);

/* ------------------------------------------------------------------------------------------------------------------
 * Environment variables.  None is needed: the defaults are what the tests and the bench run.  They are tuning and
 * diagnostic aids, read once per process unless noted (the first call that looks at them fixes the value for every context):
 *   MOON_DECODE_TRACE=1            text sessions record per-workgroup time stamps of the last layer launch of a greedy call
 *                                  and print a per-role timeline to stderr (allocated at session creation)
 *   MOON_LAYER_QKV_WGS=n           decode mode 0: workgroups that take qkv rows (default: the attention and output workgroups)
 *   MOON_LAYER_FC1_OUT_ROWS=n      decode mode 0: fc1 rows per output wavefront (default: about a third of an fc1-only wavefront's
 *                                  share, at least one; 0 is allowed)
 *   MOON_GEMM_KERNEL=regs|dma|dma256|w114|w212|w221  forces one of the MFMA product kernels where the shape allows it (default: by shape)
 *   MOON_GEMM_EPILOGUE=direct      the product kernels store their tile without the pass through LDS (default: through LDS)
 *   MOON_SAMPLE_SEPARATE=1         sampled loops with top_k <= 3: the LM-head launch leaves every token to sample_kernel instead of
 *                                  deciding it where it provably can (read at every call, so a test can compare the two in one process)
 *   MOON_GEMM_NO_PAIR=1            text prefill: a block's out_proj and fc2 run as launches of their own instead of one joint launch
 *                                  (read at every call); the two forms split K differently, so their f32 sums, and with them a few
 *                                  f16 roundings, differ
 *   MOON_GEMM_KN_TRANSPOSE=1       products with a [K, N] second operand always run over a transposed copy instead of reading the operand
 *                                  in place where the shape allows (read at every call; the same bits either way)
 *   MOON_GEMM_NO_ROPE=1            text prefill: the qkv projection and the rotation + cache update run as two launches instead of
 *                                  one (read at every call; the same bits either way)
 * Every other setting gives the same results, bit for bit; only the time changes. */

#ifdef __cplusplus
}
#endif
#endif /* MOONHIP_H */
