// extern "C" entry points for the per-op boundary: host-pointer drop-ins for the reference's src/core ops
// and their device-pointer twins.  Host-pointer ops stage operands into growable device buffers
// (or use a registered resident weight), launch, copy the result back and wait.
#include "moon_internal.hpp"
#include <cstring>

int launch_decode_attention_plain(moon_ctx *ctx, const half_t *q, const half_t *k, const half_t *v, half_t *out, size_t H,
                                  size_t kv_len, size_t D);

namespace {

enum { ST_A = 0, ST_B = 1, ST_C = 2, ST_AUX = 3, ST_MASK = 4, ST_AUX2 = 5 };

int stage_in(moon_ctx *ctx, int slot, const void *host, size_t bytes, void **dptr) {
    MOON_TRY(moon_grow(ctx, ctx->stage[slot], bytes ? bytes : 16));
    *dptr = ctx->stage[slot].ptr;
    if (bytes && bytes <= MOON_PIN_BYTES) { // small operands through page-locked memory: the copy is queued, not waited for
        if (!ctx->pin_up[slot] && hipHostMalloc(&ctx->pin_up[slot], MOON_PIN_BYTES, hipHostMallocDefault) != hipSuccess) {
            ctx->pin_up[slot] = nullptr;
            (void)hipGetLastError();
        }
        if (ctx->pin_up[slot]) {
            memcpy(ctx->pin_up[slot], host, bytes);
            host = ctx->pin_up[slot];
        }
    }
    if (bytes) MOON_HIP(ctx, hipMemcpyAsync(*dptr, host, bytes, hipMemcpyHostToDevice, ctx->stream));
    return MOON_OK;
}

int stage_out(moon_ctx *ctx, int slot, size_t bytes, void **dptr) {
    MOON_TRY(moon_grow(ctx, ctx->stage[slot], bytes ? bytes : 16));
    *dptr = ctx->stage[slot].ptr;
    return MOON_OK;
}

int fetch(moon_ctx *ctx, void *host, const void *dptr, size_t bytes) {
    void *dst = host;
    if (bytes && bytes <= MOON_PIN_BYTES) {
        if (!ctx->pin_down && hipHostMalloc(&ctx->pin_down, MOON_PIN_BYTES, hipHostMallocDefault) != hipSuccess) {
            ctx->pin_down = nullptr;
            (void)hipGetLastError();
        }
        if (ctx->pin_down) dst = ctx->pin_down;
    }
    if (bytes) MOON_HIP(ctx, hipMemcpyAsync(dst, dptr, bytes, hipMemcpyDeviceToHost, ctx->stream));
    MOON_HIP(ctx, hipStreamSynchronize(ctx->stream));
    if (dst != host) memcpy(host, dst, bytes);
    return MOON_OK;
}

// resident weight if this exact host buffer was registered, else a staged copy.  A registered weight that is used as
// B[K,N] (hgemm.matmul's layout, hgemm.zig:210-216) gets an [N,K] copy on its first such use, kept until it is
// unregistered, and *b_layout becomes MOON_B_NK: the product then runs without a transpose pass per call.
int weight_in(moon_ctx *ctx, int slot, const moon_f16 *host, size_t n_elems, const half_t **dptr, int *b_layout = nullptr, size_t K = 0,
              size_t N = 0) {
    auto it = ctx->resident.find(host);
    if (it != ctx->resident.end() && it->second.n_elems == n_elems) {
        moon_ctx::Resident &r = it->second;
        if (b_layout && *b_layout == MOON_B_KN && K * N == n_elems && K > 1 && N > 1) {
            if (!r.dptr_t || r.t_k != K || r.t_n != N) {
                if (r.dptr_t) {
                    MOON_HIP(ctx, hipStreamSynchronize(ctx->stream));
                    MOON_HIP(ctx, hipFree(r.dptr_t));
                    r.dptr_t = nullptr;
                }
                MOON_HIP(ctx, hipMalloc(&r.dptr_t, n_elems * sizeof(moon_f16)));
                MOON_TRY(launch_transpose(ctx, (const half_t *)r.dptr, (half_t *)r.dptr_t, K, N));
                r.t_k = K;
                r.t_n = N;
            }
            *dptr = (const half_t *)r.dptr_t;
            *b_layout = MOON_B_NK;
            return MOON_OK;
        }
        *dptr = (const half_t *)r.dptr;
        return MOON_OK;
    }
    void *d = nullptr;
    MOON_TRY(stage_in(ctx, slot, host, n_elems * sizeof(moon_f16), &d));
    *dptr = (const half_t *)d;
    return MOON_OK;
}

int linear_dev(moon_ctx *ctx, const half_t *a, size_t M, size_t K, const half_t *b, size_t N, int b_layout, const half_t *bias,
               int epilogue, half_t *c) {
    if (M == 1 && b_layout == MOON_B_NK) return launch_gemv_nt(ctx, a, b, bias, c, N, K, epilogue);
    return launch_gemm(ctx, a, b, bias, c, M, N, K, b_layout, epilogue);
}

int linear_host(moon_ctx *ctx, const moon_f16 *a, size_t M, size_t K, const moon_f16 *b, size_t N, int b_layout,
                const moon_f16 *bias, int epilogue, moon_f16 *c) {
    if (!ctx) return MOON_EINVAL;
    std::lock_guard<std::mutex> lock(ctx->mu);
    if ((!a && M * K) || (!b && N * K) || (!c && M * N)) return moon_fail(ctx, MOON_EINVAL, "linear: null operand");
    if (epilogue != MOON_EPI_NONE && !bias) return moon_fail(ctx, MOON_EINVAL, "linear: epilogue needs a bias");
    if (M * N == 0) return MOON_OK;
    MOON_HIP(ctx, hipSetDevice(ctx->device));
    void *da = nullptr, *dc = nullptr, *dbias = nullptr;
    const half_t *db = nullptr;
    MOON_TRY(stage_in(ctx, ST_A, a, M * K * sizeof(moon_f16), &da));
    MOON_TRY(weight_in(ctx, ST_B, b, N * K, &db, &b_layout, K, N));
    if (bias) MOON_TRY(stage_in(ctx, ST_AUX, bias, N * sizeof(moon_f16), &dbias));
    MOON_TRY(stage_out(ctx, ST_C, M * N * sizeof(moon_f16), &dc));
    MOON_TRY(linear_dev(ctx, (const half_t *)da, M, K, db, N, b_layout, (const half_t *)dbias, epilogue, (half_t *)dc));
    return fetch(ctx, c, dc, M * N * sizeof(moon_f16));
}

// true if mask[q_len, stride] equals createAttentionMask(kv_len - q_len, q_len) (attention.zig:256-281)
bool is_causal_mask(const uint8_t *mask, size_t stride, size_t q_len, size_t kv_len) {
    if (kv_len < q_len) return false;
    const size_t pos = kv_len - q_len;
    for (size_t i = 0; i < q_len; i++)
        for (size_t j = 0; j < kv_len; j++)
            if ((mask[i * stride + j] != 0) != (j <= pos + i)) return false;
    return true;
}

bool is_all_true(const uint8_t *mask, size_t n) {
    for (size_t i = 0; i < n; i++)
        if (!mask[i]) return false;
    return true;
}

int sdpa_host(moon_ctx *ctx, const moon_f16 *q, const moon_f16 *k, const moon_f16 *v, const uint8_t *mask, size_t mask_stride,
              moon_f16 *out, size_t H, size_t Lq, size_t Lkv, size_t D, bool single) {
    if (!ctx) return MOON_EINVAL;
    std::lock_guard<std::mutex> lock(ctx->mu);
    if (!q || !k || !v || !out) return moon_fail(ctx, MOON_EINVAL, "sdpa: null operand");
    if (single && Lkv > 2048) return moon_fail(ctx, MOON_ESEQ_TOO_LONG, "singleMaskedSDPA: kv_len %zu > 2048 (SequenceTooLong)", Lkv);
    if (mask && mask_stride < Lkv) return moon_fail(ctx, MOON_ESHAPE, "sdpa: mask row stride %zu < kv_len %zu", mask_stride, Lkv);
    if (H * Lq * D == 0) return MOON_OK;
    if (Lkv == 0) return moon_fail(ctx, MOON_EINVAL_DIM, "sdpa: kv_len is 0");
    MOON_HIP(ctx, hipSetDevice(ctx->device));
    long causal_pos = -1;
    const uint8_t *mask_to_send = mask;
    if (mask) {
        if (is_causal_mask(mask, mask_stride, Lq, Lkv)) {
            causal_pos = (long)(Lkv - Lq);
            mask_to_send = nullptr;
        } else if (Lq == 1 && is_all_true(mask, Lkv)) {
            mask_to_send = nullptr;
        }
    }
    void *dq, *dk, *dv, *dout, *dmask = nullptr;
    MOON_TRY(stage_in(ctx, ST_A, q, H * Lq * D * sizeof(moon_f16), &dq));
    MOON_TRY(stage_in(ctx, ST_B, k, H * Lkv * D * sizeof(moon_f16), &dk));
    MOON_TRY(stage_in(ctx, ST_AUX, v, H * Lkv * D * sizeof(moon_f16), &dv));
    MOON_TRY(stage_out(ctx, ST_C, H * Lq * D * sizeof(moon_f16), &dout));
    size_t dstride = 0;
    if (mask_to_send) {
        if (mask_stride == Lkv) {
            MOON_TRY(stage_in(ctx, ST_MASK, mask_to_send, Lq * Lkv, &dmask));
        } else { // compact the strided rows
            MOON_TRY(moon_grow(ctx, ctx->stage[ST_MASK], Lq * Lkv));
            dmask = ctx->stage[ST_MASK].ptr;
            MOON_HIP(ctx, hipMemcpy2DAsync(dmask, Lkv, mask_to_send, mask_stride, Lkv, Lq, hipMemcpyHostToDevice, ctx->stream));
        }
        dstride = Lkv;
    }
    if (Lq == 1 && !mask_to_send && D == 64 && Lkv <= 2048) {
        MOON_TRY(launch_decode_attention_plain(ctx, (const half_t *)dq, (const half_t *)dk, (const half_t *)dv, (half_t *)dout, H, Lkv, D));
    } else {
        MOON_TRY(launch_sdpa(ctx, (const half_t *)dq, (const half_t *)dk, (const half_t *)dv, (half_t *)dout, H, Lq, Lkv, D, Lkv * D,
                             causal_pos, (const uint8_t *)dmask, dstride, false));
    }
    return fetch(ctx, out, dout, H * Lq * D * sizeof(moon_f16));
}

} // namespace

// ------------------------------------------------------------------ matrix products
extern "C" int moon_hgemm(moon_ctx *ctx, const moon_f16 *a, size_t a_rows, size_t a_cols, const moon_f16 *b, size_t b_rows,
                          size_t b_cols, moon_f16 *c) {
    if (!ctx) return MOON_EINVAL;
    if (b_rows != a_cols)
        return moon_fail(ctx, MOON_ESHAPE, "hgemm: A [%zu,%zu] x B [%zu,%zu] (IncompatibleTensorShapes)", a_rows, a_cols, b_rows, b_cols);
    return linear_host(ctx, a, a_rows, a_cols, b, b_cols, MOON_B_KN, nullptr, MOON_EPI_NONE, c);
}

extern "C" int moon_hgemm_trans(moon_ctx *ctx, const moon_f16 *a, size_t a_rows, size_t a_cols, const moon_f16 *b_t,
                                size_t bt_rows, size_t bt_cols, moon_f16 *c) {
    if (!ctx) return MOON_EINVAL;
    if (bt_cols != a_cols)
        return moon_fail(ctx, MOON_ESHAPE, "hgemm_trans: A [%zu,%zu] x B_t [%zu,%zu] (IncompatibleTensorShapes)", a_rows, a_cols,
                         bt_rows, bt_cols);
    return linear_host(ctx, a, a_rows, a_cols, b_t, bt_rows, MOON_B_NK, nullptr, MOON_EPI_NONE, c);
}

extern "C" int moon_linear(moon_ctx *ctx, const moon_f16 *a, size_t M, size_t K, const moon_f16 *b, size_t N, int b_layout,
                           const moon_f16 *bias, int epilogue, moon_f16 *c) {
    if (!ctx) return MOON_EINVAL;
    if (b_layout != MOON_B_KN && b_layout != MOON_B_NK) return moon_fail(ctx, MOON_EINVAL, "linear: unknown B layout %d", b_layout);
    if (epilogue < MOON_EPI_NONE || epilogue > MOON_EPI_BIAS_GELU) return moon_fail(ctx, MOON_EINVAL, "linear: unknown epilogue %d", epilogue);
    return linear_host(ctx, a, M, K, b, N, b_layout, bias, epilogue, c);
}

// ------------------------------------------------------------------ attention
extern "C" int moon_sdpa_maskless(moon_ctx *ctx, const moon_f16 *q, const moon_f16 *k, const moon_f16 *v, moon_f16 *out,
                                  size_t n_heads, size_t q_len, size_t kv_len, size_t head_dim) {
    return sdpa_host(ctx, q, k, v, nullptr, 0, out, n_heads, q_len, kv_len, head_dim, false);
}

extern "C" int moon_sdpa_masked(moon_ctx *ctx, const moon_f16 *q, const moon_f16 *k, const moon_f16 *v, const uint8_t *mask,
                                size_t mask_stride, moon_f16 *out, size_t n_heads, size_t q_len, size_t kv_len, size_t head_dim) {
    if (ctx && !mask) return moon_fail(ctx, MOON_EINVAL, "multiMaskedSDPA: mask is null");
    return sdpa_host(ctx, q, k, v, mask, mask_stride, out, n_heads, q_len, kv_len, head_dim, false);
}

extern "C" int moon_sdpa_single(moon_ctx *ctx, const moon_f16 *q, const moon_f16 *k, const moon_f16 *v, const uint8_t *mask,
                                moon_f16 *out, size_t n_heads, size_t kv_len, size_t head_dim) {
    if (ctx && !mask) return moon_fail(ctx, MOON_EINVAL, "singleMaskedSDPA: mask is null");
    return sdpa_host(ctx, q, k, v, mask, kv_len, out, n_heads, 1, kv_len, head_dim, true);
}

extern "C" int moon_rope_apply(moon_ctx *ctx, const moon_f16 *x, moon_f16 *out, size_t n_heads, size_t seq_len, size_t head_dim,
                               const float *freqs_cis, size_t table_rows, size_t freq_pairs, const size_t *position_ids,
                               size_t rot_dim) {
    if (!ctx) return MOON_EINVAL;
    std::lock_guard<std::mutex> lock(ctx->mu);
    if (!x || !out || !freqs_cis || !position_ids) return moon_fail(ctx, MOON_EINVAL, "applyRotEmb: null operand");
    if (rot_dim != freq_pairs * 2) return moon_fail(ctx, MOON_EROT_DIM, "applyRotEmb: rot_dim %zu != 2*%zu (InvalidRotationDimension)", rot_dim, freq_pairs);
    if (rot_dim > head_dim) return moon_fail(ctx, MOON_EROT_DIM, "applyRotEmb: rot_dim %zu > head_dim %zu", rot_dim, head_dim);
    for (size_t s = 0; s < seq_len; s++)
        if (position_ids[s] >= table_rows) return moon_fail(ctx, MOON_ESEQ_TOO_LONG, "applyRotEmb: position %zu outside the table (%zu rows)", position_ids[s], table_rows);
    const size_t n = n_heads * seq_len * head_dim;
    if (!n) return MOON_OK;
    MOON_HIP(ctx, hipSetDevice(ctx->device));
    void *dx, *dout, *dtab, *dpos;
    static_assert(sizeof(size_t) == sizeof(uint64_t), "usize is 64-bit");
    MOON_TRY(stage_in(ctx, ST_A, x, n * sizeof(moon_f16), &dx));
    MOON_TRY(stage_in(ctx, ST_B, freqs_cis, table_rows * freq_pairs * 2 * sizeof(float), &dtab));
    MOON_TRY(stage_in(ctx, ST_AUX, position_ids, seq_len * sizeof(uint64_t), &dpos));
    MOON_TRY(stage_out(ctx, ST_C, n * sizeof(moon_f16), &dout));
    MOON_TRY(launch_rope_apply(ctx, (const half_t *)dx, (half_t *)dout, n_heads, seq_len, head_dim, (const float *)dtab,
                               (const uint64_t *)dpos, 0, rot_dim));
    return fetch(ctx, out, dout, n * sizeof(moon_f16));
}

// ------------------------------------------------------------------ normalisation / element-wise
extern "C" int moon_layernorm(moon_ctx *ctx, const moon_f16 *x, const moon_f16 *gamma, const moon_f16 *beta, moon_f16 *y,
                              size_t rows, size_t dim, float eps) {
    if (!ctx) return MOON_EINVAL;
    std::lock_guard<std::mutex> lock(ctx->mu);
    if (!(eps > 0.0f)) return moon_fail(ctx, MOON_EEPS, "layerNorm: eps must be > 0 (InvalidEpsilon)");
    if (!x || !gamma || !beta || !y) return moon_fail(ctx, MOON_EINVAL, "layerNorm: null operand");
    if (rows * dim == 0) return MOON_OK;
    MOON_HIP(ctx, hipSetDevice(ctx->device));
    void *dx, *dg, *db, *dy;
    MOON_TRY(stage_in(ctx, ST_A, x, rows * dim * sizeof(moon_f16), &dx));
    MOON_TRY(stage_in(ctx, ST_B, gamma, dim * sizeof(moon_f16), &dg));
    MOON_TRY(stage_in(ctx, ST_AUX, beta, dim * sizeof(moon_f16), &db));
    MOON_TRY(stage_out(ctx, ST_C, rows * dim * sizeof(moon_f16), &dy));
    MOON_TRY(launch_layernorm(ctx, (const half_t *)dx, (const half_t *)dg, (const half_t *)db, (half_t *)dy, rows, dim, eps));
    return fetch(ctx, y, dy, rows * dim * sizeof(moon_f16));
}

extern "C" int moon_gelu(moon_ctx *ctx, moon_f16 *x, size_t n) {
    if (!ctx) return MOON_EINVAL;
    std::lock_guard<std::mutex> lock(ctx->mu);
    if (!x && n) return moon_fail(ctx, MOON_EINVAL, "gelu: null operand");
    if (!n) return MOON_OK;
    MOON_HIP(ctx, hipSetDevice(ctx->device));
    void *dx;
    MOON_TRY(stage_in(ctx, ST_A, x, n * sizeof(moon_f16), &dx));
    MOON_TRY(launch_gelu(ctx, (half_t *)dx, n));
    return fetch(ctx, x, dx, n * sizeof(moon_f16));
}

extern "C" int moon_bias_add(moon_ctx *ctx, moon_f16 *a, const moon_f16 *b, size_t rows, size_t cols) {
    if (!ctx) return MOON_EINVAL;
    std::lock_guard<std::mutex> lock(ctx->mu);
    if ((!a || !b) && rows * cols) return moon_fail(ctx, MOON_EINVAL, "broadcast_add: null operand");
    if (rows * cols == 0) return MOON_OK;
    MOON_HIP(ctx, hipSetDevice(ctx->device));
    void *da, *db;
    MOON_TRY(stage_in(ctx, ST_A, a, rows * cols * sizeof(moon_f16), &da));
    MOON_TRY(stage_in(ctx, ST_B, b, cols * sizeof(moon_f16), &db));
    MOON_TRY(launch_bias_add(ctx, (half_t *)da, (const half_t *)db, rows, cols));
    return fetch(ctx, a, da, rows * cols * sizeof(moon_f16));
}

extern "C" int moon_add(moon_ctx *ctx, moon_f16 *a, const moon_f16 *b, size_t n) {
    if (!ctx) return MOON_EINVAL;
    std::lock_guard<std::mutex> lock(ctx->mu);
    if ((!a || !b) && n) return moon_fail(ctx, MOON_EINVAL, "add: null operand");
    if (!n) return MOON_OK;
    MOON_HIP(ctx, hipSetDevice(ctx->device));
    void *da, *db;
    MOON_TRY(stage_in(ctx, ST_A, a, n * sizeof(moon_f16), &da));
    MOON_TRY(stage_in(ctx, ST_B, b, n * sizeof(moon_f16), &db));
    MOON_TRY(launch_add(ctx, (half_t *)da, (const half_t *)db, n));
    return fetch(ctx, a, da, n * sizeof(moon_f16));
}

extern "C" int moon_argmax(moon_ctx *ctx, const moon_f16 *logits, size_t n, size_t *index) {
    if (!ctx) return MOON_EINVAL;
    std::lock_guard<std::mutex> lock(ctx->mu);
    if (!logits || !index) return moon_fail(ctx, MOON_EINVAL, "argmax: null operand");
    if (!n) return moon_fail(ctx, MOON_EINVAL, "argmax: empty tensor (EmptyTensor)");
    MOON_HIP(ctx, hipSetDevice(ctx->device));
    void *dl, *di;
    MOON_TRY(stage_in(ctx, ST_A, logits, n * sizeof(moon_f16), &dl));
    MOON_TRY(stage_out(ctx, ST_C, sizeof(uint32_t), &di));
    MOON_TRY(launch_argmax(ctx, (const half_t *)dl, n, (uint32_t *)di));
    uint32_t idx = 0;
    MOON_TRY(fetch(ctx, &idx, di, sizeof(idx)));
    *index = idx;
    return MOON_OK;
}

extern "C" int moon_image_patches(moon_ctx *ctx, const uint8_t *image, size_t height, size_t width, size_t channels, size_t patch_size,
                                  moon_f16 *patches) {
    if (!ctx) return MOON_EINVAL;
    std::lock_guard<std::mutex> lock(ctx->mu);
    if (!image || !patches) return moon_fail(ctx, MOON_EINVAL, "image_patches: null operand");
    MOON_HIP(ctx, hipSetDevice(ctx->device));
    if (!patch_size || height % patch_size || width % patch_size || !height || !width || !channels)
        return moon_fail(ctx, MOON_EINVAL_DIM, "image_patches: %zu x %zu x %zu is not a whole number of %zu x %zu patches (InvalidPatchSize)", height,
                         width, channels, patch_size, patch_size);
    const size_t dim = channels * patch_size * patch_size, rows = 2 * (height / patch_size) * (width / patch_size);
    void *di, *dp;
    MOON_TRY(stage_in(ctx, ST_A, image, height * width * channels, &di));
    MOON_TRY(stage_out(ctx, ST_C, rows * dim * sizeof(moon_f16), &dp));
    MOON_TRY(launch_image_patches(ctx, (const uint8_t *)di, (half_t *)dp, height, width, channels, patch_size, 2, dim));
    return fetch(ctx, patches, dp, rows * dim * sizeof(moon_f16));
}

extern "C" void moon_sampling_config_default(moon_sampling_config *cfg) {
    if (!cfg) return;
    cfg->method = MOON_SAMPLE_GREEDY;
    cfg->temperature = 0.5f;
    cfg->top_k = 3;
    cfg->min_p = 0.05f;
}

// logits on the device; the index comes back through the C staging slot
static int sample_dev(moon_ctx *ctx, const half_t *dl, size_t n, const moon_sampling_config *cfg, float u, size_t *index) {
    void *di;
    MOON_TRY(stage_out(ctx, ST_C, sizeof(uint32_t), &di));
    if (cfg->method == MOON_SAMPLE_GREEDY)
        MOON_TRY(launch_argmax(ctx, dl, n, (uint32_t *)di));
    else
        MOON_TRY(launch_sample(ctx, dl, n, cfg, u, nullptr, nullptr, nullptr, (uint32_t *)di));
    uint32_t idx = 0;
    MOON_TRY(fetch(ctx, &idx, di, sizeof(idx)));
    *index = idx;
    return MOON_OK;
}

extern "C" int moon_sample(moon_ctx *ctx, const moon_f16 *logits, size_t n, const moon_sampling_config *cfg, float u, size_t *index) {
    if (!ctx) return MOON_EINVAL;
    std::lock_guard<std::mutex> lock(ctx->mu);
    if (!logits || !index || !cfg) return moon_fail(ctx, MOON_EINVAL, "sample: null operand");
    if (!n) return moon_fail(ctx, MOON_EINVAL, "sample: empty tensor (EmptyTensor)");
    MOON_HIP(ctx, hipSetDevice(ctx->device));
    void *dl;
    MOON_TRY(stage_in(ctx, ST_A, logits, n * sizeof(moon_f16), &dl));
    return sample_dev(ctx, (const half_t *)dl, n, cfg, u, index);
}

extern "C" int moon_dev_sample(moon_ctx *ctx, const void *logits, size_t n, const moon_sampling_config *cfg, float u, size_t *index) {
    if (!ctx) return MOON_EINVAL;
    std::lock_guard<std::mutex> lock(ctx->mu);
    if (!logits || !index || !cfg) return moon_fail(ctx, MOON_EINVAL, "dev_sample: null operand");
    if (!n) return moon_fail(ctx, MOON_EINVAL, "dev_sample: empty tensor (EmptyTensor)");
    MOON_HIP(ctx, hipSetDevice(ctx->device));
    return sample_dev(ctx, (const half_t *)logits, n, cfg, u, index);
}

extern "C" int moon_sample_f32(moon_ctx *ctx, const float *logits, size_t n, const moon_sampling_config *cfg, float u, size_t *index) {
    if (!ctx) return MOON_EINVAL;
    std::lock_guard<std::mutex> lock(ctx->mu);
    if (!logits || !index || !cfg) return moon_fail(ctx, MOON_EINVAL, "sample_f32: null operand");
    if (!n) return moon_fail(ctx, MOON_EINVAL, "sample_f32: empty tensor (EmptyTensor)");
    MOON_HIP(ctx, hipSetDevice(ctx->device));
    void *dl, *di;
    MOON_TRY(stage_in(ctx, ST_A, logits, n * sizeof(float), &dl));
    MOON_TRY(stage_out(ctx, ST_C, sizeof(uint32_t), &di));
    if (cfg->method == MOON_SAMPLE_GREEDY)
        MOON_TRY(launch_argmax_f32(ctx, (const float *)dl, n, (uint32_t *)di));
    else
        MOON_TRY(launch_sample(ctx, nullptr, n, cfg, u, nullptr, nullptr, nullptr, (uint32_t *)di, 0, (const float *)dl));
    uint32_t idx = 0;
    MOON_TRY(fetch(ctx, &idx, di, sizeof(idx)));
    *index = idx;
    return MOON_OK;
}

extern "C" int moon_argmax_f32(moon_ctx *ctx, const float *logits, size_t n, size_t *index) {
    if (!ctx) return MOON_EINVAL;
    std::lock_guard<std::mutex> lock(ctx->mu);
    if (!logits || !index) return moon_fail(ctx, MOON_EINVAL, "argmax_f32: null operand");
    if (!n) return moon_fail(ctx, MOON_EINVAL, "argmax_f32: empty tensor (EmptyTensor)");
    MOON_HIP(ctx, hipSetDevice(ctx->device));
    void *dl, *di;
    MOON_TRY(stage_in(ctx, ST_A, logits, n * sizeof(float), &dl));
    MOON_TRY(stage_out(ctx, ST_C, sizeof(uint32_t), &di));
    MOON_TRY(launch_argmax_f32(ctx, (const float *)dl, n, (uint32_t *)di));
    uint32_t idx = 0;
    MOON_TRY(fetch(ctx, &idx, di, sizeof(idx)));
    *index = idx;
    return MOON_OK;
}

// ------------------------------------------------------------------ device-pointer ops
extern "C" int moon_dev_linear(moon_ctx *ctx, const void *a, size_t M, size_t K, const void *b, size_t N, int b_layout,
                               const void *bias, int epilogue, void *c) {
    if (!ctx) return MOON_EINVAL;
    std::lock_guard<std::mutex> lock(ctx->mu);
    if (!a || !b || !c) return moon_fail(ctx, MOON_EINVAL, "dev_linear: null operand");
    if (b_layout != MOON_B_KN && b_layout != MOON_B_NK) return moon_fail(ctx, MOON_EINVAL, "dev_linear: unknown B layout %d", b_layout);
    return linear_dev(ctx, (const half_t *)a, M, K, (const half_t *)b, N, b_layout, (const half_t *)bias, epilogue, (half_t *)c);
}

extern "C" int moon_dev_sdpa(moon_ctx *ctx, const void *q, const void *k, const void *v, void *out, size_t n_heads, size_t q_len,
                             size_t kv_len, size_t head_dim, long causal_pos, const void *mask, size_t mask_stride) {
    if (!ctx) return MOON_EINVAL;
    std::lock_guard<std::mutex> lock(ctx->mu);
    if (!q || !k || !v || !out) return moon_fail(ctx, MOON_EINVAL, "dev_sdpa: null operand");
    return launch_sdpa(ctx, (const half_t *)q, (const half_t *)k, (const half_t *)v, (half_t *)out, n_heads, q_len, kv_len, head_dim,
                       kv_len * head_dim, causal_pos, (const uint8_t *)mask, mask_stride, false);
}

extern "C" int moon_dev_decode_attention(moon_ctx *ctx, const void *qkv, void *cache_k, void *cache_v, const void *freqs_cis,
                                         void *out, size_t n_heads, size_t head_dim, size_t rot_dim, size_t max_seq, size_t pos) {
    if (!ctx) return MOON_EINVAL;
    std::lock_guard<std::mutex> lock(ctx->mu);
    if (!qkv || !cache_k || !cache_v || !freqs_cis || !out) return moon_fail(ctx, MOON_EINVAL, "dev_decode_attention: null operand");
    return launch_decode_attention(ctx, (const half_t *)qkv, (half_t *)cache_k, (half_t *)cache_v, (const float *)freqs_cis,
                                   (half_t *)out, n_heads, head_dim, rot_dim, max_seq, pos, nullptr);
}

extern "C" int moon_dev_rope_table(moon_ctx *ctx, void *table, size_t rot_dim, size_t end, float theta) {
    if (!ctx) return MOON_EINVAL;
    std::lock_guard<std::mutex> lock(ctx->mu);
    if (!table) return moon_fail(ctx, MOON_EINVAL, "dev_rope_table: null table");
    if (!rot_dim || rot_dim % 2) return moon_fail(ctx, MOON_EROT_DIM, "dev_rope_table: rot_dim %zu must be even and positive", rot_dim);
    if (rot_dim / 2 * end > 0x7fffffffull) return moon_fail(ctx, MOON_EINVAL_DIM, "dev_rope_table: table too large");
    return launch_rope_table(ctx, (float *)table, rot_dim, end, theta);
}

extern "C" int moon_dev_layernorm(moon_ctx *ctx, const void *x, const void *gamma, const void *beta, void *y, size_t rows,
                                  size_t dim, float eps) {
    if (!ctx) return MOON_EINVAL;
    std::lock_guard<std::mutex> lock(ctx->mu);
    if (!x || !gamma || !beta || !y) return moon_fail(ctx, MOON_EINVAL, "dev_layernorm: null operand");
    return launch_layernorm(ctx, (const half_t *)x, (const half_t *)gamma, (const half_t *)beta, (half_t *)y, rows, dim, eps);
}
