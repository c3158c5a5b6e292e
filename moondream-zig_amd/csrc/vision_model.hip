// Device-resident vision encoder session: the block loop of VisionModel.vision_encoder with attention_block and
// mlp (vision_model.zig:231-271, 273-343, 345-364).  The moondream.bin vision layout stores matrices [L, in, out]
// (weights.zig:459-474); they are transposed once at load time to the k-contiguous [out, in] form the GEMM kernel
// stages without a transposition.  Activations stay on the device for all blocks.
// The MLP's hidden width is held padded to a multiple of 64 (4304 -> 4352: fc1 gets zero rows and zero biases, so its
// output carries gelu(0) = 0 there; fc2 gets zero columns): every row of the fc1 activations and of the fc2 weights then
// starts on a 128-byte line, and the 64-wide k-tiles that the fc2 product copies into LDS are whole lines instead of
// pieces of two.  The added terms are exact zeros, so no result changes.
#include "moon_internal.hpp"

#include <vector>

struct moon_vision_model {
    moon_ctx *ctx = nullptr;
    moon_vision_config cfg{};
    size_t fp = 0; // hidden_dim rounded up to a multiple of 64
    // matrices held transposed: [L][out][in] (fc1: [L][fp][dim], fc2: [L][dim][fp]; fc1_b: [L][fp])
    half_t *qkv_w = nullptr, *qkv_b = nullptr, *out_w = nullptr, *out_b = nullptr, *fc1_w = nullptr, *fc1_b = nullptr,
           *fc2_w = nullptr, *fc2_b = nullptr, *n1_w = nullptr, *n1_b = nullptr, *n2_w = nullptr, *n2_b = nullptr,
           *no_w = nullptr, *no_b = nullptr;
    // activations for up to cap_tokens rows
    size_t cap_tokens = 0;
    half_t *x = nullptr, *ln = nullptr, *qkv = nullptr, *q = nullptr, *k = nullptr, *v = nullptr, *attn = nullptr, *proj = nullptr,
           *fc1 = nullptr, *mlp = nullptr;
    std::vector<void *> allocs;     // weights
    std::vector<void *> act_allocs; // activations
    // front and back ends of encode_image, once attached: matrices transposed to [out][in]; the patch-embedding matrix and
    // the patches are zero padded in k to a multiple of 64 (588 -> 640) so that the product takes the matrix-core kernel
    // and its rows start on 128-byte lines
    bool io = false;
    moon_vision_io_config io_cfg{};
    size_t kp = 0; // padded patch_dim
    half_t *pe_w = nullptr, *pe_b = nullptr, *pos = nullptr, *p1_w = nullptr, *p1_b = nullptr, *p2_w = nullptr, *p2_b = nullptr;
    half_t *patches_pad = nullptr, *emb = nullptr, *enc = nullptr, *cat = nullptr, *hid = nullptr, *img_out = nullptr;
};

namespace {

int dalloc(moon_vision_model *m, std::vector<void *> &list, size_t n, half_t **p) {
    MOON_HIP(m->ctx, hipMalloc((void **)p, (n ? n : 8) * sizeof(half_t)));
    list.push_back(*p);
    return MOON_OK;
}

int check_cfg(moon_ctx *ctx, const moon_vision_config *c) {
    if (!c) return moon_fail(ctx, MOON_EINVAL, "vision model: null config");
    if (!c->dim || !c->hidden_dim || !c->n_layers || !c->n_heads || !c->head_dim) return moon_fail(ctx, MOON_EINVAL_DIM, "vision model: zero dimension");
    if (c->n_heads * c->head_dim != c->dim) return moon_fail(ctx, MOON_EINVAL_DIM, "vision model: n_heads*head_dim != dim");
    if (c->head_dim > 256) return moon_fail(ctx, MOON_EINVAL_DIM, "vision model: head_dim > 256");
    if (!(c->ln_eps > 0.0f)) return moon_fail(ctx, MOON_EEPS, "vision model: ln_eps must be > 0");
    return MOON_OK;
}

int alloc_weights(moon_vision_model *m) {
    const size_t L = m->cfg.n_layers, d = m->cfg.dim, f = m->fp;
    MOON_TRY(dalloc(m, m->allocs, L * 3 * d * d, &m->qkv_w));
    MOON_TRY(dalloc(m, m->allocs, L * 3 * d, &m->qkv_b));
    MOON_TRY(dalloc(m, m->allocs, L * d * d, &m->out_w));
    MOON_TRY(dalloc(m, m->allocs, L * d, &m->out_b));
    MOON_TRY(dalloc(m, m->allocs, L * d * f, &m->fc1_w));
    MOON_TRY(dalloc(m, m->allocs, L * f, &m->fc1_b));
    MOON_TRY(dalloc(m, m->allocs, L * f * d, &m->fc2_w));
    MOON_TRY(dalloc(m, m->allocs, L * d, &m->fc2_b));
    MOON_TRY(dalloc(m, m->allocs, L * d, &m->n1_w));
    MOON_TRY(dalloc(m, m->allocs, L * d, &m->n1_b));
    MOON_TRY(dalloc(m, m->allocs, L * d, &m->n2_w));
    MOON_TRY(dalloc(m, m->allocs, L * d, &m->n2_b));
    MOON_TRY(dalloc(m, m->allocs, d, &m->no_w));
    MOON_TRY(dalloc(m, m->allocs, d, &m->no_b));
    return MOON_OK;
}

int ensure_activations(moon_vision_model *m, size_t tokens) {
    if (tokens <= m->cap_tokens) return MOON_OK;
    (void)hipStreamSynchronize(m->ctx->stream);
    for (void *p : m->act_allocs) (void)hipFree(p);
    m->act_allocs.clear();
    m->cap_tokens = 0;
    const size_t d = m->cfg.dim, f = m->fp;
    MOON_TRY(dalloc(m, m->act_allocs, tokens * d, &m->x));
    MOON_TRY(dalloc(m, m->act_allocs, tokens * d, &m->ln));
    MOON_TRY(dalloc(m, m->act_allocs, tokens * 3 * d, &m->qkv));
    MOON_TRY(dalloc(m, m->act_allocs, tokens * d, &m->q));
    MOON_TRY(dalloc(m, m->act_allocs, tokens * d, &m->k));
    MOON_TRY(dalloc(m, m->act_allocs, tokens * d, &m->v));
    MOON_TRY(dalloc(m, m->act_allocs, tokens * d, &m->attn));
    MOON_TRY(dalloc(m, m->act_allocs, tokens * d, &m->proj));
    MOON_TRY(dalloc(m, m->act_allocs, tokens * f, &m->fc1));
    MOON_TRY(dalloc(m, m->act_allocs, tokens * d, &m->mlp));
    m->cap_tokens = tokens;
    return MOON_OK;
}

void free_all(moon_vision_model *m) {
    (void)hipStreamSynchronize(m->ctx->stream);
    for (void *p : m->allocs) (void)hipFree(p);
    for (void *p : m->act_allocs) (void)hipFree(p);
    m->allocs.clear();
    m->act_allocs.clear();
}

// per-layer transposition [L][in][out] (tmp, device) -> [L][out][in]
int transpose_layers(moon_vision_model *m, const half_t *tmp, half_t *dst, size_t L, size_t in, size_t out) {
    for (size_t l = 0; l < L; l++) MOON_TRY(launch_transpose(m->ctx, tmp + l * in * out, dst + l * in * out, in, out));
    return MOON_OK;
}

int encode_dev(moon_vision_model *m, const half_t *x_in, size_t T, half_t *out) {
    moon_ctx *ctx = m->ctx;
    const size_t d = m->cfg.dim, f = m->fp, H = m->cfg.n_heads, D = m->cfg.head_dim; // (f: the padded hidden width)
    MOON_TRY(ensure_activations(m, T));
    MOON_HIP(ctx, hipMemcpyAsync(m->x, x_in, T * d * sizeof(half_t), hipMemcpyDeviceToDevice, ctx->stream));
    // Every LayerNorm but the first follows a product that has just finished the rows it normalises (out_proj + residual ->
    // ln2; fc2 + residual -> the next block's ln1, or the final LayerNorm): it is handed to that product, which folds it into
    // its split-K reduction where it has one (launch_gemm), instead of a launch that re-reads x.
    if (m->cfg.n_layers == 0) return launch_layernorm(ctx, m->x, m->no_w, m->no_b, out, T, d, m->cfg.ln_eps);
    MOON_TRY(launch_layernorm(ctx, m->x, m->n1_w, m->n1_b, m->ln, T, d, m->cfg.ln_eps));
    for (size_t l = 0; l < m->cfg.n_layers; l++) {
        // x += attention_block(layerNorm(x))   (vision_model.zig:239-248)
        MOON_TRY(launch_gemm(ctx, m->ln, m->qkv_w + l * 3 * d * d, m->qkv_b + l * 3 * d, m->qkv, T, 3 * d, d, MOON_B_NK, MOON_EPI_BIAS));
        bool packed = false; // the matrix-core kernel reads q, k, v in place; other shapes are split into [H, T, D] tensors first
        MOON_TRY(launch_sdpa_packed_qkv(ctx, m->qkv, m->attn, H, T, D, &packed));
        if (!packed) {
            MOON_TRY(launch_split_heads(ctx, m->qkv, 3 * d, 0, m->q, T, H, D));
            MOON_TRY(launch_split_heads(ctx, m->qkv, 3 * d, d, m->k, T, H, D));
            MOON_TRY(launch_split_heads(ctx, m->qkv, 3 * d, 2 * d, m->v, T, H, D));
            MOON_TRY(launch_sdpa(ctx, m->q, m->k, m->v, m->attn, H, T, T, D, T * D, -1, nullptr, 0, true));
        }
        // x += mlp(layerNorm(x))               (vision_model.zig:253-262)
        const GemmLayerNorm ln2{m->n2_w + l * d, m->n2_b + l * d, m->ln, m->cfg.ln_eps};
        MOON_TRY(launch_gemm(ctx, m->attn, m->out_w + l * d * d, m->out_b + l * d, m->x, T, d, d, MOON_B_NK, 3 /* bias, then += into x */, m->x, &ln2));
        MOON_TRY(launch_gemm(ctx, m->ln, m->fc1_w + l * d * f, m->fc1_b + l * f, m->fc1, T, f, d, MOON_B_NK, MOON_EPI_BIAS_GELU));
        const bool last = l + 1 == m->cfg.n_layers; // the final LayerNorm (vision_model.zig:266) or the next block's first
        const GemmLayerNorm next{last ? m->no_w : m->n1_w + (l + 1) * d, last ? m->no_b : m->n1_b + (l + 1) * d, last ? out : m->ln, m->cfg.ln_eps};
        MOON_TRY(launch_gemm(ctx, m->fc1, m->fc2_w + l * f * d, m->fc2_b + l * d, m->x, T, d, f, MOON_B_NK, 3 /* bias, then += into x */, m->x, &next));
    }
    return MOON_OK;
}

// encode_image (vision_model.zig:186-229): patches[2T, patch_dim] on the device -> out[T, out_dim] on the device
static int encode_image_padded(moon_vision_model *m, half_t *out);

int encode_image_dev(moon_vision_model *m, const half_t *patches, half_t *out) {
    moon_ctx *ctx = m->ctx;
    const size_t T = m->io_cfg.tokens, K = m->io_cfg.patch_dim, Kp = m->kp, R = 2 * T;
    MOON_HIP(ctx, hipMemcpy2DAsync(m->patches_pad, Kp * sizeof(half_t), patches, K * sizeof(half_t), K * sizeof(half_t), R,
                                   hipMemcpyDeviceToDevice, ctx->stream)); // (the pad columns stay zero)
    return encode_image_padded(m, out);
}

// VisionModel.vision_encoder (vision_model.zig:204-271) from m->patches_pad[2T, kp] on: m->enc[2T, dim]
static int vision_encoder_padded(moon_vision_model *m) {
    moon_ctx *ctx = m->ctx;
    const size_t d = m->cfg.dim, T = m->io_cfg.tokens, Kp = m->kp, R = 2 * T;
    // patch embedding: x = patches . W + b, then += pos_embedding on each crop (:219-229)
    MOON_TRY(launch_gemm(ctx, m->patches_pad, m->pe_w, m->pe_b, m->emb, R, d, Kp, MOON_B_NK, MOON_EPI_BIAS));
    for (size_t img = 0; img < 2; img++) MOON_TRY(launch_add(ctx, m->emb + img * T * d, m->pos, T * d));
    // the encoder blocks and the final LayerNorm on all 2T rows (:231-270)
    return encode_dev(m, m->emb, R, m->enc);
}

// from m->patches_pad[2T, kp] on
static int encode_image_padded(moon_vision_model *m, half_t *out) {
    moon_ctx *ctx = m->ctx;
    const size_t d = m->cfg.dim, T = m->io_cfg.tokens;
    MOON_TRY(vision_encoder_padded(m));
    // concat(output_0, output_1) along the features (:189-196), then encode_mlp (:366-387)
    for (size_t img = 0; img < 2; img++)
        MOON_HIP(ctx, hipMemcpy2DAsync(m->cat + img * d, 2 * d * sizeof(half_t), m->enc + img * T * d, d * sizeof(half_t), d * sizeof(half_t), T,
                                       hipMemcpyDeviceToDevice, ctx->stream));
    MOON_TRY(launch_gemm(ctx, m->cat, m->p1_w, m->p1_b, m->hid, T, m->io_cfg.proj_hidden, 2 * d, MOON_B_NK, MOON_EPI_BIAS_GELU));
    return launch_gemm(ctx, m->hid, m->p2_w, m->p2_b, out, T, m->io_cfg.out_dim, m->io_cfg.proj_hidden, MOON_B_NK, MOON_EPI_BIAS);
}

int io_attach(moon_vision_model *m, const moon_vision_io_config *cfg, const moon_vision_io_weights *w, bool synthetic, uint64_t seed,
              float std_dev) {
    moon_ctx *ctx = m->ctx;
    if (!cfg) return moon_fail(ctx, MOON_EINVAL, "vision io: null config");
    if (!cfg->patch_dim || !cfg->tokens || !cfg->proj_hidden || !cfg->out_dim) return moon_fail(ctx, MOON_EINVAL_DIM, "vision io: zero dimension");
    if (m->io) return moon_fail(ctx, MOON_EINVAL, "vision io: already attached");
    if (!synthetic) {
        if (!w) return moon_fail(ctx, MOON_EINVAL, "vision io: null weights");
        const void *ptrs[] = {w->v_patch_embedding_linear_w, w->v_patch_embedding_linear_b, w->v_pos_embedding, w->v_proj_fc1_w,
                              w->v_proj_fc1_b, w->v_proj_fc2_w, w->v_proj_fc2_b};
        for (const void *p : ptrs)
            if (!p) return moon_fail(ctx, MOON_EINVAL, "vision io: a weight pointer is null");
    }
    MOON_HIP(ctx, hipSetDevice(ctx->device));
    const size_t d = m->cfg.dim, T = cfg->tokens, K = cfg->patch_dim, Kp = (K + 63) / 64 * 64, Hp = cfg->proj_hidden, O = cfg->out_dim;
    m->io_cfg = *cfg;
    m->kp = Kp;
    MOON_TRY(dalloc(m, m->allocs, d * Kp, &m->pe_w));
    MOON_TRY(dalloc(m, m->allocs, d, &m->pe_b));
    MOON_TRY(dalloc(m, m->allocs, T * d, &m->pos));
    MOON_TRY(dalloc(m, m->allocs, Hp * 2 * d, &m->p1_w));
    MOON_TRY(dalloc(m, m->allocs, Hp, &m->p1_b));
    MOON_TRY(dalloc(m, m->allocs, O * Hp, &m->p2_w));
    MOON_TRY(dalloc(m, m->allocs, O, &m->p2_b));
    MOON_TRY(dalloc(m, m->allocs, 2 * T * Kp, &m->patches_pad));
    MOON_TRY(dalloc(m, m->allocs, 2 * T * d, &m->emb));
    MOON_TRY(dalloc(m, m->allocs, 2 * T * d, &m->enc));
    MOON_TRY(dalloc(m, m->allocs, T * 2 * d, &m->cat));
    MOON_TRY(dalloc(m, m->allocs, T * Hp, &m->hid));
    MOON_TRY(dalloc(m, m->allocs, T * O, &m->img_out));
    MOON_HIP(ctx, hipMemsetAsync(m->patches_pad, 0, 2 * T * Kp * sizeof(half_t), ctx->stream));
    MOON_HIP(ctx, hipMemsetAsync(m->pe_w, 0, d * Kp * sizeof(half_t), ctx->stream));
    size_t biggest = K * d;
    if (2 * d * Hp > biggest) biggest = 2 * d * Hp;
    if (Hp * O > biggest) biggest = Hp * O;
    half_t *tmp = nullptr, *tmp_t = nullptr; // a matrix in the file layout, and the patch matrix transposed before padding
    if (hipMalloc((void **)&tmp, biggest * sizeof(half_t)) != hipSuccess || hipMalloc((void **)&tmp_t, K * d * sizeof(half_t)) != hipSuccess) {
        if (tmp) (void)hipFree(tmp);
        return moon_fail(ctx, MOON_ENOMEM, "vision io: staging allocation failed");
    }
    int rc = MOON_OK;
    // stream numbers = 120 + declaration order of moon_vision_io_weights
    auto stage = [&](const moon_f16 *src, size_t n, uint64_t stream) { // -> tmp
        if (rc != MOON_OK) return;
        if (synthetic) rc = launch_fill_normal(ctx, tmp, n, seed, stream, std_dev);
        else if (hipMemcpyAsync(tmp, src, n * sizeof(half_t), hipMemcpyHostToDevice, ctx->stream) != hipSuccess)
            rc = moon_fail(ctx, MOON_EHIP, "vision io: weight upload failed");
    };
    auto vec = [&](half_t *dst, const moon_f16 *src, size_t n, uint64_t stream) {
        if (rc != MOON_OK) return;
        if (synthetic) rc = launch_fill_normal(ctx, dst, n, seed, stream, std_dev);
        else if (hipMemcpyAsync(dst, src, n * sizeof(half_t), hipMemcpyHostToDevice, ctx->stream) != hipSuccess)
            rc = moon_fail(ctx, MOON_EHIP, "vision io: weight upload failed");
    };
    stage(w ? w->v_patch_embedding_linear_w : nullptr, K * d, 120);
    if (rc == MOON_OK) rc = launch_transpose(ctx, tmp, tmp_t, K, d); // [K][d] -> [d][K]
    if (rc == MOON_OK && hipMemcpy2DAsync(m->pe_w, Kp * sizeof(half_t), tmp_t, K * sizeof(half_t), K * sizeof(half_t), d, hipMemcpyDeviceToDevice,
                                          ctx->stream) != hipSuccess)
        rc = moon_fail(ctx, MOON_EHIP, "vision io: padding the patch matrix failed");
    vec(m->pe_b, w ? w->v_patch_embedding_linear_b : nullptr, d, 121);
    vec(m->pos, w ? w->v_pos_embedding : nullptr, T * d, 122);
    stage(w ? w->v_proj_fc1_w : nullptr, 2 * d * Hp, 123);
    if (rc == MOON_OK) rc = launch_transpose(ctx, tmp, m->p1_w, 2 * d, Hp);
    vec(m->p1_b, w ? w->v_proj_fc1_b : nullptr, Hp, 124);
    stage(w ? w->v_proj_fc2_w : nullptr, Hp * O, 125);
    if (rc == MOON_OK) rc = launch_transpose(ctx, tmp, m->p2_w, Hp, O);
    vec(m->p2_b, w ? w->v_proj_fc2_b : nullptr, O, 126);
    if (rc == MOON_OK && hipStreamSynchronize(ctx->stream) != hipSuccess) rc = moon_fail(ctx, MOON_EHIP, "vision io: weight setup failed");
    (void)hipStreamSynchronize(ctx->stream);
    (void)hipFree(tmp);
    (void)hipFree(tmp_t);
    if (rc == MOON_OK) m->io = true;
    return rc;
}

} // namespace

extern "C" void moon_vision_io_config_default(moon_vision_io_config *cfg) {
    if (!cfg) return;
    cfg->patch_dim = 14 * 14 * 3;
    cfg->tokens = 729;
    cfg->proj_hidden = 8192;
    cfg->out_dim = 2048;
}

extern "C" int moon_vision_io_attach(moon_vision_model *m, const moon_vision_io_config *cfg, const moon_vision_io_weights *w) {
    if (!m) return MOON_EINVAL;
    std::lock_guard<std::mutex> lock(m->ctx->mu);
    return io_attach(m, cfg, w, false, 0, 0.0f);
}

extern "C" int moon_vision_io_attach_synthetic(moon_vision_model *m, const moon_vision_io_config *cfg, uint64_t seed, float std_dev) {
    if (!m) return MOON_EINVAL;
    std::lock_guard<std::mutex> lock(m->ctx->mu);
    return io_attach(m, cfg, nullptr, true, seed, std_dev);
}

extern "C" int moon_vision_encode_image_dev(moon_vision_model *m, const void *patches, void *out) {
    if (!m) return MOON_EINVAL;
    std::lock_guard<std::mutex> lock(m->ctx->mu);
    if (!m->io) return moon_fail(m->ctx, MOON_EINVAL, "vision_encode_image: no front / back end attached (moon_vision_io_attach)");
    if (!patches || !out) return moon_fail(m->ctx, MOON_EINVAL, "vision_encode_image: null operand");
    MOON_HIP(m->ctx, hipSetDevice(m->ctx->device));
    return encode_image_dev(m, (const half_t *)patches, (half_t *)out);
}

extern "C" int moon_vision_encode_image(moon_vision_model *m, const moon_f16 *patches, moon_f16 *out) {
    if (!m) return MOON_EINVAL;
    moon_ctx *ctx = m->ctx;
    std::lock_guard<std::mutex> lock(ctx->mu);
    if (!m->io) return moon_fail(ctx, MOON_EINVAL, "vision_encode_image: no front / back end attached (moon_vision_io_attach)");
    if (!patches || !out) return moon_fail(ctx, MOON_EINVAL, "vision_encode_image: null operand");
    MOON_HIP(ctx, hipSetDevice(ctx->device));
    const size_t in_bytes = 2 * m->io_cfg.tokens * m->io_cfg.patch_dim * sizeof(moon_f16);
    MOON_TRY(moon_grow(ctx, ctx->stage[0], in_bytes));
    MOON_HIP(ctx, hipMemcpyAsync(ctx->stage[0].ptr, patches, in_bytes, hipMemcpyHostToDevice, ctx->stream));
    MOON_TRY(encode_image_dev(m, (const half_t *)ctx->stage[0].ptr, m->img_out));
    MOON_HIP(ctx, hipMemcpyAsync(out, m->img_out, m->io_cfg.tokens * m->io_cfg.out_dim * sizeof(moon_f16), hipMemcpyDeviceToHost, ctx->stream));
    MOON_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return MOON_OK;
}

extern "C" int moon_vision_encoder(moon_vision_model *m, const moon_f16 *patches, moon_f16 *out) {
    if (!m) return MOON_EINVAL;
    moon_ctx *ctx = m->ctx;
    std::lock_guard<std::mutex> lock(ctx->mu);
    if (!m->io) return moon_fail(ctx, MOON_EINVAL, "vision_encoder: no front / back end attached (moon_vision_io_attach)");
    if (!patches || !out) return moon_fail(ctx, MOON_EINVAL, "vision_encoder: null operand");
    MOON_HIP(ctx, hipSetDevice(ctx->device));
    const size_t T = m->io_cfg.tokens, K = m->io_cfg.patch_dim, R = 2 * T, in_bytes = R * K * sizeof(moon_f16);
    MOON_TRY(moon_grow(ctx, ctx->stage[0], in_bytes));
    MOON_HIP(ctx, hipMemcpyAsync(ctx->stage[0].ptr, patches, in_bytes, hipMemcpyHostToDevice, ctx->stream));
    MOON_HIP(ctx, hipMemcpy2DAsync(m->patches_pad, m->kp * sizeof(half_t), ctx->stage[0].ptr, K * sizeof(half_t), K * sizeof(half_t), R,
                                   hipMemcpyDeviceToDevice, ctx->stream)); // (the pad columns stay zero)
    MOON_TRY(vision_encoder_padded(m));
    MOON_HIP(ctx, hipMemcpyAsync(out, m->enc, R * m->cfg.dim * sizeof(moon_f16), hipMemcpyDeviceToHost, ctx->stream));
    MOON_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return MOON_OK;
}

// encode_image from the resized image on (vision_model.zig:129-229): the normalised patches are written straight into the
// padded operand of the patch-embedding GEMM
extern "C" int moon_vision_encode_image_u8(moon_vision_model *m, const uint8_t *image, moon_f16 *out) {
    if (!m) return MOON_EINVAL;
    moon_ctx *ctx = m->ctx;
    std::lock_guard<std::mutex> lock(ctx->mu);
    if (!m->io) return moon_fail(ctx, MOON_EINVAL, "vision_encode_image_u8: no front / back end attached (moon_vision_io_attach)");
    if (!image || !out) return moon_fail(ctx, MOON_EINVAL, "vision_encode_image_u8: null operand");
    size_t grid = 0, patch = 0;
    while (grid * grid < m->io_cfg.tokens) grid++;
    while (3 * patch * patch < m->io_cfg.patch_dim) patch++;
    if (grid * grid != m->io_cfg.tokens || 3 * patch * patch != m->io_cfg.patch_dim)
        return moon_fail(ctx, MOON_EINVAL_DIM, "vision_encode_image_u8: %zu tokens of %zu values are not a square grid of square RGB patches",
                         m->io_cfg.tokens, m->io_cfg.patch_dim);
    MOON_HIP(ctx, hipSetDevice(ctx->device));
    const size_t side = grid * patch, in_bytes = side * side * 3;
    MOON_TRY(moon_grow(ctx, ctx->stage[0], in_bytes));
    MOON_HIP(ctx, hipMemcpyAsync(ctx->stage[0].ptr, image, in_bytes, hipMemcpyHostToDevice, ctx->stream));
    MOON_TRY(launch_image_patches(ctx, (const uint8_t *)ctx->stage[0].ptr, m->patches_pad, side, side, 3, patch, 2, m->kp));
    MOON_TRY(encode_image_padded(m, m->img_out));
    MOON_HIP(ctx, hipMemcpyAsync(out, m->img_out, m->io_cfg.tokens * m->io_cfg.out_dim * sizeof(moon_f16), hipMemcpyDeviceToHost, ctx->stream));
    MOON_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return MOON_OK;
}

extern "C" void moon_vision_config_default(moon_vision_config *cfg) {
    if (!cfg) return;
    cfg->dim = 1152;
    cfg->hidden_dim = 4304;
    cfg->n_layers = 27;
    cfg->n_heads = 16;
    cfg->head_dim = 72;
    cfg->ln_eps = 1.00135803e-5f;
}

static int vision_create(moon_ctx *ctx, const moon_vision_config *cfg, const moon_vision_weights *w, bool synthetic, uint64_t seed,
                         float std_dev, moon_vision_model **out) {
    if (!ctx || !out) return MOON_EINVAL;
    std::lock_guard<std::mutex> lock(ctx->mu);
    *out = nullptr;
    MOON_TRY(check_cfg(ctx, cfg));
    if (!synthetic) {
        if (!w) return moon_fail(ctx, MOON_EINVAL, "vision model: null weights");
        const void *ptrs[] = {w->v_Wqkv_w, w->v_Wqkv_b, w->v_out_proj_w, w->v_out_proj_b, w->v_fc1_w, w->v_fc1_b, w->v_fc2_w,
                              w->v_fc2_b, w->v_norm1_w, w->v_norm1_b, w->v_norm2_w, w->v_norm2_b, w->v_norm_out_w, w->v_norm_out_b};
        for (const void *p : ptrs)
            if (!p) return moon_fail(ctx, MOON_EINVAL, "vision model: a weight pointer is null");
    }
    MOON_HIP(ctx, hipSetDevice(ctx->device));
    moon_vision_model *m = new moon_vision_model();
    m->ctx = ctx;
    m->cfg = *cfg;
    m->fp = (cfg->hidden_dim + 63) / 64 * 64;
    const size_t L = cfg->n_layers, d = cfg->dim, f = cfg->hidden_dim, fp = m->fp;
    int rc = alloc_weights(m);
    half_t *tmp = nullptr; // staging for one matrix family in the file layout, then one padded fc2 matrix
    size_t biggest = L * 3 * d * d;
    if (L * d * f > biggest) biggest = L * d * f;
    if (rc == MOON_OK && hipMalloc((void **)&tmp, (biggest + fp * d) * sizeof(half_t)) != hipSuccess)
        rc = moon_fail(ctx, MOON_ENOMEM, "vision model: staging allocation failed");
    half_t *pad = tmp ? tmp + biggest : nullptr; // [fp][d]
    // stream numbers = 100 + declaration order of moon_vision_weights
    auto mat = [&](half_t *dst, const moon_f16 *src, size_t in, size_t outn, uint64_t stream) {
        if (rc != MOON_OK) return;
        if (synthetic) {
            rc = launch_fill_normal(ctx, tmp, L * in * outn, seed, stream, std_dev);
        } else if (hipMemcpyAsync(tmp, src, L * in * outn * sizeof(half_t), hipMemcpyHostToDevice, ctx->stream) != hipSuccess) {
            rc = moon_fail(ctx, MOON_EHIP, "vision model: weight upload failed");
        }
        if (rc == MOON_OK) rc = transpose_layers(m, tmp, dst, L, in, outn);
    };
    auto vec = [&](half_t *dst, const moon_f16 *src, size_t n, uint64_t stream, int kind /*0 random, 1 ones, 2 zeros*/) {
        if (rc != MOON_OK) return;
        if (!synthetic) {
            if (hipMemcpyAsync(dst, src, n * sizeof(half_t), hipMemcpyHostToDevice, ctx->stream) != hipSuccess)
                rc = moon_fail(ctx, MOON_EHIP, "vision model: weight upload failed");
        } else if (kind == 0) {
            rc = launch_fill_normal(ctx, dst, n, seed, stream, std_dev);
        } else {
            rc = launch_fill_const(ctx, dst, n, kind == 1 ? 1.0f : 0.0f);
        }
    };
    mat(m->qkv_w, w ? w->v_Wqkv_w : nullptr, d, 3 * d, 100);
    vec(m->qkv_b, w ? w->v_Wqkv_b : nullptr, L * 3 * d, 101, 0);
    mat(m->out_w, w ? w->v_out_proj_w : nullptr, d, d, 102);
    vec(m->out_b, w ? w->v_out_proj_b : nullptr, L * d, 103, 0);
    // stage(): one matrix family into tmp in the file layout, without transposing
    auto stage = [&](const moon_f16 *src, size_t n, uint64_t stream) {
        if (rc != MOON_OK) return;
        if (synthetic) rc = launch_fill_normal(ctx, tmp, n, seed, stream, std_dev);
        else if (hipMemcpyAsync(tmp, src, n * sizeof(half_t), hipMemcpyHostToDevice, ctx->stream) != hipSuccess)
            rc = moon_fail(ctx, MOON_EHIP, "vision model: weight upload failed");
    };
    auto hip_ok = [&](hipError_t e) {
        if (rc == MOON_OK && e != hipSuccess) rc = moon_fail(ctx, MOON_EHIP, "vision model: weight setup failed: %s", hipGetErrorString(e));
    };
    if (fp == f) {
        mat(m->fc1_w, w ? w->v_fc1_w : nullptr, d, f, 104);
        vec(m->fc1_b, w ? w->v_fc1_b : nullptr, L * f, 105, 0);
        mat(m->fc2_w, w ? w->v_fc2_w : nullptr, f, d, 106);
    } else {
        // fc1 [d][f] -> the first f rows of [fp][d], the rest zero; its bias the first f of fp
        if (rc == MOON_OK) rc = launch_fill_const(ctx, m->fc1_w, L * fp * d, 0.0f);
        stage(w ? w->v_fc1_w : nullptr, L * d * f, 104);
        for (size_t l = 0; l < L && rc == MOON_OK; l++) rc = launch_transpose(ctx, tmp + l * d * f, m->fc1_w + l * fp * d, d, f);
        if (rc == MOON_OK) rc = launch_fill_const(ctx, m->fc1_b, L * fp, 0.0f);
        stage(w ? w->v_fc1_b : nullptr, L * f, 105);
        if (rc == MOON_OK)
            hip_ok(hipMemcpy2DAsync(m->fc1_b, fp * sizeof(half_t), tmp, f * sizeof(half_t), f * sizeof(half_t), L, hipMemcpyDeviceToDevice, ctx->stream));
        // fc2 [f][d] -> zero rows appended to [fp][d], then transposed to [d][fp]
        stage(w ? w->v_fc2_w : nullptr, L * f * d, 106);
        if (rc == MOON_OK) rc = launch_fill_const(ctx, pad, fp * d, 0.0f);
        for (size_t l = 0; l < L && rc == MOON_OK; l++) {
            hip_ok(hipMemcpyAsync(pad, tmp + l * f * d, f * d * sizeof(half_t), hipMemcpyDeviceToDevice, ctx->stream));
            if (rc == MOON_OK) rc = launch_transpose(ctx, pad, m->fc2_w + l * d * fp, fp, d);
        }
    }
    vec(m->fc2_b, w ? w->v_fc2_b : nullptr, L * d, 107, 0);
    vec(m->n1_w, w ? w->v_norm1_w : nullptr, L * d, 108, 1);
    vec(m->n1_b, w ? w->v_norm1_b : nullptr, L * d, 109, 2);
    vec(m->n2_w, w ? w->v_norm2_w : nullptr, L * d, 110, 1);
    vec(m->n2_b, w ? w->v_norm2_b : nullptr, L * d, 111, 2);
    vec(m->no_w, w ? w->v_norm_out_w : nullptr, d, 112, 1);
    vec(m->no_b, w ? w->v_norm_out_b : nullptr, d, 113, 2);
    if (rc == MOON_OK && hipStreamSynchronize(ctx->stream) != hipSuccess) rc = moon_fail(ctx, MOON_EHIP, "vision model: weight setup failed");
    if (tmp) {
        (void)hipStreamSynchronize(ctx->stream);
        (void)hipFree(tmp);
    }
    if (rc != MOON_OK) {
        free_all(m);
        delete m;
        return rc;
    }
    *out = m;
    return MOON_OK;
}

extern "C" int moon_vision_model_create(moon_ctx *ctx, const moon_vision_config *cfg, const moon_vision_weights *w,
                                        moon_vision_model **out) {
    return vision_create(ctx, cfg, w, false, 0, 0.0f, out);
}

extern "C" int moon_vision_model_create_synthetic(moon_ctx *ctx, const moon_vision_config *cfg, uint64_t seed, float std_dev,
                                                  moon_vision_model **out) {
    return vision_create(ctx, cfg, nullptr, true, seed, std_dev, out);
}

extern "C" void moon_vision_model_destroy(moon_vision_model *m) {
    if (!m) return;
    {
        std::lock_guard<std::mutex> lock(m->ctx->mu);
        free_all(m);
    }
    delete m;
}

extern "C" int moon_vision_encode_dev(moon_vision_model *m, const void *x, size_t tokens, void *out) {
    if (!m) return MOON_EINVAL;
    std::lock_guard<std::mutex> lock(m->ctx->mu);
    if (!x || !out) return moon_fail(m->ctx, MOON_EINVAL, "vision_encode: null operand");
    if (!tokens) return MOON_OK;
    MOON_HIP(m->ctx, hipSetDevice(m->ctx->device));
    return encode_dev(m, (const half_t *)x, tokens, (half_t *)out);
}

extern "C" int moon_vision_encode(moon_vision_model *m, const moon_f16 *x, size_t tokens, moon_f16 *out) {
    if (!m) return MOON_EINVAL;
    moon_ctx *ctx = m->ctx;
    std::lock_guard<std::mutex> lock(ctx->mu);
    if (!x || !out) return moon_fail(ctx, MOON_EINVAL, "vision_encode: null operand");
    if (!tokens) return MOON_OK;
    MOON_HIP(ctx, hipSetDevice(ctx->device));
    const size_t bytes = tokens * m->cfg.dim * sizeof(moon_f16);
    MOON_TRY(moon_grow(ctx, ctx->stage[0], bytes));
    MOON_TRY(moon_grow(ctx, ctx->stage[2], bytes));
    MOON_HIP(ctx, hipMemcpyAsync(ctx->stage[0].ptr, x, bytes, hipMemcpyHostToDevice, ctx->stream));
    MOON_TRY(encode_dev(m, (const half_t *)ctx->stage[0].ptr, tokens, (half_t *)ctx->stage[2].ptr));
    MOON_HIP(ctx, hipMemcpyAsync(out, ctx->stage[2].ptr, bytes, hipMemcpyDeviceToHost, ctx->stream));
    MOON_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return MOON_OK;
}
