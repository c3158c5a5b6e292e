// Device-resident text decoder session: TextModel.text_encoder / text_decoder / attention_block / mlp /
// lm_head (text_model.zig:106-345) with its KVCache (text_model.zig:349-539) and the greedy loop of
// moondream.zig:323-368.  Weights are uploaded once in the moondream.bin text layout ([L, out, in] rows,
// weights.zig:439-454), which is already the k-contiguous [N,K] form both the GEMV and the GEMM kernels read.
// Activations and the cache never leave the device; a decode step enqueues kernels only (token id and position
// are read from device memory), so the loop needs no host synchronisation until the ids are fetched.
#include "moon_internal.hpp"

#include <cstdlib>
#include <cstring>
#include <algorithm>
#include <vector>

// fused decode kernels (decode_fused.hip)
bool decode_fused_supported(size_t d, size_t ffn);
int launch_decode_ln_gemv(moon_ctx *ctx, const half_t *x, const uint32_t *token, const half_t *gamma, const half_t *beta, float eps,
                          size_t d, const half_t *W1, const half_t *b1, half_t *y1, size_t N1, const half_t *W2, const half_t *b2,
                          half_t *y2, size_t N2);
int launch_decode_out_fc2(moon_ctx *ctx, const half_t *attn, const half_t *fc1, const half_t *Wo, const half_t *bo, const half_t *W2,
                          const half_t *b2, half_t *hidden, const half_t *hidden_src, const uint32_t *token, size_t d, size_t ffn);
int launch_decode_attention_merged(moon_ctx *ctx, const half_t *qkv, half_t *cache_k, half_t *cache_v, const float *table, float *partial,
                                   half_t *out, uint32_t *head_count, uint32_t count_target, size_t H, size_t D, size_t rot_dim,
                                   size_t max_seq, size_t pos, const uint32_t *pos_dev, size_t head_stride = 1);
int launch_argmax_record(moon_ctx *ctx, const half_t *logits, size_t n, uint32_t *state, uint32_t *out_ids);
size_t decode_lm_head_words(moon_ctx *ctx);
int launch_decode_lm_head(moon_ctx *ctx, const half_t *x, const half_t *gamma, const half_t *beta, float eps, size_t d, const half_t *W,
                          const half_t *bias, half_t *logits, size_t V, uint32_t *exchange, uint32_t generation, uint32_t *state,
                          uint32_t *out_ids, uint32_t bump, const moon_sampling_config *top_k_cfg = nullptr, const float *u_dev = nullptr,
                          uint32_t *decided = nullptr);
bool decode_lm_head_top_k_supported(moon_ctx *ctx, size_t top_k, size_t V);
bool decode_front_supported(moon_ctx *ctx, size_t d, size_t H, size_t D);
bool decode_layer_supported(moon_ctx *ctx, size_t d, size_t ffn, size_t H, size_t D);
size_t decode_layer_sync_words(size_t H);
int launch_decode_layer(moon_ctx *ctx, const half_t *x, const uint32_t *token, const half_t *gamma, const half_t *beta, float eps, size_t d,
                        const half_t *Wqkv, const half_t *bqkv, half_t *qkv, const half_t *W1, const half_t *b1, half_t *fc1, size_t ffn,
                        const half_t *Wo, const half_t *bo, const half_t *W2, const half_t *b2, half_t *hidden, const half_t *hidden_src,
                        half_t *cache_k, half_t *cache_v, const float *table, float *partial, half_t *attn_out, uint32_t *head_count,
                        uint32_t head_target, uint32_t *sync, uint32_t generation, uint32_t *error, size_t H, size_t rot_dim, size_t max_seq,
                        size_t pos, const uint32_t *pos_dev, long long *trace);
int launch_decode_front(moon_ctx *ctx, const half_t *x, const uint32_t *token, const half_t *gamma, const half_t *beta, float eps, size_t d,
                        const half_t *Wqkv, const half_t *bqkv, half_t *qkv, const half_t *W1, const half_t *b1, half_t *fc1, size_t ffn,
                        half_t *cache_k, half_t *cache_v, const float *table, float *partial, half_t *attn_out, uint32_t *head_count,
                        uint32_t head_target, uint32_t *qkv_count, uint32_t qkv_target, uint32_t *error, size_t H, size_t rot_dim,
                        size_t max_seq, size_t pos, const uint32_t *pos_dev);

// Per-kernel timing of the fused decode step: a HIP event pair on the library's stream around every launch of one
// step, read back after the step has finished.
enum { PROF_LN_GEMV = 0, PROF_ATTN = 1, PROF_OUT_FC2 = 2, PROF_LM_HEAD = 3, PROF_ARGMAX = 4, PROF_BUMP = 5, PROF_KINDS = 6 };
struct StepProfiler {
    std::vector<hipEvent_t> events;
    std::vector<int> kinds; // kind of the launch between events[2i] and events[2i+1]
    double sum_ms[PROF_KINDS] = {};
    size_t count[PROF_KINDS] = {};
};

struct moon_text_model {
    moon_ctx *ctx = nullptr;
    moon_text_config cfg{};
    // weights
    half_t *wte = nullptr, *ln_w = nullptr, *ln_b = nullptr, *qkv_w = nullptr, *qkv_b = nullptr, *out_w = nullptr, *out_b = nullptr,
           *fc1_w = nullptr, *fc1_b = nullptr, *fc2_w = nullptr, *fc2_b = nullptr, *lin_w = nullptr, *lin_b = nullptr,
           *lno_w = nullptr, *lno_b = nullptr;
    half_t *cache_k = nullptr, *cache_v = nullptr; // [L][H][max_seq][D]
    float *freqs = nullptr;                        // [max_seq][rot_dim/2][2]
    // activations
    half_t *hidden = nullptr, *ln_in = nullptr, *qkv = nullptr, *q_rot = nullptr, *attn = nullptr, *attn_proj = nullptr,
           *fc1 = nullptr, *mlp = nullptr, *logits = nullptr, *ln_last = nullptr;
    uint32_t *ids_dev = nullptr;   // [max_seq] prompt ids / generated ids
    uint32_t *ids_pinned = nullptr; // [max_seq] page-locked host memory the prompt ids are copied from (a copy from pageable memory blocks the call)
    uint32_t *host_words = nullptr; // [64] page-locked: where the calls' small results land (error words, a token, the loop's state)
    // page-locked staging for what the per-token calls move (a row of embeddings up; a hidden row, the logits, the ids down):
    // a copy between device memory and the caller's pageable memory blocks the call for tens of microseconds
    unsigned char *stage_up = nullptr, *stage_down = nullptr; // STAGE_BYTES each
    float *u_dev = nullptr;        // [max_seq] the sampling loop's random numbers, one per step
    uint32_t *state_dev = nullptr; // [0] position (KV length), [1] tokens recorded, [2] current token, [3] stopped, [4] eos id + 1 (record_token)
    size_t cur_len = 0, last_n = 0;
    bool cache_invalid = false;    // a fused decode kernel gave up on a wait: positions may be missing from the cache until moon_text_reset
    int decode_mode = 0;           // 0: one kernel per layer where the device holds it (default); 2: three kernels per layer; 3: two
    float *attn_partial = nullptr; // [H][8][66]
    // fused per-layer decode kernels
    bool fused = false;              // shape supported by decode_fused.hip
    uint32_t *head_count = nullptr;  // [L][H] "splits finished" counters, monotonically increasing
    std::vector<uint32_t> attn_launches; // per layer: decode-attention launches so far
    bool front = false;               // LayerNorm + qkv + fc1 + attention can run as one launch
    uint32_t *front_sync = nullptr;   // [L][H] qkv-row counters, one 128-byte line each (monotonic), then one error word
    std::vector<uint32_t> front_launches; // per layer: front-kernel launches since the counters were last cleared
    bool whole_layer = false;         // a whole layer can run as one launch (decode_layer_kernel)
    uint32_t *layer_sync = nullptr;   // [L][decode_layer_sync_words] counters (monotonic), then one error word
    size_t layer_sync_words = 0;
    std::vector<uint32_t> layer_launches;
    uint32_t *lm_exchange = nullptr;  // arg-max pairs of the LM head's workgroups, then their counter (monotonic)
    uint32_t lm_launches = 0;
    long long *layer_trace = nullptr; // [grid][8] stamps of the most recent layer launch when MOON_DECODE_TRACE is set
    struct StepProfiler *prof = nullptr;  // set only inside moon_text_greedy_profile
    std::vector<void *> allocs;
};

namespace {

constexpr size_t STAGE_BYTES = size_t(256) << 10; // (the logits of a 51,200-word vocabulary are 100 KB)

__global__ void bump_pos_kernel(uint32_t *state) {
    if (!state[3]) state[0] += 1;
}
// two neighbouring words (the loop's position and step count; also used to raise an error word next to a counter's tail)
__global__ void set_state_kernel(uint32_t *state, uint32_t pos, uint32_t step) {
    state[0] = pos;
    state[1] = step;
}
// the generation loop's state before its first step (record_token): position, no tokens yet, not stopped, eos id + 1 (0: none)
__global__ void start_loop_kernel(uint32_t *state, uint32_t pos, uint32_t eos_plus1) {
    state[0] = pos;
    state[1] = 0;
    state[3] = 0;
    state[4] = eos_plus1;
}

int dalloc(moon_text_model *m, size_t bytes, void **p) {
    MOON_HIP(m->ctx, hipMalloc(p, bytes ? bytes : 16));
    m->allocs.push_back(*p);
    return MOON_OK;
}
template <class T> int dalloc_t(moon_text_model *m, size_t n, T **p) { return dalloc(m, n * sizeof(T), (void **)p); }

// Host -> device, queued on the context's stream: small pieces go through the page-locked staging buffer (free again at the
// call's final synchronisation; one use per call), large ones straight from the caller's memory.
int copy_up(moon_text_model *m, void *dst_dev, const void *src_host, size_t bytes) {
    if (bytes <= STAGE_BYTES && m->stage_up) {
        memcpy(m->stage_up, src_host, bytes);
        src_host = m->stage_up;
    }
    MOON_HIP(m->ctx, hipMemcpyAsync(dst_dev, src_host, bytes, hipMemcpyHostToDevice, m->ctx->stream));
    return MOON_OK;
}
// Device -> host and the synchronisation that ends the call
int copy_down_sync(moon_text_model *m, void *dst_host, const void *src_dev, size_t bytes) {
    const bool staged = bytes <= STAGE_BYTES && m->stage_down;
    MOON_HIP(m->ctx, hipMemcpyAsync(staged ? (void *)m->stage_down : dst_host, src_dev, bytes, hipMemcpyDeviceToHost, m->ctx->stream));
    MOON_HIP(m->ctx, hipStreamSynchronize(m->ctx->stream));
    if (staged) memcpy(dst_host, m->stage_down, bytes);
    return MOON_OK;
}

struct Sizes {
    size_t L, d, ffn, V, H, D, S;
};
Sizes sizes(const moon_text_config &c) { return {c.n_layers, c.dim, c.hidden_dim, c.vocab, c.n_heads, c.head_dim, c.max_seq}; }

int check_cfg(moon_ctx *ctx, const moon_text_config *c) {
    if (!c) return moon_fail(ctx, MOON_EINVAL, "text model: null config");
    if (!c->vocab || !c->dim || !c->hidden_dim || !c->n_layers || !c->n_heads || !c->head_dim || !c->max_seq)
        return moon_fail(ctx, MOON_EINVAL_DIM, "text model: zero dimension");
    if (c->n_heads * c->head_dim != c->dim) return moon_fail(ctx, MOON_EINVAL_DIM, "text model: n_heads*head_dim != dim");
    if (c->head_dim != 64) return moon_fail(ctx, MOON_EINVAL_DIM, "text model: head_dim must be 64 (attention.zig:248)");
    if (c->rot_dim > c->head_dim || c->rot_dim % 2) return moon_fail(ctx, MOON_EROT_DIM, "text model: bad rot_dim");
    if (c->max_seq > 2048) return moon_fail(ctx, MOON_ESEQ_TOO_LONG, "text model: max_seq > 2048 (attention.zig:252)");
    if (!(c->ln_eps > 0.0f)) return moon_fail(ctx, MOON_EEPS, "text model: ln_eps must be > 0");
    return MOON_OK;
}

int alloc_all(moon_text_model *m) {
    const Sizes z = sizes(m->cfg);
    MOON_TRY(dalloc_t(m, z.V * z.d, &m->wte));
    MOON_TRY(dalloc_t(m, z.L * z.d, &m->ln_w));
    MOON_TRY(dalloc_t(m, z.L * z.d, &m->ln_b));
    MOON_TRY(dalloc_t(m, z.L * 3 * z.d * z.d, &m->qkv_w));
    MOON_TRY(dalloc_t(m, z.L * 3 * z.d, &m->qkv_b));
    MOON_TRY(dalloc_t(m, z.L * z.d * z.d, &m->out_w));
    MOON_TRY(dalloc_t(m, z.L * z.d, &m->out_b));
    MOON_TRY(dalloc_t(m, z.L * z.ffn * z.d, &m->fc1_w));
    MOON_TRY(dalloc_t(m, z.L * z.ffn, &m->fc1_b));
    MOON_TRY(dalloc_t(m, z.L * z.d * z.ffn, &m->fc2_w));
    MOON_TRY(dalloc_t(m, z.L * z.d, &m->fc2_b));
    MOON_TRY(dalloc_t(m, z.V * z.d, &m->lin_w));
    MOON_TRY(dalloc_t(m, z.V, &m->lin_b));
    MOON_TRY(dalloc_t(m, z.d, &m->lno_w));
    MOON_TRY(dalloc_t(m, z.d, &m->lno_b));
    MOON_TRY(dalloc_t(m, z.L * z.H * z.S * z.D, &m->cache_k));
    MOON_TRY(dalloc_t(m, z.L * z.H * z.S * z.D, &m->cache_v));
    MOON_TRY(dalloc_t(m, z.S * (m->cfg.rot_dim / 2) * 2 + 2, &m->freqs));
    MOON_TRY(dalloc_t(m, z.S * z.d, &m->hidden));
    MOON_TRY(dalloc_t(m, z.S * z.d, &m->ln_in));
    MOON_TRY(dalloc_t(m, z.S * 3 * z.d, &m->qkv));
    MOON_TRY(dalloc_t(m, z.S * z.d, &m->q_rot));
    MOON_TRY(dalloc_t(m, z.S * z.d, &m->attn));
    MOON_TRY(dalloc_t(m, z.S * z.d, &m->attn_proj));
    MOON_TRY(dalloc_t(m, z.S * z.ffn, &m->fc1));
    MOON_TRY(dalloc_t(m, z.S * z.d, &m->mlp));
    MOON_TRY(dalloc_t(m, z.V, &m->logits));
    MOON_TRY(dalloc_t(m, z.d, &m->ln_last));
    MOON_TRY(dalloc_t(m, z.S, &m->ids_dev));
    MOON_HIP(m->ctx, hipHostMalloc((void **)&m->ids_pinned, z.S * sizeof(uint32_t), hipHostMallocDefault));
    MOON_HIP(m->ctx, hipHostMalloc((void **)&m->host_words, 64 * sizeof(uint32_t), hipHostMallocDefault));
    MOON_HIP(m->ctx, hipHostMalloc((void **)&m->stage_up, STAGE_BYTES, hipHostMallocDefault));
    MOON_HIP(m->ctx, hipHostMalloc((void **)&m->stage_down, STAGE_BYTES, hipHostMallocDefault));
    MOON_TRY(dalloc_t(m, z.S, &m->u_dev));
    MOON_TRY(dalloc_t(m, 8, &m->state_dev));
    MOON_TRY(launch_fill_uniform_u32(m->ctx, m->state_dev, 8, 0, 0, 1)); // zeros
    MOON_TRY(dalloc_t(m, z.H * 8 * 66, &m->attn_partial));
    m->fused = decode_fused_supported(z.d, z.ffn);
    MOON_TRY(dalloc_t(m, z.L * z.H, &m->head_count));
    MOON_TRY(launch_fill_uniform_u32(m->ctx, m->head_count, z.L * z.H, 0, 0, 1)); // zeros
    m->attn_launches.assign(z.L, 0);
    m->front = m->fused && decode_front_supported(m->ctx, z.d, z.H, z.D);
    MOON_TRY(dalloc_t(m, z.L * z.H * 32 + 1, &m->front_sync));
    MOON_TRY(launch_fill_uniform_u32(m->ctx, m->front_sync, z.L * z.H * 32 + 1, 0, 0, 1)); // zeros
    m->front_launches.assign(z.L, 0);
    m->whole_layer = m->fused && decode_layer_supported(m->ctx, z.d, z.ffn, z.H, z.D);
    m->layer_sync_words = decode_layer_sync_words(z.H);
    MOON_TRY(dalloc_t(m, z.L * m->layer_sync_words + 1, &m->layer_sync));
    MOON_TRY(launch_fill_uniform_u32(m->ctx, m->layer_sync, z.L * m->layer_sync_words + 1, 0, 0, 1)); // zeros
    m->layer_launches.assign(z.L, 0);
    MOON_TRY(dalloc_t(m, decode_lm_head_words(m->ctx), &m->lm_exchange));
    MOON_TRY(launch_fill_uniform_u32(m->ctx, m->lm_exchange, decode_lm_head_words(m->ctx), 0, 0, 1)); // zeros
    if (getenv("MOON_DECODE_TRACE")) {
        MOON_TRY(dalloc_t(m, size_t(4096) * 8, &m->layer_trace));
        MOON_TRY(launch_fill_uniform_u32(m->ctx, (uint32_t *)m->layer_trace, size_t(4096) * 16, 0, 0, 1));
    }
    MOON_TRY(launch_rope_table(m->ctx, m->freqs, m->cfg.rot_dim, z.S, m->cfg.rope_theta));
    // a fresh cache reads as zeros, like the reference's zero-length cache never reads beyond current_len
    MOON_TRY(launch_fill_const(m->ctx, m->cache_k, z.L * z.H * z.S * z.D, 0.0f));
    MOON_TRY(launch_fill_const(m->ctx, m->cache_v, z.L * z.H * z.S * z.D, 0.0f));
    hipLaunchKernelGGL(set_state_kernel, dim3(1), dim3(1), 0, m->ctx->stream, m->state_dev, 0u, 0u);
    MOON_HIP(m->ctx, hipGetLastError());
    return MOON_OK;
}

void free_all(moon_text_model *m) {
    (void)hipStreamSynchronize(m->ctx->stream);
    for (void *p : m->allocs) (void)hipFree(p);
    m->allocs.clear();
    if (m->ids_pinned) (void)hipHostFree(m->ids_pinned);
    if (m->host_words) (void)hipHostFree(m->host_words);
    if (m->stage_up) (void)hipHostFree(m->stage_up);
    if (m->stage_down) (void)hipHostFree(m->stage_down);
    m->stage_up = m->stage_down = nullptr;
    m->ids_pinned = nullptr;
    m->host_words = nullptr;
}

// Counters, exchange buffers and error words of the fused decode kernels back to their initial state (fill kernels in
// stream order, no memset), and the host's launch counts with them.  A kernel that gave up on a wait leaves counters
// short of the targets the host has already moved on to; nothing that is cleared here survives such a launch.
int clear_sync_state(moon_text_model *m) {
    const Sizes z = sizes(m->cfg);
    moon_ctx *ctx = m->ctx;
    MOON_TRY(launch_fill_uniform_u32(ctx, m->head_count, z.L * z.H, 0, 0, 1));
    MOON_TRY(launch_fill_uniform_u32(ctx, m->front_sync, z.L * z.H * 32 + 1, 0, 0, 1));
    MOON_TRY(launch_fill_uniform_u32(ctx, m->layer_sync, z.L * m->layer_sync_words + 1, 0, 0, 1));
    MOON_TRY(launch_fill_uniform_u32(ctx, m->lm_exchange, decode_lm_head_words(ctx), 0, 0, 1));
    m->attn_launches.assign(z.L, 0);
    m->front_launches.assign(z.L, 0);
    m->layer_launches.assign(z.L, 0);
    m->lm_launches = 0;
    return MOON_OK;
}

struct ProfScope {
    moon_text_model *m;
    ProfScope(moon_text_model *model, int kind) : m(model) {
        if (!m->prof) return;
        StepProfiler &p = *m->prof;
        const size_t i = p.kinds.size();
        while (p.events.size() < 2 * (i + 1)) {
            hipEvent_t e;
            if (hipEventCreate(&e) != hipSuccess) { m = nullptr; return; }
            p.events.push_back(e);
        }
        p.kinds.push_back(kind);
        (void)hipEventRecord(p.events[2 * i], m->ctx->stream);
    }
    ~ProfScope() {
        if (m && m->prof) (void)hipEventRecord(m->prof->events[2 * m->prof->kinds.size() - 1], m->ctx->stream);
    }
};

// one decoder layer on n rows of m->hidden appended at position pos (text_model.zig:150-172)
// token_dev: (decode only) the layer input is row token_dev[0] of the embedding table instead of m->hidden
// chain_ln (rows of a prompt only): the LayerNorm of this layer's input is already in m->ln_in unless this is the first layer,
// and unless this is the last layer the fc2 product finishes the block itself: its split-K reduction adds the bias, the
// attention branch (reducing out_proj's split K on the way) and the residual and normalises the new rows with the next
// layer's LayerNorm (one launch instead of five; launch_gemm falls back to the separate launches, same arithmetic, where a
// product takes no split K).
int layer_forward(moon_text_model *m, size_t layer, size_t n, size_t pos, bool pos_on_device, const uint32_t *token_dev = nullptr,
                  bool chain_ln = false) {
    moon_ctx *ctx = m->ctx;
    const Sizes z = sizes(m->cfg);
    const half_t *ln_w = m->ln_w + layer * z.d, *ln_b = m->ln_b + layer * z.d;
    const half_t *qkv_w = m->qkv_w + layer * 3 * z.d * z.d, *qkv_b = m->qkv_b + layer * 3 * z.d;
    const half_t *out_w = m->out_w + layer * z.d * z.d, *out_b = m->out_b + layer * z.d;
    const half_t *fc1_w = m->fc1_w + layer * z.ffn * z.d, *fc1_b = m->fc1_b + layer * z.ffn;
    const half_t *fc2_w = m->fc2_w + layer * z.d * z.ffn, *fc2_b = m->fc2_b + layer * z.d;
    half_t *ck = m->cache_k + layer * z.H * z.S * z.D, *cv = m->cache_v + layer * z.H * z.S * z.D;

    if (n == 1 && m->fused) {
        // three kernels: LN + qkv + fc1;  rope + append + attention (+ merge);  out_proj + fc2 + both residual adds
        const half_t *x = token_dev ? m->wte : m->hidden;
        const int mode = m->decode_mode;
        if (m->whole_layer && mode == 0) {
            // one kernel for the layer
            const uint32_t head_target = ++m->attn_launches[layer] * 8u;
            const uint32_t generation = ++m->layer_launches[layer];
            ProfScope scope(m, PROF_LN_GEMV);
            return launch_decode_layer(ctx, x, token_dev, ln_w, ln_b, m->cfg.ln_eps, z.d, qkv_w, qkv_b, m->qkv, fc1_w, fc1_b, m->fc1, z.ffn, out_w,
                                       out_b, fc2_w, fc2_b, m->hidden, x, ck, cv, m->freqs, m->attn_partial, m->attn, m->head_count + layer * z.H,
                                       head_target, m->layer_sync + layer * m->layer_sync_words, generation,
                                       m->layer_sync + z.L * m->layer_sync_words, z.H, m->cfg.rot_dim, z.S, pos,
                                       pos_on_device ? m->state_dev : nullptr, m->layer_trace);
        }
        if (m->front && (mode == 0 || mode == 3)) {
            // two kernels: LN + qkv + fc1 with the attention hidden under the fc1 stream;  out_proj + fc2 + residual adds
            const uint32_t head_target = ++m->attn_launches[layer] * 8u;
            const uint32_t qkv_target = ++m->front_launches[layer] * (uint32_t)(3 * z.D);
            {
                ProfScope scope(m, PROF_LN_GEMV);
                MOON_TRY(launch_decode_front(ctx, x, token_dev, ln_w, ln_b, m->cfg.ln_eps, z.d, qkv_w, qkv_b, m->qkv, fc1_w, fc1_b, m->fc1, z.ffn,
                                             ck, cv, m->freqs, m->attn_partial, m->attn, m->head_count + layer * z.H, head_target,
                                             m->front_sync + layer * z.H * 32, qkv_target, m->front_sync + z.L * z.H * 32, z.H, m->cfg.rot_dim, z.S, pos,
                                             pos_on_device ? m->state_dev : nullptr));
            }
            ProfScope scope(m, PROF_OUT_FC2);
            return launch_decode_out_fc2(ctx, m->attn, m->fc1, out_w, out_b, fc2_w, fc2_b, m->hidden, x, token_dev, z.d, z.ffn);
        }
        {
            ProfScope scope(m, PROF_LN_GEMV);
            MOON_TRY(launch_decode_ln_gemv(ctx, x, token_dev, ln_w, ln_b, m->cfg.ln_eps, z.d, qkv_w, qkv_b, m->qkv, 3 * z.d, fc1_w, fc1_b,
                                           m->fc1, z.ffn));
        }
        const uint32_t target = ++m->attn_launches[layer] * 8u;
        {
            ProfScope scope(m, PROF_ATTN);
            MOON_TRY(launch_decode_attention_merged(ctx, m->qkv, ck, cv, m->freqs, m->attn_partial, m->attn, m->head_count + layer * z.H,
                                                    target, z.H, z.D, m->cfg.rot_dim, z.S, pos, pos_on_device ? m->state_dev : nullptr));
        }
        ProfScope scope(m, PROF_OUT_FC2);
        return launch_decode_out_fc2(ctx, m->attn, m->fc1, out_w, out_b, fc2_w, fc2_b, m->hidden, x, token_dev, z.d, z.ffn);
    }
    if (token_dev) MOON_TRY(launch_embed(ctx, m->wte, token_dev, m->hidden, 1, z.d));
    if (!chain_ln || layer == 0) MOON_TRY(launch_layernorm(ctx, m->hidden, ln_w, ln_b, m->ln_in, n, z.d, m->cfg.ln_eps));
    if (n == 1) {
        MOON_TRY(launch_gemv_nt(ctx, m->ln_in, qkv_w, qkv_b, m->qkv, 3 * z.d, z.d, MOON_EPI_BIAS));
        MOON_TRY(launch_decode_attention(ctx, m->qkv, ck, cv, m->freqs, m->attn, z.H, z.D, m->cfg.rot_dim, z.S, pos,
                                         pos_on_device ? m->state_dev : nullptr));
        MOON_TRY(launch_gemv_nt(ctx, m->attn, out_w, out_b, m->attn_proj, z.d, z.d, MOON_EPI_BIAS));
        MOON_TRY(launch_gemv_nt(ctx, m->ln_in, fc1_w, fc1_b, m->fc1, z.ffn, z.d, MOON_EPI_BIAS_GELU));
        MOON_TRY(launch_gemv_nt(ctx, m->fc1, fc2_w, fc2_b, m->mlp, z.d, z.ffn, MOON_EPI_BIAS));
    } else {
        bool roped = false; // the projection with the rotation and the cache update in its epilogue, where the shape has that form
        MOON_TRY(launch_gemm_qkv_rope(ctx, m->ln_in, qkv_w, qkv_b, n, z.d, m->q_rot, ck, cv, m->freqs, z.H, z.D, m->cfg.rot_dim, z.S, pos, &roped));
        if (!roped) {
            MOON_TRY(launch_gemm(ctx, m->ln_in, qkv_w, qkv_b, m->qkv, n, 3 * z.d, z.d, MOON_B_NK, MOON_EPI_BIAS));
            MOON_TRY(launch_qkv_rope_cache(ctx, m->qkv, m->q_rot, ck, cv, m->freqs, n, z.H, z.D, m->cfg.rot_dim, z.S, pos));
        }
        MOON_TRY(launch_sdpa(ctx, m->q_rot, ck, cv, m->attn, z.H, n, pos + n, z.D, z.S * z.D, (long)pos, nullptr, 0, true));
        const bool finish_in_fc2 = chain_ln;
        if (finish_in_fc2) {
            // out_proj and fc2 as one launch (each alone leaves a quarter of the device idle at 768 rows), finished together
            // with the LayerNorm that comes next: the next block's, or after the last block the model's final one (which the
            // LM head applies to the one row it needs by itself; here it only keeps the last block on the same launches)
            MOON_TRY(launch_gemm(ctx, m->ln_in, fc1_w, fc1_b, m->fc1, n, z.ffn, z.d, MOON_B_NK, MOON_EPI_BIAS_GELU));
            const bool last = layer + 1 == z.L;
            GemmLayerNorm next{last ? m->lno_w : m->ln_w + (layer + 1) * z.d, last ? m->lno_b : m->ln_b + (layer + 1) * z.d, m->ln_in, m->cfg.ln_eps};
            next.add = m->attn_proj;
            next.add_scratch = m->mlp;
            bool done = false;
            MOON_TRY(launch_gemm_pair_ln(ctx, m->attn, out_w, out_b, z.d, m->fc1, fc2_w, fc2_b, z.ffn, m->hidden, m->hidden, n, z.d, next, &done));
            if (done) return MOON_OK;
            // (otherwise the products one by one; fc1 is in place already)
            const float *out_partial = nullptr;
            int out_splits = 0;
            MOON_TRY(launch_gemm_partials(ctx, m->attn, out_w, n, z.d, z.d, MOON_B_NK, &out_partial, &out_splits));
            if (!out_splits) MOON_TRY(launch_gemm(ctx, m->attn, out_w, out_b, m->attn_proj, n, z.d, z.d, MOON_B_NK, MOON_EPI_BIAS));
            else {
                next.add_partial = out_partial;
                next.add_splits = out_splits;
                next.add_bias = out_b;
            }
            return launch_gemm(ctx, m->fc1, fc2_w, fc2_b, m->hidden, n, z.d, z.ffn, MOON_B_NK, 3 /* bias, then += into hidden */, m->hidden, &next);
        }
        MOON_TRY(launch_gemm(ctx, m->attn, out_w, out_b, m->attn_proj, n, z.d, z.d, MOON_B_NK, MOON_EPI_BIAS));
        MOON_TRY(launch_gemm(ctx, m->ln_in, fc1_w, fc1_b, m->fc1, n, z.ffn, z.d, MOON_B_NK, MOON_EPI_BIAS_GELU));
        MOON_TRY(launch_gemm(ctx, m->fc1, fc2_w, fc2_b, m->mlp, n, z.d, z.ffn, MOON_B_NK, MOON_EPI_BIAS));
    }
    return launch_residual2(ctx, m->hidden, m->attn_proj, m->mlp, n * z.d);
}

// lm_head on row `row` of hidden (text_model.zig:325-345)
int lm_head(moon_text_model *m, size_t row) {
    const Sizes z = sizes(m->cfg);
    ProfScope scope(m, PROF_LM_HEAD);
    if (m->fused)
        return launch_decode_ln_gemv(m->ctx, m->hidden + row * z.d, nullptr, m->lno_w, m->lno_b, m->cfg.ln_eps, z.d, m->lin_w, m->lin_b,
                                     m->logits, z.V, nullptr, nullptr, nullptr, 0);
    MOON_TRY(launch_layernorm(m->ctx, m->hidden + row * z.d, m->lno_w, m->lno_b, m->ln_last, 1, z.d, m->cfg.ln_eps));
    return launch_gemv_nt(m->ctx, m->ln_last, m->lin_w, m->lin_b, m->logits, z.V, z.d, MOON_EPI_BIAS);
}

} // namespace

extern "C" void moon_text_config_default(moon_text_config *cfg) {
    if (!cfg) return;
    cfg->vocab = 51200;
    cfg->dim = 2048;
    cfg->hidden_dim = 8192;
    cfg->n_layers = 24;
    cfg->n_heads = 32;
    cfg->head_dim = 64;
    cfg->rot_dim = 32; // head_dim * partial_rotary_factor (config.zig:12, text_model.zig:185)
    cfg->max_seq = 2048;
    cfg->rope_theta = 10000.0f;
    cfg->ln_eps = 1.00135803e-5f; // 1e-5 rounded to f16, as layerNorm(f16, ..., eps) receives it (text_model.zig:28,154-160)
}

extern "C" int moon_text_model_create(moon_ctx *ctx, const moon_text_config *cfg, const moon_text_weights *w, moon_text_model **out) {
    if (!ctx || !out) return MOON_EINVAL;
    std::lock_guard<std::mutex> lock(ctx->mu);
    *out = nullptr;
    MOON_TRY(check_cfg(ctx, cfg));
    if (!w) return moon_fail(ctx, MOON_EINVAL, "text model: null weights");
    const void *ptrs[] = {w->word_token_embedding, w->t_ln_w, w->t_ln_b, w->t_Wqkv_w, w->t_Wqkv_b, w->t_out_proj_w, w->t_out_proj_b,
                          w->t_fc1_w, w->t_fc1_b, w->t_fc2_w, w->t_fc2_b, w->t_linear_w, w->t_linear_b, w->t_ln_out_w, w->t_ln_out_b};
    for (const void *p : ptrs)
        if (!p) return moon_fail(ctx, MOON_EINVAL, "text model: a weight pointer is null");
    MOON_HIP(ctx, hipSetDevice(ctx->device));
    moon_text_model *m = new moon_text_model();
    m->ctx = ctx;
    m->cfg = *cfg;
    int rc = alloc_all(m);
    const Sizes z = sizes(m->cfg);
    auto up = [&](half_t *dst, const moon_f16 *src, size_t n) {
        if (rc != MOON_OK) return;
        hipError_t e = hipMemcpyAsync(dst, src, n * sizeof(moon_f16), hipMemcpyHostToDevice, ctx->stream);
        if (e != hipSuccess) rc = moon_fail(ctx, MOON_EHIP, "weight upload: %s", hipGetErrorString(e));
    };
    up(m->wte, w->word_token_embedding, z.V * z.d);
    up(m->ln_w, w->t_ln_w, z.L * z.d);
    up(m->ln_b, w->t_ln_b, z.L * z.d);
    up(m->qkv_w, w->t_Wqkv_w, z.L * 3 * z.d * z.d);
    up(m->qkv_b, w->t_Wqkv_b, z.L * 3 * z.d);
    up(m->out_w, w->t_out_proj_w, z.L * z.d * z.d);
    up(m->out_b, w->t_out_proj_b, z.L * z.d);
    up(m->fc1_w, w->t_fc1_w, z.L * z.ffn * z.d);
    up(m->fc1_b, w->t_fc1_b, z.L * z.ffn);
    up(m->fc2_w, w->t_fc2_w, z.L * z.d * z.ffn);
    up(m->fc2_b, w->t_fc2_b, z.L * z.d);
    up(m->lin_w, w->t_linear_w, z.V * z.d);
    up(m->lin_b, w->t_linear_b, z.V);
    up(m->lno_w, w->t_ln_out_w, z.d);
    up(m->lno_b, w->t_ln_out_b, z.d);
    if (rc == MOON_OK) {
        hipError_t e = hipStreamSynchronize(ctx->stream);
        if (e != hipSuccess) rc = moon_fail(ctx, MOON_EHIP, "weight upload sync: %s", hipGetErrorString(e));
    }
    if (rc != MOON_OK) {
        free_all(m);
        delete m;
        return rc;
    }
    *out = m;
    return MOON_OK;
}

extern "C" int moon_text_model_create_synthetic(moon_ctx *ctx, const moon_text_config *cfg, uint64_t seed, float std_dev,
                                                moon_text_model **out) {
    if (!ctx || !out) return MOON_EINVAL;
    std::lock_guard<std::mutex> lock(ctx->mu);
    *out = nullptr;
    MOON_TRY(check_cfg(ctx, cfg));
    MOON_HIP(ctx, hipSetDevice(ctx->device));
    moon_text_model *m = new moon_text_model();
    m->ctx = ctx;
    m->cfg = *cfg;
    int rc = alloc_all(m);
    const Sizes z = sizes(m->cfg);
    // stream numbers = declaration order of moon_text_weights
    auto rnd = [&](half_t *dst, size_t n, uint64_t stream) {
        if (rc == MOON_OK) rc = launch_fill_normal(ctx, dst, n, seed, stream, std_dev);
    };
    auto cst = [&](half_t *dst, size_t n, float v) {
        if (rc == MOON_OK) rc = launch_fill_const(ctx, dst, n, v);
    };
    rnd(m->wte, z.V * z.d, 0);
    cst(m->ln_w, z.L * z.d, 1.0f);
    cst(m->ln_b, z.L * z.d, 0.0f);
    rnd(m->qkv_w, z.L * 3 * z.d * z.d, 3);
    rnd(m->qkv_b, z.L * 3 * z.d, 4);
    rnd(m->out_w, z.L * z.d * z.d, 5);
    rnd(m->out_b, z.L * z.d, 6);
    rnd(m->fc1_w, z.L * z.ffn * z.d, 7);
    rnd(m->fc1_b, z.L * z.ffn, 8);
    rnd(m->fc2_w, z.L * z.d * z.ffn, 9);
    rnd(m->fc2_b, z.L * z.d, 10);
    rnd(m->lin_w, z.V * z.d, 11);
    rnd(m->lin_b, z.V, 12);
    cst(m->lno_w, z.d, 1.0f);
    cst(m->lno_b, z.d, 0.0f);
    if (rc == MOON_OK) {
        hipError_t e = hipStreamSynchronize(ctx->stream);
        if (e != hipSuccess) rc = moon_fail(ctx, MOON_EHIP, "synthetic weights: %s", hipGetErrorString(e));
    }
    if (rc != MOON_OK) {
        free_all(m);
        delete m;
        return rc;
    }
    *out = m;
    return MOON_OK;
}

extern "C" void moon_text_model_destroy(moon_text_model *m) {
    if (!m) return;
    {
        std::lock_guard<std::mutex> lock(m->ctx->mu);
        free_all(m);
    }
    delete m;
}

extern "C" int moon_text_reset(moon_text_model *m) {
    if (!m) return MOON_EINVAL;
    std::lock_guard<std::mutex> lock(m->ctx->mu);
    m->cur_len = 0;
    m->last_n = 0;
    MOON_HIP(m->ctx, hipSetDevice(m->ctx->device));
    if (m->cache_invalid) MOON_TRY(clear_sync_state(m)); // after a failed wait: counters and targets start over together
    m->cache_invalid = false;
    hipLaunchKernelGGL(set_state_kernel, dim3(1), dim3(1), 0, m->ctx->stream, m->state_dev, 0u, 0u);
    MOON_HIP(m->ctx, hipGetLastError());
    return MOON_OK;
}

extern "C" size_t moon_text_position(const moon_text_model *m) { return m ? m->cur_len : 0; }

// n rows already in m->hidden: the layers, the bookkeeping and, for a single row, the fused kernels' error words
static int forward_rows_locked(moon_text_model *m, size_t n_ids) {
    moon_ctx *ctx = m->ctx;
    for (size_t l = 0; l < m->cfg.n_layers; l++) MOON_TRY(layer_forward(m, l, n_ids, m->cur_len, false, nullptr, n_ids > 1));
    m->cur_len += n_ids;
    m->last_n = n_ids;
    hipLaunchKernelGGL(set_state_kernel, dim3(1), dim3(1), 0, ctx->stream, m->state_dev, (uint32_t)m->cur_len, 0u);
    MOON_HIP(ctx, hipGetLastError());
    // a single token takes the fused decode kernels, whose waits between workgroups are bounded: look at their error words
    volatile uint32_t *wait_error = m->host_words; // (page-locked: the copies are queued like the kernels, one synchronisation for all)
    wait_error[0] = wait_error[1] = 0;
    if (n_ids == 1 && m->fused) {
        MOON_HIP(ctx, hipMemcpyAsync(m->host_words, m->layer_sync + m->cfg.n_layers * m->layer_sync_words, sizeof(uint32_t), hipMemcpyDeviceToHost,
                                     ctx->stream));
        MOON_HIP(ctx, hipMemcpyAsync(m->host_words + 1, m->front_sync + m->cfg.n_layers * m->cfg.n_heads * 32, sizeof(uint32_t), hipMemcpyDeviceToHost,
                                     ctx->stream));
    }
    MOON_HIP(ctx, hipStreamSynchronize(ctx->stream));
    if (wait_error[0] || wait_error[1]) { // as in the generation loop: the token's cache row may be missing
        m->cur_len -= n_ids;
        m->cache_invalid = true;
        m->last_n = 0;
        (void)clear_sync_state(m);
        return moon_fail(ctx, MOON_EHIP, "fused decode kernel: a wait between its phases timed out; the session needs moon_text_reset");
    }
    return MOON_OK;
}

extern "C" int moon_text_forward(moon_text_model *m, const uint32_t *ids, size_t n_ids) {
    if (!m) return MOON_EINVAL;
    moon_ctx *ctx = m->ctx;
    std::lock_guard<std::mutex> lock(ctx->mu);
    if (!ids && n_ids) return moon_fail(ctx, MOON_EINVAL, "text_forward: null ids");
    if (!n_ids) return moon_fail(ctx, MOON_EINVAL_DIM, "text_forward: empty input (InvalidInputShape)");
    if (m->cache_invalid) return moon_fail(ctx, MOON_EHIP, "text_forward: an earlier decode call failed; call moon_text_reset first");
    if (m->cur_len + n_ids > m->cfg.max_seq)
        return moon_fail(ctx, MOON_ESEQ_TOO_LONG, "text_forward: %zu + %zu tokens > max_seq %zu (SequenceTooLong)", m->cur_len, n_ids, m->cfg.max_seq);
    for (size_t i = 0; i < n_ids; i++)
        if (ids[i] >= m->cfg.vocab) return moon_fail(ctx, MOON_ETOKEN, "text_forward: token id %u >= vocab %zu (TokenIdOutOfBounds)", ids[i], m->cfg.vocab);
    MOON_HIP(ctx, hipSetDevice(ctx->device));
    memcpy(m->ids_pinned, ids, n_ids * sizeof(uint32_t)); // (every call ends with the stream drained: the buffer is free)
    MOON_HIP(ctx, hipMemcpyAsync(m->ids_dev, m->ids_pinned, n_ids * sizeof(uint32_t), hipMemcpyHostToDevice, ctx->stream));
    MOON_TRY(launch_embed(ctx, m->wte, m->ids_dev, m->hidden, n_ids, m->cfg.dim));
    return forward_rows_locked(m, n_ids);
}

extern "C" int moon_text_forward_embeds(moon_text_model *m, const moon_f16 *embeds, size_t n_rows) {
    if (!m) return MOON_EINVAL;
    moon_ctx *ctx = m->ctx;
    std::lock_guard<std::mutex> lock(ctx->mu);
    if (!embeds && n_rows) return moon_fail(ctx, MOON_EINVAL, "text_forward_embeds: null input");
    if (!n_rows) return moon_fail(ctx, MOON_EINVAL_DIM, "text_forward_embeds: empty input (InvalidInputShape)");
    if (m->cache_invalid) return moon_fail(ctx, MOON_EHIP, "text_forward_embeds: an earlier decode call failed; call moon_text_reset first");
    if (m->cur_len + n_rows > m->cfg.max_seq)
        return moon_fail(ctx, MOON_ESEQ_TOO_LONG, "text_forward_embeds: %zu + %zu rows > max_seq %zu (SequenceTooLong)", m->cur_len, n_rows, m->cfg.max_seq);
    MOON_HIP(ctx, hipSetDevice(ctx->device));
    MOON_TRY(copy_up(m, m->hidden, embeds, n_rows * m->cfg.dim * sizeof(moon_f16)));
    return forward_rows_locked(m, n_rows);
}

extern "C" int moon_text_embed(moon_text_model *m, const uint32_t *ids, size_t n_ids, moon_f16 *embeds) {
    if (!m) return MOON_EINVAL;
    moon_ctx *ctx = m->ctx;
    std::lock_guard<std::mutex> lock(ctx->mu);
    if ((!ids || !embeds) && n_ids) return moon_fail(ctx, MOON_EINVAL, "text_embed: null argument");
    if (n_ids > m->cfg.max_seq) return moon_fail(ctx, MOON_ESEQ_TOO_LONG, "text_embed: %zu ids > seq_len %zu (SequenceTooLong)", n_ids, m->cfg.max_seq);
    for (size_t i = 0; i < n_ids; i++)
        if (ids[i] >= m->cfg.vocab) return moon_fail(ctx, MOON_ETOKEN, "text_embed: token id %u >= vocab %zu (TokenIdOutOfBounds)", ids[i], m->cfg.vocab);
    if (!n_ids) return MOON_OK;
    MOON_HIP(ctx, hipSetDevice(ctx->device));
    // through buffers the session's state does not live in: the ids behind the loop's random numbers, the rows in the
    // MLP scratch (both are rewritten by whatever call uses them next)
    uint32_t *ids_tmp = reinterpret_cast<uint32_t *>(m->u_dev);
    MOON_TRY(copy_up(m, ids_tmp, ids, n_ids * sizeof(uint32_t)));
    MOON_TRY(launch_embed(ctx, m->wte, ids_tmp, m->mlp, n_ids, m->cfg.dim));
    return copy_down_sync(m, embeds, m->mlp, n_ids * m->cfg.dim * sizeof(moon_f16));
}

extern "C" int moon_text_logits(moon_text_model *m, moon_f16 *logits) {
    if (!m) return MOON_EINVAL;
    moon_ctx *ctx = m->ctx;
    std::lock_guard<std::mutex> lock(ctx->mu);
    if (!logits) return moon_fail(ctx, MOON_EINVAL, "text_logits: null output");
    if (!m->last_n) return moon_fail(ctx, MOON_EINVAL, "text_logits: no forward pass yet");
    MOON_HIP(ctx, hipSetDevice(ctx->device));
    MOON_TRY(lm_head(m, m->last_n - 1));
    return copy_down_sync(m, logits, m->logits, m->cfg.vocab * sizeof(moon_f16));
}

extern "C" int moon_text_hidden(moon_text_model *m, moon_f16 *hidden, size_t n_rows) {
    if (!m) return MOON_EINVAL;
    moon_ctx *ctx = m->ctx;
    std::lock_guard<std::mutex> lock(ctx->mu);
    if (!hidden) return moon_fail(ctx, MOON_EINVAL, "text_hidden: null output");
    if (n_rows > m->last_n) return moon_fail(ctx, MOON_EINVAL_DIM, "text_hidden: %zu rows requested, last forward had %zu", n_rows, m->last_n);
    return copy_down_sync(m, hidden, m->hidden, n_rows * m->cfg.dim * sizeof(moon_f16));
}

// MOON_DECODE_TRACE: where the workgroups of the last whole-layer launch spent their time, by role (microseconds after
// the first workgroup started; mean and latest over the role's workgroups)
static void print_layer_trace(moon_text_model *m) {
    const Sizes z = sizes(m->cfg);
    const int cus = m->ctx->cu_count > 0 ? m->ctx->cu_count : 256;
    const size_t grid = size_t(4) * cus, n_attn = z.H * 8, n_out = (z.d + 3) / 4;
    if (grid > 4096) return;
    std::vector<long long> t(grid * 8);
    if (hipMemcpy(t.data(), m->layer_trace, t.size() * sizeof(long long), hipMemcpyDeviceToHost) != hipSuccess) return;
    long long t0 = t[0];
    for (size_t b = 0; b < grid; b++) t0 = std::min(t0, t[b * 8]);
    struct Role { const char *name; size_t lo, hi; int n; const char *stamps[6]; };
    const Role roles[3] = {{"attention", 0, n_attn, 4, {"start", "qkv rows reported", "head's q,k,v complete", "task done"}},
                           {"output", n_attn, n_attn + n_out, 6, {"start", "qkv rows reported", "fc1 rows reported", "all fc1 written", "all heads merged", "hidden written"}},
                           {"fc1 only", n_attn + n_out, grid, 3, {"start", "qkv rows reported", "fc1 rows reported"}}};
    fprintf(stderr, "[moonhip layer trace] last layer launch of the last step, %zu workgroups\n", grid);
    for (const Role &r : roles) {
        fprintf(stderr, "  %-9s (%4zu workgroups):", r.name, r.hi - r.lo);
        for (int i = 0; i < r.n; i++) {
            double sum = 0, mx = 0;
            for (size_t b = r.lo; b < r.hi; b++) {
                const double us = (double)(t[b * 8 + i] - t0) * 0.01;
                sum += us;
                mx = std::max(mx, us);
            }
            fprintf(stderr, "  %s %.1f/%.1f", r.stamps[i], sum / (double)(r.hi - r.lo), mx);
        }
        fprintf(stderr, "\n");
    }
}

// sampling == nullptr: greedy.  Otherwise sampling.sample with u[step] in place of the arg-max (the per-launch kernels only).
// eos_plus1 != 0: the loop ends when that token (id + 1) comes up; it is not recorded (moondream.zig:341).  *n_out (if set)
// receives the number of tokens recorded; with an end-of-sequence token set, the host looks at the device's state every
// EOS_CHUNK steps so that at most that many steps are queued behind the stop.
constexpr size_t EOS_CHUNK = 8;
static int greedy_locked(moon_text_model *m, size_t n_steps, uint32_t *out_ids, const moon_sampling_config *sampling = nullptr,
                         const float *u = nullptr, uint32_t eos_plus1 = 0, size_t *n_out = nullptr) {
    moon_ctx *ctx = m->ctx;
    if (!out_ids && n_steps) return moon_fail(ctx, MOON_EINVAL, "text_greedy: null output");
    if (m->cache_invalid) return moon_fail(ctx, MOON_EHIP, "text_greedy: an earlier decode call failed; call moon_text_reset first");
    if (!m->last_n) return moon_fail(ctx, MOON_EINVAL, "text_greedy: no prefill yet");
    if (!n_steps) return MOON_OK;
    if (m->cur_len + n_steps > m->cfg.max_seq)
        return moon_fail(ctx, MOON_ESEQ_TOO_LONG, "text_greedy: %zu + %zu tokens > max_seq %zu (SequenceTooLong)", m->cur_len, n_steps, m->cfg.max_seq);
    MOON_HIP(ctx, hipSetDevice(ctx->device));
    if (sampling) MOON_TRY(copy_up(m, m->u_dev, u, n_steps * sizeof(float)));
    uint32_t *state = m->state_dev;
    hipLaunchKernelGGL(start_loop_kernel, dim3(1), dim3(1), 0, ctx->stream, state, (uint32_t)m->cur_len, eos_plus1);
    MOON_HIP(ctx, hipGetLastError());
    if (n_out) *n_out = 0;
    const int mode = m->decode_mode;
    const bool use_layer = m->whole_layer && mode == 0;
    if (use_layer) { // counters count up for the life of the model: clear them long before 32 bits are used up (192 per launch)
        const Sizes z = sizes(m->cfg);
        if ((uint64_t(m->layer_launches[0]) + n_steps + 1) * 192ull > 0x7fffffffull) {
            MOON_TRY(launch_fill_uniform_u32(ctx, m->layer_sync, z.L * m->layer_sync_words, 0, 0, 1));
            m->layer_launches.assign(z.L, 0);
        }
    }
    const bool use_front = !use_layer && m->front && (mode == 0 || mode == 3);
    if (use_front) { // the row counters count up for the life of the model: clear them long before 32 bits are used up
        const Sizes z = sizes(m->cfg);
        const uint64_t per_launch = 3 * z.D;
        if ((uint64_t(m->front_launches[0]) + n_steps + 1) * per_launch > 0x7fffffffull) {
            MOON_TRY(launch_fill_uniform_u32(ctx, m->front_sync, z.L * z.H * 32, 0, 0, 1));
            m->front_launches.assign(z.L, 0);
        }
    }
    size_t row = m->last_n - 1;
    const bool lm_argmax = m->fused && !sampling; // LM head, arg-max and the loop's bookkeeping in one launch
    // top_k with a few candidates: the LM-head launch decides the token wherever that is provably the reference's choice and
    // says so in state[6]; sample_kernel behind it then has nothing to do
    const bool lm_topk = m->fused && sampling && sampling->method == MOON_SAMPLE_TOP_K && !getenv("MOON_SAMPLE_SEPARATE") &&
                         decode_lm_head_top_k_supported(ctx, std::min(sampling->top_k, m->cfg.vocab), m->cfg.vocab);
    if ((lm_argmax || lm_topk) && (uint64_t(m->lm_launches) + n_steps + 1) * 4096ull > 0x7fffffffull) { // its counter counts up for the life of the model
        MOON_TRY(launch_fill_uniform_u32(ctx, m->lm_exchange, decode_lm_head_words(ctx), 0, 0, 1));
        m->lm_launches = 0;
    }
    for (size_t step = 0; step < n_steps; step++) {
        if (lm_argmax) {
            const Sizes z = sizes(m->cfg);
            ProfScope scope(m, PROF_LM_HEAD);
            // token -> state[2], ids[state[1]++]; the position moves on here for every step but the first
            MOON_TRY(launch_decode_lm_head(ctx, m->hidden + row * z.d, m->lno_w, m->lno_b, m->cfg.ln_eps, z.d, m->lin_w, m->lin_b, m->logits, z.V,
                                           m->lm_exchange, ++m->lm_launches, state, m->ids_dev, step > 0 ? 1u : 0u));
        } else if (lm_topk) {
            const Sizes z = sizes(m->cfg);
            {
                ProfScope scope(m, PROF_LM_HEAD);
                MOON_TRY(launch_decode_lm_head(ctx, m->hidden + row * z.d, m->lno_w, m->lno_b, m->cfg.ln_eps, z.d, m->lin_w, m->lin_b, m->logits, z.V,
                                               m->lm_exchange, ++m->lm_launches, state, m->ids_dev, step > 0 ? 1u : 0u, sampling, m->u_dev, state + 6));
            }
            ProfScope scope(m, PROF_ARGMAX);
            MOON_TRY(launch_sample(ctx, m->logits, m->cfg.vocab, sampling, 0.f, m->u_dev, state, m->ids_dev, nullptr, step > 0 ? 1u : 0u, nullptr,
                                   state + 6));
        } else {
            MOON_TRY(lm_head(m, row));
            ProfScope scope(m, PROF_ARGMAX);
            if (sampling) // u_dev[state[1]] decides; token -> state[2], ids[state[1]++]; the position moves on for every step but the first
                MOON_TRY(launch_sample(ctx, m->logits, m->cfg.vocab, sampling, 0.f, m->u_dev, state, m->ids_dev, nullptr, step > 0 ? 1u : 0u));
            else
                MOON_TRY(launch_argmax_record(ctx, m->logits, m->cfg.vocab, state, m->ids_dev)); // token -> state[2], ids[state[1]++]
        }
        for (size_t l = 0; l < m->cfg.n_layers; l++) MOON_TRY(layer_forward(m, l, 1, m->cur_len + step, true, l == 0 ? state + 2 : nullptr));
        if (!lm_argmax && !sampling) {
            ProfScope scope(m, PROF_BUMP);
            hipLaunchKernelGGL(bump_pos_kernel, dim3(1), dim3(1), 0, ctx->stream, state);
            MOON_HIP(ctx, hipGetLastError());
        }
        row = 0;
        if (m->prof) { // read this step's event pairs back before they are reused
            StepProfiler &p = *m->prof;
            MOON_HIP(ctx, hipStreamSynchronize(ctx->stream));
            for (size_t i = 0; i < p.kinds.size(); i++) {
                float ms = 0.f;
                MOON_HIP(ctx, hipEventElapsedTime(&ms, p.events[2 * i], p.events[2 * i + 1]));
                p.sum_ms[p.kinds[i]] += ms;
                p.count[p.kinds[i]]++;
            }
            p.kinds.clear();
        }
        if (eos_plus1 && (step + 1) % EOS_CHUNK == 0 && step + 1 < n_steps) { // has the end-of-sequence token come up?
            volatile uint32_t *st = m->host_words + 16;
            MOON_HIP(ctx, hipMemcpyAsync(m->host_words + 16, state, 4 * sizeof(uint32_t), hipMemcpyDeviceToHost, ctx->stream));
            MOON_HIP(ctx, hipStreamSynchronize(ctx->stream));
            if (st[3]) break;
        }
    }
    // everything the call brings back lands in page-locked memory (queued like the kernels), one synchronisation for all of it
    volatile uint32_t *words = m->host_words;
    words[20] = 0; words[21] = (uint32_t)n_steps; words[22] = 0; words[23] = 0; // the loop's final state where no copy is asked for
    words[24] = 0;                                                            // the error word
    if (eos_plus1) MOON_HIP(ctx, hipMemcpyAsync(m->host_words + 20, state, 4 * sizeof(uint32_t), hipMemcpyDeviceToHost, ctx->stream));
    const bool ids_staged = n_steps * sizeof(uint32_t) <= STAGE_BYTES;
    MOON_HIP(ctx, hipMemcpyAsync(ids_staged ? (void *)m->stage_down : (void *)out_ids, m->ids_dev, n_steps * sizeof(uint32_t), hipMemcpyDeviceToHost, ctx->stream));
    if (use_layer)
        MOON_HIP(ctx, hipMemcpyAsync(m->host_words + 24, m->layer_sync + m->cfg.n_layers * m->layer_sync_words, sizeof(uint32_t), hipMemcpyDeviceToHost,
                                     ctx->stream));
    if (use_front)
        MOON_HIP(ctx, hipMemcpyAsync(m->host_words + 24, m->front_sync + m->cfg.n_layers * m->cfg.n_heads * 32, sizeof(uint32_t), hipMemcpyDeviceToHost, ctx->stream));
    MOON_HIP(ctx, hipStreamSynchronize(ctx->stream));
    if (ids_staged) memcpy(out_ids, m->stage_down, n_steps * sizeof(uint32_t));
    const uint32_t front_error = words[24];
    const uint32_t final_state[4] = {words[20], words[21], words[22], words[23]};
    if (front_error != 0) {
        // Workgroups that gave up skipped their counter updates and the cache append of their position: the counters
        // are cleared here, the cache and the position stay unusable until moon_text_reset.
        m->cache_invalid = true;
        m->last_n = 0;
        (void)clear_sync_state(m);
        return moon_fail(ctx, MOON_EHIP, "fused decode kernel: a wait between its phases timed out; the session needs moon_text_reset");
    }
    // every recorded token went through the layers and sits in the cache; after a stop the launches queued behind it have
    // overwritten the hidden state and the logits, so the session then needs a forward pass before the next loop
    const size_t recorded = final_state[1];
    m->cur_len += recorded;
    m->last_n = final_state[3] ? 0 : 1;
    if (n_out) *n_out = recorded;
    if (use_layer && m->layer_trace) print_layer_trace(m);
    return MOON_OK;
}

extern "C" int moon_text_greedy(moon_text_model *m, size_t n_steps, uint32_t *out_ids) {
    if (!m) return MOON_EINVAL;
    std::lock_guard<std::mutex> lock(m->ctx->mu);
    return greedy_locked(m, n_steps, out_ids);
}

extern "C" int moon_text_sample(moon_text_model *m, const moon_sampling_config *cfg, const float *u, size_t n_steps, uint32_t *out_ids) {
    if (!m) return MOON_EINVAL;
    moon_ctx *ctx = m->ctx;
    std::lock_guard<std::mutex> lock(ctx->mu);
    if (!cfg) return moon_fail(ctx, MOON_EINVAL, "text_sample: null config");
    if (cfg->method == MOON_SAMPLE_GREEDY) return greedy_locked(m, n_steps, out_ids);
    if (!u && n_steps) return moon_fail(ctx, MOON_EINVAL, "text_sample: null random numbers");
    if (cfg->method < MOON_SAMPLE_MULTINOMIAL || cfg->method > MOON_SAMPLE_MIN_P)
        return moon_fail(ctx, MOON_EINVAL, "text_sample: unknown method %d", cfg->method);
    // the checks launch_sample makes at every step, before anything runs
    if (cfg->temperature != 1.0f && !(cfg->temperature > 0.f))
        return moon_fail(ctx, MOON_ETEMPERATURE, "text_sample: temperature %g (InvalidTemperature)", (double)cfg->temperature);
    if (cfg->method == MOON_SAMPLE_TOP_K && (!cfg->top_k || std::min(cfg->top_k, m->cfg.vocab) > 1024))
        return moon_fail(ctx, MOON_EINVAL, "text_sample: top_k %zu (1 to 1024 candidates are sorted on the device)", cfg->top_k);
    return greedy_locked(m, n_steps, out_ids, cfg, u);
}

extern "C" int moon_text_generate(moon_text_model *m, const moon_sampling_config *cfg, const float *u, size_t max_tokens, uint32_t eos_token,
                                  uint32_t *out_ids, size_t *n_out) {
    if (!m) return MOON_EINVAL;
    moon_ctx *ctx = m->ctx;
    std::lock_guard<std::mutex> lock(ctx->mu);
    if (!n_out) return moon_fail(ctx, MOON_EINVAL, "text_generate: null count");
    *n_out = 0;
    if (eos_token >= m->cfg.vocab) return moon_fail(ctx, MOON_ETOKEN, "text_generate: end-of-sequence id %u >= vocab %zu", eos_token, m->cfg.vocab);
    // the reference stops at position 2048 (moondream.zig:324) instead of failing: so does this loop
    if (m->cur_len >= m->cfg.max_seq) return MOON_OK;
    max_tokens = std::min(max_tokens, m->cfg.max_seq - m->cur_len);
    const bool greedy = !cfg || cfg->method == MOON_SAMPLE_GREEDY;
    if (!greedy) {
        if (!u && max_tokens) return moon_fail(ctx, MOON_EINVAL, "text_generate: null random numbers");
        if (cfg->method < MOON_SAMPLE_MULTINOMIAL || cfg->method > MOON_SAMPLE_MIN_P)
            return moon_fail(ctx, MOON_EINVAL, "text_generate: unknown method %d", cfg->method);
        if (cfg->temperature != 1.0f && !(cfg->temperature > 0.f))
            return moon_fail(ctx, MOON_ETEMPERATURE, "text_generate: temperature %g (InvalidTemperature)", (double)cfg->temperature);
        if (cfg->method == MOON_SAMPLE_TOP_K && (!cfg->top_k || std::min(cfg->top_k, m->cfg.vocab) > 1024))
            return moon_fail(ctx, MOON_EINVAL, "text_generate: top_k %zu (1 to 1024 candidates are sorted on the device)", cfg->top_k);
    }
    return greedy_locked(m, max_tokens, out_ids, greedy ? nullptr : cfg, greedy ? nullptr : u, eos_token + 1u, n_out);
}

extern "C" int moon_text_next_token(moon_text_model *m, const moon_sampling_config *cfg, float u, uint32_t *token) {
    if (!m) return MOON_EINVAL;
    moon_ctx *ctx = m->ctx;
    std::lock_guard<std::mutex> lock(ctx->mu);
    if (!token) return moon_fail(ctx, MOON_EINVAL, "text_next_token: null output");
    if (!m->last_n) return moon_fail(ctx, MOON_EINVAL, "text_next_token: no forward pass yet");
    MOON_HIP(ctx, hipSetDevice(ctx->device));
    MOON_TRY(lm_head(m, m->last_n - 1));
    uint32_t *out = m->state_dev + 5; // a word of the loop's state that the loop itself does not use
    if (!cfg || cfg->method == MOON_SAMPLE_GREEDY) MOON_TRY(launch_argmax(ctx, m->logits, m->cfg.vocab, out));
    else MOON_TRY(launch_sample(ctx, m->logits, m->cfg.vocab, cfg, u, nullptr, nullptr, nullptr, out));
    MOON_HIP(ctx, hipMemcpyAsync(m->host_words + 8, out, sizeof(uint32_t), hipMemcpyDeviceToHost, ctx->stream));
    MOON_HIP(ctx, hipStreamSynchronize(ctx->stream));
    *token = const_cast<volatile uint32_t *>(m->host_words)[8];
    return MOON_OK;
}

extern "C" int moon_text_greedy_profile(moon_text_model *m, size_t n_steps, uint32_t *out_ids, float *avg_us, size_t *launches) {
    if (!m) return MOON_EINVAL;
    moon_ctx *ctx = m->ctx;
    std::lock_guard<std::mutex> lock(ctx->mu);
    if (!avg_us || !launches) return moon_fail(ctx, MOON_EINVAL, "text_greedy_profile: null output");
    if (!m->fused) return moon_fail(ctx, MOON_EINVAL, "text_greedy_profile: only the fused per-layer kernels can be timed per launch");
    StepProfiler prof;
    m->prof = &prof;
    const int rc = greedy_locked(m, n_steps, out_ids);
    m->prof = nullptr;
    for (hipEvent_t e : prof.events) (void)hipEventDestroy(e);
    if (rc != MOON_OK) return rc;
    for (int k = 0; k < PROF_KINDS; k++) {
        launches[k] = prof.count[k];
        avg_us[k] = prof.count[k] ? (float)(prof.sum_ms[k] * 1e3 / (double)prof.count[k]) : 0.f;
    }
    return MOON_OK;
}

// Raises the error word that the fused decode kernels' waits look at, as a kernel does when its wait expires.  For tests
// of the recovery path: every kernel still runs to its end, a workgroup that has to poll a counter for long leaves early.
extern "C" int moon_text_debug_raise_wait_error(moon_text_model *m) {
    if (!m) return MOON_EINVAL;
    moon_ctx *ctx = m->ctx;
    std::lock_guard<std::mutex> lock(ctx->mu);
    const Sizes z = sizes(m->cfg);
    MOON_HIP(ctx, hipSetDevice(ctx->device));
    // the word before each error word is unused (the tail of a counter line, or of the last counter copy): writes {0, 1} to (tail, error word)
    hipLaunchKernelGGL(set_state_kernel, dim3(1), dim3(1), 0, ctx->stream, m->layer_sync + z.L * m->layer_sync_words - 1, 0u, 1u);
    MOON_HIP(ctx, hipGetLastError());
    hipLaunchKernelGGL(set_state_kernel, dim3(1), dim3(1), 0, ctx->stream, m->front_sync + z.L * z.H * 32 - 1, 0u, 1u);
    MOON_HIP(ctx, hipGetLastError());
    return MOON_OK;
}

extern "C" int moon_text_set_decode_mode(moon_text_model *m, int mode) {
    if (!m) return MOON_EINVAL;
    std::lock_guard<std::mutex> lock(m->ctx->mu);
    if (mode != 0 && mode != 2 && mode != 3)
        return moon_fail(m->ctx, MOON_EINVAL, "decode mode must be 0 (one kernel per layer), 2 (three kernels per layer) or 3 (two kernels per layer)");
    m->decode_mode = mode;
    return MOON_OK;
}

extern "C" size_t moon_text_weight_bytes_per_token(const moon_text_model *m) {
    if (!m) return 0;
    const Sizes z = sizes(m->cfg);
    const size_t per_layer = 2 * z.d + 3 * z.d * z.d + 3 * z.d + z.d * z.d + z.d + z.ffn * z.d + z.ffn + z.d * z.ffn + z.d;
    return (z.L * per_layer + 2 * z.d + z.V * z.d + z.V) * sizeof(moon_f16);
}
