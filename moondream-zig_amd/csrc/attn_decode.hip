// Single-token causal attention over the KV cache with the rotary step and the cache append fused in --
// replaces rope.applyRotEmb on q,k (rope.zig:130-272), LayerCache.updateCache / getActiveCache
// (text_model.zig:436-515), createAttentionMask(pos,1) (attention.zig:256-281, all true) and
// attention.singleMaskedSDPA (attention.zig:564-642, 759-811) of one decode step.
//
// HBM bound: the step streams kv_len*D*2*2 bytes of K and V per head exactly once.  The key range is split
// over DEC_SPLITS workgroups per head (32 heads x 8 = 256 workgroups, one per CU); 8 lanes share a key (16 B
// each) so a wavefront load covers 8 consecutive keys = 1 KiB contiguous.  Each split produces an
// un-normalised partial (o, m, l) in f32; a second kernel merges the partials in a fixed order.
// The cache is read in place in the reference layout [n_heads][max_seq][head_dim]; no "active" copy is made.
#include "attn_decode.hpp"
#include <mutex>

namespace {

template <int D, bool FUSED>
__global__ __launch_bounds__(256) void decode_attn_partial_kernel(const half_t *__restrict__ qkv, half_t *__restrict__ ck,
                                                                   half_t *__restrict__ cv, const float *__restrict__ table,
                                                                   float *__restrict__ partial, int H, int rot_dim, int max_seq,
                                                                   int pos_arg, const uint32_t *__restrict__ pos_dev) {
    const int pos = pos_dev ? (int)*pos_dev : pos_arg;
    const int h = blockIdx.x / DEC_SPLITS, split = blockIdx.x % DEC_SPLITS;
    DecodeAttnPrefetch<> pf;
    decode_attn_prefetch<D>(pf, ck, cv, max_seq, pos, FUSED, h, split);
    decode_attn_task<D, FUSED>(qkv, ck, cv, table, partial, H, rot_dim, max_seq, pos, h, split, pf);
}

template <int D>
__global__ void decode_attn_merge_kernel(const float *__restrict__ partial, half_t *__restrict__ out) {
    const int h = blockIdx.x, d = threadIdx.x;
    out[h * D + d] = decode_attn_merge<D>(partial + size_t(h) * DEC_SPLITS * (D + 2), d);
}

} // namespace

int launch_decode_attention_merged(moon_ctx *ctx, const half_t *qkv, half_t *cache_k, half_t *cache_v, const float *table, float *partial,
                                   half_t *out, uint32_t *head_count, uint32_t count_target, size_t H, size_t D, size_t rot_dim,
                                   size_t max_seq, size_t pos, const uint32_t *pos_dev, size_t head_stride = 1);

int launch_decode_attention(moon_ctx *ctx, const half_t *qkv, half_t *cache_k, half_t *cache_v, const float *table, half_t *out,
                            size_t H, size_t D, size_t rot_dim, size_t max_seq, size_t pos, const uint32_t *pos_dev) {
    if (D != 64) return moon_fail(ctx, MOON_EINVAL_DIM, "decode attention: head_dim %zu unsupported (64 only)", D);
    if (rot_dim > D || rot_dim % 2) return moon_fail(ctx, MOON_EROT_DIM, "decode attention: bad rot_dim %zu", rot_dim);
    if (max_seq > 2048 || pos >= max_seq)
        return moon_fail(ctx, MOON_ESEQ_TOO_LONG, "decode attention: pos %zu >= max_seq %zu (limit 2048)", pos, max_seq);
    // One launch: the split that finishes a head last merges it (the kernel of the text session's three-kernel decode
    // mode).  Its per-head counters sit behind the partials and count up from launch to launch.
    const size_t partial_bytes = (H * DEC_SPLITS * (D + 2) * sizeof(float) + 255) & ~size_t(255);
    // (the heads' counters 4,352 bytes apart: all splits of all heads count in at about the same time, and atomics on one line
    // are served one after the other)
    constexpr size_t HEAD_STRIDE = 1088;
    MOON_TRY(moon_grow(ctx, ctx->work[1], partial_bytes + H * HEAD_STRIDE * sizeof(uint32_t)));
    float *partial = (float *)ctx->work[1].ptr;
    uint32_t *head_count = reinterpret_cast<uint32_t *>(reinterpret_cast<char *>(ctx->work[1].ptr) + partial_bytes);
    if (ctx->attn_cnt_buf != (void *)head_count || ctx->attn_cnt_heads != H || ctx->attn_cnt_launches >= (1u << 28)) {
        MOON_TRY(launch_fill_uniform_u32(ctx, head_count, H * HEAD_STRIDE, 0, 0, 1)); // zeros, in stream order
        ctx->attn_cnt_buf = head_count;
        ctx->attn_cnt_heads = H;
        ctx->attn_cnt_launches = 0;
    }
    const uint32_t target = ++ctx->attn_cnt_launches * (uint32_t)DEC_SPLITS;
    return launch_decode_attention_merged(ctx, qkv, cache_k, cache_v, table, partial, out, head_count, target, H, D, rot_dim, max_seq, pos, pos_dev, HEAD_STRIDE);
}

// q[H,64] already rotated, k,v[H][kv_len][64] contiguous: singleMaskedSDPA with an all-true mask.
int launch_decode_attention_plain(moon_ctx *ctx, const half_t *q, const half_t *k, const half_t *v, half_t *out, size_t H,
                                  size_t kv_len, size_t D) {
    if (D != 64 || kv_len == 0 || kv_len > 2048) return moon_fail(ctx, MOON_EINVAL_DIM, "plain decode attention: unsupported shape");
    MOON_TRY(moon_grow(ctx, ctx->work[1], H * DEC_SPLITS * (D + 2) * sizeof(float)));
    float *partial = (float *)ctx->work[1].ptr;
    ctx->attn_cnt_buf = nullptr; // these partials may cover the other path's counters: it clears them before its next launch
    hipLaunchKernelGGL((decode_attn_partial_kernel<64, false>), dim3((unsigned)(H * DEC_SPLITS)), dim3(256), 0, ctx->stream, q,
                       const_cast<half_t *>(k), const_cast<half_t *>(v), (const float *)nullptr, partial, (int)H, 0, (int)kv_len,
                       (int)kv_len - 1, (const uint32_t *)nullptr);
    MOON_HIP(ctx, hipGetLastError());
    hipLaunchKernelGGL(decode_attn_merge_kernel<64>, dim3((unsigned)H), dim3(64), 0, ctx->stream, partial, out);
    MOON_HIP(ctx, hipGetLastError());
    MOON_NOTE_KERNEL(ctx, "decode_attn_partial_kernel<64,false> + decode_attn_merge_kernel<64>");
    return MOON_OK;
}

// ---------------------------------------------------------------------------------------------------------------
// The same step for callers that cannot allocate device memory (code under HIP graph capture, serving loops, harnesses
// that forbid hipMalloc): the split partials live in a file-scope device array instead of the context's grown workspace.
// Every device the library runs on holds its own copy of the array (MOON_NOALLOC_MAX_HEADS * DEC_SPLITS * 66 floats =
// 270,336 bytes) until the process ends.  In host code the array's name is only a handle: the device address is asked
// for once per device (decode_attention_static_init, called with that device current when a context is created) and
// only that address is ever handed to a kernel.  Every launch writes all partials of its n_heads before its merge
// kernel reads them (a split without keys writes m = -inf, l = 0, o = 0), so nothing of an earlier call is read and
// nothing needs clearing; two calls that overlap on one device (different contexts or streams) race on the array.
constexpr size_t MOON_NOALLOC_MAX_HEADS = 128;
constexpr int MOON_NOALLOC_MAX_DEVICES = 64;
static __device__ __align__(256) float scratch[MOON_NOALLOC_MAX_HEADS * DEC_SPLITS * (64 + 2)];
static float *g_scratch_ptr[MOON_NOALLOC_MAX_DEVICES]; // device address of `scratch` on each device, null until asked for
static std::mutex g_scratch_mu;

int decode_attention_static_init(moon_ctx *ctx) {
    if (ctx->device < 0 || ctx->device >= MOON_NOALLOC_MAX_DEVICES) return MOON_OK; // the no-alloc entry point reports it
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (g_scratch_ptr[ctx->device]) return MOON_OK;
    float *p = nullptr;
    MOON_HIP(ctx, hipGetSymbolAddress((void **)&p, HIP_SYMBOL(scratch))); // the current device's copy
    g_scratch_ptr[ctx->device] = p;
    return MOON_OK;
}

extern "C" int moon_dev_decode_attention_noalloc(moon_ctx *ctx, const void *qkv, void *cache_k, void *cache_v, const void *freqs_cis,
                                                 void *out, size_t n_heads, size_t head_dim, size_t rot_dim, size_t max_seq, size_t pos) {
    if (!ctx) return MOON_EINVAL;
    std::lock_guard<std::mutex> lock(ctx->mu);
    if (!qkv || !cache_k || !cache_v || !freqs_cis || !out) return moon_fail(ctx, MOON_EINVAL, "dev_decode_attention_noalloc: null operand");
    if (head_dim != 64) return moon_fail(ctx, MOON_EINVAL_DIM, "decode attention: head_dim %zu unsupported (64 only)", head_dim);
    if (!n_heads || n_heads > MOON_NOALLOC_MAX_HEADS)
        return moon_fail(ctx, MOON_EINVAL_DIM, "dev_decode_attention_noalloc: n_heads %zu outside 1..%zu (the static workspace holds %zu heads)",
                         n_heads, MOON_NOALLOC_MAX_HEADS, MOON_NOALLOC_MAX_HEADS);
    if (rot_dim > head_dim || rot_dim % 2) return moon_fail(ctx, MOON_EROT_DIM, "decode attention: bad rot_dim %zu", rot_dim);
    if (max_seq > 2048 || pos >= max_seq)
        return moon_fail(ctx, MOON_ESEQ_TOO_LONG, "decode attention: pos %zu >= max_seq %zu (limit 2048)", pos, max_seq);
    float *partial = nullptr;
    if (ctx->device >= 0 && ctx->device < MOON_NOALLOC_MAX_DEVICES) {
        std::lock_guard<std::mutex> slock(g_scratch_mu);
        partial = g_scratch_ptr[ctx->device];
    }
    if (!partial) return moon_fail(ctx, MOON_EHIP, "dev_decode_attention_noalloc: no static workspace on device %d", ctx->device);
    hipLaunchKernelGGL((decode_attn_partial_kernel<64, true>), dim3((unsigned)(n_heads * DEC_SPLITS)), dim3(256), 0, ctx->stream,
                       (const half_t *)qkv, (half_t *)cache_k, (half_t *)cache_v, (const float *)freqs_cis, partial, (int)n_heads,
                       (int)rot_dim, (int)max_seq, (int)pos, (const uint32_t *)nullptr);
    MOON_HIP(ctx, hipGetLastError());
    hipLaunchKernelGGL(decode_attn_merge_kernel<64>, dim3((unsigned)n_heads), dim3(64), 0, ctx->stream, partial, (half_t *)out);
    MOON_HIP(ctx, hipGetLastError());
    MOON_NOTE_KERNEL(ctx, "decode_attn_partial_kernel<64,true> + decode_attn_merge_kernel<64>");
    return MOON_OK;
}
