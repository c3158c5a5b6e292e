// Shape-generic scaled-dot-product attention (any head_dim <= 256, any mask) -- the fallback behind
// attention.multiMasklessSDPA / multiMaskedSDPA / singleMaskedSDPA (attention.zig:125-234, 416-541, 759-811)
// for shapes and masks the matrix-core kernel does not cover.  One wavefront per query row: scores for
// the whole key range are kept in LDS (kv_len <= 4096), softmax as ops.softmax does it (max, exp clamped
// to 0 below -88, reciprocal of the sum; ops.zig:1574-1601), then o = sum_j p_j v_j in key order.
#include "epilogue.hpp"

namespace {

constexpr int GEN_MAX_KV = 4096;

__global__ __launch_bounds__(256) void sdpa_generic_kernel(const half_t *__restrict__ q, const half_t *__restrict__ k,
                                                            const half_t *__restrict__ v, half_t *__restrict__ out, int H, int Lq,
                                                            int Lkv, int D, size_t kv_head_stride, long causal_pos,
                                                            const uint8_t *__restrict__ mask, size_t mask_stride, int out_merged,
                                                            float scale) {
    extern __shared__ float smem[]; // [4 waves][Lkv] scores, then [4][D] q rows
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int row_raw = blockIdx.x * 4 + wave; // query row within the head
    const bool active = row_raw < Lq;
    const int row = active ? row_raw : Lq - 1; // idle waves redo the last row and drop the result (keeps barriers uniform)
    const int h = blockIdx.y;
    float *sc = smem + size_t(wave) * Lkv;
    float *sq = smem + size_t(4) * Lkv + size_t(wave) * D;
    for (int d = lane; d < D; d += 64) sq[d] = (float)q[(size_t(h) * Lq + row) * D + d];
    __syncthreads();
    const half_t *kh = k + size_t(h) * kv_head_stride;
    const half_t *vh = v + size_t(h) * kv_head_stride;

    float mx = -INFINITY;
    for (int j = lane; j < Lkv; j += 64) {
        const half_t *kr = kh + size_t(j) * D;
        float s = 0.0f;
        for (int d = 0; d < D; d++) s = fmaf(sq[d], (float)kr[d], s);
        s *= scale; // scale applied after the product (attention.zig:192-194, 487-489)
        bool visible = true;
        if (causal_pos >= 0) visible = (long)j <= causal_pos + row;
        if (mask) visible = visible && mask[size_t(row) * mask_stride + j] != 0;
        if (!visible) s = -INFINITY;
        sc[j] = s;
        mx = fmaxf(mx, s);
    }
    mx = wave_max(mx);
    float sum = 0.0f;
    for (int j = lane; j < Lkv; j += 64) {
        const float d = sc[j] - mx;
        const float e = (d > -88.0f) ? __expf(d) : 0.0f;
        sc[j] = e;
        sum += e;
    }
    sum = wave_sum(sum);
    // a fully masked row has sum == 0: the reference leaves -inf scores in place and its P.V product is NaN
    const float inv = (sum > 0.0f) ? 1.0f / sum : __builtin_nanf("");
    __syncthreads(); // the probabilities written above are read by other lanes below
    for (int d = lane; d < D; d += 64) {
        float o = 0.0f;
        for (int j = 0; j < Lkv; j++) o = fmaf(sc[j] * inv, (float)vh[size_t(j) * D + d], o);
        const size_t oi = out_merged ? (size_t(row) * H + h) * D + d : (size_t(h) * Lq + row) * D + d;
        if (active) out[oi] = (half_t)o;
    }
}

} // namespace

int launch_sdpa_generic(moon_ctx *ctx, const half_t *q, const half_t *k, const half_t *v, half_t *out, size_t H, size_t Lq,
                        size_t Lkv, size_t D, size_t kv_head_stride, long causal_pos, const uint8_t *mask, size_t mask_stride,
                        bool out_merged) {
    if (!H || !Lq || !D) return MOON_OK;
    if (!Lkv) return moon_fail(ctx, MOON_EINVAL_DIM, "sdpa: kv_len is 0");
    if (Lkv > GEN_MAX_KV) return moon_fail(ctx, MOON_ESEQ_TOO_LONG, "sdpa: kv_len %zu > %d", Lkv, GEN_MAX_KV);
    if (D > 256) return moon_fail(ctx, MOON_EINVAL_DIM, "sdpa: head_dim %zu > 256", D);
    if (H > 65535) return moon_fail(ctx, MOON_EINVAL_DIM, "sdpa: too many heads");
    const size_t shmem = (4 * Lkv + 4 * D) * sizeof(float);
    if (shmem > 48 * 1024)
        MOON_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void *>(sdpa_generic_kernel),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem));
    const float scale = 1.0f / sqrtf((float)D);
    hipLaunchKernelGGL(sdpa_generic_kernel, dim3((unsigned)((Lq + 3) / 4), (unsigned)H), dim3(256), shmem, ctx->stream, q, k, v, out,
                       (int)H, (int)Lq, (int)Lkv, (int)D, kv_head_stride, causal_pos, mask, mask_stride, out_merged ? 1 : 0, scale);
    MOON_HIP(ctx, hipGetLastError());
    MOON_NOTE_KERNEL(ctx, "sdpa_generic_kernel");
    return MOON_OK;
}

int launch_sdpa_mfma(moon_ctx *ctx, const half_t *q, const half_t *k, const half_t *v, half_t *out, size_t H, size_t Lq,
                     size_t Lkv, size_t D, size_t kv_head_stride, long causal_pos, bool out_merged, bool *handled);

int launch_sdpa(moon_ctx *ctx, const half_t *q, const half_t *k, const half_t *v, half_t *out, size_t H, size_t Lq, size_t Lkv,
                size_t D, size_t kv_head_stride, long causal_pos, const uint8_t *mask, size_t mask_stride, bool out_merged) {
    if (!mask) {
        bool handled = false;
        MOON_TRY(launch_sdpa_mfma(ctx, q, k, v, out, H, Lq, Lkv, D, kv_head_stride, causal_pos, out_merged, &handled));
        if (handled) return MOON_OK;
    }
    return launch_sdpa_generic(ctx, q, k, v, out, H, Lq, Lkv, D, kv_head_stride, causal_pos, mask, mask_stride, out_merged);
}
