// Normalisation, element-wise, rotary, layout and arg-max kernels around the matrix products.
// All are HBM/latency bound; each rounds to f16 exactly where the reference op does.
#include "norm.hpp"

namespace {

// ops.layerNorm, one workgroup per row (see norm.hpp)
__global__ __launch_bounds__(256) void layernorm_kernel(const half_t *__restrict__ x, const half_t *__restrict__ gamma,
                                                         const half_t *__restrict__ beta, half_t *__restrict__ y,
                                                         int dim, float eps) {
    __shared__ float sm[16];
    layernorm_row(x + size_t(blockIdx.x) * dim, gamma, beta, y + size_t(blockIdx.x) * dim, dim, eps, sm);
}

__global__ void gelu_kernel(half_t *x, size_t n) {
    size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    const size_t stride = size_t(gridDim.x) * blockDim.x;
    for (; i < n; i += stride) x[i] = (half_t)gelu_f32((float)x[i]);
}

__global__ void bias_add_kernel(half_t *a, const half_t *__restrict__ b, size_t rows, size_t cols) {
    size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    const size_t n = rows * cols, stride = size_t(gridDim.x) * blockDim.x;
    for (; i < n; i += stride) a[i] = (half_t)((float)a[i] + (float)b[i % cols]);
}

__global__ void add_kernel(half_t *a, const half_t *__restrict__ b, size_t n) {
    size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    const size_t stride = size_t(gridDim.x) * blockDim.x;
    for (; i < n; i += stride) a[i] = (half_t)((float)a[i] + (float)b[i]);
}

// text_model.zig:170-171: attn += mlp (f16), hidden += attn (f16)
__global__ void residual2_kernel(half_t *hidden, const half_t *__restrict__ attn, const half_t *__restrict__ mlp, size_t n) {
    size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    const size_t stride = size_t(gridDim.x) * blockDim.x;
    for (; i < n; i += stride) {
        const half_t a = (half_t)((float)attn[i] + (float)mlp[i]);
        hidden[i] = (half_t)((float)hidden[i] + (float)a);
    }
}

// sampling.argmax (sampling.zig:257-273): strict '>' scan from index 0, i.e. the lowest index among
// equal maxima; NaN never wins.  Single workgroup (51200 logits = 100 KiB).
template <class T>
__global__ __launch_bounds__(1024) void argmax_kernel(const T *__restrict__ logits, int n, uint32_t *out) {
    __shared__ float sv[16];
    __shared__ int si[16];
    float best = -INFINITY;
    int idx = 0x7fffffff;
    bool any = false;
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        const float v = (float)logits[i];
        if (v > best || (!any && v == best)) { // first occurrence within this thread's ascending scan
            best = v;
            idx = i;
            any = true;
        }
    }
    // reduce (value desc, index asc)
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        const float ov = __shfl_xor(best, off, 64);
        const int oi = __shfl_xor(idx, off, 64);
        if (ov > best || (ov == best && oi < idx)) {
            best = ov;
            idx = oi;
        }
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0) {
        sv[wave] = best;
        si[wave] = idx;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        const int nw = (blockDim.x + 63) >> 6;
        for (int w = 1; w < nw; w++)
            if (sv[w] > best || (sv[w] == best && si[w] < idx)) {
                best = sv[w];
                idx = si[w];
            }
        // the reference starts from max_val = data[0], max_idx = 0: if nothing compares greater
        // (all NaN, or all -inf) index 0 is returned
        const float first = (float)logits[0];
        *out = (idx == 0x7fffffff || first != first) ? 0u : (uint32_t)idx; // a NaN at index 0 is never displaced
    }
}

// text_encoder (text_model.zig:121-134): row gather
__global__ void embed_kernel(const half_t *__restrict__ wte, const uint32_t *__restrict__ ids, half_t *out, int dim) {
    const uint32_t id = ids[blockIdx.x];
    const half_t *src = wte + size_t(id) * dim;
    half_t *dst = out + size_t(blockIdx.x) * dim;
    for (int i = threadIdx.x; i < dim; i += blockDim.x) dst[i] = src[i];
}

// rope.precomputeFreqsCis (rope.zig:32-128): [end, rot_dim/2, 2] f32 (cos, sin).  The reference's steps are f32: power =
// 2i/dim, inv = 1/pow(theta, power), angle = p * inv, then cos and sin.  An f32 pow that is one ulp off moves the angle of
// the last rows by 1e-4 rad, so each transcendental is evaluated in f64 on its f32 argument and rounded once: the
// correctly rounded f32 result (32768 entries, once per model).
__global__ void rope_table_kernel(float *table, int half_pairs, int end, int dim, float theta) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= half_pairs * end) return;
    const int p = i / half_pairs, f = i % half_pairs;
    const float power = (float)(2 * f) / (float)dim;
    const float inv = 1.0f / (float)pow((double)theta, (double)power);
    const float ang = (float)p * inv;
    table[2 * i] = (float)cos((double)ang);
    table[2 * i + 1] = (float)sin((double)ang);
}

// rope.applyRotEmb (rope.zig:130-272) on [H,S,D]; one thread per (h,s,d<D) element slot
__global__ void rope_apply_kernel(const half_t *__restrict__ x, half_t *__restrict__ out, int H, int S, int D,
                                  const float *__restrict__ table, const uint64_t *__restrict__ position_ids,
                                  size_t pos0, int rot_dim) {
    const size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    const size_t total = size_t(H) * S * D;
    if (i >= total) return;
    const int d = int(i % D);
    const int s = int((i / D) % S);
    const int half = rot_dim >> 1;
    if (d >= rot_dim) {
        out[i] = x[i];
        return;
    }
    if (d >= half) return; // the partner thread writes both
    const size_t p = position_ids ? (size_t)position_ids[s] : pos0 + s;
    const float c = table[(p * half + d) * 2], sn = table[(p * half + d) * 2 + 1];
    half_t o_r, o_i;
    rotate_pair((float)x[i], (float)x[i + half], c, sn, o_r, o_i);
    out[i] = o_r;
    out[i + half] = o_i;
}

// Prefill glue: qkv[S, 3*H*D] -> rotated q [H,S,D]; rotated k and v written straight into the cache
// [H][max_seq][D] at pos0+s (text_model.zig:198-262 without the intermediate copies).
__global__ void qkv_rope_cache_kernel(const half_t *__restrict__ qkv, half_t *__restrict__ q_out, half_t *__restrict__ ck,
                                      half_t *__restrict__ cv, const float *__restrict__ table, int S, int H, int D,
                                      int rot_dim, int max_seq, size_t pos0) {
    const size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    const size_t total = size_t(S) * H * D;
    if (i >= total) return;
    const int d = int(i % D);
    const int h = int((i / D) % H);
    const int s = int(i / (size_t(D) * H));
    const size_t hd = size_t(H) * D;
    const half_t *row = qkv + size_t(s) * 3 * hd;
    const size_t col = size_t(h) * D + d;
    const size_t qo = (size_t(h) * S + s) * D + d;
    const size_t co = (size_t(h) * max_seq + pos0 + s) * D + d;
    const int half = rot_dim >> 1;
    cv[co] = row[2 * hd + col];
    if (d >= rot_dim) {
        q_out[qo] = row[col];
        ck[co] = row[hd + col];
        return;
    }
    if (d >= half) return;
    const size_t p = pos0 + s;
    const float c = table[(p * half + d) * 2], sn = table[(p * half + d) * 2 + 1];
    half_t o_r, o_i;
    rotate_pair((float)row[col], (float)row[col + half], c, sn, o_r, o_i);
    q_out[qo] = o_r;
    q_out[qo + half] = o_i;
    rotate_pair((float)row[hd + col], (float)row[hd + col + half], c, sn, o_r, o_i);
    ck[co] = o_r;
    ck[co + half] = o_i;
}

// The same in 16-byte pieces: thread (s, h, g) copies granule g (8 halfs) of v, and of q and k where they are not rotated;
// granules below rot_dim / 2 rotate themselves against their partners rot_dim / 2 further on and write both.
// Needs D % 8 == 0, rot_dim % 16 == 0 and 16-byte aligned rows (checked by the launcher).
__global__ __launch_bounds__(256) void qkv_rope_cache_vec_kernel(const half_t *__restrict__ qkv, half_t *__restrict__ q_out,
                                                                  half_t *__restrict__ ck, half_t *__restrict__ cv,
                                                                  const float *__restrict__ table, int S, int H, int D, int rot_dim,
                                                                  int max_seq, size_t pos0) {
    const int G = D >> 3;
    const size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= size_t(S) * H * G) return;
    const int g = int(i % G), h = int((i / G) % H), s = int(i / (size_t(G) * H));
    const size_t hd = size_t(H) * D;
    const half_t *row = qkv + size_t(s) * 3 * hd + size_t(h) * D + 8 * g;
    const size_t qo = (size_t(h) * S + s) * D + 8 * g, co = (size_t(h) * max_seq + pos0 + s) * D + 8 * g;
    const int half = rot_dim >> 1;
    *reinterpret_cast<half8_t *>(cv + co) = *reinterpret_cast<const half8_t *>(row + 2 * hd);
    if (8 * g >= rot_dim) {
        *reinterpret_cast<half8_t *>(q_out + qo) = *reinterpret_cast<const half8_t *>(row);
        *reinterpret_cast<half8_t *>(ck + co) = *reinterpret_cast<const half8_t *>(row + hd);
        return;
    }
    if (8 * g >= half) return;
    const half8_t qr = *reinterpret_cast<const half8_t *>(row), qi = *reinterpret_cast<const half8_t *>(row + half);
    const half8_t kr = *reinterpret_cast<const half8_t *>(row + hd), ki = *reinterpret_cast<const half8_t *>(row + hd + half);
    const float4 *t = reinterpret_cast<const float4 *>(table + ((pos0 + s) * half + 8 * g) * 2); // (cos, sin) of 8 consecutive d
    half8_t oqr, oqi, okr, oki;
#pragma unroll
    for (int e = 0; e < 4; e++) {
        const float4 cs = t[e]; // d = 8g + 2e, 8g + 2e + 1
        half_t a, b;
        rotate_pair((float)qr[2 * e], (float)qi[2 * e], cs.x, cs.y, a, b);
        oqr[2 * e] = a; oqi[2 * e] = b;
        rotate_pair((float)qr[2 * e + 1], (float)qi[2 * e + 1], cs.z, cs.w, a, b);
        oqr[2 * e + 1] = a; oqi[2 * e + 1] = b;
        rotate_pair((float)kr[2 * e], (float)ki[2 * e], cs.x, cs.y, a, b);
        okr[2 * e] = a; oki[2 * e] = b;
        rotate_pair((float)kr[2 * e + 1], (float)ki[2 * e + 1], cs.z, cs.w, a, b);
        okr[2 * e + 1] = a; oki[2 * e + 1] = b;
    }
    *reinterpret_cast<half8_t *>(q_out + qo) = oqr;
    *reinterpret_cast<half8_t *>(q_out + qo + half) = oqi;
    *reinterpret_cast<half8_t *>(ck + co) = okr;
    *reinterpret_cast<half8_t *>(ck + co + half) = oki;
}

__global__ void merge_heads_kernel(const half_t *__restrict__ x, half_t *__restrict__ out, int S, int H, int D) {
    const size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= size_t(S) * H * D) return;
    const int d = int(i % D), h = int((i / D) % H), s = int(i / (size_t(D) * H));
    out[i] = x[(size_t(h) * S + s) * D + d];
}

__global__ void split_heads_kernel(const half_t *__restrict__ qkv, size_t row_stride, size_t col_off,
                                   half_t *__restrict__ out, int S, int H, int D) {
    const size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= size_t(S) * H * D) return;
    const int d = int(i % D), s = int((i / D) % S), h = int(i / (size_t(D) * S));
    out[i] = qkv[size_t(s) * row_stride + col_off + size_t(h) * D + d];
}

inline unsigned grid_for(size_t n, unsigned block = 256, unsigned cap = 65535u * 16) {
    size_t g = (n + block - 1) / block;
    return (unsigned)(g < 1 ? 1 : (g > cap ? cap : g));
}

} // namespace

int launch_layernorm(moon_ctx *ctx, const half_t *x, const half_t *gamma, const half_t *beta, half_t *y, size_t rows,
                     size_t dim, float eps) {
    if (!(eps > 0.0f)) return moon_fail(ctx, MOON_EEPS, "layerNorm: eps must be > 0 (InvalidEpsilon)");
    if (!rows || !dim) return MOON_OK;
    hipLaunchKernelGGL(layernorm_kernel, dim3((unsigned)rows), dim3(256), 0, ctx->stream, x, gamma, beta, y, (int)dim, eps);
    MOON_HIP(ctx, hipGetLastError());
    return MOON_OK;
}
int launch_gelu(moon_ctx *ctx, half_t *x, size_t n) {
    if (!n) return MOON_OK;
    hipLaunchKernelGGL(gelu_kernel, dim3(grid_for(n, 256, 8192)), dim3(256), 0, ctx->stream, x, n);
    MOON_HIP(ctx, hipGetLastError());
    return MOON_OK;
}
int launch_bias_add(moon_ctx *ctx, half_t *a, const half_t *b, size_t rows, size_t cols) {
    if (!rows || !cols) return MOON_OK;
    hipLaunchKernelGGL(bias_add_kernel, dim3(grid_for(rows * cols, 256, 8192)), dim3(256), 0, ctx->stream, a, b, rows, cols);
    MOON_HIP(ctx, hipGetLastError());
    return MOON_OK;
}
int launch_add(moon_ctx *ctx, half_t *a, const half_t *b, size_t n) {
    if (!n) return MOON_OK;
    hipLaunchKernelGGL(add_kernel, dim3(grid_for(n, 256, 8192)), dim3(256), 0, ctx->stream, a, b, n);
    MOON_HIP(ctx, hipGetLastError());
    return MOON_OK;
}
int launch_residual2(moon_ctx *ctx, half_t *hidden, const half_t *attn, const half_t *mlp, size_t n) {
    if (!n) return MOON_OK;
    hipLaunchKernelGGL(residual2_kernel, dim3(grid_for(n, 256, 8192)), dim3(256), 0, ctx->stream, hidden, attn, mlp, n);
    MOON_HIP(ctx, hipGetLastError());
    return MOON_OK;
}
// Everything encode_image does to the resized image before the patch embedding (vision_model.zig:129-184,
// reshape_handler.zig:5-129), one output element per thread: u8 -> f16 (exact), the image taken `copies` times
// (createPatches fills both crops from the same pixels), /255 in f16, (x - 0.5) / 0.5 in f16, and the rearrangement
// "b c (h p) (w q) -> b (h w) (c p q)".  Each f16 operation is an f32 operation rounded to f16, which for +, -, /
// of f16 operands gives the correctly rounded f16 result.  out rows are `pitch` halfs apart.
__global__ __launch_bounds__(256) void image_patches_kernel(const uint8_t *__restrict__ image, half_t *__restrict__ out, int H, int W, int C,
                                                            int P, int copies, int pitch) {
    const int wp = W / P, T = (H / P) * wp, dim = C * P * P;
    const size_t total = size_t(copies) * T * dim;
    for (size_t e = size_t(blockIdx.x) * blockDim.x + threadIdx.x; e < total; e += size_t(gridDim.x) * blockDim.x) {
        const int col = (int)(e % dim);
        const size_t row = e / dim; // copy * T + patch
        const int patch = (int)(row % T);
        const int pw = col % P, ph = (col / P) % P, c = col / (P * P);
        const int y = (patch / wp) * P + ph, x = (patch % wp) * P + pw;
        const half_t v = (half_t)(float)image[(size_t(y) * W + x) * C + c];
        const half_t scaled = (half_t)__fdiv_rn((float)v, 255.0f);   // val /= 255 (vision_model.zig:167-169)
        const half_t centred = (half_t)((float)scaled - 0.5f);       // (x - mean) / std, mean = std = 0.5 (reshape_handler.zig:90)
        out[row * pitch + col] = (half_t)__fdiv_rn((float)centred, 0.5f);
    }
}

int launch_image_patches(moon_ctx *ctx, const uint8_t *image, half_t *out, size_t H, size_t W, size_t C, size_t P, size_t copies, size_t pitch) {
    if (!H || !W || !C || !P || !copies) return moon_fail(ctx, MOON_EINVAL_DIM, "image_patches: zero dimension");
    if (H % P || W % P) return moon_fail(ctx, MOON_EINVAL_DIM, "image_patches: %zu x %zu is not a whole number of %zu x %zu patches (InvalidPatchSize)", H, W, P, P);
    const size_t dim = C * P * P, total = copies * (H / P) * (W / P) * dim;
    if (pitch < dim || H > 32768 || W > 32768 || C > 16 || total > 0x7fffffffull) return moon_fail(ctx, MOON_EINVAL, "image_patches: size out of range");
    const size_t blocks = (total + 255) / 256;
    hipLaunchKernelGGL(image_patches_kernel, dim3((unsigned)(blocks < 4096 ? blocks : 4096)), dim3(256), 0, ctx->stream, image, out, (int)H, (int)W, (int)C,
                       (int)P, (int)copies, (int)pitch);
    MOON_HIP(ctx, hipGetLastError());
    return MOON_OK;
}

int launch_argmax(moon_ctx *ctx, const half_t *logits, size_t n, uint32_t *index_out) {
    if (!n || n > 0x7fffffff) return moon_fail(ctx, MOON_EINVAL, "argmax: empty or oversized tensor");
    hipLaunchKernelGGL(argmax_kernel<half_t>, dim3(1), dim3(1024), 0, ctx->stream, logits, (int)n, index_out);
    MOON_HIP(ctx, hipGetLastError());
    return MOON_OK;
}
int launch_argmax_f32(moon_ctx *ctx, const float *logits, size_t n, uint32_t *index_out) {
    if (!n || n > 0x7fffffff) return moon_fail(ctx, MOON_EINVAL, "argmax: empty or oversized tensor");
    hipLaunchKernelGGL(argmax_kernel<float>, dim3(1), dim3(1024), 0, ctx->stream, logits, (int)n, index_out);
    MOON_HIP(ctx, hipGetLastError());
    return MOON_OK;
}
int launch_embed(moon_ctx *ctx, const half_t *wte, const uint32_t *ids, half_t *out, size_t n_ids, size_t dim) {
    if (!n_ids) return MOON_OK;
    hipLaunchKernelGGL(embed_kernel, dim3((unsigned)n_ids), dim3(256), 0, ctx->stream, wte, ids, out, (int)dim);
    MOON_HIP(ctx, hipGetLastError());
    return MOON_OK;
}
int launch_rope_table(moon_ctx *ctx, float *table, size_t rot_dim, size_t end, float theta) {
    const size_t n = (rot_dim / 2) * end;
    if (!n) return MOON_OK;
    hipLaunchKernelGGL(rope_table_kernel, dim3(grid_for(n)), dim3(256), 0, ctx->stream, table, (int)(rot_dim / 2), (int)end,
                       (int)rot_dim, theta);
    MOON_HIP(ctx, hipGetLastError());
    return MOON_OK;
}
int launch_rope_apply(moon_ctx *ctx, const half_t *x, half_t *out, size_t H, size_t S, size_t D, const float *table,
                      const uint64_t *position_ids, size_t pos0, size_t rot_dim) {
    const size_t n = H * S * D;
    if (!n) return MOON_OK;
    hipLaunchKernelGGL(rope_apply_kernel, dim3(grid_for(n)), dim3(256), 0, ctx->stream, x, out, (int)H, (int)S, (int)D, table,
                       position_ids, pos0, (int)rot_dim);
    MOON_HIP(ctx, hipGetLastError());
    return MOON_OK;
}
int launch_qkv_rope_cache(moon_ctx *ctx, const half_t *qkv, half_t *q_out, half_t *cache_k, half_t *cache_v,
                          const float *table, size_t S, size_t H, size_t D, size_t rot_dim, size_t max_seq, size_t pos0) {
    const size_t n = S * H * D;
    if (!n) return MOON_OK;
    const uintptr_t ptrs = reinterpret_cast<uintptr_t>(qkv) | reinterpret_cast<uintptr_t>(q_out) | reinterpret_cast<uintptr_t>(cache_k) |
                           reinterpret_cast<uintptr_t>(cache_v) | reinterpret_cast<uintptr_t>(table);
    if (D % 8 == 0 && rot_dim % 16 == 0 && rot_dim <= D && ptrs % 16 == 0) {
        hipLaunchKernelGGL(qkv_rope_cache_vec_kernel, dim3(grid_for(n / 8)), dim3(256), 0, ctx->stream, qkv, q_out, cache_k, cache_v, table,
                           (int)S, (int)H, (int)D, (int)rot_dim, (int)max_seq, pos0);
        MOON_HIP(ctx, hipGetLastError());
        return MOON_OK;
    }
    hipLaunchKernelGGL(qkv_rope_cache_kernel, dim3(grid_for(n)), dim3(256), 0, ctx->stream, qkv, q_out, cache_k, cache_v, table,
                       (int)S, (int)H, (int)D, (int)rot_dim, (int)max_seq, pos0);
    MOON_HIP(ctx, hipGetLastError());
    return MOON_OK;
}
int launch_merge_heads(moon_ctx *ctx, const half_t *x, half_t *out, size_t S, size_t H, size_t D) {
    const size_t n = S * H * D;
    if (!n) return MOON_OK;
    hipLaunchKernelGGL(merge_heads_kernel, dim3(grid_for(n)), dim3(256), 0, ctx->stream, x, out, (int)S, (int)H, (int)D);
    MOON_HIP(ctx, hipGetLastError());
    return MOON_OK;
}
int launch_split_heads(moon_ctx *ctx, const half_t *qkv, size_t row_stride, size_t col_off, half_t *out, size_t S, size_t H,
                       size_t D) {
    const size_t n = S * H * D;
    if (!n) return MOON_OK;
    hipLaunchKernelGGL(split_heads_kernel, dim3(grid_for(n)), dim3(256), 0, ctx->stream, qkv, row_stride, col_off, out, (int)S,
                       (int)H, (int)D);
    MOON_HIP(ctx, hipGetLastError());
    return MOON_OK;
}
