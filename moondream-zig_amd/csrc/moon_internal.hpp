// Internal declarations shared by the HIP translation units of libmoonhip.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <map>
#include <mutex>
#include <string>

#include "moonhip.h"

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));

// A device buffer that only ever grows; used for staging host-pointer calls and for workspaces.
constexpr size_t MOON_PIN_BYTES = size_t(256) << 10;
struct GrowBuf {
    void *ptr = nullptr;
    size_t cap = 0;
};

struct moon_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    hipEvent_t ev_start = nullptr, ev_stop = nullptr;
    std::mutex mu;
    std::string err;
    int cu_count = 0;
    char last_kernel[96] = ""; // moon_last_kernel: what the latest product / attention launch dispatched (set by the launchers)
    char gemm_kernel[8] = ""; // moon_set_gemm_kernel / MOON_GEMM_KERNEL: a product kernel to take where the shape allows it ("": by shape)
    // staging for host-pointer ops: a, b, c, bias/aux, mask
    GrowBuf stage[6];
    // page-locked host memory that the host-pointer entry points copy small operands and results through (allocated at first
    // use, MOON_PIN_BYTES each, one per staging slot and one for results): a copy between device memory and the caller's
    // pageable memory blocks the call for tens of microseconds.  Free again at the synchronisation that ends every such call.
    void *pin_up[6] = {nullptr, nullptr, nullptr, nullptr, nullptr, nullptr};
    void *pin_down = nullptr;
    // kernel workspaces (split-K partials, attention partials, transposed B)
    GrowBuf work[4]; // 0: split-K partials, 1: decode-attention partials, 2: transposed operands, 3: split-K partials kept for a later launch
    // stand-alone decode attention in one launch: per-head "splits finished" counters behind the partials in work[1]
    // (monotonic over launches; cleared whenever the buffer or the head count changes)
    void *attn_cnt_buf = nullptr;
    size_t attn_cnt_heads = 0;
    uint32_t attn_cnt_launches = 0;
    struct Resident {
        void *dptr;
        size_t n_elems;
        void *dptr_t = nullptr;    // [N,K] copy of a weight used as B[K,N] (hgemm.matmul's layout), made on its first such use
        size_t t_k = 0, t_n = 0;
    };
    std::map<const void *, Resident> resident;
};

int moon_fail(moon_ctx *ctx, int code, const char *fmt, ...);
// Notes what a launcher dispatched, for moon_last_kernel (a few dozen nanoseconds per call).
#define MOON_NOTE_KERNEL(ctx, ...) snprintf((ctx)->last_kernel, sizeof (ctx)->last_kernel, __VA_ARGS__)
int moon_grow(moon_ctx *ctx, GrowBuf &b, size_t bytes);

#define MOON_HIP(ctx, expr)                                                                          \
    do {                                                                                             \
        hipError_t _e = (expr);                                                                      \
        if (_e != hipSuccess)                                                                        \
            return moon_fail((ctx), (_e == hipErrorOutOfMemory) ? MOON_ENOMEM : MOON_EHIP,           \
                             "%s failed: %s (%s:%d)", #expr, hipGetErrorString(_e), __FILE__, __LINE__); \
    } while (0)

#define MOON_TRY(expr)               \
    do {                             \
        int _rc = (expr);            \
        if (_rc != MOON_OK) return _rc; \
    } while (0)

// Bookkeeping of the on-device generation loop (moondream.zig:323-368), one thread at the end of the kernel that picked the
// token.  state: [0] position (KV length), [1] tokens recorded so far, [2] current token, [3] 1 once the end-of-sequence
// token has come up, [4] that token's id + 1 (0: none).  The position moves on by `bump` (the append of the previous
// step's token); the end-of-sequence token is neither recorded nor does anything move after it (moondream.zig:341 breaks
// out of the loop there): the launches that the host had already queued behind it keep appending to the one position after
// the last valid one, which the session never reads.
#if defined(__HIPCC__)
__device__ __forceinline__ void record_token(uint32_t *state, uint32_t *out_ids, uint32_t tok, uint32_t bump) {
    if (state[3]) return;
    state[0] += bump;
    state[2] = tok;
    if (state[4] == tok + 1u) {
        state[3] = 1u;
        return;
    }
    if (out_ids) {
        out_ids[state[1]] = tok;
        state[1] += 1;
    }
}
#endif

// ---- kernel launchers (all asynchronous on ctx->stream, device pointers) ----

// y[N] = epi(x[K] . W[N,K]); K % 8 == 0 takes the 128-bit path.
int launch_gemv_nt(moon_ctx *ctx, const half_t *x, const half_t *W, const half_t *bias, half_t *y,
                   size_t N, size_t K, int epilogue);
// C[M,N] = epi(A[M,K] x B) with B[N,K] (b_layout NK) or B[K,N] (KN); MFMA kernel, generic fallback for odd K.
// epilogue: a MOON_EPI_* value, or the internal MOON_EPI_BIAS_RESID (3): C = f16(resid + f16(f16(acc) + bias)), resid may be C.
// ln: a LayerNorm of the finished rows of C into ln->out (the reference's next op on this tensor, vision_model.zig:239, 253,
// 266): fused into the split-K reduction where the product takes that path, a launch of its own otherwise.
// add (with epilogue 3 only): a second addend, C = f16(resid + f16(add + t)), t the product after its bias: the two adds of the
// decoder's parallel block (text_model.zig:170-171); add_scratch: M x N halfs the library may use where that is not fused.
struct GemmLayerNorm {
    const half_t *gamma, *beta;
    half_t *out;
    float eps;
    const half_t *add = nullptr;
    half_t *add_scratch = nullptr;
    // the second addend as the split-K partials of an earlier product that launch_gemm_partials left behind, with that product's
    // bias: add = f16(f16(sum of the partials) + add_bias) is then formed on the fly (add must still name M x N halfs, which
    // receive it where the epilogue is not fused)
    const float *add_partial = nullptr;
    int add_splits = 0;
    const half_t *add_bias = nullptr;
};
// The split-K product of launch_gemm without its reduction: the f32 partials [splits][M][N] stay in a workspace of the context
// (valid until the next call of this function) for a later launch_gemm to fold in through GemmLayerNorm::add_partial.
// *splits = 0 (nothing launched) where the shape does not take the split-K path.
int launch_gemm_partials(moon_ctx *ctx, const half_t *A, const half_t *B, size_t M, size_t N, size_t K, int b_layout, const float **partial,
                         int *splits);
int launch_gemm(moon_ctx *ctx, const half_t *A, const half_t *B, const half_t *bias, half_t *C,
                size_t M, size_t N, size_t K, int b_layout, int epilogue, const half_t *resid = nullptr, const GemmLayerNorm *ln = nullptr);
// A decoder block's qkv projection [M, K] . [3 * H * D, K]^T + bias with launch_qkv_rope_cache folded into its epilogue: the
// rotated q goes to q_out [H][M][D], the rotated k and v to rows pos0 .. pos0 + M - 1 of the cache [H][max_seq][D]; the
// projection itself is not written anywhere.  The same bits as the two launches.  Only for D = 64 and the shapes that take the
// 256- or 192-row product kernels; *done says whether anything was launched.
int launch_gemm_qkv_rope(moon_ctx *ctx, const half_t *A, const half_t *W, const half_t *bias, size_t M, size_t K, half_t *q_out, half_t *cache_k,
                         half_t *cache_v, const float *table, size_t H, size_t D, size_t rot_dim, size_t max_seq, size_t pos0, bool *done);
// Two products with the same [M, N] result in ONE launch, then the launch that finishes both, as launch_gemm does with
// ln->add_partial set: C = f16(resid + f16(add + t)), add = f16(f16(A_add . B_add^T) + bias_add), t = f16(f16(A . B^T) + bias),
// and the LayerNorm of the finished rows into ln.out (ln.add must name M x N halfs all the same).  Both B operands are [N, K].
// Only for shapes where that fills the device in one round (M >= 192, N <= 2048, K's multiples of 64, 16-byte aligned
// operands); *done says whether anything was launched, and if not the caller runs the products one by one.
int launch_gemm_pair_ln(moon_ctx *ctx, const half_t *A_add, const half_t *B_add, const half_t *bias_add, size_t K_add, const half_t *A, const half_t *B,
                        const half_t *bias, size_t K, const half_t *resid, half_t *C, size_t M, size_t N, const GemmLayerNorm &ln, bool *done);

int launch_layernorm(moon_ctx *ctx, const half_t *x, const half_t *gamma, const half_t *beta, half_t *y,
                     size_t rows, size_t dim, float eps);
int launch_gelu(moon_ctx *ctx, half_t *x, size_t n);
int launch_bias_add(moon_ctx *ctx, half_t *a, const half_t *b, size_t rows, size_t cols);
int launch_add(moon_ctx *ctx, half_t *a, const half_t *b, size_t n);
// a = f16(a + f16(b + c))  -- the parallel-block residual (text_model.zig:170-171)
int launch_residual2(moon_ctx *ctx, half_t *hidden, const half_t *attn, const half_t *mlp, size_t n);
int launch_argmax(moon_ctx *ctx, const half_t *logits, size_t n, uint32_t *index_out);
int launch_argmax_f32(moon_ctx *ctx, const float *logits, size_t n, uint32_t *index_out);
// resized u8 image [H,W,C] -> normalised f16 patches [copies * (H/P)*(W/P), C*P*P], rows `pitch` halfs apart
int launch_image_patches(moon_ctx *ctx, const uint8_t *image, half_t *out, size_t H, size_t W, size_t C, size_t P, size_t copies, size_t pitch);
// logits_f32: the row as f32 instead of f16 (then logits is unused).
// sampling.sample for the methods other than greedy: u, or u_dev[state ? state[1] : 0] when u_dev is set; the token goes to
// out[0] (if out) and, if state, to state[2] and out_ids[state[1]++], and state[0] += bump_pos (the decode loop's bookkeeping).
// skip_if: a device word; when it is not 0 as the kernel starts, the kernel does nothing (the step's token is decided already).
int launch_sample(moon_ctx *ctx, const half_t *logits, size_t n, const moon_sampling_config *cfg, float u, const float *u_dev,
                  uint32_t *state, uint32_t *out_ids, uint32_t *out, uint32_t bump_pos = 0, const float *logits_f32 = nullptr,
                  const uint32_t *skip_if = nullptr);
int launch_embed(moon_ctx *ctx, const half_t *wte, const uint32_t *ids, half_t *out, size_t n_ids, size_t dim);
int launch_rope_table(moon_ctx *ctx, float *table, size_t rot_dim, size_t end, float theta);
// x,out [H,S,D]; position_ids on device (u64) or, if null, pos0 + s.
int launch_rope_apply(moon_ctx *ctx, const half_t *x, half_t *out, size_t H, size_t S, size_t D,
                      const float *table, const uint64_t *position_ids, size_t pos0, size_t rot_dim);
// prefill: split qkv[S,3*H*D] -> rotated q [H,S,D] (scratch), rotated k and v appended into the cache at pos0.
int launch_qkv_rope_cache(moon_ctx *ctx, const half_t *qkv, half_t *q_out, half_t *cache_k, half_t *cache_v,
                          const float *table, size_t S, size_t H, size_t D, size_t rot_dim, size_t max_seq, size_t pos0);
// [H,S,D] -> [S,H*D]
int launch_merge_heads(moon_ctx *ctx, const half_t *x, half_t *out, size_t S, size_t H, size_t D);
// [S, row_stride] columns col_off.. -> [H,S,D]
int launch_split_heads(moon_ctx *ctx, const half_t *qkv, size_t row_stride, size_t col_off, half_t *out,
                       size_t S, size_t H, size_t D);

int launch_fill_normal(moon_ctx *ctx, half_t *dst, size_t n, uint64_t seed, uint64_t stream, float std_dev);
int launch_fill_const(moon_ctx *ctx, half_t *dst, size_t n, float value);
int launch_fill_uniform_u32(moon_ctx *ctx, uint32_t *dst, size_t n, uint64_t seed, uint64_t stream, uint32_t modulo);

// generic attention: q[H,Lq,D] k,v with head stride kv_head_stride elements (so a cache can be read in place);
// out_merged: write [Lq, H*D] instead of [H,Lq,D].
int launch_sdpa_packed_qkv(moon_ctx *ctx, const half_t *qkv, half_t *out, size_t H, size_t T, size_t D, bool *handled);
int launch_sdpa(moon_ctx *ctx, const half_t *q, const half_t *k, const half_t *v, half_t *out, size_t H,
                size_t Lq, size_t Lkv, size_t D, size_t kv_head_stride, long causal_pos, const uint8_t *mask,
                size_t mask_stride, bool out_merged);
int launch_decode_attention(moon_ctx *ctx, const half_t *qkv, half_t *cache_k, half_t *cache_v, const float *table,
                            half_t *out, size_t H, size_t D, size_t rot_dim, size_t max_seq, size_t pos,
                            const uint32_t *pos_dev);
// asks for the device address of the static workspace of moon_dev_decode_attention_noalloc on ctx->device (once per device)
int decode_attention_static_init(moon_ctx *ctx);
int launch_sdpa_generic(moon_ctx *ctx, const half_t *q, const half_t *k, const half_t *v, half_t *out, size_t H, size_t Lq,
                        size_t Lkv, size_t D, size_t kv_head_stride, long causal_pos, const uint8_t *mask, size_t mask_stride,
                        bool out_merged);
// dst[cols, rows] = transpose(src[rows, cols])
int launch_transpose(moon_ctx *ctx, const half_t *src, half_t *dst, size_t rows, size_t cols);
