// Decode-time GEMV, y[N] = epi(x[K] . W[N,K]) -- replaces hgemm_trans.matmul's M==1 path
// (hgemm_trans.zig:430-455, processVectorChunk :55-118).
//
// Bandwidth bound: W is read exactly once with 128-bit loads (64 lanes x 16 B = one contiguous 1 KiB
// segment of a weight row per instruction), f32 accumulation, one wavefront owns ROWS consecutive
// rows so ROWS x UNROLL loads are in flight per lane before the first use.  x is re-read through
// the vector L1 (4-16 KiB, hot).  The 64-lane reduction order is fixed, so results are
// deterministic.  Algorithmic traffic per launch: N*K*2 (W) + K*2 (x) + N*2 (bias) + N*2 (y) bytes.
#include "epilogue.hpp"

namespace {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float dot8(const u32x4 &w, const u32x4 &x, float acc) {
    const half2_t *wp = reinterpret_cast<const half2_t *>(&w);
    const half2_t *xp = reinterpret_cast<const half2_t *>(&x);
#pragma unroll
    for (int i = 0; i < 4; i++) {
        acc = fmaf((float)wp[i][0], (float)xp[i][0], acc);
        acc = fmaf((float)wp[i][1], (float)xp[i][1], acc);
    }
    return acc;
}

template <int ROWS, int UNROLL, int EPI>
__global__ __launch_bounds__(256) void gemv_nt_kernel(const half_t *__restrict__ x, const half_t *__restrict__ W,
                                                       const half_t *__restrict__ bias, half_t *__restrict__ y,
                                                       int N, int K) {
    const int lane = threadIdx.x & 63;
    const int wave = (blockIdx.x * 4) + (threadIdx.x >> 6);
    const int row0 = wave * ROWS;
    if (row0 >= N) return;
    const int granules = K >> 3; // 16-byte pieces per row
    const u32x4 *xg = reinterpret_cast<const u32x4 *>(x);
    const u32x4 *wrow[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; r++) {
        const int row = min(row0 + r, N - 1); // tail rows re-read the last row; their result is dropped
        wrow[r] = reinterpret_cast<const u32x4 *>(W + size_t(row) * K);
    }
    float acc[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; r++) acc[r] = 0.0f;

    for (int g0 = lane; g0 < granules; g0 += 64 * UNROLL) {
        u32x4 wv[UNROLL][ROWS];
        u32x4 xv[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; u++) {
            const int g = g0 + 64 * u;
            const bool ok = g < granules;
            xv[u] = u32x4{0, 0, 0, 0};
#pragma unroll
            for (int r = 0; r < ROWS; r++) wv[u][r] = u32x4{0, 0, 0, 0};
            if (ok) {
                xv[u] = xg[g];
#pragma unroll
                for (int r = 0; r < ROWS; r++) wv[u][r] = __builtin_nontemporal_load(wrow[r] + g);
            }
        }
#pragma unroll
        for (int u = 0; u < UNROLL; u++)
#pragma unroll
            for (int r = 0; r < ROWS; r++) acc[r] = dot8(wv[u][r], xv[u], acc[r]);
    }
#pragma unroll
    for (int r = 0; r < ROWS; r++) acc[r] = wave_sum(acc[r]);
    if (lane == 0) {
#pragma unroll
        for (int r = 0; r < ROWS; r++)
            if (row0 + r < N) y[row0 + r] = apply_epilogue<EPI>(acc[r], bias, size_t(row0 + r));
    }
}

// Any K (no alignment assumption): one wave per row, scalar loads.
template <int EPI>
__global__ __launch_bounds__(256) void gemv_nt_generic_kernel(const half_t *__restrict__ x, const half_t *__restrict__ W,
                                                               const half_t *__restrict__ bias, half_t *__restrict__ y,
                                                               int N, int K) {
    const int lane = threadIdx.x & 63;
    const int row = (blockIdx.x * 4) + (threadIdx.x >> 6);
    if (row >= N) return;
    float acc = 0.0f;
    for (int k = lane; k < K; k += 64) acc = fmaf((float)W[size_t(row) * K + k], (float)x[k], acc);
    acc = wave_sum(acc);
    if (lane == 0) y[row] = apply_epilogue<EPI>(acc, bias, size_t(row));
}

template <int EPI>
int launch_epi(moon_ctx *ctx, const half_t *x, const half_t *W, const half_t *bias, half_t *y, int N, int K) {
    const bool vec = (K % 8 == 0) && ((reinterpret_cast<uintptr_t>(W) | reinterpret_cast<uintptr_t>(x)) % 16 == 0);
    if (!vec) {
        hipLaunchKernelGGL(gemv_nt_generic_kernel<EPI>, dim3((N + 3) / 4), dim3(256), 0, ctx->stream, x, W, bias, y, N, K);
    } else if (K >= 4096) {
        constexpr int ROWS = 1, UNROLL = 8;
        hipLaunchKernelGGL((gemv_nt_kernel<ROWS, UNROLL, EPI>), dim3((N + 4 * ROWS - 1) / (4 * ROWS)), dim3(256), 0,
                           ctx->stream, x, W, bias, y, N, K);
    } else {
        constexpr int ROWS = 2, UNROLL = 4;
        hipLaunchKernelGGL((gemv_nt_kernel<ROWS, UNROLL, EPI>), dim3((N + 4 * ROWS - 1) / (4 * ROWS)), dim3(256), 0,
                           ctx->stream, x, W, bias, y, N, K);
    }
    MOON_HIP(ctx, hipGetLastError());
    MOON_NOTE_KERNEL(ctx, "%s", !vec ? "gemv_nt_generic_kernel" : K >= 4096 ? "gemv_nt_kernel<1,8>" : "gemv_nt_kernel<2,4>");
    return MOON_OK;
}

} // namespace

int launch_gemv_nt(moon_ctx *ctx, const half_t *x, const half_t *W, const half_t *bias, half_t *y, size_t N, size_t K,
                   int epilogue) {
    if (N == 0) return MOON_OK;
    if (N > 0x7fffffff || K > 0x7fffffff) return moon_fail(ctx, MOON_EINVAL_DIM, "gemv: dimension too large");
    if (epilogue != MOON_EPI_NONE && !bias) return moon_fail(ctx, MOON_EINVAL, "gemv: epilogue needs a bias");
    switch (epilogue) {
    case MOON_EPI_NONE: return launch_epi<MOON_EPI_NONE>(ctx, x, W, bias, y, (int)N, (int)K);
    case MOON_EPI_BIAS: return launch_epi<MOON_EPI_BIAS>(ctx, x, W, bias, y, (int)N, (int)K);
    case MOON_EPI_BIAS_GELU: return launch_epi<MOON_EPI_BIAS_GELU>(ctx, x, W, bias, y, (int)N, (int)K);
    default: return moon_fail(ctx, MOON_EINVAL, "gemv: unknown epilogue %d", epilogue);
    }
}
