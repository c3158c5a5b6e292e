// What the matrix-product kernels of gemm.hip and gemm_wide.hpp share: tile constants, the LDS swizzle, the argument block.
#pragma once
#include "epilogue.hpp"

namespace {

constexpr int BM = 128, BN = 128, BK = 64;
constexpr int TILE_HALFS = 128 * BK; // one 128-row operand tile

// Operand tiles sit in LDS as [row][64 halfs]; the 16-byte granules of a row are XOR-swizzled by (row >> 1) & 7, which makes
// the 128-bit operand reads of 32 consecutive rows and the 128-bit staging writes bank-conflict free.
__device__ __forceinline__ int swz(int row, int granule) { return granule ^ ((row >> 1) & 7); }

struct GemmArgs {
    const half_t *A;  // [M,K]
    const half_t *Bt; // [N,K]
    const half_t *bias;
    const half_t *resid; // [M,N] added after the bias for MOON_EPI_BIAS_RESID (may be C itself)
    half_t *C;        // [M,N]
    float *partial;   // [splits][M][N] when splits > 1
    int M, N, K;
    int tiles_m, tiles_n, splits, k_per_split; // k_per_split is a multiple of BK
    int a_bytes, bt_bytes; // sizes of A and Bt (the wavefront-specialised kernels address them as buffers; < 2^31)
    int lds_epilogue; // write the tile through LDS in full lines (needs 16-byte aligned C / bias / resid rows)
    int super_m, super_n; // gemm_wide.hpp: tiles are dealt in blocks of super_m x super_n tiles (>= 1 each)
    // the *_rope kernels only: the product is a decoder block's qkv projection [M, 3 * H * 64]; instead of C they write the
    // rotated q [H][M][64] and the cache rows [H][max_seq][64] of k (rotated) and v at positions pos0 .. pos0 + M - 1
    half_t *rope_q, *rope_ck, *rope_cv;
    const float *rope_table; // [max_seq][rot_dim / 2][2] (cos, sin)
    int rope_H, rope_dim, rope_max_seq, rope_pos0;
};

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

} // namespace
