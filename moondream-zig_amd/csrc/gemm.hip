// FP16 GEMM on the matrix cores, C[M,N] = epi(A[M,K] x B) -- replaces hgemm.matmul (hgemm.zig:362-426,
// B[K,N]) and the tiled path of hgemm_trans.matmul (hgemm_trans.zig:457-487, B[N,K]).
//
// Tile: 128 (m) x 128 (n) x 64 (k), four multiplying wavefronts in a 2x2 grid, each owning a 64x64 sub-tile as 2x2
// v_mfma_f32_32x32x16_f16 accumulators (64 f32 VGPRs); a 256 x 128 tile (128x64 sub-tiles) for shapes with more tiles
// than CUs.  Both operands are staged k-contiguous in LDS ([row][64 halfs], 16-byte granules XOR-swizzled by
// (row>>1)&7 so the 128-bit operand reads of 32 consecutive rows and the 128-bit staging writes are bank-conflict
// free), several k-tiles deep, with one barrier per k-tile.  Three kernels share this: two specialised by wavefront
// (loaders that copy global -> LDS directly, multipliers that only read LDS and issue MFMAs) and a register-staged one
// (256 threads, two workgroups per CU) for whatever those do not take.
// The weight rows feed the MFMA "A" operand and the activation rows the "B" operand, so every lane ends up
// holding 4 consecutive n for one m.  f32 accumulation over the whole K, one rounding to f16 (then the bias / GELU
// roundings) exactly as the reference does.
//
// B[K,N] inputs (vision layout) are first transposed to [N,K] by a bandwidth-bound kernel into a
// workspace; resident model weights are transposed once at load time instead.
// Small grids (tiles < CUs) split K across workgroups: f32 partials to a workspace, then a fixed-order
// reduction applies the epilogue (deterministic, no atomics).
#include <atomic>
#include <cstring>

#include "gemm_wide.hpp"

namespace {

// Writes one wavefront's 64x64 accumulators: f16 with the epilogue, or f32 partials when K is split.
// D[i][j] of an accumulator: i (weight row n) = 8*(v/4) + 4*(lane/32) + v%4, j (activation row m) = lane%32
template <int EPI>
__device__ __forceinline__ void gemm_store_tile(const GemmArgs &p, const float16_t (&acc)[2][2], int m0, int n0, int wm, int wn, int frag_row,
                                                int frag_g, int split) {
    const bool vec_store = (p.N % 4 == 0);
#pragma unroll
    for (int ni = 0; ni < 2; ni++)
#pragma unroll
        for (int mi = 0; mi < 2; mi++) {
            const int m = m0 + wm * 64 + mi * 32 + frag_row;
            if (m >= p.M) continue;
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const int n = n0 + wn * 64 + ni * 32 + 8 * q + 4 * frag_g;
                if (n >= p.N) continue;
                if (p.splits > 1) {
                    float *dst = p.partial + (size_t(split) * p.M + m) * p.N + n;
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        if (n + e < p.N) dst[e] = acc[ni][mi][4 * q + e];
                } else if (vec_store && n + 3 < p.N) {
                    half4_t o;
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        o[e] = apply_residual<EPI>(apply_epilogue<EPI>(acc[ni][mi][4 * q + e], p.bias, size_t(n + e)), p.resid, size_t(m) * p.N + n + e);
                    *reinterpret_cast<half4_t *>(p.C + size_t(m) * p.N + n) = o;
                } else {
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        if (n + e < p.N)
                            p.C[size_t(m) * p.N + n + e] =
                                apply_residual<EPI>(apply_epilogue<EPI>(acc[ni][mi][4 * q + e], p.bias, size_t(n + e)), p.resid, size_t(m) * p.N + n + e);
                }
            }
        }
}

// The same tile written through LDS: the accumulators hold, per lane, four consecutive n of one m, which straight to
// memory means 8-byte pieces 2N bytes apart (64 store instructions per wavefront, none of them a full line).  Here the
// wavefront parks its 64x64 tile in LDS as f16 (the matmul's own rounding), [m][n] with a pitch of 68 halfs, reads it
// back eight consecutive n per lane, applies the rest of the epilogue and stores 16 bytes per lane: eight lanes cover
// a 128-byte row segment, eight instructions the tile.  scratch: 64 * 68 halfs owned by this wavefront.  Needs
// N % 8 == 0 and no split of K.
constexpr int EPI_PITCH = 68;
template <int EPI, int MB = 2> // MB: 32-row blocks of m in the sub-tile (2: 64 rows; 1: 32 rows)
__device__ __forceinline__ void gemm_store_tile_lds(const GemmArgs &p, const float16_t (&acc)[2][MB], int m0, int n0, int wm, int wn, int lane,
                                                    half_t *scratch) {
    const int frag_row = lane & 31, frag_g = lane >> 5;
#pragma unroll
    for (int ni = 0; ni < 2; ni++)
#pragma unroll
        for (int mi = 0; mi < MB; mi++)
#pragma unroll
            for (int q = 0; q < 4; q++) {
                half4_t o;
#pragma unroll
                for (int e = 0; e < 4; e++) o[e] = (half_t)acc[ni][mi][4 * q + e];
                *reinterpret_cast<half4_t *>(scratch + (mi * 32 + frag_row) * EPI_PITCH + ni * 32 + 8 * q + 4 * frag_g) = o;
            }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // the wavefront reads back what its own lanes wrote
    const int nl = (lane & 7) * 8, n = n0 + wn * 64 + nl; // this lane's eight columns
    if (n >= p.N) return;
    half8_t bias = {0, 0, 0, 0, 0, 0, 0, 0};
    if (EPI >= MOON_EPI_BIAS) bias = *reinterpret_cast<const half8_t *>(p.bias + n);
#pragma unroll
    for (int r = 0; r < 4 * MB; r++) {
        const int ml = r * 8 + (lane >> 3), m = m0 + wm * 64 + ml;
        if (m >= p.M) continue;
        const half8_t t = *reinterpret_cast<const half8_t *>(scratch + ml * EPI_PITCH + nl);
        half8_t res = {0, 0, 0, 0, 0, 0, 0, 0};
        if (EPI == MOON_EPI_BIAS_RESID) res = *reinterpret_cast<const half8_t *>(p.resid + size_t(m) * p.N + n);
        half8_t o;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            half_t v = apply_epilogue_v<EPI>((float)t[e], bias[e]); // (float)t[e] rounds back to t[e]: the matmul result as parked
            if (EPI == MOON_EPI_BIAS_RESID) v = (half_t)((float)res[e] + (float)v);
            o[e] = v;
        }
        *reinterpret_cast<half8_t *>(p.C + size_t(m) * p.N + n) = o;
    }
}

// A wavefront's 64x64 f32 partial tile of a split K, written in full lines the same way: half of the tile (32 rows m) at a
// time through 32 * 68 floats of LDS, four consecutive n per lane on the way out.  Needs N % 4 == 0.
template <int EPI, int MB = 2> // MB: 32-row blocks of m in the sub-tile, as in gemm_store_tile_lds
__device__ __forceinline__ void gemm_store_partial_lds(const GemmArgs &p, const float16_t (&acc)[2][MB], int m0, int n0, int wm, int wn, int lane,
                                                       int split, float *scratch) {
    const int frag_row = lane & 31, frag_g = lane >> 5;
    const int nl = (lane & 15) * 4, n = n0 + wn * 64 + nl;
#pragma unroll
    for (int mi = 0; mi < MB; mi++) {
#pragma unroll
        for (int ni = 0; ni < 2; ni++)
#pragma unroll
            for (int q = 0; q < 4; q++) {
                float4 o = {acc[ni][mi][4 * q], acc[ni][mi][4 * q + 1], acc[ni][mi][4 * q + 2], acc[ni][mi][4 * q + 3]};
                *reinterpret_cast<float4 *>(scratch + frag_row * EPI_PITCH + ni * 32 + 8 * q + 4 * frag_g) = o;
            }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if (n < p.N) {
#pragma unroll
            for (int r = 0; r < 8; r++) {
                const int ml = r * 4 + (lane >> 4), m = m0 + wm * 64 + mi * 32 + ml;
                if (m >= p.M) continue;
                *reinterpret_cast<float4 *>(p.partial + (size_t(split) * p.M + m) * p.N + n) = *reinterpret_cast<const float4 *>(scratch + ml * EPI_PITCH + nl);
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // the reads are done before the other half overwrites the rows
    }
}

template <int EPI>
__global__ __launch_bounds__(256) void gemm_nt_mfma_kernel(GemmArgs p) {
    __shared__ __attribute__((aligned(16))) half_t lds[2][2][TILE_HALFS]; // [buffer][operand: 0 = act (m), 1 = weight (n)]

    // XCD-aware tile order: consecutive workgroup ids land on different XCDs (round robin over 8), so give
    // each XCD a contiguous run of tiles that share weight column tiles in its own L2.
    const int tiles = p.tiles_m * p.tiles_n;
    const int total = tiles * p.splits;
    const int per_xcd = (total + 7) / 8;
    int wg = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
    if (wg >= total) return;
    const int split = wg / tiles;
    const int tile = wg % tiles;
    const int tn = tile / p.tiles_m, tm = tile % p.tiles_m;
    const int m0 = tm * BM, n0 = tn * BN;
    const int k_begin = split * p.k_per_split;
    const int k_end = min(p.K, k_begin + p.k_per_split);
    const int n_ktiles = (k_end - k_begin + BK - 1) / BK;

    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm = wave & 1, wn = wave >> 1;

    // staging assignment: granule c of rows r, r+32, r+64, r+96 of both operand tiles
    const int sc = t & 7, sr = t >> 3;
    const half_t *a_src[4], *w_src[4];
    int lds_off[4];
#pragma unroll
    for (int q = 0; q < 4; q++) {
        const int r = sr + 32 * q;
        a_src[q] = p.A + size_t(min(m0 + r, p.M - 1)) * p.K + sc * 8;
        w_src[q] = p.Bt + size_t(min(n0 + r, p.N - 1)) * p.K + sc * 8;
        lds_off[q] = r * BK + swz(r, sc) * 8;
    }

    uint4 ra[4], rw[4];
    auto load_tile = [&](int kt) {
        const int k = k_begin + kt * BK + sc * 8;
        const bool ok = k < k_end; // K % 8 == 0, so a granule is either fully inside or outside
#pragma unroll
        for (int q = 0; q < 4; q++) {
            ra[q] = make_uint4(0, 0, 0, 0);
            rw[q] = make_uint4(0, 0, 0, 0);
            if (ok) {
                ra[q] = *reinterpret_cast<const uint4 *>(a_src[q] + k_begin + kt * BK);
                rw[q] = *reinterpret_cast<const uint4 *>(w_src[q] + k_begin + kt * BK);
            }
        }
    };
    auto store_tile = [&](int buf) {
#pragma unroll
        for (int q = 0; q < 4; q++) {
            *reinterpret_cast<uint4 *>(&lds[buf][0][lds_off[q]]) = ra[q];
            *reinterpret_cast<uint4 *>(&lds[buf][1][lds_off[q]]) = rw[q];
        }
    };

    float16_t acc[2][2]; // [ni][mi]
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;

    const int frag_row = lane & 31, frag_g = lane >> 5;

    if (n_ktiles > 0) {
        load_tile(0);
        store_tile(0);
    }
    __syncthreads();

    for (int kt = 0; kt < n_ktiles; kt++) {
        const int buf = kt & 1;
        if (kt + 1 < n_ktiles) load_tile(kt + 1);
#pragma unroll
        for (int s = 0; s < BK / 16; s++) {
            half8_t fa[2], fw[2];
#pragma unroll
            for (int i = 0; i < 2; i++) {
                const int rm = wm * 64 + i * 32 + frag_row;
                const int rn = wn * 64 + i * 32 + frag_row;
                fa[i] = *reinterpret_cast<const half8_t *>(&lds[buf][0][rm * BK + swz(rm, 2 * s + frag_g) * 8]);
                fw[i] = *reinterpret_cast<const half8_t *>(&lds[buf][1][rn * BK + swz(rn, 2 * s + frag_g) * 8]);
            }
#pragma unroll
            for (int ni = 0; ni < 2; ni++)
#pragma unroll
                for (int mi = 0; mi < 2; mi++)
                    acc[ni][mi] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fw[ni], fa[mi], acc[ni][mi], 0, 0, 0);
        }
        if (kt + 1 < n_ktiles) store_tile(buf ^ 1);
        __syncthreads();
    }

    if (p.splits == 1 && p.N % 8 == 0 && p.lds_epilogue) // both staging buffers are free now
        gemm_store_tile_lds<EPI>(p, acc, m0, n0, wm, wn, lane, &lds[0][0][0] + size_t(t >> 6) * 64 * EPI_PITCH);
    else if (p.splits > 1 && p.N % 4 == 0 && p.lds_epilogue)
        gemm_store_partial_lds<EPI>(p, acc, m0, n0, wm, wn, lane, split, reinterpret_cast<float *>(&lds[0][0][0]) + size_t(t >> 6) * 32 * EPI_PITCH);
    else
        gemm_store_tile<EPI>(p, acc, m0, n0, wm, wn, frag_row, frag_g, split);
}

// The epilogue of the wavefront-specialised 128 x 128 kernel, shared by all eight wavefronts (the loaders have nothing
// else left to do, and with GELU the epilogue is VALU work): the multipliers park the whole tile in LDS as f16,
// [m][n] with a pitch of 136 halfs; after a barrier every thread takes eight consecutive n of four rows, applies the rest
// of the epilogue and stores 16 bytes (sixteen threads cover a 256-byte row segment).
constexpr int TILE_PITCH = 136;
__device__ __forceinline__ void gemm_park_tile(const float16_t (&acc)[2][2], int wm, int wn, int lane, half_t *scratch) {
    const int frag_row = lane & 31, frag_g = lane >> 5;
#pragma unroll
    for (int ni = 0; ni < 2; ni++)
#pragma unroll
        for (int mi = 0; mi < 2; mi++)
#pragma unroll
            for (int q = 0; q < 4; q++) {
                half4_t o;
#pragma unroll
                for (int e = 0; e < 4; e++) o[e] = (half_t)acc[ni][mi][4 * q + e];
                *reinterpret_cast<half4_t *>(scratch + (wm * 64 + mi * 32 + frag_row) * TILE_PITCH + wn * 64 + ni * 32 + 8 * q + 4 * frag_g) = o;
            }
}
template <int EPI, int ROWS = 128> // ROWS: rows of the parked tile (32 per pass of the 512 threads)
__device__ __forceinline__ void gemm_tile_out(const GemmArgs &p, int m0, int n0, int t, const half_t *scratch) {
    const int nl = (t & 15) * 8, n = n0 + nl;
    if (n >= p.N) return;
    half8_t bias = {0, 0, 0, 0, 0, 0, 0, 0};
    if (EPI >= MOON_EPI_BIAS) bias = *reinterpret_cast<const half8_t *>(p.bias + n);
#pragma unroll
    for (int r = 0; r < ROWS / 32; r++) {
        const int ml = r * 32 + (t >> 4), m = m0 + ml;
        if (m >= p.M) continue;
        const half8_t v = *reinterpret_cast<const half8_t *>(scratch + ml * TILE_PITCH + nl);
        half8_t res = {0, 0, 0, 0, 0, 0, 0, 0};
        if (EPI == MOON_EPI_BIAS_RESID) res = *reinterpret_cast<const half8_t *>(p.resid + size_t(m) * p.N + n);
        half8_t o;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            half_t x = apply_epilogue_v<EPI>((float)v[e], bias[e]); // (float)v[e] rounds back to v[e]: the matmul result as parked
            if (EPI == MOON_EPI_BIAS_RESID) x = (half_t)((float)res[e] + (float)x);
            o[e] = x;
        }
        *reinterpret_cast<half8_t *>(p.C + size_t(m) * p.N + n) = o;
    }
}

// gemm_tile_out for a qkv projection, with what qkv_rope_cache_vec_kernel does to the finished rows folded in (the same
// values, roundings and rotations: the results are the same bits), so that the projection never goes to memory unrotated.
// The tile's 128 columns are two whole heads of q, k or v (heads are 64 wide, tiles start at multiples of 128).  A thread
// finishes eight consecutive columns of a row; where those are rotated it also forms the eight partner values, rot_dim / 2
// further on or back in the same head, from the parked tile and their bias.
template <int ROWS>
__device__ __forceinline__ void gemm_tile_out_rope(const GemmArgs &p, int m0, int n0, int t, const half_t *scratch) {
    const int nl = (t & 15) * 8, n = n0 + nl, d0 = nl & 63; // d0: first of the eight columns within its head
    if (n >= p.N) return;
    const int hd = p.rope_H * 64;
    const int region = n / hd, head = (n - region * hd) >> 6; // 0: q, 1: k, 2: v
    const int half = p.rope_dim >> 1;
    const bool rotated = region < 2 && d0 < p.rope_dim, low = d0 < half;
    const int shift = low ? half : -half; // to the partner's columns (where rotated)
    const half8_t bias = *reinterpret_cast<const half8_t *>(p.bias + n);
    half8_t biasp = bias;
    if (rotated) biasp = *reinterpret_cast<const half8_t *>(p.bias + n + shift);
    half_t *dst0 = (region == 0 ? p.rope_q + size_t(head) * p.M * 64 : (region == 1 ? p.rope_ck : p.rope_cv) + (size_t(head) * p.rope_max_seq + p.rope_pos0) * 64) + d0;
#pragma unroll
    for (int r = 0; r < ROWS / 32; r++) {
        const int ml = r * 32 + (t >> 4), m = m0 + ml;
        if (m >= p.M) continue;
        const half8_t v = *reinterpret_cast<const half8_t *>(scratch + ml * TILE_PITCH + nl);
        half8_t o;
#pragma unroll
        for (int e = 0; e < 8; e++) o[e] = apply_epilogue_v<MOON_EPI_BIAS>((float)v[e], bias[e]);
        if (rotated) {
            const half8_t vp = *reinterpret_cast<const half8_t *>(scratch + ml * TILE_PITCH + nl + shift);
            const float4 *tab = reinterpret_cast<const float4 *>(p.rope_table + ((size_t)(p.rope_pos0 + m) * half + (low ? d0 : d0 - half)) * 2);
#pragma unroll
            for (int e4 = 0; e4 < 4; e4++) {
                const float4 cs = tab[e4]; // (cos, sin) of two consecutive d
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    const int e = 2 * e4 + j;
                    const float c = j ? cs.z : cs.x, sn = j ? cs.w : cs.y;
                    const half_t mine = o[e], other = apply_epilogue_v<MOON_EPI_BIAS>((float)vp[e], biasp[e]);
                    half_t a, b;
                    if (low) {
                        rotate_pair((float)mine, (float)other, c, sn, a, b);
                        o[e] = a;
                    } else {
                        rotate_pair((float)other, (float)mine, c, sn, a, b);
                        o[e] = b;
                    }
                }
            }
        }
        *reinterpret_cast<half8_t *>(dst0 + size_t(m) * 64) = o;
    }
}

// The same tile computation, specialised by wavefront.  A 512-thread workgroup holds four LOADER wavefronts and four
// MULTIPLIER wavefronts, one of each per SIMD, so the hardware interleaves their instruction streams:
//   * loaders copy the operand tiles global -> LDS with buffer_load_dwordx4 ... lds (every lane names a 16-byte source,
//     the 64 destinations are consecutive in LDS; no registers are spent on staging).  DMA_STAGES - 1 k-tiles (96 KiB) are
//     in flight per workgroup.  The XOR swizzle moves to the source side: the lane that fills physical granule pg of row
//     r fetches logical granule pg ^ ((r >> 1) & 7).  A wavefront's loads retire in order, so "at most 8*n outstanding"
//     means its part of the tile n behind the newest has landed.
//   * multipliers only read operand slices from LDS and issue MFMAs, software pipelined across slices and k-tiles.
// One barrier per k-tile, executed by all eight wavefronts, publishes tile kt+1 (loaders arrive once it has landed) and
// frees the buffer of tile kt (multipliers arrive once they have read it); the loaders then refill that buffer.
// The tile moves 32 KiB per k-tile for 16 MFMAs per SIMD (0.26 us at the ~2 GHz the clock settles at under MFMA load),
// i.e. needs ~125 B/ns from the CU's load path, which is about what that path delivers from the L2.
// Needs K % 16 == 0: a partial last k-tile runs fewer 16-wide steps; what its copies fetch beyond K is never multiplied.
constexpr int DMA_STAGES = 4;
constexpr int DMA_THREADS = 512;
constexpr size_t DMA_LDS_BYTES = size_t(DMA_STAGES) * 2 * TILE_HALFS * sizeof(half_t);

// BKN: the second operand is [K, N] (hgemm.zig's layout) and is read as it lies.  Its tile sits in LDS as [k][128 n]; a
// loader instruction copies four k-rows of 256 bytes, the 16-byte granules of row r XOR-ed with 2 * (r & 3) on the source
// side, and the multipliers fetch their operand slices with the transposing LDS load (ds_read_b64_tr_b16: the 16 lanes of a
// quarter-wavefront name a 4 x 16 block, four halfs each, and lane i receives column i of its four rows), two per slice in
// place of one 16-byte read.  Same products in the same order as with the [N, K] operand: the same bits.  Needs N % 8 == 0.
template <int EPI, bool BKN = false>
__global__ __launch_bounds__(DMA_THREADS) void gemm_nt_dma_kernel(GemmArgs p) {
    extern __shared__ __attribute__((aligned(16))) half_t lds_dma[]; // [stage][operand: 0 = act (m), 1 = weight (n)][TILE_HALFS]

    const int tiles = p.tiles_m * p.tiles_n;
    const int total = tiles * p.splits;
    const int per_xcd = (total + 7) / 8;
    int wg = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
    if (wg >= total) return;
    const int split = wg / tiles;
    const int tile = wg % tiles;
    const int tn = tile / p.tiles_m, tm = tile % p.tiles_m;
    const int m0 = tm * BM, n0 = tn * BN;
    const int k_begin = split * p.k_per_split;
    const int k_end = min(p.K, k_begin + p.k_per_split);
    const int n_ktiles = (k_end - k_begin + BK - 1) / BK;
    if (n_ktiles <= 0) return;

    const int t = threadIdx.x, lane = t & 63;
    const int role_wave = (t >> 6) & 3; // index within the role
    const bool loader = t >= 256;

    if (loader) {
        // this wavefront fills rows [32*role_wave, +32) of both tiles, 8 rows per instruction.  The copies use the buffer
        // form: a scalar descriptor of the whole operand, one 32-bit offset register per lane (fixed over the k-tiles) and
        // a scalar offset for the k-tile.  With 64-bit addresses in registers (two per lane) the copies of a wavefront
        // whose SIMD also feeds the matrix core ran at half their rate (measured 66 against 117 B/ns per CU).  Reads past
        // the end of the operand return zero, so a partial last k-tile needs no clamping (what lies beyond K is never
        // multiplied).
        int off_a[4], off_w[4]; // byte offset of the granule this lane fetches, at k = 0
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int r = 32 * role_wave + 8 * j + (lane >> 3);
            const int g8 = swz(r, lane & 7) * 8;
            off_a[j] = (min(m0 + r, p.M - 1) * p.K + g8) * 2;
            off_w[j] = (min(n0 + r, p.N - 1) * p.K + g8) * 2;
            if (BKN) { // k-rows 16 * role_wave + 4 * j .. + 3 of the tile: lane -> (row, physical granule); columns past N are never stored
                const int rk = 16 * role_wave + 4 * j + (lane >> 4), pg = lane & 15;
                off_w[j] = (rk * p.N + n0 + (pg ^ (2 * (rk & 3))) * 8) * 2;
            }
        }
        auto issue = [&](int kt) {
            half_t *stage = lds_dma + size_t(kt % DMA_STAGES) * 2 * TILE_HALFS;
            // the k-tile enters through the descriptors' base and size: the range check that turns reads past the end of the
            // operand into zeros does not see an instruction's scalar offset
            const int k_off = (k_begin + kt * BK) * 2;
            const int kw_off = BKN ? (k_begin + kt * BK) * p.N * 2 : k_off; // (rows of [K, N] past K lie past the end: zeros)
            const __amdgpu_buffer_rsrc_t rs_a =
                __builtin_amdgcn_make_buffer_rsrc(const_cast<char *>(reinterpret_cast<const char *>(p.A)) + k_off, 0, p.a_bytes - k_off, 0x00020000);
            const __amdgpu_buffer_rsrc_t rs_w =
                __builtin_amdgcn_make_buffer_rsrc(const_cast<char *>(reinterpret_cast<const char *>(p.Bt)) + kw_off, 0, p.bt_bytes - kw_off, 0x00020000);
#pragma unroll
            for (int j = 0; j < 4; j++) {
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_a, (__attribute__((address_space(3))) void *)(stage + (32 * role_wave + 8 * j) * BK), 16,
                                                         off_a[j], 0, 0, 0);
                __builtin_amdgcn_raw_ptr_buffer_load_lds(
                    rs_w, (__attribute__((address_space(3))) void *)(stage + TILE_HALFS + (32 * role_wave + 8 * j) * BK), 16, off_w[j], 0, 0, 0);
            }
        };
        int issued = 0; // k-tiles whose copies have been issued
        // this wavefront's part of tile kt has landed once at most 8 * (issued - 1 - kt) of its copies are outstanding
        auto wait_tile = [&](int kt) {
            const int newer = issued - 1 - kt;
            if (newer >= 2) wait_vmcnt<16>();
            else if (newer == 1) wait_vmcnt<8>();
            else wait_vmcnt<0>();
        };
        for (; issued < DMA_STAGES - 1 && issued < n_ktiles; issued++) issue(issued);
        wait_tile(0);
        lds_barrier(); // tile 0 is visible
        for (int kt = 0; kt < n_ktiles; kt++) {
            // past the barrier that published tile kt nobody reads tile kt-1 any more: its buffer takes tile kt + DMA_STAGES - 1
            if (issued < n_ktiles) {
                issue(issued);
                issued++;
            }
            if (kt + 1 < n_ktiles) {
                wait_tile(kt + 1);
                lds_barrier(); // publishes tile kt+1
            }
        }
        if (!(p.splits == 1 && p.N % 8 == 0 && p.lds_epilogue)) return;
        // the loaders take their half of the epilogue once the multipliers have parked the tile
        const int last = (n_ktiles - 1) % DMA_STAGES, free0 = last == 0 ? 1 : last == 1 ? 2 : 0;
        lds_barrier();
        gemm_tile_out<EPI>(p, m0, n0, t, lds_dma + size_t(free0) * 2 * TILE_HALFS);
        return;
    }

    const int wm = role_wave & 1, wn = role_wave >> 1;
    const int frag_row = lane & 31, frag_g = lane >> 5;
    float16_t acc[2][2]; // [ni][mi]
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;

    // LDS byte offsets (within a stage) of this lane's operand slices: [16-wide step][row block]
    unsigned off_a[BK / 16][2], off_w[BK / 16][2];
#pragma unroll
    for (int s = 0; s < BK / 16; s++)
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const int rm = wm * 64 + i * 32 + frag_row;
            const int rn = wn * 64 + i * 32 + frag_row;
            off_a[s][i] = (rm * BK + swz(rm, 2 * s + frag_g) * 8) * 2;
            off_w[s][i] = (TILE_HALFS + rn * BK + swz(rn, 2 * s + frag_g) * 8) * 2;
        }
    // BKN: where this lane points the transposing loads of n-block ni, for the first four k of its slice of step 0 (step s and
    // the second four add (16 s + 4 q) rows of 256 bytes): row 8 * frag_g + i / 4, columns 4 * (i % 4) .. + 3 of the 16 the
    // lane's quarter-wavefront covers, i = lane % 16
    unsigned off_wk[2];
#pragma unroll
    for (int ni = 0; ni < 2; ni++) {
        const int i = lane & 15, row = 8 * frag_g + (i >> 2);
        const int c = wn * 8 + ni * 4 + ((lane >> 4) & 1) * 2 + ((i & 3) >> 1); // 16-byte granule of the row
        off_wk[ni] = (TILE_HALFS + row * BN + (c ^ (2 * (row & 3))) * 8 + (i & 1) * 4) * 2;
    }
    // The operand reads and the waits for them are written out by hand.  Left to the compiler the reads sink below the
    // MFMAs of the step before (into the registers those just consumed) and are waited for at once, and the wait at the
    // head of the loop is for everything outstanding, so the LDS latency is paid several times per k-tile with the matrix
    // core idle.  The compiler does not count reads issued from asm statements, so it adds no waits of its own for them;
    // each wait statement names the registers it guards as operands, which keeps their use behind it.
    constexpr unsigned STAGE_BYTES = 2 * TILE_HALFS * sizeof(half_t);
    // (BKN: fw[ni] arrives as two 8-byte halves, wk[ni][0..1])
    struct Frag {
        half8_t fa[2], fw[2];
        half4_t wk[2][2];
    };
    auto read_frags = [&](int kt, int s, Frag &f) {
        const unsigned sb = unsigned(kt % DMA_STAGES) * STAGE_BYTES;
#pragma unroll
        for (int i = 0; i < 2; i++) {
            asm volatile("ds_read_b128 %0, %1" : "=v"(f.fa[i]) : "v"(sb + off_a[s][i]));
            if (!BKN) asm volatile("ds_read_b128 %0, %1" : "=v"(f.fw[i]) : "v"(sb + off_w[s][i]));
            else {
#pragma unroll
                for (int q = 0; q < 2; q++)
                    asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(f.wk[i][q]) : "v"(sb + off_wk[i] + unsigned(16 * s + 4 * q) * (BN * 2)));
            }
        }
    };
    // all but the newest group of reads (the one issued last: four reads, six with BKN) have landed; f belongs to an older group
    auto wait_older = [&](Frag &f) {
        if (!BKN) asm volatile("s_waitcnt lgkmcnt(4)" : "+v"(f.fa[0]), "+v"(f.fa[1]), "+v"(f.fw[0]), "+v"(f.fw[1])::"memory");
        else
            asm volatile("s_waitcnt lgkmcnt(6)" : "+v"(f.fa[0]), "+v"(f.fa[1]), "+v"(f.wk[0][0]), "+v"(f.wk[0][1]), "+v"(f.wk[1][0]), "+v"(f.wk[1][1])::"memory");
    };
    auto wait_all = [&](Frag &f) {
        if (!BKN) asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(f.fa[0]), "+v"(f.fa[1]), "+v"(f.fw[0]), "+v"(f.fw[1])::"memory");
        else
            asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(f.fa[0]), "+v"(f.fa[1]), "+v"(f.wk[0][0]), "+v"(f.wk[0][1]), "+v"(f.wk[1][0]), "+v"(f.wk[1][1])::"memory");
    };
    auto multiply = [&](const Frag &f) {
#pragma unroll
        for (int ni = 0; ni < 2; ni++) {
            const half8_t w = BKN ? __builtin_shufflevector(f.wk[ni][0], f.wk[ni][1], 0, 1, 2, 3, 4, 5, 6, 7) : f.fw[ni];
#pragma unroll
            for (int mi = 0; mi < 2; mi++) acc[ni][mi] = __builtin_amdgcn_mfma_f32_32x32x16_f16(w, f.fa[mi], acc[ni][mi], 0, 0, 0);
        }
    };

    Frag fr[2];
    lds_barrier(); // tile 0 is visible
    read_frags(0, 0, fr[0]);
    // At the top of a k-tile the reads of its first slice into fr[0] are in flight.  Every slice is requested one
    // step (four MFMAs) before it is multiplied; the barrier that publishes tile kt+1 (and hands the buffer of tile kt
    // back to the loaders, hence the wait for this wavefront's last reads of it) is passed with the MFMAs of the third
    // slice queued, and the first slice of tile kt+1 is fetched under the MFMAs of the fourth.
    // Full k-tiles with a successor first, in a loop of one basic block; then the last tile, full or partial (with the
    // partial tile as a second path inside the loop the accumulators end up in different registers on the two paths and
    // are copied, 64 registers each way, every iteration, with the matrix core drained in between).  The scheduling
    // fences keep the MFMAs of a step where they are written: between the reads of the next slice and the wait for it.
    const int last_steps = ((k_end - k_begin) - (n_ktiles - 1) * BK) / 16; // 16-wide steps of the last k-tile (1..4)
    auto first_three = [&](int kt) {
        read_frags(kt, 1, fr[1]);
        wait_older(fr[0]);
        multiply(fr[0]);
        __builtin_amdgcn_sched_barrier(0);
        read_frags(kt, 2, fr[0]);
        wait_older(fr[1]);
        multiply(fr[1]);
        __builtin_amdgcn_sched_barrier(0);
        read_frags(kt, 3, fr[1]);
        wait_older(fr[0]);
        multiply(fr[0]);
        __builtin_amdgcn_sched_barrier(0);
    };
    for (int kt = 0; kt + 1 < n_ktiles; kt++) {
        first_three(kt);
        wait_all(fr[1]);
        __builtin_amdgcn_s_barrier();
        read_frags(kt + 1, 0, fr[0]);
        multiply(fr[1]);
        __builtin_amdgcn_sched_barrier(0);
    }
    if (last_steps == BK / 16) {
        first_three(n_ktiles - 1);
        wait_all(fr[1]);
        multiply(fr[1]);
    } else { // fr[0] will hold its first slice
        wait_all(fr[0]);
        multiply(fr[0]);
        for (int s = 1; s < last_steps; s++) {
            read_frags(n_ktiles - 1, s, fr[0]);
            wait_all(fr[0]);
            multiply(fr[0]);
        }
    }
    if (p.splits == 1 && p.N % 8 == 0 && p.lds_epilogue) {
        // two neighbouring stages that the last k-tile does not occupy (every copy into them has landed)
        const int last = (n_ktiles - 1) % DMA_STAGES, free0 = last == 0 ? 1 : last == 1 ? 2 : 0;
        half_t *scratch = lds_dma + size_t(free0) * 2 * TILE_HALFS; // 128 x 136 halfs: 34 KiB of the two free stages
        gemm_park_tile(acc, wm, wn, lane, scratch);
        lds_barrier(); // all eight wavefronts: the tile is parked
        gemm_tile_out<EPI>(p, m0, n0, t, scratch);
    } else if (p.splits > 1 && p.N % 4 == 0 && p.lds_epilogue) {
        const int last = (n_ktiles - 1) % DMA_STAGES, free0 = last == 0 ? 1 : last == 1 ? 2 : 0;
        gemm_store_partial_lds<EPI>(p, acc, m0, n0, wm, wn, lane, split,
                                    reinterpret_cast<float *>(lds_dma + size_t(free0) * 2 * TILE_HALFS) + size_t(role_wave) * 32 * EPI_PITCH);
    } else
        gemm_store_tile<EPI>(p, acc, m0, n0, wm, wn, frag_row, frag_g, split);
}

// The wavefront-specialised kernel on a 256 (m) x 128 (n) x 64 tile, for shapes with more 128 x 128 tiles than CUs.
// While a SIMD's matrix core is kept busy its wavefronts' vector loads run at about half their usual rate (measured:
// ~65 B/ns per CU against ~125 B/ns), so a 128 x 128 tile, which needs 512 bytes per MFMA, cannot keep the matrix cores
// more than half busy; this tile needs 384.  Four multiplier wavefronts in a 2 (m) x 2 (n) grid own 128 x 64 sub-tiles
// (4 x 2 accumulators of 32 x 32, 128 registers), four loader wavefronts copy the 48 KiB of a k-tile (12 instructions
// each), three stages (144 KiB, two k-tiles in flight).  Needs K % 64 == 0, N % 8 == 0, 16-byte aligned rows of C / bias
// / resid, no split of K.  MI = 3 is the same kernel on a 192 x 128 tile (multipliers own 96 x 64): M = 768 splits into
// four row blocks instead of three, which fills more CUs.
constexpr int DMA2_STAGES = 3;
template <int MI> struct Dma2 {
    static constexpr int BM2 = 64 * MI;
    static constexpr int STAGE2_HALFS = (BM2 + BN) * BK;
    static constexpr size_t LDS_BYTES = size_t(DMA2_STAGES) * STAGE2_HALFS * sizeof(half_t);
    static constexpr int A_LOADS = 2 * MI; // copies of activation rows per loader wavefront and k-tile (8 rows each)
};

// PARTIAL: the workgroup multiplies k-tiles [kt0, kt0 + n_ktiles) of tile `wg` only and leaves the f32 sums in slab `split` of
// p.partial (no epilogue); otherwise the whole of K, and wg is taken from the workgroup index.
// ROPE: the epilogue of a qkv projection that writes the rotated q and the cache rows (gemm_tile_out_rope) instead of C.
// BKN: the second operand is [K, N], read in place as in gemm_nt_dma_kernel<EPI, true>.
template <int EPI, int MI, bool PARTIAL = false, bool ROPE = false, bool BKN = false>
__device__ __forceinline__ void gemm_nt_dma2_body(const GemmArgs &p, int wg_arg = 0, int kt0 = 0, int n_ktiles_arg = 0, int split = 0) {
    static_assert(MI == 3 || MI == 4, "192- or 256-row tiles");
    static_assert(!PARTIAL || EPI == MOON_EPI_NONE, "partial sums take no epilogue");
    static_assert(!ROPE || (EPI == MOON_EPI_BIAS && !PARTIAL), "the rotating epilogue follows a bias");
    constexpr int BM2 = Dma2<MI>::BM2, STAGE2_HALFS = Dma2<MI>::STAGE2_HALFS, A_LOADS = Dma2<MI>::A_LOADS;
    constexpr bool SHARED_EPILOGUE = (EPI == MOON_EPI_BIAS_GELU || ROPE) && !PARTIAL; // all eight wavefronts finish the tile
    static_assert(size_t(BM2) * TILE_PITCH <= size_t(DMA2_STAGES) * STAGE2_HALFS, "the parked tile fits the staging area");
    extern __shared__ __attribute__((aligned(16))) half_t lds2[]; // [stage][act: 256 rows | weight: 128 rows][64 halfs]

    const int total = p.tiles_m * p.tiles_n;
    const int per_xcd = (total + 7) / 8;
    // (workgroup id -> tile as in the 128 x 128 kernel: the ids an XCD receives cover a contiguous run of tiles)
    const int wg = PARTIAL ? wg_arg : (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
    if (wg >= total) return;
    const int tn = wg / p.tiles_m, tm = wg % p.tiles_m;
    const int m0 = tm * BM2, n0 = tn * BN;
    const int n_ktiles = PARTIAL ? n_ktiles_arg : p.K / BK;

    const int t = threadIdx.x, lane = t & 63;
    const int role_wave = (t >> 6) & 3;
    const bool loader = t >= 256;

    if (loader) {
        // this wavefront fills activation rows [16*MI*role_wave, +16*MI) and weight rows [32*role_wave, +32), 8 rows per
        // instruction (buffer form: scalar descriptor, one offset register per lane, scalar k offset)
        const __amdgpu_buffer_rsrc_t rs_a = __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t *>(p.A), 0, p.a_bytes, 0x00020000);
        const __amdgpu_buffer_rsrc_t rs_w = __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t *>(p.Bt), 0, p.bt_bytes, 0x00020000);
        int off_a[A_LOADS], off_w[4];
#pragma unroll
        for (int j = 0; j < A_LOADS; j++) {
            const int r = 16 * MI * role_wave + 8 * j + (lane >> 3);
            off_a[j] = (min(m0 + r, p.M - 1) * p.K + swz(r, lane & 7) * 8) * 2;
        }
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int r = 32 * role_wave + 8 * j + (lane >> 3);
            off_w[j] = (min(n0 + r, p.N - 1) * p.K + swz(r, lane & 7) * 8) * 2;
            if (BKN) { // k-rows 16 * role_wave + 4 * j .. + 3 of the tile; columns past N re-read the row's last granule and are never stored
                const int rk = 16 * role_wave + 4 * j + (lane >> 4), pg = lane & 15;
                off_w[j] = (rk * p.N + min(n0 + (pg ^ (2 * (rk & 3))) * 8, p.N - 8)) * 2;
            }
        }
        auto issue = [&](int kt) {
            half_t *stage = lds2 + size_t(kt % DMA2_STAGES) * STAGE2_HALFS;
            const int k_off = (kt0 + kt) * BK * 2;
            const int kw_off = BKN ? (kt0 + kt) * BK * p.N * 2 : k_off;
#pragma unroll
            for (int j = 0; j < A_LOADS; j++)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_a, (__attribute__((address_space(3))) void *)(stage + (16 * MI * role_wave + 8 * j) * BK),
                                                         16, off_a[j], k_off, 0, 0);
#pragma unroll
            for (int j = 0; j < 4; j++)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(
                    rs_w, (__attribute__((address_space(3))) void *)(stage + BM2 * BK + (32 * role_wave + 8 * j) * BK), 16, off_w[j], kw_off, 0, 0);
        };
        int issued = 0;
        // this wavefront's part of tile kt has landed once at most (A_LOADS + 4) * (issued - 1 - kt) of its copies are outstanding
        auto wait_tile = [&](int kt) {
            if (issued - 1 - kt >= 1) wait_vmcnt<A_LOADS + 4>();
            else wait_vmcnt<0>();
        };
        for (; issued < DMA2_STAGES - 1 && issued < n_ktiles; issued++) issue(issued);
        wait_tile(0);
        lds_barrier(); // tile 0 is visible
        for (int kt = 0; kt < n_ktiles; kt++) {
            if (issued < n_ktiles) { // the buffer of tile kt-1 is free past the barrier that published tile kt
                issue(issued);
                issued++;
            }
            if (kt + 1 < n_ktiles) {
                wait_tile(kt + 1);
                lds_barrier(); // publishes tile kt+1
            }
        }
        if constexpr (SHARED_EPILOGUE) { // the loaders take their half of the epilogue (see the multipliers' end)
            lds_barrier();               // the multipliers have read the last k-tile
            lds_barrier();               // ... and parked the tile
            if constexpr (ROPE) gemm_tile_out_rope<BM2>(p, m0, n0, t, lds2);
            else gemm_tile_out<EPI, BM2>(p, m0, n0, t, lds2);
        }
        return;
    }

    const int wm = role_wave & 1, wn = role_wave >> 1;
    const int frag_row = lane & 31, frag_g = lane >> 5;
    float16_t acc[2][MI]; // [ni][mi]
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < MI; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;

    unsigned off_a[BK / 16][MI], off_w[BK / 16][2]; // LDS byte offsets (within a stage) of this lane's operand slices
#pragma unroll
    for (int s = 0; s < BK / 16; s++) {
#pragma unroll
        for (int i = 0; i < MI; i++) {
            const int rm = wm * 32 * MI + i * 32 + frag_row;
            off_a[s][i] = (rm * BK + swz(rm, 2 * s + frag_g) * 8) * 2;
        }
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const int rn = wn * 64 + i * 32 + frag_row;
            off_w[s][i] = (BM2 * BK + rn * BK + swz(rn, 2 * s + frag_g) * 8) * 2;
        }
    }
    unsigned off_wk[2]; // BKN: see gemm_nt_dma_kernel
#pragma unroll
    for (int ni = 0; ni < 2; ni++) {
        const int i = lane & 15, row = 8 * frag_g + (i >> 2);
        const int c = wn * 8 + ni * 4 + ((lane >> 4) & 1) * 2 + ((i & 3) >> 1);
        off_wk[ni] = (BM2 * BK + row * BN + (c ^ (2 * (row & 3))) * 8 + (i & 1) * 4) * 2;
    }
    // (reads and waits by hand, as in the 128 x 128 kernel: MI + 2 reads per slice, one slice ahead of its 2 * MI MFMAs)
    constexpr unsigned STAGE_BYTES = STAGE2_HALFS * sizeof(half_t);
    struct Frag {
        half8_t fa[MI], fw[2];
        half4_t wk[2][2]; // BKN: fw[ni] arrives as two 8-byte halves
    };
    auto read_frags = [&](int kt, int s, Frag &f) {
        const unsigned sb = unsigned(kt % DMA2_STAGES) * STAGE_BYTES;
#pragma unroll
        for (int i = 0; i < MI; i++) asm volatile("ds_read_b128 %0, %1" : "=v"(f.fa[i]) : "v"(sb + off_a[s][i]));
#pragma unroll
        for (int i = 0; i < 2; i++) {
            if (!BKN) asm volatile("ds_read_b128 %0, %1" : "=v"(f.fw[i]) : "v"(sb + off_w[s][i]));
            else {
#pragma unroll
                for (int q = 0; q < 2; q++)
                    asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(f.wk[i][q]) : "v"(sb + off_wk[i] + unsigned(16 * s + 4 * q) * (BN * 2)));
            }
        }
    };
    // (all but the newest group of reads have landed: MI + 2 reads a group, MI + 4 with BKN)
    auto wait_older = [&](Frag &f) {
        if constexpr (!BKN) {
            if constexpr (MI == 4)
                asm volatile("s_waitcnt lgkmcnt(6)" : "+v"(f.fa[0]), "+v"(f.fa[1]), "+v"(f.fa[2]), "+v"(f.fa[MI - 1]), "+v"(f.fw[0]), "+v"(f.fw[1])::"memory");
            else
                asm volatile("s_waitcnt lgkmcnt(5)" : "+v"(f.fa[0]), "+v"(f.fa[1]), "+v"(f.fa[2]), "+v"(f.fw[0]), "+v"(f.fw[1])::"memory");
        } else {
            if constexpr (MI == 4)
                asm volatile("s_waitcnt lgkmcnt(8)" : "+v"(f.fa[0]), "+v"(f.fa[1]), "+v"(f.fa[2]), "+v"(f.fa[MI - 1]), "+v"(f.wk[0][0]), "+v"(f.wk[0][1]), "+v"(f.wk[1][0]), "+v"(f.wk[1][1])::"memory");
            else
                asm volatile("s_waitcnt lgkmcnt(7)" : "+v"(f.fa[0]), "+v"(f.fa[1]), "+v"(f.fa[2]), "+v"(f.wk[0][0]), "+v"(f.wk[0][1]), "+v"(f.wk[1][0]), "+v"(f.wk[1][1])::"memory");
        }
    };
    auto wait_all = [&](Frag &f) {
        if constexpr (!BKN) {
            if constexpr (MI == 4)
                asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(f.fa[0]), "+v"(f.fa[1]), "+v"(f.fa[2]), "+v"(f.fa[MI - 1]), "+v"(f.fw[0]), "+v"(f.fw[1])::"memory");
            else
                asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(f.fa[0]), "+v"(f.fa[1]), "+v"(f.fa[2]), "+v"(f.fw[0]), "+v"(f.fw[1])::"memory");
        } else {
            if constexpr (MI == 4)
                asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(f.fa[0]), "+v"(f.fa[1]), "+v"(f.fa[2]), "+v"(f.fa[MI - 1]), "+v"(f.wk[0][0]), "+v"(f.wk[0][1]), "+v"(f.wk[1][0]), "+v"(f.wk[1][1])::"memory");
            else
                asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(f.fa[0]), "+v"(f.fa[1]), "+v"(f.fa[2]), "+v"(f.wk[0][0]), "+v"(f.wk[0][1]), "+v"(f.wk[1][0]), "+v"(f.wk[1][1])::"memory");
        }
    };
    auto multiply = [&](const Frag &f) {
        half8_t w[2];
#pragma unroll
        for (int ni = 0; ni < 2; ni++) w[ni] = BKN ? __builtin_shufflevector(f.wk[ni][0], f.wk[ni][1], 0, 1, 2, 3, 4, 5, 6, 7) : f.fw[ni];
#pragma unroll
        for (int mi = 0; mi < MI; mi++)
#pragma unroll
            for (int ni = 0; ni < 2; ni++) acc[ni][mi] = __builtin_amdgcn_mfma_f32_32x32x16_f16(w[ni], f.fa[mi], acc[ni][mi], 0, 0, 0);
    };

    Frag fr[2];
    lds_barrier(); // tile 0 is visible
    read_frags(0, 0, fr[0]);
    auto first_three = [&](int kt) {
        read_frags(kt, 1, fr[1]);
        wait_older(fr[0]);
        multiply(fr[0]);
        __builtin_amdgcn_sched_barrier(0);
        read_frags(kt, 2, fr[0]);
        wait_older(fr[1]);
        multiply(fr[1]);
        __builtin_amdgcn_sched_barrier(0);
        read_frags(kt, 3, fr[1]);
        wait_older(fr[0]);
        multiply(fr[0]);
        __builtin_amdgcn_sched_barrier(0);
    };
    for (int kt = 0; kt + 1 < n_ktiles; kt++) { // (every k-tile is a full one)
        first_three(kt);
        wait_all(fr[1]);
        __builtin_amdgcn_s_barrier();
        read_frags(kt + 1, 0, fr[0]);
        multiply(fr[1]);
        __builtin_amdgcn_sched_barrier(0);
    }
    first_three(n_ktiles - 1);
    wait_all(fr[1]);
    multiply(fr[1]);
    if constexpr (SHARED_EPILOGUE) {
        // With GELU the epilogue is VALU work and the loaders have nothing left to do: the multipliers park the whole tile in
        // LDS as f16 ([m][n], pitch 136 halfs, from the start of the staging area, which is free once every multiplier has
        // read the last k-tile), and all eight wavefronts finish it, eight consecutive n of BM2 / 32 rows per thread.
        lds_barrier();
#pragma unroll
        for (int ni = 0; ni < 2; ni++)
#pragma unroll
            for (int mi = 0; mi < MI; mi++)
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    half4_t o;
#pragma unroll
                    for (int e = 0; e < 4; e++) o[e] = (half_t)acc[ni][mi][4 * q + e];
                    *reinterpret_cast<half4_t *>(lds2 + (wm * 32 * MI + mi * 32 + frag_row) * TILE_PITCH + wn * 64 + ni * 32 + 8 * q + 4 * frag_g) = o;
                }
        lds_barrier();
        if constexpr (ROPE) gemm_tile_out_rope<BM2>(p, m0, n0, t, lds2);
        else gemm_tile_out<EPI, BM2>(p, m0, n0, t, lds2);
        return;
    }
    if constexpr (PARTIAL) {
        // the stage after the last k-tile's is free (every copy into it has landed and been read): 32 x 68 floats per wavefront
        float *fscratch = reinterpret_cast<float *>(lds2 + size_t(n_ktiles % DMA2_STAGES) * STAGE2_HALFS) + size_t(role_wave) * 32 * EPI_PITCH;
        static_assert(size_t(4) * 32 * EPI_PITCH * sizeof(float) <= size_t(STAGE2_HALFS) * sizeof(half_t), "the four wavefronts' slots fit a stage");
        {
            float16_t part[2][2];
#pragma unroll
            for (int ni = 0; ni < 2; ni++)
#pragma unroll
                for (int mi = 0; mi < 2; mi++) part[ni][mi] = acc[ni][mi];
            gemm_store_partial_lds<EPI>(p, part, m0 + wm * 32 * MI - wm * 64, n0, wm, wn, lane, split, fscratch);
        }
        if constexpr (MI == 4) {
            float16_t part[2][2];
#pragma unroll
            for (int ni = 0; ni < 2; ni++)
#pragma unroll
                for (int mi = 0; mi < 2; mi++) part[ni][mi] = acc[ni][MI - 2 + mi];
            gemm_store_partial_lds<EPI>(p, part, m0 + wm * 32 * MI + 64 - wm * 64, n0, wm, wn, lane, split, fscratch);
        } else {
            float16_t part[2][1];
#pragma unroll
            for (int ni = 0; ni < 2; ni++) part[ni][0] = acc[ni][MI - 1];
            gemm_store_partial_lds<EPI, 1>(p, part, m0 + wm * 32 * MI + 64 - wm * 64, n0, wm, wn, lane, split, fscratch);
        }
        return;
    }
    // the stage after the last k-tile's is free (every copy into it has landed and been read): 64 x 68 halfs per wavefront
    half_t *scratch = lds2 + size_t(n_ktiles % DMA2_STAGES) * STAGE2_HALFS + size_t(role_wave) * 64 * EPI_PITCH;
    { // the first 64 rows of the sub-tile
        float16_t part[2][2];
#pragma unroll
        for (int ni = 0; ni < 2; ni++)
#pragma unroll
            for (int mi = 0; mi < 2; mi++) part[ni][mi] = acc[ni][mi];
        gemm_store_tile_lds<EPI>(p, part, m0 + wm * 32 * MI - wm * 64, n0, wm, wn, lane, scratch);
    }
    if constexpr (MI == 4) { // the other 64
        float16_t part[2][2];
#pragma unroll
        for (int ni = 0; ni < 2; ni++)
#pragma unroll
            for (int mi = 0; mi < 2; mi++) part[ni][mi] = acc[ni][MI - 2 + mi];
        gemm_store_tile_lds<EPI>(p, part, m0 + wm * 32 * MI + 64 - wm * 64, n0, wm, wn, lane, scratch);
    } else { // the other 32
        float16_t part[2][1];
#pragma unroll
        for (int ni = 0; ni < 2; ni++) part[ni][0] = acc[ni][MI - 1];
        gemm_store_tile_lds<EPI, 1>(p, part, m0 + wm * 32 * MI + 64 - wm * 64, n0, wm, wn, lane, scratch);
    }
}

// (the two tile heights as kernels of their own with one template parameter, like the other kernels of this file)
template <int EPI, bool BKN = false>
__global__ __launch_bounds__(DMA_THREADS) void gemm_nt_dma256_kernel(GemmArgs p) {
    gemm_nt_dma2_body<EPI, 4, false, false, BKN>(p);
}
template <int EPI, bool BKN = false>
__global__ __launch_bounds__(DMA_THREADS) void gemm_nt_dma192_kernel(GemmArgs p) {
    gemm_nt_dma2_body<EPI, 3, false, false, BKN>(p);
}

// A decoder block's qkv projection with the rotation and the cache update in its epilogue (one kernel per tile height)
__global__ __launch_bounds__(DMA_THREADS) void gemm_nt_dma256_rope_kernel(GemmArgs p) {
    gemm_nt_dma2_body<MOON_EPI_BIAS, 4, false, true>(p);
}
__global__ __launch_bounds__(DMA_THREADS) void gemm_nt_dma192_rope_kernel(GemmArgs p) {
    gemm_nt_dma2_body<MOON_EPI_BIAS, 3, false, true>(p);
}

// TWO products with the same [M, N] result shape in one launch, each with its own split of K, f32 partial sums only (the
// decoder block's out_proj and fc2, whose results are added: text_model.zig:163-171).  Alone, each of them leaves a
// quarter of the compute units idle at 768 rows (192 workgroups); together their 192 x 128 tiles times the splits fill all of
// them.  Workgroups [0, units0) take problem 0 (tile = unit % tiles, split = unit / tiles), the others problem 1.
struct GemmPairArgs {
    GemmArgs p[2];
    int units0, units_total;
};
__global__ __launch_bounds__(DMA_THREADS) void gemm_nt_dma192_pair_kernel(GemmPairArgs a) {
    const int per_xcd = (a.units_total + 7) / 8;
    const int unit = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
    if (unit >= a.units_total) return;
    const bool first = unit < a.units0;
    const GemmArgs &p = first ? a.p[0] : a.p[1];
    const int u = first ? unit : unit - a.units0;
    const int tiles = p.tiles_m * p.tiles_n;
    const int split = u / tiles, tile = u % tiles;
    const int k_begin = split * p.k_per_split, k_end = min(p.K, k_begin + p.k_per_split);
    if (k_end <= k_begin) return;
    gemm_nt_dma2_body<MOON_EPI_NONE, 3, true>(p, tile, k_begin / BK, (k_end - k_begin) / BK, split);
}

template <int EPI>
__global__ void splitk_reduce_kernel(const float *__restrict__ partial, const half_t *__restrict__ bias, const half_t *resid, half_t *C,
                                     size_t MN, int N, int splits) {
    size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= MN) return;
    float s = partial[i];
    for (int k = 1; k < splits; k++) s += partial[size_t(k) * MN + i];
    C[i] = apply_residual<EPI>(apply_epilogue<EPI>(s, bias, i % N), resid, i);
}
// The same sums (same order over the splits), eight consecutive outputs of a row per thread: 32-byte reads of every
// partial, a 16-byte store.  Needs N % 8 == 0 and 16-byte aligned C / bias / resid.
template <int EPI>
__global__ __launch_bounds__(256) void splitk_reduce8_kernel(const float *__restrict__ partial, const half_t *__restrict__ bias,
                                                             const half_t *resid, half_t *C, size_t MN, int N, int splits) {
    const size_t i = (size_t(blockIdx.x) * blockDim.x + threadIdx.x) * 8;
    if (i >= MN) return;
    float4 a = *reinterpret_cast<const float4 *>(partial + i), b = *reinterpret_cast<const float4 *>(partial + i + 4);
    for (int k = 1; k < splits; k++) {
        const float4 c = *reinterpret_cast<const float4 *>(partial + size_t(k) * MN + i), d = *reinterpret_cast<const float4 *>(partial + size_t(k) * MN + i + 4);
        a.x += c.x; a.y += c.y; a.z += c.z; a.w += c.w;
        b.x += d.x; b.y += d.y; b.z += d.z; b.w += d.w;
    }
    const float s[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
    const size_t n = i % N;
    half8_t bv = {0, 0, 0, 0, 0, 0, 0, 0}, rv = {0, 0, 0, 0, 0, 0, 0, 0}, o;
    if (EPI >= MOON_EPI_BIAS) bv = *reinterpret_cast<const half8_t *>(bias + n);
    if (EPI == MOON_EPI_BIAS_RESID) rv = *reinterpret_cast<const half8_t *>(resid + i);
#pragma unroll
    for (int e = 0; e < 8; e++) {
        half_t v = apply_epilogue_v<EPI>(s[e], bv[e]);
        if (EPI == MOON_EPI_BIAS_RESID) v = (half_t)((float)rv[e] + (float)v);
        o[e] = v;
    }
    *reinterpret_cast<half8_t *>(C + i) = o;
}

// The split-K reduction followed by the LayerNorm of the finished rows, one 256-thread workgroup per row of C (N <= 2048,
// N % 8 == 0): the sums and the epilogue are those of splitk_reduce8_kernel (same order over the splits); the row stays in
// registers (eight columns per thread) and ops.layerNorm (ops.zig:1063-1419: f32 mean, biased variance,
// y = f16((x*rstd - mean*rstd)*gamma + beta)) is applied to the f16 values just written to C, into ln_out.  Replaces a
// LayerNorm launch that would re-read C.  Row sums: per wavefront, then the four wavefronts' in a fixed order.
// add (with the residual epilogue only): a second addend, C = f16(resid + f16(add + t)) with t the product after its bias:
// the two adds of the decoder's parallel block (text_model.zig:170-171) with the product as the MLP branch.
constexpr int LN_FUSE_MAX_N = 2048;
template <int EPI>
__global__ __launch_bounds__(256) void splitk_reduce_ln_kernel(const float *__restrict__ partial, const half_t *__restrict__ bias, const half_t *resid,
                                                               const half_t *__restrict__ add, const float *__restrict__ add_partial, int add_splits,
                                                               const half_t *__restrict__ add_bias, half_t *C, const half_t *__restrict__ gamma,
                                                               const half_t *__restrict__ beta, half_t *__restrict__ ln_out, int M, int N, int splits,
                                                               float eps) {
    __shared__ float s_part[2][4];
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6, row = blockIdx.x;
    const size_t MN = size_t(M) * N, base = size_t(row) * N;
    const int n = t * 8;
    const bool mine = n < N;
    half8_t v = {0, 0, 0, 0, 0, 0, 0, 0}, g = v, bt = v;
    float sum = 0.0f;
    if (mine) {
        const size_t i = base + n;
        float4 a = *reinterpret_cast<const float4 *>(partial + i), b = *reinterpret_cast<const float4 *>(partial + i + 4);
        for (int k = 1; k < splits; k++) {
            const float4 c = *reinterpret_cast<const float4 *>(partial + size_t(k) * MN + i),
                         d = *reinterpret_cast<const float4 *>(partial + size_t(k) * MN + i + 4);
            a.x += c.x; a.y += c.y; a.z += c.z; a.w += c.w;
            b.x += d.x; b.y += d.y; b.z += d.z; b.w += d.w;
        }
        const float s[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
        half8_t bv = {0, 0, 0, 0, 0, 0, 0, 0}, rv = {0, 0, 0, 0, 0, 0, 0, 0}, av = {0, 0, 0, 0, 0, 0, 0, 0};
        if (EPI >= MOON_EPI_BIAS) bv = *reinterpret_cast<const half8_t *>(bias + n);
        if (EPI == MOON_EPI_BIAS_RESID) rv = *reinterpret_cast<const half8_t *>(resid + i);
        if (EPI == MOON_EPI_BIAS_RESID && add_partial) { // the other product's reduction and bias, as splitk_reduce8_kernel<MOON_EPI_BIAS> does them
            float4 pa = *reinterpret_cast<const float4 *>(add_partial + i), pb = *reinterpret_cast<const float4 *>(add_partial + i + 4);
            for (int k = 1; k < add_splits; k++) {
                const float4 c = *reinterpret_cast<const float4 *>(add_partial + size_t(k) * MN + i),
                             d = *reinterpret_cast<const float4 *>(add_partial + size_t(k) * MN + i + 4);
                pa.x += c.x; pa.y += c.y; pa.z += c.z; pa.w += c.w;
                pb.x += d.x; pb.y += d.y; pb.z += d.z; pb.w += d.w;
            }
            const float sa[8] = {pa.x, pa.y, pa.z, pa.w, pb.x, pb.y, pb.z, pb.w};
            const half8_t abv = *reinterpret_cast<const half8_t *>(add_bias + n);
#pragma unroll
            for (int e = 0; e < 8; e++) av[e] = apply_epilogue_v<MOON_EPI_BIAS>(sa[e], abv[e]);
        } else if (EPI == MOON_EPI_BIAS_RESID && add) av = *reinterpret_cast<const half8_t *>(add + i);
        g = *reinterpret_cast<const half8_t *>(gamma + n);
        bt = *reinterpret_cast<const half8_t *>(beta + n);
#pragma unroll
        for (int e = 0; e < 8; e++) {
            half_t o = apply_epilogue_v<EPI>(s[e], bv[e]);
            if (EPI == MOON_EPI_BIAS_RESID && (add || add_partial)) o = (half_t)((float)av[e] + (float)o); // attn += mlp (text_model.zig:170)
            if (EPI == MOON_EPI_BIAS_RESID) o = (half_t)((float)rv[e] + (float)o);
            v[e] = o;
            sum += (float)o;
        }
        *reinterpret_cast<half8_t *>(C + i) = v;
    }
    sum = wave_sum(sum);
    if (lane == 0) s_part[0][wave] = sum;
    __syncthreads();
    const float mean = ((s_part[0][0] + s_part[0][1]) + (s_part[0][2] + s_part[0][3])) / (float)N;
    float m2 = 0.0f;
    if (mine) {
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const float d = (float)v[e] - mean;
            m2 = fmaf(d, d, m2);
        }
    }
    m2 = wave_sum(m2);
    if (lane == 0) s_part[1][wave] = m2;
    __syncthreads();
    const float var = ((s_part[1][0] + s_part[1][1]) + (s_part[1][2] + s_part[1][3])) / (float)N;
    const float rstd = 1.0f / sqrtf(var + eps);
    if (mine) {
#pragma clang fp contract(off)
        const float mean_rstd = mean * rstd; // ops.zig:1301, 1330-1333: separate multiplies and adds
        half8_t o;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const float x = (float)v[e] * rstd - mean_rstd;
            o[e] = (half_t)(x * (float)g[e] + (float)bt[e]);
        }
        *reinterpret_cast<half8_t *>(ln_out + base + n) = o;
    }
}

// Any shape / alignment: one thread per output, sequential-k f32 accumulation.
template <int EPI>
__global__ void gemm_generic_kernel(const half_t *__restrict__ A, const half_t *__restrict__ B, const half_t *__restrict__ bias,
                                    const half_t *resid, half_t *C, int M, int N, int K, int b_is_nk) {
    const size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= size_t(M) * N) return;
    const int m = int(i / N), n = int(i % N);
    float acc = 0.0f;
    if (b_is_nk)
        for (int k = 0; k < K; k++) acc = fmaf((float)A[size_t(m) * K + k], (float)B[size_t(n) * K + k], acc);
    else
        for (int k = 0; k < K; k++) acc = fmaf((float)A[size_t(m) * K + k], (float)B[size_t(k) * N + n], acc);
    C[i] = apply_residual<EPI>(apply_epilogue<EPI>(acc, bias, size_t(n)), resid, i);
}

// B[K,N] -> Bt[N,K], 64x64 tiles through LDS
__global__ __launch_bounds__(256) void transpose_kernel(const half_t *__restrict__ src, half_t *__restrict__ dst, int rows, int cols) {
    __shared__ half_t tile[64][66];
    const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
    for (int i = threadIdx.x; i < 64 * 64; i += 256) {
        const int r = i / 64, c = i % 64;
        if (r0 + r < rows && c0 + c < cols) tile[r][c] = src[size_t(r0 + r) * cols + c0 + c];
    }
    __syncthreads();
    for (int i = threadIdx.x; i < 64 * 64; i += 256) {
        const int c = i / 64, r = i % 64;
        if (r0 + r < rows && c0 + c < cols) dst[size_t(c0 + c) * rows + r0 + r] = tile[r][c];
    }
}

// ln: optional LayerNorm of the finished rows of C into ln->out.  *ln_done says whether it was fused (into the split-K
// reduction); if not, the caller runs it as a launch of its own.  With ln->add set only the fused form can apply the
// epilogue: where the product does not take it, nothing is launched and GEMM_NOT_FUSED comes back.
constexpr int GEMM_NOT_FUSED = -1000;
template <int EPI>
int run_gemm(moon_ctx *ctx, const half_t *A, const half_t *B, const half_t *bias, const half_t *resid, half_t *C, int M, int N, int K,
             int b_layout, const GemmLayerNorm *ln, bool *ln_done, const float **keep_partial = nullptr, int *keep_splits = nullptr) {
    // keep_partial: run the split-K product only and leave its partials in work[3] (see launch_gemm_partials); like a second
    // addend this is all or nothing
    const bool must_fuse = (ln && ln->add) || keep_partial;
    const bool aligned = (K % 8 == 0) && (reinterpret_cast<uintptr_t>(A) % 16 == 0) && (reinterpret_cast<uintptr_t>(B) % 16 == 0) &&
                         (reinterpret_cast<uintptr_t>(C) % 8 == 0) && K > 0;
    if (!aligned) {
        if (must_fuse) return GEMM_NOT_FUSED;
        const size_t mn = size_t(M) * N;
        hipLaunchKernelGGL(gemm_generic_kernel<EPI>, dim3((unsigned)((mn + 255) / 256)), dim3(256), 0, ctx->stream, A, B, bias, resid, C,
                           M, N, K, b_layout == MOON_B_NK ? 1 : 0);
        MOON_NOTE_KERNEL(ctx, "gemm_generic_kernel");
        MOON_HIP(ctx, hipGetLastError());
        return MOON_OK;
    }
    const half_t *Bt = B;
    GemmArgs p;
    p.A = A;
    p.Bt = Bt;
    p.bias = bias;
    p.resid = resid;
    p.C = C;
    p.partial = nullptr;
    p.M = M;
    p.N = N;
    p.K = K;
    const size_t buf_max = (size_t(1) << 31) - 4096; // 32-bit offsets, with room for a granule past the last row
    const bool buffers_ok = size_t(M) * K * 2 < buf_max && size_t(N) * K * 2 < buf_max;
    p.super_m = p.super_n = 1;
    p.a_bytes = buffers_ok ? int(size_t(M) * K * 2) : 0;
    p.bt_bytes = buffers_ok ? int(size_t(N) * K * 2) : 0;
    {
        static const char *e = getenv("MOON_GEMM_EPILOGUE");
        const bool al = reinterpret_cast<uintptr_t>(C) % 16 == 0 && // (the split-K workspace is allocated by the library: aligned)
                         (!bias || reinterpret_cast<uintptr_t>(bias) % 16 == 0) &&
                        (!resid || reinterpret_cast<uintptr_t>(resid) % 16 == 0);
        p.lds_epilogue = al && !(e && !strcmp(e, "direct")) ? 1 : 0;
    }
    p.tiles_m = (M + BM - 1) / BM;
    p.tiles_n = (N + BN - 1) / BN;
    const int tiles = p.tiles_m * p.tiles_n;
    const int cus = ctx->cu_count > 0 ? ctx->cu_count : 256;
    const char *force = ctx->gemm_kernel[0] ? ctx->gemm_kernel : nullptr;
    // The kernels with 128 x 128 accumulators per wavefront (gemm_wide.hpp)
    const bool wide_ok = buffers_ok && K % 16 == 0 && N % 8 == 0 && p.lds_epilogue;
    int wide = 0; // 114: 128 x 128 tiles, 212: 256 x 128, 221: 256 x 256
    // Default: 256 x 256 tiles where they fill every CU at least once (measured 5 % faster than the 256 x 128 kernel at
    // 4096^3); the other two arrangements measured equal to or slower than the wavefront-specialised kernels on every shape
    // of the two models (their sum over the four wavefronts costs what their k-loop saves) and are only taken when named.
    if (wide_ok && !force && size_t((M + 255) / 256) * ((N + 255) / 256) >= size_t(cus) && !must_fuse) wide = 221;
    if (wide_ok && force && !strcmp(force, "w114")) wide = 114;
    if (wide_ok && force && !strcmp(force, "w212")) wide = 212;
    if (wide_ok && force && !strcmp(force, "w221")) wide = 221;
    // A [K, N] operand is read as it lies by the wavefront-specialised kernels (the 128 x 128 one up to one tile per compute
    // unit, the 192- / 256-row ones beyond); the other kernels get a transposed copy first.  MOON_GEMM_KN_TRANSPOSE: always the copy.
    const bool native_kn = b_layout == MOON_B_KN && N % 8 == 0 && K % 16 == 0 && buffers_ok && !force && !wide && !getenv("MOON_GEMM_KN_TRANSPOSE") &&
                           (tiles <= cus || (K % BK == 0 && p.lds_epilogue));
    if (b_layout == MOON_B_KN && !native_kn) {
        MOON_TRY(moon_grow(ctx, ctx->work[2], size_t(N) * K * sizeof(half_t)));
        hipLaunchKernelGGL(transpose_kernel, dim3((N + 63) / 64, (K + 63) / 64), dim3(256), 0, ctx->stream, B,
                           (half_t *)ctx->work[2].ptr, K, N);
        MOON_HIP(ctx, hipGetLastError());
        Bt = (const half_t *)ctx->work[2].ptr;
        p.Bt = Bt;
    }
    if (wide) {
        const int tm = wide == 114 ? 128 : 256, tn = wide == 221 ? 256 : 128;
        p.tiles_m = (M + tm - 1) / tm;
        p.tiles_n = (N + tn - 1) / tn;
        const int wtiles = p.tiles_m * p.tiles_n;
        wide_super_tiles(p.tiles_m, p.tiles_n, tm, tn, &p.super_m, &p.super_n);
        int splits = 1;
        if (wtiles * 2 <= cus && K >= 1024) {
            splits = cus / wtiles;
            if (splits > K / 512) splits = K / 512;
            if (splits > 8) splits = 8;
            if (splits < 1) splits = 1;
        }
        int kps = (K + splits - 1) / splits;
        kps = (kps + BK - 1) / BK * BK;
        splits = (K + kps - 1) / kps;
        p.splits = splits;
        p.k_per_split = kps;
        const bool ln_ok = splits > 1 && ln && N <= LN_FUSE_MAX_N && reinterpret_cast<uintptr_t>(ln->gamma) % 16 == 0 &&
                           reinterpret_cast<uintptr_t>(ln->beta) % 16 == 0 && reinterpret_cast<uintptr_t>(ln->out) % 16 == 0 &&
                           (!ln->add || reinterpret_cast<uintptr_t>(ln->add) % 16 == 0);
        if (keep_partial) {
            if (splits <= 1) return GEMM_NOT_FUSED;
        } else if (must_fuse && !ln_ok) return GEMM_NOT_FUSED;
        if (splits > 1) {
            GrowBuf &ws = ctx->work[keep_partial ? 3 : 0];
            MOON_TRY(moon_grow(ctx, ws, size_t(splits) * M * N * sizeof(float)));
            p.partial = (float *)ws.ptr;
        }
        const int total = wtiles * splits;
        const dim3 grid(((total + 7) / 8) * 8);
        const int dev = ctx->device >= 0 && ctx->device < 64 ? ctx->device : -1;
        // (with a split K the kernel writes partials and applies no epilogue: one instantiation serves every EPI)
        auto go = [&](auto kern, size_t lds_bytes, std::atomic<bool> *attr_set) -> int {
            if (dev < 0 || !attr_set[dev].load()) { // this much dynamic LDS needs the opt-in once per device and instantiation
                MOON_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
                if (dev >= 0) attr_set[dev].store(true);
            }
            hipLaunchKernelGGL(kern, grid, dim3(256), lds_bytes, ctx->stream, p);
            MOON_HIP(ctx, hipGetLastError());
            return MOON_OK;
        };
        static std::atomic<bool> set114[64], set212[64], set221[64];
        if (wide == 114) MOON_TRY(go(gemm_nt_wide_kernel<EPI, 1, 1, 4, 64>, WideCfg<1, 1, 4, 64>::LDS_BYTES, set114));
        else if (wide == 212) MOON_TRY(go(gemm_nt_wide_kernel<EPI, 2, 1, 2, 64>, WideCfg<2, 1, 2, 64>::LDS_BYTES, set212));
        else MOON_TRY(go(gemm_nt_wide_kernel<EPI, 2, 2, 1, 32>, WideCfg<2, 2, 1, 32>::LDS_BYTES, set221));
        MOON_NOTE_KERNEL(ctx, "gemm_nt_wide_kernel<%s> %d workgroups, k split %d", wide == 114 ? "1,1,4,64" : wide == 212 ? "2,1,2,64" : "2,2,1,32", total, splits);
        if (keep_partial) {
            *keep_partial = p.partial;
            *keep_splits = splits;
            return MOON_OK;
        }
        if (splits > 1) {
            const size_t mn = size_t(M) * N;
            if (ln_ok) {
                hipLaunchKernelGGL(splitk_reduce_ln_kernel<EPI>, dim3((unsigned)M), dim3(256), 0, ctx->stream, p.partial, bias, resid, ln->add,
                                   ln->add_partial, ln->add_splits, ln->add_bias, C, ln->gamma, ln->beta, ln->out, M, N, splits, ln->eps);
                *ln_done = true;
            } else
                hipLaunchKernelGGL(splitk_reduce8_kernel<EPI>, dim3((unsigned)((mn / 8 + 255) / 256)), dim3(256), 0, ctx->stream, p.partial, bias,
                                   resid, C, mn, N, splits);
            MOON_HIP(ctx, hipGetLastError());
        }
        return MOON_OK;
    }
    // More 128 x 128 tiles than CUs: the 256 x 128 kernel (MOON_GEMM_KERNEL=regs|dma keeps the 128 x 128 ones).
    if (tiles > cus && buffers_ok && K % BK == 0 && N % 8 == 0 && p.lds_epilogue && !(force && (!strcmp(force, "regs") || !strcmp(force, "dma")))) {
        if (must_fuse) return GEMM_NOT_FUSED;
        // 192-row tiles where they fill more CUs in one round than 256-row tiles do (M = 768: four row blocks, not three)
        const int t256 = ((M + 255) / 256) * p.tiles_n, t192 = ((M + 191) / 192) * p.tiles_n;
        const bool use192 = t192 <= cus && t192 > t256 && size_t((M + 191) / 192) * 192 <= size_t((M + 255) / 256) * 256 &&
                            !(force && !strcmp(force, "dma256"));
        p.tiles_m = use192 ? (M + 191) / 192 : (M + 255) / 256;
        p.splits = 1;
        p.k_per_split = K;
        const int total = p.tiles_m * p.tiles_n;
        const size_t lds_bytes = use192 ? Dma2<3>::LDS_BYTES : Dma2<4>::LDS_BYTES;
        // the opt-in to this much dynamic LDS is per device and per kernel (here: per epilogue instantiation); setting it twice is harmless
        static std::atomic<bool> attr_set[4][64];
        const int dev = ctx->device >= 0 && ctx->device < 64 ? ctx->device : -1;
        const int which = (use192 ? 1 : 0) + (native_kn ? 2 : 0);
        if (dev < 0 || !attr_set[which][dev].load()) {
            const void *kern = native_kn ? (use192 ? reinterpret_cast<const void *>(gemm_nt_dma192_kernel<EPI, true>) : reinterpret_cast<const void *>(gemm_nt_dma256_kernel<EPI, true>))
                                         : (use192 ? reinterpret_cast<const void *>(gemm_nt_dma192_kernel<EPI>) : reinterpret_cast<const void *>(gemm_nt_dma256_kernel<EPI>));
            MOON_HIP(ctx, hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
            if (dev >= 0) attr_set[which][dev].store(true);
        }
        const dim3 grid2(((total + 7) / 8) * 8);
        if (native_kn) {
            if (use192) hipLaunchKernelGGL((gemm_nt_dma192_kernel<EPI, true>), grid2, dim3(DMA_THREADS), lds_bytes, ctx->stream, p);
            else hipLaunchKernelGGL((gemm_nt_dma256_kernel<EPI, true>), grid2, dim3(DMA_THREADS), lds_bytes, ctx->stream, p);
        } else if (use192) hipLaunchKernelGGL(gemm_nt_dma192_kernel<EPI>, grid2, dim3(DMA_THREADS), lds_bytes, ctx->stream, p);
        else hipLaunchKernelGGL(gemm_nt_dma256_kernel<EPI>, grid2, dim3(DMA_THREADS), lds_bytes, ctx->stream, p);
        MOON_NOTE_KERNEL(ctx, "%s%s %d workgroups", use192 ? "gemm_nt_dma192_kernel" : "gemm_nt_dma256_kernel", native_kn ? " ([K,N] operand read in place)" : "", total);
        MOON_HIP(ctx, hipGetLastError());
        return MOON_OK;
    }
    int splits = 1;
    if (tiles * 2 <= cus && K >= 1024) {
        splits = cus / tiles;
        const int max_by_k = K / 512;
        if (splits > max_by_k) splits = max_by_k;
        if (splits > 8) splits = 8;
        if (splits < 1) splits = 1;
    }
    int kps = (K + splits - 1) / splits;
    kps = (kps + BK - 1) / BK * BK;
    splits = (K + kps - 1) / kps;
    p.splits = splits;
    p.k_per_split = kps;
    const bool ln_ok = splits > 1 && ln && N % 8 == 0 && N <= LN_FUSE_MAX_N && p.lds_epilogue && reinterpret_cast<uintptr_t>(ln->gamma) % 16 == 0 &&
                       reinterpret_cast<uintptr_t>(ln->beta) % 16 == 0 && reinterpret_cast<uintptr_t>(ln->out) % 16 == 0 &&
                       (!ln->add || reinterpret_cast<uintptr_t>(ln->add) % 16 == 0);
    if (keep_partial) {
        if (splits <= 1 || N % 8 || !p.lds_epilogue) return GEMM_NOT_FUSED;
    } else if (must_fuse && !ln_ok) return GEMM_NOT_FUSED;
    if (splits > 1) {
        GrowBuf &ws = ctx->work[keep_partial ? 3 : 0];
        MOON_TRY(moon_grow(ctx, ws, size_t(splits) * M * N * sizeof(float)));
        p.partial = (float *)ws.ptr;
    }
    const int total = tiles * splits;
    const int grid = ((total + 7) / 8) * 8;
    // Which kernel: with at most one workgroup per CU the wavefront-specialised kernel is faster (its loaders keep 96 KiB
    // in flight for the lone workgroup); with more tiles than CUs two register-staged workgroups share a CU and overlap
    // each other's stalls, which measures faster.  K % 16 != 0 needs the register-staged kernel.
    // MOON_GEMM_KERNEL=regs|dma overrides the choice (for measurements).
    bool use_dma = K % 16 == 0 && total <= cus && buffers_ok;
    if (force && !strcmp(force, "regs")) use_dma = false;
    if (force && !strcmp(force, "dma")) use_dma = K % 16 == 0 && buffers_ok;
    if (native_kn && !use_dma) return moon_fail(ctx, MOON_EINVAL, "gemm: no kernel for this [K, N] operand"); // (cannot happen: the same conditions)
    if (use_dma) {
        static std::atomic<bool> attr_set[2][64]; // 128 KiB of dynamic LDS needs the opt-in once per device (and per instantiation)
        const int dev = ctx->device >= 0 && ctx->device < 64 ? ctx->device : -1;
        if (dev < 0 || !attr_set[native_kn ? 1 : 0][dev].load()) {
            const void *kern = native_kn ? reinterpret_cast<const void *>(gemm_nt_dma_kernel<EPI, true>) : reinterpret_cast<const void *>(gemm_nt_dma_kernel<EPI>);
            MOON_HIP(ctx, hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)DMA_LDS_BYTES));
            if (dev >= 0) attr_set[native_kn ? 1 : 0][dev].store(true);
        }
        if (native_kn) hipLaunchKernelGGL((gemm_nt_dma_kernel<EPI, true>), dim3(grid), dim3(DMA_THREADS), DMA_LDS_BYTES, ctx->stream, p);
        else hipLaunchKernelGGL(gemm_nt_dma_kernel<EPI>, dim3(grid), dim3(DMA_THREADS), DMA_LDS_BYTES, ctx->stream, p);
    } else {
        hipLaunchKernelGGL(gemm_nt_mfma_kernel<EPI>, dim3(grid), dim3(256), 0, ctx->stream, p);
    }
    MOON_NOTE_KERNEL(ctx, "%s %d workgroups, k split %d%s", native_kn ? "gemm_nt_dma_kernel ([K,N] operand read in place)" : use_dma ? "gemm_nt_dma_kernel" : "gemm_nt_mfma_kernel", total, splits,
                     splits > 1 ? (ln_ok ? " + splitk_reduce_ln_kernel" : " + splitk_reduce kernel") : "");
    MOON_HIP(ctx, hipGetLastError());
    if (keep_partial) {
        *keep_partial = p.partial;
        *keep_splits = splits;
        return MOON_OK;
    }
    if (splits > 1) {
        const size_t mn = size_t(M) * N;
        if (ln_ok) {
            hipLaunchKernelGGL(splitk_reduce_ln_kernel<EPI>, dim3((unsigned)M), dim3(256), 0, ctx->stream, p.partial, bias, resid, ln->add,
                               ln->add_partial, ln->add_splits, ln->add_bias, C, ln->gamma, ln->beta, ln->out, M, N, splits, ln->eps);
            *ln_done = true;
        } else if (N % 8 == 0 && p.lds_epilogue)
            hipLaunchKernelGGL(splitk_reduce8_kernel<EPI>, dim3((unsigned)((mn / 8 + 255) / 256)), dim3(256), 0, ctx->stream, p.partial, bias,
                               resid, C, mn, N, splits);
        else
            hipLaunchKernelGGL(splitk_reduce_kernel<EPI>, dim3((unsigned)((mn + 255) / 256)), dim3(256), 0, ctx->stream, p.partial, bias, resid,
                               C, mn, N, splits);
        MOON_HIP(ctx, hipGetLastError());
    }
    return MOON_OK;
}

} // namespace

int launch_gemm(moon_ctx *ctx, const half_t *A, const half_t *B, const half_t *bias, half_t *C, size_t M, size_t N, size_t K,
                int b_layout, int epilogue, const half_t *resid, const GemmLayerNorm *ln) {
    if (M == 0 || N == 0) return MOON_OK;
    if (M > 0x3fffffff || N > 0x3fffffff || K > 0x3fffffff) return moon_fail(ctx, MOON_EINVAL_DIM, "gemm: dimension too large");
    if (epilogue != MOON_EPI_NONE && !bias) return moon_fail(ctx, MOON_EINVAL, "gemm: epilogue needs a bias");
    if (b_layout != MOON_B_KN && b_layout != MOON_B_NK) return moon_fail(ctx, MOON_EINVAL, "gemm: unknown B layout %d", b_layout);
    if (ln && (!ln->gamma || !ln->beta || !ln->out)) return moon_fail(ctx, MOON_EINVAL, "gemm: the LayerNorm that follows needs gamma, beta and an output");
    if (ln && !(ln->eps > 0.0f)) return moon_fail(ctx, MOON_EEPS, "gemm: the LayerNorm that follows needs eps > 0");
    if (ln && ln->add && (epilogue != MOON_EPI_BIAS_RESID || !ln->add_scratch))
        return moon_fail(ctx, MOON_EINVAL, "gemm: a second addend needs the residual epilogue and a scratch buffer");
    if (ln && ln->add_partial && (!ln->add || !ln->add_bias || ln->add_splits < 2 || N % 8 || reinterpret_cast<uintptr_t>(ln->add_bias) % 16))
        return moon_fail(ctx, MOON_EINVAL, "gemm: partials as the second addend need their bias, their split count and a destination");
    bool ln_done = false;
    int rc;
    switch (epilogue) {
    case MOON_EPI_NONE: rc = run_gemm<MOON_EPI_NONE>(ctx, A, B, bias, nullptr, C, (int)M, (int)N, (int)K, b_layout, ln, &ln_done); break;
    case MOON_EPI_BIAS: rc = run_gemm<MOON_EPI_BIAS>(ctx, A, B, bias, nullptr, C, (int)M, (int)N, (int)K, b_layout, ln, &ln_done); break;
    case MOON_EPI_BIAS_GELU: rc = run_gemm<MOON_EPI_BIAS_GELU>(ctx, A, B, bias, nullptr, C, (int)M, (int)N, (int)K, b_layout, ln, &ln_done); break;
    case MOON_EPI_BIAS_RESID:
        if (!resid) return moon_fail(ctx, MOON_EINVAL, "gemm: the residual epilogue needs a residual");
        rc = run_gemm<MOON_EPI_BIAS_RESID>(ctx, A, B, bias, resid, C, (int)M, (int)N, (int)K, b_layout, ln, &ln_done);
        break;
    default: return moon_fail(ctx, MOON_EINVAL, "gemm: unknown epilogue %d", epilogue);
    }
    if (rc == GEMM_NOT_FUSED) { // the same arithmetic as separate launches: t = product + bias; C = f16(resid + f16(add + t)); LayerNorm
        if (ln->add_partial) {
            const size_t mn = M * N;
            hipLaunchKernelGGL(splitk_reduce8_kernel<MOON_EPI_BIAS>, dim3((unsigned)((mn / 8 + 255) / 256)), dim3(256), 0, ctx->stream, ln->add_partial,
                               ln->add_bias, nullptr, const_cast<half_t *>(ln->add), mn, (int)N, ln->add_splits);
            MOON_HIP(ctx, hipGetLastError());
        }
        MOON_TRY(run_gemm<MOON_EPI_BIAS>(ctx, A, B, bias, nullptr, ln->add_scratch, (int)M, (int)N, (int)K, b_layout, nullptr, &ln_done));
        if (C != resid) MOON_HIP(ctx, hipMemcpyAsync(C, resid, M * N * sizeof(half_t), hipMemcpyDeviceToDevice, ctx->stream));
        MOON_TRY(launch_residual2(ctx, C, ln->add, ln->add_scratch, M * N));
        return launch_layernorm(ctx, C, ln->gamma, ln->beta, ln->out, M, N, ln->eps);
    }
    if (rc != MOON_OK || !ln || ln_done) return rc;
    return launch_layernorm(ctx, C, ln->gamma, ln->beta, ln->out, M, N, ln->eps);
}

int launch_gemm_partials(moon_ctx *ctx, const half_t *A, const half_t *B, size_t M, size_t N, size_t K, int b_layout, const float **partial,
                         int *splits) {
    *partial = nullptr;
    *splits = 0;
    if (M == 0 || N == 0 || M > 0x3fffffff || N > 0x3fffffff || K > 0x3fffffff) return MOON_OK;
    if (b_layout != MOON_B_KN && b_layout != MOON_B_NK) return moon_fail(ctx, MOON_EINVAL, "gemm: unknown B layout %d", b_layout);
    bool ln_done = false;
    // (C only enters the alignment checks of the shared code: the workspace itself is what gets written)
    const int rc = run_gemm<MOON_EPI_NONE>(ctx, A, B, nullptr, nullptr, reinterpret_cast<half_t *>(ctx->work[3].ptr), (int)M, (int)N, (int)K, b_layout,
                                           nullptr, &ln_done, partial, splits);
    if (rc == GEMM_NOT_FUSED) {
        *partial = nullptr;
        *splits = 0;
        return MOON_OK;
    }
    return rc;
}

int launch_gemm_qkv_rope(moon_ctx *ctx, const half_t *A, const half_t *W, const half_t *bias, size_t M, size_t K, half_t *q_out, half_t *cache_k,
                         half_t *cache_v, const float *table, size_t H, size_t D, size_t rot_dim, size_t max_seq, size_t pos0, bool *done) {
    *done = false;
    const int cus = ctx->cu_count > 0 ? ctx->cu_count : 256;
    const size_t N = 3 * H * D, buf_max = (size_t(1) << 31) - 4096;
    const auto al16 = [](const void *q) { return reinterpret_cast<uintptr_t>(q) % 16 == 0; };
    if (ctx->gemm_kernel[0] || getenv("MOON_GEMM_NO_ROPE")) return MOON_OK; // (a kernel was named for measurements, or the fusion switched off)
    if (D != 64 || !H || rot_dim % 16 || rot_dim > D || !M || M > 0x3fffffff || K % BK || !K || pos0 + M > max_seq || max_seq > 0x3fffffff) return MOON_OK;
    if (M * K * 2 >= buf_max || N * K * 2 >= buf_max) return MOON_OK;
    if (!al16(A) || !al16(W) || !al16(bias) || !al16(q_out) || !al16(cache_k) || !al16(cache_v) || !al16(table)) return MOON_OK;
    // the shapes that launch_gemm gives to the 256- and 192-row kernels: more 128 x 128 tiles than compute units
    const int tiles_n = (int)((N + BN - 1) / BN);
    if (size_t((M + BM - 1) / BM) * tiles_n <= size_t(cus)) return MOON_OK;
    const int t256 = (int)((M + 255) / 256) * tiles_n, t192 = (int)((M + 191) / 192) * tiles_n;
    const bool use192 = t192 <= cus && t192 > t256 && ((M + 191) / 192) * 192 <= ((M + 255) / 256) * 256;
    GemmArgs p;
    p.A = A;
    p.Bt = W;
    p.bias = bias;
    p.resid = nullptr;
    p.C = nullptr;
    p.partial = nullptr;
    p.M = (int)M;
    p.N = (int)N;
    p.K = (int)K;
    p.tiles_m = (int)(use192 ? (M + 191) / 192 : (M + 255) / 256);
    p.tiles_n = tiles_n;
    p.splits = 1;
    p.k_per_split = (int)K;
    p.a_bytes = (int)(M * K * 2);
    p.bt_bytes = (int)(N * K * 2);
    p.lds_epilogue = 1;
    p.super_m = p.super_n = 1;
    p.rope_q = q_out;
    p.rope_ck = cache_k;
    p.rope_cv = cache_v;
    p.rope_table = table;
    p.rope_H = (int)H;
    p.rope_dim = (int)rot_dim;
    p.rope_max_seq = (int)max_seq;
    p.rope_pos0 = (int)pos0;
    const int total = p.tiles_m * p.tiles_n;
    const size_t lds_bytes = use192 ? Dma2<3>::LDS_BYTES : Dma2<4>::LDS_BYTES;
    static std::atomic<bool> attr_set[2][64];
    const int dev = ctx->device >= 0 && ctx->device < 64 ? ctx->device : -1;
    if (dev < 0 || !attr_set[use192 ? 1 : 0][dev].load()) {
        const void *kern = use192 ? reinterpret_cast<const void *>(gemm_nt_dma192_rope_kernel) : reinterpret_cast<const void *>(gemm_nt_dma256_rope_kernel);
        MOON_HIP(ctx, hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
        if (dev >= 0) attr_set[use192 ? 1 : 0][dev].store(true);
    }
    const dim3 grid(((total + 7) / 8) * 8);
    if (use192) hipLaunchKernelGGL(gemm_nt_dma192_rope_kernel, grid, dim3(DMA_THREADS), lds_bytes, ctx->stream, p);
    else hipLaunchKernelGGL(gemm_nt_dma256_rope_kernel, grid, dim3(DMA_THREADS), lds_bytes, ctx->stream, p);
    MOON_NOTE_KERNEL(ctx, "%s %d workgroups", use192 ? "gemm_nt_dma192_rope_kernel" : "gemm_nt_dma256_rope_kernel", total);
    MOON_HIP(ctx, hipGetLastError());
    *done = true;
    return MOON_OK;
}

int launch_gemm_pair_ln(moon_ctx *ctx, const half_t *A_add, const half_t *B_add, const half_t *bias_add, size_t K_add, const half_t *A, const half_t *B,
                        const half_t *bias, size_t K, const half_t *resid, half_t *C, size_t M, size_t N, const GemmLayerNorm &ln, bool *done) {
    *done = false;
    const int cus = ctx->cu_count > 0 ? ctx->cu_count : 256;
    const size_t buf_max = (size_t(1) << 31) - 4096;
    const auto al16 = [](const void *q) { return reinterpret_cast<uintptr_t>(q) % 16 == 0; };
    if (ctx->gemm_kernel[0] || getenv("MOON_GEMM_NO_PAIR")) return MOON_OK; // (a kernel was named for measurements: the products run one by one)
    if (M < 192 || M > 0x3fffffff || N % 8 || N > (size_t)LN_FUSE_MAX_N || K % BK || K_add % BK || !K || !K_add) return MOON_OK;
    if (M * K * 2 >= buf_max || N * K * 2 >= buf_max || M * K_add * 2 >= buf_max || N * K_add * 2 >= buf_max) return MOON_OK;
    if (!al16(A) || !al16(B) || !al16(A_add) || !al16(B_add) || !al16(bias) || !al16(bias_add) || !al16(resid) || !al16(C) || !al16(ln.gamma) ||
        !al16(ln.beta) || !al16(ln.out) || !ln.add || !al16(ln.add))
        return MOON_OK;
    const int tiles_m = (int)((M + 191) / 192), tiles_n = (int)((N + BN - 1) / BN), tiles = tiles_m * tiles_n;
    if (tiles * 2 > cus) return MOON_OK;
    // splits (s_add, s): all workgroups in one round, the longest run of k-tiles as short as it gets
    const int kt_add = (int)(K_add / BK), kt = (int)(K / BK);
    int best_a = 0, best_s = 0, best_len = 1 << 30;
    for (int sa = 1; sa <= 8 && sa <= kt_add; sa++)
        for (int s = 1; s <= 8 && s <= kt; s++) {
            if (tiles * (sa + s) > cus) continue;
            const int len = std::max((kt_add + sa - 1) / sa, (kt + s - 1) / s);
            if (len < best_len || (len == best_len && sa + s < best_a + best_s)) {
                best_len = len;
                best_a = sa;
                best_s = s;
            }
        }
    if (!best_a) return MOON_OK;
    GemmPairArgs a;
    const auto fill = [&](GemmArgs &p, const half_t *Ap, const half_t *Bp, size_t Kp, int splits, GrowBuf &ws) -> int {
        p.A = Ap;
        p.Bt = Bp;
        p.bias = nullptr;
        p.resid = nullptr;
        p.C = nullptr;
        p.M = (int)M;
        p.N = (int)N;
        p.K = (int)Kp;
        p.tiles_m = tiles_m;
        p.tiles_n = tiles_n;
        const int ktp = (int)(Kp / BK);
        p.k_per_split = (ktp + splits - 1) / splits * BK;
        p.splits = (int)((Kp + p.k_per_split - 1) / p.k_per_split);
        p.a_bytes = (int)(M * Kp * 2);
        p.bt_bytes = (int)(N * Kp * 2);
        p.lds_epilogue = 1;
        p.super_m = p.super_n = 1;
        MOON_TRY(moon_grow(ctx, ws, size_t(p.splits) * M * N * sizeof(float)));
        p.partial = (float *)ws.ptr;
        return MOON_OK;
    };
    MOON_TRY(fill(a.p[0], A_add, B_add, K_add, best_a, ctx->work[3]));
    MOON_TRY(fill(a.p[1], A, B, K, best_s, ctx->work[0]));
    a.units0 = tiles * a.p[0].splits;
    a.units_total = a.units0 + tiles * a.p[1].splits;
    static std::atomic<bool> attr_set[64];
    const int dev = ctx->device >= 0 && ctx->device < 64 ? ctx->device : -1;
    if (dev < 0 || !attr_set[dev].load()) {
        MOON_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_nt_dma192_pair_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                          (int)Dma2<3>::LDS_BYTES));
        if (dev >= 0) attr_set[dev].store(true);
    }
    hipLaunchKernelGGL(gemm_nt_dma192_pair_kernel, dim3(((a.units_total + 7) / 8) * 8), dim3(DMA_THREADS), Dma2<3>::LDS_BYTES, ctx->stream, a);
    MOON_NOTE_KERNEL(ctx, "gemm_nt_dma192_pair_kernel %d + %d workgroups, k splits %d and %d + splitk_reduce_ln_kernel", a.units0, a.units_total - a.units0,
                     a.p[0].splits, a.p[1].splits);
    MOON_HIP(ctx, hipGetLastError());
    hipLaunchKernelGGL(splitk_reduce_ln_kernel<MOON_EPI_BIAS_RESID>, dim3((unsigned)M), dim3(256), 0, ctx->stream, a.p[1].partial, bias, resid, ln.add,
                       a.p[0].partial, a.p[0].splits, bias_add, C, ln.gamma, ln.beta, ln.out, (int)M, (int)N, a.p[1].splits, ln.eps);
    MOON_HIP(ctx, hipGetLastError());
    *done = true;
    return MOON_OK;
}

// dst[cols, rows] = src[rows, cols]^T
int launch_transpose(moon_ctx *ctx, const half_t *src, half_t *dst, size_t rows, size_t cols) {
    if (!rows || !cols) return MOON_OK;
    hipLaunchKernelGGL(transpose_kernel, dim3((unsigned)((cols + 63) / 64), (unsigned)((rows + 63) / 64)), dim3(256), 0, ctx->stream,
                       src, dst, (int)rows, (int)cols);
    MOON_HIP(ctx, hipGetLastError());
    return MOON_OK;
}
