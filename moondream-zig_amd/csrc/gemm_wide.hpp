// FP16 GEMM, C[M,N] = epi(A[M,K] x Bt[N,K]^T), with 128 x 128 accumulators per wavefront -- the tiled path of
// hgemm_trans.matmul (hgemm_trans.zig:457-487) and, after the re-layout of B, hgemm.matmul (hgemm.zig:362-426).
//
// Why another kernel: with 64 x 64 per wavefront every v_mfma_f32_32x32x16_f16 needs one 16-byte-per-lane operand read
// from LDS.  A wavefront that owns 128 x 128 (4 x 4 accumulators = 256 accumulation registers, so one wavefront per SIMD
// and 256 threads per workgroup) issues 8 operand reads per 16 MFMAs.  The four wavefronts of a workgroup are arranged
// WM x WN x WK:
//   WM x WN wavefronts tile the workgroup's (128 WM) x (128 WN) output; WK wavefronts share one output tile and split
//   each k-tile between them (16-wide steps wk*KS .. wk*KS+KS-1), their accumulators being summed through LDS once, after
//   the k-loop, in a fixed order.
//   1 x 1 x 4 (k-tile 64): 128 x 128 per workgroup, for shapes with about as many such tiles as CUs,
//   2 x 1 x 2 (k-tile 64): 256 x 128,   2 x 2 x 1 (k-tile 32): 256 x 256, for large shapes.
// There are no loader wavefronts: every wavefront copies its share of the next k-tiles global -> LDS with
// buffer_load_dwordx4 ... lds (no staging registers), STAGES k-tiles deep, one barrier per k-tile.  With a single
// wavefront per SIMD nothing else fills the matrix core while that wavefront issues other instructions, so the operand
// reads of the next step and the copies are placed one by one between the MFMAs of the current step, where their issue
// cycles are hidden.  Operand reads and their waits are written by hand (see gemm.hip for why).
// Needs K % 16 == 0, N % 8 == 0, 16-byte aligned rows of C / bias / resid, operands below 2 GiB.
#pragma once
#include <type_traits>

#include "gemm_common.hpp"

// Timing experiments only (results are wrong when non-zero): 1 no MFMAs, 2 no copies after the first stages, 4 no operand
// reads, 8 no barrier per k-tile, 16 time stamps (100 MHz counter) of the phases into p.partial (no split K then).  The
// library is built with 0.
#ifndef WIDE_TUNE
#define WIDE_TUNE 0
#endif
#ifndef WIDE_DMA_SLOTS
#define WIDE_DMA_SLOTS 0
#endif

namespace {

template <int WM, int WN, int WK, int BKT> struct WideCfg {
    static_assert(WM * WN * WK == 4, "four wavefronts");
    static_assert(BKT == 64 || BKT == 32, "k-tiles of 64 or 32");
    static constexpr int TM = 128 * WM;
    static constexpr int TN = 128 * WN;
    static constexpr int ROW_BYTES = BKT * 2;              // a staged row
    static constexpr int GRAN = BKT / 8;                   // 16-byte granules per row
    static constexpr int ROWS_PER_COPY = 1024 / ROW_BYTES; // one copy instruction moves 1 KiB
    static constexpr unsigned STAGE_BYTES = (TM + TN) * ROW_BYTES;
    static constexpr int STAGES = STAGE_BYTES <= 32768 ? 5 : STAGE_BYTES <= 49152 ? 3 : 2;
    static constexpr size_t LDS_BYTES = size_t(STAGES) * STAGE_BYTES;
    static constexpr int DA = TM / 4 / ROWS_PER_COPY; // copies per wavefront and k-tile: activation rows
    static constexpr int DW = TN / 4 / ROWS_PER_COPY; // ... weight rows
    static constexpr int DPW = DA + DW;
    static constexpr int KS = BKT / 16 / WK; // 16-wide steps of a k-tile per wavefront
    static_assert(KS >= 1, "every wavefront has a step");
    static_assert((STAGES - 1) * DPW < 64, "the copies in flight fit the counter");
};

// Granule swizzle of a staged row: makes the 128-bit operand reads of 32 consecutive rows and the 1 KiB copies conflict free.
template <int BKT> __device__ __forceinline__ int wide_swz(int row, int granule) {
    return BKT == 64 ? granule ^ ((row >> 1) & 7) : granule ^ ((row >> 2) & 3);
}

template <int OFF> __device__ __forceinline__ void ds_read_b128_at(half8_t &dst, unsigned addr) {
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF));
}

// at most n of this wavefront's copies outstanding (they retire in order)
__device__ __forceinline__ void wide_wait_copies(int n) {
    if (n >= 32) wait_vmcnt<32>();
    else if (n >= 24) wait_vmcnt<24>();
    else if (n >= 16) wait_vmcnt<16>();
    else if (n >= 12) wait_vmcnt<12>();
    else if (n >= 8) wait_vmcnt<8>();
    else wait_vmcnt<0>();
}

__device__ __forceinline__ float acc_read(const float &a) { // the value where the MFMAs left it (an accumulation register)
    float r;
    asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(r) : "a"(a));
    return r;
}

// Host side: the block of tiles (sm x sn) in which gemm_nt_wide_kernel deals its tiles.  An XCD receives a contiguous run of
// about tiles / 8 tiles; the block is chosen so that such a run touches few distinct operand rows per k-tile (sm * TM
// activation rows + sn * TN weight rows), which is what its L2 has to hold and the fabric has to deliver.
inline void wide_super_tiles(int tiles_m, int tiles_n, int tile_rows_m, int tile_rows_n, int *sm_out, int *sn_out) {
    const int per_xcd = (tiles_m * tiles_n + 7) / 8;
    long best = -1;
    int bm = tiles_m, bn = 1;
    for (int sm = 1; sm <= tiles_m; sm++) {
        int sn = (per_xcd + sm - 1) / sm;
        if (sn > tiles_n) sn = tiles_n;
        if (sn < 1) sn = 1;
        long cost = long(sm) * tile_rows_m + long(sn) * tile_rows_n;
        if (tiles_m % sm) cost += tile_rows_m / 2;             // ragged blocks at the bottom
        if (sm * sn != per_xcd) cost += tile_rows_m / 4;       // runs that straddle blocks
        if (best < 0 || cost < best) {
            best = cost;
            bm = sm;
            bn = sn;
        }
    }
    *sm_out = bm;
    *sn_out = bn;
}

constexpr int WIDE_PITCH_H = 136; // halfs per parked row of 128 n (f16 tile on its way out)
constexpr int WIDE_PITCH_H2 = 72; // ... of 64 n
constexpr int WIDE_PITCH_F = 132; // floats per parked row of 128 n (f32 partials of a split K)
constexpr int WIDE_PITCH_F2 = 68; // ... of 64 n

template <int EPI, int WM, int WN, int WK, int BKT>
__global__ __launch_bounds__(256) void gemm_nt_wide_kernel(GemmArgs p) {
    // The body is compiled in the device pass only.  The host pass needs nothing but the stub, and it mishandles this body:
    // after the first instantiation it drops the stubs of further instantiations that differ in EPI only, without a
    // diagnostic (the device-only builtins and register constraints inside the nested generic lambdas).
#if defined(__HIP_DEVICE_COMPILE__)
    using Cfg = WideCfg<WM, WN, WK, BKT>;
    constexpr int TM = Cfg::TM, TN = Cfg::TN, STAGES = Cfg::STAGES, DPW = Cfg::DPW, KS = Cfg::KS, ROW_BYTES = Cfg::ROW_BYTES;
    constexpr unsigned STAGE_BYTES = Cfg::STAGE_BYTES;
    constexpr int BLK = 32 * ROW_BYTES; // bytes between the 32-row blocks of a staged operand
    extern __shared__ __attribute__((aligned(16))) char lds_wide[];

    // workgroup -> (split, tile): the ids an XCD receives (round robin over 8) cover a contiguous run of tiles, m fastest,
    // so the workgroups of one XCD share weight panels in its L2
    const int tiles = p.tiles_m * p.tiles_n;
    const int total = tiles * p.splits;
    const int per_xcd = (total + 7) / 8;
    const int wg = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
    if (wg >= total) return;
    const int split = wg / tiles;
    const int tile_id = wg % tiles;
    // tile order: blocks of SM x SN tiles, m fastest inside a block and over the blocks of a block column.  With more tile rows
    // than SM an XCD's run then covers a squarer patch (fewer distinct operand rows per k-tile through its L2) than a plain
    // m-fastest order would.
    int tn, tm;
    {
        const int SM = p.super_m, SN = p.super_n;
        const int full_cols = p.tiles_n / SN * SN; // tile columns that lie in full-width block columns
        const int in_full = full_cols * p.tiles_m;
        if (tile_id < in_full) {
            const int bc = tile_id / (SN * p.tiles_m), r = tile_id % (SN * p.tiles_m); // block column, index within it
            const int full_rows = p.tiles_m / SM * SM;
            if (r < full_rows * SN) {
                const int br = r / (SM * SN), q = r % (SM * SN);
                tm = br * SM + q % SM;
                tn = bc * SN + q / SM;
            } else { // the ragged block at the bottom of the column
                const int q = r - full_rows * SN, h = p.tiles_m - full_rows;
                tm = full_rows + q % h;
                tn = bc * SN + q / h;
            }
        } else { // the ragged block column at the right: m fastest
            const int q = tile_id - in_full;
            tm = q % p.tiles_m;
            tn = full_cols + q / p.tiles_m;
        }
    }
    const int m0 = tm * TM, n0 = tn * TN;
    const int k_begin = split * p.k_per_split;
    const int k_end = min(p.K, k_begin + p.k_per_split);
    const int n_ktiles = (k_end - k_begin + BKT - 1) / BKT;
    if (n_ktiles <= 0) return;

    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
#if WIDE_TUNE & 16
    long long stamp[5];
    stamp[0] = wall_clock64();
#endif
    const int wk = wave % WK, wmn = wave / WK, wm = wmn % WM, wn = wmn / WM;
    const int frag_row = lane & 31, frag_g = lane >> 5;

    // ---- copies global -> LDS: this wavefront fills activation rows [wave*TM/4, +TM/4) and weight rows [wave*TN/4, +TN/4)
    // of every stage, 1 KiB per instruction, buffer form (scalar descriptor, one offset register per lane and
    // instruction).  The swizzle sits on the source side: the lane that fills physical
    // granule pg of row r fetches the logical granule that the swizzle maps there.  Rows past M / N repeat the last row
    // (never stored); reads past the end of the operand return zero.
    // (the lambdas below capture pointers to these arrays, not the arrays: an array whose bound depends on the template
    // parameters, captured by a lambda, makes the host pass reject or silently drop this kernel's stub)
    int off_a_[Cfg::DA], off_w_[Cfg::DW];
#pragma unroll
    for (int j = 0; j < Cfg::DA; j++) {
        const int r = wave * (TM / 4) + Cfg::ROWS_PER_COPY * j + lane / Cfg::GRAN;
        off_a_[j] = (min(m0 + r, p.M - 1) * p.K + wide_swz<BKT>(r, lane % Cfg::GRAN) * 8) * 2;
    }
#pragma unroll
    for (int j = 0; j < Cfg::DW; j++) {
        const int r = wave * (TN / 4) + Cfg::ROWS_PER_COPY * j + lane / Cfg::GRAN;
        off_w_[j] = (min(n0 + r, p.N - 1) * p.K + wide_swz<BKT>(r, lane % Cfg::GRAN) * 8) * 2;
    }
    const int *const off_a = off_a_, *const off_w = off_w_;
    // Copy number j of the DPW copies that this wavefront issues per k-tile (the first DA fill activation rows).  (A lambda
    // of the kernel, not a __device__ function template: the host pass marks such a template invalid at its first use because
    // of the device-only builtins, and the second kernel instantiation that calls it then fails to compile.)
    // The k-tile enters through the descriptor's base (and shortens its size), not through the instruction's scalar offset:
    // the hardware's range check does not see the scalar offset, and with it a partial last k-tile could reach up to 112
    // bytes past the end of the operand instead of reading zeros.
    auto issue_copy = [&](int j, char *stage, int k_off) {
        if (j < Cfg::DA) {
            const __amdgpu_buffer_rsrc_t rs_a =
                __builtin_amdgcn_make_buffer_rsrc(const_cast<char *>(reinterpret_cast<const char *>(p.A)) + k_off, 0, p.a_bytes - k_off, 0x00020000);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(
                rs_a, (__attribute__((address_space(3))) void *)(stage + (wave * (TM / 4) + Cfg::ROWS_PER_COPY * j) * ROW_BYTES), 16, off_a[j], 0, 0, 0);
        } else {
            const __amdgpu_buffer_rsrc_t rs_w =
                __builtin_amdgcn_make_buffer_rsrc(const_cast<char *>(reinterpret_cast<const char *>(p.Bt)) + k_off, 0, p.bt_bytes - k_off, 0x00020000);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(
                rs_w, (__attribute__((address_space(3))) void *)(stage + (TM + wave * (TN / 4) + Cfg::ROWS_PER_COPY * (j - Cfg::DA)) * ROW_BYTES), 16,
                off_w[j - Cfg::DA], 0, 0, 0);
        }
    };
    int issued = 0;           // k-tiles whose copies have been issued
    unsigned issue_stage = 0; // byte offset of the stage the next copies fill
    auto issue_begin = [&]() { return (k_begin + issued * BKT) * 2; };
    auto issue_end = [&]() {
        issued++;
        issue_stage = issue_stage + STAGE_BYTES == STAGES * STAGE_BYTES ? 0u : issue_stage + STAGE_BYTES;
    };

    // ---- operand reads: LDS byte offsets (within a stage) of this lane's slices for its KS steps
    unsigned off_fa_[Cfg::KS], off_fw_[Cfg::KS];
#pragma unroll
    for (int j = 0; j < KS; j++) {
        const int g = wide_swz<BKT>(frag_row, 2 * (wk * KS + j) + frag_g);
        off_fa_[j] = (wm * 128 + frag_row) * ROW_BYTES + g * 16;
        off_fw_[j] = (TM + wn * 128 + frag_row) * ROW_BYTES + g * 16;
    }
    const unsigned *const off_fa = off_fa_, *const off_fw = off_fw_;
    // read number i (0..7) of a step: activation block 0, the four weight blocks, activation blocks 1..3
    auto read_one = [&](int i, unsigned aa, unsigned ww, half8_t (&fa)[4], half8_t (&fw)[4]) {
        if (WIDE_TUNE & 4) return;
        switch (i) {
        case 0: ds_read_b128_at<0>(fa[0], aa); break;
        case 1: ds_read_b128_at<0>(fw[0], ww); break;
        case 2: ds_read_b128_at<BLK>(fw[1], ww); break;
        case 3: ds_read_b128_at<2 * BLK>(fw[2], ww); break;
        case 4: ds_read_b128_at<3 * BLK>(fw[3], ww); break;
        case 5: ds_read_b128_at<BLK>(fa[1], aa); break;
        case 6: ds_read_b128_at<2 * BLK>(fa[2], aa); break;
        default: ds_read_b128_at<3 * BLK>(fa[3], aa); break;
        }
    };
    // everything this wavefront has read has landed; the registers the wait guards are its operands
    auto wait_reads = [&](half8_t (&fa)[4], half8_t (&fw)[4]) {
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(fa[0]), "+v"(fa[1]), "+v"(fa[2]), "+v"(fa[3]), "+v"(fw[0]), "+v"(fw[1]), "+v"(fw[2]), "+v"(fw[3])::"memory");
    };

    float16_t acc[4][4]; // [ni][mi]; D[i][j] of one: i (weight row n) = 8*(v/4) + 4*(lane/32) + v%4, j (activation row m) = lane%32
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;

    half8_t fa[2][4], fw[2][4];
    // One 16-wide step: the 16 MFMAs on register set C, and between them, one at a time, the eight operand reads of the
    // next step into the other set (RD) and this k-tile's copies (DMA).
    auto step = [&](auto cc, auto rdc, auto dmac, unsigned aa, unsigned ww) {
        constexpr int C = decltype(cc)::value;
        constexpr bool RD = decltype(rdc)::value != 0, DMA = decltype(dmac)::value != 0;
        const int k_off = issue_begin();
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int mi = i >> 2, ni = i & 3;
            if (!(WIDE_TUNE & 1)) acc[ni][mi] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fw[C][ni], fa[C][mi], acc[ni][mi], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            if (RD && i < 8) {
                read_one(i, aa, ww, fa[C ^ 1], fw[C ^ 1]);
                __builtin_amdgcn_sched_barrier(0);
            }
#if WIDE_DMA_SLOTS == 1
            if (DMA && !(WIDE_TUNE & 2) && i >= 8) { // the copies in the second half of the step, the reads in the first
#pragma unroll
                for (int j = ((i - 8) * DPW) / 8; j < ((i - 7) * DPW) / 8; j++) issue_copy(j, lds_wide + issue_stage, k_off);
                __builtin_amdgcn_sched_barrier(0);
            }
#else
            if (DMA && !(WIDE_TUNE & 2)) { // the copies spread evenly over the step
#pragma unroll
                for (int j = (i * DPW) / 16; j < ((i + 1) * DPW) / 16; j++) issue_copy(j, lds_wide + issue_stage, k_off);
                __builtin_amdgcn_sched_barrier(0);
            }
#endif
        }
        if (DMA) issue_end();
        // The reads were issued at least eight MFMAs ago and have landed: the wait costs nothing here, and it makes the
        // registers hold their values before control flow can merge.  (The compiler takes the outputs of the read statements
        // for written when they are issued; a register copy that it inserts where two paths join would otherwise copy what
        // has not arrived yet.)
        if (RD) wait_reads(fa[C ^ 1], fw[C ^ 1]);
    };
    using c0 = std::integral_constant<int, 0>;
    using c1 = std::integral_constant<int, 1>;
    // One k-tile that has a successor (all such tiles are full).  On entry its first step's operands are in set P0.  At the
    // start of its last step the wavefront has all its operands of this tile in registers: it waits for its
    // own copies of tile kt+1 (at most `allow` copies outstanding), passes the barrier that publishes that tile and frees
    // this tile's stage, and during the step requests the first step of tile kt+1 and (DMA) refills this tile's stage with
    // tile kt + STAGES.
    auto full_tile = [&](auto p0c, auto dmac, unsigned sb, unsigned sb_next, int allow) {
        constexpr int P0 = decltype(p0c)::value;
#pragma unroll
        for (int j = 0; j + 1 < KS; j++) {
            if ((P0 + j) & 1) step(c1{}, c1{}, c0{}, sb + off_fa[j + 1 < KS ? j + 1 : 0], sb + off_fw[j + 1 < KS ? j + 1 : 0]);
            else step(c0{}, c1{}, c0{}, sb + off_fa[j + 1 < KS ? j + 1 : 0], sb + off_fw[j + 1 < KS ? j + 1 : 0]);
        }
        constexpr int PL = (P0 + KS - 1) & 1;
        if (!(WIDE_TUNE & 2)) wide_wait_copies(allow);
        if (!(WIDE_TUNE & 8)) __builtin_amdgcn_s_barrier();
        step(std::integral_constant<int, PL>{}, c1{}, dmac, sb_next + off_fa[0], sb_next + off_fw[0]);
    };
    // The last k-tile, full or partial: straight-line code over all KS steps (no second path for the accumulators to be
    // merged from); the steps of this wavefront that lie beyond K multiply zeros (what the copies fetched there is dropped).
    const int last_steps = ((k_end - k_begin) - (n_ktiles - 1) * BKT + 15) / 16; // 16-wide steps of the last k-tile
    const int n_my = max(0, min(KS, last_steps - wk * KS));
    auto last_tile = [&](unsigned sb) {
#pragma unroll
        for (int j = 0; j < KS; j++) {
            const int par = j & 1;
            if (j >= n_my) {
#pragma unroll
                for (int i = 0; i < 4; i++)
#pragma unroll
                    for (int e = 0; e < 8; e++) {
                        fa[par][i][e] = (half_t)0.0f;
                        fw[par][i][e] = (half_t)0.0f;
                    }
            }
            const unsigned aa = sb + off_fa[j + 1 < KS ? j + 1 : 0], ww = sb + off_fw[j + 1 < KS ? j + 1 : 0];
            if (j + 1 < KS) {
                if (par) step(c1{}, c1{}, c0{}, aa, ww);
                else step(c0{}, c1{}, c0{}, aa, ww);
            } else {
                if (par) step(c1{}, c0{}, c0{}, aa, ww);
                else step(c0{}, c0{}, c0{}, aa, ww);
            }
        }
    };

    // ---- the k-loop.  Iteration kt < n_dma refills its stage (tile kt + STAGES); the rest drain.
    {
        const int first = min(STAGES, n_ktiles);
        for (int i = 0; i < first; i++) {
            const int k_off = issue_begin();
#pragma unroll
            for (int j = 0; j < DPW; j++) issue_copy(j, lds_wide + issue_stage, k_off);
            issue_end();
        }
        wide_wait_copies((first - 1) * DPW);
        __builtin_amdgcn_s_barrier(); // tile 0 is visible
#if WIDE_TUNE & 16
        stamp[1] = wall_clock64();
#endif
        const int n_full = n_ktiles - 1;             // k-tiles with a successor
        const int n_dma = max(0, n_ktiles - STAGES); // ... of which the first n_dma issue copies
        constexpr int STEADY = (STAGES - 2) * DPW;   // copies that may be outstanding when tile kt+1 is needed, in steady state
        unsigned sb = 0;
        auto next_sb = [&](unsigned s) { return s + STAGE_BYTES == STAGES * STAGE_BYTES ? 0u : s + STAGE_BYTES; };
        auto drain_allow = [&](int kt) { return (n_ktiles - 2 - kt) * DPW; }; // tiles kt+2 .. n_ktiles-1 may still be on their way
        int kt = 0;
        if constexpr (KS % 2 == 1) {
            // the register set of a tile's first step alternates from tile to tile: start so that the last tile finds its
            // first step in set 0
            if (n_full & 1) {
#pragma unroll
                for (int i = 0; i < 8; i++) read_one(i, off_fa[0], off_fw[0], fa[1], fw[1]);
                wait_reads(fa[1], fw[1]);
                const unsigned s1 = next_sb(sb);
                if (n_dma > 0) full_tile(c1{}, c1{}, sb, s1, STEADY);
                else full_tile(c1{}, c0{}, sb, s1, drain_allow(0));
                sb = s1;
                kt = 1;
            } else {
#pragma unroll
                for (int i = 0; i < 8; i++) read_one(i, off_fa[0], off_fw[0], fa[0], fw[0]);
                wait_reads(fa[0], fw[0]);
            }
            for (; kt + 1 < n_dma; kt += 2) {
                const unsigned s1 = next_sb(sb), s2 = next_sb(s1);
                full_tile(c0{}, c1{}, sb, s1, STEADY);
                full_tile(c1{}, c1{}, s1, s2, STEADY);
                sb = s2;
            }
            if (kt < n_dma) { // the pair that holds the last copying tile
                const unsigned s1 = next_sb(sb), s2 = next_sb(s1);
                full_tile(c0{}, c1{}, sb, s1, STEADY);
                full_tile(c1{}, c0{}, s1, s2, drain_allow(kt + 1));
                sb = s2;
                kt += 2;
            }
            for (; kt < n_full; kt += 2) {
                const unsigned s1 = next_sb(sb), s2 = next_sb(s1);
                full_tile(c0{}, c0{}, sb, s1, drain_allow(kt));
                full_tile(c1{}, c0{}, s1, s2, drain_allow(kt + 1));
                sb = s2;
            }
        } else {
#pragma unroll
            for (int i = 0; i < 8; i++) read_one(i, off_fa[0], off_fw[0], fa[0], fw[0]);
            wait_reads(fa[0], fw[0]);
            for (; kt < n_dma; kt++) {
                const unsigned s1 = next_sb(sb);
                full_tile(c0{}, c1{}, sb, s1, STEADY);
                sb = s1;
            }
            for (; kt < n_full; kt++) {
                const unsigned s1 = next_sb(sb);
                full_tile(c0{}, c0{}, sb, s1, drain_allow(kt));
                sb = s1;
            }
        }
        last_tile(sb);
    }
#if WIDE_TUNE & 16
    stamp[2] = wall_clock64();
#endif
    __builtin_amdgcn_s_barrier(); // every wavefront holds its last operands in registers: the staging area is free
#if WIDE_TUNE & 16
    stamp[3] = wall_clock64();
#endif

    // ---- the way out.  The accumulators hold, per lane, four consecutive n of one m, which straight to memory would be
    // 8-byte pieces 2N bytes apart.  A wavefront parks a block row (32 m x NW n) in its own LDS region, [m][n], reads it
    // back as full row segments, applies the epilogue and stores 16 bytes per lane.  With a split K the f32 partials go out
    // the same way.  vals[ni][v]: the finished sums of the block row's NI 32 x 32 blocks.
    auto store_rows = [&](auto nic, const float (&vals)[decltype(nic)::value][16], int mrow0, int ncol0, char *scratch) {
        constexpr int NI = decltype(nic)::value, NW = 32 * NI;
        constexpr int PH = NI == 4 ? WIDE_PITCH_H : WIDE_PITCH_H2, PF = NI == 4 ? WIDE_PITCH_F : WIDE_PITCH_F2;
        if (p.splits == 1) {
            half_t *sc = reinterpret_cast<half_t *>(scratch);
#pragma unroll
            for (int ni = 0; ni < NI; ni++)
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    half4_t o;
#pragma unroll
                    for (int e = 0; e < 4; e++) o[e] = (half_t)vals[ni][4 * q + e];
                    *reinterpret_cast<half4_t *>(sc + frag_row * PH + ni * 32 + 8 * q + 4 * frag_g) = o;
                }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // the wavefront reads back what its own lanes wrote
            constexpr int LPR = NW / 8; // lanes per row (16 or 8), 8 columns each
            const int nl = (lane % LPR) * 8, n = ncol0 + nl;
            if (n < p.N) {
                half8_t bias = {0, 0, 0, 0, 0, 0, 0, 0};
                if (EPI >= MOON_EPI_BIAS) bias = *reinterpret_cast<const half8_t *>(p.bias + n);
#pragma unroll
                for (int r = 0; r < 32 * LPR / 64; r++) {
                    const int ml = r * (64 / LPR) + lane / LPR, m = mrow0 + ml;
                    if (m >= p.M) continue;
                    const half8_t v = *reinterpret_cast<const half8_t *>(sc + ml * PH + nl);
                    half8_t res = {0, 0, 0, 0, 0, 0, 0, 0};
                    if (EPI == MOON_EPI_BIAS_RESID) res = *reinterpret_cast<const half8_t *>(p.resid + size_t(m) * p.N + n);
                    half8_t o;
#pragma unroll
                    for (int e = 0; e < 8; e++) {
                        half_t x = apply_epilogue_v<EPI>((float)v[e], bias[e]); // (float)v[e] rounds back to v[e]: the product as parked
                        if (EPI == MOON_EPI_BIAS_RESID) x = (half_t)((float)res[e] + (float)x);
                        o[e] = x;
                    }
                    *reinterpret_cast<half8_t *>(p.C + size_t(m) * p.N + n) = o;
                }
            }
        } else {
            float *sc = reinterpret_cast<float *>(scratch);
#pragma unroll
            for (int ni = 0; ni < NI; ni++)
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const float4 o = {vals[ni][4 * q], vals[ni][4 * q + 1], vals[ni][4 * q + 2], vals[ni][4 * q + 3]};
                    *reinterpret_cast<float4 *>(sc + frag_row * PF + ni * 32 + 8 * q + 4 * frag_g) = o;
                }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            constexpr int LPR = NW / 4; // lanes per row (32 or 16), 4 columns each
            const int nl = (lane % LPR) * 4, n = ncol0 + nl;
            if (n < p.N) {
#pragma unroll
                for (int r = 0; r < 32 * LPR / 64; r++) {
                    const int ml = r * (64 / LPR) + lane / LPR, m = mrow0 + ml;
                    if (m >= p.M) continue;
                    *reinterpret_cast<float4 *>(p.partial + (size_t(split) * p.M + m) * p.N + n) = *reinterpret_cast<const float4 *>(sc + ml * PF + nl);
                }
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // read back before the next block row is parked
        __builtin_amdgcn_sched_barrier(0);
    };

    if constexpr (WK == 1) {
        // every wavefront owns its 128 x 128: four block rows, each through this wavefront's 32 KiB of the staging area
        char *scratch = lds_wide + size_t(wave) * 32768;
        auto out_row = [&](auto mic) {
            constexpr int mi = decltype(mic)::value;
            float vals[4][16];
#pragma unroll
            for (int ni = 0; ni < 4; ni++)
#pragma unroll
                for (int v = 0; v < 16; v++) vals[ni][v] = acc_read(acc[ni][mi][v]);
            store_rows(std::integral_constant<int, 4>{}, vals, m0 + wm * 128 + mi * 32, n0 + wn * 128, scratch);
        };
        out_row(std::integral_constant<int, 0>{});
        out_row(std::integral_constant<int, 1>{});
        out_row(std::integral_constant<int, 2>{});
        out_row(std::integral_constant<int, 3>{});
    } else {
        // ---- sum over the WK wavefronts that share an output tile.  Block row mi belongs to the wavefront with
        // wk == mi % WK.  Two rounds, each over two of the four 32-wide column blocks: every wavefront writes the blocks it
        // does not own to LDS ([4 registers][lane][4 floats] per 32 x 32 block, 4 KiB, straight from the accumulation
        // registers), barrier, every owner adds what the others left for it to its own, in the order wk = 0, 1, .. whoever
        // the owner is, and sends the finished half block row on its way; barrier before the regions are rewritten.
        // Which accumulators a wavefront keeps depends on its wk, and accumulators are registers, so this code exists once
        // per value of wk.  LDS: [wavefront][foreign block row f][column block of the round] blocks, then 9 KiB of parking
        // space per wavefront.
        constexpr int NF = WK == 4 ? 3 : 2;    // foreign block rows per wavefront
        constexpr unsigned XW = NF * 2 * 4096; // bytes a wavefront writes per round
        static_assert(4 * XW + 4 * 9216 <= Cfg::LDS_BYTES, "exchange and parking space fit the staging area");
        char *park = lds_wide + 4 * XW + size_t(wave) * 9216;
        auto finish = [&](auto wkc) {
            constexpr int WKV = decltype(wkc)::value;
#pragma unroll
            for (int round = 0; round < 2; round++) {
                // foreign blocks out
                const unsigned mine = wave * XW + lane * 16;
#pragma unroll
                for (int mi = 0; mi < 4; mi++) {
                    if (mi % WK == WKV) continue;
                    const int f = WK == 4 ? (mi < WKV ? mi : mi - 1) : (mi >> 1);
#pragma unroll
                    for (int h = 0; h < 2; h++) {
                        const int ni = 2 * round + h;
#pragma unroll
                        for (int q = 0; q < 4; q++) {
                            const float4 o = {acc_read(acc[ni][mi][4 * q]), acc_read(acc[ni][mi][4 * q + 1]), acc_read(acc[ni][mi][4 * q + 2]),
                                              acc_read(acc[ni][mi][4 * q + 3])};
                            *reinterpret_cast<float4 *>(lds_wide + mine + unsigned((f * 2 + h) * 4096 + q * 1024)) = o;
                        }
                    }
                }
                lds_barrier();
                // own block rows in
#pragma unroll
                for (int mi = 0; mi < 4; mi++) {
                    if (mi % WK != WKV) continue;
                    float vals[2][16];
#pragma unroll
                    for (int h = 0; h < 2; h++) {
                        const int ni = 2 * round + h;
#pragma unroll
                        for (int src = 0; src < WK; src++) {
                            if (src == WKV) {
#pragma unroll
                                for (int v = 0; v < 16; v++) {
                                    const float own = acc_read(acc[ni][mi][v]);
                                    vals[h][v] = src == 0 ? own : vals[h][v] + own;
                                }
                            } else {
                                const int f = WK == 4 ? (mi < src ? mi : mi - 1) : (mi >> 1);
                                const float *theirs = reinterpret_cast<const float *>(lds_wide + size_t(wmn * WK + src) * XW + (f * 2 + h) * 4096) + lane * 4;
#pragma unroll
                                for (int q = 0; q < 4; q++) {
                                    const float4 v = *reinterpret_cast<const float4 *>(theirs + q * 256);
                                    if (src == 0) {
                                        vals[h][4 * q] = v.x;
                                        vals[h][4 * q + 1] = v.y;
                                        vals[h][4 * q + 2] = v.z;
                                        vals[h][4 * q + 3] = v.w;
                                    } else {
                                        vals[h][4 * q] += v.x;
                                        vals[h][4 * q + 1] += v.y;
                                        vals[h][4 * q + 2] += v.z;
                                        vals[h][4 * q + 3] += v.w;
                                    }
                                }
                            }
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    store_rows(std::integral_constant<int, 2>{}, vals, m0 + wm * 128 + mi * 32, n0 + wn * 128 + round * 64, park);
                }
                if (round == 0) lds_barrier(); // everything of this round has been read
            }
        };
        if constexpr (WK == 2) {
            if (wk == 0) finish(std::integral_constant<int, 0>{});
            else finish(std::integral_constant<int, 1>{});
        } else {
            if (wk == 0) finish(std::integral_constant<int, 0>{});
            else if (wk == 1) finish(std::integral_constant<int, 1>{});
            else if (wk == 2) finish(std::integral_constant<int, 2>{});
            else finish(std::integral_constant<int, 3>{});
        }
    }
#if WIDE_TUNE & 16
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    stamp[4] = wall_clock64();
    if (lane == 0 && p.partial && p.splits == 1)
        for (int i = 0; i < 5; i++) reinterpret_cast<long long *>(p.partial)[(size_t(blockIdx.x) * 4 + wave) * 5 + i] = stamp[i];
#endif
#endif // __HIP_DEVICE_COMPILE__
}

} // namespace
