// Matrix-core attention for multi-token queries: the causal prefill of the text decoder (32 heads x 64,
// attention.multiMaskedSDPA with the mask of createAttentionMask, attention.zig:256-281, 416-541) and the
// non-causal 729-token vision attention (16 heads x 72, attention.multiMasklessSDPA, attention.zig:125-234).
//
// One 256-thread workgroup owns 32 query rows of one head.  Its four wavefronts split the key range in tiles
// of 64 keys (wave w takes tiles w, w+4, ...), each running an online-softmax pass of its own over private LDS
// staging, so the main loop has no workgroup barrier; the four partial results (m, l, O) are merged through
// LDS at the end.  Per tile a wave computes, with v_mfma_f32_32x32x16_f16 and f32 accumulation,
//     S^T[key][q] = K . Q^T          (keys are the MFMA rows, so a lane holds 32 scores of ONE query and the
//                                      row maximum / sum are in-register reductions plus one cross-half exchange)
//     O^T[d][q]  += V^T . P^T        (P rounded to f16 for the matrix core; V is staged row-major and transposed by
//                                      the LDS load that feeds the matrix core)
// The scale 1/sqrt(D) multiplies the f32 product (attention.zig:192-194, 487-489), masked scores are -inf, the
// result is divided by the f32 row sum and rounded once to f16.
#include "epilogue.hpp"

#include <atomic>

namespace {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));

constexpr int FA_Q = 32;     // query rows per workgroup
constexpr int FA_KT = 64;    // keys per tile
constexpr int FA_WAVES = 4;

template <int D>
struct FaCfg {
    static constexpr int DK = (D + 15) / 16 * 16; // contraction length of K.Q^T, zero padded
    static constexpr int KSTEPS = DK / 16;
    static constexpr int DT = (D + 31) / 32;      // 32-row tiles of O^T, rows >= D are zero
    static constexpr int G = D / 8;               // 16-byte granules per row
    static constexpr int KS = DK + 8;             // K tile row stride in halfs: 36 or 44 dwords, conflict-free b128 reads
    // The V tile stays row-major, [key][d], and is read with the transposing LDS load (ds_read_tr16_b64).  Per half-wavefront
    // such a load touches 4 consecutive keys x 32 consecutive d: with D = 64 the rows are unpadded (32 dwords) and the 16-byte
    // granule c of key row r sits at granule c ^ 2*(r & 3), so those 4 x 4 granules fall on distinct banks and the b128
    // stores of two consecutive rows do too; otherwise the row stride is 48 dwords (rows 0..3 start at banks 0, 48, 32, 16).
    static constexpr bool V_SWIZZLE = (D == 64);
    static constexpr int VS = V_SWIZZLE ? D : 96; // V tile row stride in halfs
    static constexpr int K_HALFS = FA_KT * KS;
    static constexpr int V_HALFS = FA_KT * VS;
    // the K tile and the V tile of a wavefront share their LDS: K is only read before the scores, V only after
    static constexpr int WAVE_HALFS = K_HALFS > V_HALFS ? K_HALFS : V_HALFS;
    static constexpr int K_LOADS = (FA_KT * G + 63) / 64;       // 16-byte loads per lane for a K tile
    static constexpr bool FA_FULL_K = (FA_KT * G) % 64 == 0;    // every lane takes part in every K load
    // merge of the four wavefronts: O as [wave][q][SD] floats over the tiles (row stride D + 4: the 16-byte accesses of 16
    // consecutive q fall on distinct banks), the maxima and sums [wave][q] behind them in an area of their own
    static constexpr int SD = D + 4;
    static constexpr size_t MERGE_BYTES = size_t(FA_WAVES) * FA_Q * SD * sizeof(float);
    static constexpr size_t TILE_BYTES = size_t(FA_WAVES) * WAVE_HALFS * sizeof(half_t);
    static constexpr size_t ML_OFFSET = TILE_BYTES > MERGE_BYTES ? TILE_BYTES : MERGE_BYTES;
    static constexpr size_t LDS_BYTES = ML_OFFSET + 2 * FA_WAVES * FA_Q * sizeof(float);
};

struct FaArgs {
    const half_t *q, *k, *v;
    half_t *out;
    int H, Lq, Lkv;
    size_t q_head_stride, q_row_stride;   // element (h, r, d) of q sits at q[h * q_head_stride + r * q_row_stride + d]
    size_t kv_head_stride, kv_row_stride; // same for k and v
    long causal_pos; // key j is visible to query row r when causal_pos < 0 or j <= causal_pos + r
    int out_merged;  // 0: out[h][r][d], 1: out[r][h][d]
    float scale;
};

template <int D>
struct FaTileRegs {
    u32x4 k[FaCfg<D>::K_LOADS];
    u32x4 v[FaCfg<D>::K_LOADS];
};

// The K / V rows of a head are addressed as a buffer: a scalar descriptor of the head's rows, one 32-bit byte offset per
// lane that does not change from tile to tile, and the tile's first row as the scalar offset (fewer address registers
// and instructions than a 64-bit pointer per load, and the loads of a wavefront whose SIMD feeds the matrix core issue
// faster in this form).  Rows past the head's last read as zero (the descriptor ends there); their scores are masked.
typedef unsigned int fa_u32x4 __attribute__((ext_vector_type(4)));
template <int D>
__device__ __forceinline__ void fa_load_k(FaTileRegs<D> &r, __amdgpu_buffer_rsrc_t rs, int row_bytes, int key0, int lane) {
    using C = FaCfg<D>;
    const int tile_off = __builtin_amdgcn_readfirstlane(key0 * row_bytes); // (the same in every lane: a scalar operand)
#pragma unroll
    for (int i = 0; i < C::K_LOADS; i++) {
        const int g = i * 64 + lane;
        if (C::FA_FULL_K || g < FA_KT * C::G) {
            const int row = g / C::G, c = g % C::G;
            r.k[i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rs, row * row_bytes + c * 16, tile_off, 0));
        }
    }
}
template <int D>
__device__ __forceinline__ void fa_load_v(FaTileRegs<D> &r, __amdgpu_buffer_rsrc_t rs, int row_bytes, int key0, int lane) {
    using C = FaCfg<D>;
    const int tile_off = __builtin_amdgcn_readfirstlane(key0 * row_bytes);
#pragma unroll
    for (int i = 0; i < C::K_LOADS; i++) {
        const int g = i * 64 + lane;
        if (C::FA_FULL_K || g < FA_KT * C::G) {
            const int row = g / C::G, c = g % C::G;
            r.v[i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rs, row * row_bytes + c * 16, tile_off, 0));
        }
    }
}

template <int D>
__device__ __forceinline__ void fa_store_k(const FaTileRegs<D> &r, half_t *Ks, int lane) {
    using C = FaCfg<D>;
#pragma unroll
    for (int i = 0; i < C::K_LOADS; i++) {
        const int g = i * 64 + lane;
        if (C::FA_FULL_K || g < FA_KT * C::G) {
            const int row = g / C::G, c = g % C::G;
            *reinterpret_cast<u32x4 *>(Ks + row * C::KS + c * 8) = r.k[i];
        }
    }
    if (C::DK > D) { // zero padding of the contraction, columns [D, DK): one row per lane (the V tile overwrote it)
        static_assert(C::DK - D == 8 || C::DK == D, "one 16-byte granule of padding");
        *reinterpret_cast<u32x4 *>(Ks + lane * C::KS + D) = u32x4{0, 0, 0, 0};
    }
}
template <int D>
__device__ __forceinline__ void fa_store_v(const FaTileRegs<D> &r, half_t *Vs, int lane) {
    using C = FaCfg<D>;
#pragma unroll
    for (int i = 0; i < C::K_LOADS; i++) {
        const int g = i * 64 + lane;
        if (C::FA_FULL_K || g < FA_KT * C::G) {
            const int row = g / C::G, c = g % C::G;
            const int cs = C::V_SWIZZLE ? (c ^ (2 * (row & 3))) : c;
            *reinterpret_cast<u32x4 *>(Vs + row * C::VS + cs * 8) = r.v[i];
        }
    }
}
// Transposing LDS load: the 16 lanes of a quarter-wavefront each name 4 consecutive halfs; lane i of the quarter receives
// element i % 4 of the halfs named by lanes i / 4, i / 4 + 4, i / 4 + 8, i / 4 + 12.  When lane n names key n / 4, d-columns
// 4 * (n % 4) .. + 3 of a 4 x 16 block of row-major V, lane i ends up with column i of keys 0..3: V^T as the matrix core reads it.
__device__ __forceinline__ half4_t fa_read_tr(const half_t *p) {
    typedef short short4_t __attribute__((ext_vector_type(4)));
    return __builtin_bit_cast(half4_t, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4_t *)(p)));
}

template <int D>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void flash_attn_kernel(FaArgs p) {
    using C = FaCfg<D>;
    extern __shared__ __attribute__((aligned(16))) half_t smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6); // (wave: a scalar)
    const int col = lane & 31, hf = lane >> 5;
    const bool causal = p.causal_pos >= 0;
    // Workgroups are dealt to the eight accelerator dies round robin, and each die has an L2 of its own: when the count
    // divides, die x takes the x-th eighth of the (head, query block) list, so a head's K and V are fetched into one or two
    // L2s instead of all eight.
    int item = (int)(blockIdx.y * gridDim.x + blockIdx.x);
    const int n_items = (int)(gridDim.x * gridDim.y);
    if (n_items % 8 == 0) item = (item % 8) * (n_items / 8) + item / 8;
    int h = item / (int)gridDim.x, bx = item % (int)gridDim.x;
    // Late query blocks see the most keys: start them first.  Where a die's share is whole heads, its workgroups walk the
    // query blocks of all its heads together (block 23 of heads 0-3, block 22 of heads 0-3, ...): what is still to start when
    // the first workgroups leave is then the lightest blocks of every head, not all of the last head's.
    if (causal && n_items % 8 == 0 && (n_items / 8) % (int)gridDim.x == 0) {
        const int per_die = n_items / 8, heads_per_die = per_die / (int)gridDim.x, j = item % per_die;
        h = (item / per_die) * heads_per_die + j % heads_per_die;
        bx = j / heads_per_die;
    }
    const int qb = causal ? (int)gridDim.x - 1 - bx : bx;
    const int q0 = qb * FA_Q;
    half_t *Ks = smem + wave * C::WAVE_HALFS;
    half_t *Vs = Ks; // (shared with the K tile)
    // where this lane points the transposing loads of O^T row tile dt (see fa_read_tr): key 4*hf + (lane % 16) / 4 of the 8 keys
    // of a contraction half-step, d-columns 32*dt + 16*((lane / 16) % 2) + 4*(lane % 4) .. + 3.  Rows of O^T at or past D are
    // dropped, so the lanes that would name columns past the row name its last four instead.
    int voff[C::DT];
    {
        const int rq = (lane & 15) >> 2;
#pragma unroll
        for (int dt = 0; dt < C::DT; dt++) {
            int colh = 32 * dt + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
            if (C::V_SWIZZLE) colh = (((colh >> 3) ^ (2 * rq)) << 3) | (colh & 7);
            else colh = min(colh, D - 4);
            voff[dt] = (4 * hf + rq) * C::VS + colh;
        }
    }
    // this head's rows: (Lkv - 1) row strides and one row of D halfs
    const int row_bytes = (int)p.kv_row_stride * 2, head_bytes = (p.Lkv - 1) * row_bytes + D * 2;
    const __amdgpu_buffer_rsrc_t kh = __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t *>(p.k + size_t(h) * p.kv_head_stride), 0, head_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t vh = __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t *>(p.v + size_t(h) * p.kv_head_stride), 0, head_bytes, 0x00020000);

    // keys any row of this block can see
    long kv_end = p.Lkv;
    if (causal && p.causal_pos + q0 + FA_Q < kv_end) kv_end = p.causal_pos + q0 + FA_Q;
    const int n_tiles = (int)((kv_end + FA_KT - 1) / FA_KT);

    // The first K tile is requested before the query rows and the first V tile after them: the scores wait for K and Q only,
    // and the one round trip to memory that this wavefront cannot hide covers all three.
    FaTileRegs<D> regs;
    if (wave < n_tiles) fa_load_k<D>(regs, kh, row_bytes, wave * FA_KT, lane);

    // this lane's query row as the MFMA "B" operand: Q[q0 + col][16*s + 8*hf .. +7]
    half8_t qf[C::KSTEPS];
    {
        const int qrow = min(q0 + col, p.Lq - 1);
        const half_t *qp = p.q + size_t(h) * p.q_head_stride + size_t(qrow) * p.q_row_stride;
#pragma unroll
        for (int s = 0; s < C::KSTEPS; s++) {
            const int d = 16 * s + 8 * hf;
#pragma unroll
            for (int e = 0; e < 8; e++) qf[s][e] = (half_t)0.0f;
            if (d < D) qf[s] = *reinterpret_cast<const half8_t *>(qp + d);
        }
    }
    if (wave < n_tiles) fa_load_v<D>(regs, vh, row_bytes, wave * FA_KT, lane);

    float16_t o[C::DT];
#pragma unroll
    for (int dt = 0; dt < C::DT; dt++)
#pragma unroll
        for (int v = 0; v < 16; v++) o[dt][v] = 0.0f;
    float m_run = -INFINITY, l_run = 0.0f; // l_run: this lane's half of the row sum

    for (int t = wave; t < n_tiles; t += FA_WAVES) {
        asm volatile("" ::: "memory"); // the V tile of the previous iteration has been read: the K tile takes its place
        fa_store_k<D>(regs, Ks, lane);
        if (t + FA_WAVES < n_tiles) fa_load_k<D>(regs, kh, row_bytes, (t + FA_WAVES) * FA_KT, lane);
        const int key0 = t * FA_KT;

        float16_t s[2];
#pragma unroll
        for (int kt = 0; kt < 2; kt++) {
#pragma unroll
            for (int v = 0; v < 16; v++) s[kt][v] = 0.0f;
#pragma unroll
            for (int st = 0; st < C::KSTEPS; st++) {
                const half8_t a = *reinterpret_cast<const half8_t *>(Ks + (32 * kt + col) * C::KS + 16 * st + 8 * hf);
                s[kt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, qf[st], s[kt], 0, 0, 0);
            }
        }
        // s[kt][v] = score of key key0 + 32*kt + 8*(v/4) + 4*hf + v%4 against query q0 + col
        const bool edge = (key0 + FA_KT > p.Lkv) || (causal && (long)(key0 + FA_KT - 1) > p.causal_pos + q0);
        float mx = -INFINITY;
        // Scores stay unscaled in s; the scale (times log2 e) enters in the one fma that feeds exp2.  The running maximum
        // m_run is kept in those units (scaled, base 2).
        if (edge) { // (a tile that needs no masking takes the other path: no compare, no branch per score)
            const long last_visible = causal ? min((long)p.Lkv - 1, p.causal_pos + q0 + col) : (long)p.Lkv - 1;
#pragma unroll
            for (int kt = 0; kt < 2; kt++)
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    const int key = key0 + 32 * kt + 8 * (v >> 2) + 4 * hf + (v & 3);
                    const float x = (long)key > last_visible ? -INFINITY : s[kt][v];
                    s[kt][v] = x;
                    mx = fmaxf(mx, x);
                }
        } else {
#pragma unroll
            for (int kt = 0; kt < 2; kt++)
#pragma unroll
                for (int v = 0; v < 16; v++) mx = fmaxf(mx, s[kt][v]);
        }
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        const float c2 = p.scale * 1.4426950408889634f; // > 0: the maximum of the scaled scores is the scaled maximum
        const float m_new = fmaxf(m_run, mx * c2);
        const float m_use = (m_new == -INFINITY) ? 0.0f : m_new; // a row that has seen no key yet
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_use);
        m_run = m_new;
        float psum = 0.0f;
#pragma unroll
        for (int kt = 0; kt < 2; kt++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const float e = __builtin_amdgcn_exp2f(__builtin_fmaf(s[kt][v], c2, -m_use));
                s[kt][v] = e;
                psum += e;
            }
        l_run = l_run * alpha + psum;
        // (rows of O^T at or past D are never read: in the last row tile only the registers of rows below D are rescaled;
        // the others hold whatever accumulates, each on its own)
#pragma unroll
        for (int dt = 0; dt < C::DT; dt++)
#pragma unroll
            for (int v = 0; v < 16; v++)
                if (32 * dt + 8 * (v >> 2) < D) o[dt][v] *= alpha;

        asm volatile("" ::: "memory"); // the K tile has been read (LDS serves a wavefront in order): V takes its place
        fa_store_v<D>(regs, Vs, lane);
        if (t + FA_WAVES < n_tiles) fa_load_v<D>(regs, vh, row_bytes, (t + FA_WAVES) * FA_KT, lane);
        // O^T += V^T . P^T : contraction step (kt, sp) uses the keys a lane already holds in s[kt][8*sp .. 8*sp+7],
        // i.e. key0 + 32*kt + 16*sp + {4*hf + 0..3, 8 + 4*hf + 0..3}
#pragma unroll
        for (int kt = 0; kt < 2; kt++)
#pragma unroll
            for (int sp = 0; sp < 2; sp++) {
                half8_t pb;
#pragma unroll
                for (int e = 0; e < 8; e++) pb[e] = (half_t)s[kt][8 * sp + e];
#pragma unroll
                for (int dt = 0; dt < C::DT; dt++) {
                    const half_t *vp = Vs + voff[dt] + (32 * kt + 16 * sp) * C::VS;
                    const half4_t lo = fa_read_tr(vp);
                    const half4_t hi = fa_read_tr(vp + 8 * C::VS);
                    half8_t a;
                    a[0] = lo[0]; a[1] = lo[1]; a[2] = lo[2]; a[3] = lo[3];
                    a[4] = hi[0]; a[5] = hi[1]; a[6] = hi[2]; a[7] = hi[3];
                    o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, pb, o[dt], 0, 0, 0);
                }
            }
    }

    // merge the four waves' partial results
    const float l_wave = l_run + __shfl_xor(l_run, 32);
    float *so = reinterpret_cast<float *>(smem);                                                        // [wave][q][SD]
    float *sm = reinterpret_cast<float *>(reinterpret_cast<char *>(smem) + C::ML_OFFSET);               // [wave][q]
    float *sl = sm + FA_WAVES * FA_Q;                                                                   // [wave][q]
    if (hf == 0) {
        sm[wave * FA_Q + col] = m_run;
        sl[wave * FA_Q + col] = l_wave;
    }
    __syncthreads(); // every wave is done with its staging area, which O takes over, and has published its maximum
    float m_all = -INFINITY;
#pragma unroll
    for (int w = 0; w < FA_WAVES; w++) m_all = fmaxf(m_all, sm[w * FA_Q + col]);
    const float f = (m_run == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f(m_run - m_all); // (maxima are in base-2 units)
#pragma unroll
    for (int dt = 0; dt < C::DT; dt++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int d = 32 * dt + 8 * j + 4 * hf; // o[dt][4*j .. 4*j+3] are rows d .. d+3 of O^T
            if (32 * dt + 8 * j < D) {
                float4 r;
                r.x = o[dt][4 * j] * f;
                r.y = o[dt][4 * j + 1] * f;
                r.z = o[dt][4 * j + 2] * f;
                r.w = o[dt][4 * j + 3] * f;
                *reinterpret_cast<float4 *>(so + (wave * FA_Q + col) * C::SD + d) = r;
            }
        }
    __syncthreads();
    {
        const int q = tid & 31;
        float l_all = 0.0f;
#pragma unroll
        for (int w = 0; w < FA_WAVES; w++) {
            const float mw = sm[w * FA_Q + q];
            if (mw != -INFINITY) l_all += __builtin_amdgcn_exp2f(mw - m_all) * sl[w * FA_Q + q];
        }
        const float inv = 1.0f / l_all;
        const int row = q0 + q;
        if (row < p.Lq) {
            for (int dg = tid >> 5; dg < C::G; dg += 8) {
                float acc[8];
#pragma unroll
                for (int e = 0; e < 8; e++) acc[e] = 0.0f;
#pragma unroll
                for (int w = 0; w < FA_WAVES; w++) {
                    const float4 a = *reinterpret_cast<const float4 *>(so + (w * FA_Q + q) * C::SD + dg * 8);
                    const float4 b = *reinterpret_cast<const float4 *>(so + (w * FA_Q + q) * C::SD + dg * 8 + 4);
                    acc[0] += a.x; acc[1] += a.y; acc[2] += a.z; acc[3] += a.w;
                    acc[4] += b.x; acc[5] += b.y; acc[6] += b.z; acc[7] += b.w;
                }
                half8_t r;
#pragma unroll
                for (int e = 0; e < 8; e++) r[e] = (half_t)(acc[e] * inv);
                const size_t oi = p.out_merged ? (size_t(row) * p.H + h) * D + dg * 8 : (size_t(h) * p.Lq + row) * D + dg * 8;
                *reinterpret_cast<half8_t *>(p.out + oi) = r;
            }
        }
    }
}

template <int D>
int launch_flash(moon_ctx *ctx, const FaArgs &p) {
    using C = FaCfg<D>;
    static std::atomic<bool> attr_set[64]; // the opt-in to this much dynamic LDS is per device (and per instantiation)
    const int dev = ctx->device >= 0 && ctx->device < 64 ? ctx->device : -1;
    if (dev < 0 || !attr_set[dev].load()) {
        MOON_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void *>(flash_attn_kernel<D>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                          (int)C::LDS_BYTES));
        if (dev >= 0) attr_set[dev].store(true);
    }
    hipLaunchKernelGGL(flash_attn_kernel<D>, dim3((unsigned)((p.Lq + FA_Q - 1) / FA_Q), (unsigned)p.H), dim3(256), C::LDS_BYTES, ctx->stream, p);
    MOON_HIP(ctx, hipGetLastError());
    MOON_NOTE_KERNEL(ctx, "flash_attn_kernel<%d> %d workgroups", D, (int)((p.Lq + FA_Q - 1) / FA_Q) * (int)p.H);
    return MOON_OK;
}

} // namespace

// Takes the call when the shape is one the matrix-core kernel is built for; otherwise *handled stays false and the
// caller falls back to the shape-generic kernel.
int launch_sdpa_mfma(moon_ctx *ctx, const half_t *q, const half_t *k, const half_t *v, half_t *out, size_t H, size_t Lq, size_t Lkv,
                     size_t D, size_t kv_head_stride, long causal_pos, bool out_merged, bool *handled) {
    *handled = false;
    if ((D != 64 && D != 72) || Lq < 16 || Lkv == 0 || H == 0 || H > 65535) return MOON_OK;
    if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out) % 16 || (kv_head_stride * sizeof(half_t)) % 16) return MOON_OK;
    if (Lkv * D * sizeof(half_t) >= (size_t(1) << 31)) return MOON_OK; // a head's rows are addressed with 32-bit offsets
    FaArgs p{q, k, v, out, (int)H, (int)Lq, (int)Lkv, Lq * D, D, kv_head_stride, D, causal_pos, out_merged ? 1 : 0, 1.0f / sqrtf((float)D)};
    *handled = true;
    return D == 64 ? launch_flash<64>(ctx, p) : launch_flash<72>(ctx, p);
}

// Non-causal attention straight from a packed projection qkv[T][3 * H * D] (row = q | k | v, heads side by side inside each
// third: vision_model.zig:285-314 splits and transposes it into three tensors first) to the merged layout out[T][H * D]
// that the output projection reads (vision_model.zig:326-335).  *handled stays false for shapes the kernel does not cover.
int launch_sdpa_packed_qkv(moon_ctx *ctx, const half_t *qkv, half_t *out, size_t H, size_t T, size_t D, bool *handled) {
    *handled = false;
    if ((D != 64 && D != 72) || T < 16 || H == 0 || H > 65535) return MOON_OK;
    if (((uintptr_t)qkv | (uintptr_t)out) % 16) return MOON_OK;
    const size_t d = H * D;
    if (T * 3 * d * sizeof(half_t) >= (size_t(1) << 31)) return MOON_OK; // (32-bit offsets within a head's rows)
    FaArgs p{qkv, qkv + d, qkv + 2 * d, out, (int)H, (int)T, (int)T, D, 3 * d, D, 3 * d, -1, 1, 1.0f / sqrtf((float)D)};
    *handled = true;
    return D == 64 ? launch_flash<64>(ctx, p) : launch_flash<72>(ctx, p);
}
