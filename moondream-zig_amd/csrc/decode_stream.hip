// The greedy decode loop of the 24-layer decoder as ONE launch whose weight stream never stops (text_model.zig:106-345 with
// its KVCache :349-539 and the loop of moondream.zig:323-368): LM head, arg-max, embedding gather and per layer LayerNorm,
// qkv, partial rotary, cache append, attention, fc1 + GELU, out_proj, fc2 and both residual adds.
//
// 512 workgroups of 512 threads, two per compute unit, all resident for the whole call.  The two workgroups of a unit
// (head h, key split s) have different jobs, and between them they stream a fixed 1/256 of every matrix:
//   the ATTENTION workgroup owns everything that waits for other workgroups:
//     qkv      rows q, k, v [h*64 + s*8 + 0..7]: 24 rows of 4 KiB, 3 per wavefront
//     K, V     keys of split s of head h: about kv_len / 8 keys of 128 B each, twice
//     out^T    rows [h*64 + s*8 + 0..7] of out_proj^T ([d][d], row k = out_w[:, k]): the head's attention output times its rows
//     and reduces 8 elements of the new hidden state from everybody's partial sums
//   the MLP workgroup waits for nothing but the layer's hidden state:
//     fc1      rows [u*32, +32), 4 per wavefront; g_j = gelu(row j . ln + b) goes to LDS
//     fc2^T    the SAME 32 rows, stored transposed ([ffn][d]): g_j times row j accumulates the workgroup's share of
//              fc2(fc1) in registers -- the 8192-wide vector never leaves the workgroup and nothing waits for it
//   both take a share of the LM head's 51200 rows.
// out^T and fc2^T rows are read in column slices: a chunk is 256 columns of two adjacent rows (lanes 0-31 one row, lanes
// 32-63 the next), wavefront w owns columns [256 w, +256), so after one cross-lane add lane i < 32 of wavefront w holds
// elements 8 (32 w + i) .. +7 of the workgroup's partial vector: exactly what reducer 32 w + i needs, no LDS reduction.
// Every byte reaches its wavefront through a ring of 8 KiB of LDS (8 chunks of 1 KiB) filled by direct global -> LDS
// loads (no registers in between, buffer form: scalar descriptor + scalar offset + a per-lane offset).  The order of
// chunks is fixed for the whole call, so a wavefront can always request the next ones, whatever it is doing: it keeps
// AHEAD chunks requested beyond the one it reads, and while it waits for another workgroup's data it tops the ring up.
// Loads return in order, so a chunk has landed when at most AHEAD - 1 younger requests are outstanding, and everything
// requested before a poll has landed when the poll returns.
// What crosses workgroups per layer (device-coherent accesses; readers poll):
//   E2  q, k, v of the new token among the 8 attention workgroups of a head (192 values, each word tagged)
//   E3  the 8 split partials (o[64], m, l) of a head, merged by each of the 8 workgroups for itself (tagged words)
//   E4  8 f32 partial sums of fc2 (MLP workgroups) and 8 of out_proj (attention workgroups) per reducer, then a flag per
//       source wavefront; reducer r adds its 2 x 256 sources in a fixed order, applies the reference's rounding points
//       (f16 after each product, after each bias, after attn + mlp, after the residual) and publishes 8 elements of
//   E1  the new hidden state (2048 tagged values), which every workgroup polls
// Arithmetic: q, k, v, fc1 and LM-head rows are the dot products of gemv.hip (same lanes, same order); out_proj and fc2
// are summed in another order than there (per workgroup over its rows, then over workgroups), inside the reference's own
// freedom (its f32 summation order is not defined, hgemm_trans.zig:101), with every f16 rounding point kept.
// Every wait is bounded: when one expires the error word is raised, all later waits return at once, every wavefront
// still runs to the end of the call (on meaningless data), and the host reports the failure.
#include "decode_stream.hpp"
#include "norm.hpp"

namespace {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned long long u64;
typedef __amdgpu_buffer_rsrc_t rsrc_t;

constexpr int W = STREAM_THREADS / 64; // wavefronts per workgroup
static_assert(W == 8 && STREAM_GRID == 512, "the work split below is written for 2 x 256 workgroups of eight wavefronts");
constexpr int UNITS = STREAM_GRID / 2; // (head, split) pairs = reducers
constexpr int D_ = STREAM_D, HD = STREAM_HD, H_ = STREAM_H, SPL = 8;
constexpr int NQ = 24 / W;            // qkv rows per wavefront (attention workgroup)
constexpr int NF = 32 / W;            // fc1 rows per wavefront (MLP workgroup)
constexpr int NI = 256 / (8 * W);     // key chunks per wavefront: 8 keys per chunk, up to 256 keys per split
constexpr int RING = 8;               // chunks of 1 KiB per wavefront
constexpr int AHEAD = 6;              // chunks requested beyond the one being read
constexpr int AUX_NT = 2;             // non-temporal: the weights are read once per token
constexpr int AUX_SC1 = 16;           // device-coherent: written through to / read from beyond the per-XCD L2

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

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
// acc[i] += a * w[i]
__device__ __forceinline__ void axpy8(float (&acc)[8], float a, const u32x4 &w) {
    const half_t *h = reinterpret_cast<const half_t *>(&w);
#pragma unroll
    for (int i = 0; i < 8; i++) acc[i] = fmaf(a, (float)h[i], acc[i]);
}

__device__ __forceinline__ u64 ld64(const u64 *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void st64(u64 *p, u64 v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ uint32_t ld32(const uint32_t *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void st32(uint32_t *p, uint32_t v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ u64 pack_f(float v, uint32_t tag) { return ((u64)tag << 32) | (u64)__float_as_uint(v); }
__device__ __forceinline__ uint32_t pack_h(half_t v, uint32_t tag16) { return (tag16 << 16) | (uint32_t)__builtin_bit_cast(unsigned short, v); }
__device__ __forceinline__ half_t unpack_h(uint32_t w) { return __builtin_bit_cast(half_t, (unsigned short)(w & 0xffffu)); }

__device__ __forceinline__ void argmax_merge(float &best, int &idx, float ov, int oi) {
    if (ov > best || (ov == best && oi < idx)) {
        best = ov;
        idx = oi;
    }
}

// LDS map (bytes)
constexpr int LDS_RING = 0;                       // [W][RING] chunks of 1 KiB
constexpr int LDS_HID = W * RING * 1024;          // [2048] f16 hidden state as received
constexpr int LDS_X = LDS_HID + 4096;             // [2048] f16 LayerNorm output
constexpr int LDS_MISC = LDS_X + 4096;            // floats, see below
constexpr int M_RED16 = 0, M_SQ = 16, M_SATTN = 80, M_SCORE = 144, M_SRED = 400 /* [8][64] */, M_PART = 912 /* 528 */, M_G = 1440 /* 32 */,
              M_R4 = 1472 /* [4][16] */, M_BEST = 1536, M_IDX = 1544, M_TOK = 1552, M_QKVRAW = 1560 /* 192 halves = 96 floats */,
              M_KNEW = 1656 /* 64 halves */, M_VNEW = 1688 /* 64 halves */, M_END = 1720;
constexpr int LDS_BYTES = LDS_MISC + 7168;        // 79 KiB: exactly two workgroups per compute unit
static_assert(M_END * 4 <= 7168, "LDS map");

// LayerNorm of the 2048-wide row in s_hid into s_x: threads 0..255 hold 8 elements each and follow the arithmetic and
// summation order of layernorm_regs; every thread of the workgroup calls it.
__device__ __forceinline__ void ln_2048(const half_t *s_hid, const u32x4 &gv, const u32x4 &bv, half_t *s_x, float eps, float *s_red) {
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const bool act = t < 256;
    float xv[8];
    u32x4 raw = {0, 0, 0, 0};
    if (act) raw = *reinterpret_cast<const u32x4 *>(s_hid + 8 * t);
    const half_t *xh = reinterpret_cast<const half_t *>(&raw);
    float s = 0.0f;
#pragma unroll
    for (int k = 0; k < 8; k++) {
        xv[k] = (float)xh[k];
        s += xv[k];
    }
    s = wave_sum(s);
    lds_barrier();
    if (lane == 0) s_red[wave] = s;
    lds_barrier();
    float tot = 0.0f;
#pragma unroll
    for (int w = 0; w < 4; w++) tot += s_red[w];
    const float mean = tot / (float)D_;
    float m2 = 0.0f;
#pragma unroll
    for (int k = 0; k < 8; k++) {
        const float d = xv[k] - mean;
        m2 = fmaf(d, d, m2);
    }
    m2 = wave_sum(m2);
    lds_barrier();
    if (lane == 0) s_red[wave] = m2;
    lds_barrier();
    tot = 0.0f;
#pragma unroll
    for (int w = 0; w < 4; w++) tot += s_red[w];
    const float var = tot / (float)D_;
    const float rstd = 1.0f / sqrtf(var + eps);
    if (act) {
#pragma clang fp contract(off)
        const float mean_rstd = mean * rstd;
        const half_t *gh = reinterpret_cast<const half_t *>(&gv), *bh = reinterpret_cast<const half_t *>(&bv);
        u32x4 out = {0, 0, 0, 0};
        half_t *oh = reinterpret_cast<half_t *>(&out);
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const float n = xv[k] * rstd - mean_rstd;
            oh[k] = (half_t)(n * (float)gh[k] + (float)bh[k]);
        }
        *reinterpret_cast<u32x4 *>(s_x + 8 * t) = out;
    }
    lds_barrier();
}

__global__ __launch_bounds__(STREAM_THREADS) __attribute__((amdgpu_waves_per_eu(4, 4))) void decode_stream_kernel(StreamParams p) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    half_t *s_hid = reinterpret_cast<half_t *>(smem + LDS_HID);
    half_t *s_x = reinterpret_cast<half_t *>(smem + LDS_X);
    float *s_m = reinterpret_cast<float *>(smem + LDS_MISC);
    float *s_red16 = s_m + M_RED16, *sq = s_m + M_SQ, *sattn = s_m + M_SATTN, *sscore = s_m + M_SCORE, *sred = s_m + M_SRED,
          *spart = s_m + M_PART, *sg = s_m + M_G, *sr4 = s_m + M_R4, *s_best = s_m + M_BEST;
    int *s_idx = reinterpret_cast<int *>(s_m + M_IDX), *s_tok = reinterpret_cast<int *>(s_m + M_TOK);
    half_t *s_qkvraw = reinterpret_cast<half_t *>(s_m + M_QKVRAW), *sk_new = reinterpret_cast<half_t *>(s_m + M_KNEW),
           *sv_new = reinterpret_cast<half_t *>(s_m + M_VNEW);

    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6); // the wavefront index as a scalar
    const uint32_t lane_off = (uint32_t)lane * 16u;                              // a chunk of 1 KiB in a row
    const uint32_t pair_off = (uint32_t)(lane >> 5) * 4096u + (uint32_t)(lane & 31) * 16u; // 512 B of each of two adjacent rows
    const bool mlp = (blockIdx.x & 1) != 0; // the workgroup's job
    const int u = blockIdx.x >> 1, h = u >> 3, s = u & 7;
    const int L = p.L, half_rot = p.rot_dim >> 1;
    unsigned char *ring = smem + LDS_RING + wave * (RING * 1024);
    int aborted = p.timeout_ticks < 0 ? 1 : 0; // (a negative bound: a timing build that waits for nobody)

    // rows of this wavefront, the same in every layer
    const int qx0 = wave * NQ, q_first = min(NQ, 8 - (qx0 & 7)); // qkv rows: entries qx0 .. +NQ-1 of the unit's list [q rows h*64 + s*8 + 0..7
    auto qkv_row = [&](int r) {                                  // | the same k rows | the same v rows]
        const int x = qx0 + r;
        return (x >> 3) * D_ + h * HD + s * 8 + (x & 7);
    };
    const int frow0 = u * 32 + wave * NF; // fc1 rows frow0 .. +NF-1
    const int gw = blockIdx.x * W + wave;
    int lm0, lm1; // LM head rows of this wavefront
    {
        const int nw = STREAM_GRID * W, qq = p.V / nw, rr = p.V % nw;
        lm0 = gw * qq + min(gw, rr);
        lm1 = lm0 + qq + (gw < rr ? 1 : 0);
    }
    const int lm_chunks = 4 * (lm1 - lm0);

    // ---------------------------------------------------------------------------------------------- the chunk stream
    // Every streamed weight lives in one allocation (at most 4 GiB): one descriptor, 32-bit byte offsets.  The wavefront's
    // chunk sequence is a list of runs with a constant stride.  Per step: its LM-head rows (one run, the rows are
    // adjacent); then per layer, attention workgroup: its qkv rows (one or two runs), its K chunks, its V chunks, its
    // slice of the 8 out_proj^T rows (4 chunks of two rows); MLP workgroup: its fc1 rows (one run), its slice of the 32
    // fc2^T rows (16 chunks of two rows).
    const rsrc_t r_w = __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t *>(p.w_base), 0, (int)(uint32_t)p.w_bytes, 0x00020000);
    const rsrc_t r_rp = __builtin_amdgcn_make_buffer_rsrc(p.rp, 0, (int)(STREAM_RP_FLOATS * sizeof(float)), 0x00020000);
    unsigned issued = 0, consumed = 0; // chunks requested / read so far by this wavefront
    int g_step = 0, g_l = lm_chunks > 0 ? -1 : 0, g_run = 0; // the next run: step, layer (-1: LM head), run within the layer
    rsrc_t run_rs = r_w;
    uint32_t run_off = 0, run_stride = 0;
    int run_left = 0;      // chunks of the current run not yet requested
    bool run_pair = false; // chunks of two half rows (pair_off) instead of 1 KiB in a row (lane_off)
    const int n_runs = mlp ? 2 : 5;
    // describes the next run (possibly an empty one); false at the end of the call
    auto next_run = [&]() -> bool {
        if (g_step >= p.n_steps) return false;
        const int l = g_l;
        run_rs = r_w;
        run_stride = 1024u;
        run_pair = false;
        if (l < 0) {
            run_off = p.off_lin + (uint32_t)lm0 * 4096u;
            run_left = lm_chunks;
            g_l = 0;
            g_run = 0;
            return true;
        }
        if (mlp) {
            if (g_run == 0) { // fc1 rows frow0 .. +NF-1
                run_off = p.off_fc1 + (uint32_t)(l * STREAM_FFN + frow0) * 4096u;
                run_left = 4 * NF;
            } else { // columns [256 wave, +256) of fc2^T rows u*32 + 0..31, two rows per chunk
                run_off = p.off_fc2t + (uint32_t)(l * STREAM_FFN + u * 32) * 4096u + (uint32_t)wave * 512u;
                run_stride = 8192u;
                run_left = 16;
                run_pair = true;
            }
            if (p.debug & 1) run_left = 0;
        } else {
            switch (g_run) {
            case 0: // qkv rows of the first part
                run_off = p.off_qkv + (uint32_t)(l * 3 * D_ + (qx0 >> 3) * D_ + h * HD + s * 8 + (qx0 & 7)) * 4096u;
                run_left = 4 * q_first;
                break;
            case 1: // ... and of the next part
                run_off = p.off_qkv + (uint32_t)(l * 3 * D_ + ((qx0 >> 3) + 1) * D_ + h * HD + s * 8) * 4096u;
                run_left = 4 * (NQ - q_first);
                break;
            case 2: // K: 8 keys per chunk, rows j0 + wave*8 + 64 i .. +7 of head h; nothing at or beyond the new position is read
            case 3: { // V
                const int pos = p.pos0 + g_step, kv_len = pos + 1, per = (kv_len + SPL - 1) / SPL;
                const int j0 = s * per, j1 = min(kv_len, j0 + per);
                const half_t *base = (g_run == 2 ? p.cache_k : p.cache_v) + (size_t(l) * H_ + h) * p.max_seq * HD;
                run_rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t *>(base), 0, __builtin_amdgcn_readfirstlane(min(j1, pos) * (HD * 2)), 0x00020000);
                run_off = (uint32_t)(j0 + wave * 8) * (HD * 2);
                run_stride = 8 * W * HD * 2;
                run_left = NI;
                break;
            }
            default: // columns [256 wave, +256) of out_proj^T rows h*64 + s*8 + 0..7, two rows per chunk
                run_off = p.off_outt + (uint32_t)(l * D_ + h * HD + s * 8) * 4096u + (uint32_t)wave * 512u;
                run_stride = 8192u;
                run_left = 4;
                run_pair = true;
                break;
            }
        }
        if (++g_run >= n_runs) {
            g_run = 0;
            if (++g_l >= L) {
                g_l = lm_chunks > 0 ? -1 : 0;
                g_step++;
            }
        }
        return true;
    };
    // requests the next chunk of the wavefront's sequence into the next ring slot; false when the ring is full or the call's
    // last chunk has been requested
    auto request_next = [&]() -> bool {
        if (issued - consumed >= (unsigned)RING) return false;
        while (run_left == 0)
            if (!next_run()) return false;
        auto lds = (__attribute__((address_space(3))) void *)(ring + (issued & (RING - 1)) * 1024);
        if (run_pair) __builtin_amdgcn_raw_ptr_buffer_load_lds(run_rs, lds, 16, pair_off, run_off, 0, AUX_NT);
        else __builtin_amdgcn_raw_ptr_buffer_load_lds(run_rs, lds, 16, lane_off, run_off, 0, AUX_NT);
        run_off += run_stride;
        run_left--;
        issued++;
        return true;
    };
    auto top_up = [&](unsigned ahead) {
        while (issued - consumed < ahead && request_next()) {
        }
    };
    // the next chunk of the sequence: this lane's 16 bytes of it
    auto read_chunk = [&]() -> u32x4 {
        // AHEAD - 1 requests are younger than this chunk (more only if a poll has returned since they were made); at the end
        // of the call, when there is nothing left to request, fewer are, and everything outstanding is waited for
        if (issued - consumed >= (unsigned)AHEAD) wait_vmcnt<AHEAD - 1>();
        else wait_vmcnt<0>();
        const u32x4 v = *reinterpret_cast<const u32x4 *>(ring + (consumed & (RING - 1)) * 1024 + lane_off);
        consumed++;
        top_up(AHEAD);
        return v;
    };
    // Wave-uniform bounded wait: poll() performs the wavefront's loads and says, per lane, whether its words carry the tag.
    // While they do not, the ring is topped up.  Returns when every lane's do, or when the wait is given up (aborted is then
    // set and stays set: all later waits of this wavefront return after a single poll).
    auto wave_wait = [&](auto poll) {
        long long t0 = 0;
        for (unsigned n = 1;; n++) {
            const bool ok = poll();
            if (aborted || __builtin_amdgcn_ballot_w64(!ok) == 0) return;
            top_up(RING);
            if ((n & 31u) == 0) {
                if (__builtin_amdgcn_readfirstlane((int)ld32(p.error)) != 0) {
                    aborted = 1;
                    return;
                }
                const long long now = wall_clock64();
                if (t0 == 0) t0 = now;
                else if (now - t0 > p.timeout_ticks) {
                    st32(p.error, 1u);
                    aborted = 1;
                    return;
                }
            }
        }
    };
    // hidden state published by the reducers of the layer-step with this tag -> s_hid (every thread: 4 elements)
    auto receive_hidden = [&](uint32_t tag) {
        const u64 *src = reinterpret_cast<const u64 *>(p.hid_t) + 2 * t;
        const uint32_t t16 = tag & 0xffffu;
        u64 a = 0, c = 0;
        wave_wait([&]() {
            a = ld64(src);
            c = ld64(src + 1);
            return ((uint32_t)(a >> 16 & 0xffffu) == t16) & ((uint32_t)(a >> 48) == t16) & ((uint32_t)(c >> 16 & 0xffffu) == t16) & ((uint32_t)(c >> 48) == t16);
        });
        const u64 v = (a & 0xffffull) | ((a >> 32 & 0xffffull) << 16) | ((c & 0xffffull) << 32) | ((c >> 32 & 0xffffull) << 48);
        *reinterpret_cast<u64 *>(s_hid + 4 * t) = v;
    };
    // dot product of the next row of the sequence (4 chunks) with the vector in xv, summed over the wavefront
    auto row_dot = [&](const u32x4 (&xv)[4]) -> float {
        float acc = 0.0f;
#pragma unroll
        for (int c = 0; c < 4; c++) acc = dot8(read_chunk(), xv[c], acc);
        return wave_sum(acc);
    };
    // E4, source side: lanes 0-31 of wavefront w hold elements 8 (32 w + lane) .. +7 of the workgroup's partial vector: 32
    // bytes into the source's 8 KiB block for reducer 32 w + lane (its slot rotated by the source index, so that the lines
    // a reducer reads are not 8 KiB apart), then, once the wavefront's stores have been acknowledged, the wavefront's flag
    auto publish_partial = [&](const float (&acc)[8], int kind, uint32_t tag) {
        if (lane < 32) {
            const uint32_t r = 32u * wave + lane, slot = (r + (uint32_t)u) & 255u;
            const uint32_t off = (((uint32_t)kind * UNITS + (uint32_t)u) * UNITS + slot) * 32u;
            __builtin_amdgcn_raw_buffer_store_b128(u32x4{__float_as_uint(acc[0]), __float_as_uint(acc[1]), __float_as_uint(acc[2]), __float_as_uint(acc[3])},
                                                   r_rp, (int)off, 0, AUX_SC1);
            __builtin_amdgcn_raw_buffer_store_b128(u32x4{__float_as_uint(acc[4]), __float_as_uint(acc[5]), __float_as_uint(acc[6]), __float_as_uint(acc[7])},
                                                   r_rp, (int)(off + 16u), 0, AUX_SC1);
        }
        wait_vmcnt<0>();
        if (lane == 0) st32(p.rp_flag + (kind * UNITS + u) * W + wave, tag);
    };

    top_up(AHEAD);
    for (int step = 0; step < p.n_steps; step++) {
        const int pos = p.pos0 + step;
        const bool tracing = p.trace && step == p.n_steps - 1 && t == 0;
        float rope_c = 1.0f, rope_s = 0.0f; // thread d < rot_dim: (cos, sin) of its pair at this position
        if (!mlp && t < p.rot_dim) {
            const int fi = t < half_rot ? t : t - half_rot;
            rope_c = p.freqs[(size_t(pos) * half_rot + fi) * 2];
            rope_s = p.freqs[(size_t(pos) * half_rot + fi) * 2 + 1];
        }
        // ------------------------------------------------------------------------------------------------ LM head + arg-max
        {
            u32x4 gv = {0, 0, 0, 0}, bv = {0, 0, 0, 0};
            if (t < 256) {
                gv = *reinterpret_cast<const u32x4 *>(p.lno_w + 8 * t);
                bv = *reinterpret_cast<const u32x4 *>(p.lno_b + 8 * t);
            }
            const int n_rows = lm1 - lm0;
            half_t bias_lane = (half_t)0.0f; // lane i holds the bias of row lm0 + i (rows beyond 64: reloaded below)
            if (lane < n_rows) bias_lane = p.lin_b[lm0 + lane];
            if (step == 0) {
                if (t < 256) {
                    const u32x4 v = *reinterpret_cast<const u32x4 *>(p.hidden_first + 8 * t);
                    *reinterpret_cast<u32x4 *>(s_hid + 8 * t) = v;
                }
            } else {
                receive_hidden(p.gen0 + (uint32_t)(step * L)); // after layer L-1 of the step before
            }
            lds_barrier();
            ln_2048(s_hid, gv, bv, s_x, p.eps, s_red16);
            u32x4 xv[4];
#pragma unroll
            for (int c = 0; c < 4; c++) xv[c] = *reinterpret_cast<const u32x4 *>(s_x + (c * 64 + lane) * 8);
            float best = -INFINITY;
            int best_i = 0x7fffffff;
            bool any = false;
#pragma unroll 1
            for (int i = 0; i < n_rows; i++) {
                if (i > 0 && (i & 63) == 0) bias_lane = (i + lane < n_rows) ? p.lin_b[lm0 + i + lane] : (half_t)0.0f; // (huge vocabularies only)
                const float dot = row_dot(xv);
                const half_t bias = __builtin_bit_cast(half_t, (unsigned short)__builtin_amdgcn_readlane((int)__builtin_bit_cast(unsigned short, bias_lane), i & 63));
                const int n = lm0 + i;
                const half_t v = apply_epilogue_v<MOON_EPI_BIAS>(dot, bias);
                if (lane == 0) p.logits[n] = v;
                float f = (float)v;
                if (n == 0 && f != f) f = INFINITY; // the reference starts from logits[0] and only moves on "greater"
                if (f > best || (!any && f == best)) {
                    best = f;
                    best_i = n;
                    any = true;
                }
            }
            if (lane == 0) {
                s_best[wave] = best;
                s_idx[wave] = best_i;
            }
            lds_barrier();
            const uint32_t atag = (p.gen0 + (uint32_t)(step * L) + 1u) & 0xffffu;
            if (t == 0) {
                for (int w = 1; w < W; w++) argmax_merge(best, best_i, s_best[w], s_idx[w]);
                st64(p.am_t + blockIdx.x, (u64)pack_h((half_t)best, atag) | ((u64)(uint32_t)best_i << 32));
            }
            {
                u64 pr = 0; // 512 pairs, one per thread
                wave_wait([&]() {
                    pr = ld64(p.am_t + t);
                    return (uint32_t)(pr >> 16 & 0xffffu) == atag;
                });
                best = (float)unpack_h((uint32_t)pr);
                best_i = (int)(uint32_t)(pr >> 32);
#pragma unroll
                for (int off = 32; off >= 1; off >>= 1) argmax_merge(best, best_i, __shfl_xor(best, off, 64), __shfl_xor(best_i, off, 64));
            }
            lds_barrier(); // s_best / s_idx of the first round have been read
            if (lane == 0) {
                s_best[wave] = best;
                s_idx[wave] = best_i;
            }
            lds_barrier();
            if (t == 0) {
                for (int w = 1; w < W; w++) argmax_merge(best, best_i, s_best[w], s_idx[w]);
                uint32_t tok = best_i == 0x7fffffff ? 0u : (uint32_t)best_i;
                if (tok >= (uint32_t)p.V) tok = 0u; // only after a failed wait
                *s_tok = (int)tok;
                if (blockIdx.x == 0) p.out_ids[step] = tok;
            }
            lds_barrier();
            // text_encoder (text_model.zig:121-134): the layer-0 input is the token's embedding row
            const uint32_t token = (uint32_t)*s_tok;
            if (t < 256) {
                const u32x4 e = *reinterpret_cast<const u32x4 *>(p.wte + size_t(token) * D_ + 8 * t);
                *reinterpret_cast<u32x4 *>(s_hid + 8 * t) = e;
            }
            lds_barrier();
        }

        for (int l = 0; l < L; l++) {
            const uint32_t tag = p.gen0 + (uint32_t)(step * L + l) + 1u, tag16 = tag & 0xffffu;
            long long *tr = tracing ? p.trace + (size_t(l) * STREAM_GRID + blockIdx.x) * 8 : nullptr;
            if (tr) tr[0] = wall_clock64();
            // small vectors of the layer: requested here, in front of the wait for the hidden state, whose poll they precede
            u32x4 gv = {0, 0, 0, 0}, bv = {0, 0, 0, 0};
            if (t < 256) {
                gv = *reinterpret_cast<const u32x4 *>(p.ln_w + size_t(l) * D_ + 8 * t);
                bv = *reinterpret_cast<const u32x4 *>(p.ln_b + size_t(l) * D_ + 8 * t);
            }
            half_t bias_lane = (half_t)0.0f; // lanes 0 .. 3: biases of the wavefront's qkv rows (attention) / fc1 rows (MLP)
            if (mlp) {
                if (lane < NF) bias_lane = p.fc1_b[size_t(l) * STREAM_FFN + frow0 + lane];
            } else if (lane < NQ) bias_lane = p.qkv_b[size_t(l) * 3 * D_ + qkv_row(lane)];
            half_t bo = (half_t)0.0f, b2 = (half_t)0.0f; // reducer: biases of its 8 elements
            if (!mlp && t < 8) {
                bo = p.out_b[size_t(l) * D_ + 8 * u + t];
                b2 = p.fc2_b[size_t(l) * D_ + 8 * u + t];
            }
            auto lane_bias = [&](int k) {
                return __builtin_bit_cast(half_t, (unsigned short)__builtin_amdgcn_readlane((int)__builtin_bit_cast(unsigned short, bias_lane), k));
            };
            // E1: the hidden state of this layer (layer 0: the embedding row, already in s_hid)
            if (l > 0) {
                receive_hidden(tag - 1u);
                lds_barrier();
            }
            if (tr) tr[1] = wall_clock64();
            ln_2048(s_hid, gv, bv, s_x, p.eps, s_red16);
            u32x4 xv[4];
#pragma unroll
            for (int c = 0; c < 4; c++) xv[c] = *reinterpret_cast<const u32x4 *>(s_x + (c * 64 + lane) * 8);

            if (mlp) {
                // ------------------------------------------------------------------------------------------ the MLP half
                // fc1 rows of the wavefront: g_j = gelu(row . ln + bias) -> LDS
#pragma unroll 1
                for (int i = 0; i < ((p.debug & 1) ? 0 : NF); i++) {
                    const float dot = row_dot(xv);
                    const half_t g = apply_epilogue_v<MOON_EPI_BIAS_GELU>(dot, lane_bias(i));
                    if (lane == 0) sg[wave * NF + i] = (float)g;
                }
                if (tr) tr[2] = wall_clock64();
                lds_barrier();
                // fc2^T: lanes 0-31 take row 2c, lanes 32-63 row 2c + 1 of chunk c, columns 256 wave + 8 (lane & 31) .. +7
                float acc2[8];
#pragma unroll
                for (int i = 0; i < 8; i++) acc2[i] = 0.0f;
#pragma unroll 1
                for (int c = 0; c < ((p.debug & 1) ? 0 : 16); c++) axpy8(acc2, sg[2 * c + (lane >> 5)], read_chunk());
#pragma unroll
                for (int i = 0; i < 8; i++) acc2[i] += __shfl_xor(acc2[i], 32, 64); // even rows + odd rows
                if (tr) tr[3] = wall_clock64();
                publish_partial(acc2, 0, tag);
                if (tr) tr[6] = wall_clock64();
                lds_barrier(); // sg is rewritten in the next layer
                continue;
            }

            // ------------------------------------------------------------------------------------------ the attention half
            // q, k, v rows of the wavefront -> E2
#pragma unroll 1
            for (int r = 0; r < NQ; r++) {
                const float dot = row_dot(xv);
                const half_t v = apply_epilogue_v<MOON_EPI_BIAS>(dot, lane_bias(r));
                if (lane == 0) st32(p.qkv_t + qkv_row(r), pack_h(v, tag16));
            }
            if (tr) tr[2] = wall_clock64();
            half_t *ck = p.cache_k + size_t(l) * H_ * p.max_seq * HD, *cv = p.cache_v + size_t(l) * H_ * p.max_seq * HD;
            const int kv_len = pos + 1, per = (kv_len + SPL - 1) / SPL;
            const int j0 = s * per, j1 = min(kv_len, j0 + per), nkeys = max(j1 - j0, 0);
            { // E2: q | k | v of head h, 96 pairs of tagged values; every wavefront waits for them, the first one keeps them
                const u64 *src = reinterpret_cast<const u64 *>(p.qkv_t);
                const int part = lane >> 5, pair = lane & 31; // first load: q (lanes 0-31) and k (32-63); second load: v
                u64 a = 0, c = 0;
                wave_wait([&]() {
                    a = ld64(src + (part * D_ + h * HD) / 2 + pair);
                    c = ld64(src + (2 * D_ + h * HD) / 2 + pair);
                    return ((uint32_t)(a >> 16 & 0xffffu) == tag16) & ((uint32_t)(a >> 48) == tag16) & ((uint32_t)(c >> 16 & 0xffffu) == tag16) &
                           ((uint32_t)(c >> 48) == tag16);
                });
                if (wave == 0) {
                    uint32_t *raw = reinterpret_cast<uint32_t *>(s_qkvraw);
                    raw[part * 32 + pair] = (uint32_t)(a & 0xffffu) | ((uint32_t)(a >> 32 & 0xffffu) << 16);
                    if (lane < 32) raw[64 + pair] = (uint32_t)(c & 0xffffu) | ((uint32_t)(c >> 32 & 0xffffu) << 16);
                }
            }
            if (tr) tr[3] = wall_clock64();
            lds_barrier();
            if (t < HD) {
#pragma clang fp contract(off)
                // rope.zig:223-224 on the first rot_dim dims of q and k; q stays f16-rounded like the reference's tensor
                const int d = t;
                const half_t *qr_ = s_qkvraw, *kr_ = s_qkvraw + HD, *vr_ = s_qkvraw + 2 * HD;
                sv_new[d] = vr_[d];
                if (d >= p.rot_dim) {
                    sq[d] = (float)qr_[d];
                    sk_new[d] = kr_[d];
                } else {
                    const int fi = d < half_rot ? d : d - half_rot;
                    const float c = rope_c, sn = rope_s;
                    const float qr = (float)qr_[fi], qi = (float)qr_[fi + half_rot], kr = (float)kr_[fi], ki = (float)kr_[fi + half_rot];
                    if (d < half_rot) {
                        sq[d] = (float)(half_t)(qr * c - qi * sn);
                        sk_new[d] = (half_t)(kr * c - ki * sn);
                    } else {
                        sq[d] = (float)(half_t)(qr * sn + qi * c);
                        sk_new[d] = (half_t)(kr * sn + ki * c);
                    }
                }
            }
            lds_barrier();
            if (pos >= j0 && pos < j1 && t < HD) { // updateCache (text_model.zig:476-515): this split owns the new position
                st_h<true>(ck + (size_t(h) * p.max_seq + pos) * HD + t, sk_new[t]);
                st_h<true>(cv + (size_t(h) * p.max_seq + pos) * HD + t, sv_new[t]);
                wait_vmcnt<0>(); // in memory before this workgroup publishes anything further
            }
            {
                const int g = lane >> 3, e = lane & 7;
                float qf[8];
#pragma unroll
                for (int i = 0; i < 8; i++) qf[i] = sq[8 * e + i];
#pragma unroll 1
                for (int i = 0; i < NI; i++) {
                    const int j = j0 + wave * 8 + g + 8 * W * i;
                    u32x4 kk = read_chunk(); // zeros at and beyond min(j1, pos)
                    if (j == pos) kk = *reinterpret_cast<const u32x4 *>(&sk_new[8 * e]);
                    const half_t *kh = reinterpret_cast<const half_t *>(&kk);
                    float sc = 0.0f;
#pragma unroll
                    for (int x = 0; x < 8; x++) sc = fmaf(qf[x], (float)kh[x], sc);
                    sc += __shfl_xor(sc, 1, 64);
                    sc += __shfl_xor(sc, 2, 64);
                    sc += __shfl_xor(sc, 4, 64);
                    if (e == 0 && j < j1) sscore[j - j0] = sc * 0.125f; // 1/sqrt(64), attention.zig:569
                }
                lds_barrier();
                // softmax statistics of the split, by every wavefront for itself (same values in each)
                float m = -INFINITY;
#pragma unroll
                for (int i = 0; i < 4; i++)
                    if (lane + 64 * i < nkeys) m = fmaxf(m, sscore[lane + 64 * i]);
                m = wave_max(m);
                float lsum = 0.0f;
#pragma unroll
                for (int i = 0; i < 4; i++)
                    if (lane + 64 * i < nkeys) lsum += __expf(sscore[lane + 64 * i] - m);
                lsum = wave_sum(lsum);
                float acc[8];
#pragma unroll
                for (int x = 0; x < 8; x++) acc[x] = 0.0f;
#pragma unroll 1
                for (int i = 0; i < NI; i++) {
                    const int j = j0 + wave * 8 + g + 8 * W * i;
                    u32x4 vv = read_chunk();
                    if (j == pos) vv = *reinterpret_cast<const u32x4 *>(&sv_new[8 * e]);
                    if (j < j1) {
                        const half_t *vh = reinterpret_cast<const half_t *>(&vv);
                        const float pj = __expf(sscore[j - j0] - m);
#pragma unroll
                        for (int x = 0; x < 8; x++) acc[x] = fmaf(pj, (float)vh[x], acc[x]);
                    }
                }
#pragma unroll
                for (int x = 0; x < 8; x++) {
                    acc[x] += __shfl_xor(acc[x], 8, 64);
                    acc[x] += __shfl_xor(acc[x], 16, 64);
                    acc[x] += __shfl_xor(acc[x], 32, 64);
                }
                if (g == 0) {
#pragma unroll
                    for (int x = 0; x < 8; x++) sred[wave * HD + 8 * e + x] = acc[x];
                }
                lds_barrier();
                u64 *dst = p.ap_t + (size_t(h) * SPL + s) * 66;
                if (t < HD) {
                    const float o = ((sred[0 * HD + t] + sred[1 * HD + t]) + (sred[2 * HD + t] + sred[3 * HD + t])) +
                                    ((sred[4 * HD + t] + sred[5 * HD + t]) + (sred[6 * HD + t] + sred[7 * HD + t]));
                    st64(dst + t, pack_f(o, tag));
                } else if (t == HD) st64(dst + HD, pack_f(m, tag));
                else if (t == HD + 1) st64(dst + HD + 1, pack_f(lsum, tag));
            }
            if (tr) tr[4] = wall_clock64();
            // E3: the 8 partials of the head, 528 words
            {
                const u64 *src = p.ap_t + size_t(h) * SPL * 66;
                u64 a = 0, c = pack_f(0.0f, tag);
                wave_wait([&]() {
                    a = ld64(src + t);
                    if (t < 16) c = ld64(src + 512 + t);
                    return ((uint32_t)(a >> 32) == tag) & ((uint32_t)(c >> 32) == tag);
                });
                spart[t] = __uint_as_float((uint32_t)a);
                if (t < 16) spart[512 + t] = __uint_as_float((uint32_t)c);
            }
            lds_barrier();
            if (t < HD) { // merge in split order (attention.zig:601-615: normalise by the reciprocal of the sum)
                float ms_[SPL], m = -INFINITY;
#pragma unroll
                for (int x = 0; x < SPL; x++) {
                    ms_[x] = spart[x * 66 + HD];
                    m = fmaxf(m, ms_[x]);
                }
                float lt = 0.0f, o = 0.0f;
#pragma unroll
                for (int x = 0; x < SPL; x++) {
                    const float wgt = (ms_[x] == -INFINITY) ? 0.0f : __expf(ms_[x] - m);
                    lt = fmaf(spart[x * 66 + HD + 1], wgt, lt);
                    o = fmaf(spart[x * 66 + t], wgt, o);
                }
                sattn[t] = (float)(half_t)f32_round(o * (1.0f / lt));
            }
            lds_barrier();
            if (tr) tr[5] = wall_clock64();
            // out_proj^T: chunk c holds rows 2c (lanes 0-31) and 2c + 1 (lanes 32-63) of this split's 8, columns 256 wave + ..
            float acco[8];
#pragma unroll
            for (int i = 0; i < 8; i++) acco[i] = 0.0f;
#pragma unroll 1
            for (int c = 0; c < 4; c++) axpy8(acco, sattn[s * 8 + 2 * c + (lane >> 5)], read_chunk());
#pragma unroll
            for (int i = 0; i < 8; i++) acco[i] += __shfl_xor(acco[i], 32, 64);
            publish_partial(acco, 1, tag);
            if (tr) tr[6] = wall_clock64();
            // E4, reducer side: this workgroup reduces elements 8u .. 8u+7.  Thread t < 256 takes source unit t: 8 sums of fc2
            // from its MLP workgroup, 8 of out_proj from its attention workgroup, both written by their wavefront u / 32
            float part[16];
#pragma unroll
            for (int i = 0; i < 16; i++) part[i] = 0.0f;
            if (wave < 4) {
                const uint32_t *flag0 = p.rp_flag + (0 * UNITS + t) * W + (u >> 5), *flag1 = p.rp_flag + (1 * UNITS + t) * W + (u >> 5);
                wave_wait([&]() { return (ld32(flag0) == tag) & (ld32(flag1) == tag); });
                const uint32_t slot = (uint32_t)((u + t) & 255);
                u32x4 v[4];
#pragma unroll
                for (int k = 0; k < 2; k++) {
                    const uint32_t off = (((uint32_t)k * UNITS + (uint32_t)t) * UNITS + slot) * 32u;
                    v[2 * k] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(r_rp, (int)off, 0, AUX_SC1));
                    v[2 * k + 1] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(r_rp, (int)(off + 16u), 0, AUX_SC1));
                }
#pragma unroll
                for (int i = 0; i < 4; i++)
#pragma unroll
                    for (int j = 0; j < 4; j++) part[4 * i + j] = __uint_as_float(v[i][j]);
                // sum over the 256 sources in a fixed order: over the lanes of a wavefront, then over the four wavefronts
#pragma unroll
                for (int i = 0; i < 16; i++) part[i] = wave_sum(part[i]);
                if (lane == 0) {
#pragma unroll
                    for (int i = 0; i < 16; i++) sr4[wave * 16 + i] = part[i];
                }
            }
            lds_barrier();
            if (wave == 0) {
                float tot = 0.0f;
                if (lane < 16) tot = (sr4[lane] + sr4[16 + lane]) + (sr4[32 + lane] + sr4[48 + lane]);
                const int e = lane & 7;
                const float fsum = __shfl(tot, e, 64), osum = __shfl(tot, 8 + e, 64);
                const half_t ao = apply_epilogue_v<MOON_EPI_BIAS>(osum, bo);       // attn_out = out_proj(attn) + bias
                const half_t ml = apply_epilogue_v<MOON_EPI_BIAS>(fsum, b2);       // mlp_out = fc2(fc1) + bias
                const half_t am = (half_t)((float)ao + (float)ml);                 // attn_out += mlp_out   (text_model.zig:170)
                const half_t hn = (half_t)((float)s_hid[8 * u + e] + (float)am);   // hidden += attn_out     (text_model.zig:171)
                const uint32_t wd = pack_h(hn, tag16);
                const uint32_t wd_hi = (uint32_t)__shfl_down((int)wd, 1, 64);
                if (lane < 8 && (lane & 1) == 0) st64(reinterpret_cast<u64 *>(p.hid_t) + 4 * u + (lane >> 1), (u64)wd | ((u64)wd_hi << 32));
            }
            lds_barrier(); // s_hid is overwritten by the next layer's hidden state
            if (tr) tr[7] = wall_clock64();
        }
    }
    // the hidden state after the last step, for the calls that follow (plain stores, visible at the end of the launch)
    if (blockIdx.x == 0) {
        receive_hidden(p.gen0 + (uint32_t)(p.n_steps * L));
        lds_barrier();
        if (t < 256) *reinterpret_cast<u32x4 *>(p.hidden_out + 8 * t) = *reinterpret_cast<const u32x4 *>(s_hid + 8 * t);
    }
}

} // namespace

bool decode_stream_supported(moon_ctx *ctx, size_t d, size_t ffn, size_t H, size_t D, size_t max_seq, size_t L, size_t V) {
    if (d != STREAM_D || ffn != STREAM_FFN || H != STREAM_H || D != STREAM_HD || max_seq > 2048) return false;
    if (2 * ctx->cu_count < STREAM_GRID) return false; // two workgroups per compute unit, all resident
    // the kernel addresses every streamed matrix with a 32-bit byte offset from one base
    if ((L * (3 * d * d + 2 * ffn * d + d * d) + V * d) * 2 >= (size_t(1) << 32) - 4096) return false;
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(decode_stream_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    int per_cu = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, reinterpret_cast<const void *>(decode_stream_kernel), STREAM_THREADS, LDS_BYTES) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    return per_cu >= 2;
}

int launch_decode_stream(moon_ctx *ctx, const StreamParams &p) {
    if (p.n_steps <= 0) return MOON_OK;
    if (p.rot_dim > STREAM_HD || p.rot_dim % 2) return moon_fail(ctx, MOON_EROT_DIM, "decode stream: bad rot_dim %d", p.rot_dim);
    if (p.max_seq > 2048 || p.pos0 + p.n_steps > p.max_seq)
        return moon_fail(ctx, MOON_ESEQ_TOO_LONG, "decode stream: %d + %d positions > max_seq %d (limit 2048)", p.pos0, p.n_steps, p.max_seq);
    if (p.V <= 0 || p.L <= 0) return moon_fail(ctx, MOON_EINVAL_DIM, "decode stream: empty model");
    // the attribute is per device; decode_stream_supported has set it on this one when the session was created
    hipLaunchKernelGGL(decode_stream_kernel, dim3(STREAM_GRID), dim3(STREAM_THREADS), LDS_BYTES, ctx->stream, p);
    MOON_HIP(ctx, hipGetLastError());
    return MOON_OK;
}
