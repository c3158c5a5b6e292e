// The three kernels of one decoder layer at decode time (one token), and the LM head:
//   decode_ln_gemv_kernel      ln = LN(hidden);  y1 = ln.W1^T + b1  [and  y2 = gelu(ln.W2^T + b2)]
//                              (text_model.zig:154-160 + 193-196 + 310-315; with one matrix: lm_head, :331-342)
//   decode_attn_merged_kernel  rope + cache append + attention, the last split of a head merges it (:198-294)
//   decode_out_fc2_kernel      hidden += (attn.Wo^T + bo) + (fc1.Wfc2^T + b2)                       (:296-299, 317-320, 170-171)
// All are HBM bound: every weight byte is read once with 128-bit non-temporal loads, 8-20 loads in flight per
// lane, 2048 wavefronts (two 256-thread workgroups per CU).  Arithmetic, rounding points and summation orders are
// those of gemv.hip / norm.hpp / attn_decode.hpp, so the fused and the unfused paths produce the same bits.
#include "attn_decode.hpp"
#include "norm.hpp"
#include "sample_quick.hpp"
#include <algorithm>
#include <cmath>
#include <cstdlib>

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

__device__ __forceinline__ void split_rows(int n_rows, int n_waves, int w, int &begin, int &end) {
    const int q = n_rows / n_waves, r = n_rows % n_waves;
    begin = w * q + min(w, r);
    end = begin + q + (w < r ? 1 : 0);
}

// A wavefront's rows in up to two matrices of the same row length K, walked in groups of RG rows whose CH x RG
// 16-byte loads per lane are requested together (CH = ceil(K / 512) pieces of 64 lanes x 16 bytes per row).
template <int CH, int RG>
struct RowGroups {
    const half_t *W[2];
    int r0[2], n[2]; // first row and row count in each matrix
    int K, granules, total;
    u32x4 w[RG][CH];
    const half_t *bias[2];
    half_t bias_lane; // lane j < RG: bias of row j of the loaded group
    __device__ __forceinline__ void init(const half_t *W1, int a0, int a1, const half_t *W2, int b0, int b1, int K_,
                                         const half_t *bias1 = nullptr, const half_t *bias2 = nullptr) {
        W[0] = W1; W[1] = W2;
        bias[0] = bias1; bias[1] = bias2;
        bias_lane = (half_t)0.0f;
        r0[0] = a0; n[0] = a1 - a0;
        r0[1] = b0; n[1] = b1 - b0;
        K = K_;
        granules = K_ >> 3;
        total = n[0] + n[1];
    }
    // row i of the concatenated list -> (matrix, row)
    __device__ __forceinline__ void locate(int i, int &m, int &row) const {
        m = i < n[0] ? 0 : 1;
        row = i < n[0] ? r0[0] + i : r0[1] + (i - n[0]);
    }
    __device__ __forceinline__ void load(int first, int lane) {
        if (lane < RG && first + lane < total) { // the epilogue's bias values travel with the group
            int m, row;
            locate(first + lane, m, row);
            if (bias[m]) bias_lane = bias[m][row];
        }
#pragma unroll
        for (int j = 0; j < RG; j++) {
            int m, row;
            locate(min(first + j, total - 1), m, row); // rows past the end re-read the last row; their result is dropped
            const u32x4 *src = reinterpret_cast<const u32x4 *>(W[m] + size_t(row) * K);
#pragma unroll
            for (int c = 0; c < CH; c++) {
                const int g = c * 64 + lane;
                w[j][c] = u32x4{0, 0, 0, 0};
                if (g < granules && first + j < total) w[j][c] = __builtin_nontemporal_load(src + g);
            }
        }
    }
    // pieces [c0, c1) of the one row `first` (and, with c0 == 0, the row's bias), a wait after every CHUNK of them but
    // the last
    template <int CHUNK, int SLEEP = 0>
    __device__ __forceinline__ void load_pieces(int first, int lane, int c0, int c1) {
        static_assert(RG == 1, "one row");
        if (c0 == 0 && lane < RG && first + lane < total) {
            int m, row;
            locate(first + lane, m, row);
            if (bias[m]) bias_lane = bias[m][row];
        }
        int m, row;
        locate(min(first, total - 1), m, row);
        const u32x4 *src = reinterpret_cast<const u32x4 *>(W[m] + size_t(row) * K);
#pragma unroll
        for (int c = 0; c < CH; c++) {
            if (c < c0 || c >= c1) continue;
            const int g = c * 64 + lane;
            w[0][c] = u32x4{0, 0, 0, 0};
            if (g < granules && first < total) w[0][c] = __builtin_nontemporal_load(src + g);
            // A pause between two requests: the pieces wait for the fc1 vector anyway, and the less this wavefront has queued
            // the sooner the unit's dependent accesses are served (0.622 ms per token with 6 x 64 cycles, 0.632 / 0.628 / 0.640
            // with 4 / 8 / 10, 0.640-0.650 with none; before, the integer division of a run-time CHUNK happened to fill the gap).
            if (SLEEP > 0) __builtin_amdgcn_s_sleep(SLEEP);
            if (c + 1 < c1 && (c + 1 - c0) % CHUNK == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
    }
    // done(matrix, row, dot, bias) is called by all lanes
    template <class Done>
    __device__ __forceinline__ void consume(int first, const u32x4 (&xv)[CH], Done done) {
        const half_t group_bias = bias_lane;
#pragma unroll
        for (int j = 0; j < RG; j++) {
            float s = 0.0f;
#pragma unroll
            for (int c = 0; c < CH; c++) s = dot8(w[j][c], xv[c], s);
            s = wave_sum(s);
            const half_t b = __builtin_bit_cast(half_t, (unsigned short)__builtin_amdgcn_readlane((int)__builtin_bit_cast(unsigned short, group_bias), j));
            if (first + j < total) {
                int m, row;
                locate(first + j, m, row);
                done(m, row, s, b);
            }
        }
    }
};

template <int CH>
__device__ __forceinline__ void load_x(u32x4 (&xv)[CH], const half_t *x_lds, int K, int lane) {
#pragma unroll
    for (int c = 0; c < CH; c++) {
        const int g = c * 64 + lane;
        xv[c] = u32x4{0, 0, 0, 0};
        if (g < (K >> 3)) xv[c] = *reinterpret_cast<const u32x4 *>(x_lds + size_t(g) * 8);
    }
}

struct LnGemvArgs {
    const half_t *x;           // [d] hidden vector (or an embedding table)
    const uint32_t *token;     // if not null: x = x + token[0] * d (embedding lookup on the device)
    const half_t *gamma, *beta;
    const half_t *W1, *b1;     // [N1, d]
    half_t *y1;
    const half_t *W2, *b2;     // [N2, d], may be null (N2 = 0)
    half_t *y2;
    int d, N1, N2;
    float eps;
};

// TWO: both matrices (a decoder layer's qkv + fc1); otherwise W1 alone (the LM head), a kernel of its own name so
// that profiles tell the two apart
template <int CH, bool TWO>
__global__ __launch_bounds__(256) void decode_ln_gemv_kernel(LnGemvArgs p) {
    extern __shared__ __attribute__((aligned(16))) half_t s_ln[]; // [d]
    __shared__ float s_red[16];
    constexpr int RG = 4;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n_waves = gridDim.x * 4, gw = blockIdx.x * 4 + wave;
    const half_t *x = p.token ? p.x + size_t(p.token[0]) * p.d : p.x;
    // LayerNorm inputs first (small, cached), then the first group of weight rows, then the LayerNorm arithmetic:
    // loads return in issue order, so the weights stream in while the statistics are reduced
    LnInput ln_in; // all of the LayerNorm input is requested before any of it is waited for
    ln_request<true>(ln_in, x, p.gamma, p.beta, p.d); // d % 8 == 0, rows of the model's own buffers
    int a0, a1, b0 = 0, b1 = 0;
    split_rows(p.N1, n_waves, gw, a0, a1);
    if (TWO) split_rows(p.N2, n_waves, gw, b0, b1);
    RowGroups<CH, RG> rows;
    rows.init(p.W1, a0, a1, p.W2, b0, b1, p.d, p.b1, p.b2);
    if (rows.total > 0) rows.load(0, lane);
    layernorm_regs(ln_in, s_ln, p.d, p.eps, s_red);
    lds_barrier();
    u32x4 xv[CH];
    load_x<CH>(xv, s_ln, p.d, lane);
    for (int first = 0; first < rows.total; first += RG) {
        rows.consume(first, xv, [&](int m, int n, float dot, half_t b) {
            if (lane == 0) {
                if (m == 0) p.y1[n] = apply_epilogue_v<MOON_EPI_BIAS>(dot, b);
                else p.y2[n] = apply_epilogue_v<MOON_EPI_BIAS_GELU>(dot, b);
            }
        });
        if (first + RG < rows.total) rows.load(first + RG, lane);
    }
}

// Final LayerNorm + LM head + greedy arg-max in one launch (text_model.zig:325-345; sampling.argmax, sampling.zig:257-273,
// first maximum wins, a NaN at index 0 is never displaced), with the greedy loop's bookkeeping:
// state[2] = token, out_ids[state[1]++] = token, state[0] += bump.  Every wavefront keeps the first maximum of its
// (ascending) rows; a workgroup stores its (value, index) pair, and the workgroup that counts in last merges the pairs.
struct LmHeadArgs {
    LnGemvArgs g;                  // y1 = logits, one matrix
    unsigned long long *partials;  // [grid] value bits << 32 | index, device-coherent
    uint32_t *counter;             // root (leaves complete), then 32 leaf lines (workgroups that stored their pair); monotonic over launches
    uint32_t generation;           // launches so far, this one included
    uint32_t *state;
    uint32_t *out_ids;
    uint32_t bump;
    // TOPK (the sampled loop with top_k < QUICK_KEYS): partials hold QUICK_WORDS words per workgroup instead of one
    int top_k;
    float temperature, scale, inv_t; // scale: 1 / temperature when that is exact, else 0 (as sample_kernel takes it); inv_t: roughly 1 / temperature
    const float *u_dev;              // u = u_dev[state[1]]
    uint32_t *decided;               // 1: the token is recorded; 0: sample_kernel has to run
};
constexpr int QUICK_WORDS = QUICK_KEYS + 1; // per workgroup: the keys, then (sum bits << 32 | max bits); a bad row travels as a NaN sum
constexpr int QUICK_MAX_GRID = 1024;        // the merging workgroup's threads take four workgroups' words each, all requested at once
__device__ __forceinline__ void argmax_merge(float &best, int &idx, float ov, int oi) {
    if (ov > best || (ov == best && oi < idx)) {
        best = ov;
        idx = oi;
    }
}
template <int CH>
__global__ __launch_bounds__(256) void decode_lm_head_kernel(LmHeadArgs a) {
    extern __shared__ __attribute__((aligned(16))) half_t s_ln[]; // [d]
    __shared__ float s_red[16];
    __shared__ float s_best[4];
    __shared__ int s_idx[4];
    __shared__ int s_last;
    constexpr int RG = 4;
    const LnGemvArgs &p = a.g;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n_waves = gridDim.x * 4, gw = blockIdx.x * 4 + wave;
    LnInput ln_in; // all of the LayerNorm input is requested before any of it is waited for
    ln_request<true>(ln_in, p.x, p.gamma, p.beta, p.d); // d % 8 == 0, rows of the model's own buffers
    int a0, a1;
    split_rows(p.N1, n_waves, gw, a0, a1);
    RowGroups<CH, RG> rows;
    rows.init(p.W1, a0, a1, nullptr, 0, 0, p.d, p.b1);
    if (rows.total > 0) rows.load(0, lane);
    layernorm_regs(ln_in, s_ln, p.d, p.eps, s_red);
    lds_barrier();
    u32x4 xv[CH];
    load_x<CH>(xv, s_ln, p.d, lane);
    float best = -INFINITY;
    int best_i = 0x7fffffff;
    bool any = false;
    for (int first = 0; first < rows.total; first += RG) {
        rows.consume(first, xv, [&](int, int n, float dot, half_t b) {
            const half_t v = apply_epilogue_v<MOON_EPI_BIAS>(dot, b);
            if (lane == 0) p.y1[n] = v;
            float f = (float)v;
            if (n == 0 && f != f) f = INFINITY; // the reference starts from logits[0] and only moves on "greater": a NaN there stays
            if (f > best || (!any && f == best)) {
                best = f;
                best_i = n;
                any = true;
            }
        });
        if (first + RG < rows.total) rows.load(first + RG, lane);
    }
    if (lane == 0) {
        s_best[wave] = best;
        s_idx[wave] = best_i;
    }
    lds_barrier();
    if (tid == 0) {
        for (int w = 1; w < 4; w++) argmax_merge(best, best_i, s_best[w], s_idx[w]);
        const unsigned long long pair = ((unsigned long long)__float_as_uint(best) << 32) | (unsigned)best_i;
        __hip_atomic_store(a.partials + blockIdx.x, pair, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // the pair has reached memory before the workgroup counts in
        // two-level count (a single word would serialise a thousand atomics at the end of the launch): 32 leaves on
        // lines of their own, whoever completes a leaf counts it in at the root
        const unsigned leaves = gridDim.x < 32u ? gridDim.x : 32u, leaf = blockIdx.x % leaves;
        const unsigned members = gridDim.x / leaves + (leaf < gridDim.x % leaves ? 1u : 0u);
        const uint32_t old = __hip_atomic_fetch_add(a.counter + (1 + leaf) * 32, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        s_last = 0;
        if (old + 1 == a.generation * members) {
            const uint32_t done = __hip_atomic_fetch_add(a.counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            s_last = done + 1 == a.generation * leaves ? 1 : 0;
        }
    }
    lds_barrier();
    if (!s_last) return;
    best = -INFINITY;
    best_i = 0x7fffffff;
    for (int i = tid; i < (int)gridDim.x; i += 256) { // ascending within the thread, merged by (value, then lower index)
        const unsigned long long pair = __hip_atomic_load(a.partials + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        argmax_merge(best, best_i, __uint_as_float((unsigned)(pair >> 32)), (int)(unsigned)(pair & 0xffffffffu));
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) argmax_merge(best, best_i, __shfl_xor(best, off, 64), __shfl_xor(best_i, off, 64));
    lds_barrier();
    if (lane == 0) {
        s_best[wave] = best;
        s_idx[wave] = best_i;
    }
    lds_barrier();
    if (tid == 0) {
        for (int w = 1; w < 4; w++) argmax_merge(best, best_i, s_best[w], s_idx[w]);
        const uint32_t tok = best_i == 0x7fffffff ? 0u : (uint32_t)best_i;
        record_token(a.state, a.out_ids, tok, a.bump);
    }
}

// The same launch for the sampled loop with top_k < QUICK_KEYS (the reference CLI's default is top_k 3, moondream.zig:64-65):
// LayerNorm + LM head, logits to HBM, and per workgroup the QUICK_KEYS largest logits, the maximum and a rough sum of
// exps; the workgroup that counts in last merges those and decides the token where quick_top_k can prove that it is the
// reference's (sample_quick.hpp), recording it like the arg-max kernel does and setting *decided; otherwise *decided is 0
// and sample_kernel, launched behind this kernel either way, evaluates the row in full.
template <int CH>
__global__ __launch_bounds__(256) void decode_lm_head_topk_kernel(LmHeadArgs a) {
    extern __shared__ __attribute__((aligned(16))) half_t s_ln[]; // [d]
    __shared__ float s_red[16];
    __shared__ unsigned long long s_keys[4][QUICK_KEYS];
    __shared__ half_t s_logit[4][64];
    __shared__ float s_mx[4], s_sum[4];
    __shared__ unsigned s_bad[4];
    __shared__ int s_last;
    constexpr int RG = 4;
    const LnGemvArgs &p = a.g;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n_waves = gridDim.x * 4, gw = blockIdx.x * 4 + wave;
    LnInput ln_in;
    ln_request<true>(ln_in, p.x, p.gamma, p.beta, p.d);
    int a0, a1;
    split_rows(p.N1, n_waves, gw, a0, a1);
    RowGroups<CH, RG> rows;
    rows.init(p.W1, a0, a1, nullptr, 0, 0, p.d, p.b1);
    if (rows.total > 0) rows.load(0, lane);
    layernorm_regs(ln_in, s_ln, p.d, p.eps, s_red);
    lds_barrier();
    u32x4 xv[CH];
    load_x<CH>(xv, s_ln, p.d, lane);
    const float inv_t = a.inv_t;
    // Inside the row loop a logit only goes to LDS (the loop is the launch's weight stream: anything more between two row
    // groups delays the next requests); afterwards lane j takes the wavefront's j-th logit and the wavefront reduces.
    for (int first = 0; first < rows.total; first += RG) {
        rows.consume(first, xv, [&](int, int n, float dot, half_t b) {
            const half_t v = apply_epilogue_v<MOON_EPI_BIAS>(dot, b);
            if (lane == 0) {
                p.y1[n] = v;
                s_logit[wave][n - a0] = v;
            }
        });
        if (first + RG < rows.total) rows.load(first + RG, lane);
    }
    QuickTop q; // after the reduction every lane of the wavefront holds the same values
    quick_init(q);
    {
        const bool have = lane < rows.total; // rows.total <= 64 (checked by the launcher)
        const half_t v = have ? s_logit[wave][lane] : __builtin_bit_cast(half_t, (unsigned short)0xfc00);
        const unsigned hb = __builtin_bit_cast(unsigned short, v);
        q.bad = __ballot(have && (hb & 0x7c00u) == 0x7c00u && hb != 0xfc00u) ? 1u : 0u;
        unsigned long long key = have ? quick_key(v, a0 + lane) : 0ull;
#pragma unroll
        for (int r = 0; r < QUICK_KEYS; r++) { // the largest key left, QUICK_KEYS times
            unsigned long long best = key;
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1) {
                const unsigned lo = __shfl_xor((unsigned)best, off, 64), hi = __shfl_xor((unsigned)(best >> 32), off, 64);
                const unsigned long long o = ((unsigned long long)hi << 32) | lo;
                best = o > best ? o : best;
            }
            q.key[r] = best;
            if (key == best) key = 0;
        }
        if (q.key[0]) {
            const float mx = (float)quick_key_logit(q.key[0]), f = (float)v;
            float e = have && f > -INFINITY && mx > -INFINITY ? __expf((f - mx) * inv_t) : 0.f;
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1) e += __shfl_xor(e, off, 64);
            q.mx = mx;
            q.sum = e;
        }
    }
    auto publish = [&]() __attribute__((always_inline)) { // this wavefront's q -> LDS (inlined: q stays in registers)
        if (lane == 0) {
#pragma unroll
            for (int j = 0; j < QUICK_KEYS; j++) s_keys[wave][j] = q.key[j];
            s_mx[wave] = q.mx;
            s_sum[wave] = q.sum;
            s_bad[wave] = q.bad;
        }
    };
    auto gather = [&]() __attribute__((always_inline)) { // thread 0: the other three wavefronts' q merged into its own
        for (int w = 1; w < 4; w++) {
            QuickTop o;
#pragma unroll
            for (int j = 0; j < QUICK_KEYS; j++) o.key[j] = s_keys[w][j];
            o.mx = s_mx[w];
            o.sum = s_sum[w];
            o.bad = s_bad[w];
            quick_merge(q, o, inv_t);
        }
    };
    publish();
    lds_barrier();
    if (tid == 0) {
        gather();
        unsigned long long *mine = a.partials + size_t(blockIdx.x) * QUICK_WORDS;
#pragma unroll
        for (int j = 0; j < QUICK_KEYS; j++) __hip_atomic_store(mine + j, q.key[j], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const float sum_word = q.bad ? __uint_as_float(0x7fc00000u) : q.sum;
        __hip_atomic_store(mine + QUICK_KEYS, ((unsigned long long)__float_as_uint(sum_word) << 32) | __float_as_uint(q.mx), __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // the words have reached memory before the workgroup counts in
        const unsigned leaves = gridDim.x < 32u ? gridDim.x : 32u, leaf = blockIdx.x % leaves;
        const unsigned members = gridDim.x / leaves + (leaf < gridDim.x % leaves ? 1u : 0u);
        const uint32_t old = __hip_atomic_fetch_add(a.counter + (1 + leaf) * 32, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        s_last = 0;
        if (old + 1 == a.generation * members) {
            const uint32_t done = __hip_atomic_fetch_add(a.counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            s_last = done + 1 == a.generation * leaves ? 1 : 0;
        }
    }
    lds_barrier();
    if (!s_last) return;
    quick_init(q);
    {
        constexpr int PER = QUICK_MAX_GRID / 256;
        unsigned long long words[PER][QUICK_WORDS]; // every word is requested before the first is looked at
#pragma unroll
        for (int i = 0; i < PER; i++) {
            const int g = tid + i * 256;
            const unsigned long long *theirs = a.partials + size_t(g < (int)gridDim.x ? g : 0) * QUICK_WORDS;
#pragma unroll
            for (int j = 0; j < QUICK_WORDS; j++) words[i][j] = __hip_atomic_load(theirs + j, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
#pragma unroll
        for (int i = 0; i < PER; i++) {
            if (tid + i * 256 >= (int)gridDim.x) continue;
            QuickTop o;
#pragma unroll
            for (int j = 0; j < QUICK_KEYS; j++) o.key[j] = words[i][j];
            o.mx = __uint_as_float((unsigned)words[i][QUICK_KEYS]);
            o.sum = __uint_as_float((unsigned)(words[i][QUICK_KEYS] >> 32));
            o.bad = o.sum != o.sum ? 1u : 0u;
            if (o.bad) o.sum = 0.f;
            quick_merge(q, o, inv_t);
        }
    }
    // over the wavefront: a butterfly in which both partners merge the other's q into their own (the keys are distinct
    // except for the empty key 0, and merging is symmetric: both end with the same q)
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        QuickTop o;
#pragma unroll
        for (int j = 0; j < QUICK_KEYS; j++) {
            const unsigned lo = __shfl_xor((unsigned)q.key[j], off, 64), hi = __shfl_xor((unsigned)(q.key[j] >> 32), off, 64);
            o.key[j] = ((unsigned long long)hi << 32) | lo;
        }
        o.mx = __shfl_xor(q.mx, off, 64);
        o.sum = __shfl_xor(q.sum, off, 64);
        o.bad = __shfl_xor(q.bad, off, 64);
        quick_merge(q, o, inv_t);
    }
    lds_barrier();
    publish();
    lds_barrier();
    if (tid == 0) {
        gather();
        uint32_t tok = 0;
        const float u = a.u_dev[a.state[1]];
        const bool ok = quick_top_k(q, a.top_k, a.temperature, a.scale, u, &tok);
        if (ok) record_token(a.state, a.out_ids, tok, a.bump);
        *a.decided = ok ? 1u : 0u;
    }
}

// ---------------------------------------------------------------------------------------------------------------
// LayerNorm + qkv + fc1 AND the attention of the same layer in one launch.
// Every workgroup computes a share of the qkv rows first and reports them on a device-wide counter.  The first
// H * DEC_SPLITS workgroups then each take one (head, key split) attention task: they request their K and V rows,
// wait until the counter says that q, k and v are complete, and run the task; the other workgroups stream the fc1
// rows meanwhile, so the attention's dependent chain (q.k -> softmax -> p.v -> merge by the last split of a head) is
// hidden under the fc1 weight stream instead of costing a launch of its own.
// Only the attention workgroups ever wait, and they are the first H * DEC_SPLITS of the grid; every other workgroup runs
// to completion without waiting for anyone.  So the launch makes progress as long as the device can hold more than
// H * DEC_SPLITS workgroups of this kernel at once (checked by decode_front_supported: 4 per CU on 256 CUs against 256
// waiting ones), whether or not the whole grid is resident: the slots that finished workgroups free are taken by the
// ones still to start.  An ordinary launch is therefore enough (a cooperative launch costs tens of microseconds).
// The wait is bounded all the same: on a timeout the error word is raised, every waiting workgroup leaves, and the
// host reports the failure.
struct FrontArgs {
    LnGemvArgs g;            // y1 = qkv (written with device-coherent stores), y2 = fc1
    half_t *ck, *cv;         // this layer's cache [H][max_seq][64]
    const float *table;
    float *partial;          // [H][DEC_SPLITS][64 + 2]
    half_t *attn_out;        // [H * 64]
    uint32_t *head_count;    // [H] splits finished, monotonic over launches
    uint32_t head_target;
    uint32_t *qkv_count;     // [H] lines: q, k and v rows of the head written, monotonic over launches
    uint32_t qkv_target;     // a head's value once this launch has written its 3 * 64 rows
    uint32_t *error;
    int H, rot_dim, max_seq, pos;
    const uint32_t *pos_dev;
};

constexpr long long FRONT_TIMEOUT_TICKS = 100000000LL; // 1 s of the 100 MHz wall clock
constexpr int FRONT_COUNTER_STRIDE = 32;               // uint32 slots per 128-byte line: one line per head

template <int CH, int PF>
__global__ __launch_bounds__(256) void decode_front_kernel(FrontArgs a) {
    extern __shared__ __attribute__((aligned(16))) half_t s_ln[]; // [d]
    __shared__ float s_red[16];
    __shared__ int s_ok;
    constexpr int RG = 4;
    const LnGemvArgs &p = a.g;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n_waves = gridDim.x * 4, gw = blockIdx.x * 4 + wave;
    const int attn_groups = a.H * DEC_SPLITS;
    const bool attn_wg = (int)blockIdx.x < attn_groups;
    const half_t *x = p.token ? p.x + size_t(p.token[0]) * p.d : p.x;
    LnInput ln_in; // all of the LayerNorm input is requested before any of it is waited for
    ln_request<true>(ln_in, x, p.gamma, p.beta, p.d); // d % 8 == 0, rows of the model's own buffers
    int a0, a1, b0 = 0, b1 = 0;
    split_rows(p.N1, n_waves, gw, a0, a1);
    if (!attn_wg) split_rows(p.N2, n_waves - attn_groups * 4, gw - attn_groups * 4, b0, b1); // fc1 rows go to the other workgroups
    RowGroups<CH, RG> rows;
    rows.init(p.W1, a0, a1, p.W2, b0, b1, p.d, p.b1, p.b2);
    if (rows.total > 0) rows.load(0, lane);
    layernorm_regs(ln_in, s_ln, p.d, p.eps, s_red);
    lds_barrier();
    u32x4 xv[CH];
    load_x<CH>(xv, s_ln, p.d, lane);
    // all qkv rows of a wavefront sit in its first group (N1 <= RG * wavefronts, checked by the launcher)
    for (int first = 0; first < rows.total || first == 0; first += RG) {
        if (first < rows.total)
            rows.consume(first, xv, [&](int m, int n, float dot, half_t b) {
                if (lane == 0) {
                    if (m == 0) st_h<true>(p.y1 + n, apply_epilogue_v<MOON_EPI_BIAS>(dot, b));
                    else p.y2[n] = apply_epilogue_v<MOON_EPI_BIAS_GELU>(dot, b);
                }
            });
        if (first == 0) {
            // This workgroup's qkv rows are written: once the stores are acknowledged, count them in -- one atomic per
            // head segment the rows fall into (consecutive rows: at most two), on a counter line of that head's own,
            // so that the thousand reports of a launch spread over H addresses instead of queueing on one.
            // No load is in flight here (the next group is requested below): the wait covers the stores only.
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            lds_barrier();
            if (tid == 0) {
                int r0, r1, dummy;
                split_rows(p.N1, n_waves, blockIdx.x * 4, r0, dummy);
                split_rows(p.N1, n_waves, blockIdx.x * 4 + 3, dummy, r1);
                while (r0 < r1) {
                    const int seg_end = min(r1, (r0 / 64 + 1) * 64);
                    const int head = (r0 / 64) % a.H;
                    __hip_atomic_fetch_add(a.qkv_count + head * FRONT_COUNTER_STRIDE, (uint32_t)(seg_end - r0), __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_AGENT);
                    r0 = seg_end;
                }
            }
        }
        if (first + RG < rows.total) rows.load(first + RG, lane);
    }
    if (!attn_wg) return;

    const int pos = a.pos_dev ? (int)*a.pos_dev : a.pos;
    const int h = blockIdx.x / DEC_SPLITS, split = blockIdx.x % DEC_SPLITS;
    DecodeAttnPrefetch<PF> pf;
    decode_attn_prefetch<64, PF>(pf, a.ck, a.cv, a.max_seq, pos, true, h, split); // independent of the new token: in flight during the wait
    if (tid == 0) {
        // the counter alone is polled; the clock and the error word are looked at once in 64 polls
        const long long t0 = wall_clock64();
        int ok = 1;
        for (unsigned polls = 1;; polls++) {
            if (__hip_atomic_load(a.qkv_count + h * FRONT_COUNTER_STRIDE, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >= a.qkv_target) break;
            if ((polls & 63u) == 0) {
                if (__hip_atomic_load(a.error, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) {
                    ok = 0;
                    break;
                }
                if (wall_clock64() - t0 > FRONT_TIMEOUT_TICKS) {
                    __hip_atomic_store(a.error, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    ok = 0;
                    break;
                }
            }
        }
        s_ok = ok;
    }
    lds_barrier();
    if (!s_ok) return;
    // q, k and v of this head are complete
    decode_attn_task<64, true, true, PF>(p.y1, a.ck, a.cv, a.table, a.partial, a.H, a.rot_dim, a.max_seq, pos, h, split, pf, a.head_count,
                                     a.head_target, a.attn_out);
}

// ---------------------------------------------------------------------------------------------------------------
// A whole decoder layer in ONE launch (text_model.zig:150-172): LayerNorm, qkv, attention, fc1 + GELU, out_proj, fc2 and
// both residual adds.  Workgroups take roles by index; only consumers ever wait, on counters that producers bump:
//   every workgroup    LayerNorm (redundantly), then its share of the qkv rows -> per-head "rows written" counters
//   [0, A)             A = H * DEC_SPLITS attention tasks: wait for the head's q, k, v rows, attend over the cache; the
//                      split that finishes a head last merges it and counts the head as done
//   [A, A + O)         O = d / 4 output workgroups (one hidden element per wavefront): a few fc1 rows, then the
//                      wavefront requests its out_proj row and its fc2 row (20 KiB, in flight during the waits), waits
//                      for "all fc1 rows written" and "all heads done", and writes hidden += out_proj(attn) + fc2(fc1)
//   [A + O, grid)      the remaining fc1 rows (several times as many per wavefront as the output workgroups take)
// The weight stream of a later phase is always requested before the wait for the earlier phase's vector, so HBM stays
// busy across the three dependent exchanges that otherwise cost a kernel launch each.  Arithmetic, rounding points and
// summation orders are those of the separate kernels: the results are bit-identical.
// Progress: waiting workgroups occupy at most A + O of the device's slots and every producer runs to completion
// without waiting, so the launch finishes whenever the device holds more than A + O workgroups of this kernel at once
// (checked on the host).  Every wait is bounded all the same: timeout -> error word -> every waiter leaves.
struct LayerArgs {
    LnGemvArgs g;            // y1 = qkv and y2 = fc1, both written with device-coherent stores
    const half_t *Wo, *bo;   // [d, d]
    const half_t *W2, *b2;   // [d, ffn]
    half_t *hidden;          // [d] written at the end
    const half_t *hidden_src; // old hidden for the residual (hidden itself, or an embedding table with g.token)
    half_t *ck, *cv;
    const float *table;
    float *partial;
    half_t *attn_out;        // [d], device-coherent
    uint32_t *head_count;    // [H] splits finished (monotonic)
    uint32_t head_target;
    uint32_t *sync;          // counter lines of LAYER_SYNC_* below (monotonic), 32 uint32 per line
    uint32_t generation;     // launches of this layer so far, this one included
    uint32_t *error;
    int H, rot_dim, max_seq, pos, ffn;
    const uint32_t *pos_dev;
    long long *trace;        // optional [grid][8] wall-clock stamps of thread 0 (tuning aid), or null
    int qkv_wgs;             // workgroups that take qkv rows (the first ones)
    int fc1_rows_out;        // fc1 rows the output workgroups take; the fc1-only workgroups take the rest
};
// 1 KiB pieces of an output wavefront's fc2 row requested at a time, each lot waited for before the next is asked for (the shorter the queue in
// front of a dependent access of this compute unit, the sooner it is served; 2 and 1 measured 3 and 12 % slower, 8 and 16 slower too)
constexpr int LAYER_OUT_CHUNK = 4;
constexpr int LAYER_PIECE_SLEEP = 6; // units of 64 cycles between two piece requests (see RowGroups::load_pieces)
constexpr int LAYER_LINE = 32;                       // uint32 per 128-byte line
constexpr int LAYER_SYNC_FC1_LEAF = 0;               // lines 0..31: fc1 workgroups reported, 32 leaves
constexpr int LAYER_FC1_LEAVES = 32;
constexpr int LAYER_SYNC_QKV = LAYER_FC1_LEAVES;     // then one line per head: q, k, v rows written; then one per head: q rows written
// The two counters that all the output workgroups wait for ("fc1 leaves complete", "heads merged") exist in LAYER_COPIES copies
// each: whoever completes a leaf or merges a head adds to every copy (one atomic instruction, a lane per copy), and an output
// workgroup polls the copy of its index.  512 workgroups polling one line keep the memory channel that holds it busy (a poll
// is a read at the memory side), and everything else that lives in that channel, a 128th of the weight stream included,
// waits behind them: with the polls of these two counters replaced by fixed delays (timing only) the launch was 4.7 %
// shorter.  The copies are LAYER_COPY_STRIDE words apart (4 KiB + 256 B), which lands them in different channels whether the
// channels interleave by 256 bytes or by pages.
constexpr int LAYER_COPIES = 64;
constexpr int LAYER_COPY_STRIDE = 1088;
constexpr int LAYER_BCAST_FC1 = 0, LAYER_BCAST_HEADS = 1; // sets of copies, behind the lines above
__host__ __device__ inline int layer_bcast_offset(size_t H) { return (int)(LAYER_SYNC_QKV + 2 * H) * LAYER_LINE; }
inline int layer_sync_words(size_t H) { return layer_bcast_offset(H) + 2 * LAYER_COPIES * LAYER_COPY_STRIDE; }

// thread 0 of the workgroup polls *word until it reaches target; the clock and the error word are looked at once in
// 64 polls.  Returns (to every thread) whether the wait succeeded.
__device__ __forceinline__ bool wait_reached(uint32_t *word, uint32_t target, uint32_t *error, int *s_flag) {
    lds_barrier();
    if (threadIdx.x == 0) {
        const long long t0 = wall_clock64();
        int ok = 1;
        for (unsigned polls = 1;; polls++) {
            if (__hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >= target) break;
            if ((polls & 63u) == 0) {
                if (__hip_atomic_load(error, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) {
                    ok = 0;
                    break;
                }
                if (wall_clock64() - t0 > FRONT_TIMEOUT_TICKS) {
                    __hip_atomic_store(error, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    ok = 0;
                    break;
                }
            }
        }
        *s_flag = ok;
    }
    lds_barrier();
    return *s_flag != 0;
}


// FC1_GROUP: fc1 rows a wavefront requests together.  The fewer bytes a compute unit has queued, the sooner the small
// dependent accesses of the attention chain issued from it are served (two measured 3 % slower than one).
// PF: 32-key steps of an attention task whose K and V rows are requested before the wait for q (decode_attn_prefetch); the
// host picks the instantiation that covers a split at the launch's position.
template <int CH_D, int CH_F, int FC1_GROUP, int PF>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4, 4))) void decode_layer_kernel(LayerArgs a) {
    extern __shared__ __attribute__((aligned(16))) half_t smem[]; // [d] LayerNorm output; then [ffn] fc1
    __shared__ float s_red[16];
    __shared__ int s_flag;
    const LnGemvArgs &p = a.g;
    half_t *s_ln = smem, *s_fc1 = smem + p.d;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int gw = blockIdx.x * 4 + wave;
    const int n_attn = a.H * DEC_SPLITS, n_out = (p.d + 3) / 4;
    const int b = blockIdx.x;
    const bool attn_wg = b < n_attn, out_wg = !attn_wg && b < n_attn + n_out;
    const int n_fc1_wgs = gridDim.x - n_attn;
    uint32_t *bcast = a.sync + layer_bcast_offset(a.H);
    auto stamp = [&](int i) {
        if (a.trace && tid == 0) a.trace[size_t(b) * 8 + i] = wall_clock64();
    };
    stamp(0);

    const half_t *x = p.token ? p.x + size_t(p.token[0]) * p.d : p.x;
    LnInput ln_in; // all of the LayerNorm input is requested before any of it is waited for
    ln_request<true>(ln_in, x, p.gamma, p.beta, p.d); // d % 8 == 0, rows of the model's own buffers
    // qkv rows: all wavefronts (at most two each, one group).  They come first and alone: the attention chain hangs on
    // them, and a wavefront can only have its stores acknowledged once every load it issued earlier has returned.
    // Only the first qkv_wgs workgroups take qkv rows: those are served first by their compute unit, so the rows are all in
    // (and the chain under way) sooner than if the last workgroup of every unit had a share as well.
    const int qkv_waves = a.qkv_wgs * 4;
    int a0 = 0, a1 = 0;
    if (b < a.qkv_wgs) split_rows(p.N1, qkv_waves, gw, a0, a1);
    RowGroups<CH_D, 2> qrows;
    qrows.init(p.W1, a0, a1, nullptr, 0, 0, p.d, p.b1);
    if (qrows.total > 0) qrows.load(0, lane);
    layernorm_regs(ln_in, s_ln, p.d, p.eps, s_red);
    lds_barrier();
    u32x4 xv[CH_D];
    load_x<CH_D>(xv, s_ln, p.d, lane);
    for (int first = 0; first < qrows.total; first += 2) {
        qrows.consume(first, xv, [&](int, int n, float dot, half_t bias) {
            if (lane == 0) st_h<true>(p.y1 + n, apply_epilogue_v<MOON_EPI_BIAS>(dot, bias));
        });
        if (first + 2 < qrows.total) qrows.load(first + 2, lane);
    }
    // The workgroup's qkv rows are written: once the stores are acknowledged count them in, one atomic per head segment
    // they fall into (consecutive rows: at most two), each head on a line of its own.  No load is in flight here.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    lds_barrier();
    if (tid == 0 && b < a.qkv_wgs) {
        int r0, r1, dummy;
        split_rows(p.N1, qkv_waves, b * 4, r0, dummy);
        split_rows(p.N1, qkv_waves, b * 4 + 3, dummy, r1);
        while (r0 < r1) {
            const int seg_end = min(r1, (r0 / 64 + 1) * 64);
            const int head = (r0 / 64) % a.H;
            __hip_atomic_fetch_add(a.sync + (LAYER_SYNC_QKV + head) * LAYER_LINE, (uint32_t)(seg_end - r0), __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
            if (r0 < a.H * 64) // a q row: the splits that do not hold the new token's position wait for these alone
                __hip_atomic_fetch_add(a.sync + (LAYER_SYNC_QKV + a.H + head) * LAYER_LINE, (uint32_t)(seg_end - r0), __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
            r0 = seg_end;
        }
    }
    stamp(1); // qkv rows reported

    if (attn_wg) {
        const int pos = a.pos_dev ? (int)*a.pos_dev : a.pos;
        const int h = b / DEC_SPLITS, split = b % DEC_SPLITS;
        // K and V rows do not depend on the new token: wavefronts 1-3 request theirs before the wait.  Wavefront 0 polls,
        // and a poll returns in order behind whatever the wavefront has in flight, so it requests its rows afterwards.
        // The attention chain is what the launch waits for longest: its wavefronts' instructions go first where they share a SIMD
        // with streaming wavefronts (0.589 against 0.591-0.592 ms per token).
        __builtin_amdgcn_s_setprio(3);
        DecodeAttnPrefetch<PF> pf;
        if (wave != 0) decode_attn_prefetch<64, PF>(pf, a.ck, a.cv, a.max_seq, pos, true, h, split);
        // The cached keys need q only; k and v of the new token are one more key, which the last split holds alone
        // (decode_attn_range).  So that split waits for all of the head's rows, the others for its q rows.
        if (split == DEC_SPLITS - 1) {
            if (!wait_reached(a.sync + (LAYER_SYNC_QKV + h) * LAYER_LINE, a.generation * 192u, a.error, &s_flag)) return;
        } else {
            if (!wait_reached(a.sync + (LAYER_SYNC_QKV + a.H + h) * LAYER_LINE, a.generation * 64u, a.error, &s_flag)) return;
        }
        if (wave == 0) decode_attn_prefetch<64, PF>(pf, a.ck, a.cv, a.max_seq, pos, true, h, split);
        stamp(2); // what this split needs of the head's q, k, v is complete
        decode_attn_task<64, true, true, PF>(p.y1, a.ck, a.cv, a.table, a.partial, a.H, a.rot_dim, a.max_seq, pos, h, split, pf, a.head_count,
                                         a.head_target, a.attn_out, bcast + LAYER_BCAST_HEADS * LAYER_COPIES * LAYER_COPY_STRIDE, LAYER_COPIES, LAYER_COPY_STRIDE);
        stamp(3); // task (and possibly the head's merge) done
        return;
    }

    // fc1 rows: the output wavefronts take fc1_rows_out of them between themselves, the fc1-only wavefronts the rest
    {
        int b0, b1;
        const int w_out = n_out * 4, w_fc1 = (gridDim.x - n_attn - n_out) * 4;
        const int rows_out = a.fc1_rows_out;
        if (out_wg) split_rows(rows_out, w_out, gw - n_attn * 4, b0, b1);
        else {
            split_rows(p.N2 - rows_out, w_fc1, gw - (n_attn + n_out) * 4, b0, b1);
            b0 += rows_out;
            b1 += rows_out;
        }
        RowGroups<CH_D, FC1_GROUP> frows;
        frows.init(p.W2, b0, b1, nullptr, 0, 0, p.d, p.b2);
        constexpr int fstep = FC1_GROUP;
        if (frows.total > 0) frows.load(0, lane);
        for (int first = 0; first < frows.total; first += fstep) {
            frows.consume(first, xv, [&](int, int n, float dot, half_t bias) {
                if (lane == 0) st_h<true>(p.y2 + n, apply_epilogue_v<MOON_EPI_BIAS_GELU>(dot, bias));
            });
            if (first + fstep < frows.total) frows.load(first + fstep, lane);
        }
    }
    // this workgroup's fc1 rows are written: report on the two-level counter (32 leaves, then the root)
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    lds_barrier();
    if (wave == 0) {
        int leaf_done = 0;
        if (lane == 0) {
            const unsigned idx = (unsigned)(b - n_attn);
            const unsigned leaves = n_fc1_wgs < LAYER_FC1_LEAVES ? n_fc1_wgs : LAYER_FC1_LEAVES;
            const unsigned leaf = idx % leaves;
            const unsigned members = n_fc1_wgs / leaves + (leaf < (unsigned)n_fc1_wgs % leaves ? 1u : 0u);
            const unsigned old = __hip_atomic_fetch_add(a.sync + (LAYER_SYNC_FC1_LEAF + leaf) * LAYER_LINE, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            leaf_done = old + 1 == a.generation * members;
        }
        if (__builtin_amdgcn_readfirstlane(leaf_done)) // the leaf is complete: count it on every copy of the root, a lane per copy
            __hip_atomic_fetch_add(bcast + (LAYER_BCAST_FC1 * LAYER_COPIES + lane) * LAYER_COPY_STRIDE, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    stamp(2); // fc1 rows reported
    if (!out_wg) return;

    // output row of this wavefront; its two weight rows are requested now and arrive during the waits
    const int n = (b - n_attn) * 4 + __builtin_amdgcn_readfirstlane(wave); // (the same in every lane: row addresses stay scalar)
    const bool have_row = n < p.d;
    RowGroups<CH_D, 1> out_row;
    RowGroups<CH_F, 1> fc2_row;
    out_row.init(a.Wo, have_row ? n : 0, have_row ? n + 1 : 0, nullptr, 0, 0, p.d, a.bo);
    fc2_row.init(a.W2, have_row ? n : 0, have_row ? n + 1 : 0, nullptr, 0, 0, a.ffn, a.b2);
    const half_t *hsrc = p.token ? a.hidden_src + size_t(p.token[0]) * p.d : a.hidden_src;
    int hid_bits = 0, bias_o_bits = 0, bias_f_bits = 0;
    if (have_row) {
        const half_t hid = hsrc[n];
        out_row.load(0, lane);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // the out_proj row is in before the fc2 row is asked for
        fc2_row.template load_pieces<CH_F, 0>(0, lane, 0, 0); // (no piece yet: the row's bias alone)
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        // lane 0's old hidden value and the two rows' biases are all here now: as scalars they need no vector register
        // until the end of the launch
        hid_bits = __builtin_amdgcn_readfirstlane((int)__builtin_bit_cast(unsigned short, hid));
        bias_o_bits = __builtin_amdgcn_readfirstlane((int)__builtin_bit_cast(unsigned short, out_row.bias_lane));
        bias_f_bits = __builtin_amdgcn_readfirstlane((int)__builtin_bit_cast(unsigned short, fc2_row.bias_lane));
        fc2_row.template load_pieces<LAYER_OUT_CHUNK, LAYER_PIECE_SLEEP>(0, lane, 0, CH_F);
    }
    const unsigned fc1_leaves = n_fc1_wgs < LAYER_FC1_LEAVES ? n_fc1_wgs : LAYER_FC1_LEAVES;
    if (!wait_reached(bcast + (LAYER_BCAST_FC1 * LAYER_COPIES + b % LAYER_COPIES) * LAYER_COPY_STRIDE, a.generation * fc1_leaves, a.error, &s_flag)) return;
    stamp(3); // all fc1 rows written
    // The fc1 vector: four 16-byte loads per thread, one round trip.  They are workgroup-scope loads (sc0), which the die's L2
    // serves: every byte of the vector was written through to memory (sc1 stores) before the counter this workgroup has just
    // waited for was raised, and no workgroup reads a line of it before that, so the first of a die's 64 output workgroups to
    // ask takes the line from memory as it is and the others share it.  Device-scope loads, which pass the L2, cost 8 MB of
    // fabric traffic per launch at the moment the weight stream ends (0.585 against 0.578 ms per token, in 8-byte pieces, each
    // waited for).  (While all 512 output workgroups polled one counter line, anything that brought them to the next wait
    // sooner made the launch longer, this copy in one round trip included: 0.610 ms.)
    {
        static_assert(CH_F % 4 == 0, "ffn = 512 CH_F halfs in 16-byte pieces over 256 threads");
        u32x4 v[CH_F / 4];
#pragma unroll
        for (int k = 0; k < CH_F / 4; k++)
            asm volatile("global_load_dwordx4 %0, %1, off sc0" : "=v"(v[k]) : "v"(p.y2 + size_t(tid + 256 * k) * 8) : "memory");
#pragma unroll
        for (int k = 0; k < CH_F / 4; k++) asm volatile("s_waitcnt vmcnt(0)" : "+v"(v[k])::"memory");
#pragma unroll
        for (int k = 0; k < CH_F / 4; k++) reinterpret_cast<u32x4 *>(s_fc1)[tid + 256 * k] = v[k];
    }
    lds_barrier();
    // the fc2 row's product is taken before the wait for the heads (the fc1 vector is complete microseconds before the last head):
    // what follows that wait is the launch's last hop
    float dot_f = 0.0f; // pieces in the same order as RowGroups::consume
    if (have_row) {
#pragma unroll
        for (int c = 0; c < CH_F; c++) {
            const int g = c * 64 + lane;
            // (ffn is a multiple of 512 here, decode_layer_supported: every lane has its piece.  A guarded read would put each
            // piece behind a branch of its own, and the compiler then keeps all sixteen in registers that are not there.)
            const u32x4 xg = *reinterpret_cast<const u32x4 *>(s_fc1 + size_t(g) * 8);
            dot_f = dot8(fc2_row.w[0][c], xg, dot_f);
        }
        dot_f = wave_sum(dot_f);
    }
    if (!wait_reached(bcast + (LAYER_BCAST_HEADS * LAYER_COPIES + b % LAYER_COPIES) * LAYER_COPY_STRIDE, a.generation * (uint32_t)a.H, a.error, &s_flag)) return;
    stamp(4); // all heads merged
    if (!have_row) return;
    const half_t bias_o = __builtin_bit_cast(half_t, (unsigned short)bias_o_bits), bias_f = __builtin_bit_cast(half_t, (unsigned short)bias_f_bits);
    const half_t hid = __builtin_bit_cast(half_t, (unsigned short)hid_bits);
    // The attention output goes straight into each wavefront's registers, a lane fetching the pieces that meet its pieces of the
    // out_proj row (d is a multiple of 512: every lane has them): four times the requests of one copy into LDS per workgroup, but
    // no LDS round trip and no barrier behind the last wait (0.5831 against 0.5869 ms per token).  Same pieces in the same order
    // as RowGroups::consume.  Workgroup-scope loads through the die's L2, like the fc1 vector's: the heads were written through
    // before the counter rose.
    float dot_o = 0.0f;
    {
        u32x4 xa[CH_D];
#pragma unroll
        for (int c = 0; c < CH_D; c++)
            asm volatile("global_load_dwordx4 %0, %1, off sc0" : "=v"(xa[c]) : "v"(a.attn_out + size_t(c * 64 + lane) * 8) : "memory");
#pragma unroll
        for (int c = 0; c < CH_D; c++) asm volatile("s_waitcnt vmcnt(0)" : "+v"(xa[c])::"memory");
#pragma unroll
        for (int c = 0; c < CH_D; c++) dot_o = dot8(out_row.w[0][c], xa[c], dot_o);
        dot_o = wave_sum(dot_o);
    }
    if (lane == 0) {
        const half_t ao = apply_epilogue_v<MOON_EPI_BIAS>(dot_o, bias_o);
        const half_t m = apply_epilogue_v<MOON_EPI_BIAS>(dot_f, bias_f);
        const half_t am = (half_t)((float)ao + (float)m); // attn_out += mlp_out
        a.hidden[n] = (half_t)((float)hid + (float)am);   // hidden += attn_out
    }
    stamp(5);
}

struct OutFc2Args {
    const half_t *attn;  // [d]
    const half_t *fc1;   // [ffn]
    const half_t *Wo, *bo;   // [d, d]
    const half_t *W2, *b2;   // [d, ffn]
    half_t *hidden;          // [d], updated in place
    const half_t *hidden_src; // where the old hidden value is read (hidden itself, or an embedding table)
    const uint32_t *token;    // if not null: hidden_src += token[0] * d
    int d, ffn;
};

template <int CH_D, int CH_F>
__global__ __launch_bounds__(256) void decode_out_fc2_kernel(OutFc2Args p) {
    extern __shared__ __attribute__((aligned(16))) half_t smem[];
    half_t *s_attn = smem, *s_fc1 = smem + p.d;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n_waves = gridDim.x * 4, gw = blockIdx.x * 4 + wave;
    int r0, r1;
    split_rows(p.d, n_waves, gw, r0, r1);
    // the two activation vectors (cached) are requested first, then the weight rows of this wavefront's first output
    constexpr int STAGE = 6; // 16-byte pieces per thread: (d + ffn) * 2 / 16 / 256 <= 6 for d + ffn <= 12288
    u32x4 staged[STAGE];
    const int nd = p.d / 8, nf = p.ffn / 8;
#pragma unroll
    for (int k = 0; k < STAGE; k++) {
        const int i = tid + 256 * k;
        staged[k] = u32x4{0, 0, 0, 0};
        if (i < nd) staged[k] = reinterpret_cast<const u32x4 *>(p.attn)[i];
        else if (i < nd + nf) staged[k] = reinterpret_cast<const u32x4 *>(p.fc1)[i - nd];
    }
    RowGroups<CH_D, 1> out_row;
    RowGroups<CH_F, 1> fc2_row;
    out_row.init(p.Wo, r0, r1, nullptr, 0, 0, p.d, p.bo);
    fc2_row.init(p.W2, r0, r1, nullptr, 0, 0, p.ffn, p.b2);
    const half_t *hsrc = p.token ? p.hidden_src + size_t(p.token[0]) * p.d : p.hidden_src;
    half_t hid_lane = (half_t)0.0f; // old hidden value of row r0 + lane
    if (lane < r1 - r0) hid_lane = hsrc[r0 + lane];
    if (r1 > r0) {
        out_row.load(0, lane);
        fc2_row.load(0, lane);
    }
#pragma unroll
    for (int k = 0; k < STAGE; k++) {
        const int i = tid + 256 * k;
        if (i < nd + nf) reinterpret_cast<u32x4 *>(smem)[i] = staged[k]; // s_fc1 follows s_attn
    }
    for (int i = tid + 256 * STAGE; i < nd + nf; i += 256)
        reinterpret_cast<u32x4 *>(smem)[i] = i < nd ? reinterpret_cast<const u32x4 *>(p.attn)[i] : reinterpret_cast<const u32x4 *>(p.fc1)[i - nd];
    lds_barrier();
    u32x4 xa[CH_D], xf[CH_F];
    load_x<CH_D>(xa, s_attn, p.d, lane);
    load_x<CH_F>(xf, s_fc1, p.ffn, lane);
    for (int i = 0; i < r1 - r0; i++) {
        half_t a = (half_t)0.0f;
        out_row.consume(i, xa, [&](int, int, float dot, half_t b) { a = apply_epilogue_v<MOON_EPI_BIAS>(dot, b); });
        const half_t hid = __builtin_bit_cast(half_t, (unsigned short)__builtin_amdgcn_readlane((int)__builtin_bit_cast(unsigned short, hid_lane), i & 63));
        fc2_row.consume(i, xf, [&](int, int n, float dot, half_t b) {
            if (lane == 0) {
                const half_t m = apply_epilogue_v<MOON_EPI_BIAS>(dot, b);
                const half_t am = (half_t)((float)a + (float)m);  // attn_out += mlp_out
                p.hidden[n] = (half_t)((float)hid + (float)am);   // hidden += attn_out
            }
        });
        if (i + 1 < r1 - r0) {
            out_row.load(i + 1, lane);
            fc2_row.load(i + 1, lane);
        }
    }
}

template <int D, int PF>
__global__ __launch_bounds__(256) void decode_attn_merged_kernel(const half_t *__restrict__ qkv, half_t *__restrict__ ck,
                                                                  half_t *__restrict__ cv, const float *__restrict__ table,
                                                                  float *__restrict__ partial, half_t *__restrict__ out,
                                                                  uint32_t *head_count, uint32_t count_target, int H, int rot_dim,
                                                                  int max_seq, int pos_arg, const uint32_t *__restrict__ pos_dev, int head_stride) {
    const int pos = pos_dev ? (int)*pos_dev : pos_arg;
    const int h = blockIdx.x / DEC_SPLITS, split = blockIdx.x % DEC_SPLITS;
    DecodeAttnPrefetch<PF> pf;
    decode_attn_prefetch<D, PF>(pf, ck, cv, max_seq, pos, true, h, split);
    // device-coherent partials and a per-head counter: whichever split finishes a head last merges it
    decode_attn_task<D, true, true, PF>(qkv, ck, cv, table, partial, H, rot_dim, max_seq, pos, h, split, pf, head_count, count_target, out, nullptr, 1, 0,
                                        head_stride);
}

// sampling.argmax (sampling.zig:257-273) + bookkeeping of the greedy loop: state[2] = token, out_ids[state[1]++] = token.
__global__ __launch_bounds__(1024) void argmax_record_kernel(const half_t *__restrict__ logits, int n, uint32_t *state, uint32_t *out_ids) {
    __shared__ float sv[16];
    __shared__ int si[16];
    float best = -INFINITY;
    int idx = 0x7fffffff;
    bool any = false;
    const int n8 = n / 8;
    for (int g = threadIdx.x; g < n8; g += blockDim.x) { // 8 logits per 16-byte load, ascending within the thread
        const u32x4 v = reinterpret_cast<const u32x4 *>(logits)[g];
        const half_t *h = reinterpret_cast<const half_t *>(&v);
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const float f = (float)h[e];
            if (f > best || (!any && f == best)) {
                best = f;
                idx = g * 8 + e;
                any = true;
            }
        }
    }
    for (int i = n8 * 8 + threadIdx.x; i < n; i += blockDim.x) {
        const float f = (float)logits[i];
        if (f > best || (f == best && i < idx) || (!any && f == best)) {
            best = f;
            idx = i;
            any = true;
        }
    }
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
        const float first = (float)logits[0];
        const uint32_t tok = (idx == 0x7fffffff || first != first) ? 0u : (uint32_t)idx; // a NaN at index 0 is never displaced
        record_token(state, out_ids, tok, 0u);
    }
}

inline int pieces(size_t K) { return (int)((K / 8 + 63) / 64); }
constexpr int LN_GEMV_GROUPS_PER_CU = 4, OUT_FC2_GROUPS_PER_CU = 2;

} // namespace

bool decode_fused_supported(size_t d, size_t ffn) {
    const int cd = pieces(d), cf = pieces(ffn);
    return d % 8 == 0 && ffn % 8 == 0 && d <= 256 * LN_REGS && ((cd == 4 && cf == 16) || (cd == 1 && (cf == 2 || cf == 4)) || (cd == 2 && cf == 8));
}


// Can a whole layer run as one launch of decode_layer_kernel on this device?
bool decode_layer_supported(moon_ctx *ctx, size_t d, size_t ffn, size_t H, size_t D) {
    if (D != 64 || pieces(d) != 4 || pieces(ffn) != 16 || H * D != d || d % 512 || ffn % 512) return false; // (whole 1 KiB pieces)
    const int cus = ctx->cu_count > 0 ? ctx->cu_count : 256;
    const int grid = LN_GEMV_GROUPS_PER_CU * cus;
    const int waiting = (int)(H * DEC_SPLITS + (d + 3) / 4); // attention and output workgroups
    if (waiting >= grid || 3 * d > size_t(16) * grid) return false;
    int per_cu = 0;
    const void *kernels[5] = {reinterpret_cast<const void *>(decode_layer_kernel<4, 16, 1, 4>), reinterpret_cast<const void *>(decode_layer_kernel<4, 16, 1, 5>),
                              reinterpret_cast<const void *>(decode_layer_kernel<4, 16, 1, 6>), reinterpret_cast<const void *>(decode_layer_kernel<4, 16, 1, 8>),
                              reinterpret_cast<const void *>(decode_layer_kernel<4, 16, 1, 10>)};
    for (const void *k : kernels) {
        if (hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)((d + ffn) * sizeof(half_t))) != hipSuccess) return false;
        int n = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, k, 256, (d + ffn) * sizeof(half_t)) != hipSuccess) return false;
        per_cu = per_cu == 0 ? n : std::min(per_cu, n);
    }
    return per_cu * cus > waiting; // producers always find a slot
}
size_t decode_layer_sync_words(size_t H) { return (size_t)layer_sync_words(H); }

int launch_decode_layer(moon_ctx *ctx, const half_t *x, const uint32_t *token, const half_t *gamma, const half_t *beta, float eps, size_t d,
                        const half_t *Wqkv, const half_t *bqkv, half_t *qkv, const half_t *W1, const half_t *b1, half_t *fc1, size_t ffn,
                        const half_t *Wo, const half_t *bo, const half_t *W2, const half_t *b2, half_t *hidden, const half_t *hidden_src,
                        half_t *cache_k, half_t *cache_v, const float *table, float *partial, half_t *attn_out, uint32_t *head_count,
                        uint32_t head_target, uint32_t *sync, uint32_t generation, uint32_t *error, size_t H, size_t rot_dim, size_t max_seq,
                        size_t pos, const uint32_t *pos_dev, long long *trace) {
    if (rot_dim > 64 || rot_dim % 2) return moon_fail(ctx, MOON_EROT_DIM, "decode attention: bad rot_dim %zu", rot_dim);
    if (max_seq > 2048 || pos >= max_seq)
        return moon_fail(ctx, MOON_ESEQ_TOO_LONG, "decode attention: pos %zu >= max_seq %zu (limit 2048)", pos, max_seq);
    LayerArgs a;
    a.trace = trace;
    {
        const long long n_attn = (long long)(H * DEC_SPLITS), n_out = (long long)((d + 3) / 4), grid_wgs = (long long)LN_GEMV_GROUPS_PER_CU * (ctx->cu_count > 0 ? ctx->cu_count : 256);
        const long long w_out = n_out * 4, w_fc1 = (grid_wgs - n_attn - n_out) * 4;
        static long long qkv_wgs = -1, r_o = -1;
        if (qkv_wgs < 0) {
            const char *e = getenv("MOON_LAYER_QKV_WGS");
            qkv_wgs = e ? atoll(e) : 0;
            const char *f = getenv("MOON_LAYER_FC1_OUT_ROWS");
            r_o = f ? atoll(f) + 1 : 0; // (kept as rows + 1 so that 0 rows can be asked for)
        }
        // by default the fc1-only workgroups, the last to be served on every compute unit, take no qkv rows
        const long long qkv_default = 3 * (long long)d <= 64 * (n_attn + n_out) ? n_attn + n_out : grid_wgs;
        // an fc1-only wavefront takes about three times the fc1 rows of an output wavefront, which has its 20 KiB of out_proj
        // and fc2 rows to request as well; whole rows per output wavefront, at least one (moondream: 1 and 6 rows; 2 and 4
        // measured 0.598 against 0.592 ms per token, none and 8 0.673)
        const long long per_out_wave = w_fc1 > 0 ? std::max<long long>(1, (long long)ffn / (w_out + 3 * w_fc1)) : (long long)ffn;
        const long long default_rows_out = std::min<long long>((long long)ffn, w_out * per_out_wave);
        a.qkv_wgs = (int)(qkv_wgs > 0 && qkv_wgs <= grid_wgs && 3 * (long long)d <= 64 * qkv_wgs ? qkv_wgs : qkv_default);
        a.fc1_rows_out = (int)(r_o > 0 && w_fc1 > 0 ? std::min<long long>((long long)ffn, w_out * (r_o - 1)) : default_rows_out);
    }
    a.g = LnGemvArgs{x, token, gamma, beta, Wqkv, bqkv, qkv, W1, b1, fc1, (int)d, (int)(3 * d), (int)ffn, eps};
    a.Wo = Wo;
    a.bo = bo;
    a.W2 = W2;
    a.b2 = b2;
    a.hidden = hidden;
    a.hidden_src = hidden_src;
    a.ck = cache_k;
    a.cv = cache_v;
    a.table = table;
    a.partial = partial;
    a.attn_out = attn_out;
    a.head_count = head_count;
    a.head_target = head_target;
    a.sync = sync;
    a.generation = generation;
    a.error = error;
    a.H = (int)H;
    a.rot_dim = (int)rot_dim;
    a.max_seq = (int)max_seq;
    a.pos = (int)pos;
    a.ffn = (int)ffn;
    a.pos_dev = pos_dev;
    const unsigned grid = (unsigned)(LN_GEMV_GROUPS_PER_CU * (ctx->cu_count > 0 ? ctx->cu_count : 256));
    // The instantiation whose attention tasks request all their K and V rows before the wait for q: the pos cached keys go to
    // DEC_SPLITS - 1 splits, 32 keys per prefetch step (a step too few costs a dependent round trip per 32 keys inside the
    // attention chain: 0.628 instead of 0.598 ms per token at 900-1030 cached keys; steps too many cost 1-2 % at short
    // contexts).  pos is the host's count; a loop that has stopped at an end-of-sequence token only over-provides.
    const size_t per_split = (pos + DEC_SPLITS - 2) / (DEC_SPLITS - 1), steps = (per_split + 31) / 32;
    const size_t lds = (d + ffn) * sizeof(half_t);
    if (steps <= 4) hipLaunchKernelGGL((decode_layer_kernel<4, 16, 1, 4>), dim3(grid), dim3(256), lds, ctx->stream, a);
    else if (steps <= 5) hipLaunchKernelGGL((decode_layer_kernel<4, 16, 1, 5>), dim3(grid), dim3(256), lds, ctx->stream, a);
    else if (steps <= 6) hipLaunchKernelGGL((decode_layer_kernel<4, 16, 1, 6>), dim3(grid), dim3(256), lds, ctx->stream, a);
    else if (steps <= 8) hipLaunchKernelGGL((decode_layer_kernel<4, 16, 1, 8>), dim3(grid), dim3(256), lds, ctx->stream, a);
    else hipLaunchKernelGGL((decode_layer_kernel<4, 16, 1, 10>), dim3(grid), dim3(256), lds, ctx->stream, a);
    MOON_HIP(ctx, hipGetLastError());
    return MOON_OK;
}

// Can the layer's front kernel (LayerNorm + qkv + fc1 + attention) run on this device?  It needs head_dim 64 and room
// for well more workgroups than there are attention tasks (the only ones that wait).
bool decode_front_supported(moon_ctx *ctx, size_t d, size_t H, size_t D) {
    if (D != 64 || pieces(d) != 4 || H * D != d) return false;
    const int cus = ctx->cu_count > 0 ? ctx->cu_count : 256;
    const int grid = LN_GEMV_GROUPS_PER_CU * cus;
    if ((int)(H * DEC_SPLITS) >= grid || 3 * d > size_t(16) * grid) return false; // every wavefront's qkv rows fit its first group
    int per_cu = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, reinterpret_cast<const void *>(decode_front_kernel<4, 10>), 256, d * sizeof(half_t)) !=
        hipSuccess)
        return false;
    return per_cu * cus >= 2 * (int)(H * DEC_SPLITS);
}

int launch_decode_front(moon_ctx *ctx, const half_t *x, const uint32_t *token, const half_t *gamma, const half_t *beta, float eps, size_t d,
                        const half_t *Wqkv, const half_t *bqkv, half_t *qkv, const half_t *W1, const half_t *b1, half_t *fc1, size_t ffn,
                        half_t *cache_k, half_t *cache_v, const float *table, float *partial, half_t *attn_out, uint32_t *head_count,
                        uint32_t head_target, uint32_t *qkv_count, uint32_t qkv_target, uint32_t *error, size_t H, size_t rot_dim,
                        size_t max_seq, size_t pos, const uint32_t *pos_dev) {
    if (rot_dim > 64 || rot_dim % 2) return moon_fail(ctx, MOON_EROT_DIM, "decode attention: bad rot_dim %zu", rot_dim);
    if (max_seq > 2048 || pos >= max_seq)
        return moon_fail(ctx, MOON_ESEQ_TOO_LONG, "decode attention: pos %zu >= max_seq %zu (limit 2048)", pos, max_seq);
    FrontArgs a;
    a.g = LnGemvArgs{x, token, gamma, beta, Wqkv, bqkv, qkv, W1, b1, fc1, (int)d, (int)(3 * d), (int)ffn, eps};
    a.ck = cache_k;
    a.cv = cache_v;
    a.table = table;
    a.partial = partial;
    a.attn_out = attn_out;
    a.head_count = head_count;
    a.head_target = head_target;
    a.qkv_count = qkv_count;
    a.qkv_target = qkv_target;
    a.error = error;
    a.H = (int)H;
    a.rot_dim = (int)rot_dim;
    a.max_seq = (int)max_seq;
    a.pos = (int)pos;
    a.pos_dev = pos_dev;
    const unsigned grid = (unsigned)(LN_GEMV_GROUPS_PER_CU * (ctx->cu_count > 0 ? ctx->cu_count : 256));
    if ((pos + DEC_SPLITS - 2) / (DEC_SPLITS - 1) <= 128) hipLaunchKernelGGL((decode_front_kernel<4, 4>), dim3(grid), dim3(256), d * sizeof(half_t), ctx->stream, a);
    else hipLaunchKernelGGL((decode_front_kernel<4, 10>), dim3(grid), dim3(256), d * sizeof(half_t), ctx->stream, a);
    MOON_HIP(ctx, hipGetLastError());
    return MOON_OK;
}

// ln = LN(x); y1 = ln.W1^T + b1; optionally y2 = gelu(ln.W2^T + b2).  token: optional device token id selecting row token*d of x.
int launch_decode_ln_gemv(moon_ctx *ctx, const half_t *x, const uint32_t *token, const half_t *gamma, const half_t *beta, float eps,
                          size_t d, const half_t *W1, const half_t *b1, half_t *y1, size_t N1, const half_t *W2, const half_t *b2,
                          half_t *y2, size_t N2) {
    LnGemvArgs p{x, token, gamma, beta, W1, b1, y1, W2, b2, y2, (int)d, (int)N1, (int)N2, eps};
    const unsigned grid = (unsigned)(LN_GEMV_GROUPS_PER_CU * (ctx->cu_count > 0 ? ctx->cu_count : 256));
    const size_t shmem = d * sizeof(half_t);
    switch (pieces(d)) {
    case 1:
        if (N2 > 0) hipLaunchKernelGGL((decode_ln_gemv_kernel<1, true>), dim3(grid), dim3(256), shmem, ctx->stream, p);
        else hipLaunchKernelGGL((decode_ln_gemv_kernel<1, false>), dim3(grid), dim3(256), shmem, ctx->stream, p);
        break;
    case 2:
        if (N2 > 0) hipLaunchKernelGGL((decode_ln_gemv_kernel<2, true>), dim3(grid), dim3(256), shmem, ctx->stream, p);
        else hipLaunchKernelGGL((decode_ln_gemv_kernel<2, false>), dim3(grid), dim3(256), shmem, ctx->stream, p);
        break;
    case 4:
        if (N2 > 0) hipLaunchKernelGGL((decode_ln_gemv_kernel<4, true>), dim3(grid), dim3(256), shmem, ctx->stream, p);
        else hipLaunchKernelGGL((decode_ln_gemv_kernel<4, false>), dim3(grid), dim3(256), shmem, ctx->stream, p);
        break;
    default: return moon_fail(ctx, MOON_EINVAL_DIM, "fused decode: unsupported dim %zu", d);
    }
    MOON_HIP(ctx, hipGetLastError());
    return MOON_OK;
}

// words of the LM head's arg-max exchange: a pair per workgroup (two words each), then the counter lines
size_t decode_lm_head_words(moon_ctx *ctx) { return size_t(2 * QUICK_WORDS) * LN_GEMV_GROUPS_PER_CU * (ctx->cu_count > 0 ? ctx->cu_count : 256) + 33 * 32; }
// (a wavefront of that launch keeps its logits one per lane)
bool decode_lm_head_top_k_supported(moon_ctx *ctx, size_t top_k, size_t V) {
    const size_t grid = size_t(LN_GEMV_GROUPS_PER_CU) * (ctx->cu_count > 0 ? ctx->cu_count : 256);
    return top_k >= 1 && top_k + 1 <= (size_t)QUICK_KEYS && V >= (size_t)QUICK_KEYS && V <= size_t(64) * 4 * grid && grid <= (size_t)QUICK_MAX_GRID;
}
int launch_decode_lm_head(moon_ctx *ctx, const half_t *x, const half_t *gamma, const half_t *beta, float eps, size_t d, const half_t *W,
                          const half_t *bias, half_t *logits, size_t V, uint32_t *exchange, uint32_t generation, uint32_t *state,
                          uint32_t *out_ids, uint32_t bump, const moon_sampling_config *top_k_cfg, const float *u_dev, uint32_t *decided) {
    const unsigned grid = (unsigned)(LN_GEMV_GROUPS_PER_CU * (ctx->cu_count > 0 ? ctx->cu_count : 256));
    if (!V || V > 0x7fffffff) return moon_fail(ctx, MOON_EINVAL, "argmax: empty or oversized tensor");
    if (top_k_cfg && (!decode_lm_head_top_k_supported(ctx, top_k_cfg->top_k, V) || !u_dev || !decided || !state))
        return moon_fail(ctx, MOON_EINVAL, "lm head: top_k %zu cannot be decided in the LM-head kernel", top_k_cfg->top_k);
    if ((unsigned long long)generation * grid > 0xffffffffull) return moon_fail(ctx, MOON_EINVAL, "lm head: launch counter out of range");
    LmHeadArgs a;
    a.g = LnGemvArgs{x, nullptr, gamma, beta, W, bias, logits, nullptr, nullptr, nullptr, (int)d, (int)V, 0, eps};
    a.partials = reinterpret_cast<unsigned long long *>(exchange);
    a.counter = exchange + size_t(2 * QUICK_WORDS) * grid;
    a.generation = generation;
    a.state = state;
    a.out_ids = out_ids;
    a.bump = bump;
    a.top_k = 0;
    a.temperature = a.inv_t = 1.f;
    a.scale = 0.f;
    a.u_dev = nullptr;
    a.decided = nullptr;
    const size_t shmem = d * sizeof(half_t);
    if (top_k_cfg) {
        a.top_k = (int)top_k_cfg->top_k;
        a.temperature = top_k_cfg->temperature;
        a.inv_t = 1.0f / top_k_cfg->temperature;
        int exponent = 0; // as launch_sample: dividing by a power of two is a multiplication by its reciprocal, bit for bit
        a.scale = (std::frexp(top_k_cfg->temperature, &exponent) == 0.5f && exponent > -100 && exponent < 100) ? 1.0f / top_k_cfg->temperature : 0.f;
        a.u_dev = u_dev;
        a.decided = decided;
        switch (pieces(d)) {
        case 1: hipLaunchKernelGGL((decode_lm_head_topk_kernel<1>), dim3(grid), dim3(256), shmem, ctx->stream, a); break;
        case 2: hipLaunchKernelGGL((decode_lm_head_topk_kernel<2>), dim3(grid), dim3(256), shmem, ctx->stream, a); break;
        case 4: hipLaunchKernelGGL((decode_lm_head_topk_kernel<4>), dim3(grid), dim3(256), shmem, ctx->stream, a); break;
        default: return moon_fail(ctx, MOON_EINVAL_DIM, "fused decode: unsupported dim %zu", d);
        }
        MOON_HIP(ctx, hipGetLastError());
        return MOON_OK;
    }
    switch (pieces(d)) {
    case 1: hipLaunchKernelGGL((decode_lm_head_kernel<1>), dim3(grid), dim3(256), shmem, ctx->stream, a); break;
    case 2: hipLaunchKernelGGL((decode_lm_head_kernel<2>), dim3(grid), dim3(256), shmem, ctx->stream, a); break;
    case 4: hipLaunchKernelGGL((decode_lm_head_kernel<4>), dim3(grid), dim3(256), shmem, ctx->stream, a); break;
    default: return moon_fail(ctx, MOON_EINVAL_DIM, "fused decode: unsupported dim %zu", d);
    }
    MOON_HIP(ctx, hipGetLastError());
    return MOON_OK;
}

int launch_decode_out_fc2(moon_ctx *ctx, const half_t *attn, const half_t *fc1, const half_t *Wo, const half_t *bo, const half_t *W2,
                          const half_t *b2, half_t *hidden, const half_t *hidden_src, const uint32_t *token, size_t d, size_t ffn) {
    OutFc2Args p{attn, fc1, Wo, bo, W2, b2, hidden, hidden_src, token, (int)d, (int)ffn};
    const unsigned grid = (unsigned)(OUT_FC2_GROUPS_PER_CU * (ctx->cu_count > 0 ? ctx->cu_count : 256));
    if (d > size_t(16) * grid) return moon_fail(ctx, MOON_EINVAL_DIM, "fused decode: dim %zu too large", d);
    const size_t shmem = (d + ffn) * sizeof(half_t);
    const int cd = pieces(d), cf = pieces(ffn);
    if (cd == 4 && cf == 16) hipLaunchKernelGGL((decode_out_fc2_kernel<4, 16>), dim3(grid), dim3(256), shmem, ctx->stream, p);
    else if (cd == 1 && cf == 2) hipLaunchKernelGGL((decode_out_fc2_kernel<1, 2>), dim3(grid), dim3(256), shmem, ctx->stream, p);
    else if (cd == 1 && cf == 4) hipLaunchKernelGGL((decode_out_fc2_kernel<1, 4>), dim3(grid), dim3(256), shmem, ctx->stream, p);
    else if (cd == 2 && cf == 8) hipLaunchKernelGGL((decode_out_fc2_kernel<2, 8>), dim3(grid), dim3(256), shmem, ctx->stream, p);
    else return moon_fail(ctx, MOON_EINVAL_DIM, "fused decode: unsupported dim %zu / hidden_dim %zu", d, ffn);
    MOON_HIP(ctx, hipGetLastError());
    return MOON_OK;
}

// head_count: H persistent counters of this layer; count_target = DEC_SPLITS x (number of launches on them so far, this one included)
int launch_decode_attention_merged(moon_ctx *ctx, const half_t *qkv, half_t *cache_k, half_t *cache_v, const float *table, float *partial,
                                   half_t *out, uint32_t *head_count, uint32_t count_target, size_t H, size_t D, size_t rot_dim,
                                   size_t max_seq, size_t pos, const uint32_t *pos_dev, size_t head_stride) {
    if (D != 64) return moon_fail(ctx, MOON_EINVAL_DIM, "decode attention: head_dim %zu unsupported (64 only)", D);
    if (max_seq > 2048 || pos >= max_seq) return moon_fail(ctx, MOON_ESEQ_TOO_LONG, "decode attention: pos %zu >= max_seq %zu (limit 2048)", pos, max_seq);
    // (two prefetch depths: up to 4 steps of 32 keys per split, which is 896 cached keys, and everything beyond; see launch_decode_layer)
    if ((pos + DEC_SPLITS - 2) / (DEC_SPLITS - 1) <= 128)
        hipLaunchKernelGGL((decode_attn_merged_kernel<64, 4>), dim3((unsigned)(H * DEC_SPLITS)), dim3(256), 0, ctx->stream, qkv, cache_k, cache_v, table,
                           partial, out, head_count, count_target, (int)H, (int)rot_dim, (int)max_seq, (int)pos, pos_dev, (int)head_stride);
    else
        hipLaunchKernelGGL((decode_attn_merged_kernel<64, 10>), dim3((unsigned)(H * DEC_SPLITS)), dim3(256), 0, ctx->stream, qkv, cache_k, cache_v, table,
                           partial, out, head_count, count_target, (int)H, (int)rot_dim, (int)max_seq, (int)pos, pos_dev, (int)head_stride);
    MOON_HIP(ctx, hipGetLastError());
    MOON_NOTE_KERNEL(ctx, "decode_attn_merged_kernel<64> %d workgroups", (int)(H * DEC_SPLITS));
    return MOON_OK;
}

int launch_argmax_record(moon_ctx *ctx, const half_t *logits, size_t n, uint32_t *state, uint32_t *out_ids) {
    if (!n || n > 0x7fffffff) return moon_fail(ctx, MOON_EINVAL, "argmax: empty or oversized tensor");
    hipLaunchKernelGGL(argmax_record_kernel, dim3(1), dim3(1024), 0, ctx->stream, logits, (int)n, state, out_ids);
    MOON_HIP(ctx, hipGetLastError());
    return MOON_OK;
}
