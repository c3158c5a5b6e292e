// Token sampling on the device: sampling.sample of the reference (src/utils/sampling.zig:353-389) for its
// multinomial, top_k and min_p methods, on one row of f16 logits that already sits in HBM (the LM head's output),
// so a decode loop never copies 100 KiB of logits to the host to pick one index.
//
// One workgroup of 1024 threads; thread t owns the contiguous indices [t*C, (t+1)*C).  Up to 65536 logits the
// probabilities are computed once and stay in registers (C is a compile-time constant); beyond that they are recomputed
// from the logits wherever they are needed.  The reference draws one number from its PRNG per call (rng.float(f32));
// that number is an argument here (u, or u_dev[step]), the generator stays with the caller.  Probabilities are formed
// with the reference's operations in the reference's order per element (f32 divide by the temperature, subtract the
// maximum, exp with the -88 cut-off, multiply by 1/sum).  The reference's sums over the whole vocabulary are sequential
// f32 loops (ops.zig:1585-1592, sampling.zig:139-147, 281-294, 200-214), and which candidate a draw lands on depends on
// their rounding; seq_prefix below evaluates such a loop bit for bit with 1024 threads, so the index is the reference's.
// That evaluation costs a few hundred microseconds, so the kernel first takes its sums the fast way and keeps the answer
// only where it provably cannot depend on how they were rounded (the draw clear of the running sums next to it by more
// than any evaluation can move them, the candidate set clear of its thresholds); otherwise it runs the exact one.  With
// the reference's default (top_k 3) the exact path is taken on a few draws in 10^5.
#pragma clang fp contract(off)
#include "moon_internal.hpp"
#include "sample_quick.hpp"
#include "seq_sum.hpp"

#include <atomic>
#include <cmath>
#include <type_traits>

namespace {

constexpr int ST = 1024;    // threads
constexpr int COPIES = 32;  // histogram copies, one per LDS bank, so that equal digits of different lanes do not queue up

struct SampleArgs {
    const half_t *logits;
    const float *logits_f32; // when set: the row as f32 (the type sampling.sample takes, sampling.zig:353); logits is unused
    int n, method, k;
    float temperature, min_p, u;
    float scale;        // 1 / temperature when that is exact (a power of two), else 0: the division is then a multiplication
    const float *u_dev; // when set: u = u_dev[state ? state[1] : 0]
    uint32_t *state;    // decode loop bookkeeping: state[2] = token, out_ids[state[1]++] = token, state[0] += bump_pos
    uint32_t bump_pos;
    uint32_t *out_ids;
    uint32_t *out;      // when set: out[0] = token
    const uint32_t *skip_if; // when set and *skip_if != 0: the token of this step is already decided, nothing to do
};

struct SampleShared {
    float s16[16];
    int s16i[16];
    float scan[ST];
    unsigned hist[256 * COPIES];
    unsigned digit_count[256];
    unsigned long long cand[ST];
    unsigned sel[3];
    int first, last, result;
    unsigned count;
    unsigned map0[16], map1[16]; // seq_prefix: the wavefronts' composed maps
    float seq_s;                 // seq_prefix: the running sum at the start of chunk seq_cur
    int seq_cross;
    int safe;                    // the quick path's result is provably the exact path's
};

__device__ __forceinline__ float block_max(float v, float *s16) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    __syncthreads(); // s16 may still be read from the previous reduction
    if ((threadIdx.x & 63) == 0) s16[threadIdx.x >> 6] = v;
    __syncthreads();
    float r = s16[0];
#pragma unroll
    for (int w = 1; w < ST / 64; w++) r = fmaxf(r, s16[w]);
    return r;
}
__device__ __forceinline__ float block_sum(float v, float *s16) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) s16[threadIdx.x >> 6] = v;
    __syncthreads();
    float r = s16[0];
#pragma unroll
    for (int w = 1; w < ST / 64; w++) r += s16[w];
    return r;
}
__device__ __forceinline__ int block_min_int(int v, int *s16) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v = min(v, __shfl_xor(v, off, 64));
    __syncthreads();
    if ((threadIdx.x & 63) == 0) s16[threadIdx.x >> 6] = v;
    __syncthreads();
    int r = s16[0];
#pragma unroll
    for (int w = 1; w < ST / 64; w++) r = min(r, s16[w]);
    return r;
}

// A sequential f32 sum  s = 0; for i: s += w_i  over non-negative terms, evaluated bit for bit by the workgroup.
// While s stays inside one binade [2^b, 2^(b+1)) it is an integer S in [2^23, 2^24) times ulp = 2^(b-23), and adding w
// rounds S + w / ulp to an integer: S + E when the fraction of w / ulp is below a half, S + E + 1 when above, and to the
// even one of the two on a tie.  So every term is a map S -> S + c[S & 1] with two small integers c[0], c[1]; such maps
// compose associatively (the parity after the first map picks the second map's entry), which a scan over the 1024
// threads' chunks evaluates exactly.  Nothing is trusted past the first chunk in which S would reach 2^24 (s leaves the
// binade, the ulp changes) or a term is not smaller than the binade itself: the thread that owns that chunk runs the
// plain float loop over it, and the next phase starts behind it with the new binade.  A sum crosses a few dozen binades
// at most, most of them inside the first chunks.
// each(f) calls f(i, w_i) for the thread's own indices in ascending order.  On return sh.scan[t] holds the running sum
// BEFORE chunk t (exact), and the function returns the total.
template <class Each>
__device__ __forceinline__ float seq_prefix(Each each, SampleShared &sh) {
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    __syncthreads();
    if (t == 0) sh.seq_s = 0.f;
    int cur = 0;  // chunks before cur are done: sh.scan[0..cur) are final
    int win = 64; // chunks looked at per phase: doubled whenever a phase ends without leaving its binade, so that the terms
                  // are visited two or three times in all rather than once per binade
    __syncthreads();
    while (cur < ST) {
        const float s = sh.seq_s;
        const unsigned sbits = __float_as_uint(s);
        int sb = (int)((sbits >> 23) & 255u);
        if (sb <= 1) sb = 0;
        const unsigned S0 = sb ? ((sbits & 0x7fffffu) | 0x800000u) : 0u;
        const int wend = min(cur + win, ST);
        const bool mine = t >= cur && t < wend;
        SeqMap m{0u, 0u};
        if (mine)
            each([&](int, float w) {
                m = seq_compose(m, seq_elem(w, sb));
            });
        SeqMap inc = m; // inclusive scan over the threads in ascending order
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            SeqMap o;
            o.c0 = __shfl_up(inc.c0, off, 64);
            o.c1 = __shfl_up(inc.c1, off, 64);
            if (lane >= off) inc = seq_compose(o, inc);
        }
        if (lane == 63) {
            sh.map0[wave] = inc.c0;
            sh.map1[wave] = inc.c1;
        }
        if (t == 0) sh.seq_cross = ST;
        __syncthreads();
        SeqMap before{0u, 0u};
        for (int w = 0; w < wave; w++) before = seq_compose(before, SeqMap{sh.map0[w], sh.map1[w]});
        inc = seq_compose(before, inc);
        SeqMap exc; // everything before this thread's chunk
        exc.c0 = __shfl_up(inc.c0, 1, 64);
        exc.c1 = __shfl_up(inc.c1, 1, 64);
        if (lane == 0) exc = before;
        const unsigned p = S0 & 1u;
        const unsigned start = S0 + (p ? exc.c1 : exc.c0), end = S0 + (p ? inc.c1 : inc.c0);
        // sb == 0: S counts nothing, a non-zero term anywhere in the chunk shows as >= SEQ_BIG
        if (mine && end >= SEQ_BIG) atomicMin(&sh.seq_cross, t);
        __syncthreads();
        const int x = sh.seq_cross;
        if (mine && t <= x) sh.scan[t] = sb ? __uint_as_float(((unsigned)sb << 23) | (start & 0x7fffffu)) : s;
        if (x == ST) { // the window stayed inside the binade
            if (t == wend - 1) sh.seq_s = sb ? __uint_as_float(((unsigned)sb << 23) | (end & 0x7fffffu)) : s;
            cur = wend;
            win = min(2 * win, ST);
        } else {
            if (t == x) { // the plain loop over the chunk that leaves the binade
                float v = sh.scan[t];
                each([&](int, float w) { v += w; });
                sh.seq_s = v;
            }
            cur = x + 1;
        }
        __syncthreads();
    }
    return sh.seq_s;
}

// The candidate walk of multinomial_sampling / min_p_sampling (sampling.zig:276-297, 199-218): candidates in index
// order with weight wt(probability) (0 = not a candidate; adding 0 changes nothing, so skipping them is the same loop),
// r = u * (sum of the weights), first candidate with r < running sum.  each(f) calls f(i, probability) for the thread's
// own indices in ascending order.  The running sums at the chunk starts and the total are the reference's bits
// (seq_prefix); the one chunk whose end is the first above r is walked with the same float additions.  Returns -1 when r
// is not below the total (the caller's fall-back).
template <class Each, class Wt>
__device__ __forceinline__ int walk_exact(Each each, Wt wt, float u, SampleShared &sh) {
    const int t = threadIdx.x;
    const float total = seq_prefix([&](auto f) { each([&](int i, float pi) { f(i, wt(pi)); }); }, sh);
    const float r = u * total;
    if (t == 0) sh.first = ST;
    __syncthreads();
    const float end = t + 1 < ST ? sh.scan[t + 1] : total; // the running sum behind this chunk
    if (r < end) atomicMin(&sh.first, t);
    __syncthreads();
    const int c = sh.first;
    if (c == ST) return -1;
    if (t == c) {
        float cum = sh.scan[c];
        int res = -1;
        each([&](int i, float pi) {
            if (res < 0) {
                cum += wt(pi);
                if (r < cum) res = i;
            }
        });
        sh.result = res;
    }
    __syncthreads();
    return sh.result;
}

// The quick form of the same walk: sequential sums inside a chunk, a scan over the 1024 chunk sums, the chunk that holds
// r walked by one thread.  Its sums are not the reference's bits, so it only answers when the answer cannot depend on them:
// with m candidates, the running sums and r = u * total, taken in any order and with any 1 / sum behind the probabilities
// (every probability is one multiplication by the same factor, so the factor cancels in r against a running sum up to the
// roundings), stay within (6 m + 32) 2^-24 of the total of their exact values; if r keeps at least that distance from the
// two running sums around the chosen candidate, every such evaluation names this candidate.  Otherwise sh.safe is
// cleared and the caller takes the exact path.  m: the number of candidates (the caller counts them).
template <class Each, class Wt>
__device__ __forceinline__ int walk_quick(Each each, Wt wt, float u, unsigned m, SampleShared &sh) {
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    float cs = 0.f;
    each([&](int, float pi) { cs += wt(pi); });
    float incl = cs;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const float o = __shfl_up(incl, off, 64);
        if (lane >= off) incl += o;
    }
    __syncthreads();
    if (lane == 63) sh.s16[wave] = incl;
    if (t == 0) sh.first = ST;
    __syncthreads();
    float base = 0.f, total = 0.f;
    for (int wv = 0; wv < ST / 64; wv++) {
        if (wv == wave) base = total;
        total += sh.s16[wv];
    }
    incl = base + incl;
    sh.scan[t] = incl;
    const float r = u * total;
    if (cs > 0.f && r < incl) atomicMin(&sh.first, t);
    __syncthreads();
    const int c = sh.first;
    const float tol = (6.0f * (float)m + 32.0f) * 0x1p-24f * total;
    if (c == ST || !(tol < 0.25f * total)) { // r not clearly below the total, or too many candidates for the bound to say anything
        if (t == 0) sh.safe = 0;
        __syncthreads();
        return -1;
    }
    if (t == c) { // walk this chunk from the running sum the chunk before it ended on
        float cum = c ? sh.scan[c - 1] : 0.f, below = cum;
        int res = -1;
        each([&](int i, float pi) {
            const float w = wt(pi);
            if (res < 0 && w > 0.f) {
                below = cum;
                cum += w;
                if (r < cum) res = i;
            }
        });
        sh.result = res;
        if (res < 0 || !(r - below > tol) || !(cum - r > tol)) sh.safe = 0;
    }
    __syncthreads();
    return sh.result;
}

// top_k_sampling (sampling.zig:300-339) for k <= 1024.  Order of the reference's stable descending sort = descending
// order of the 64-bit key (probability bits, ~index): probabilities are not negative, so their bit patterns order like
// their values, and among equal probabilities the lower index has the larger key.  Keys are distinct, so the k largest
// are exactly the keys >= the k-th largest, which a radix select finds 8 bits at a time without sorting the vocabulary;
// those k are then sorted (bitonic, in LDS) and walked by one thread with the reference's sequential sums.
// QUICK: each() yields the exps (not the probabilities), scale is a 1 / sum that need not be the reference's bits, and
// k + 1 keys are selected.  Ordering by the exps is the reference's ordering by the probabilities (one multiplication of
// every exp by the same factor, rounded: monotone) unless two different exps are so close that the factor can round them
// to one value, where the index would decide instead: any two neighbours among the k + 1 must be equal or more than
// 2^-21 apart in relative terms.  The draw must keep (6 k + 32) 2^-24 of the total away from the running sums around the
// chosen candidate (the factor cancels in r against a running sum up to the roundings).  Both hold: the index is what
// the exact evaluation returns; else sh.safe is cleared.
template <bool QUICK, class Each>
__device__ __forceinline__ int top_k_walk(Each each, unsigned k, float scale, float u, SampleShared &sh) {
    const int t = threadIdx.x, copy = t & (COPIES - 1);
    const unsigned nsel = QUICK ? k + 1 : k; // the caller makes sure that nsel fits ST and the row
    unsigned k_rem = nsel, digit = 0;
    // One pass of the select: count, per value of an 8-bit digit, the keys that still match everything decided so far
    // (digit_if_match gives the digit, or -1), then move on to the digit whose bucket holds the k_rem-th largest of them.
    // True when every key of that bucket is among the k: nothing below this digit needs looking at.
    auto pass = [&](auto digit_if_match) {
        for (int e = t; e < 256 * COPIES; e += ST) sh.hist[e] = 0;
        __syncthreads();
        each([&](int i, float pi) {
            const int d = digit_if_match(i, pi);
            if (d >= 0) atomicAdd(&sh.hist[d * COPIES + copy], 1u);
        });
        __syncthreads();
        if (t < 256) {
            unsigned c = 0;
            for (int e = 0; e < COPIES; e++) c += sh.hist[t * COPIES + ((e + t) & (COPIES - 1))];
            sh.digit_count[t] = c;
        }
        __syncthreads();
        if (t < 64) { // lane l looks at digits 255-4l .. 252-4l, a scan over the lanes counts the keys in higher digits
            unsigned c[4], mine = 0;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                c[e] = sh.digit_count[255 - 4 * t - e];
                mine += c[e];
            }
            unsigned incl = mine;
#pragma unroll
            for (int off = 1; off < 64; off <<= 1) {
                const unsigned o = __shfl_up(incl, off, 64);
                if (t >= off) incl += o;
            }
            const unsigned long long reached = __ballot(incl >= k_rem);
            if (reached && t == __builtin_ctzll(reached)) {
                unsigned above = incl - mine;
                int e = 0;
                for (; e < 3; e++) {
                    if (above + c[e] >= k_rem) break;
                    above += c[e];
                }
                sh.sel[0] = (unsigned)(255 - 4 * t - e);
                sh.sel[1] = above;
                sh.sel[2] = c[e];
            }
        }
        __syncthreads();
        digit = sh.sel[0];
        k_rem -= sh.sel[1];
        const bool whole_bucket = sh.sel[2] == k_rem;
        __syncthreads();
        return whole_bucket;
    };
    // the probability's bits first, 8 at a time; the index only if the k-th largest probability is shared and not all
    // of its holders fit (then the lower indices win: larger ~index)
    unsigned vprefix = 0, vmask = 0, iprefix = 0, imask = 0;
    bool whole = false;
    for (int shift = 24; shift >= 0 && !whole; shift -= 8) {
        whole = pass([&](int, float pi) {
            const unsigned b = __float_as_uint(pi);
            return (b & vmask) == vprefix ? (int)((b >> shift) & 255u) : -1;
        });
        vprefix |= digit << shift;
        vmask |= 255u << shift;
    }
    for (int shift = 24; shift >= 0 && !whole; shift -= 8) {
        whole = pass([&](int i, float pi) {
            const unsigned x = ~(unsigned)i;
            return (__float_as_uint(pi) == vprefix && (x & imask) == iprefix) ? (int)((x >> shift) & 255u) : -1;
        });
        iprefix |= digit << shift;
        imask |= 255u << shift;
    }
    if (t == 0) sh.count = 0;
    sh.cand[t] = 0; // below every real key (a real key's low word is ~index, never 0)
    __syncthreads();
    each([&](int i, float pi) {
        const unsigned b = __float_as_uint(pi), x = ~(unsigned)i;
        if (b > vprefix || (b == vprefix && x >= iprefix)) {
            const unsigned pos = atomicAdd(&sh.count, 1u);
            if (pos < (unsigned)ST) *reinterpret_cast<uint2 *>(&sh.cand[pos]) = make_uint2(x, b); // low word ~index, high word the probability's bits
        }
    });
    unsigned P = 1;
    while (P < nsel) P <<= 1;
    // Bitonic sort, descending, one key per thread: partners less than a wavefront apart trade keys through shuffles,
    // the others through LDS.
    __syncthreads();
    unsigned long long key = sh.cand[t];
    for (unsigned size = 2; size <= P; size <<= 1)
        for (unsigned stride = size >> 1; stride > 0; stride >>= 1) {
            unsigned long long other;
            if (stride >= 64) {
                __syncthreads();
                sh.cand[t] = key;
                __syncthreads();
                other = sh.cand[(unsigned)t ^ stride];
            } else {
                const unsigned lo_w = __shfl_xor((unsigned)key, (int)stride, 64), hi_w = __shfl_xor((unsigned)(key >> 32), (int)stride, 64);
                other = ((unsigned long long)hi_w << 32) | lo_w;
            }
            const bool descending = ((unsigned)t & size) == 0, lower = ((unsigned)t & stride) == 0;
            const bool keep_larger = lower == descending;
            key = (keep_larger == (other > key)) ? other : key;
        }
    __syncthreads();
    sh.cand[t] = key;
    __syncthreads();
    // Running sums in the reference's order (sampling.zig:323-338), taken once by one thread (16 candidates are read ahead
    // of the dependent additions) and kept; every thread then tests its own candidate against r = u * total, and the
    // lowest position that passes wins.  Places past k hold probability 0: adding them changes nothing, so no step of the
    // loop is conditional.  Falls back to the last of the k.
    if (QUICK) { // neighbours among the k + 1: equal, or clearly apart
        if ((unsigned)t + 1 < nsel) {
            const float a = __uint_as_float((unsigned)(sh.cand[t] >> 32)), b = __uint_as_float((unsigned)(sh.cand[t + 1] >> 32));
            if (a != b && !(a - b > a * 0x1p-21f)) sh.safe = 0;
        }
    }
    if (t == 0) {
        float cum = 0.f, w[16], w_next[16];
        auto weight = [&](unsigned j) {
            const float x = __uint_as_float((unsigned)(sh.cand[j] >> 32));
            return QUICK ? (j < k ? x * scale : 0.f) : x; // the probability: one multiplication (ops.zig:1598)
        };
#pragma unroll
        for (int e = 0; e < 16; e++) w[e] = weight(e);
        for (unsigned j0 = 0; j0 < k; j0 += 16) {
            const unsigned j1 = j0 + 16 < (unsigned)ST ? j0 + 16 : 0; // the block after this one, read while this one is added up
#pragma unroll
            for (int e = 0; e < 16; e++) w_next[e] = weight(j1 + e);
#pragma unroll
            for (int e = 0; e < 16; e++) {
                cum += w[e];
                sh.scan[j0 + e] = cum;
            }
#pragma unroll
            for (int e = 0; e < 16; e++) w[e] = w_next[e];
        }
        sh.first = (int)k - 1;
    }
    __syncthreads();
    const float total = sh.scan[k - 1], r = u * total;
    if ((unsigned)t < k && r < sh.scan[t]) atomicMin(&sh.first, t);
    __syncthreads();
    const int first = sh.first;
    if (QUICK && t == 0) {
        const float tol = (6.0f * (float)k + 32.0f) * 0x1p-24f * total, below = first ? sh.scan[first - 1] : 0.f;
        if (!(r - below > tol) || !(sh.scan[first] - r > tol) || !(tol < 0.25f * total)) sh.safe = 0;
    }
    return (int)~(unsigned)sh.cand[first];
}

// J > 0: J (even) logits per thread, probabilities kept in registers; the logits pointer is 4-byte aligned.
// J == 0: any size and alignment, probabilities recomputed from the logits at every use.
template <int J, int METHOD>
__global__ __launch_bounds__(ST) void sample_kernel(SampleArgs p) {
    extern __shared__ __attribute__((aligned(16))) unsigned char dyn_lds[]; // the staged logits, then SampleShared
    SampleShared &sh = *reinterpret_cast<SampleShared *>(dyn_lds);
    if (p.skip_if && *p.skip_if) return; // (the same word for every thread: the whole workgroup leaves)
    const int t = threadIdx.x, n = p.n;
    const half_t *__restrict__ logits = p.logits;
    const float *__restrict__ logits_f32 = p.logits_f32;
    auto lg = [&](int i) { return logits_f32 ? logits_f32[i] : (float)logits[i]; };
    const float temperature = p.temperature;
    const float u = p.u_dev ? p.u_dev[p.state ? p.state[1] : 0] : p.u;
    const int C = J ? J : (n + ST - 1) / ST, lo = min(n, t * C), hi = min(n, lo + C); // the J == 0 kernel's chunk
    float v[J ? J : 1];

    // apply_temperature (sampling.zig:342-350) happens only for a temperature other than 1 (sampling.zig:363-366)
    // (dividing by a power of two and multiplying by its reciprocal round alike: both are exact up to the same overflow / underflow)
    const float scale = p.scale;
    auto x_of = [&](float logit) { return temperature == 1.0f ? logit : scale != 0.f ? logit * scale : __fdiv_rn(logit, temperature); };
    // the maximum of the scaled logits is the scaled maximum: dividing by a positive number keeps the order
    float mx = -INFINITY;
    if constexpr (J > 0) {
        // Coalesced 4-byte loads (two logits) into LDS, then every thread reads its own chunk of J/2 words back.  A chunk
        // starts every PITCH words, an odd number, so the 64 lanes of a wavefront read from different banks.  Places past
        // the end hold -inf: probability 0, never a candidate of a walk, and in top_k's order (probability, then lower
        // index first) behind every real logit, so nothing below needs to know where the row ends.
        constexpr int HW = J / 2, PITCH = HW + (HW % 2 == 0 ? 1 : 0);
        constexpr uint32_t NEG_INF2 = 0xfc00fc00u;
        uint32_t *stage = reinterpret_cast<uint32_t *>(dyn_lds);
        const uint32_t *pairs = reinterpret_cast<const uint32_t *>(logits);
#pragma unroll 5
        for (int w = t; w < ST * HW; w += ST) {
            uint32_t raw = NEG_INF2;
            if (2 * w + 1 < n)
                raw = pairs[w];
            else if (2 * w < n)
                raw = reinterpret_cast<const uint16_t *>(logits)[2 * w] | 0xfc000000u;
            stage[(w / HW) * PITCH + (w % HW)] = raw;
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < J; j += 2) {
            const uint32_t raw = stage[t * PITCH + j / 2];
            v[j] = (float)__builtin_bit_cast(half_t, (uint16_t)(raw & 0xffffu));
            v[j + 1] = (float)__builtin_bit_cast(half_t, (uint16_t)(raw >> 16));
            mx = fmaxf(mx, fmaxf(v[j], v[j + 1]));
        }
        __syncthreads(); // sh lives in the same memory
    } else {
        for (int i = lo; i < hi; i++) mx = fmaxf(mx, lg(i));
    }
    mx = x_of(block_max(mx, sh.s16));
    auto e_of = [&](float logit) {
        const float d = x_of(logit) - mx;
        return d > -88.0f ? sampling_expf(d) : 0.f; // ops.zig:1589-1590, sampling.zig:145
    };
    if constexpr (J > 0) {
#pragma unroll
        for (int j = 0; j < J; j++) v[j] = e_of(v[j]);
    }
    // v[] holds the exps from here on; a probability is one multiplication, exp * (1 / sum) (ops.zig:1598, sampling.zig:150-153)
    float inv = 1.f;
    bool normalise = true;
    // f(i, exp of i) for the thread's own indices, ascending
    auto each_exp = [&](auto f) {
        if constexpr (J > 0) {
            int first = t * J;
            asm volatile("" : "+v"(first)); // or the compiler keeps every index (and what callers derive from it) in a register of its own across the passes
#pragma unroll
            for (int j = 0; j < J; j++) f(first + j, v[j]);
        } else {
            for (int i = lo; i < hi; i++) f(i, e_of(lg(i)));
        }
    };
    // f(i, probability of i)
    auto each = [&](auto f) { each_exp([&](int i, float e) { f(i, normalise ? e * inv : e); }); };
    // the same as a loop that stays a loop: the phases of seq_prefix run it many times, and fifty unrolled copies of their
    // body each time cost more registers than a lane has
    // (over a copy of the exps that is made when the exact path is entered: indexing by a loop variable puts an array in
    // scratch memory, and the quick path's unrolled passes should keep theirs in registers)
    float vs[J ? J : 1];
    auto each_exp_rolled = [&](auto f) {
        if constexpr (J > 0) {
#pragma unroll 1
            for (int j = 0; j < J; j++) f(t * J + j, vs[j]);
        } else {
            each_exp(f);
        }
    };
    auto each_rolled = [&](auto f) { each_exp_rolled([&](int i, float e) { f(i, normalise ? e * inv : e); }); };

    // One evaluation of the method with the current 1 / sum.  quick: sums in whatever order is fast, and sh.safe is cleared
    // unless the result provably does not depend on that (see walk_quick / top_k_walk); exact: the reference's loops, bit
    // for bit.
    auto run = [&](auto quick_tag) -> int {
        constexpr bool QUICK = decltype(quick_tag)::value;
        int token;
        if constexpr (METHOD == MOON_SAMPLE_MULTINOMIAL) { // multinomial_sampling (sampling.zig:276-297); falls back to the last index
            if constexpr (QUICK) {
                token = walk_quick(each, [](float pi) { return pi; }, u, (unsigned)n, sh);
            } else {
                token = walk_exact(each_rolled, [](float pi) { return pi; }, u, sh);
                if (token < 0) token = n - 1;
            }
        } else if constexpr (METHOD == MOON_SAMPLE_MIN_P) { // min_p_sampling (sampling.zig:114-219)
            float max_prob = 0.f;
            each([&](int, float pi) { max_prob = fmaxf(max_prob, pi); });
            max_prob = block_max(max_prob, sh.s16);
            const float threshold = p.min_p * max_prob;
            int first_valid = 0x7fffffff, first_max = 0x7fffffff;
            each([&](int i, float pi) {
                if (pi >= threshold) first_valid = min(first_valid, i);
                if (pi == max_prob) first_max = min(first_max, i);
            });
            first_valid = block_min_int(first_valid, sh.s16i);
            unsigned m = 0;
            if constexpr (QUICK) {
                // Which indices are candidates, and which is the first maximum, must not depend on the factor either: an exp
                // equal to the largest one or clearly below it, and clearly on one side of min_p times the largest one.
                float e_max = 0.f;
                each_exp([&](int, float e) { e_max = fmaxf(e_max, e); });
                e_max = block_max(e_max, sh.s16);
                const float edge = p.min_p * e_max;
                int close = 0, count = 0;
                each_exp([&](int, float e) {
                    if (e != e_max && !(e_max - e > e_max * 0x1p-21f)) close = 1;
                    if (fabsf(e - edge) <= edge * 0x1p-20f) close = 1;
                    if (e > edge) count++;
                });
                if (close) sh.safe = 0;
                m = (unsigned)block_sum((float)count, sh.s16); // at most 2^24 of them: the float sum is the integer
            }
            if (first_valid == 0x7fffffff) { // nothing reaches the threshold: keep the first maximum (sampling.zig:183-197)
                token = block_min_int(first_max, sh.s16i);
                if (token == 0x7fffffff) token = 0; // not-a-number logits
            } else if constexpr (QUICK) {
                token = walk_quick(each, [&](float pi) { return pi >= threshold ? pi : 0.f; }, u, m, sh);
            } else {
                token = walk_exact(each_rolled, [&](float pi) { return pi >= threshold ? pi : 0.f; }, u, sh);
                if (token < 0) token = first_valid; // sampling.zig:217-218
            }
        } else {
            const unsigned k = (unsigned)min(p.k, n);
            if constexpr (QUICK) {
                if (k + 1 > (unsigned)n || k + 1 > (unsigned)ST) { // no (k+1)-th key to compare the k-th with
                    if (t == 0) sh.safe = 0;
                    token = 0;
                } else {
                    token = top_k_walk<true>(each_exp, k, inv, u, sh);
                }
            } else {
                token = top_k_walk<false>(each, k, 1.f, u, sh);
            }
        }
        return token;
    };

    // the quick attempt: the sum of the exps as a tree
    if (t == 0) sh.safe = 1;
    float sum = 0.f;
    each_exp([&](int, float e) { sum += e; });
    sum = block_sum(sum, sh.s16); // (its barriers also publish sh.safe)
    inv = __fdiv_rn(1.0f, sum);
    if (!(sum > 0.f) && t == 0) sh.safe = 0; // not-a-number logits: the exact path decides
    __syncthreads();
    int token = run(std::true_type{});
    __syncthreads();
    if (!sh.safe) {
        if constexpr (J > 0) {
#pragma unroll
            for (int j = 0; j < J; j++) vs[j] = v[j];
        }
        // the sum of the exps in the reference's sequential order (ops.zig:1585-1592; sampling.zig:139-147 for min_p)
        sum = seq_prefix(each_exp_rolled, sh);
        inv = __fdiv_rn(1.0f, sum);
        // ops.softmax normalises only a positive sum (ops.zig:1595; otherwise it leaves its input, the scaled logits, in place:
        // only a not-a-number logit gets there, and the exps stand in here); min_p always does (sampling.zig:150)
        normalise = METHOD == MOON_SAMPLE_MIN_P || sum > 0.f;
        token = run(std::false_type{});
    }
    if (t == 0) {
        if (p.out) p.out[0] = (uint32_t)token;
        if (p.state) record_token(p.state, p.out_ids, (uint32_t)token, p.bump_pos); // as the fused LM-head + arg-max kernel does
    }
}

template <int J, int METHOD>
hipError_t launch_sample_kernel_m(hipStream_t stream, const SampleArgs &a) {
    constexpr size_t stage_bytes = size_t(ST) * (J / 2 + ((J / 2) % 2 == 0 ? 1 : 0)) * 4;
    constexpr size_t lds_bytes = stage_bytes > sizeof(SampleShared) ? stage_bytes : sizeof(SampleShared);
    static std::atomic<bool> allowed[64]; // per device: the kernel has been allowed this much dynamic LDS (setting it twice is harmless)
    int device = 0;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess) return e;
    if (device < 0 || device >= 64 || !allowed[device].load()) {
        e = hipFuncSetAttribute(reinterpret_cast<const void *>(sample_kernel<J, METHOD>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
        if (e != hipSuccess) return e;
        if (device >= 0 && device < 64) allowed[device].store(true);
    }
    hipLaunchKernelGGL((sample_kernel<J, METHOD>), dim3(1), dim3(ST), lds_bytes, stream, a);
    return hipGetLastError();
}
template <int J>
hipError_t launch_sample_kernel(hipStream_t stream, const SampleArgs &a) {
    if (a.method == MOON_SAMPLE_MULTINOMIAL) return launch_sample_kernel_m<J, MOON_SAMPLE_MULTINOMIAL>(stream, a);
    if (a.method == MOON_SAMPLE_MIN_P) return launch_sample_kernel_m<J, MOON_SAMPLE_MIN_P>(stream, a);
    return launch_sample_kernel_m<J, MOON_SAMPLE_TOP_K>(stream, a);
}

} // namespace

// sampling.sample for methods multinomial / top_k / min_p; greedy goes to the arg-max kernels (it ignores the temperature).
int launch_sample(moon_ctx *ctx, const half_t *logits, size_t n, const moon_sampling_config *cfg, float u, const float *u_dev,
                  uint32_t *state, uint32_t *out_ids, uint32_t *out, uint32_t bump_pos, const float *logits_f32, const uint32_t *skip_if) {
    if (!cfg) return moon_fail(ctx, MOON_EINVAL, "sample: null config");
    if (!n || n > 0x3fffffff) return moon_fail(ctx, MOON_EINVAL, "sample: empty or oversized tensor");
    if (cfg->method < MOON_SAMPLE_MULTINOMIAL || cfg->method > MOON_SAMPLE_MIN_P)
        return moon_fail(ctx, MOON_EINVAL, "sample: unknown method %d", cfg->method);
    if (cfg->temperature != 1.0f && !(cfg->temperature > 0.f))
        return moon_fail(ctx, MOON_ETEMPERATURE, "sample: temperature %g (InvalidTemperature)", (double)cfg->temperature);
    size_t k = 0;
    if (cfg->method == MOON_SAMPLE_TOP_K) {
        if (!cfg->top_k) return moon_fail(ctx, MOON_EINVAL, "sample: top_k of 0 leaves nothing to draw from");
        k = cfg->top_k < n ? cfg->top_k : n;
        if (k > (size_t)ST) return moon_fail(ctx, MOON_EINVAL, "sample: top_k %zu (at most %d candidates are sorted on the device)", k, ST);
    }
    SampleArgs a;
    a.logits = logits; a.logits_f32 = logits_f32; a.n = (int)n; a.method = cfg->method; a.k = (int)k;
    a.temperature = cfg->temperature; a.min_p = cfg->min_p; a.u = u; a.u_dev = u_dev;
    int exponent = 0;
    a.scale = (std::frexp(cfg->temperature, &exponent) == 0.5f && exponent > -100 && exponent < 100) ? 1.0f / cfg->temperature : 0.f;
    a.state = state; a.out_ids = out_ids; a.out = out; a.bump_pos = bump_pos; a.skip_if = skip_if;
    const size_t per_thread = (n + ST - 1) / ST;
    const bool in_registers = !logits_f32 && per_thread <= 64 && (reinterpret_cast<uintptr_t>(logits) & 3) == 0;
    hipError_t e;
    if (!in_registers) e = launch_sample_kernel<0>(ctx->stream, a);
    else if (per_thread <= 4) e = launch_sample_kernel<4>(ctx->stream, a);
    else if (per_thread <= 16) e = launch_sample_kernel<16>(ctx->stream, a);
    else if (per_thread <= 32) e = launch_sample_kernel<32>(ctx->stream, a);
    else if (per_thread <= 50) e = launch_sample_kernel<50>(ctx->stream, a);
    else e = launch_sample_kernel<64>(ctx->stream, a);
    MOON_HIP(ctx, e);
    return MOON_OK;
}
