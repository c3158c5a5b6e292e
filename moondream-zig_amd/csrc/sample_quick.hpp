// What the sampling kernel (sample.hip) and the LM-head kernel of the sampled decode loop (decode_fused.hip) share: the
// exp both use, and top_k's decision from the k + 1 largest logits alone, kept only where it provably is the reference's.
#pragma once
#include "moon_internal.hpp"

namespace {

// exp of the sampling paths: the classic libm expf (k = round(x / ln 2), x - k ln2 in two parts, c = x - x^2 (P1 + x^2 P2),
// 1 + (x c / (2 - c) - lo + hi), scaled by 2^k) spelled out in separate IEEE f32 operations (contraction is off in this
// function), because which candidate a draw lands on depends on the last bit of every term: the device and the
// checker share this definition instead of each trusting its own library's expf.
__device__ __forceinline__ float sampling_expf(float x) {
#pragma clang fp contract(off)
    const float ln2hi = 6.9314575195e-1f, ln2lo = 1.4286067653e-6f, invln2 = 1.4426950216e+0f, P1 = 1.6666625440e-1f, P2 = -2.7667332906e-3f;
    const unsigned ux = __float_as_uint(x);
    const int sign = (int)(ux >> 31);
    const unsigned hx = ux & 0x7fffffffu;
    if (hx > 0x7f800000u) return x;
    if (hx >= 0x42b17218u && !sign) return x * 0x1p127f;
    if (sign && hx >= 0x42cff1b5u) return 0.0f;
    float hi, lo, xr;
    int k;
    if (hx > 0x3eb17218u) {
        if (hx > 0x3f851592u) k = (int)(invln2 * x + (sign ? -0.5f : 0.5f));
        else k = 1 - sign - sign;
        hi = x - (float)k * ln2hi;
        lo = (float)k * ln2lo;
        xr = hi - lo;
    } else if (hx > 0x39000000u) {
        k = 0;
        hi = x;
        lo = 0.0f;
        xr = x;
    } else
        return 1.0f + x;
    const float xx = xr * xr;
    const float c = xr - xx * (P1 + xx * P2);
    const float y = 1.0f + (__fdiv_rn(xr * c, 2.0f - c) - lo + hi);
    return k == 0 ? y : ldexpf(y, k);
}

// ---- top_k decided from the k + 1 largest logits (the sampled decode loop, k < QUICK_KEYS)
// Where the LM head's workgroups already hold the logits, each keeps its QUICK_KEYS largest as keys (logit in an order-
// preserving code, ~index: larger logit first, then lower index, the order of the reference's stable descending sort
// wherever the probability is a strictly increasing function of the logit), its maximum and a rough sum of exps; the
// workgroup that finishes last merges them and calls quick_top_k below.  Everything that is not provably the reference's
// answer is left to sample_kernel, which runs afterwards unless told that the token is decided.
constexpr int QUICK_KEYS = 4;

struct QuickTop {
    unsigned long long key[QUICK_KEYS]; // descending; 0 = none
    float mx, sum;                      // largest logit seen (-inf: none) and the sum of exp((logit - mx) * inv_t), roughly
    unsigned bad;                       // a logit that is not a number, or +inf: nothing here applies
};
__device__ __forceinline__ void quick_init(QuickTop &q) {
#pragma unroll
    for (int j = 0; j < QUICK_KEYS; j++) q.key[j] = 0;
    q.mx = -INFINITY;
    q.sum = 0.f;
    q.bad = 0;
}
__device__ __forceinline__ unsigned long long quick_key(half_t v, int index) {
    const unsigned hb = __builtin_bit_cast(unsigned short, v);
    const unsigned ord = (hb & 0x8000u) ? (~hb & 0xffffu) : (hb | 0x8000u);
    return ((unsigned long long)ord << 32) | (unsigned)~(unsigned)index;
}
__device__ __forceinline__ half_t quick_key_logit(unsigned long long key) {
    const unsigned ord = (unsigned)(key >> 32);
    const unsigned hb = (ord & 0x8000u) ? (ord & 0x7fffu) : (~ord & 0xffffu);
    return __builtin_bit_cast(half_t, (unsigned short)hb);
}
__device__ __forceinline__ void quick_insert(QuickTop &q, unsigned long long x) {
    if (x > q.key[QUICK_KEYS - 1]) {
        q.key[QUICK_KEYS - 1] = x;
#pragma unroll
        for (int j = QUICK_KEYS - 1; j > 0; j--) {
            const unsigned long long a = q.key[j - 1], b = q.key[j];
            q.key[j - 1] = a > b ? a : b;
            q.key[j] = a > b ? b : a;
        }
    }
}
// the rough sum: exp by the hardware, any order (top_k's result does not depend on it beyond what quick_top_k allows for)
__device__ __forceinline__ void quick_add_sum(QuickTop &q, float mx, float sum, float inv_t) {
    if (!(sum > 0.f)) return;
    if (mx > q.mx) {
        q.sum = q.sum * __expf((q.mx - mx) * inv_t) + sum; // (q.sum is 0 while q.mx is -inf: exp gives 0, not a NaN)
        q.mx = mx;
    } else
        q.sum += sum * __expf((mx - q.mx) * inv_t);
}
__device__ __forceinline__ void quick_add(QuickTop &q, half_t v, int index, float inv_t) {
    const unsigned hb = __builtin_bit_cast(unsigned short, v);
    if ((hb & 0x7c00u) == 0x7c00u && hb != 0xfc00u) q.bad = 1; // NaN or +inf
    quick_insert(q, quick_key(v, index));
    const float f = (float)v;
    if (f > -INFINITY) quick_add_sum(q, f, 1.f, inv_t);
}
__device__ __forceinline__ void quick_merge(QuickTop &q, const QuickTop &o, float inv_t) {
#pragma unroll
    for (int j = 0; j < QUICK_KEYS; j++) quick_insert(q, o.key[j]);
    quick_add_sum(q, o.mx, o.sum, inv_t);
    q.bad |= o.bad;
}

// top_k_sampling (sampling.zig:300-339) on the merged keys of the whole row, the way sample_kernel's quick evaluation does
// it: probabilities = exp * (1 / sum) with a sum that need not be the reference's bits (the factor cancels between
// r = u * total and the running sums up to the roundings), sequential running sums over the k largest, first candidate
// with r < running sum.  The answer stands only if
//   * neighbours among the k + 1 largest have the same logit (same exp, the lower index first in either order) or exps
//     more than 2^-20 apart in relative terms: then ordering by logit is ordering by probability, and no logit outside
//     the k reaches the k-th probability (expf is monotone to within an ulp or two);
//   * the k-th and the (k+1)-th differ: among equal probabilities at the edge the reference keeps the lower indices of ALL
//     that share the probability, which may include lower logits that this selection never looked at;
//   * r keeps (6 k + 32) 2^-24 of the total away from the running sums around the chosen candidate.
// Returns false otherwise (and for k + 1 > QUICK_KEYS, fewer than k + 1 logits, bad logits, all exps zero).
__device__ __forceinline__ bool quick_top_k(const QuickTop &q, int k, float temperature, float scale, float u, uint32_t *token) {
#pragma clang fp contract(off)
    if (k < 1 || k + 1 > QUICK_KEYS || q.bad || !(q.sum > 0.f)) return false;
    bool safe = true;
#pragma unroll
    for (int j = 0; j < QUICK_KEYS; j++)
        if (j <= k && q.key[j] == 0) safe = false;
    auto x_of = [&](float logit) { return temperature == 1.0f ? logit : scale != 0.f ? logit * scale : __fdiv_rn(logit, temperature); };
    const float mx = x_of((float)quick_key_logit(q.key[0]));
    float e[QUICK_KEYS];
#pragma unroll
    for (int j = 0; j < QUICK_KEYS; j++) {
        const float d = x_of((float)quick_key_logit(q.key[j])) - mx;
        e[j] = d > -88.0f ? sampling_expf(d) : 0.f; // ops.zig:1589-1590
    }
#pragma unroll
    for (int j = 0; j + 1 < QUICK_KEYS; j++) {
        const bool same_logit = (q.key[j] >> 32) == (q.key[j + 1] >> 32);
        if (j + 1 <= k && (same_logit ? j + 1 == k : !(e[j] - e[j + 1] > e[j] * 0x1p-20f))) safe = false;
    }
    const float inv = __fdiv_rn(1.0f, q.sum);
    float cum = 0.f, scan[QUICK_KEYS];
#pragma unroll
    for (int j = 0; j < QUICK_KEYS; j++) {
        cum += j < k ? e[j] * inv : 0.f;
        scan[j] = cum;
    }
    const float total = cum, r = u * total;
    int first = k - 1;
#pragma unroll
    for (int j = QUICK_KEYS - 1; j >= 0; j--)
        if (j < k && r < scan[j]) first = j;
    float below = 0.f, at = 0.f;
    unsigned long long chosen = 0;
#pragma unroll
    for (int j = 0; j < QUICK_KEYS; j++) {
        if (j == first - 1) below = scan[j];
        if (j == first) {
            at = scan[j];
            chosen = q.key[j];
        }
    }
    const float tol = (6.0f * (float)k + 32.0f) * 0x1p-24f * total;
    if (!(r - below > tol) || !(at - r > tol) || !(tol < 0.25f * total)) safe = false;
    *token = ~(uint32_t)chosen;
    return safe;
}

} // namespace
