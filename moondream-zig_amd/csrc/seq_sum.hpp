// The arithmetic behind the sampler's bit-exact sequential sums (sample.hip: seq_prefix), kept free of device-only calls so
// that a host program can check it against a plain float loop (tests/cxx/seq_sum_check.cpp).
//
// A sequential f32 sum  s = 0; for i: s += w_i  over non-negative terms: while s stays inside one binade [2^b, 2^(b+1)) it is
// an integer S in [2^23, 2^24) times ulp = 2^(b-23), and adding w rounds S + w / ulp to an integer: S + E when the fraction
// of w / ulp is below a half, S + E + 1 when above, and to the even one of the two on a tie.  So every term is a map
// S -> S + c[S & 1] with two small integers c[0], c[1]; such maps compose associatively (the parity after the first map
// picks the second map's entry).  A map says nothing once S would reach 2^24 (s leaves the binade, the ulp changes) or a
// term is not smaller than the binade itself: its entries are then >= SEQ_BIG.
#pragma once

#if defined(__HIPCC__)
#define SEQ_FN __host__ __device__ __forceinline__
#else
#define SEQ_FN inline
#endif

namespace {

struct SeqMap {
    unsigned c0, c1;
};
constexpr unsigned SEQ_BIG = 1u << 24, SEQ_CAP = 1u << 26;
SEQ_FN unsigned seq_min_u(unsigned a, unsigned b) { return a < b ? a : b; }
SEQ_FN SeqMap seq_compose(SeqMap a, SeqMap b) { // a first, then b
    SeqMap r;
    r.c0 = seq_min_u(a.c0 + ((a.c0 & 1u) ? b.c1 : b.c0), SEQ_CAP);
    r.c1 = seq_min_u(a.c1 + (((1u + a.c1) & 1u) ? b.c1 : b.c0), SEQ_CAP);
    return r;
}
// sb: biased exponent of the running sum, 0 when the sum is zero or below the second normal binade (then every non-zero
// term ends the phase).  Branch-free: this runs for every term in every phase.
SEQ_FN SeqMap seq_elem(float w, int sb) {
    const unsigned bits = __builtin_bit_cast(unsigned, w);
    const unsigned ebf = (bits >> 23) & 255u;
    const unsigned em = (bits & 0x7fffffu) | (ebf ? 0x800000u : 0u); // subnormal: no implicit bit, exponent as for 1
    const int k = sb - (int)(ebf ? ebf : 1u);                        // w / ulp = em / 2^k
    const unsigned kc = (unsigned)(k < 1 ? 1 : k > 25 ? 25 : k);
    const unsigned E = em >> kc, frac = em & ((1u << kc) - 1u), half = 1u << (kc - 1u); // em < 2^24: E is 0 from k = 24 on
    const unsigned up = frac > half ? 1u : 0u, tie = frac == half ? 1u : 0u;
    SeqMap m{E + up + (tie & E), E + up + (tie & ~E)}; // tie: to the even neighbour, which depends on the parity of S + E
    const bool zero = (bits << 1) == 0u;
    const bool big = !zero && (sb == 0 || k <= 0); // no binade to count in, or a term not smaller than the binade itself
    m.c0 = zero ? 0u : big ? SEQ_BIG : m.c0;
    m.c1 = zero ? 0u : big ? SEQ_BIG : m.c1;
    return m;
}

} // namespace
