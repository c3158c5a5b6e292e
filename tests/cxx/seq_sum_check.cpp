// Host check of the map arithmetic behind the sampler's sequential sums (moondream-zig_amd/csrc/seq_sum.hpp) against the
// plain loop  s += w  in IEEE binary32: for a start sum s0 in a normal binade and a list of non-negative terms, the
// composition of the terms' maps applied to s0's integer mantissa either gives the loop's result bit for bit, or says
// (entry >= SEQ_BIG) that the sum leaves the binade somewhere in the list, in which case the loop must indeed have left
// it or met a term as large as the binade.  Term lists: random magnitudes around every distance from the ulp, exact ties
// at half an ulp on both parities, terms of one ulp, subnormals, zeros, terms that are the binade itself, and long runs of
// tiny terms that are rounded away one by one (the case a tree sum gets wrong).  Associativity of the composition is
// checked by composing the same list in random groupings.
#include "seq_sum.hpp"

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <random>
#include <vector>

static float from_bits(uint32_t b) {
    float f;
    std::memcpy(&f, &b, 4);
    return f;
}
static uint32_t bits_of(float f) {
    uint32_t b;
    std::memcpy(&b, &f, 4);
    return b;
}

static int failures = 0;
static long checked = 0, left_binade = 0;

// one list against the loop; returns false on a mismatch
static bool check_list(float s0, const std::vector<float> &w, std::mt19937_64 &rng) {
    const uint32_t sbits = bits_of(s0);
    int sb = (int)((sbits >> 23) & 255u);
    if (sb <= 1) sb = 0;
    const uint32_t S0 = sb ? ((sbits & 0x7fffffu) | 0x800000u) : 0u;
    // left fold
    SeqMap m{0u, 0u};
    for (float x : w) m = seq_compose(m, seq_elem(x, sb));
    // a random grouping of the same list: ((..)(..))(..) must give the same map while it stays below the cap
    SeqMap g{0u, 0u};
    for (size_t i = 0; i < w.size();) {
        size_t len = 1 + rng() % 7;
        SeqMap part{0u, 0u};
        for (size_t j = i; j < i + len && j < w.size(); j++) part = seq_compose(part, seq_elem(w[j], sb));
        g = seq_compose(g, part);
        i += len;
    }
    const uint32_t end = S0 + ((S0 & 1u) ? m.c1 : m.c0), end_g = S0 + ((S0 & 1u) ? g.c1 : g.c0);
    // the loop, with the first index at which it leaves the binade (or meets a term not below the binade)
    volatile float s = s0;
    bool left = false;
    for (float x : w) {
        if (x != 0.f && (sb == 0 || bits_of(x) >= ((uint32_t)sb << 23))) left = true;
        s = s + x;
        if ((int)((bits_of(s) >> 23) & 255u) != sb) left = true;
    }
    checked++;
    if (end < SEQ_BIG) {
        const float predicted = sb ? from_bits(((uint32_t)sb << 23) | (end & 0x7fffffu)) : s0;
        if (left || bits_of(predicted) != bits_of(s) || end_g != end) {
            if (failures < 10)
                std::printf("MISMATCH s0=%a n=%zu loop=%a predicted=%a left=%d end=%u grouped=%u\n", (double)s0, w.size(), (double)s, (double)predicted,
                            (int)left, end, end_g);
            failures++;
            return false;
        }
    } else {
        left_binade++;
        if (!left || end_g < SEQ_BIG) { // the maps gave up although the loop stayed inside, or the grouping disagrees
            if (failures < 10) std::printf("SPURIOUS s0=%a n=%zu loop=%a end=%u grouped=%u\n", (double)s0, w.size(), (double)s, end, end_g);
            failures++;
            return false;
        }
    }
    return true;
}

int main() {
    std::mt19937_64 rng(12345);
    auto uniform = [&](double a, double b) { return a + (b - a) * (double)(rng() >> 11) / 9007199254740992.0; };
    for (int round = 0; round < 20000; round++) {
        // a start sum in a random normal binade (exponents 2 .. 200), random mantissa, both parities
        const int sb = 2 + (int)(rng() % 199);
        const uint32_t mant = (uint32_t)(rng() & 0x7fffffu);
        const float s0 = from_bits(((uint32_t)sb << 23) | mant);
        const float ulp = std::ldexp(1.0f, sb - 127 - 23);
        std::vector<float> w;
        const int kind = round % 8, n = 1 + (int)(rng() % 300);
        for (int i = 0; i < n; i++) {
            float x = 0.f;
            switch (kind) {
            case 0: x = (float)(uniform(0, 4) * ulp); break;                                     // around the ulp
            case 1: x = (float)std::ldexp(uniform(0.5, 1.0), sb - 127 - (int)(rng() % 40)); break; // every distance below the binade
            case 2: x = (rng() & 1) ? 0.5f * ulp : 1.5f * ulp; break;                             // exact ties
            case 3: x = (rng() % 3 == 0) ? 0.f : ulp * (float)(rng() % 5); break;                 // zeros and whole ulps
            case 4: x = (float)(uniform(0, 0.499) * ulp); break;                                  // all rounded away, one by one
            case 5: x = from_bits((uint32_t)(rng() % 0x00800000u)); break;                         // subnormals
            case 6: x = (i == n / 2) ? std::ldexp(1.0f, sb - 127) : (float)(uniform(0, 2) * ulp); break; // one term as large as the binade
            default: x = (float)(uniform(0.4999, 0.5001) * ulp * (double)(1 + rng() % 3)); break; // next to the ties
            }
            w.push_back(x);
        }
        check_list(s0, w, rng);
    }
    // sums that start from zero or from below the normal range: every non-zero term ends the phase
    for (int round = 0; round < 200; round++) {
        std::vector<float> w{0.f, 0.f, from_bits((uint32_t)(1 + rng() % 1000)), 1.0f};
        check_list(round % 2 ? 0.f : from_bits((uint32_t)(rng() % 0x00800000u)), w, rng);
    }
    std::printf("%ld lists checked, %ld of them leave the binade, %d failures\n", checked, left_binade, failures);
    return failures ? 1 : 0;
}
