// Host-side exact integer helpers used to build the context's constant tables.
// Product code: independent of the test oracle (different algorithms where the mathematics allows it:
// extended Euclid for inverses, power tables in natural order scattered by bit reversal).
#pragma once
#include <stdint.h>
#include <cmath>
#include <vector>

namespace ckks_host {

typedef uint64_t u64;
typedef unsigned __int128 u128;

inline u64 mulmod(u64 a, u64 b, u64 m) { return (u64)(((u128)a * b) % m); }
inline u64 addmod(u64 a, u64 b, u64 m) { u64 s = a + b; return (s >= m || s < a) ? s - m : s; }
inline u64 powmod(u64 a, u64 e, u64 m) {
    u64 r = 1 % m;
    a %= m;
    for (; e; e >>= 1, a = mulmod(a, a, m))
        if (e & 1) r = mulmod(r, a, m);
    return r;
}
// modular inverse by the extended Euclidean algorithm (gcd(a, m) must be 1)
inline u64 invmod(u64 a, u64 m) {
    __int128 r0 = m, r1 = a % m, s0 = 0, s1 = 1;
    while (r1 != 0) {
        __int128 qq = r0 / r1, t = r0 - qq * r1;
        r0 = r1; r1 = t;
        t = s0 - qq * s1; s0 = s1; s1 = t;
    }
    if (s0 < 0) s0 += m;
    return (u64)s0;
}
// floor(x * 2^64 / m): companion word of Shoup's multiplication (Utils.cuh:40-45)
inline u64 shoup(u64 x, u64 m) { return (u64)((((u128)x) << 64) / m); }
// floor(2^128 / m) for odd m (Context_23.cuh:67-70)
inline void barrett_mu(u64 m, u64& hi, u64& lo) {
    u128 mu = (~(u128)0) / m;
    hi = (u64)(mu >> 64);
    lo = (u64)mu;
}
inline uint32_t bitrev(uint32_t x, int bits) {
    x = ((x & 0xaaaaaaaau) >> 1) | ((x & 0x55555555u) << 1);
    x = ((x & 0xccccccccu) >> 2) | ((x & 0x33333333u) << 2);
    x = ((x & 0xf0f0f0f0u) >> 4) | ((x & 0x0f0f0f0fu) << 4);
    x = ((x & 0xff00ff00u) >> 8) | ((x & 0x00ff00ffu) << 8);
    x = (x >> 16) | (x << 16);
    return bits ? x >> (32 - bits) : 0;
}

// Generator choice of the reference (Utils.cuh:63-96).  The 2N-th root psi = g^((q-1)/2N) fixes the VALUES of a
// transform, so the rule has to be followed to the letter, including its trial-division bound
// (i < sqrt(n) on the shrinking cofactor, compared in double) that can leave a prime square as one "factor".
inline u64 reference_generator(u64 q) {
    std::vector<u64> fac;
    u64 n = q - 1;
    if (n % 2 == 0) fac.push_back(2);
    while (n % 2 == 0) n /= 2;
    for (u64 i = 3; (double)i < std::sqrt((double)n); i++) {
        if (n % i == 0) fac.push_back(i);
        while (n % i == 0) n /= i;
    }
    if (n > 2) fac.push_back(n);
    for (u64 r = 2; r < q; r++) {
        bool ok = true;
        for (u64 f : fac)
            if (powmod(r, (q - 1) / f, q) == 1) { ok = false; break; }
        if (ok) return r;
    }
    return 0;
}
// psi with psi^M = 1 of exact order M (Utils.cuh:98-109); 0 if M does not divide q-1
inline u64 mth_root(u64 M, u64 q) {
    if ((q - 1) % M) return 0;
    return powmod(reference_generator(q), (q - 1) / M, q);
}
// product of v[lo..hi) modulo m, leaving out index `skip` (-1: none)
inline u64 prod_mod(const std::vector<u64>& v, int lo, int hi, int skip, u64 m) {
    u64 r = 1 % m;
    for (int i = lo; i < hi; i++)
        if (i != skip) r = mulmod(r, v[i] % m, m);
    return r;
}

}  // namespace ckks_host
