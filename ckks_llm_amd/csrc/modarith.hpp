// Device-side modular arithmetic for gfx950.
//
// Two arithmetic back ends share the NTT / conversion kernels:
//   * IntArith  - u64 lazy Harvey butterflies with Shoup multiplication, any odd prime q < 2^62.
//                 Same value ranges as the reference's CTBased_butterfly / GSBased_butterfly
//                 (ntt_60bit.cuh:293-318) and mulMod_shoup (uint128.cuh:169-179).
//   * F64Arith  - butterflies on IEEE doubles holding exact signed integers (CDNA4 issues FP64 FMA at
//                 full rate while 64-bit integer multiply-high costs about eight half-rate
//                 instructions).  Valid for q < 2^50; see ntt.hip for the range analysis.
// Outputs of every kernel are canonical residues in [0, q), so both back ends are bit-identical.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef uint64_t u64;
typedef unsigned __int128 u128;

namespace ckks {

// Conditional subtraction with the reference's exact semantics (uint128.cuh:143-147): the decision is the sign
// bit of a - q, so out-of-range inputs (a >= 2^63 + q) map the same way as in the reference.
__device__ __forceinline__ u64 csub(u64 a, u64 q) {
    u64 t = a - q;
    return t + (q & (u64)((long long)t >> 63));
}

// a * w mod q in [0, 2q) for any a < 2^64, w < q, ws = floor(w * 2^64 / q)
__device__ __forceinline__ u64 mul_shoup_lazy(u64 a, u64 w, u64 ws, u64 q) {
    return a * w - __umul64hi(a, ws) * q;
}
// canonical result; uint128.cuh:169-179
__device__ __forceinline__ u64 mul_shoup(u64 a, u64 w, u64 ws, u64 q) {
    return csub(mul_shoup_lazy(a, w, ws, q), q);
}

struct u128w {
    u64 lo, hi;
};
__device__ __forceinline__ void mac128(u128w& acc, u64 a, u64 b) {   // acc += a*b (mod 2^128), uint128.cuh:297-307
    u64 lo = a * b, hi = __umul64hi(a, b);
    acc.lo += lo;
    acc.hi += hi + (acc.lo < lo);
}
__device__ __forceinline__ void sub128_64(u128w& acc, u64 b) {        // uint128.cuh:273-283
    u64 lo = acc.lo - b;
    acc.hi -= (acc.lo < b);
    acc.lo = lo;
}
// 128 -> 64 bit Barrett with mu = floor(2^128/q) = (mu_hi, mu_lo); same quotient estimate as
// singleBarrett_new (uint128.cuh:182-212): the low word of a.lo*mu.lo is dropped.
__device__ __forceinline__ u64 barrett128(u128w a, u64 q, u64 mu_hi, u64 mu_lo) {
    u64 tmp = __umul64hi(a.lo, mu_lo);
    u64 p_lo = a.lo * mu_hi, p_hi = __umul64hi(a.lo, mu_hi);
    u64 t2 = p_lo + tmp;
    u64 res = p_hi + (t2 < p_lo);
    u64 r_lo = a.hi * mu_lo, r_hi = __umul64hi(a.hi, mu_lo);
    u64 t3 = r_lo + t2;
    res += r_hi + (t3 < r_lo);
    res += a.hi * mu_hi;
    u64 r = a.lo - res * q;
    return csub(r, q);
}
// uint128.cuh:214-225
__device__ __forceinline__ u64 barrett64(u64 a, u64 q, u64 mu_hi) {
    u64 s = __umul64hi(mu_hi, a);
    return csub(a - s * q, q);
}
__device__ __forceinline__ u64 negate_mod(u64 a, u64 q) { return a == 0 ? 0 : q - a; }   // uint128.cuh:309-313

}  // namespace ckks
