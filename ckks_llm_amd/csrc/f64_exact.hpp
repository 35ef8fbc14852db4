// Exact integer arithmetic in IEEE doubles: the primitives that the FP64 transform back ends, the FP64 basis conversions, the
// fused key switch and the PPMM epilogue are built from, as functions that compile for the device and for the host.
//
// Every value these functions handle is an integer held in a double; the results are exact as long as every integer involved
// stays below 2^53 and the quotient estimate rint(a w / q) is close enough for h - c q to be representable.  The reference guards
// its modular arithmetic with range assertions that a compile-time switch turns on (uint128.cuh:19, 175-177, 209-211, 222-224);
// the counterpart here is the host build with CKKS_F64_RANGE_CHECK defined: every primitive then reports its operands and results
// to a checker (ckks::range, implemented by the host program that includes this header), which verifies them with 128-bit
// integers.  On the device and in ordinary host builds the hooks expand to nothing.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef uint64_t u64;

#define CKKS_HD __host__ __device__ __forceinline__

#if defined(CKKS_F64_RANGE_CHECK) && !defined(__HIP_DEVICE_COMPILE__)
namespace ckks {
namespace range {
// x is an integer below 2^53 in magnitude
void value(double x, const char* where);
// a, w integers below 2^53; h + l = a w exactly; c an integer; fma(-c, q, h) = h - c q exactly; r = that + l exactly, r = a w (mod q)
void mulmod(double a, double w, double q, double h, double l, double c, double r, const char* where);
// c an integer; r = x - c q exactly and within (q + 1) / 2 + slack of zero
void balance(double x, double q, double c, double r, const char* where);
// res = x mod q in [0, q)
void canonical(double x, double q, u64 res, const char* where);
// |x| < limit: the precondition of a bit-pattern conversion
void below(double x, double limit, const char* where);
}  // namespace range
}  // namespace ckks
#define CKKS_RANGE(call) ::ckks::range::call
#else
#define CKKS_RANGE(call) ((void)0)
#endif

namespace ckks {

CKKS_HD double f64_from_bits(u64 b) { return __builtin_bit_cast(double, b); }
CKKS_HD u64 f64_bits(double d) { return __builtin_bit_cast(u64, d); }

// integer x < 2^52 -> double: the word is the mantissa of 2^52 + x
CKKS_HD double exact_u2d(u64 x) { return f64_from_bits(0x4330000000000000ull | x) - 4503599627370496.0; }
// integer in [0, 2^52) held in a double -> the integer: the mantissa of 2^52 + r
CKKS_HD u64 bits52(double r) {
    CKKS_RANGE(below(r - 2251799813685248.0, 2251799813685248.5, "bits52: 0 <= r < 2^52"));
    return f64_bits(r + 4503599627370496.0) & 0xFFFFFFFFFFFFFull;
}
// a w mod q, within (0.5 + |a| 2^-52) q of zero (the quotient estimate is off by less than |a w| 2^-52 / q + 2^-53 |c|):
// h + l is the exact product, c q and h - c q are exact
CKKS_HD double mulmod_f64(double a, double w, double q, double qinv) {
    const double h = a * w;
    const double l = __builtin_fma(a, w, -h);
    const double c = __builtin_rint(h * qinv);
    const double r = __builtin_fma(-c, q, h) + l;
    CKKS_RANGE(mulmod(a, w, q, h, l, c, r, "mulmod_f64"));
    return r;
}
// x - rint(x / q) q: within (q + 1) / 2 of zero for |x| < 2^53
CKKS_HD double balance_f64(double x, double q, double qinv) {
    const double c = __builtin_rint(x * qinv);
    const double r = __builtin_fma(-c, q, x);
    CKKS_RANGE(balance(x, q, c, r, "balance_f64"));
    return r;
}
// any integer |r| < 2^52 -> its residue in [0, q), as a double
CKKS_HD double canon_f64(double x, double q, double qinv) {
    double r = balance_f64(x, q, qinv);
    r = r < 0.0 ? r + q : r;
    CKKS_RANGE(canonical(x, q, (u64)r, "canon_f64"));
    return r;
}

}  // namespace ckks

// ------------------------------------------------------------------------------------------------------------
// The per-coefficient sums of the exact RNS conversions (BasisConv.cuh:18-58) in this arithmetic, as the conversion kernels
// call them.  MAXS: compile-time bound of the source count (the loops are unrolled over it).
// ------------------------------------------------------------------------------------------------------------
namespace ckks {

// scaled source residue y_j = [x (D/d_j)^-1] mod d_j, canonical, for source primes below 2^41
CKKS_HD double conv_f64_scale(u64 xin, double hatinv, double d, double dinv) { return canon_f64(mulmod_f64(exact_u2d(xin), hatinv, d, dinv), d, dinv); }
// residue of sum_j y_j (D/d_j) - v D modulo a target prime below 2^41: |v| <= nsrc and |D mod r| <= r/2, every term within
// 0.51 r of zero
template <int MAXS>
CKKS_HD u64 conv_f64_target(const double (&y)[MAXS], int nsrc, const double* hat, double v, double dmod, double r, double rinv) {
    double acc = -v * dmod;
    CKKS_RANGE(value(acc, "conv_f64_target: v D"));
#pragma unroll
    for (int j = 0; j < MAXS; j++)
        if (j < nsrc) {
            acc += mulmod_f64(y[j], hat[j], r, rinv);
            CKKS_RANGE(value(acc, "conv_f64_target: running sum"));
        }
    return bits52(canon_f64(acc, r, rinv));
}
// Sources of any width, targets below 2^50: the scaled residue (an integer below 2^62 formed in integer arithmetic) enters as
// y = yh 2^31 + yl, each part with its own constant ((D/d_j) and (D/d_j) 2^31 mod r, balanced); every term lies within 0.51 r
// of zero and the running sum is balanced after every four sources.  Returns the canonical residue as a double.
CKKS_HD void conv_split_parts(u64 y, double& yl, double& yh) {
    yl = exact_u2d(y & 0x7fffffffull);
    yh = exact_u2d(y >> 31);
}
template <int MAXS>
CKKS_HD double conv_split_target(const double (&yl)[MAXS], const double (&yh)[MAXS], int nsrc, const double* hat, const double* hat31, double v,
                                 double dmod, double r, double rinv) {
    double acc = -mulmod_f64(v, dmod, r, rinv);
#pragma unroll
    for (int j = 0; j < MAXS; j++)
        if (j < nsrc) {
            acc += mulmod_f64(yl[j], hat[j], r, rinv) + mulmod_f64(yh[j], hat31[j], r, rinv);
            CKKS_RANGE(value(acc, "conv_split_target: running sum"));
            if ((j & 3) == 3) acc = balance_f64(acc, r, rinv);
        }
    return canon_f64(acc, r, rinv);
}

}  // namespace ckks

// ------------------------------------------------------------------------------------------------------------
// Recombination of the anti-diagonal sums of the digit-plane PPMM (PPMM_kernel.cuh:93-252 computes the same residues with 128-bit
// accumulation), one output at a time.  S[e] = sum over (d + j = e) and k of plaintext digit d times residue digit j: an int32
// with |S[e]| <= DW Kpad 2^14 (at most DW digit pairs per k on a diagonal, each product at most 2^14); the launcher admits
// DW Kpad <= 2^14, so |S[e]| <= 2^28 and every group y = S[4g] + 256 S[4g+1] + 2^16 S[4g+2] + 2^24 S[4g+3] is exact below 2^53.  The contraction kernel carries out exactly these operations in this order on four outputs
// at a time, interleaved; these functions are the per-output statement of it that the host range check drives.
//   c32, c64: 2^32 and 2^64 mod q, balanced;  qli: q_last^-1 mod q, balanced;  r_last: the last prime's residue of the same
//   output, used as an integer without reduction modulo q as in PPMM_kernel.cuh:243-247 (last = true: no rescale)
// ------------------------------------------------------------------------------------------------------------
namespace ckks {

template <int ND>
CKKS_HD u64 ppmm_recombine(const int (&S)[ND], double q, double qinv, double c32, double qli, bool last, u64 r_last) {
    static_assert(ND >= 5 && ND <= 8, "two groups of diagonals");
    double y0 = (double)S[3], y1 = (double)S[ND - 1];
    for (int e = 2; e >= 0; e--) { y0 = __builtin_fma(y0, 256.0, (double)S[e]); CKKS_RANGE(value(y0, "ppmm_recombine: y0")); }
    for (int e = ND - 2; e >= 4; e--) { y1 = __builtin_fma(y1, 256.0, (double)S[e]); CKKS_RANGE(value(y1, "ppmm_recombine: y1")); }
    // |y0 + (y1 2^32 mod q)| < 2^53 + 0.51 q: one exact addition, one reduction
    double t = y0 + mulmod_f64(y1, c32, q, qinv);
    CKKS_RANGE(value(t, "ppmm_recombine: y0 + y1 2^32"));
    t = balance_f64(t, q, qinv);
    if (!last) {
        t -= __builtin_fma((double)(unsigned)(r_last >> 32), 4294967296.0, (double)(unsigned)r_last);
        CKKS_RANGE(value(t, "ppmm_recombine: r_i - r_last"));
        t = mulmod_f64(t, qli, q, qinv);
    }
    const double res = t < 0.0 ? t + q : t;
    const u64 ures = f64_bits(res + 4503599627370496.0) & 0xFFFFFFFFFFull;
    CKKS_RANGE(below(res - 0.5 * q, 0.5 * q + 0.5, "ppmm_recombine: result in [0, q)"));
    return ures;
}
// q < 2^50: three groups; y0 and y1 are balanced first so that the products with 2^32 and 2^64 mod q keep their quotients below 2^49
template <int ND>
CKKS_HD u64 ppmm_recombine_wide(const int (&S)[ND], double q, double qinv, double c32, double c64, double qli, bool last, double r_last) {
    static_assert(ND >= 5, "at least two groups of diagonals");
    constexpr int E1 = ND - 1 < 7 ? ND - 1 : 7;
    double y0 = (double)S[3], y1 = (double)S[E1], y2 = ND > 8 ? (double)S[ND - 1] : 0.0;
    for (int e = 2; e >= 0; e--) { y0 = __builtin_fma(y0, 256.0, (double)S[e]); CKKS_RANGE(value(y0, "ppmm_recombine_wide: y0")); }
    for (int e = E1 - 1; e >= 4; e--) { y1 = __builtin_fma(y1, 256.0, (double)S[e]); CKKS_RANGE(value(y1, "ppmm_recombine_wide: y1")); }
    for (int e = ND - 2; e >= 8; e--) { y2 = __builtin_fma(y2, 256.0, (double)S[e]); CKKS_RANGE(value(y2, "ppmm_recombine_wide: y2")); }
    y0 = balance_f64(y0, q, qinv);
    y1 = balance_f64(y1, q, qinv);
    y1 = mulmod_f64(y1, c32, q, qinv);
    y2 = mulmod_f64(y2, c64, q, qinv);
    double t = y0 + y1 + y2;
    CKKS_RANGE(value(t, "ppmm_recombine_wide: sum of the groups"));
    t = balance_f64(t, q, qinv);
    if (!last) {
        t -= r_last;
        CKKS_RANGE(value(t, "ppmm_recombine_wide: r_i - r_last"));
        t = balance_f64(mulmod_f64(t, qli, q, qinv), q, qinv);
    }
    const double res = t < 0.0 ? t + q : t;
    return bits52(res);
}

}  // namespace ckks
