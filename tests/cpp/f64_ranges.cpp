// Host build of the library's exact-integer FP64 arithmetic with its range hooks switched on (CKKS_F64_RANGE_CHECK): whole
// forward and inverse transforms, the conversion sums, a ModDown sum and the PPMM recombination run here on the CPU through the
// very functions the kernels compile (ckks_llm_amd/csrc/f64_exact.hpp, ntt_core.hpp), and every operand and result passes
// through the checker below, which redoes the step in 128-bit integers.  The counterpart of the reference's in-kernel range
// assertions (uint128.cuh:19, 175-177, 209-211, 222-224).  Built by tests/cpp/Makefile with hipcc in host-only mode (no GPU
// code is generated or run), optionally under AddressSanitizer and UBSan; driven by tests/test_f64_ranges.py through ctypes.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "../../ckks_llm_amd/csrc/ntt_core.hpp"

typedef __int128 i128;

namespace {
struct Stats {
    long checks = 0, violations = 0;
    double max_abs = 0.0;            // largest |integer| seen
    double max_ratio = 0.0;          // largest |mulmod result| / q
    double max_balance_ratio = 0.0;  // largest |balance result| / q
    char first[256] = {0};
} g;

void fail(const char* where, const char* what, double a, double b) {
    if (g.violations++ == 0) snprintf(g.first, sizeof g.first, "%s: %s (%.17g, %.17g)", where, what, a, b);
}
bool is_int53(double x) { return std::fabs(x) < 9007199254740992.0 && x == std::nearbyint(x); }
i128 as_int(double x) { return (i128)x; }       // exact for integer-valued doubles below 2^127
i128 iabs(i128 x) { return x < 0 ? -x : x; }
}  // namespace

namespace ckks {
namespace range {
void value(double x, const char* where) {
    g.checks++;
    if (!is_int53(x)) fail(where, "not an integer below 2^53", x, 0);
    g.max_abs = std::fmax(g.max_abs, std::fabs(x));
}
void mulmod(double a, double w, double q, double h, double l, double c, double r, const char* where) {
    g.checks++;
    if (!is_int53(a) || !is_int53(w)) { fail(where, "operand not an integer below 2^53", a, w); return; }
    g.max_abs = std::fmax(g.max_abs, std::fmax(std::fabs(a), std::fabs(w)));
    const i128 P = as_int(a) * as_int(w);
    if (h != std::nearbyint(h) || l != std::nearbyint(l) || as_int(h) + as_int(l) != P) { fail(where, "h + l is not the exact product", h, l); return; }
    if (c != std::nearbyint(c)) { fail(where, "quotient estimate is not an integer", c, 0); return; }
    const i128 T = as_int(h) - as_int(c) * as_int(q);
    if (iabs(T) >= ((i128)1 << 53)) { fail(where, "h - c q does not fit 53 bits", (double)T, c); return; }
    if (__builtin_fma(-c, q, h) != (double)T) { fail(where, "fma(-c, q, h) is not h - c q", (double)T, __builtin_fma(-c, q, h)); return; }
    const i128 R = T + as_int(l);
    if (iabs(R) >= ((i128)1 << 53) || (double)R != r) { fail(where, "result is not (h - c q) + l", (double)R, r); return; }
    if ((P - R) % as_int(q) != 0) { fail(where, "result is not congruent to the product", r, q); return; }
    g.max_ratio = std::fmax(g.max_ratio, std::fabs(r) / q);
    if (std::fabs(r) >= q) fail(where, "result not within q of zero", r, q);
}
void balance(double x, double q, double c, double r, const char* where) {
    g.checks++;
    if (!is_int53(x)) { fail(where, "operand not an integer below 2^53", x, 0); return; }
    g.max_abs = std::fmax(g.max_abs, std::fabs(x));
    if (c != std::nearbyint(c)) { fail(where, "quotient estimate is not an integer", c, 0); return; }
    const i128 R = as_int(x) - as_int(c) * as_int(q);
    if ((double)R != r || iabs(R) >= ((i128)1 << 53)) { fail(where, "result is not x - c q", (double)R, r); return; }
    g.max_balance_ratio = std::fmax(g.max_balance_ratio, std::fabs(r) / q);
    // within (q + 1) / 2 of zero, plus what the rounding of x (1/q) (relative error below 2^-52) can move the estimate across a half
    if (2 * iabs(R) > as_int(q) + 1 + (i128)std::ceil(std::fabs(x) * 4.440892098500626e-16)) fail(where, "result not within (q + 1) / 2 + |x| 2^-52 of zero", r, q);
}
void canonical(double x, double q, u64 res, const char* where) {
    g.checks++;
    if (!is_int53(x)) { fail(where, "operand not an integer below 2^53", x, 0); return; }
    i128 m = as_int(x) % as_int(q);
    if (m < 0) m += as_int(q);
    if ((i128)res != m) fail(where, "not the residue in [0, q)", x, (double)res);
}
void below(double x, double limit, const char* where) {
    g.checks++;
    if (!(std::fabs(x) < limit)) fail(where, "precondition of a bit-pattern conversion", x, limit);
}
}  // namespace range
}  // namespace ckks

using namespace ckks;

namespace {
double balanced_double(u64 x, u64 q) { return x > q / 2 ? -(double)(q - x) : (double)x; }      // as the context builds its FP64 tables

PrimeConst prime_const(u64 q, u64 n_inv, u64 w1n) {
    PrimeConst p;
    memset(&p, 0, sizeof p);
    p.q = q; p.n_inv = n_inv; p.w1n = w1n;
    p.qd = (double)q; p.qinv_d = 1.0 / (double)q;
    p.n_inv_d = balanced_double(n_inv, q); p.w1n_d = balanced_double(w1n, q);
    return p;
}

// What lies between the two passes of a transform: 0 the values as the pass leaves them (8-byte words in place), 1 the 40-bit
// form, 2 the 36-bit form of the resident transform
template <class AR>
double through_mid_fwd(const AR& ar, double x, int form) {
    if (form == 1) {
        const u64 e = ar.lazy40 ? ar.enc40_raw(x) : ar.enc40(x);
        return ar.dec40((unsigned)e, (unsigned)(e >> 32));
    }
    if (form == 2) {
        const u64 e = ar.enc36(x);
        return ar.dec36((unsigned)e, (unsigned)(e >> 32));
    }
    return ar.from_mid(ar.to_mid_fwd(x));
}
template <class AR>
double through_mid_inv(const AR& ar, double x, int form) {
    if (form == 1) {
        const u64 e = ar.enc40(x);
        return ar.dec40((unsigned)e, (unsigned)(e >> 32));
    }
    if (form == 2) {
        const u64 e = ar.enc36(x);
        return ar.dec36((unsigned)e, (unsigned)(e >> 32));
    }
    return ar.from_mid(ar.to_mid_inv(x));
}

// One limb through both passes, with the tile shapes, register rounds and exchange points of strided_tile and row_tile
// (ntt.hip): N = N1 N2 row-major, strided pass on columns (twiddle offset 1), row pass on rows (offset N1 + row).
template <class AR, int SA, int SB>
void transform(const AR& ar, const double* tw, u64* data, bool inverse, int form) {
    typedef StridedCfg<SA, SB> CS;
    typedef RowCfg<SA, SB> CR;
    constexpr int N1 = 1 << SA, N2 = 1 << SB;
    std::vector<double> mid((size_t)N1 * N2);
    auto strided_fwd = [&]() {
        constexpr int S1 = CS::S1, R = CS::R, G = CS::G;
        std::vector<double> col(N1);
        for (int c = 0; c < N2; c++) {
            for (int g = 0; g < G; g++) {
                double v[R];
                for (int j = 0; j < R; j++) v[j] = ar.from_canonical(data[(size_t)(g + j * G) * N2 + c]);
                fwd_spread<AR, SA, S1>(v, tw, 1u, ar);
                ar.round_end(v);
                for (int j = 0; j < R; j++) col[g + j * G] = v[j];
            }
            for (int g = 0; g < G; g++) {
                double v[R];
                for (int j = 0; j < R; j++) v[j] = col[g * R + j];
                fwd_packed<AR, SA, S1>(v, tw, 1u, (unsigned)g, ar);
                for (int j = 0; j < R; j++) mid[(size_t)(g * R + j) * N2 + c] = through_mid_fwd(ar, v[j], form);
            }
        }
    };
    auto row_fwd = [&]() {
        constexpr int S1 = CR::S1, R = CR::R, U = CR::U;
        std::vector<double> row(N2);
        for (int r = 0; r < N1; r++) {
            const unsigned tw_off = (unsigned)(N1 + r);
            for (int u = 0; u < U; u++) {
                double v[R];
                for (int j = 0; j < R; j++) v[j] = mid[(size_t)r * N2 + u + j * U];
                fwd_spread<AR, SB, S1>(v, tw, tw_off, ar);
                ar.round_end(v);
                for (int j = 0; j < R; j++) row[u + j * U] = v[j];
            }
            for (int u = 0; u < U; u++) {
                double v[R];
                for (int j = 0; j < R; j++) v[j] = row[u * R + j];
                fwd_packed<AR, SB, S1>(v, tw, tw_off, (unsigned)u, ar);
                for (int j = 0; j < R; j++) data[(size_t)r * N2 + u * R + j] = ar.to_canonical_fwd(v[j]);
            }
        }
    };
    auto row_inv = [&]() {
        constexpr int S1 = CR::S1, R = CR::R, U = CR::U;
        std::vector<double> row(N2);
        for (int r = 0; r < N1; r++) {
            const unsigned tw_off = (unsigned)(N1 + r);
            for (int u = 0; u < U; u++) {
                double v[R];
                for (int j = 0; j < R; j++) v[j] = ar.from_canonical(data[(size_t)r * N2 + u * R + j]);
                inv_packed<AR, SB, S1>(v, tw, tw_off, (unsigned)u, ar);
                ar.round_end(v);
                for (int j = 0; j < R; j++) row[u * R + j] = v[j];
            }
            for (int u = 0; u < U; u++) {
                double v[R];
                for (int j = 0; j < R; j++) v[j] = row[u + j * U];
                inv_spread<AR, SB, S1, 0>(v, tw, tw_off, ar);
                for (int j = 0; j < R; j++) mid[(size_t)r * N2 + u + j * U] = through_mid_inv(ar, v[j], form);
            }
        }
    };
    auto strided_inv = [&]() {
        constexpr int S1 = CS::S1, R = CS::R, G = CS::G;
        std::vector<double> col(N1);
        for (int c = 0; c < N2; c++) {
            for (int g = 0; g < G; g++) {
                double v[R];
                for (int j = 0; j < R; j++) v[j] = mid[(size_t)(g * R + j) * N2 + c];
                inv_packed<AR, SA, S1>(v, tw, 1u, (unsigned)g, ar);
                ar.round_end(v);
                for (int j = 0; j < R; j++) col[g * R + j] = v[j];
            }
            for (int g = 0; g < G; g++) {
                double v[R];
                for (int j = 0; j < R; j++) v[j] = col[g + j * G];
                inv_spread<AR, SA, S1, 1>(v, tw, 1u, ar);
                for (int j = 0; j < R / 2; j++) {
                    u64 ox, oy;
                    ar.gs_last(v[j], v[j + R / 2], ox, oy);
                    data[(size_t)(g + j * G) * N2 + c] = ox;
                    data[(size_t)(g + (j + R / 2) * G) * N2 + c] = oy;
                }
            }
        }
    };
    if (!inverse) { strided_fwd(); row_fwd(); }
    else { row_inv(); strided_inv(); }
}

template <class AR>
int transform_logn(const AR& ar, const double* tw, u64* data, int logN, bool inverse, int form) {
    switch (logN) {
        case 8: transform<AR, 4, 4>(ar, tw, data, inverse, form); return 0;
        case 10: transform<AR, 5, 5>(ar, tw, data, inverse, form); return 0;
        case 12: transform<AR, 6, 6>(ar, tw, data, inverse, form); return 0;
        case 13: transform<AR, 7, 6>(ar, tw, data, inverse, form); return 0;
        case 16: transform<AR, 8, 8>(ar, tw, data, inverse, form); return 0;
        default: return 1;
    }
}
}  // namespace

extern "C" {

void f64r_reset() { g = Stats(); }
// out: checks, violations; dout: max |integer|, max |mulmod result| / q, max |balance result| / q
void f64r_stats(long* out, double* dout, char* first, int first_cap) {
    out[0] = g.checks; out[1] = g.violations;
    dout[0] = g.max_abs; dout[1] = g.max_ratio; dout[2] = g.max_balance_ratio;
    if (first && first_cap > 0) { strncpy(first, g.first, (size_t)first_cap - 1); first[first_cap - 1] = 0; }
}

// One limb of N = 2^logN words, in place.  table: the forward (psi_table) or inverse (psiinv_table) twiddles of the prime as the
// context holds them, canonical; n_inv = N^-1 mod q.  wide: the back end for primes up to 2^50.  form: see through_mid_fwd.
int f64r_ntt(int wide, int form, uint64_t q, const uint64_t* table, uint64_t n_inv, uint64_t* data, int logN, int inverse) {
    const long N = 1l << logN;
    std::vector<double> tw((size_t)N);
    for (long k = 0; k < N; k++) tw[(size_t)k] = balanced_double(table[k], q);
    const PrimeConst pc = prime_const(q, n_inv, table[1]);
    if (wide) return transform_logn(F64WideArith(pc), tw.data(), data, logN, inverse != 0, form);
    return transform_logn(F64Arith(pc), tw.data(), data, logN, inverse != 0, form);
}

// Exact conversion of `count` coefficients from nsrc source primes to ntgt target primes, all below 2^41 (conv_kernel_f64):
// in [nsrc][count], out [ntgt][count]; hatinv[j] = (D/d_j)^-1 mod d_j, hat[k][j] = (D/d_j) mod r_k, dmod[k] = D mod r_k.
int f64r_conv(int nsrc, int ntgt, const uint64_t* d, const uint64_t* r, const uint64_t* hatinv, const uint64_t* hat, const uint64_t* dmod,
              const uint64_t* in, uint64_t* out, long count) {
    if (nsrc > 16 || nsrc < 1) return 1;
    for (long x = 0; x < count; x++) {
        double y[16], vv = 0.0;
        for (int j = 0; j < 16; j++) {
            y[j] = 0.0;
            if (j < nsrc) {
                y[j] = conv_f64_scale(in[(long)j * count + x], balanced_double(hatinv[j], d[j]), (double)d[j], 1.0 / (double)d[j]);
                vv += y[j] / (double)d[j];
            }
        }
        const double v = (double)(int)vv;
        for (int k = 0; k < ntgt; k++) {
            double hat_d[16];
            for (int j = 0; j < nsrc; j++) hat_d[j] = balanced_double(hat[(long)k * nsrc + j], r[k]);
            out[(long)k * count + x] = conv_f64_target<16>(y, nsrc, hat_d, v, balanced_double(dmod[k], r[k]), (double)r[k], 1.0 / (double)r[k]);
        }
    }
    return 0;
}
// Sources of any width (scaled in integers: y[j][x] are the scaled residues), targets below 2^50 (conv_kernel_split);
// hat31[k][j] = (D/d_j) 2^31 mod r_k.
int f64r_conv_split(int nsrc, int ntgt, const uint64_t* d, const uint64_t* r, const uint64_t* hat, const uint64_t* hat31, const uint64_t* dmod,
                    const uint64_t* y, uint64_t* out, long count) {
    if (nsrc > 16 || nsrc < 1) return 1;
    for (long x = 0; x < count; x++) {
        double yl[16], yh[16], vv = 0.0;
        for (int j = 0; j < 16; j++) {
            yl[j] = yh[j] = 0.0;
            if (j < nsrc) {
                const u64 w = y[(long)j * count + x];
                vv += (double)w / (double)d[j];
                conv_split_parts(w, yl[j], yh[j]);
            }
        }
        const double v = (double)(int)vv;
        for (int k = 0; k < ntgt; k++) {
            double hat_d[16], hat31_d[16];
            for (int j = 0; j < nsrc; j++) {
                hat_d[j] = balanced_double(hat[(long)k * nsrc + j], r[k]);
                hat31_d[j] = balanced_double(hat31[(long)k * nsrc + j], r[k]);
            }
            out[(long)k * count + x] = bits52(conv_split_target<16>(yl, yh, nsrc, hat_d, hat31_d, v, balanced_double(dmod[k], r[k]), (double)r[k], 1.0 / (double)r[k]));
        }
    }
    return 0;
}

// ModDown of the fused key switch (BasisConv.cuh:257-326; ks_moddown_strided_kernel / ks_back_kernel with pre-scaled special-prime
// coefficients): out = (own - sum_i x_i pHat_i) P^-1 mod q for `count` coefficients; x [K][count] residues of the special primes
// p_i (which may exceed q), own [count] residues modulo q.
int f64r_moddown(int wide, uint64_t q, int K, const uint64_t* x, const uint64_t* phat, uint64_t pinv, const uint64_t* own, uint64_t* out, long count) {
    const PrimeConst pc = prime_const(q, 1, 1);
    bool failed = false;
    auto run = [&](const auto& ar) {
        for (long n = 0; n < count; n++) {
            double acc = 0.0;
            for (int i = 0; i < K; i++) {
                if (K == 1) acc = exact_u2d(x[n]);
                else acc += ar.mulmod(exact_u2d(x[(long)i * count + n]), wide ? balanced_double(phat[i], q) : exact_u2d(phat[i]));
                range::value(acc, "moddown: running sum");
            }
            const double t = ar.q - canon_f64(acc, ar.q, ar.qinv) + exact_u2d(own[n]);
            range::value(t, "moddown: own - sum");
            const double v = ar.mulmod(t, wide ? balanced_double(pinv, q) : exact_u2d(pinv));
            out[n] = wide ? F64WideArith(pc).canon_wide(v) : ar.canon_any(v);
            // the form of the key switch's last launch: the sum starts from minus the own coefficient
            double acc2 = -exact_u2d(own[n]);
            for (int i = 0; i < K; i++) {
                if (K == 1) acc2 += exact_u2d(x[n]);
                else acc2 += ar.mulmod(exact_u2d(x[(long)i * count + n]), wide ? balanced_double(phat[i], q) : exact_u2d(phat[i]));
                range::value(acc2, "moddown: running sum from -own");
            }
            const double v2 = ar.mulmod(ar.q - canon_f64(acc2, ar.q, ar.qinv), wide ? balanced_double(pinv, q) : exact_u2d(pinv));
            const uint64_t out2 = wide ? F64WideArith(pc).canon_wide(v2) : ar.canon_any(v2);
            if (out2 != out[n]) { failed = true; return; }
        }
    };
    if (wide) run(F64WideArith(pc));
    else run(F64Arith(pc));
    return failed ? 2 : 0;
}

// Recombination of the digit-plane PPMM: S [count][ND] anti-diagonal sums, r_last [count] residues of the last prime (ignored when
// last != 0); c32 = 2^32 mod q, c64 = 2^64 mod q, qli = q_last^-1 mod q (canonical here, balanced inside as the launcher does).
int f64r_ppmm(int wide, int ND, uint64_t q, uint64_t c32, uint64_t c64, uint64_t qli, int last, const int* S, const uint64_t* r_last, uint64_t* out, long count) {
    const double qd = (double)q, qinv = 1.0 / qd, c32d = balanced_double(c32, q), c64d = balanced_double(c64, q), qlid = balanced_double(qli, q);
    for (long n = 0; n < count; n++) {
        const int* s = S + n * ND;
        const u64 rl = last ? 0 : r_last[n];
#define NARROW(D) case D: { int t[D]; memcpy(t, s, sizeof t); out[n] = ppmm_recombine<D>(t, qd, qinv, c32d, qlid, last != 0, rl); break; }
#define WIDE(D) case D: { int t[D]; memcpy(t, s, sizeof t); out[n] = ppmm_recombine_wide<D>(t, qd, qinv, c32d, c64d, qlid, last != 0, exact_u2d(rl)); break; }
        if (!wide) {
            switch (ND) { NARROW(7) NARROW(8) default: return 1; }
        } else {
            switch (ND) { WIDE(9) default: return 1; }
        }
#undef NARROW
#undef WIDE
    }
    return 0;
}

}  // extern "C"

#ifdef F64R_MAIN
// Stand-alone run for the sanitizer build: f64_ranges_san.bin q:logN:wide:form ...  Each argument is one limb taken through the
// forward and the inverse transform on worst-case and random words; the round trip must give the words back with no range
// violation.  Tables: psi_table[bitrev(i)] = psi^i, psiinv_table[bitrev(i)] = psi^-i with N^-1 folded into entry 1 (Utils.cuh:160-203).
#include <cstdlib>

#include "../../ckks_llm_amd/csrc/host_math.hpp"

int main(int argc, char** argv) {
    namespace H = ckks_host;
    int bad = 0;
    for (int a = 1; a < argc; a++) {
        unsigned long long q = 0;
        int logN = 0, wide = 0, form = 0;
        if (sscanf(argv[a], "%llu:%d:%d:%d", &q, &logN, &wide, &form) != 4) { fprintf(stderr, "bad argument %s\n", argv[a]); return 2; }
        const long N = 1l << logN;
        const u64 psi = H::mth_root(2 * (u64)N, q);
        if (!psi) { fprintf(stderr, "%llu has no 2N-th root for logN %d\n", q, logN); return 2; }
        const u64 psi_inv = H::invmod(psi, q), n_inv = H::invmod((u64)N % q, q);
        std::vector<u64> fwd((size_t)N), inv((size_t)N);
        u64 p = 1, pi = 1;
        for (long i = 0; i < N; i++) {
            const uint32_t r = H::bitrev((uint32_t)i, logN);
            fwd[r] = p; inv[r] = pi;
            p = H::mulmod(p, psi, q); pi = H::mulmod(pi, psi_inv, q);
        }
        inv[1] = H::mulmod(inv[1], n_inv, q);
        for (int pattern = 0; pattern < 4; pattern++) {
            std::vector<u64> data((size_t)N), orig;
            unsigned long long s = 88172645463325252ull + (unsigned)pattern;
            for (long i = 0; i < N; i++) {
                s ^= s << 13; s ^= s >> 7; s ^= s << 17;
                data[(size_t)i] = pattern == 0 ? q - 1 : pattern == 1 ? ((i & 1) ? q - 1 : 0) : pattern == 2 ? (q / 2 + (u64)(i & 1)) : s % q;
            }
            orig = data;
            f64r_reset();
            if (f64r_ntt(wide, form, q, fwd.data(), n_inv, data.data(), logN, 0) || f64r_ntt(wide, form, q, inv.data(), n_inv, data.data(), logN, 1)) {
                fprintf(stderr, "unsupported logN %d\n", logN);
                return 2;
            }
            const bool same = data == orig;
            printf("q=%llu logN=%d wide=%d form=%d pattern=%d: %ld checks, %ld violations, max |x| = 2^%.2f, round trip %s%s%s\n", q, logN, wide, form, pattern,
                   g.checks, g.violations, std::log2(g.max_abs), same ? "ok" : "DIFFERS", g.violations ? " first: " : "", g.first);
            if (g.violations || !same) bad++;
        }
    }
    return bad ? 1 : 0;
}
#endif
