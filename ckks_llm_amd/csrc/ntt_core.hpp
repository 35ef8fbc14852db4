// Device code shared by the transform kernels: arithmetic back ends, the register-resident axis transforms of a tile,
// the inter-pass forms and the limb addressing rule of Context_23::ToNTTInplace / FromNTTInplace (ntt_60bit.cuh:446-455).
#pragma once
#include <type_traits>

#include "context.hpp"
#include "f64_exact.hpp"

namespace ckks {

// ------------------------------------------------------------------------------------------------------------
// arithmetic back ends
// ------------------------------------------------------------------------------------------------------------
struct IntArith {
    typedef u64 V;
    typedef ulonglong2 TW;
    u64 q, q2;
    u64 n_inv, n_inv_s, w1n, w1n_s;
    __device__ __forceinline__ IntArith(const PrimeConst& pc)
        : q(pc.q), q2(pc.q * 2), n_inv(pc.n_inv), n_inv_s(pc.n_inv_s), w1n(pc.w1n), w1n_s(pc.w1n_s) {}
    __device__ __forceinline__ V from_canonical(u64 x) const { return x; }
    __device__ __forceinline__ V from_mid(u64 x) const { return x; }
    __device__ __forceinline__ u64 to_mid_fwd(V x) const { return x; }          // lazy [0,4q)
    __device__ __forceinline__ u64 to_mid_inv(V x) const { return x; }          // lazy [0,2q)
    static constexpr bool lazy40 = false;
    __device__ __forceinline__ u64 enc40(V x) const { return x; }               // the compact inter-pass form is FP64-only
    __device__ __forceinline__ u64 enc40_raw(V x) const { return x; }
    __device__ __forceinline__ V dec40(unsigned lo, unsigned) const { return lo; }
    __device__ __forceinline__ u64 to_canonical_fwd(V x) const { return csub(csub(x, q2), q); }
    template <int R> __device__ __forceinline__ void round_end(V (&)[R]) const {}          // lazy ranges hold for a whole pass
    // Harvey lazy butterflies; ranges as ntt_60bit.cuh:293-318
    __device__ __forceinline__ void ct(V& x, V& y, TW w) const {
        x = x >= q2 ? x - q2 : x;
        u64 t = mul_shoup_lazy(y, w.x, w.y, q);
        y = x + q2 - t;
        x = x + t;
    }
    __device__ __forceinline__ void gs(V& x, V& y, TW w) const {
        u64 s = x + y, d = x + q2 - y;
        x = s >= q2 ? s - q2 : s;
        y = mul_shoup_lazy(d, w.x, w.y, q);
    }
    // last inverse stage with N^-1 folded in (ntt_60bit.cuh:890-897); canonical outputs
    __device__ __forceinline__ void gs_last(V& x, V& y, u64& ox, u64& oy) const {
        u64 s = x + y, d = x + q2 - y;
        ox = mul_shoup(s, n_inv, n_inv_s, q);
        oy = mul_shoup(d, w1n, w1n_s, q);
    }
};

struct F64Arith {
    typedef double V;
    typedef double TW;
    double q, qinv, hqinv, n_inv, w1n;
    bool lazy40;               // q < 2^36.5: the values between the passes of a forward transform (|x| < 5.1 q) fit 40 bits as they are
    CKKS_HD F64Arith(const PrimeConst& pc)
        : q(pc.qd), qinv(pc.qinv_d), hqinv(0.5 * pc.qinv_d), n_inv(pc.n_inv_d), w1n(pc.w1n_d), lazy40(pc.qd < 97184015999.0) {}
    // canonical residue (below 2^52) -> double: the word is the mantissa of 2^52 + x
    CKKS_HD V from_canonical(u64 x) const { return exact_u2d(x); }
    CKKS_HD V from_mid(u64 x) const { return f64_from_bits(x); }
    CKKS_HD u64 to_mid_fwd(V x) const { return f64_bits(x); }
    CKKS_HD V mulmod(V a, TW w) const { return mulmod_f64(a, w, q, qinv); }          // result in (-0.51 q, 0.51 q)
    CKKS_HD V balance(V x) const { return balance_f64(x, q, qinv); }
    CKKS_HD static u64 bits52(V r) { return ::ckks::bits52(r); }
    CKKS_HD u64 canon(V r) const {               // r in (-q, q) -> [0, q)
        r = r < 0.0 ? r + q : r;
        return bits52(r);
    }
    // any integer |x| < 2^10 q -> [0, q) without a sign fix-up: (x + 1/2) / q is at least 1/(2q) > 2^-42 away from every integer
    // and the product is off by less than 2^-42, so the floor is exactly floor(x / q)
    CKKS_HD u64 canon_any(V x) const {
        const double c = __builtin_floor(__builtin_fma(x, qinv, hqinv));
        const u64 res = bits52(__builtin_fma(-c, q, x));
        CKKS_RANGE(canonical(x, q, res, "F64Arith::canon_any"));
        return res;
    }
    CKKS_HD u64 to_mid_inv(V x) const { return f64_bits(balance(x)); }
    // 40-bit form of a balanced value (q < 2^39, so |r| < 2^38.1): r + 2^39 read from the low mantissa bits of r + 2^52 + 2^39
    CKKS_HD u64 enc40(V x) const { return enc40_raw(balance(x)); }
    CKKS_HD u64 enc40_raw(V x) const {                                                 // |x| < 2^39
        CKKS_RANGE(below(x, 549755813888.0, "F64Arith::enc40_raw"));
        return f64_bits(x + 4504149383184384.0) & 0xFFFFFFFFFFull;
    }
    // 36-bit form of a balanced value (q < 2^36, so |r| < 2^35): r + 2^35 read from the low mantissa bits of r + 2^52 + 2^35
    CKKS_HD u64 enc36(V x) const {
        const V r = balance(x);
        CKKS_RANGE(below(r, 34359738368.0, "F64Arith::enc36"));
        return f64_bits(r + 4503633987108864.0) & 0xFFFFFFFFFull;
    }
    CKKS_HD V dec36(unsigned lo, unsigned hi4) const { return f64_from_bits(0x4330000000000000ull | ((u64)hi4 << 32) | lo) - 4503633987108864.0; }
    CKKS_HD V dec40(unsigned lo, unsigned hi8) const { return f64_from_bits(0x4330000000000000ull | ((u64)hi8 << 32) | lo) - 4504149383184384.0; }
    CKKS_HD u64 to_canonical_fwd(V x) const { return canon_any(x); }
    template <int R> CKKS_HD void round_end(V (&)[R]) const {}          // q < 2^41: the ranges hold for a whole pass
    CKKS_HD void ct(V& x, V& y, TW w) const {
        double t = mulmod(y, w);
        y = x - t;
        x = x + t;
        CKKS_RANGE(value(x, "F64Arith::ct sum"));
        CKKS_RANGE(value(y, "F64Arith::ct difference"));
    }
    CKKS_HD void gs(V& x, V& y, TW w) const {
        double s = x + y, d = x - y;
        CKKS_RANGE(value(s, "F64Arith::gs sum"));
        CKKS_RANGE(value(d, "F64Arith::gs difference"));
        x = s;
        y = mulmod(d, w);
    }
    CKKS_HD void gs_last(V& x, V& y, u64& ox, u64& oy) const {
        double s = x + y, d = x - y;
        CKKS_RANGE(value(s, "F64Arith::gs_last sum"));
        CKKS_RANGE(value(d, "F64Arith::gs_last difference"));
        ox = canon_any(mulmod(s, n_inv));
        oy = canon_any(mulmod(d, w1n));
    }
};

// FP64 back end for primes up to 2^50 (the reference's own 49-bit Q and P primes, Params.cuh:84-171).  Same exact-integer
// arithmetic as F64Arith; what changes is how far a value may drift from zero before it is brought back, because every
// integer involved must stay below 2^53 and the quotient estimate of mulmod loses accuracy as its operand grows:
//   mulmod(y, w), |w| <= q/2, |y| <= b q: the estimate rint(fl(fl(y w) fl(1/q))) is off by at most 0.5 + 3 * 2^-53 * b q / 2
//   < 0.5 + 0.19 b, so the result lies within (0.5 + 0.19 b) q of zero and h - c q, an integer below 2^53, is exact.
//   forward (x +- t): from |x| <= q/2 four stages reach 1.2, 1.9, 2.8, 3.8 q; inverse (sums double): from q/2 four stages
//   reach 8 q < 2^53.  So every value is balanced to (-q/2, q/2] when it is loaded, after each register round of at most four
//   stages (round_end) and before it is stored between the passes; the last stage of an inverse transform multiplies sums
//   of at most 8 q (results within 2 q of zero) and canonicalises by a balance and one conditional addition.
struct F64WideArith : F64Arith {
    double half;
    CKKS_HD F64WideArith(const PrimeConst& pc) : F64Arith(pc), half(0.5 * pc.qd) {}
    CKKS_HD V from_canonical(u64 x) const {
        const double d = F64Arith::from_canonical(x);
        return d > half ? d - q : d;
    }
    CKKS_HD u64 canon_wide(V x) const {            // any integer |x| < 2^53 -> [0, q)
        const double r = balance(x);                                   // within (q + 1) / 2 of zero
        const u64 res = bits52(r < 0.0 ? r + q : r);
        CKKS_RANGE(canonical(x, q, res, "F64WideArith::canon_wide"));
        return res;
    }
    CKKS_HD u64 to_mid_fwd(V x) const { return f64_bits(balance(x)); }
    CKKS_HD u64 to_canonical_fwd(V x) const { return canon_wide(x); }
    template <int R> CKKS_HD void round_end(V (&v)[R]) const {
#pragma unroll
        for (int j = 0; j < R; j++) v[j] = balance(v[j]);
    }
    CKKS_HD void gs_last(V& x, V& y, u64& ox, u64& oy) const {
        double s = x + y, d = x - y;
        CKKS_RANGE(value(s, "F64WideArith::gs_last sum"));
        CKKS_RANGE(value(d, "F64WideArith::gs_last difference"));
        ox = canon_wide(mulmod(s, n_inv));
        oy = canon_wide(mulmod(d, w1n));
    }
};

// ------------------------------------------------------------------------------------------------------------
// S-stage axis transforms on R = 2^S1 register values (S1 = ceil(S/2))
//   "spread" layout : register j holds axis position  g + j * (AX / R)
//   "packed" layout : register j holds axis position  g * R + j
// Twiddle of forward stage s (0 <= s < S) for axis position e (pair partner e + AX/2^(s+1)):
//   tw[(tw_off << s) + (e >> (S - s))],  tw_off = 1 for the strided pass, N1 + row for the row pass.
// ------------------------------------------------------------------------------------------------------------
template <class AR, int S, int S1>
CKKS_HD void fwd_spread(typename AR::V (&v)[1 << S1], const typename AR::TW* __restrict__ tw, unsigned tw_off,
                                           const AR& ar) {
    constexpr int R = 1 << S1;
#pragma unroll
    for (int s = 0; s < S1; s++) {
        const int half = R >> (s + 1);
#pragma unroll
        for (int j = 0; j < R; j++) {
            if ((j & half) == 0) {
                typename AR::TW w = tw[(tw_off << s) + (j >> (S1 - s))];
                ar.ct(v[j], v[j + half], w);
            }
        }
    }
}
template <class AR, int S, int S1>
CKKS_HD void fwd_packed(typename AR::V (&v)[1 << S1], const typename AR::TW* __restrict__ tw, unsigned tw_off,
                                           unsigned g, const AR& ar) {
    constexpr int R = 1 << S1;
#pragma unroll
    for (int s = S1; s < S; s++) {
        const int dist = 1 << (S - s - 1);
#pragma unroll
        for (int j = 0; j < R; j++) {
            if ((j & dist) == 0) {
                typename AR::TW w = tw[(tw_off << s) + ((g * R + j) >> (S - s))];
                ar.ct(v[j], v[j + dist], w);
            }
        }
    }
}
// inverse: same index structure, stages in the opposite order, Gentleman-Sande butterflies
template <class AR, int S, int S1>
CKKS_HD void inv_packed(typename AR::V (&v)[1 << S1], const typename AR::TW* __restrict__ tw, unsigned tw_off,
                                           unsigned g, const AR& ar) {
    constexpr int R = 1 << S1;
#pragma unroll
    for (int s = S - 1; s >= S1; s--) {
        const int dist = 1 << (S - s - 1);
#pragma unroll
        for (int j = 0; j < R; j++) {
            if ((j & dist) == 0) {
                typename AR::TW w = tw[(tw_off << s) + ((g * R + j) >> (S - s))];
                ar.gs(v[j], v[j + dist], w);
            }
        }
    }
}
template <class AR, int S, int S1, int S_STOP>
CKKS_HD void inv_spread(typename AR::V (&v)[1 << S1], const typename AR::TW* __restrict__ tw, unsigned tw_off,
                                           const AR& ar) {
    constexpr int R = 1 << S1;
#pragma unroll
    for (int s = S1 - 1; s >= S_STOP; s--) {
        const int half = R >> (s + 1);
#pragma unroll
        for (int j = 0; j < R; j++) {
            if ((j & half) == 0) {
                typename AR::TW w = tw[(tw_off << s) + (j >> (S1 - s))];
                ar.gs(v[j], v[j + half], w);
            }
        }
    }
}

struct NttArgs {
    u64* data;
    const PrimeConst* primes;
    const void* tw;            // [prime][N] twiddles of the back end in use
    int start_poly_idx, start_mod_idx, poly_num, mod_num, poly_mod_len;
    long batch_stride_limbs;
    unsigned limb_base, limbs_total;      // this launch covers limbs limb_base .. limb_base + gridDim.y - 1 of limbs_total
    char* mid;                            // compact inter-pass buffer (MID_LIMB_BYTES per limb of the launch) or nullptr
    int reverse = 0;                      // take the limbs of the launch from the last to the first (see launch_passes)
    long out_delta = 0;                   // paired transform with the 5-byte inter-pass form: its second pass writes out_delta words behind data
    // Forward transforms of polynomials that exist only as scattered MLWE samples (the embedding of the ring packing): when
    // embed_mlwe is set the first pass takes coefficient pos of polynomial y from sample (pos mod k) / gap, coefficient
    // pos / k (zero where pos mod k is no multiple of gap), lifted around zero from q0 to p0 on the limbs of the first prime.
    const u64* const* embed_mlwe = nullptr;
    u64 embed_p0 = 0, embed_q0 = 0;
    int embed_logk = 0, embed_loggap = 0, embed_n1 = 0;
    int embed_no_wrap = 0;                // q0 / 2 < p0: the lift p0 - (q0 - x) never wraps, the reference's `% p0` is the identity
};

// Compact inter-pass form (N = 2^16, FP64 back end, q < 2^39): 5 bytes per value instead of 8, in a separate buffer laid out
// for BOTH passes: piece (cb, rb) = the 16 x 16 block of columns 16cb.. and rows 16rb.., 1280 bytes:
//   lo words  [r_local][c_local]            1024 B
//   hi bytes  forward transforms: [r_local / 4][c_local] dwords, byte r_local % 4; inverse transforms: [r_local][c_local]   256 B
// The strided pass (tile = cb) touches pieces (cb, 0..15), the row pass (tile = rb) pieces (0..15, rb); in all four access
// patterns 16 lanes cover 64 contiguous bytes.
// Accesses to data that another workgroup of the SAME launch writes or reads (the paired transform): relaxed atomics at agent
// scope, i.e. ordinary loads and stores that are carried out at the level of the memory hierarchy all compute units share.
template <bool SHARED, class T>
__device__ __forceinline__ void put(T* p, T v) {
    if (SHARED) __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else *p = v;
}
template <bool SHARED, class T>
__device__ __forceinline__ T get(const T* p) {
    if (SHARED) return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return *p;
}
constexpr int MID_PIECE_BYTES = 1280;
constexpr long MID_LIMB_BYTES = 256l * MID_PIECE_BYTES;
__device__ __forceinline__ char* mid_piece(char* mid_limb, unsigned cb, unsigned rb) { return mid_limb + (cb * 16 + rb) * MID_PIECE_BYTES; }
// Forward first pass, lane (cl, g) holding rows 16g .. 16g+15 of column cl of tile cb: writes its 16 values into piece (cb, g).
template <class AR, bool SHARED = false>
__device__ __forceinline__ void mid_store_columns(char* mid_limb, unsigned cb, unsigned g, unsigned cl, const typename AR::V (&v)[16], const AR& ar) {
    char* piece = mid_piece(mid_limb, cb, g);
    unsigned hi[4] = {0, 0, 0, 0};
    u64 e[16];
    if (ar.lazy40) {                 // uniform over the workgroup: small primes skip the reduction before the 40-bit form
#pragma unroll
        for (int j = 0; j < 16; j++) e[j] = ar.enc40_raw(v[j]);
    } else {
#pragma unroll
        for (int j = 0; j < 16; j++) e[j] = ar.enc40(v[j]);
    }
#pragma unroll
    for (int j = 0; j < 16; j++) {
        put<SHARED>(reinterpret_cast<unsigned*>(piece + (j * 16 + cl) * 4), (unsigned)e[j]);
        hi[j >> 2] |= (unsigned)(e[j] >> 32) << (8 * (j & 3));
    }
#pragma unroll
    for (int jg = 0; jg < 4; jg++) put<SHARED>(reinterpret_cast<unsigned*>(piece + 1024 + (jg * 16 + cl) * 4), hi[jg]);
}
// Forward second pass, lane (u, rl) of row tile rb taking columns u + 16j of row 16 rb + rl: element (rl, u) of piece (j, rb).
// The raw words are returned undecoded so that a caller can request them ahead of their use.
template <bool SHARED = false>
__device__ __forceinline__ void mid_load_row_raw(const char* mid_limb, unsigned rb, unsigned rl, unsigned u, unsigned (&lo)[16], unsigned (&hi)[16]) {
#pragma unroll
    for (int j = 0; j < 16; j++) {
        const char* piece = mid_piece(const_cast<char*>(mid_limb), j, rb);
        lo[j] = get<SHARED>(reinterpret_cast<const unsigned*>(piece + (rl * 16 + u) * 4));
        hi[j] = get<SHARED>(reinterpret_cast<const unsigned*>(piece + 1024 + ((rl >> 2) * 16 + u) * 4));
    }
}
template <class AR>
__device__ __forceinline__ typename AR::V mid_decode_row(const AR& ar, unsigned lo, unsigned hi, unsigned rl) {
    return ar.dec40(lo, (hi >> (8 * (rl & 3))) & 0xffu);
}
// Inverse first pass (row pass) output in the inverse layout of the high bytes: bytes [r_local][c_local].
template <class AR, bool SHARED = false>
__device__ __forceinline__ void mid_store_row_inverse(char* mid_limb, unsigned rb, unsigned rl, unsigned u, const typename AR::V (&v)[16], const AR& ar) {
#pragma unroll
    for (int j = 0; j < 16; j++) {
        char* piece = mid_piece(mid_limb, j, rb);
        const u64 e = ar.enc40(v[j]);
        put<SHARED>(reinterpret_cast<unsigned*>(piece + (rl * 16 + u) * 4), (unsigned)e);
        put<SHARED>(reinterpret_cast<unsigned char*>(piece + 1024 + rl * 16 + u), (unsigned char)(e >> 32));
    }
}

// The two forms in which a stage-fused launch hands a forward transform's first pass to the kernel that runs its second:
// the 5-byte pieces above (primes below 2^39) and, for wider primes, the limb itself as it lies between the passes of an
// in-place transform (balanced doubles, row-major).  request() fetches lane (u, rl)'s sixteen words of row tile rb undecoded,
// so that a caller can ask for them ahead of their use.
struct MidPieces {
    static constexpr long LIMB_BYTES = MID_LIMB_BYTES;
    struct Raw { unsigned lo[16], hi[16]; };
    template <class AR, bool SHARED = false>
    static __device__ __forceinline__ void store_columns(char* mid_limb, unsigned cb, unsigned g, unsigned cl, const double (&v)[16], const AR& ar) {
        mid_store_columns<AR, SHARED>(mid_limb, cb, g, cl, v, ar);
    }
    template <bool SHARED = false>
    static __device__ __forceinline__ void request(const char* mid_limb, unsigned rb, unsigned rl, unsigned u, Raw& r) {
        mid_load_row_raw<SHARED>(mid_limb, rb, rl, u, r.lo, r.hi);
    }
    template <class AR>
    static __device__ __forceinline__ double decode(const AR& ar, const Raw& r, int j, unsigned rl) { return mid_decode_row(ar, r.lo[j], r.hi[j], rl); }
};
struct MidLimb {
    static constexpr long LIMB_BYTES = 65536l * 8;
    struct Raw { u64 w[16]; };
    template <class AR, bool SHARED = false>
    static __device__ __forceinline__ void store_columns(char* mid_limb, unsigned cb, unsigned g, unsigned cl, const double (&v)[16], const AR& ar) {
        u64* col = reinterpret_cast<u64*>(mid_limb) + cb * 16 + cl;
#pragma unroll
        for (int j = 0; j < 16; j++) put<SHARED>(col + (long)(g * 16 + j) * 256, ar.to_mid_fwd(v[j]));
    }
    template <bool SHARED = false>
    static __device__ __forceinline__ void request(const char* mid_limb, unsigned rb, unsigned rl, unsigned u, Raw& r) {
        const u64* row = reinterpret_cast<const u64*>(mid_limb) + (long)(rb * 16 + rl) * 256 + u;
#pragma unroll
        for (int j = 0; j < 16; j++) r.w[j] = get<SHARED>(row + j * 16);
    }
    template <class AR>
    static __device__ __forceinline__ double decode(const AR& ar, const Raw& r, int j, unsigned) { return ar.from_mid(r.w[j]); }
};

// limb index of this block -> base pointer and prime.  Limbs are ordered prime-major so that consecutive
// workgroups reuse one prime's twiddle table while it is hot in L2.
__device__ __forceinline__ u64* limb_ptr(const NttArgs& a, unsigned limb, long N, int& prime) {
    limb += a.limb_base;
    unsigned per_mod = a.limbs_total / a.mod_num;      // poly_num * batch
    unsigned j = limb / per_mod, r = limb % per_mod;
    unsigned y = r % a.poly_num, z = r / a.poly_num;
    prime = a.start_mod_idx + (int)j;
    return a.data + ((long)z * a.batch_stride_limbs + (long)y * a.poly_mod_len + a.start_poly_idx + j) * N;
}

// residue modulo q0 -> residue modulo p0 of the same centred value (mlweCipherEmbedding_new_kernel, PCMM_Scheme.cuh:335-339:
// x > q0/2 ? (p0 - (q0 - x)) % p0 : x).  The 64-bit remainder is a long instruction sequence; with q0 / 2 < p0 it is the identity.
__device__ __forceinline__ u64 embed_lift(u64 x, const NttArgs& a) {
    if (x <= a.embed_q0 / 2) return x;
    const u64 t = a.embed_p0 - (a.embed_q0 - x);
    return a.embed_no_wrap ? t : t % a.embed_p0;
}
__device__ __forceinline__ unsigned limb_poly(const NttArgs& a, unsigned limb) {
    limb += a.limb_base;
    return (limb % (a.limbs_total / a.mod_num)) % a.poly_num;
}

constexpr int s1_of(int S) { return (S + 1) / 2; }

// Data loads of the second pass of the fused kernel read what OTHER compute units of the same XCD stored a moment ago.
// Those stores are in the XCD's L2 (vector stores write through the L1); the reader only has to keep clear of its own L1,
// which may still hold the pre-transform contents of the same lines.  A relaxed agent-scope atomic load is an ordinary
// 8-byte load that bypasses the L1 and is served by the L2.
template <bool COHERENT>
__device__ __forceinline__ u64 load_word(const u64* p) {
    if (COHERENT) return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return *p;
}
// Final stores of such a second pass are not read again on the chip: marked non-temporal, the L2 gives their lines up first and
// keeps the lines that are still between their two passes.
template <bool STREAM>
__device__ __forceinline__ void store_word(u64* p, u64 v) {
    if (STREAM) __builtin_nontemporal_store(v, p);
    else *p = v;
}

// tile shapes of the two passes
template <int SA, int SB>
struct StridedCfg {
    static constexpr int S1 = s1_of(SA), R = 1 << S1, N1 = 1 << SA, N2 = 1 << SB, G = N1 / R;
    static constexpr int CW = N2 < 16 ? N2 : 16;
    static constexpr int THREADS = G * CW, TILES = N2 / CW, LDS_WORDS = N1 * CW;
};
template <int SA, int SB>
struct RowCfg {
    static constexpr int S1 = s1_of(SB), R = 1 << S1, N1 = 1 << SA, N2 = 1 << SB, U = N2 / R;      // U lanes per row
    static constexpr int ROWS0 = (4096 / N2) < 1 ? 1 : (4096 / N2);                                // tile of 4096 words
    static constexpr int ROWS = ROWS0 < N1 ? ROWS0 : N1;
    static constexpr int PITCH = N2 + N2 / 16;                                        // one pad word per 16: conflict-free packed reads
    static constexpr int THREADS = U * ROWS, TILES = N1 / ROWS, LDS_WORDS = ROWS * PITCH;
};
__device__ __forceinline__ int padded(int pos) { return pos + (pos >> 4); }

}  // namespace ckks
