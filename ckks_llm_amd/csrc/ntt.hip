// Batched RNS negacyclic NTT / iNTT for gfx950.
//
// Replaces Context_23::ToNTTInplace / FromNTTInplace (+ _for_externalProduct) and their eight kernels
// (Context_23.cuh:847-930, ntt_60bit.cuh:421-1318).  Same transform: forward = Cooley-Tukey, natural ->
// bit-reversed order, twiddle of stage m / group i is psi_table[m + i]; inverse = Gentleman-Sande with
// psiinv_table[h + i], scaled by N^-1; outputs fully reduced.
//
// Decomposition (N = N1 * N2, N1 = 2^SA >= N2 = 2^SB):
//   forward : "strided" pass = first SA stages on columns (elements N2 apart), a workgroup owns all N1 rows of
//             CW adjacent columns (CW*8 B = one 128 B line per row); then the "row" pass = last SB stages on
//             rows of N2 contiguous words.  Inverse runs the mirror image (row pass first).
//   Each pass keeps R = 2^ceil(S/2) values per lane in registers and does its S stages in two register rounds
//   with one LDS exchange in between; every HBM access of both passes is a full 128 B line per 16 lanes.
//   All columns of the strided pass share the same 2^SA - 1 twiddles; the row pass reads each of the other
//   N - N1 twiddles exactly once per limb.
//
// Arithmetic back ends (modarith.hpp): IntArith (any q < 2^62) and F64Arith (q < 2^41): values are exact signed
// integers in doubles, a*w mod q = fma(-rint(a*w/q), q, a*w) evaluated with the two-product trick, no
// conditional corrections inside the butterflies.  Range analysis for F64Arith (|w| <= q/2):
//   forward: each stage adds at most 0.51 q to |x|, so after 16 stages |x| < 9.2 q < 2^45; the quotient
//            estimate rint(h * qinv) is off by < 2^-8, so |a*w - c*q| < 0.51 q.
//   inverse: the sum branch doubles |x| per stage; values are reduced to (-q/2, q/2] between the two passes, so
//            |x| < 2^8 * q < 2^49 inside a pass and every integer involved stays below 2^53.
// Between the two passes of one transform the buffer holds back-end specific words (lazy residues in [0,4q) /
// [0,2q) for IntArith, raw double bit patterns for F64Arith); after the second pass it holds canonical residues.
#include <cstdlib>

#include "context.hpp"

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
    __device__ __forceinline__ u64 to_canonical_fwd(V x) const { return csub(csub(x, q2), q); }
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
    double q, qinv, n_inv, w1n;
    __device__ __forceinline__ F64Arith(const PrimeConst& pc) : q(pc.qd), qinv(pc.qinv_d), n_inv(pc.n_inv_d), w1n(pc.w1n_d) {}
    __device__ __forceinline__ V from_canonical(u64 x) const { return (double)(long long)x; }
    __device__ __forceinline__ V from_mid(u64 x) const { return __longlong_as_double((long long)x); }
    __device__ __forceinline__ u64 to_mid_fwd(V x) const { return (u64)__double_as_longlong(x); }
    __device__ __forceinline__ V mulmod(V a, TW w) const {          // result in (-0.51 q, 0.51 q)
        double h = a * w;
        double l = __builtin_fma(a, w, -h);
        double c = __builtin_rint(h * qinv);
        return __builtin_fma(-c, q, h) + l;
    }
    __device__ __forceinline__ V balance(V x) const { return __builtin_fma(-__builtin_rint(x * qinv), q, x); }
    __device__ __forceinline__ u64 canon(V r) const {               // r in (-q, q) -> [0, q)
        r = r < 0.0 ? r + q : r;
        return (u64)(long long)r;
    }
    __device__ __forceinline__ u64 to_mid_inv(V x) const { return (u64)__double_as_longlong(balance(x)); }
    __device__ __forceinline__ u64 to_canonical_fwd(V x) const { return canon(balance(x)); }
    __device__ __forceinline__ void ct(V& x, V& y, TW w) const {
        double t = mulmod(y, w);
        y = x - t;
        x = x + t;
    }
    __device__ __forceinline__ void gs(V& x, V& y, TW w) const {
        double s = x + y, d = x - y;
        x = s;
        y = mulmod(d, w);
    }
    __device__ __forceinline__ void gs_last(V& x, V& y, u64& ox, u64& oy) const {
        double s = x + y, d = x - y;
        ox = canon(mulmod(s, n_inv));
        oy = canon(mulmod(d, w1n));
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
__device__ __forceinline__ void fwd_spread(typename AR::V (&v)[1 << S1], const typename AR::TW* __restrict__ tw, unsigned tw_off,
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
__device__ __forceinline__ void fwd_packed(typename AR::V (&v)[1 << S1], const typename AR::TW* __restrict__ tw, unsigned tw_off,
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
__device__ __forceinline__ void inv_packed(typename AR::V (&v)[1 << S1], const typename AR::TW* __restrict__ tw, unsigned tw_off,
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
__device__ __forceinline__ void inv_spread(typename AR::V (&v)[1 << S1], const typename AR::TW* __restrict__ tw, unsigned tw_off,
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

constexpr int s1_of(int S) { return (S + 1) / 2; }

// ------------------------------------------------------------------------------------------------------------
// strided pass (first SA forward stages / last SA inverse stages)
// ------------------------------------------------------------------------------------------------------------
template <class AR, int SA, int SB, bool INVERSE>
__global__ __launch_bounds__(((1 << SA) >> s1_of(SA)) * ((1 << SB) < 16 ? (1 << SB) : 16)) void ntt_strided_pass(NttArgs a) {
    constexpr int S1 = s1_of(SA), R = 1 << S1, N1 = 1 << SA, N2 = 1 << SB, G = N1 / R;
    constexpr int CW = N2 < 16 ? N2 : 16;
    constexpr long N = (long)N1 * N2;
    typedef typename AR::V V;
    typedef typename AR::TW TW;
    __shared__ V lds[N1 * CW];
    int prime;
    u64* limb = limb_ptr(a, blockIdx.y, N, prime);
    const AR ar(a.primes[prime]);
    const TW* __restrict__ tw = (const TW*)a.tw + (long)prime * N;
    const unsigned cl = threadIdx.x % CW, g = threadIdx.x / CW;
    u64* col = limb + blockIdx.x * CW + cl;
    V v[R];
    if (!INVERSE) {
#pragma unroll
        for (int j = 0; j < R; j++) v[j] = ar.from_canonical(col[(long)(g + j * G) * N2]);
        fwd_spread<AR, SA, S1>(v, tw, 1u, ar);
#pragma unroll
        for (int j = 0; j < R; j++) lds[(g + j * G) * CW + cl] = v[j];
        __syncthreads();
#pragma unroll
        for (int j = 0; j < R; j++) v[j] = lds[(g * R + j) * CW + cl];
        fwd_packed<AR, SA, S1>(v, tw, 1u, g, ar);
#pragma unroll
        for (int j = 0; j < R; j++) col[(long)(g * R + j) * N2] = ar.to_mid_fwd(v[j]);
    } else {
#pragma unroll
        for (int j = 0; j < R; j++) v[j] = ar.from_mid(col[(long)(g * R + j) * N2]);
        inv_packed<AR, SA, S1>(v, tw, 1u, g, ar);
#pragma unroll
        for (int j = 0; j < R; j++) lds[(g * R + j) * CW + cl] = v[j];
        __syncthreads();
#pragma unroll
        for (int j = 0; j < R; j++) v[j] = lds[(g + j * G) * CW + cl];
        inv_spread<AR, SA, S1, 1>(v, tw, 1u, ar);
        // stage 0 (h = 1): pairs (j, j + R/2), N^-1 folded in
#pragma unroll
        for (int j = 0; j < R / 2; j++) {
            u64 ox, oy;
            ar.gs_last(v[j], v[j + R / 2], ox, oy);
            col[(long)(g + j * G) * N2] = ox;
            col[(long)(g + (j + R / 2) * G) * N2] = oy;
        }
    }
}

// ------------------------------------------------------------------------------------------------------------
// row pass (last SB forward stages / first SB inverse stages) on rows of N2 contiguous words
// ------------------------------------------------------------------------------------------------------------
template <int SB>
struct RowCfg {
    static constexpr int S1 = s1_of(SB), R = 1 << S1, N2 = 1 << SB, U = N2 / R;      // U lanes per row
    static constexpr int ROWS = (4096 / N2) < 1 ? 1 : (4096 / N2);                    // rows per workgroup (tile of 4096 words)
    static constexpr int PITCH = N2 + N2 / 16;                                        // one pad word per 16: conflict-free packed reads
};
__device__ __forceinline__ int padded(int pos) { return pos + (pos >> 4); }

template <class AR, int SA, int SB, bool INVERSE>
__global__ __launch_bounds__(RowCfg<SB>::U * (RowCfg<SB>::ROWS < (1 << SA) ? RowCfg<SB>::ROWS : (1 << SA))) void ntt_row_pass(NttArgs a) {
    typedef RowCfg<SB> C;
    constexpr int S1 = C::S1, R = C::R, N2 = C::N2, U = C::U, N1 = 1 << SA;
    constexpr int ROWS = C::ROWS < N1 ? C::ROWS : N1;
    constexpr long N = (long)N1 * N2;
    typedef typename AR::V V;
    typedef typename AR::TW TW;
    __shared__ V lds[ROWS * C::PITCH];
    int prime;
    u64* limb = limb_ptr(a, blockIdx.y, N, prime);
    const AR ar(a.primes[prime]);
    const TW* __restrict__ tw = (const TW*)a.tw + (long)prime * N;
    const unsigned u = threadIdx.x % U, rl = threadIdx.x / U;
    const unsigned row = blockIdx.x * ROWS + rl;
    u64* rp = limb + (long)row * N2;
    V* lrow = lds + rl * C::PITCH;
    const unsigned tw_off = N1 + row;
    V v[R];
    if (!INVERSE) {
#pragma unroll
        for (int j = 0; j < R; j++) v[j] = ar.from_mid(rp[u + j * U]);
        fwd_spread<AR, SB, S1>(v, tw, tw_off, ar);
#pragma unroll
        for (int j = 0; j < R; j++) lrow[padded(u + j * U)] = v[j];
        __syncthreads();
#pragma unroll
        for (int j = 0; j < R; j++) v[j] = lrow[padded(u * R + j)];
        fwd_packed<AR, SB, S1>(v, tw, tw_off, u, ar);
        __syncthreads();
        // transpose back through LDS so the global stores are coalesced
#pragma unroll
        for (int j = 0; j < R; j++) lrow[padded(u * R + j)] = v[j];
        __syncthreads();
#pragma unroll
        for (int j = 0; j < R; j++) rp[u + j * U] = ar.to_canonical_fwd(lrow[padded(u + j * U)]);
    } else {
#pragma unroll
        for (int j = 0; j < R; j++) lrow[padded(u + j * U)] = ar.from_canonical(rp[u + j * U]);
        __syncthreads();
#pragma unroll
        for (int j = 0; j < R; j++) v[j] = lrow[padded(u * R + j)];
        inv_packed<AR, SB, S1>(v, tw, tw_off, u, ar);
        __syncthreads();
#pragma unroll
        for (int j = 0; j < R; j++) lrow[padded(u * R + j)] = v[j];
        __syncthreads();
#pragma unroll
        for (int j = 0; j < R; j++) v[j] = lrow[padded(u + j * U)];
        inv_spread<AR, SB, S1, 0>(v, tw, tw_off, ar);
#pragma unroll
        for (int j = 0; j < R; j++) rp[u + j * U] = ar.to_mid_inv(v[j]);
    }
}

template <class AR, int SA, int SB>
static int launch_two_pass(ckks_ctx* c, NttArgs args, int limbs, bool inverse) {
    constexpr int N1 = 1 << SA, N2 = 1 << SB, CW = N2 < 16 ? N2 : 16;
    constexpr int RA = 1 << s1_of(SA);
    typedef RowCfg<SB> C;
    constexpr int ROWS = C::ROWS < N1 ? C::ROWS : N1;
    static const int chunk_env = getenv("CKKS_NTT_CHUNK") ? atoi(getenv("CKKS_NTT_CHUNK")) : 0;
    const int chunk = (chunk_env > 0 && !c->ev_mid_armed) ? chunk_env : limbs;
    args.limbs_total = (unsigned)limbs;
    for (int base = 0; base < limbs; base += chunk) {
        const int n = limbs - base < chunk ? limbs - base : chunk;
        args.limb_base = (unsigned)base;
        dim3 gs(N2 / CW, n), bs((N1 / RA) * CW);
        dim3 gr(N1 / ROWS, n), br(C::U * ROWS);
        if (!inverse) {
            hipLaunchKernelGGL((ntt_strided_pass<AR, SA, SB, false>), gs, bs, 0, c->stream, args);
            if (c->ev_mid_armed) (void)hipEventRecord(c->ev_mid, c->stream);
            hipLaunchKernelGGL((ntt_row_pass<AR, SA, SB, false>), gr, br, 0, c->stream, args);
        } else {
            hipLaunchKernelGGL((ntt_row_pass<AR, SA, SB, true>), gr, br, 0, c->stream, args);
            if (c->ev_mid_armed) (void)hipEventRecord(c->ev_mid, c->stream);
            hipLaunchKernelGGL((ntt_strided_pass<AR, SA, SB, true>), gs, bs, 0, c->stream, args);
        }
    }
    CKKS_HIP_TRY(hipGetLastError());
    return CKKS_OK;
}

template <class AR>
static int dispatch_logn(ckks_ctx* c, const NttArgs& args, int limbs, bool inverse) {
    switch (c->logN) {
        case 8:  return launch_two_pass<AR, 4, 4>(c, args, limbs, inverse);
        case 9:  return launch_two_pass<AR, 5, 4>(c, args, limbs, inverse);
        case 10: return launch_two_pass<AR, 5, 5>(c, args, limbs, inverse);
        case 11: return launch_two_pass<AR, 6, 5>(c, args, limbs, inverse);
        case 12: return launch_two_pass<AR, 6, 6>(c, args, limbs, inverse);
        case 13: return launch_two_pass<AR, 7, 6>(c, args, limbs, inverse);
        case 14: return launch_two_pass<AR, 7, 7>(c, args, limbs, inverse);
        case 15: return launch_two_pass<AR, 8, 7>(c, args, limbs, inverse);
        case 16: return launch_two_pass<AR, 8, 8>(c, args, limbs, inverse);
        default: set_error("NTT: logN must be in [8, 16]"); return CKKS_E_INVALID;
    }
}

int launch_ntt(ckks_ctx* c, uint64_t* dev, int start_poly_idx, int start_mod_idx, int poly_num, int mod_num,
               int poly_mod_len, long batch_stride_limbs, int batch, bool inverse) {
    if (!c || !dev) { set_error("NTT: null argument"); return CKKS_E_INVALID; }
    if (poly_num <= 0 || mod_num <= 0 || batch <= 0) return CKKS_OK;      // empty batch: nothing to do
    if (start_mod_idx < 0 || start_mod_idx + mod_num > c->nprimes || start_poly_idx < 0 || poly_mod_len < 0) {
        set_error("NTT: prime range outside the context");
        return CKKS_E_INVALID;
    }
    long limbs = (long)poly_num * mod_num * batch;
    if (limbs > 65535) { set_error("NTT: more than 65535 limbs in one call"); return CKKS_E_INVALID; }
    bool f64 = c->arith_mode == 0;
    for (int j = 0; j < mod_num && f64; j++) f64 = c->f64_ok[start_mod_idx + j] != 0;
    NttArgs args;
    args.data = (u64*)dev;
    args.primes = c->d_primes;
    args.start_poly_idx = start_poly_idx;
    args.start_mod_idx = start_mod_idx;
    args.poly_num = poly_num;
    args.mod_num = mod_num;
    args.poly_mod_len = poly_mod_len;
    args.batch_stride_limbs = batch_stride_limbs;
    if (f64) {
        args.tw = inverse ? (const void*)c->d_twd_inv : (const void*)c->d_twd_fwd;
        return dispatch_logn<F64Arith>(c, args, (int)limbs, inverse);
    }
    args.tw = inverse ? (const void*)c->d_tw_inv : (const void*)c->d_tw_fwd;
    return dispatch_logn<IntArith>(c, args, (int)limbs, inverse);
}

}  // namespace ckks
