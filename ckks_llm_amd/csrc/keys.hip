// Switching keys in the auxiliary T basis and the homomorphic operations built on the key switch (multiply, rotate, conjugate)
// for gfx950.
//
// Reference: Scheme_23::addMultKey_23 / addConjKey_23 / addLeftRotKey_23 (KeySwitch_23.cuh:21-165), mult_23 (:192-236),
// conjugate_23 (:433-468), leftRotate_23 (:556-586); kernels compute_c0c1c2 (poly_arithmetic.cuh:787-824),
// cipher_add_axbx_batch_device (:159-172, 416-420), sxsx_mul_P_3param (:526-547), sk_and_poly_LeftRot_ntt / _inv (:581-660),
// sk_and_poly_conjugate (:666-680).
//
// The key switch itself (iNTT, ModUp to T, NTT, external product, iNTT, ModUp to PQ, ModDown, NTT) is ckks_keyswitch_23; this
// file adds what surrounds it.  The reference runs the surrounding element-wise steps as separate launches (tensor product, two
// additions, two permutations); here each operation has one kernel before the switch and one after it.  All kernels stream
// 8-byte words, one lane per coefficient; the permutation reads scattered (a bit-reversed affine index) and writes in order.
#include <hip/hip_runtime.h>
#include <string>
#include <vector>

#include "context.hpp"
#include "host_math.hpp"

using namespace ckks;
namespace H = ckks_host;

namespace {

constexpr int THREADS = 256;
constexpr int MAX_DIGIT_PRIMES = 16;

__device__ __forceinline__ u64 mulmod(u64 a, u64 b, const PrimeConst& p) {
    u128w acc{0, 0};
    mac128(acc, a, b);
    return barrett128(acc, p.q, p.mu_hi, p.mu_lo);
}

// NTT slot j holds the evaluation at psi^(2*bitrev(j)+1).  The reference scatters out[j] = in[i] with
// 2*bitrev(j)+1 = pow * (2*bitrev(i)+1) mod 2N; the same map as a gather needs pow^-1: i = bitrev((pow^-1 * (2*bitrev(j)+1) mod 2N - 1) / 2).
__device__ __forceinline__ long automorph_source(long j, u64 pow_inv, int logN) {
    const u64 mask = (2ull << logN) - 1;
    const u64 e = 2ull * (__brev((uint32_t)j) >> (32 - logN)) + 1;
    const u64 src = (((pow_inv * e) & mask) - 1) >> 1;
    return (long)(__brev((uint32_t)src) >> (32 - logN));
}

// out[idx_out + t][j] = in[idx_in + t][source(j)] (+ add[idx_in + t][source(j)] when add is given), grid.z = polynomials of a pair
__global__ __launch_bounds__(THREADS) void automorph_kernel(u64* out, const u64* in, const u64* add, const PrimeConst* primes, long N, int logN,
                                                            u64 pow_inv, int idx_mod, long out_poly_stride, long in_poly_stride, int add_poly) {
    const long j = (long)blockIdx.x * THREADS + threadIdx.x;
    const int t = blockIdx.y, z = blockIdx.z;
    const long i = automorph_source(j, pow_inv, logN);
    u64 v = in[z * in_poly_stride + (long)t * N + i];
    if (add && z == add_poly) v = csub(v + add[(long)t * N + i], primes[idx_mod + t].q);
    out[z * out_poly_stride + (long)t * N + j] = v;
}
// out[t][i] = in[t][N-1-i]
__global__ __launch_bounds__(THREADS) void reverse_kernel(u64* out, const u64* in, long N) {
    const long i = (long)blockIdx.x * THREADS + threadIdx.x;
    const int t = blockIdx.y;
    out[(long)t * N + i] = in[(long)t * N + N - 1 - i];
}
// out[t][i] = out[t][i] + in[t][N-1-i] mod q
__global__ __launch_bounds__(THREADS) void add_reversed_kernel(u64* out, const u64* in, const PrimeConst* primes, long N, int idx_mod) {
    const long i = (long)blockIdx.x * THREADS + threadIdx.x;
    const int t = blockIdx.y;
    out[(long)t * N + i] = csub(out[(long)t * N + i] + in[(long)t * N + N - 1 - i], primes[idx_mod + t].q);
}

// digit i of a switching key over [P | Q]: b = (P * s_from on the digit's own primes) + e - a * s_to  (KeySwitch_23.cuh:41-50)
struct DigitConst {
    int first_prime, count;            // pqt indices first_prime .. first_prime + count - 1 carry P * s_from
    u64 pmod[MAX_DIGIT_PRIMES];        // P mod q for those primes
};
__global__ __launch_bounds__(THREADS) void swk_combine_kernel(u64* bx, const u64* ax, const u64* ex, const u64* s_to, const u64* s_from,
                                                              const PrimeConst* primes, long N, int K, DigitConst d) {
    const long i = (long)blockIdx.x * THREADS + threadIdx.x;
    const int t = blockIdx.y;                                   // pqt index
    const PrimeConst p = primes[t];
    const long o = (long)t * N + i;
    u64 v = ex[o];
    if (t >= d.first_prime && t < d.first_prime + d.count) v = csub(v + mulmod(s_from[(long)(t - K) * N + i], d.pmod[t - d.first_prime], p), p.q);
    bx[o] = csub(p.q + v - mulmod(ax[o], s_to[o], p), p.q);
}

// tensor product of two ciphertexts (compute_c0c1c2_kernel): a1*a2, b1*b2, and a1*b2 + a2*b1 through (a1+b1)(a2+b2) - a1*a2 - b1*b2
// in 128 bits, each reduced once as the reference does
__global__ __launch_bounds__(THREADS) void tensor_kernel(u64* axbx, u64* axax, u64* bxbx, const u64* a1, const u64* a2, const u64* b1, const u64* b2,
                                                         const PrimeConst* primes, long N, int K) {
    const long i = (long)blockIdx.x * THREADS + threadIdx.x;
    const int t = blockIdx.y;
    const PrimeConst p = primes[K + t];
    const long o = (long)t * N + i;
    const u64 ra1 = a1[o], ra2 = a2[o], rb1 = b1[o], rb2 = b2[o];
    u128w t1{0, 0}, t2{0, 0}, t3{0, 0};
    mac128(t1, ra1, ra2);
    mac128(t2, rb1, rb2);
    mac128(t3, ra1 + rb1, ra2 + rb2);
    // t3 -= t1; t3 -= t2 (128-bit)
    u64 lo = t3.lo - t1.lo;
    u64 hi = t3.hi - t1.hi - (t3.lo < t1.lo);
    const u64 lo2 = lo - t2.lo;
    hi = hi - t2.hi - (lo < t2.lo);
    t3.lo = lo2; t3.hi = hi;
    axax[o] = barrett128(t1, p.q, p.mu_hi, p.mu_lo);
    bxbx[o] = barrett128(t2, p.q, p.mu_hi, p.mu_lo);
    axbx[o] = barrett128(t3, p.q, p.mu_hi, p.mu_lo);
}
// cipher.a += x, cipher.b += y (cipher_add_axbx_batch_device_kernel)
__global__ __launch_bounds__(THREADS) void add_pair_kernel(u64* ax, u64* bx, const u64* x, const u64* y, const PrimeConst* primes, long N, int K) {
    const long i = (long)blockIdx.x * THREADS + threadIdx.x;
    const int t = blockIdx.y;
    const u64 q = primes[K + t].q;
    const long o = (long)t * N + i;
    ax[o] = csub(ax[o] + x[o], q);
    bx[o] = csub(bx[o] + y[o], q);
}

int need_t_basis(ckks_ctx* c, const char* who) {
    if (!c) { set_error(std::string(who) + ": null context"); return CKKS_E_INVALID; }
    if (c->t_num == 0 || c->gamma == 0 || c->p_num == 0) { set_error(std::string(who) + ": the context has no P or T basis"); return CKKS_E_INVALID; }
    return CKKS_OK;
}
int need_level(ckks_ctx* c, int l, const char* who) {
    if (l < 0 || l > c->L) { set_error(std::string(who) + ": level outside 0..L"); return CKKS_E_INVALID; }
    return CKKS_OK;
}

}  // namespace

// rotGroups[idx] = 5^idx mod 2N (Context_23.cuh:648-659)
extern "C" int ckks_rot_group(const ckks_ctx* c, long idx, uint64_t* value) {
    if (!c || !value || idx < 0) { set_error("rotGroups: bad argument"); return CKKS_E_INVALID; }
    *value = H::powmod(5, (u64)idx, 2 * (u64)c->N);
    return CKKS_OK;
}

extern "C" int ckks_poly_automorph_ntt(ckks_ctx* c, uint64_t* out, const uint64_t* in, uint64_t pow, int idx_out, int idx_in, int mod_num) {
    if (!c || !out || !in || idx_out < 0 || idx_in < 0 || mod_num < 0) { set_error("sk_and_poly_LeftRot: bad argument"); return CKKS_E_INVALID; }
    if (!(pow & 1)) { set_error("sk_and_poly_LeftRot: the exponent must be odd"); return CKKS_E_INVALID; }
    if (out == in && idx_out == idx_in) { set_error("sk_and_poly_LeftRot: not in place"); return CKKS_E_INVALID; }
    if (mod_num == 0) return CKKS_OK;
    const long N = c->N;
    const u64 pow_inv = H::invmod(pow % (2 * (u64)N), 2 * (u64)N);
    hipLaunchKernelGGL(automorph_kernel, dim3(N / THREADS, mod_num, 1), dim3(THREADS), 0, c->stream, (u64*)out + (long)idx_out * N,
                       (const u64*)in + (long)idx_in * N, (const u64*)nullptr, c->d_primes, N, c->logN, pow_inv, 0, 0L, 0L, -1);
    CKKS_HIP_TRY(hipGetLastError());
    return CKKS_OK;
}

extern "C" int ckks_poly_conjugate_ntt(ckks_ctx* c, uint64_t* out, const uint64_t* in, int idx_out, int idx_in, int mod_num) {
    if (!c || !out || !in || idx_out < 0 || idx_in < 0 || mod_num < 0) { set_error("sk_and_poly_conjugate: bad argument"); return CKKS_E_INVALID; }
    if (out == in && idx_out == idx_in) { set_error("sk_and_poly_conjugate: not in place"); return CKKS_E_INVALID; }
    if (mod_num == 0) return CKKS_OK;
    const long N = c->N;
    hipLaunchKernelGGL(reverse_kernel, dim3(N / THREADS, mod_num), dim3(THREADS), 0, c->stream, (u64*)out + (long)idx_out * N,
                       (const u64*)in + (long)idx_in * N, N);
    CKKS_HIP_TRY(hipGetLastError());
    return CKKS_OK;
}

extern "C" int ckks_keygen_switch_23(ckks_ctx* c, uint64_t* swk, const uint64_t* s_to, const uint64_t* s_from, const uint8_t* random_a,
                                     const uint8_t* random_e, uint64_t* scratch) {
    int rc = need_t_basis(c, "addSWKey_23");
    if (rc != CKKS_OK) return rc;
    if (!swk || !s_to || !s_from || !random_a || !random_e || !scratch) { set_error("addSWKey_23: null argument"); return CKKS_E_INVALID; }
    const long N = c->N;
    const int K = c->K, L = c->L, T = c->t_num, RB = c->Ri_blockNum, dnum = c->dnum, KL = K + L + 1;
    if (RB * T < KL) { set_error("addSWKey_23: a key block (Ri_blockNum * t_num limbs) is smaller than K+L+1 limbs"); return CKKS_E_INVALID; }
    if (K > MAX_DIGIT_PRIMES) { set_error("addSWKey_23: more than 16 special primes"); return CKKS_E_INVALID; }
    const size_t digit = (size_t)N * T * RB;
    uint64_t* ax = swk;
    uint64_t* bx = swk + digit * dnum;
    for (int i = 0; i < dnum; i++) {
        DigitConst d;
        d.first_prime = K + i * K;
        d.count = 0;
        for (int t = 0; t < K && i * K + t <= L; t++) d.pmod[d.count++] = c->PModqt[i * K + t];
        if ((rc = ckks_sample_gaussian(c, random_e + (size_t)i * N * 4, scratch, 0, 0, KL))) return rc;
        if ((rc = launch_ntt(c, scratch, 0, 0, 1, KL, KL, 0, 1, false))) return rc;
        if ((rc = ckks_sample_uniform(c, random_a + (size_t)i * N * KL * 8, ax + digit * i, 0, 0, KL))) return rc;
        hipLaunchKernelGGL(swk_combine_kernel, dim3(N / THREADS, KL), dim3(THREADS), 0, c->stream, (u64*)(bx + digit * i), (const u64*)(ax + digit * i),
                           (const u64*)scratch, (const u64*)s_to, (const u64*)s_from, c->d_primes, N, K, d);
        CKKS_HIP_TRY(hipGetLastError());
    }
    // a and b of every digit to the coefficient domain in one call: 2*dnum polynomials of K+L+1 limbs, T*RB limbs apart (:54-55)
    if ((rc = launch_ntt(c, swk, 0, 0, 2 * dnum, KL, T * RB, 0, 1, true))) return rc;
    for (int i = 0; i < 2 * dnum; i++) {                                                             // :57-63
        uint64_t* part = swk + digit * i;
        CKKS_HIP_TRY(hipMemcpyAsync(scratch, part, 8 * (size_t)N * KL, hipMemcpyDeviceToDevice, c->stream));
        if ((rc = ckks_modup_pq_to_t(c, part, scratch, L, 1))) return rc;
    }
    return launch_ntt(c, swk, 0, KL, dnum * RB * 2, T, T, 0, 1, false);                                // :64
}

extern "C" int ckks_mult_23(ckks_ctx* c, uint64_t* out, const uint64_t* c1, const uint64_t* c2, const uint64_t* rlk, int l, uint64_t* work,
                            uint64_t* modUp_QjtoT_temp, uint64_t* exProduct_T_temp, uint64_t* modUp_TtoQj_buffer) {
    int rc = need_t_basis(c, "mult_23");
    if (rc != CKKS_OK) return rc;
    if (l == 0) { set_error("Ciphertexts are on level 0"); return CKKS_E_STATE; }                      // KeySwitch_23.cuh:194-197
    if (!rlk) { set_error("rotKey_23 not exists"); return CKKS_E_STATE; }                              // :198-201
    if ((rc = need_level(c, l, "mult_23"))) return rc;
    if (!out || !c1 || !c2 || !work) { set_error("mult_23: null argument"); return CKKS_E_INVALID; }
    const long N = c->N;
    const int K = c->K, L1 = c->L + 1;
    u64* axbx = (u64*)work;
    u64* axax = axbx + N * L1;
    u64* bxbx = axax + N * L1;
    hipLaunchKernelGGL(tensor_kernel, dim3(N / THREADS, l + 1), dim3(THREADS), 0, c->stream, axbx, axax, bxbx, (const u64*)c1, (const u64*)c2,
                       (const u64*)c1 + N * L1, (const u64*)c2 + N * L1, c->d_primes, N, K);
    CKKS_HIP_TRY(hipGetLastError());
    // out = KeySwitch(axax) + (axbx, bxbx) (:233-234): the additions ride on the last launch of the key switch where that is one of
    // the fused forms (axbx and bxbx lie 2 (L+1) limbs apart in the work area)
    bool added = false;
    if ((rc = keyswitch_23_add(c, out, axax, rlk, l, modUp_QjtoT_temp, exProduct_T_temp, modUp_TtoQj_buffer, (const uint64_t*)axbx, 2l * L1, &added))) return rc;
    if (added) return CKKS_OK;
    hipLaunchKernelGGL(add_pair_kernel, dim3(N / THREADS, l + 1), dim3(THREADS), 0, c->stream, (u64*)out, (u64*)out + N * L1, (const u64*)axbx,
                       (const u64*)bxbx, c->d_primes, N, K);
    CKKS_HIP_TRY(hipGetLastError());
    return CKKS_OK;
}

extern "C" int ckks_rotate_23(ckks_ctx* c, uint64_t* out, const uint64_t* cipher, const uint64_t* rotkey, long rot, int l, uint64_t* work,
                              uint64_t* modUp_QjtoT_temp, uint64_t* exProduct_T_temp, uint64_t* modUp_TtoQj_buffer) {
    int rc = need_t_basis(c, "leftRotate_23");
    if (rc != CKKS_OK) return rc;
    if (!rotkey) { set_error("rotKey_23 not exists"); return CKKS_E_STATE; }                           // KeySwitch_23.cuh:558-561
    if ((rc = need_level(c, l, "leftRotate_23"))) return rc;
    if (!out || !cipher || !work || out == cipher) { set_error("leftRotate_23: null argument or out == cipher"); return CKKS_E_INVALID; }
    const long N = c->N;
    if (rot < 0 || rot > N / 2) { set_error("leftRotate_23: rotation outside 0..N/2"); return CKKS_E_INVALID; }
    const int K = c->K, L1 = c->L + 1;
    u64* a_copy = (u64*)work;                      // the switch leaves its input in the coefficient domain (the reference transforms a back, :571)
    u64* tmp = a_copy + N * L1;                    // cipher_temp_pool
    CKKS_HIP_TRY(hipMemcpyAsync(a_copy, cipher, 8 * (size_t)N * (l + 1), hipMemcpyDeviceToDevice, c->stream));
    if ((rc = ckks_keyswitch_23(c, tmp, a_copy, rotkey, l, modUp_QjtoT_temp, exProduct_T_temp, modUp_TtoQj_buffer))) return rc;
    // (tmp.a, tmp.b + b) through the slot permutation with 5^(N/2 - rot) (:582-585): its inverse is 5^rot
    const u64 pow_inv = H::powmod(5, (u64)rot, 2 * (u64)N);
    hipLaunchKernelGGL(automorph_kernel, dim3(N / THREADS, l + 1, 2), dim3(THREADS), 0, c->stream, (u64*)out, (const u64*)tmp,
                       (const u64*)cipher + N * L1, c->d_primes, N, c->logN, pow_inv, K, N * L1, N * L1, 1);
    CKKS_HIP_TRY(hipGetLastError());
    return CKKS_OK;
}

extern "C" int ckks_conjugate_23(ckks_ctx* c, uint64_t* out, const uint64_t* cipher, const uint64_t* conjkey, int l, uint64_t* work,
                                 uint64_t* modUp_QjtoT_temp, uint64_t* exProduct_T_temp, uint64_t* modUp_TtoQj_buffer) {
    int rc = need_t_basis(c, "conjugate_23");
    if (rc != CKKS_OK) return rc;
    if (!conjkey) { set_error("conjKey_23 not exists"); return CKKS_E_STATE; }                         // KeySwitch_23.cuh:435-438
    if ((rc = need_level(c, l, "conjugate_23"))) return rc;
    if (!out || !cipher || !work || out == cipher) { set_error("conjugate_23: null argument or out == cipher"); return CKKS_E_INVALID; }
    const long N = c->N;
    const int K = c->K, L1 = c->L + 1;
    u64* a_rev = (u64*)work;
    hipLaunchKernelGGL(reverse_kernel, dim3(N / THREADS, l + 1), dim3(THREADS), 0, c->stream, a_rev, (const u64*)cipher, N);                 // :455
    CKKS_HIP_TRY(hipGetLastError());
    if ((rc = ckks_keyswitch_23(c, out, a_rev, conjkey, l, modUp_QjtoT_temp, exProduct_T_temp, modUp_TtoQj_buffer))) return rc;
    hipLaunchKernelGGL(add_reversed_kernel, dim3(N / THREADS, l + 1), dim3(THREADS), 0, c->stream, (u64*)out + N * L1, (const u64*)cipher + N * L1,
                       c->d_primes, N, K);                                                                                                   // :454, 467
    CKKS_HIP_TRY(hipGetLastError());
    return CKKS_OK;
}
