// Key side of the ring-packed PCMM for gfx950: the MLWE secret derived from the RLWE secret, the repacking keys that
// mlweCipherPacking consumes, and the MLWE decryption / decoding used to inspect the samples between the steps.
//
// Reference: PCMM_Scheme::convertMLWESKfromRLWESK (PCMM_Scheme.cuh:23-48) with ringDown_kernel (ringSwitch.cuh:7-19),
// PCMM_Scheme::addRepakcingKey (PCMM_Scheme.cuh:126-224) with EmbedMLWESKtoRLWESK (:126-149), PCMM_Scheme::mlweDecrypt (:531-576),
// PCMM_Context::decodeCoeffs (PCMM_Context.cuh:149-178).
//
// Per repacking key the reference runs nine launches; here a key is one random-stream launch, one fused sampling kernel (a, and
// e + p0 * iota(s_i) in the coefficient domain), one transform and one combining kernel.  The size-N1 transforms are
// pcmm_ntt_fwd / pcmm_ntt_inv, which run every power of two N1 (the reference's run N1 = 256 only).
#include <hip/hip_runtime.h>
#include <cmath>
#include <string>

#include "context.hpp"
#include "pcmm.hpp"

using namespace ckks;

namespace {

constexpr int THREADS = 256;

__device__ __forceinline__ u64 mulmod(u64 a, u64 b, const PrimeConst& p) {
    u128w acc{0, 0};
    mac128(acc, a, b);
    return barrett128(acc, p.q, p.mu_hi, p.mu_lo);
}

// small[im][g] = big[im][g / N1 + (g % N1) * rank]: small polynomial i = g / N1 takes the big coefficients i + n * rank
__global__ __launch_bounds__(THREADS) void ring_down_kernel(const u64* big, u64* small, long N, int N1, int rank) {
    const long g = (long)blockIdx.x * THREADS + threadIdx.x;
    const int im = blockIdx.y;
    small[(long)im * N + g] = big[(long)im * N + g / N1 + (g % N1) * (long)rank];
}

// steps of the discrete Gaussian (see the sampler of the scheme: thresholds on the 32-bit word)
struct GaussSteps {
    uint32_t thr[19];
};
__device__ __forceinline__ int gauss_value(uint32_t u, const GaussSteps& g) {
    int v = 0;
#pragma unroll
    for (int k = 0; k < 19; k++) {
        v += (u >= g.thr[k]);
        v -= (~u >= g.thr[k]);
    }
    return v;
}

// one repacking key, sampling half: a[t] uniform modulo prime first+t, b[t] = e + p0 * iota(s_i) (coefficient domain), where
// iota(s_i) has coefficient n of small secret i at position n * rank, on the q limbs only (EmbedMLWESKtoRLWESK, :126-149)
__global__ __launch_bounds__(THREADS) void repack_key_sample_kernel(u64* ax, u64* bx, const uint8_t* random, const u64* mlwe_sk_coeff, const PrimeConst* primes,
                                                                    const PrimeConst* pq, long N, int N1, int rank, int first, int np, int key, GaussSteps g) {
    const long x = (long)blockIdx.x * THREADS + threadIdx.x;
    const int t = blockIdx.y;
    const PrimeConst p = primes[first + t];
    const uint32_t* ew = (const uint32_t*)random;
    const u64* aw = (const u64*)(random + 4 * N);
    double d = (double)aw[(long)t * N + x];                                            // convert_uniform_xq (Sampler_impl.cuh:13-24)
    d /= 18446744073709551616.0;
    d *= (double)(p.q - 1);
    ax[(long)t * N + x] = (u64)d;
    const int e = gauss_value(ew[x], g);
    u64 v = e < 0 ? p.q + (long long)e : (u64)e;
    if (t >= np && x % rank == 0) {
        const u64 s = mlwe_sk_coeff[(long)t * N + (long)key * N1 + x / rank];            // modulus slot t = np + (t - np)
        v = csub(v + mulmod(s, pq[0].q, p), p.q);
    }
    bx[(long)t * N + x] = v;
}
// combining half: b = b - a * s (NTT domain), s = RLWE secret limbs first.. (:214-221)
__global__ __launch_bounds__(THREADS) void repack_key_combine_kernel(u64* bx, const u64* ax, const u64* sx, const PrimeConst* primes, long N, int first) {
    const long x = (long)blockIdx.x * THREADS + threadIdx.x;
    const int t = blockIdx.y;
    const PrimeConst p = primes[first + t];
    const long o = (long)t * N + x;
    bx[o] = csub(p.q + bx[o] - mulmod(sx[(long)(first + t) * N + x], ax[o], p), p.q);
}

// plain[im][n] = b + sum_i a_i * s_i (mlweDecrypt_kernel, :531-555): 128-bit accumulation, one Barrett reduction.
// A workgroup handles 64 coefficients; its 4 waves split the rank and combine through LDS.
__global__ __launch_bounds__(THREADS) void mlwe_decrypt_kernel(u64* plain, const u64* cipher_ntt, const u64* mlwe_sk, const PrimeConst* pq, int N1, int rank,
                                                               int np) {
    __shared__ u64 part[2][4][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n = blockIdx.x * 64 + lane;
    const int im = blockIdx.y;
    const PrimeConst p = pq[np + im];
    const u64* a = cipher_ntt + (long)im * (rank + 1) * N1;
    const u64* s = mlwe_sk + (long)(np + im) * rank * N1;
    u128w acc{0, 0};
    for (int i = wave; i < rank; i += 4) mac128(acc, a[(long)i * N1 + n], s[(long)i * N1 + n]);
    part[0][wave][lane] = acc.lo;
    part[1][wave][lane] = acc.hi;
    __syncthreads();
    if (wave == 0) {
        u128w tot{a[(long)rank * N1 + n], 0};
        for (int w = 0; w < 4; w++) {
            const u64 lo = part[0][w][lane], hi = part[1][w][lane];
            tot.lo += lo;
            tot.hi += hi + (tot.lo < lo);
        }
        plain[(long)im * N1 + n] = barrett128(tot, p.q, p.mu_hi, p.mu_lo);
    }
}

// MLWEDecodeCoeffs_kernel (PCMM_Context.cuh:149-163): centred residue modulo the first ring-pack modulus over the scale
__global__ __launch_bounds__(THREADS) void mlwe_decode_kernel(double* vals, const u64* coeff, u64 mod, long long scaler, int N1) {
    const int n = blockIdx.x * THREADS + threadIdx.x;
    if (n >= N1) return;
    const u64 mi = coeff[n];
    vals[n] = mi <= (mod >> 1) ? (double)(long long)mi / (double)scaler : ((double)(long long)mi - (double)mod) / (double)scaler;
}

int shape_ok(pcmm_ctx* h, const char* who) {
    if (!h || !h->ctx) { set_error(std::string(who) + ": null handle"); return CKKS_E_INVALID; }
    if ((long)h->N1 * h->rank != h->ctx->N) { set_error(std::string(who) + ": N1 * rank must be N"); return CKKS_E_INVALID; }
    if (h->N1 % 64) { set_error(std::string(who) + ": N1 must be a multiple of 64"); return CKKS_E_INVALID; }
    return CKKS_OK;
}

}  // namespace

extern "C" int pcmm_convert_mlwe_sk(pcmm_ctx* h, uint64_t* mlwe_sk, uint64_t* rlwe_sk) {
    int rc = shape_ok(h, "convertMLWESKfromRLWESK");
    if (rc != CKKS_OK) return rc;
    if (!mlwe_sk || !rlwe_sk) { set_error("convertMLWESKfromRLWESK: null argument"); return CKKS_E_INVALID; }
    ckks_ctx* c = h->ctx;
    const long N = c->N;
    const int K = c->K, KL = c->K + c->L + 1, np = h->np, nq = h->nq;
    if (nq > KL || K + nq > KL) { set_error("convertMLWESKfromRLWESK: more ring-pack moduli than limbs of the secret"); return CKKS_E_INVALID; }
    if ((rc = launch_ntt(c, rlwe_sk, 0, 0, 1, KL, KL, 0, 1, true))) return rc;                       // :38
    // the reference's two launches (:40-43): RLWE limbs 0.. to key moduli 0.., then RLWE limbs K.. to key moduli np..
    hipLaunchKernelGGL(ring_down_kernel, dim3(N / THREADS, nq), dim3(THREADS), 0, c->stream, (const u64*)rlwe_sk, (u64*)mlwe_sk, N, h->N1, h->rank);
    hipLaunchKernelGGL(ring_down_kernel, dim3(N / THREADS, nq), dim3(THREADS), 0, c->stream, (const u64*)rlwe_sk + (long)K * N,
                       (u64*)mlwe_sk + (long)np * N, N, h->N1, h->rank);
    CKKS_HIP_TRY(hipGetLastError());
    if ((rc = launch_ntt(c, rlwe_sk, 0, 0, 1, KL, KL, 0, 1, false))) return rc;                      // :45
    return pcmm_ntt_fwd(h, mlwe_sk, h->rank, np + nq, 0, 0, 1);                                      // :47
}

extern "C" int pcmm_add_repacking_key(pcmm_ctx* h, uint64_t* keys, uint64_t* mlwe_sk, const uint64_t* rlwe_sk, const uint8_t* key32, uint64_t nonce,
                                      uint64_t* scratch) {
    int rc = shape_ok(h, "addRepakcingKey");
    if (rc != CKKS_OK) return rc;
    if (!keys || !mlwe_sk || !rlwe_sk || !key32 || !scratch) { set_error("addRepakcingKey: null argument"); return CKKS_E_INVALID; }
    ckks_ctx* c = h->ctx;
    const long N = c->N;
    const int K = c->K, np = h->np, nq = h->nq, mod_num = np + nq - 1, first = K - np;
    if (K < np || (nq - 1) / np != 1) { set_error("addRepakcingKey: dnum not supported!"); return CKKS_E_INVALID; }            // :178-180
    for (int i = 0; i < mod_num; i++)
        if (c->pqt[first + i] != h->pq[i]) { set_error("addRepakcingKey: the ring-pack primes are not the context's last special primes and first moduli"); return CKKS_E_INVALID; }
    // steps of the Gaussian: the same table as the scheme's sampler (2^32 - round(2^32 * Q(k / 3.2)))
    GaussSteps g;
    for (int k = 1; k <= 19; k++) {
        const double tail = 0.5 * std::erfc(((double)k / 3.2) / std::sqrt(2.0));
        g.thr[k - 1] = (uint32_t)(4294967296.0 - std::floor(4294967296.0 * tail + 0.5));
    }
    if ((rc = pcmm_ntt_inv(h, mlwe_sk, h->rank, np + nq, 0, 0, 1))) return rc;                        // :159
    uint8_t* rnd = (uint8_t*)scratch;
    const size_t per_key = (size_t)4 * N + (size_t)8 * N * mod_num;
    for (int i = 0; i < h->rank; i++) {
        uint64_t* ax = keys + (size_t)i * 2 * mod_num * N;
        uint64_t* bx = ax + (size_t)mod_num * N;
        if ((rc = ckks_random_bytes(c, rnd, per_key, key32, nonce + (uint64_t)i))) return rc;
        hipLaunchKernelGGL(repack_key_sample_kernel, dim3(N / THREADS, mod_num), dim3(THREADS), 0, c->stream, (u64*)ax, (u64*)bx, (const uint8_t*)rnd,
                           (const u64*)mlwe_sk, c->d_primes, h->d_pq, N, h->N1, h->rank, first, np, i, g);
        CKKS_HIP_TRY(hipGetLastError());
        if ((rc = launch_ntt(c, bx, 0, first, 1, mod_num, mod_num, 0, 1, false))) return rc;          // :211
        hipLaunchKernelGGL(repack_key_combine_kernel, dim3(N / THREADS, mod_num), dim3(THREADS), 0, c->stream, (u64*)bx, (const u64*)ax, (const u64*)rlwe_sk,
                           c->d_primes, N, first);
        CKKS_HIP_TRY(hipGetLastError());
    }
    // every modulus of the MLWE secret back to the NTT domain (the reference leaves the last one behind, :182)
    return pcmm_ntt_fwd(h, mlwe_sk, h->rank, np + nq, 0, 0, 1);
}

extern "C" int pcmm_mlwe_decrypt(pcmm_ctx* h, uint64_t* plain, uint64_t* mlwe_cipher, const uint64_t* mlwe_sk, int l) {
    int rc = shape_ok(h, "mlweDecrypt");
    if (rc != CKKS_OK) return rc;
    if (!plain || !mlwe_cipher || !mlwe_sk) { set_error("mlweDecrypt: null argument"); return CKKS_E_INVALID; }
    if (l < 0 || l + 1 > h->nq) { set_error("mlweDecrypt: level outside the ring-pack moduli"); return CKKS_E_INVALID; }
    ckks_ctx* c = h->ctx;
    if ((rc = pcmm_ntt_fwd(h, mlwe_cipher, h->rank + 1, l + 1, 0, h->np, 1))) return rc;              // :566
    hipLaunchKernelGGL(mlwe_decrypt_kernel, dim3(h->N1 / 64, l + 1), dim3(THREADS), 0, c->stream, (u64*)plain, (const u64*)mlwe_cipher, (const u64*)mlwe_sk,
                       h->d_pq, h->N1, h->rank, h->np);
    CKKS_HIP_TRY(hipGetLastError());
    return pcmm_ntt_inv(h, mlwe_cipher, h->rank + 1, l + 1, 0, h->np, 1);                             // :575
}

extern "C" int pcmm_decode_coeffs(pcmm_ctx* h, double* vals, const uint64_t* plain, uint64_t* scratch, long long scaler, int l) {
    int rc = shape_ok(h, "decodeCoeffs");
    if (rc != CKKS_OK) return rc;
    if (!vals || !plain || !scratch || scaler == 0) { set_error("decodeCoeffs: null argument or zero scale"); return CKKS_E_INVALID; }
    if (l < 0 || l + 1 > h->nq) { set_error("decodeCoeffs: level outside the ring-pack moduli"); return CKKS_E_INVALID; }
    ckks_ctx* c = h->ctx;
    CKKS_HIP_TRY(hipMemcpyAsync(scratch, plain, 8 * (size_t)h->N1 * (l + 1), hipMemcpyDeviceToDevice, c->stream));       // :175
    if ((rc = pcmm_ntt_inv(h, scratch, 1, l + 1, 0, h->np, 1))) return rc;                            // :176
    hipLaunchKernelGGL(mlwe_decode_kernel, dim3((h->N1 + THREADS - 1) / THREADS), dim3(THREADS), 0, c->stream, vals, (const u64*)scratch, h->pq[h->np], scaler,
                       h->N1);
    CKKS_HIP_TRY(hipGetLastError());
    return CKKS_OK;
}
