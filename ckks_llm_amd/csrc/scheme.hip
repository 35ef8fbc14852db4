// Randomness, samplers, pointwise limb arithmetic, key generation, encryption / decryption and coefficient encoding for gfx950:
// the steps either side of the NTT -> key switch -> PCMM path that a client of the scheme runs.
//
// Reference: RNG.cuh:18-56 + RNG_impl.cuh:72-176 (Salsa20 stream), Sampler.cuh:17-54 + Sampler_impl.cuh:13-119 (conversions),
// poly_arithmetic.cuh:101-105,395-485 (pointwise), SecretKey.cuh:18-31, Scheme_23.cuh:54-127 (keys, encryption),
// Encoder.cuh:67-186 (coefficient encode / decode).
//
// The reference issues one small launch per sampler and per pointwise step; here a key or a ciphertext is produced by one sampling
// kernel, the batched transforms, and one combining kernel.  All of it is HBM-bound streaming work: every lane handles one
// coefficient of every limb of a call, 8-byte accesses coalesced along the coefficient index.
#include <hip/hip_runtime.h>
#include <cmath>
#include <cstring>
#include <string>
#include <vector>

#include "context.hpp"
#include "host_math.hpp"

using namespace ckks;
namespace H = ckks_host;

namespace {

constexpr int THREADS = 256;

// ---------------------------------------------------------------------------------------------------------------------------------
// Salsa20/20 key stream: one lane per 64-byte block
// ---------------------------------------------------------------------------------------------------------------------------------
struct SalsaKey {
    uint32_t k[8];
};

__device__ __forceinline__ uint32_t rotl(uint32_t u, int c) { return (u << c) | (u >> (32 - c)); }

__global__ __launch_bounds__(THREADS) void salsa20_kernel(uint8_t* out, size_t n_bytes, SalsaKey key, uint64_t nonce) {
    const size_t blk = (size_t)blockIdx.x * THREADS + threadIdx.x;
    if (blk * 64 >= n_bytes) return;
    uint32_t j[16], x[16];
    j[0] = 0x61707865u; j[5] = 0x3320646eu; j[10] = 0x79622d32u; j[15] = 0x6b206574u;     // "expand 32-byte k"
#pragma unroll
    for (int i = 0; i < 4; i++) { j[1 + i] = key.k[i]; j[11 + i] = key.k[4 + i]; }
    j[6] = (uint32_t)nonce; j[7] = (uint32_t)(nonce >> 32);
    j[8] = (uint32_t)blk; j[9] = (uint32_t)((uint64_t)blk >> 32);
#pragma unroll
    for (int i = 0; i < 16; i++) x[i] = j[i];
#define QR(a, b, c, d)                 \
    x[b] ^= rotl(x[a] + x[d], 7);      \
    x[c] ^= rotl(x[b] + x[a], 9);      \
    x[d] ^= rotl(x[c] + x[b], 13);     \
    x[a] ^= rotl(x[d] + x[c], 18);
    for (int r = 0; r < 10; r++) {
        QR(0, 4, 8, 12) QR(5, 9, 13, 1) QR(10, 14, 2, 6) QR(15, 3, 7, 11)
        QR(0, 1, 2, 3) QR(5, 6, 7, 4) QR(10, 11, 8, 9) QR(15, 12, 13, 14)
    }
#undef QR
#pragma unroll
    for (int i = 0; i < 16; i++) x[i] += j[i];
    uint8_t* dst = out + blk * 64;
    if (blk * 64 + 64 <= n_bytes && (((uintptr_t)dst) & 15) == 0) {
        uint4* d4 = (uint4*)dst;
#pragma unroll
        for (int i = 0; i < 4; i++) d4[i] = make_uint4(x[4 * i], x[4 * i + 1], x[4 * i + 2], x[4 * i + 3]);
    } else {
        const size_t take = n_bytes - blk * 64 < 64 ? n_bytes - blk * 64 : 64;
        for (size_t b = 0; b < take; b++) dst[b] = (uint8_t)(x[b >> 2] >> (8 * (b & 3)));
    }
}

// ---------------------------------------------------------------------------------------------------------------------------------
// conversions of random bytes
// ---------------------------------------------------------------------------------------------------------------------------------
// Steps of the discrete Gaussian as thresholds on the 32-bit word: value >= k  <=>  u >= thr[k-1], k = 1..19; the negative side is
// the mirror image u -> ~u.  thr[k-1] = 2^32 - floor(2^32 * Q(k / 3.2) + 0.5) with Q the upper normal tail, i.e. the probability of a
// word is taken at the middle of its cell.  convert_gaussian_xq (Sampler_impl.cuh:27-70) evaluates the same step function in float
// arithmetic (trunc(3.2 * normcdfinvf(u / (2^32-1))), clamped to +-19.2); the two differ only for words within float rounding of a
// step, and an integer rule is the same on every machine.
struct GaussSteps {
    uint32_t thr[19];
};
const GaussSteps& gauss_steps() {
    static GaussSteps g = [] {
        GaussSteps s;
        for (int k = 1; k <= 19; k++) {
            const double tail = 0.5 * std::erfc(((double)k / 3.2) / std::sqrt(2.0));
            s.thr[k - 1] = (uint32_t)(4294967296.0 - std::floor(4294967296.0 * tail + 0.5));
        }
        return s;
    }();
    return g;
}
__device__ __forceinline__ int gauss_value(uint32_t u, const GaussSteps& g) {
    int v = 0;
#pragma unroll
    for (int k = 0; k < 19; k++) {
        v += (u >= g.thr[k]);
        v -= (~u >= g.thr[k]);
    }
    return v;
}
__device__ __forceinline__ u64 signed_residue(int v, u64 q) { return v < 0 ? q + (long long)v : (u64)v; }
__device__ __forceinline__ u64 zo_value(uint8_t byte, double t0, double t1, u64 q) {   // Sampler_impl.cuh:96-113
    const double d = (double)byte;
    return d < t0 ? 0 : (d < t1 ? 1 : q - 1);
}
__device__ __forceinline__ u64 uniform_value(u64 w, u64 q) {                            // Sampler_impl.cuh:13-24
    double d = (double)w;
    d /= 18446744073709551616.0;
    d *= (double)(q - 1);
    return (u64)d;
}
__device__ __forceinline__ u64 mulmod(u64 a, u64 b, const PrimeConst& p) {
    u128w acc{0, 0};
    mac128(acc, a, b);
    return barrett128(acc, p.q, p.mu_hi, p.mu_lo);
}

__global__ __launch_bounds__(THREADS) void sample_uniform_kernel(const u64* random, u64* out, const PrimeConst* primes, long N, int idx_mod) {
    const long i = (long)blockIdx.x * THREADS + threadIdx.x;
    const int t = blockIdx.y;
    out[(long)t * N + i] = uniform_value(random[(long)t * N + i], primes[idx_mod + t].q);
}
__global__ __launch_bounds__(THREADS) void sample_gaussian_kernel(const uint32_t* random, u64* out, const PrimeConst* primes, long N, int idx_mod,
                                                                  int mod_num, GaussSteps g) {
    const long i = (long)blockIdx.x * THREADS + threadIdx.x;
    const int v = gauss_value(random[i], g);
    for (int t = 0; t < mod_num; t++) out[(long)t * N + i] = signed_residue(v, primes[idx_mod + t].q);
}
__global__ __launch_bounds__(THREADS) void sample_zo_kernel(const uint8_t* random, u64* out, const PrimeConst* primes, long N, int idx_mod, int mod_num,
                                                            double t0, double t1) {
    const long i = (long)blockIdx.x * THREADS + threadIdx.x;
    const uint8_t b = random[i];
    for (int t = 0; t < mod_num; t++) out[(long)t * N + i] = zo_value(b, t0, t1, primes[idx_mod + t].q);
}
// Sparse ternary polynomial (convert_HWT, Sampler_impl.cuh:74-93): one workgroup per limb zeroes it, then lane k < h writes the
// sign of word k at its position unless a later word names the same position (the later one wins; the reference leaves that to
// a race).
__global__ __launch_bounds__(THREADS) void sample_hwt_kernel(const uint8_t* random, u64* out, const PrimeConst* primes, long N, int h, int idx_mod) {
    const int t = blockIdx.x;
    u64* limb = out + (long)t * N;
    const u64 q = primes[idx_mod + t].q;
    for (long i = threadIdx.x; i < N; i += THREADS) limb[i] = 0;
    __syncthreads();
    const uint32_t* words = (const uint32_t*)random;
    const uint8_t* signs = random + 4 * (long)h;
    for (int k = threadIdx.x; k < h; k += THREADS) {
        const uint32_t pos = words[k] & (uint32_t)(N - 1);
        bool last = true;
        for (int k2 = k + 1; k2 < h; k2++) last = last && ((words[k2] & (uint32_t)(N - 1)) != pos);
        if (last) limb[pos] = signs[k] >= 128 ? 1 : q - 1;
    }
}

// ---------------------------------------------------------------------------------------------------------------------------------
// pointwise arithmetic on limbs
// ---------------------------------------------------------------------------------------------------------------------------------
template <int OP>
__global__ __launch_bounds__(THREADS) void poly_op_kernel(u64* c, const u64* a, const u64* b, const PrimeConst* primes, long N, int idx_mod) {
    const long i = (long)blockIdx.x * THREADS + threadIdx.x;
    const int t = blockIdx.y;
    const PrimeConst p = primes[idx_mod + t];
    const u64 x = a[(long)t * N + i], y = b[(long)t * N + i];
    u64 r;
    if (OP == 0) r = mulmod(x, y, p);
    else if (OP == 1) r = csub(x + y, p.q);
    else r = csub(p.q + x - y, p.q);
    c[(long)t * N + i] = r;
}

// pk.b = e - a*s (Scheme_23.cuh:75-76), e already in pk.b
__global__ __launch_bounds__(THREADS) void pk_combine_kernel(u64* bx, const u64* ax, const u64* sx, const PrimeConst* primes, long N, int K) {
    const long i = (long)blockIdx.x * THREADS + threadIdx.x;
    const int t = blockIdx.y;
    const PrimeConst p = primes[K + t];
    const u64 as = mulmod(ax[(long)t * N + i], sx[(long)(K + t) * N + i], p);
    bx[(long)t * N + i] = csub(p.q + bx[(long)t * N + i] - as, p.q);
}

// encryption, sampling half: e0 -> a, e1 -> b (limbs 0..l of each), v -> scratch (Scheme_23.cuh:89,94,100)
__global__ __launch_bounds__(THREADS) void encrypt_sample_kernel(const uint8_t* random, u64* ax, u64* bx, u64* vx, const PrimeConst* primes, long N, int K,
                                                                 int limbs, GaussSteps g) {
    const long i = (long)blockIdx.x * THREADS + threadIdx.x;
    const uint8_t zb = random[i];
    const uint32_t* w = (const uint32_t*)(random + N);
    const int e0 = gauss_value(w[i], g), e1 = gauss_value(w[N + i], g);
    for (int t = 0; t < limbs; t++) {
        const u64 q = primes[K + t].q;
        vx[(long)t * N + i] = zo_value(zb, 128.0, 192.0, q);
        ax[(long)t * N + i] = signed_residue(e0, q);
        bx[(long)t * N + i] = signed_residue(e1, q);
    }
}
// encryption, combining half: a = v*pk.a + e0, b = v*pk.b + e1 (+ m) (Scheme_23.cuh:92-111)
__global__ __launch_bounds__(THREADS) void encrypt_combine_kernel(u64* ax, u64* bx, const u64* vx, const u64* pka, const u64* pkb, const u64* mx,
                                                                  const PrimeConst* primes, long N, int K) {
    const long i = (long)blockIdx.x * THREADS + threadIdx.x;
    const int t = blockIdx.y;
    const PrimeConst p = primes[K + t];
    const long o = (long)t * N + i;
    const u64 v = vx[o];
    ax[o] = csub(mulmod(v, pka[o], p) + ax[o], p.q);
    u64 b = csub(mulmod(v, pkb[o], p) + bx[o], p.q);
    if (mx) b = csub(b + mx[o], p.q);
    bx[o] = b;
}
// decryption: m = a*s + b on limbs 0..l, zero above (Scheme_23.cuh:124-126)
__global__ __launch_bounds__(THREADS) void decrypt_kernel(u64* mx, const u64* ax, const u64* bx, const u64* sx, const PrimeConst* primes, long N, int K,
                                                          int limbs) {
    const long i = (long)blockIdx.x * THREADS + threadIdx.x;
    const int t = blockIdx.y;
    const long o = (long)t * N + i;
    if (t >= limbs) { mx[o] = 0; return; }
    const PrimeConst p = primes[K + t];
    mx[o] = csub(mulmod(ax[o], sx[(long)(K + t) * N + i], p) + bx[o], p.q);
}

// ---------------------------------------------------------------------------------------------------------------------------------
// coefficient encoding
// ---------------------------------------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(THREADS) void encode_coeffs_kernel(u64* mx, const double* vals, const PrimeConst* primes, long N, int K, long scale) {
    const long i = (long)blockIdx.x * THREADS + threadIdx.x;
    const int t = blockIdx.y;
    const long long q = (long long)primes[K + t].q;
    const long long data = (long long)(vals[i] * (double)scale);           // Encoder.cuh:75
    const long long r = data % q;
    mx[(long)t * N + i] = r < 0 ? (u64)(r + q) : (u64)r;
}

// Decoding table of one level (device words): w[i][j] = q_0..q_{j-1} mod q_i (row i, j < i), then cinv[i] = (q_0..q_{i-1})^-1 mod q_i,
// then Q = q_0..q_l and floor(Q/2) as little-endian words.
constexpr int DECODE_MAX_LIMBS = 64;

// CRT of one coefficient to the centred integer modulo Q, then to the nearest double, divided by the scale (Encoder.cuh:128-180,
// NTL::ZZ there).  Garner's mixed-radix digits v_i (x = v_0 + v_1 q_0 + v_2 q_0 q_1 + ...) come first, Horner's rule over them gives x
// as W machine words, x > floor(Q/2) is replaced by Q - x with a sign, and the top 64 significant bits plus a sticky bit round
// correctly into the double.
template <int W>
__global__ __launch_bounds__(THREADS) void decode_coeffs_kernel(double* vals, const u64* coeff, const PrimeConst* primes, const u64* tab, long N, int logN,
                                                                int K, int limbs, int gap, double scale, int is_bitrev) {
    const long idx = (long)blockIdx.x * THREADS + threadIdx.x;
    long o = idx;
    if (is_bitrev) o = (long)(__brev((uint32_t)idx) >> (32 - logN));
    if (idx % gap) { vals[o] = 0.0; return; }                      // only coefficients j*gap and N/2 + j*gap are produced (:163-177)
    const u64* wtab = tab;
    const u64* cinv = tab + (long)limbs * limbs;
    const u64* Qw = cinv + limbs;
    const u64* Qh = Qw + W;
    u64 v[DECODE_MAX_LIMBS];
    v[0] = coeff[idx];
    for (int i = 1; i < limbs; i++) {
        const PrimeConst p = primes[K + i];
        u64 acc = 0;
        for (int j = 0; j < i; j++) {
            u64 vj = v[j];
            if (vj >= p.q) vj = barrett64(vj, p.q, p.mu_hi);
            acc = csub(acc + mulmod(vj, wtab[(long)i * limbs + j], p), p.q);
        }
        const u64 diff = csub(p.q + coeff[(long)i * N + idx] - acc, p.q);
        v[i] = mulmod(diff, cinv[i], p);
    }
    u64 x[W];
#pragma unroll
    for (int w = 0; w < W; w++) x[w] = 0;
    x[0] = v[limbs - 1];
    for (int i = limbs - 2; i >= 0; i--) {
        const u64 q = primes[K + i].q;
        u64 carry = v[i];
#pragma unroll
        for (int w = 0; w < W; w++) {
            const u64 lo = x[w] * q, hi = __umul64hi(x[w], q);
            const u64 sum = lo + carry;
            carry = hi + (sum < lo);
            x[w] = sum;
        }
    }
    // x > floor(Q/2) ?
    bool greater = false, decided = false;
#pragma unroll
    for (int w = W - 1; w >= 0; w--) {
        const u64 h = Qh[w];
        if (!decided && x[w] != h) { greater = x[w] > h; decided = true; }
    }
    if (greater) {
        u64 borrow = 0;
#pragma unroll
        for (int w = 0; w < W; w++) {
            const u64 qv = Qw[w];
            const u64 d1 = qv - x[w];
            const u64 b1 = qv < x[w];
            const u64 d2 = d1 - borrow;
            const u64 b2 = d1 < borrow;
            x[w] = d2;
            borrow = b1 | b2;
        }
    }
    // top word, the word below it, sticky bits
    u64 top = 0, next = 0;
    bool sticky = false;
    int k = 0;
    bool found = false;
#pragma unroll
    for (int w = W - 1; w >= 0; w--) {
        if (!found) {
            if (x[w] != 0) { found = true; top = x[w]; k = w; next = w > 0 ? x[w - 1] : 0; }
        } else if (w < k - 1) {
            sticky = sticky || x[w] != 0;
        }
    }
    double d = 0.0;
    if (found) {
        const int lz = __clzll((long long)top);
        u64 m = top << lz;
        if (lz) { m |= next >> (64 - lz); sticky = sticky || (next << lz) != 0; } else { sticky = sticky || next != 0; }
        if (sticky) m |= 1;
        d = ldexp(__ull2double_rn(m), 64 * k - lz);
        if (greater) d = -d;
    }
    d /= scale;
    if (is_bitrev) d *= 256;                                       // Encoder.cuh:171-173
    vals[o] = d;
}

int check_limbs(ckks_ctx* c, const void* a, const void* b, int idx_out, int idx_mod, int mod_num, const char* who) {
    if (!c || !a || !b) { set_error(std::string(who) + ": null argument"); return CKKS_E_INVALID; }
    if (idx_out < 0 || idx_mod < 0 || mod_num < 0 || idx_mod + mod_num > c->nprimes) {
        set_error(std::string(who) + ": prime range outside the context");
        return CKKS_E_INVALID;
    }
    return CKKS_OK;
}
int check_level(ckks_ctx* c, int l, const char* who) {
    if (!c) { set_error(std::string(who) + ": null context"); return CKKS_E_INVALID; }
    if (l < 0 || l > c->L) { set_error(std::string(who) + ": level outside 0..L"); return CKKS_E_INVALID; }
    return CKKS_OK;
}

// multiword helpers for the decoding table (little-endian words)
void big_mul_word(std::vector<u64>& x, u64 m) {
    u64 carry = 0;
    for (auto& w : x) {
        const u128 t = (u128)w * m + carry;
        w = (u64)t;
        carry = (u64)(t >> 64);
    }
    if (carry) x.push_back(carry);
}

}  // namespace

// ---------------------------------------------------------------------------------------------------------------------------------
// C ABI
// ---------------------------------------------------------------------------------------------------------------------------------
extern "C" int ckks_random_bytes(ckks_ctx* c, uint8_t* dev, size_t n_bytes, const uint8_t* key32, uint64_t nonce) {
    if (!c || !dev || !key32) { set_error("ckks_random_bytes: null argument"); return CKKS_E_INVALID; }
    if (n_bytes == 0) return CKKS_OK;
    SalsaKey k;
    std::memcpy(k.k, key32, 32);
    const size_t blocks = (n_bytes + 63) / 64;
    const size_t grid = (blocks + THREADS - 1) / THREADS;
    if (grid > 0x7fffffffull) { set_error("ckks_random_bytes: more than 2^37 bytes in one call"); return CKKS_E_INVALID; }
    hipLaunchKernelGGL(salsa20_kernel, dim3((unsigned)grid), dim3(THREADS), 0, c->stream, dev, n_bytes, k, nonce);
    CKKS_HIP_TRY(hipGetLastError());
    return CKKS_OK;
}

extern "C" int ckks_sample_uniform(ckks_ctx* c, const uint8_t* random, uint64_t* out, int idx_out, int idx_mod, int mod_num) {
    int rc = check_limbs(c, random, out, idx_out, idx_mod, mod_num, "uniformSampler_xq");
    if (rc != CKKS_OK || mod_num == 0) return rc;
    if (((uintptr_t)random) & 7) { set_error("uniformSampler_xq: random words must be 8-byte aligned"); return CKKS_E_INVALID; }
    hipLaunchKernelGGL(sample_uniform_kernel, dim3(c->N / THREADS, mod_num), dim3(THREADS), 0, c->stream, (const u64*)random,
                       (u64*)out + (long)idx_out * c->N, c->d_primes, c->N, idx_mod);
    CKKS_HIP_TRY(hipGetLastError());
    return CKKS_OK;
}

extern "C" int ckks_sample_gaussian(ckks_ctx* c, const uint8_t* random, uint64_t* out, int idx_out, int idx_mod, int mod_num) {
    int rc = check_limbs(c, random, out, idx_out, idx_mod, mod_num, "gaussianSampler_xq");
    if (rc != CKKS_OK || mod_num == 0) return rc;
    if (((uintptr_t)random) & 3) { set_error("gaussianSampler_xq: random words must be 4-byte aligned"); return CKKS_E_INVALID; }
    hipLaunchKernelGGL(sample_gaussian_kernel, dim3(c->N / THREADS), dim3(THREADS), 0, c->stream, (const uint32_t*)random,
                       (u64*)out + (long)idx_out * c->N, c->d_primes, c->N, idx_mod, mod_num, gauss_steps());
    CKKS_HIP_TRY(hipGetLastError());
    return CKKS_OK;
}

extern "C" int ckks_sample_zo(ckks_ctx* c, const uint8_t* random, uint64_t* out, double probability, int idx_out, int idx_mod, int mod_num) {
    int rc = check_limbs(c, random, out, idx_out, idx_mod, mod_num, "ZOSampler");
    if (rc != CKKS_OK || mod_num == 0) return rc;
    const double t0 = 256.0f * probability, t1 = 256.0f * (1 + probability) / 2;       // Sampler_impl.cuh:106-109
    hipLaunchKernelGGL(sample_zo_kernel, dim3(c->N / THREADS), dim3(THREADS), 0, c->stream, random, (u64*)out + (long)idx_out * c->N,
                       c->d_primes, c->N, idx_mod, mod_num, t0, t1);
    CKKS_HIP_TRY(hipGetLastError());
    return CKKS_OK;
}

extern "C" int ckks_sample_hwt(ckks_ctx* c, const uint8_t* random, uint64_t* out, int h, int idx_out, int idx_mod, int mod_num) {
    int rc = check_limbs(c, random, out, idx_out, idx_mod, mod_num, "HWTSampler");
    if (rc != CKKS_OK || mod_num == 0) return rc;
    if (h < 0 || h > c->N) { set_error("HWTSampler: h outside 0..N"); return CKKS_E_INVALID; }
    if (((uintptr_t)random) & 3) { set_error("HWTSampler: random words must be 4-byte aligned"); return CKKS_E_INVALID; }
    // the reference's output offset includes idx_mod (Sampler_impl.cuh:89-92)
    hipLaunchKernelGGL(sample_hwt_kernel, dim3(mod_num), dim3(THREADS), 0, c->stream, random, (u64*)out + (long)(idx_out + idx_mod) * c->N,
                       c->d_primes, c->N, h, idx_mod);
    CKKS_HIP_TRY(hipGetLastError());
    return CKKS_OK;
}

static int poly_op(ckks_ctx* c, int op, uint64_t* out, const uint64_t* a, const uint64_t* b, int idx_c, int idx_a, int idx_b, int idx_mod,
                   int mod_num, const char* who) {
    int rc = check_limbs(c, a, b, idx_c, idx_mod, mod_num, who);
    if (rc != CKKS_OK) return rc;
    if (!out || idx_a < 0 || idx_b < 0) { set_error(std::string(who) + ": bad operand"); return CKKS_E_INVALID; }
    if (mod_num == 0) return CKKS_OK;
    const long N = c->N;
    dim3 grid(N / THREADS, mod_num), block(THREADS);
    u64* pc = (u64*)out + (long)idx_c * N;
    const u64* pa = (const u64*)a + (long)idx_a * N;
    const u64* pb = (const u64*)b + (long)idx_b * N;
    if (op == 0) hipLaunchKernelGGL(poly_op_kernel<0>, grid, block, 0, c->stream, pc, pa, pb, c->d_primes, N, idx_mod);
    else if (op == 1) hipLaunchKernelGGL(poly_op_kernel<1>, grid, block, 0, c->stream, pc, pa, pb, c->d_primes, N, idx_mod);
    else hipLaunchKernelGGL(poly_op_kernel<2>, grid, block, 0, c->stream, pc, pa, pb, c->d_primes, N, idx_mod);
    CKKS_HIP_TRY(hipGetLastError());
    return CKKS_OK;
}
extern "C" int ckks_poly_mul(ckks_ctx* c, uint64_t* out, const uint64_t* a, const uint64_t* b, int idx_c, int idx_a, int idx_b, int idx_mod,
                             int mod_num) {
    return poly_op(c, 0, out, a, b, idx_c, idx_a, idx_b, idx_mod, mod_num, "barrett_batch_3param_device");
}
extern "C" int ckks_poly_add(ckks_ctx* c, uint64_t* out, const uint64_t* a, const uint64_t* b, int idx_c, int idx_a, int idx_b, int idx_mod,
                             int mod_num) {
    return poly_op(c, 1, out, a, b, idx_c, idx_a, idx_b, idx_mod, mod_num, "poly_add_3param_batch_device");
}
extern "C" int ckks_poly_sub(ckks_ctx* c, uint64_t* out, const uint64_t* a, const uint64_t* b, int idx_c, int idx_a, int idx_b, int idx_mod,
                             int mod_num) {
    return poly_op(c, 2, out, a, b, idx_c, idx_a, idx_b, idx_mod, mod_num, "poly_sub_3param_batch_device");
}

extern "C" int ckks_keygen_secret(ckks_ctx* c, uint64_t* sx, const uint8_t* random, int h) {
    if (!c) { set_error("SecretKey: null context"); return CKKS_E_INVALID; }
    const int KL = c->K + c->L + 1;
    int rc = ckks_sample_hwt(c, random, sx, h, 0, 0, KL);
    if (rc != CKKS_OK) return rc;
    return launch_ntt(c, sx, 0, 0, 1, KL, KL, 0, 1, false);
}

extern "C" int ckks_keygen_public(ckks_ctx* c, uint64_t* pk, const uint64_t* sx, const uint8_t* random_a, const uint8_t* random_e) {
    if (!c || !pk || !sx || !random_a || !random_e) { set_error("addEncKey: null argument"); return CKKS_E_INVALID; }
    const int K = c->K, L1 = c->L + 1;
    const long N = c->N;
    uint64_t* ax = pk;
    uint64_t* bx = pk + N * L1;
    int rc = ckks_sample_uniform(c, random_a, ax, 0, K, L1);
    if (rc != CKKS_OK) return rc;
    rc = ckks_sample_gaussian(c, random_e, bx, 0, K, L1);
    if (rc != CKKS_OK) return rc;
    rc = launch_ntt(c, bx, 0, K, 1, L1, L1, 0, 1, false);
    if (rc != CKKS_OK) return rc;
    hipLaunchKernelGGL(pk_combine_kernel, dim3(N / THREADS, L1), dim3(THREADS), 0, c->stream, (u64*)bx, (const u64*)ax, (const u64*)sx, c->d_primes,
                       N, K);
    CKKS_HIP_TRY(hipGetLastError());
    return CKKS_OK;
}

extern "C" int ckks_encrypt(ckks_ctx* c, uint64_t* cipher, const uint64_t* mx, const uint64_t* pk, const uint8_t* random, uint64_t* scratch,
                            int l) {
    int rc = check_level(c, l, "encryptMsg");
    if (rc != CKKS_OK) return rc;
    if (!cipher || !pk || !random || !scratch) { set_error("encryptMsg: null argument"); return CKKS_E_INVALID; }
    if (((uintptr_t)random) & 3) { set_error("encryptMsg: random words must be 4-byte aligned"); return CKKS_E_INVALID; }
    const int K = c->K, L1 = c->L + 1;
    const long N = c->N;
    u64* ax = (u64*)cipher;
    u64* bx = ax + N * L1;
    hipLaunchKernelGGL(encrypt_sample_kernel, dim3(N / THREADS), dim3(THREADS), 0, c->stream, random, ax, bx, (u64*)scratch, c->d_primes, N, K, l + 1,
                       gauss_steps());
    CKKS_HIP_TRY(hipGetLastError());
    rc = launch_ntt(c, cipher, 0, K, 2, l + 1, L1, 0, 1, false);                   // e0, e1 in place
    if (rc != CKKS_OK) return rc;
    rc = launch_ntt(c, scratch, 0, K, 1, l + 1, l + 1, 0, 1, false);               // v
    if (rc != CKKS_OK) return rc;
    hipLaunchKernelGGL(encrypt_combine_kernel, dim3(N / THREADS, l + 1), dim3(THREADS), 0, c->stream, ax, bx, (const u64*)scratch, (const u64*)pk,
                       (const u64*)pk + N * L1, (const u64*)mx, c->d_primes, N, K);
    CKKS_HIP_TRY(hipGetLastError());
    return CKKS_OK;
}

extern "C" int ckks_decrypt(ckks_ctx* c, uint64_t* mx, const uint64_t* cipher, const uint64_t* sx, int l) {
    int rc = check_level(c, l, "decryptMsg");
    if (rc != CKKS_OK) return rc;
    if (!mx || !cipher || !sx) { set_error("decryptMsg: null argument"); return CKKS_E_INVALID; }
    const int K = c->K, L1 = c->L + 1;
    const long N = c->N;
    hipLaunchKernelGGL(decrypt_kernel, dim3(N / THREADS, L1), dim3(THREADS), 0, c->stream, (u64*)mx, (const u64*)cipher, (const u64*)cipher + N * L1,
                       (const u64*)sx, c->d_primes, N, K, l + 1);
    CKKS_HIP_TRY(hipGetLastError());
    return CKKS_OK;
}

extern "C" int ckks_encode_coeffs(ckks_ctx* c, uint64_t* mx, const double* vals, long scale, int l) {
    int rc = check_level(c, l, "encode_coeffs");
    if (rc != CKKS_OK) return rc;
    if (!mx || !vals) { set_error("encode_coeffs: null argument"); return CKKS_E_INVALID; }
    const long N = c->N;
    hipLaunchKernelGGL(encode_coeffs_kernel, dim3(N / THREADS, l + 1), dim3(THREADS), 0, c->stream, (u64*)mx, vals, c->d_primes, N, c->K, scale);
    CKKS_HIP_TRY(hipGetLastError());
    return launch_ntt(c, mx, 0, c->K, 1, l + 1, c->L + 1, 0, 1, false);
}

// table of one level, built on first use and kept until the context is destroyed
static int decode_table(ckks_ctx* c, int l, const u64** tab, int* words) {
    for (auto& e : c->decode_tabs)
        if (e.level == l) { *tab = (const u64*)e.dev; *words = e.words; return CKKS_OK; }
    const int n = l + 1;
    const u64* q = c->pqt.data() + c->K;
    std::vector<u64> Q{1};
    for (int i = 0; i < n; i++) big_mul_word(Q, q[i]);
    int W = 8;
    while (W < (int)Q.size()) W *= 2;
    if (W > 32) { set_error("decode_coeffs: modulus above 2048 bits"); return CKKS_E_INVALID; }
    std::vector<u64> host((size_t)n * n + n + 2 * W, 0);
    for (int i = 0; i < n; i++) {
        u64 prod = 1 % q[i];
        for (int j = 0; j < i; j++) {
            host[(size_t)i * n + j] = prod;
            prod = H::mulmod(prod, q[j] % q[i], q[i]);
        }
        host[(size_t)n * n + i] = i ? H::invmod(prod, q[i]) : 1;
    }
    u64* Qw = host.data() + (size_t)n * n + n;
    u64* Qh = Qw + W;
    for (size_t w = 0; w < Q.size(); w++) Qw[w] = Q[w];
    for (int w = 0; w < W; w++) Qh[w] = (Qw[w] >> 1) | (w + 1 < W ? Qw[w + 1] << 63 : 0);
    void* dev = nullptr;
    CKKS_HIP_TRY(hipMalloc(&dev, host.size() * 8));
    hipError_t e = hipMemcpy(dev, host.data(), host.size() * 8, hipMemcpyHostToDevice);
    if (e != hipSuccess) { (void)hipFree(dev); return hip_fail(e, "hipMemcpy(decode table)"); }
    c->decode_tabs.push_back({l, W, dev});
    *tab = (const u64*)dev;
    *words = W;
    return CKKS_OK;
}

extern "C" int ckks_decode_coeffs(ckks_ctx* c, double* vals, const uint64_t* mx, uint64_t* scratch, double scale, int slots, int is_bitrev, int l) {
    int rc = check_level(c, l, "decode_coeffs");
    if (rc != CKKS_OK) return rc;
    if (!vals || !mx || !scratch) { set_error("decode_coeffs: null argument"); return CKKS_E_INVALID; }
    const long N = c->N;
    if (slots < 1 || slots > N / 2 || (N / 2) % slots) { set_error("decode_coeffs: slots must divide N/2"); return CKKS_E_INVALID; }
    if (l + 1 > DECODE_MAX_LIMBS) { set_error("decode_coeffs: more than 64 limbs"); return CKKS_E_INVALID; }
    if (!(scale > 0)) { set_error("decode_coeffs: scale must be positive"); return CKKS_E_INVALID; }
    const u64* tab = nullptr;
    int W = 0;
    rc = decode_table(c, l, &tab, &W);
    if (rc != CKKS_OK) return rc;
    CKKS_HIP_TRY(hipMemcpyAsync(scratch, mx, 8 * N * (size_t)(l + 1), hipMemcpyDeviceToDevice, c->stream));
    rc = launch_ntt(c, scratch, 0, c->K, 1, l + 1, l + 1, 0, 1, true);
    if (rc != CKKS_OK) return rc;
    const int gap = (int)((N / 2) / slots);
    dim3 grid((unsigned)(N / THREADS)), block(THREADS);
#define LAUNCH_DECODE(WW)                                                                                                              \
    hipLaunchKernelGGL(decode_coeffs_kernel<WW>, grid, block, 0, c->stream, vals, (const u64*)scratch, c->d_primes, tab, N, c->logN, c->K, l + 1, gap, \
                       scale, is_bitrev)
    if (W == 8) LAUNCH_DECODE(8);
    else if (W == 16) LAUNCH_DECODE(16);
    else LAUNCH_DECODE(32);
#undef LAUNCH_DECODE
    CKKS_HIP_TRY(hipGetLastError());
    return CKKS_OK;
}
