// C++ host mirror of the reference's classes for the NTT -> key switch -> PCMM path, on top of the C ABI (ckks_hip.h).
//
// Same class names, member names, argument order and addressing as the reference's headers, so that code written
// against Context_23.h / Scheme_23.h / pcmm/PCMM_Scheme.h compiles against this header with
// `using namespace ckks_llm_amd;`.  Differences, all deliberate:
//   * Context_23 has a second constructor that takes the primes (the reference only selects a compiled-in set by logN,
//     Context_23.cuh:12-113; that constructor is here too);
//   * tables live in the handle, not in process-global __constant__ symbols, so several contexts can coexist;
//   * scales are long double (the reference uses NTL::RR only for this bookkeeping, Ciphertext.cuh:23);
//   * C-ABI error codes become exceptions: std::invalid_argument where the reference throws it
//     (KeySwitch_23.cuh:194-201, Scheme_23.cuh:192-194), std::runtime_error for everything the reference never checks.
// Header-only, no HIP headers needed: any C++17 host compiler can build against it and link libckks_hip.so.
#pragma once
#include <algorithm>
#include <cmath>
#include <complex>
#include <cstddef>
#include <cstdio>
#include <cstdint>
#include <iostream>
#include <random>
#include <stdexcept>
#include <string>
#include <vector>

#include "ckks_hip.h"

namespace ckks_llm_amd {

typedef uint64_t uint64_tt;

inline void check(int rc, const char* what) {
    if (rc == CKKS_OK) return;
    std::string msg = std::string(what) + ": " + ckks_last_error();
    if (rc == CKKS_E_STATE) throw std::invalid_argument(msg);
    throw std::runtime_error(msg);
}

inline uint64_tt* device_alloc_words(size_t words) {
    void* p = nullptr;
    check(ckks_malloc(&p, sizeof(uint64_tt) * (words ? words : 1)), "ckks_malloc");
    return static_cast<uint64_tt*>(p);
}
inline void device_release(uint64_tt*& p) {
    if (!p) return;
    ckks_sync();                       // the reference synchronises around every cudaFree (Ciphertext.cuh:88-99)
    ckks_free(p);
    p = nullptr;
}

// The reference's compiled-in parameter sets (Params.cuh:11-170: logN = 13, 14, 15, 16): Q, P and T primes, gamma and the
// default plaintext precision.  Data only; the bootstrapping polynomials the same function sets are not part of this library.
struct ReferenceParams {
    std::vector<uint64_tt> q, p, t;
    int gamma = 0;
    long precision = 0;
};
inline ReferenceParams reference_params(long logN) {
    ReferenceParams r;
    switch (logN) {
    case 13:
        r.q = {
            0x4001b00001, 0xfff9c0001, 0xfff8e0001, 0xfff840001, 0xfff700001,};
        r.p = {
            0x10a19000001,};
        r.t = {
            0xffffffffffc0001, 0xfffffffff840001, 0xfffffffff6a0001,};
        r.gamma = 3; r.precision = 1l << 36;
        break;
    case 14:
        r.q = {
            0x4001b00001, 0xfff9c0001, 0xfff8e0001, 0xfff840001, 0xfff700001, 0xfff640001, 0x1000a20001, 0x1000b40001,
            0x1000f60001, 0x10011a0001,};
        r.p = {
            0x10a19000001, 0x10a3b000001,};
        r.t = {
            0xffffffffffc0001, 0xfffffffff840001, 0xfffffffff6a0001, 0xfffffffff5a0001,};
        r.gamma = 3; r.precision = 1l << 36;
        break;
    case 15:
        r.q = {
            0x20000018e0001, 0x2000001c00001, 0x2000001ca0001, 0x2000001d20001, 0x1fffffee80001, 0x1fffffede0001,
            0x1fffffec40001, 0x1fffffe780001, 0x2000000ce0001, 0x20000013a0001, 0x20000013c0001, 0x20000015a0001,};
        r.p = {
            0x2000002600001, 0x20000027e0001, 0x2000002800001, 0x20000029e0001,};
        r.t = {
            0xffffffffffc0001, 0xfffffffff840001, 0xfffffffff6a0001, 0xfffffffff5a0001, 0xfffffffff2a0001,
            0xfffffffff240001, 0xffffffffefe0001,};
        r.gamma = 4; r.precision = 1l << 49;
        break;
    case 16:
        r.q = {
            0x20000018e0001, 0x2000001c00001, 0x2000001ca0001, 0x2000001d20001, 0x1fffffee80001, 0x1fffffede0001,
            0x1fffffec40001, 0x1fffffe780001, 0x2000000ce0001, 0x20000013a0001, 0x20000013c0001, 0x20000015a0001,
            0x1ffffffea0001, 0x1ffffffd40001, 0x1ffffffba0001, 0x1ffffffb40001, 0x20000001a0001, 0x20000005e0001,
            0x2000000860001, 0x2000000b00001, 0x1ffffffb00001, 0x1ffffffa20001, 0x1ffffff780001, 0x1ffffff5c0001,
            0x1fffffe5a0001, 0x1fffffe480001, 0x1fffffde80001, 0x1fffffde20001,};
        r.p = {
            0x2000002600001, 0x20000027e0001, 0x2000002800001, 0x20000029e0001,};
        r.t = {
            0xffffffffffc0001, 0xfffffffff840001, 0xfffffffff6a0001, 0xfffffffff5a0001, 0xfffffffff2a0001,
            0xfffffffff240001, 0xffffffffefe0001, 0xffffffffeca0001,};
        r.gamma = 4; r.precision = 1l << 49;
        break;
    default:
        throw std::invalid_argument("Context_23: the reference holds parameter sets for logN = 13, 14, 15 and 16 only");
    }
    return r;
}

// Context_23 (Context_23.h:19-279): prime sets, tables, NTT and basis conversion.
// PrecisionStats / GetPrecisionStats (precision.cuh:5-249): the table of log2(1 / |computed - wanted|) that the reference's test
// programs print.  Kept as the reference computes it: MinDelta starts at 1, so the maximum precision is never reported below 0
// bits; the median of an even number n of values is the mean of the sorted values n/2 and n/2 + 1 (counting from 0) unless
// n/2 + 1 = n.  The cumulative distributions the reference fills and never prints are left out.
struct Stats {
    double Real, Imag, L2;
};
struct PrecisionStats {
    Stats MaxDelta, MinDelta, MaxPrecision, MinPrecision, MeanDelta, MeanPrecision, MedianDelta, MedianPrecision;
    std::string String() const {                                           // precision.cuh:29-44
        char buffer[512];
        snprintf(buffer, sizeof(buffer),
                 "\n _________________________________\n"
                 "|    Log2 | REAL  | IMAG  | L2    |\n"
                 "|MIN Prec | %.2f | %.2f | %.2f |\n"
                 "|MAX Prec | %.2f | %.2f | %.2f |\n"
                 "|AVG Prec | %.2f | %.2f | %.2f |\n"
                 "|MED Prec | %.2f | %.2f | %.2f |\n"
                 "===================================\n",
                 MinPrecision.Real, MinPrecision.Imag, MinPrecision.L2, MaxPrecision.Real, MaxPrecision.Imag, MaxPrecision.L2,
                 MeanPrecision.Real, MeanPrecision.Imag, MeanPrecision.L2, MedianPrecision.Real, MedianPrecision.Imag, MedianPrecision.L2);
        return std::string(buffer);
    }
};
inline Stats deltaToPrecision(const Stats& c) { return {std::log2(1 / c.Real), std::log2(1 / c.Imag), std::log2(1 / c.L2)}; }
inline PrecisionStats precision_from_deltas(std::vector<double> re, std::vector<double> im) {
    const size_t n = re.size();
    std::vector<double> l2(n);
    PrecisionStats prec;
    prec.MaxDelta = {0, 0, 0};
    prec.MinDelta = {1, 1, 1};
    prec.MeanDelta = {0, 0, 0};
    for (size_t i = 0; i < n; i++) {
        l2[i] = std::sqrt(re[i] * re[i] + im[i] * im[i]);
        prec.MeanDelta.Real += re[i]; prec.MeanDelta.Imag += im[i]; prec.MeanDelta.L2 += l2[i];
        prec.MaxDelta = {std::max(prec.MaxDelta.Real, re[i]), std::max(prec.MaxDelta.Imag, im[i]), std::max(prec.MaxDelta.L2, l2[i])};
        prec.MinDelta = {std::min(prec.MinDelta.Real, re[i]), std::min(prec.MinDelta.Imag, im[i]), std::min(prec.MinDelta.L2, l2[i])};
    }
    prec.MeanDelta = {prec.MeanDelta.Real / n, prec.MeanDelta.Imag / n, prec.MeanDelta.L2 / n};
    auto median = [n](std::vector<double>& v) {                            // calcMedian, precision.cuh:69-102
        std::sort(v.begin(), v.end());
        const size_t index = n / 2;
        return (n % 2 == 1 || index + 1 == n) ? v[index] : (v[index] + v[index + 1]) / 2;
    };
    prec.MedianDelta = {median(re), median(im), median(l2)};
    prec.MinPrecision = deltaToPrecision(prec.MaxDelta);
    prec.MaxPrecision = deltaToPrecision(prec.MinDelta);
    prec.MeanPrecision = deltaToPrecision(prec.MeanDelta);
    prec.MedianPrecision = deltaToPrecision(prec.MedianDelta);
    return prec;
}
inline PrecisionStats GetPrecisionStats(const std::vector<double>& valuesTest, const std::vector<double>& valuesWant) {      // precision.cuh:178-249
    if (valuesTest.size() < valuesWant.size() || valuesWant.empty()) throw std::invalid_argument("GetPrecisionStats: vectors of the same positive length");
    std::vector<double> re(valuesWant.size()), im(valuesWant.size(), 0.0);
    for (size_t i = 0; i < re.size(); i++) re[i] = std::abs(valuesTest[i] - valuesWant[i]);
    return precision_from_deltas(re, im);
}
inline PrecisionStats GetPrecisionStats(const std::vector<std::complex<double>>& valuesTest, const std::vector<std::complex<double>>& valuesWant) {  // :104-174
    if (valuesTest.size() < valuesWant.size() || valuesWant.empty()) throw std::invalid_argument("GetPrecisionStats: vectors of the same positive length");
    std::vector<double> re(valuesWant.size()), im(valuesWant.size());
    for (size_t i = 0; i < re.size(); i++) { re[i] = std::abs(valuesTest[i].real() - valuesWant[i].real()); im[i] = std::abs(valuesTest[i].imag() - valuesWant[i].imag()); }
    return precision_from_deltas(re, im);
}

class Context_23 {
public:
    long logN, N;
    int p_num, q_num, t_num, gamma, K, L, dnum, Ri_blockNum, Qj_blockNum;
    std::vector<uint64_tt> pVec, qVec, tVec;
    long logslots = 0, slots = 0, M = 0, Nh = 0, logNh = 0, h = 64, precision = 0;     // Context_23.h:62-89
    double sigma = 3.2;
    ckks_ctx* handle = nullptr;

    Context_23(long logN, const std::vector<uint64_tt>& p, const std::vector<uint64_tt>& q,
               const std::vector<uint64_tt>& t = {}, int gamma = 0)
        : logN(logN), N(1l << logN), p_num((int)p.size()), q_num((int)q.size()), t_num((int)t.size()), gamma(gamma),
          K((int)p.size()), L((int)q.size() - 1), pVec(p), qVec(q), tVec(t) {
        create();
    }
    // The reference's own constructor (Context_23.h:21, Context_23.cuh:12-52): the parameter set compiled in for logN, the
    // secret's Hamming weight 64 or 192 ("hamming weight error!" otherwise, Params.cuh:228).
    Context_23(long logN, long logslots, long h = 64, double sigma = 3.2)
        : logN(logN), N(1l << logN), logslots(logslots), slots(1l << logslots), h(h), sigma(sigma) {
        if (h != 64 && h != 192) throw std::invalid_argument("hamming weight error!");
        ReferenceParams r = reference_params(logN);
        pVec = r.p; qVec = r.q; tVec = r.t; gamma = r.gamma; precision = r.precision;
        p_num = K = (int)pVec.size(); q_num = (int)qVec.size(); t_num = (int)tVec.size(); L = q_num - 1;
        create();
    }
    Context_23(const Context_23&) = delete;
    Context_23& operator=(const Context_23&) = delete;
    ~Context_23() { if (handle) ckks_ctx_destroy(handle); }
    void seed_rng_from_system() {
        std::random_device rd;
        for (int i = 0; i < 32; i += 4) {
            const uint32_t w = rd();
            for (int b = 0; b < 4; b++) rng_key[i + b] = (uint8_t)(w >> (8 * b));
        }
        rng_nonce = 0;
    }

    long info(const char* name) const {
        long v = 0;
        check(ckks_ctx_info(handle, name, &v), "ckks_ctx_info");
        return v;
    }
private:
    void create() {
        M = N << 1; Nh = N >> 1; logNh = logN - 1;
        if (!slots) { slots = Nh; logslots = logNh; }
        check(ckks_ctx_create(&handle, (int)logN, pVec.data(), p_num, qVec.data(), q_num, tVec.data(), t_num, gamma), "Context_23");
        dnum = (int)info("dnum");
        Ri_blockNum = (int)info("Ri_blockNum");
        Qj_blockNum = (int)info("Qj_blockNum");
        seed_rng_from_system();
    }
public:

    // Where the reference's programs call cudaDeviceSynchronize and check the last error (Utils.cuh CUDA_CHECK): waits for the
    // context's stream and throws on anything the launches so far have reported, including a one-launch transform that gave up a wait.
    void synchronize() { check(ckks_ctx_check(handle), "synchronize"); }
    // launch form of the transforms (0 = chosen by the library); no counterpart in the reference
    void set_ntt_mode(int mode) { check(ckks_ctx_set_ntt_mode(handle, mode), "set_ntt_mode"); }

    // Context_23.h:42-45
    void ToNTTInplace(uint64_tt* device_a, int start_poly_idx, int start_mod_idx, int poly_num, int mod_num, int poly_mod_len) {
        check(ckks_ntt_fwd(handle, device_a, start_poly_idx, start_mod_idx, poly_num, mod_num, poly_mod_len), "ToNTTInplace");
    }
    void FromNTTInplace(uint64_tt* device_a, int start_poly_idx, int start_mod_idx, int poly_num, int mod_num, int poly_mod_len) {
        check(ckks_ntt_inv(handle, device_a, start_poly_idx, start_mod_idx, poly_num, mod_num, poly_mod_len), "FromNTTInplace");
    }
    void ToNTTInplace_for_externalProduct(uint64_tt* device_a, int start_poly_idx, int start_mod_idx, int poly_num, int mod_num,
                                          int poly_mod_len, int cipher_mod_num, int batch_size) {
        check(ckks_ntt_fwd_ext(handle, device_a, start_poly_idx, start_mod_idx, poly_num, mod_num, poly_mod_len, cipher_mod_num,
                               batch_size), "ToNTTInplace_for_externalProduct");
    }
    void FromNTTInplace_for_externalProduct(uint64_tt* device_a, int start_poly_idx, int start_mod_idx, int poly_num, int mod_num,
                                            int poly_mod_len, int cipher_mod_num, int batch_size) {
        check(ckks_ntt_inv_ext(handle, device_a, start_poly_idx, start_mod_idx, poly_num, mod_num, poly_mod_len, cipher_mod_num,
                               batch_size), "FromNTTInplace_for_externalProduct");
    }
    // Context_23.h:54-61
    void modUpPQtoT_23(uint64_tt* output, const uint64_tt* input, int l, int batch_size) {
        check(ckks_modup_pq_to_t(handle, output, input, l, batch_size), "modUpPQtoT_23");
    }
    void modUpQjtoT_23(uint64_tt* output, const uint64_tt* input, int l, int batch_size) {
        check(ckks_modup_qj_to_t(handle, output, input, l, batch_size), "modUpQjtoT_23");
    }
    void modUpTtoPQl_23(uint64_tt* modUp_TtoQj_buffer, const uint64_tt* exProduct_T_temp, int l, int batch_size) {
        check(ckks_modup_t_to_pql(handle, modUp_TtoQj_buffer, exProduct_T_temp, l, batch_size), "modUpTtoPQl_23");
    }
    void modDownPQltoQl_23(uint64_tt* output, const uint64_tt* modUp_TtoQj_buffer, int l, int batch_size) {
        check(ckks_moddown_pql_to_ql(handle, output, modUp_TtoQj_buffer, l, batch_size), "modDownPQltoQl_23");
    }
    void external_product_T(uint64_tt* output, const uint64_tt* cipher_modUp_QjtoT, const uint64_tt* swk_modUp_RitoT, int l) {
        check(ckks_external_product_t(handle, output, cipher_modUp_QjtoT, swk_modUp_RitoT, l), "external_product_T");
    }
    // Context_23.h:62: one switching key against batch_size digit sets
    void external_product_T_swk_reuse(uint64_tt* output, const uint64_tt* cipher_modUp_QjtoT, const uint64_tt* swk_modUp_RitoT, int l, int batch_size) {
        check(ckks_external_product_t_swk_reuse(handle, output, cipher_modUp_QjtoT, swk_modUp_RitoT, l, batch_size), "external_product_T_swk_reuse");
    }

    // RNG::generateRandom_device (RNG.cuh:18-56).  The reference draws a fresh key and nonce from rand() per call; here the
    // context holds a key and a nonce that counts the calls.  The key comes from std::random_device when the context is built, so
    // no two processes share secrets or encryption randomness; a program that must repeat a run (the parity tests) overwrites
    // rng_key with fixed bytes and resets rng_nonce before it draws anything.
    uint8_t rng_key[32];
    uint64_t rng_nonce = 0;
    void generateRandom_device(uint8_t* a, uint64_tt n) {
        check(ckks_random_bytes(handle, a, (size_t)n, rng_key, ++rng_nonce), "generateRandom_device");
    }
    // Context_23::encode_coeffs / decode_coeffs (Encoder.cuh:83-96, 113-186); vals: N device doubles
    template <class PlaintextT>
    void encode_coeffs(const double* vals, PlaintextT& msg) {
        check(ckks_encode_coeffs(handle, msg.mx_device, vals, (long)msg.scale, msg.l), "encode_coeffs");
    }
    template <class PlaintextT>
    void decode_coeffs(PlaintextT& msg, double* vals, bool is_bitRev = false) {
        uint64_tt* scratch = device_alloc_words((size_t)N * (msg.l + 1));
        int rc = ckks_decode_coeffs(handle, vals, msg.mx_device, scratch, (double)msg.scale, msg.slots, is_bitRev ? 1 : 0, msg.l);
        device_release(scratch);
        check(rc, "decode_coeffs");
    }
};

// Sampler (Sampler.cuh:12-54): conversions of random device bytes into limbs
class Sampler {
public:
    static void uniformSampler_xq(Context_23& c, const uint8_t* in, uint64_tt* out, int idx_out, int idx_mod, int mod_num) {
        check(ckks_sample_uniform(c.handle, in, out, idx_out, idx_mod, mod_num), "uniformSampler_xq");
    }
    static void gaussianSampler_xq(Context_23& c, const uint8_t* in, uint64_tt* out, int idx_out, int idx_mod, int mod_num) {
        check(ckks_sample_gaussian(c.handle, in, out, idx_out, idx_mod, mod_num), "gaussianSampler_xq");
    }
    static void HWTSampler(Context_23& c, const uint8_t* in, uint64_tt* out, int h, int idx_out, int idx_mod, int mod_num) {
        check(ckks_sample_hwt(c.handle, in, out, h, idx_out, idx_mod, mod_num), "HWTSampler");
    }
    static void ZOSampler(Context_23& c, const uint8_t* in, uint64_tt* out, double probability, int idx_out, int idx_mod, int mod_num) {
        check(ckks_sample_zo(c.handle, in, out, probability, idx_out, idx_mod, mod_num), "ZOSampler");
    }
};

// Plaintext (Plaintext.cuh:6-76): L+1 limbs, NTT domain
class Plaintext {
public:
    uint64_tt* mx_device = nullptr;
    int N = 0, l = 0, L = 0, slots = 0;
    long double scale = 0;

    Plaintext() {}
    Plaintext(int N, int L, int l, int slots, long double scale) : N(N), l(l), L(L), slots(slots), scale(scale) {
        if (l > L) std::cout << "new Plaintext error!" << std::endl;            // Plaintext.cuh:11
        mx_device = device_alloc_words((size_t)N * (L + 1));
    }
    Plaintext(const Plaintext&) = delete;
    Plaintext& operator=(const Plaintext&) = delete;
    virtual ~Plaintext() { device_release(mx_device); }
};

// SecretKey (SecretKey.cuh:9-57): sparse ternary secret of Hamming weight <= h over [P | Q], NTT domain
class SecretKey {
public:
    uint64_tt* sx_device = nullptr;
    int N, L, K;

    // h < 0: the context's Hamming weight, as the reference's SecretKey(context) takes it (SecretKey.cuh:20-29)
    explicit SecretKey(Context_23& context, int h = -1) : N((int)context.N), L(context.L), K(context.K) {
        if (h < 0) h = (int)context.h;
        sx_device = device_alloc_words((size_t)N * (K + L + 1));
        uint64_tt* rnd = device_alloc_words((size_t)(5 * h + 7) / 8 + 8);
        context.generateRandom_device(reinterpret_cast<uint8_t*>(rnd), (uint64_tt)5 * h);
        int rc = ckks_keygen_secret(context.handle, sx_device, reinterpret_cast<uint8_t*>(rnd), h);
        device_release(rnd);
        check(rc, "SecretKey");
    }
    SecretKey(const SecretKey&) = delete;
    SecretKey& operator=(const SecretKey&) = delete;
    virtual ~SecretKey() { device_release(sx_device); }
};

// Key (Key.cuh:5-24): [a | b], (L+1+K)*dnum limbs each
class Key {
public:
    uint64_tt* ax_device = nullptr;
    uint64_tt* bx_device = nullptr;
    uint64_tt* cipher_device = nullptr;
    int N = 0, L = 0, K = 0, dnum = 0;

    Key(int N, int L, int K, int dnum) : N(N), L(L), K(K), dnum(dnum) {
        cipher_device = device_alloc_words((size_t)N * (L + 1 + K) * dnum * 2);
        ax_device = cipher_device;
        bx_device = cipher_device + (size_t)N * (L + 1 + K) * dnum;
    }
    Key(const Key&) = delete;
    Key& operator=(const Key&) = delete;
    virtual ~Key() { device_release(cipher_device); }
};

// Ciphertext (Ciphertext.cuh:5-99): one device buffer [a: L+1 limbs | b: L+1 limbs].
class Ciphertext {
public:
    uint64_tt* ax_device = nullptr;
    uint64_tt* bx_device = nullptr;
    uint64_tt* cipher_device = nullptr;
    int N = 0, l = 0, L = 0, slots = 0;
    long double scale = 0;

    Ciphertext() {}
    Ciphertext(int N, int L, int l, int slots, long double scale) : N(N), l(l), L(L), slots(slots), scale(scale) {
        cipher_device = device_alloc_words((size_t)N * (L + 1) * 2);
        ax_device = cipher_device;
        bx_device = cipher_device + (size_t)N * (L + 1);
    }
    Ciphertext(const Ciphertext& c) : Ciphertext(c.N, c.L, c.l, c.slots, c.scale) {
        check(ckks_memcpy_d2d(cipher_device, c.cipher_device, sizeof(uint64_tt) * (size_t)N * (L + 1) * 2), "Ciphertext copy");
    }
    Ciphertext& operator=(const Ciphertext&) = delete;
    virtual ~Ciphertext() { device_release(cipher_device); }
};

// MLWECiphertext (pcmm/MLWECiphertext.cuh:6-78): [(L+1) moduli][a_0 .. a_{k-1}, b][N1].
class MLWECiphertext {
public:
    uint64_tt* cipher_device = nullptr;
    int N1 = 0, L = 0, l = 0, k = 0;
    long double scale = 0;

    MLWECiphertext() {}
    MLWECiphertext(int N1, int L, int l, int k, long double scale) : N1(N1), L(L), l(l), k(k), scale(scale) {
        cipher_device = device_alloc_words((size_t)N1 * (L + 1) * (k + 1));
    }
    MLWECiphertext(const MLWECiphertext&) = delete;
    MLWECiphertext& operator=(const MLWECiphertext&) = delete;
    virtual ~MLWECiphertext() { device_release(cipher_device); }
};

// Key_decomp (Key_decomp.cuh:5-24): a switching key in the T basis, [a | b] with dnum * Ri_blockNum * t_num limbs each
class Key_decomp {
public:
    uint64_tt* ax_device = nullptr;
    uint64_tt* bx_device = nullptr;
    uint64_tt* cipher_device = nullptr;
    int N = 0, dnum = 0, t_num = 0, Ri_blockNum = 0;

    Key_decomp(int N, int dnum, int t_num, int Ri_blockNum) : N(N), dnum(dnum), t_num(t_num), Ri_blockNum(Ri_blockNum) {
        cipher_device = device_alloc_words((size_t)N * dnum * t_num * Ri_blockNum * 2);
        ax_device = cipher_device;
        bx_device = cipher_device + (size_t)N * dnum * t_num * Ri_blockNum;
    }
    Key_decomp(const Key_decomp&) = delete;
    Key_decomp& operator=(const Key_decomp&) = delete;
    virtual ~Key_decomp() { device_release(cipher_device); }
};

// The members of Scheme_23 on the path (Scheme_23.h:113-182): public-key encryption, decryption, rescale, switching keys,
// multiplication, rotation, conjugation.
class Scheme_23 {
public:
    Context_23& context;
    Key* publicKey = nullptr;
    Key_decomp* rlk_23 = nullptr;
    Key_decomp* ConjKey_23 = nullptr;
    std::vector<Key_decomp*> rotKey_vec_23;
    uint64_tt* vx_enc = nullptr;
    uint8_t* in_enc = nullptr;
    long random_len_for_enc = 0;
    uint64_tt* sxsx = nullptr;
    uint64_tt* temp_mul = nullptr;
    uint64_tt* mul_work = nullptr;            // axbx1_mul, axax_mul, bxbx_mul of the reference, contiguous
    // Scheme_23::mallocMemory (Scheme_23.cuh:7-51): scratch owned by the scheme
    uint64_tt* rescale_buffer = nullptr;
    uint64_tt* modUp_QjtoT_temp = nullptr;
    uint64_tt* exProduct_T_temp = nullptr;
    uint64_tt* modUp_TtoQj_buffer = nullptr;

    explicit Scheme_23(Context_23& context) : context(context) {
        const size_t N = (size_t)context.N;
        rescale_buffer = device_alloc_words(2 * N * (context.L + 1));
        vx_enc = device_alloc_words(N * (context.L + 1));
        random_len_for_enc = (long)(N + 4 * N + 4 * N);                          // Scheme_23.cuh:38
        in_enc = reinterpret_cast<uint8_t*>(device_alloc_words((size_t)random_len_for_enc / 8));
        rotKey_vec_23.assign(N, nullptr);                                        // Scheme_23.cuh:41
        if (context.t_num > 0) {
            sxsx = device_alloc_words(N * (context.K + context.L + 1));
            temp_mul = device_alloc_words(N * (context.K + context.L + 1));
            mul_work = device_alloc_words(3 * N * (context.L + 1));
            modUp_QjtoT_temp = device_alloc_words(N * context.t_num * context.Qj_blockNum);
            exProduct_T_temp = device_alloc_words(N * context.t_num * context.Ri_blockNum * 2);
            modUp_TtoQj_buffer = device_alloc_words(N * context.t_num * context.Ri_blockNum * 2);
        }
    }
    Scheme_23(const Scheme_23&) = delete;
    ~Scheme_23() {
        delete publicKey;
        delete rlk_23;
        delete ConjKey_23;
        for (Key_decomp* k : rotKey_vec_23) delete k;
        delete cipher_temp_pool;
        device_release(sxsx);
        device_release(temp_mul);
        device_release(mul_work);
        device_release(vx_enc);
        uint64_tt* r = reinterpret_cast<uint64_tt*>(in_enc);
        device_release(r);
        device_release(rescale_buffer);
        device_release(modUp_QjtoT_temp);
        device_release(exProduct_T_temp);
        device_release(modUp_TtoQj_buffer);
    }

    // Scheme_23::addEncKey (Scheme_23.cuh:54-80): pk = (a, e - a*s)
    void addEncKey(SecretKey& secretKey) {
        const size_t N = (size_t)context.N, L1 = (size_t)context.L + 1;
        delete publicKey;
        publicKey = new Key((int)N, context.L, 0, 1);
        uint64_tt* rnd = device_alloc_words(N * L1 + N / 2);
        uint8_t* r8 = reinterpret_cast<uint8_t*>(rnd);
        context.generateRandom_device(r8, 8 * N * L1 + 4 * N);
        int rc = ckks_keygen_public(context.handle, publicKey->cipher_device, secretKey.sx_device, r8, r8 + 8 * N * L1);
        device_release(rnd);
        check(rc, "addEncKey");
    }
    // Scheme_23::encryptZero / encryptMsg (Scheme_23.cuh:82-112); a missing key throws std::invalid_argument
    void encryptZero(Ciphertext& cipher, int l, int slots) {
        cipher.l = l;
        cipher.slots = slots;
        encrypt(cipher, nullptr, l);
    }
    void encryptMsg(Ciphertext& cipher, Plaintext& message) {
        cipher.l = message.l;
        cipher.scale = message.scale;
        cipher.slots = message.slots;
        encrypt(cipher, message.mx_device, message.l);
    }
    // Scheme_23::decryptMsg (Scheme_23.cuh:114-127)
    void decryptMsg(Plaintext& plain, SecretKey& secretKey, Ciphertext& cipher) {
        plain.l = cipher.l;
        plain.scale = cipher.scale;
        plain.slots = cipher.slots;
        check(ckks_decrypt(context.handle, plain.mx_device, cipher.cipher_device, secretKey.sx_device, cipher.l), "decryptMsg");
    }

    // Scheme_23::addMultKey_23 / addConjKey_23 / addLeftRotKey_23 (KeySwitch_23.cuh:21-165)
    void addMultKey_23(SecretKey& secretKey) {
        if (rlk_23) return;
        const int K = context.K;
        check(ckks_poly_mul(context.handle, sxsx, secretKey.sx_device, secretKey.sx_device, 0, K, K, K, context.L + 1), "addMultKey_23");
        rlk_23 = switch_key(secretKey.sx_device, sxsx);
    }
    void addConjKey_23(SecretKey& secretKey) {
        if (ConjKey_23) return;
        check(ckks_poly_conjugate_ntt(context.handle, sxsx, secretKey.sx_device, 0, context.K, context.L + 1), "addConjKey_23");
        ConjKey_23 = switch_key(secretKey.sx_device, sxsx);
    }
    void addLeftRotKey_23(SecretKey& secretKey, long rot_num) {
        if (rotKey_vec_23.at((size_t)rot_num)) return;
        uint64_tt pow = 0;
        check(ckks_rot_group(context.handle, rot_num, &pow), "addLeftRotKey_23");
        check(ckks_poly_automorph_ntt(context.handle, sxsx, secretKey.sx_device, pow, 0, 0, context.K + context.L + 1), "addLeftRotKey_23");
        rotKey_vec_23[(size_t)rot_num] = switch_key(sxsx, secretKey.sx_device + (size_t)context.N * context.K);
    }
    // Scheme_23::mult_23 (KeySwitch_23.cuh:192-236); level 0 and a missing key throw std::invalid_argument
    void mult_23(Ciphertext& cipher_res, Ciphertext& cipher1, Ciphertext& cipher2) {
        const int l = cipher1.l < cipher2.l ? cipher1.l : cipher2.l;
        check(ckks_mult_23(context.handle, cipher_res.cipher_device, cipher1.cipher_device, cipher2.cipher_device,
                           rlk_23 ? rlk_23->cipher_device : nullptr, l, mul_work, modUp_QjtoT_temp, exProduct_T_temp, modUp_TtoQj_buffer), "mult_23");
        cipher_res.l = l;
        cipher_res.scale = cipher1.scale * cipher2.scale;
    }
    // Scheme_23::leftRotate_23 (KeySwitch_23.cuh:556-586)
    void leftRotate_23(Ciphertext& cipher_res, Ciphertext& cipher, long rotSlots) {
        Key_decomp* k = (rotSlots >= 0 && (size_t)rotSlots < rotKey_vec_23.size()) ? rotKey_vec_23[(size_t)rotSlots] : nullptr;
        check(ckks_rotate_23(context.handle, cipher_res.cipher_device, cipher.cipher_device, k ? k->cipher_device : nullptr, rotSlots, cipher.l,
                             mul_work, modUp_QjtoT_temp, exProduct_T_temp, modUp_TtoQj_buffer), "leftRotate_23");
        cipher_res.l = cipher.l;
        cipher_res.scale = cipher.scale;
        cipher_res.slots = cipher.slots;
    }
    // Scheme_23::rescaleAndEqual_noNTT (Scheme_23.cuh:427-440): rescale of a coefficient-domain ciphertext
    void rescaleAndEqual_noNTT(Ciphertext& cipher) {
        check(ckks_rescale_coeff(context.handle, cipher.cipher_device, cipher.l), "rescaleAndEqual_noNTT");
        cipher.scale = cipher.scale / (long double)context.qVec[(size_t)cipher.l];
        cipher.l -= 1;
    }
    // Scheme_23::conjugate_23 (KeySwitch_23.cuh:433-468)
    void conjugate_23(Ciphertext& cipher_res, Ciphertext& cipher) {
        check(ckks_conjugate_23(context.handle, cipher_res.cipher_device, cipher.cipher_device, ConjKey_23 ? ConjKey_23->cipher_device : nullptr,
                                cipher.l, mul_work, modUp_QjtoT_temp, exProduct_T_temp, modUp_TtoQj_buffer), "conjugate_23");
        cipher_res.l = cipher.l;
        cipher_res.scale = cipher.scale;
        cipher_res.slots = cipher.slots;
    }

    // Scheme_23::rescaleAndEqual (Scheme_23.cuh:369-385); throws std::invalid_argument on level 0 (:192-194 style)
    void rescaleAndEqual(Ciphertext& cipher) {
        check(ckks_rescale(context.handle, cipher.cipher_device, rescale_buffer, cipher.l), "rescaleAndEqual");
        cipher.scale /= (long double)context.qVec[cipher.l];
        cipher.l -= 1;
    }
    // ---- the in-place and derived forms: host composition over the same entry points, same words as the separate-result forms ----
    Ciphertext* cipher_temp_pool = nullptr;             // Scheme_23.cuh:27
    Ciphertext& temp_like(const Ciphertext& c) {
        if (!cipher_temp_pool) cipher_temp_pool = new Ciphertext((int)context.N, context.L, c.l, c.slots, c.scale);
        return *cipher_temp_pool;
    }
    void copy_back(Ciphertext& dst, const Ciphertext& src) {
        check(ckks_memcpy_d2d(dst.cipher_device, src.cipher_device, sizeof(uint64_tt) * (size_t)context.N * (context.L + 1) * 2), "copy back");
        dst.l = src.l;
        dst.scale = src.scale;
    }
    // KeySwitch_23.cuh:238-282
    void multAndEqual_23(Ciphertext& cipher1, Ciphertext& cipher2) {
        Ciphertext& t = temp_like(cipher1);
        mult_23(t, cipher1, cipher2);
        copy_back(cipher1, t);
    }
    // KeySwitch_23.cuh:346-388: cipher1 = cipher2^2
    void square(Ciphertext& cipher1, Ciphertext& cipher2) { mult_23(cipher1, cipher2, cipher2); }
    // KeySwitch_23.cuh:390-430
    void squareAndEqual(Ciphertext& cipher) {
        Ciphertext& t = temp_like(cipher);
        mult_23(t, cipher, cipher);
        copy_back(cipher, t);
    }
    // KeySwitch_23.cuh:473-506
    void conjugateAndEqual_23(Ciphertext& cipher) {
        Ciphertext& t = temp_like(cipher);
        conjugate_23(t, cipher);
        copy_back(cipher, t);
    }
    // KeySwitch_23.cuh:509-553
    void leftRotateAndEqual_23(Ciphertext& cipher, long rotSlots) {
        Ciphertext& t = temp_like(cipher);
        leftRotate_23(t, cipher, rotSlots);
        copy_back(cipher, t);
    }
    // KeySwitch_23.cuh:618-622: right by 2^rotSlots slots = left by N/2 - 2^rotSlots
    void rightRotateAndEqual_23(Ciphertext& cipher, long rotSlots) { leftRotateAndEqual_23(cipher, context.N / 2 - (1l << rotSlots)); }
    // KeySwitch_23.cuh:583-616: cipher += cipher rotated left by rotSlots
    void leftRotateAddSelf_23(Ciphertext& cipher, long rotSlots) {
        Ciphertext& t = temp_like(cipher);
        leftRotate_23(t, cipher, rotSlots);
        addAndEqual(cipher, t);
    }
    // Scheme_23.cuh:130-141
    void add(Ciphertext& cipher_res, Ciphertext& cipher1, Ciphertext& cipher2) {
        const int l = cipher1.l < cipher2.l ? cipher1.l : cipher2.l, L1 = context.L + 1;
        for (int z = 0; z < 2; z++)
            check(ckks_poly_add(context.handle, cipher_res.cipher_device, cipher1.cipher_device, cipher2.cipher_device, z * L1, z * L1, z * L1, context.K, l + 1), "add");
        cipher_res.l = l;
        cipher_res.scale = cipher1.scale;
    }
    // Scheme_23.cuh:143-152
    void addAndEqual(Ciphertext& cipher1, Ciphertext& cipher2) {
        const long double scale = cipher1.scale;
        add(cipher1, cipher1, cipher2);
        cipher1.scale = scale;
    }
    // Scheme_23.cuh:268-280 (the result keeps cipher1's level, as there)
    void sub(Ciphertext& cipher_res, Ciphertext& cipher1, Ciphertext& cipher2) {
        const int l = cipher1.l < cipher2.l ? cipher1.l : cipher2.l, L1 = context.L + 1;
        for (int z = 0; z < 2; z++)
            check(ckks_poly_sub(context.handle, cipher_res.cipher_device, cipher1.cipher_device, cipher2.cipher_device, z * L1, z * L1, z * L1, context.K, l + 1), "sub");
        cipher_res.l = cipher1.l;
        cipher_res.scale = cipher1.scale;
    }
    // Scheme_23.cuh:282-292
    void subAndEqual(Ciphertext& cipher1, Ciphertext& cipher2) {
        const int l = cipher1.l < cipher2.l ? cipher1.l : cipher2.l;
        sub(cipher1, cipher1, cipher2);
        cipher1.l = l;
    }
    // Scheme_23.cuh:407-425: to the coefficient domain, one coefficient-domain rescale per level, back
    void rescaleToAndEqual(Ciphertext& cipher, int level) {
        context.FromNTTInplace(cipher.cipher_device, 0, context.K, 2, cipher.l + 1, context.L + 1);
        while (cipher.l > level) rescaleAndEqual_noNTT(cipher);
        context.ToNTTInplace(cipher.cipher_device, 0, context.K, 2, cipher.l + 1, context.L + 1);
    }
    // steps 2..9 of Scheme_23::mult_23 (KeySwitch_23.cuh:219-231): d2 (NTT domain, L+1 limbs) -> out = [a | b].
    // A null key throws std::invalid_argument as the missing rotation / relinearisation key does (:198-201).
    void keySwitch_23(uint64_tt* out, uint64_tt* d2, const uint64_tt* swk, int l) {
        check(ckks_keyswitch_23(context.handle, out, d2, swk, l, modUp_QjtoT_temp, exProduct_T_temp, modUp_TtoQj_buffer), "keySwitch_23");
    }

private:
    Key_decomp* switch_key(const uint64_tt* s_to, const uint64_tt* s_from) {
        const size_t N = (size_t)context.N, KL = (size_t)context.K + context.L + 1;
        const size_t na = (size_t)context.dnum * 8 * N * KL, ne = (size_t)context.dnum * 4 * N;      // KeySwitch_23.cuh:36
        Key_decomp* key = new Key_decomp((int)N, context.dnum, context.t_num, context.Ri_blockNum);
        uint64_tt* rnd = device_alloc_words((na + ne) / 8);
        uint8_t* r8 = reinterpret_cast<uint8_t*>(rnd);
        context.generateRandom_device(r8, na + ne);
        int rc = ckks_keygen_switch_23(context.handle, key->cipher_device, s_to, s_from, r8, r8 + na, temp_mul);
        device_release(rnd);
        if (rc != CKKS_OK) delete key;
        check(rc, "addSWKey_23");
        return key;
    }
    void encrypt(Ciphertext& cipher, const uint64_tt* mx, int l) {
        if (!publicKey) throw std::invalid_argument("encryptMsg: no encryption key (addEncKey)");
        context.generateRandom_device(in_enc, (uint64_tt)random_len_for_enc);
        check(ckks_encrypt(context.handle, cipher.cipher_device, mx, publicKey->cipher_device, in_enc, vx_enc, l), "encryptMsg");
    }
};


// PlaintextT (bootstrapping/Bootstrapping_encoding.h): a plaintext over the T primes, NTT domain, t_num limbs.
class PlaintextT {
public:
    uint64_tt* mx_device = nullptr;
    int N = 0, t_num = 0;
    long double scale = 1;

    PlaintextT(int N, int t_num, long double scale) : N(N), t_num(t_num), scale(scale) { mx_device = device_alloc_words((size_t)N * t_num); }
    PlaintextT(const PlaintextT&) = delete;
    PlaintextT& operator=(const PlaintextT&) = delete;
    virtual ~PlaintextT() { device_release(mx_device); }
};

// The hoisted baby-step / giant-step part of EncodingMatrix (Bootstrapping_C2S_S2C_impl.cuh): Giant_Rotate_And_Mult_PlaintT,
// Baby_Rotate, and one level of EvalCoeffsToSlots / EvalSlotsToCoeffs around them.  The plaintext diagonals and rotation tables
// of a level come from the caller: generating them is the bootstrapping's set-up, which is not part of this library.
class EncodingMatrix {
public:
    Scheme_23& scheme;
    uint64_tt* scratch = nullptr;
    size_t scratch_words = 0;

    explicit EncodingMatrix(Scheme_23& scheme) : scheme(scheme) {}
    EncodingMatrix(const EncodingMatrix&) = delete;
    ~EncodingMatrix() { device_release(scratch); }

    // Bootstrapping_C2S_S2C_impl.cuh:93-152
    void Giant_Rotate_And_Mult_PlaintT(uint64_tt* bs_cipher_T, uint64_tt* PQ_to_T_temp, int rotNum_here, uint64_tt* modUp_QjtoT_temp,
                                       std::vector<uint64_tt*> rotKey_pointer, std::vector<int> rotSlots_vec, std::vector<uint64_tt*> plaintextT_pointer,
                                       std::vector<int> accNum_vec, int bs, int gs, int l) {
        (void)rotNum_here;                       // carried for the reference's signature; its kernel runs over gs
        if ((int)rotKey_pointer.size() < gs || (int)rotSlots_vec.size() < gs || (int)plaintextT_pointer.size() < bs * gs || (int)accNum_vec.size() < bs)
            throw std::invalid_argument("Giant_Rotate_And_Mult_PlaintT: a table is shorter than gs / bs * gs / bs");
        check(ckks_giant_rotate_mult_plain_t(scheme.context.handle, bs_cipher_T, PQ_to_T_temp, modUp_QjtoT_temp, rotKey_pointer.data(), rotSlots_vec.data(),
                                             plaintextT_pointer.data(), accNum_vec.data(), bs, gs, l), "Giant_Rotate_And_Mult_PlaintT");
    }
    // Bootstrapping_C2S_S2C_impl.cuh:203-228
    void Baby_Rotate(uint64_tt* output, uint64_tt* modUp_QjtoT_temp, uint64_tt* input, int rotNum_here, std::vector<uint64_tt*> rotKey_pointer,
                     std::vector<int> rotSlots_vec, int l) {
        if ((int)rotKey_pointer.size() < rotNum_here || (int)rotSlots_vec.size() < rotNum_here) throw std::invalid_argument("Baby_Rotate: a table is shorter than rotNum_here");
        check(ckks_baby_rotate(scheme.context.handle, output, modUp_QjtoT_temp, input, rotNum_here, rotKey_pointer.data(), rotSlots_vec.data(), l), "Baby_Rotate");
    }
    // One pass of the level loop (Bootstrapping_C2S_S2C_impl.cuh:254-382): cipher is in the COEFFICIENT domain and stays there.
    // A_s[G + j] is the plaintext of baby step G / g and rotation j, index numRotations has none (:290-300); keys come from
    // scheme.rotKey_vec_23, a missing one throws std::invalid_argument.
    void EvalLevel(std::vector<PlaintextT*>& A_s, Ciphertext& cipher, const std::vector<int>& rot_in, const std::vector<int>& rot_out, int b, int g,
                   int numRotations, bool rescale = true) {
        if ((int)rot_in.size() < g || (int)rot_out.size() < b) throw std::invalid_argument("EvalLevel: a rotation table is shorter than g / b");
        std::vector<const uint64_tt*> plain((size_t)b * g, nullptr), in_keys((size_t)g, nullptr), out_keys((size_t)b, nullptr);
        std::vector<int> acc((size_t)b, 0);
        for (int i = 0; i < b; i++)
            for (int j = 0; j < g; j++)
                if (i * g + j != numRotations && (size_t)(i * g + j) < A_s.size()) {
                    plain[(size_t)i * g + j] = A_s[(size_t)i * g + j]->mx_device;
                    acc[(size_t)i]++;
                }
        auto key = [&](int r) -> const uint64_tt* {
            if (r <= 0 || (size_t)r >= scheme.rotKey_vec_23.size() || !scheme.rotKey_vec_23[(size_t)r]) return nullptr;
            return scheme.rotKey_vec_23[(size_t)r]->cipher_device;
        };
        for (int j = 0; j < g; j++) in_keys[(size_t)j] = key(rot_in[(size_t)j]);
        for (int i = 0; i < b; i++) out_keys[(size_t)i] = key(rot_out[(size_t)i]);
        size_t words = 0;
        check(ckks_bsgs_scratch_words(scheme.context.handle, b, &words), "ckks_bsgs_scratch_words");
        if (words > scratch_words) {
            device_release(scratch);
            scratch = device_alloc_words(words);
            scratch_words = words;
        }
        check(ckks_bsgs_level_23(scheme.context.handle, cipher.cipher_device, cipher.l, plain.data(), acc.data(), rot_in.data(), in_keys.data(),
                                 rot_out.data(), out_keys.data(), b, g, scratch), "EvalLevel");
        cipher.scale *= A_s.at(0)->scale;
        if (rescale) scheme.rescaleAndEqual_noNTT(cipher);
    }
};

// MLWESecretKey (pcmm/MLWESecretKey.cuh:6-52): [L+1 moduli][k polynomials][N1]
class MLWESecretKey {
public:
    uint64_tt* sx_device = nullptr;
    int N1 = 0, L = 0, k = 0;
    MLWESecretKey(int N1, int L, int k) : N1(N1), L(L), k(k) { sx_device = device_alloc_words((size_t)N1 * k * (L + 1)); }
    MLWESecretKey(const MLWESecretKey&) = delete;
    MLWESecretKey& operator=(const MLWESecretKey&) = delete;
    virtual ~MLWESecretKey() { device_release(sx_device); }
};

// MLWEPlaintext (pcmm/MLWEPlaintext.cuh:7-60): [L+1 moduli][N1]
class MLWEPlaintext {
public:
    uint64_tt* mx_device = nullptr;
    int N1 = 0, L = 0, l = 0;
    long double scale = 0;
    MLWEPlaintext(int N1, int L, int l, long double scale) : N1(N1), L(L), l(l), scale(scale) {
        if (l > L) std::cout << "new MLWEPlaintext error!" << std::endl;
        mx_device = device_alloc_words((size_t)N1 * (L + 1));
    }
    MLWEPlaintext(const MLWEPlaintext&) = delete;
    MLWEPlaintext& operator=(const MLWEPlaintext&) = delete;
    virtual ~MLWEPlaintext() { device_release(mx_device); }
};

// PCMM_Context (pcmm/PCMM_Context.h:14-90)
class PCMM_Context {
public:
    Context_23& context;
    int N1, mlwe_rank, ringpack_p_count, ringpack_q_count, ringpack_pq_count;
    std::vector<uint64_tt> p_ringpack, q_ringpack;
    pcmm_ctx* handle = nullptr;

    PCMM_Context(int N1, int mlwe_rank, const std::vector<uint64_tt>& p_ringpack, const std::vector<uint64_tt>& q_ringpack,
                 Context_23& context)
        : context(context), N1(N1), mlwe_rank(mlwe_rank), ringpack_p_count((int)p_ringpack.size()),
          ringpack_q_count((int)q_ringpack.size()), ringpack_pq_count((int)(p_ringpack.size() + q_ringpack.size())),
          p_ringpack(p_ringpack), q_ringpack(q_ringpack) {
        check(pcmm_ctx_create(&handle, context.handle, N1, mlwe_rank, p_ringpack.data(), ringpack_p_count, q_ringpack.data(),
                              ringpack_q_count), "PCMM_Context");
    }
    PCMM_Context(const PCMM_Context&) = delete;
    ~PCMM_Context() { if (handle) pcmm_ctx_destroy(handle); }
    long info(const char* name) const {
        long v = 0;
        check(pcmm_info(handle, name, &v), "pcmm_info");
        return v;
    }
    // By default every PPMM call reads its plaintext matrix afresh, as the reference does.  A matrix declared static (one that
    // changes only through this library's copies) keeps its digit planes between calls; set_weight_cache(true) declares every
    // matrix static; a static matrix overwritten in place by other means is announced with weights_changed.
    void weights_static(const float* plain_mat, size_t bytes, bool is_static = true) {
        check(pcmm_weights_static(handle, plain_mat, bytes, is_static ? 1 : 0), "pcmm_weights_static");
    }
    void set_weight_cache(bool enabled) { check(pcmm_set_weight_cache(handle, enabled ? 1 : 0), "pcmm_set_weight_cache"); }
    void weights_changed(const float* plain_mat = nullptr) { check(pcmm_weights_changed(handle, plain_mat), "pcmm_weights_changed"); }
    // PCMM_Context.h: size-N1 transforms over the ring-pack primes, data = [mod_batch_size][mod_num][poly_num][N1]
    void ToNTTInplace(uint64_tt* data, int poly_num, int mod_num, int start_poly_idx, int start_mod_idx, int mod_batch_size) {
        check(pcmm_ntt_fwd(handle, data, poly_num, mod_num, start_poly_idx, start_mod_idx, mod_batch_size), "PCMM_Context::ToNTTInplace");
    }
    void FromNTTInplace(uint64_tt* data, int poly_num, int mod_num, int start_poly_idx, int start_mod_idx, int mod_batch_size) {
        check(pcmm_ntt_inv(handle, data, poly_num, mod_num, start_poly_idx, start_mod_idx, mod_batch_size), "PCMM_Context::FromNTTInplace");
    }
    // PCMM_Context::decodeCoeffs (PCMM_Context.cuh:165-178); vals: N1 device doubles
    void decodeCoeffs(MLWEPlaintext& msg, double* vals) {
        uint64_tt* scratch = device_alloc_words((size_t)N1 * (msg.l + 1));
        int rc = pcmm_decode_coeffs(handle, vals, msg.mx_device, scratch, (long long)msg.scale, msg.l);
        device_release(scratch);
        check(rc, "decodeCoeffs");
    }
};

// The rlweCipherDecompose / PPMM members of PCMM_Scheme (pcmm/PCMM_Scheme.h:12-48).
class PCMM_Scheme {
public:
    PCMM_Context& pcmm_context;
    Scheme_23& scheme;
    uint64_tt* ppmm_output = nullptr;          // [mat_M][ringpack_q_count][(rank+1)*N1] (PCMM_Scheme.cuh:20)
    size_t ppmm_output_words = 0;

    uint64_tt* embeded_mlwe_buffer = nullptr;  // (rank+1) big polynomials over [p0 | q0] (PCMM_Scheme.cuh:12)
    uint64_tt* mult_key_output = nullptr;      // 4 limbs; the reference borrows scheme.modUp_TtoQj_buffer (PCMM_Scheme.cuh:394)
    uint64_tt* repackingKeys = nullptr;        // rank keys [a | b] over [p0 | q0], NTT domain, one buffer (PCMM_Scheme.cuh:166-176)
    bool own_keys = false;

    PCMM_Scheme(PCMM_Context& pcmm_context, Scheme_23& scheme) : pcmm_context(pcmm_context), scheme(scheme) {
        const size_t N = (size_t)scheme.context.N;
        embeded_mlwe_buffer = device_alloc_words((size_t)(pcmm_context.mlwe_rank + 1) * N * (pcmm_context.ringpack_pq_count - 1));
        mult_key_output = device_alloc_words(2 * N * (pcmm_context.ringpack_pq_count - 1));
    }
    // The reference's signature (PCMM_Scheme.h:19).  It keeps the secret key only for coeffBitRev, a debugging member that
    // decrypts and encrypts again (PCMM_Scheme.cuh:515-528) and is not part of this library, so the key is not kept here.
    PCMM_Scheme(PCMM_Context& pcmm_context, Scheme_23& scheme, SecretKey&) : PCMM_Scheme(pcmm_context, scheme) {}
    PCMM_Scheme(const PCMM_Scheme&) = delete;
    ~PCMM_Scheme() {
        device_release(ppmm_output);
        device_release(embeded_mlwe_buffer);
        device_release(mult_key_output);
        if (own_keys) device_release(repackingKeys);
    }

    // PCMM_Scheme::convertMLWESKfromRLWESK (PCMM_Scheme.cuh:23-48)
    void convertMLWESKfromRLWESK(MLWESecretKey& mlwe_sk, SecretKey& rlwe_sk) {
        check(pcmm_convert_mlwe_sk(pcmm_context.handle, mlwe_sk.sx_device, rlwe_sk.sx_device), "convertMLWESKfromRLWESK");
    }
    // PCMM_Scheme::addRepakcingKey (PCMM_Scheme.cuh:126-224): the keys go to repackingKeys (owned), key i at i*2*m*N words;
    // key i draws from the context's stream under the nonce rng_nonce + 1 + i
    void addRepakcingKey(MLWESecretKey& mlwe_sk, SecretKey& rlwe_sk) {
        if (repackingKeys) { std::cout << "repacking keys already generated!" << std::endl; return; }      // :152-155
        Context_23& c = scheme.context;
        const size_t N = (size_t)c.N, m = (size_t)pcmm_context.ringpack_pq_count - 1;
        uint64_tt* keys = device_alloc_words(N * m * 2 * pcmm_context.mlwe_rank);
        uint64_tt* scratch = device_alloc_words(N * (m + 1));
        int rc = pcmm_add_repacking_key(pcmm_context.handle, keys, mlwe_sk.sx_device, rlwe_sk.sx_device, c.rng_key, c.rng_nonce + 1, scratch);
        c.rng_nonce += (uint64_t)pcmm_context.mlwe_rank;
        device_release(scratch);
        if (rc != CKKS_OK) device_release(keys);
        check(rc, "addRepakcingKey");
        repackingKeys = keys;
        own_keys = true;
    }
    // PCMM_Scheme::mlweDecrypt (PCMM_Scheme.cuh:557-576)
    void mlweDecrypt(MLWECiphertext& mlwe_cipher, MLWESecretKey& mlwe_sk, MLWEPlaintext& mlwe_plain) {
        mlwe_plain.l = mlwe_cipher.l;
        check(pcmm_mlwe_decrypt(pcmm_context.handle, mlwe_plain.mx_device, mlwe_cipher.cipher_device, mlwe_sk.sx_device, mlwe_cipher.l), "mlweDecrypt");
    }

    // PCMM_Scheme::mlweCipherPacking (PCMM_Scheme.cuh:361-425): k MLWE samples -> 1 RLWE ciphertext with the repacking keys
    // (from addRepakcingKey, or installed by the caller in repackingKeys).
    void mlweCipherPacking(Ciphertext& rlwe_cipher, std::vector<MLWECiphertext*> mlwe_cipher_decomposed, uint64_tt mlwe_num,
                           uint64_tt offset) {
        if (!repackingKeys) throw std::invalid_argument("mlweCipherPacking: repacking keys not exists");
        if (offset + mlwe_num > mlwe_cipher_decomposed.size()) throw std::invalid_argument("mlweCipherPacking: offset + mlwe_num exceeds the vector");
        std::vector<const uint64_tt*> ptrs(mlwe_num);
        for (uint64_tt i = 0; i < mlwe_num; i++) ptrs[i] = mlwe_cipher_decomposed[offset + i]->cipher_device;
        check(pcmm_mlwe_pack(pcmm_context.handle, rlwe_cipher.cipher_device, ptrs.data(), (int)mlwe_num, repackingKeys,
                             embeded_mlwe_buffer, mult_key_output), "mlweCipherPacking");
        rlwe_cipher.l = pcmm_context.ringpack_q_count - 1 - 1;                       // :407-409
        rlwe_cipher.scale = mlwe_cipher_decomposed[0]->scale;
    }

    // PCMM_Scheme::rlweCipherDecompose (PCMM_Scheme.cuh:90-125).  Shape errors print and return, as the reference (:103-106).
    void rlweCipherDecompose(Ciphertext& rlwe_cipher, std::vector<MLWECiphertext*> mlwe_cipher_decomposed, uint64_tt mlwe_num,
                             uint64_tt offset) {
        if (mlwe_num > (uint64_tt)pcmm_context.mlwe_rank) {
            std::cout << "rlweCipherDecompose extract number muse <= mlwe_rank" << std::endl;
            return;
        }
        if (offset + mlwe_num > mlwe_cipher_decomposed.size()) throw std::invalid_argument("rlweCipherDecompose: offset + mlwe_num exceeds the vector");
        std::vector<uint64_tt*> ptrs(mlwe_num);
        for (uint64_tt i = 0; i < mlwe_num; i++) ptrs[i] = mlwe_cipher_decomposed[offset + i]->cipher_device;
        check(pcmm_rlwe_decompose_ntt(pcmm_context.handle, rlwe_cipher.cipher_device, ptrs.data(), (int)mlwe_num, rlwe_cipher.l),
              "rlweCipherDecompose");
    }

    // PCMM_Scheme::PPMM (PPMM_kernel.cuh:254-349): plain_mat is a DEVICE pointer to mat_M x mat_N fp32, row-major.
    // scaler = (long)(q_ringpack[1] * 2^49 / scale) (:283-284); afterwards row i of the product (first modulus) is copied
    // back into mlwe_cipher_decomposed[i] and its scale becomes scale * scaler / q_ringpack[1] (:345-348).
    void PPMM(float* plain_mat, std::vector<MLWECiphertext*> mlwe_cipher_decomposed, int mat_M, int mat_N, int mat_K, int mlwe_num) {
        if (mat_K != pcmm_context.N1) { std::cout << "matrix K should be equal to N1!" << std::endl; return; }
        if (mat_N != mlwe_num) { std::cout << "matrix N should be equal to mlwe number!" << std::endl; return; }
        const int mod_num = pcmm_context.ringpack_q_count;
        const size_t C = (size_t)pcmm_context.N1 * (pcmm_context.mlwe_rank + 1);
        const size_t need = (size_t)mat_M * mod_num * C;
        if (need > ppmm_output_words) {
            device_release(ppmm_output);
            ppmm_output = device_alloc_words(need);
            ppmm_output_words = need;
        }
        std::vector<const uint64_tt*> ptrs(mlwe_num);
        for (int i = 0; i < mlwe_num; i++) ptrs[i] = mlwe_cipher_decomposed[i]->cipher_device;
        const long scaler = (long)((long double)pcmm_context.q_ringpack[1] * ppmm_target_scale / mlwe_cipher_decomposed[0]->scale);
        last_scaler = scaler;
        check(pcmm_ppmm(pcmm_context.handle, plain_mat, ptrs.data(), ppmm_output, mat_M, mat_N, mod_num, (double)scaler), "PPMM");
        const int rows = mat_M < mlwe_num ? mat_M : mlwe_num;
        for (int i = 0; i < rows; i++) {
            mlwe_cipher_decomposed[i]->scale = mlwe_cipher_decomposed[i]->scale * scaler / (long double)pcmm_context.q_ringpack[1];
            check(ckks_memcpy_d2d(mlwe_cipher_decomposed[i]->cipher_device, ppmm_output + (size_t)i * C * mod_num, sizeof(uint64_tt) * C),
                  "PPMM copy back");
        }
    }
    long last_scaler = 0;
    // scale of the product rows; the reference fixes 2^49 (PPMM_kernel.cuh:283), which suits its 50- to 60-bit ring-pack primes; a
    // caller with shorter primes lowers it so that the rows stay below q_ringpack[0] / 2
    long double ppmm_target_scale = (long double)(1ll << 49);

    // The same layer step without 8-byte MLWE samples in between (no counterpart in the reference, where rlweCipherDecompose and PPMM
    // run back to back, Bert.cuh:411-424): the gather writes the operand digit planes of the MFMA kernel directly.
    //   packedBegin(mat_N)                                   opens the planes for mat_N samples (a multiple of 64)
    //   rlweCipherDecomposePacked(cipher, mlwe_num, offset, take)  the first take (default all) of a ciphertext's mlwe_num samples -> samples offset ..
    //   PPMMPacked(plain_mat, rows, mat_M)                   the product; row i (first modulus) lands in rows[i] as PPMM leaves it
    void packedBegin(int mat_N) {
        packed_N = mat_N;
        check(pcmm_packed_begin(pcmm_context.handle, mat_N, pcmm_context.ringpack_q_count), "packedBegin");
    }
    void rlweCipherDecomposePacked(Ciphertext& rlwe_cipher, uint64_tt mlwe_num, uint64_tt offset, uint64_tt take = 0) {
        packed_scale = rlwe_cipher.scale;
        check(pcmm_rlwe_decompose_packed(pcmm_context.handle, rlwe_cipher.cipher_device, (int)offset, (int)mlwe_num, (int)(take ? take : mlwe_num),
                                         rlwe_cipher.l), "rlweCipherDecomposePacked");
    }
    void PPMMPacked(float* plain_mat, const std::vector<MLWECiphertext*>& rows, int mat_M) {
        const int mod_num = pcmm_context.ringpack_q_count;
        const size_t C = (size_t)pcmm_context.N1 * (pcmm_context.mlwe_rank + 1);
        const size_t need = (size_t)mat_M * mod_num * C;
        if (need > ppmm_output_words) {
            device_release(ppmm_output);
            ppmm_output = device_alloc_words(need);
            ppmm_output_words = need;
        }
        const long scaler = (long)((long double)pcmm_context.q_ringpack[1] * ppmm_target_scale / packed_scale);             // PPMM_kernel.cuh:283-284
        last_scaler = scaler;
        check(pcmm_ppmm_packed(pcmm_context.handle, plain_mat, ppmm_output, mat_M, (double)scaler), "PPMMPacked");
        const size_t n = rows.size() < (size_t)mat_M ? rows.size() : (size_t)mat_M;
        for (size_t i = 0; i < n; i++) {
            rows[i]->scale = packed_scale * scaler / (long double)pcmm_context.q_ringpack[1];
            check(ckks_memcpy_d2d(rows[i]->cipher_device, ppmm_output + i * C * mod_num, sizeof(uint64_tt) * C), "PPMMPacked copy back");
        }
    }
    int packed_N = 0;
    long double packed_scale = 0;
};

}  // namespace ckks_llm_amd
