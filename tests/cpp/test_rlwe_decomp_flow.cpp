// The reference's own test program for the ring-packed PCMM path (test_rlwe_decomp.cu:23-198), rewritten against the C++ host
// mirror with the same object names and the same order of calls, on the reference's logN = 15 prime set (Params.cuh) at
// N = 2^12, N1 = 256: keys, encode_coeffs, encryptMsg, rlweCipherDecompose, mlweDecrypt + decodeCoeffs of a sample, decryptMsg +
// decode_coeffs of the input, PPMM, mlweCipherPacking, decryptMsg + decode_coeffs of the result, and the comparison with the
// plain product that the reference prints through GetPrecisionStats (:195) - here asserted.  Needs a GPU.  Exit code 0 = passed.
#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <random>
#include <unistd.h>
#include <vector>

#include "../../include/ckks_llm_amd.hpp"

using namespace ckks_llm_amd;

static int failures = 0;
#define EXPECT(cond, what)                                                      \
    do {                                                                        \
        if (!(cond)) { printf("FAIL %s (line %d)\n", what, __LINE__); failures++; } \
        else printf("ok   %s\n", what);                                         \
    } while (0)

static double* device_doubles(const std::vector<double>& h) {
    void* p = nullptr;
    check(ckks_malloc(&p, h.size() * 8), "malloc");
    check(ckks_memcpy_h2d(p, h.data(), h.size() * 8), "h2d");
    return static_cast<double*>(p);
}
static std::vector<double> host_doubles(const double* d, size_t n) {
    std::vector<double> h(n);
    check(ckks_memcpy_d2h(h.data(), d, n * 8), "d2h");
    return h;
}
// worst and mean precision in bits, from GetPrecisionStats as the reference's program calls it (test_rlwe_decomp.cu:195)
static void precision_bits(const std::vector<double>& got, const std::vector<double>& want, double& worst, double& mean, bool print = false) {
    const PrecisionStats st = GetPrecisionStats(got, want);
    if (print) printf("%s", st.String().c_str());
    worst = st.MinPrecision.Real;
    mean = st.MeanPrecision.Real;
}

static int run() {
    // Params.cuh, logN = 15: q (12 primes near 2^49), p (4), t (7), gamma 4, precision 2^49; all are 1 mod 2^16, so they also serve N = 2^12
    const std::vector<uint64_tt> q = {0x20000018e0001ull, 0x2000001c00001ull, 0x2000001ca0001ull, 0x2000001d20001ull, 0x1fffffee80001ull, 0x1fffffede0001ull, 0x1fffffec40001ull, 0x1fffffe780001ull, 0x2000000ce0001ull, 0x20000013a0001ull, 0x20000013c0001ull, 0x20000015a0001ull};
    const std::vector<uint64_tt> p = {0x2000002600001ull, 0x20000027e0001ull, 0x2000002800001ull, 0x20000029e0001ull};
    const std::vector<uint64_tt> t = {0xffffffffffc0001ull, 0xfffffffff840001ull, 0xfffffffff6a0001ull, 0xfffffffff5a0001ull, 0xfffffffff2a0001ull, 0xfffffffff240001ull, 0xffffffffefe0001ull};
    const int logN = 12, PCMM_N1 = 256;
    Context_23 context(logN, p, q, t, 4);
    Scheme_23 scheme(context);
    const int N = (int)context.N, slots = N / 2, L = context.L;
    const int mlwe_rank = N / PCMM_N1;
    std::vector<uint64_tt> p_ringpack = {context.pVec[context.p_num - 1]};
    std::vector<uint64_tt> q_ringpack = {context.qVec[0], context.qVec[1]};
    const int q_ringpack_count = (int)q_ringpack.size();
    const long double precision = (long double)(1ll << 49);             // Params.cuh:58

    SecretKey sk(context, 192);
    PCMM_Context pcmm_context(PCMM_N1, mlwe_rank, p_ringpack, q_ringpack, context);
    PCMM_Scheme pcmm_scheme(pcmm_context, scheme, sk);
    const int pq_ringpack_count = pcmm_context.ringpack_pq_count;
    MLWESecretKey mlwe_sk(PCMM_N1, pq_ringpack_count - 1, mlwe_rank);
    pcmm_scheme.convertMLWESKfromRLWESK(mlwe_sk, sk);
    scheme.addEncKey(sk);
    pcmm_scheme.addRepakcingKey(mlwe_sk, sk);

    std::mt19937_64 rng(1);
    std::uniform_real_distribution<double> msg_dist(-0.1, 0.1);
    std::uniform_real_distribution<float> randnum(-1.f / 10, 1.f / 10);
    std::vector<double> real_mes_host(N);
    for (double& v : real_mes_host) v = msg_dist(rng);
    double* real_msg1 = device_doubles(real_mes_host);

    const int target_level = 1;
    const int mat_M = mlwe_rank, mat_N = mlwe_rank;
    std::vector<float> plain_mat_host((size_t)mat_M * mat_N);
    for (float& w : plain_mat_host) w = randnum(rng);
    std::vector<double> plain_gemm_host(N, 0.0);
    for (int idx_M = 0; idx_M < mat_M; idx_M++)                                              // test_rlwe_decomp.cu:86-92
        for (int idx_K = 0; idx_K < PCMM_N1; idx_K++)
            for (int idx_N = 0; idx_N < mat_N; idx_N++)
                plain_gemm_host[idx_M + idx_K * mat_M] += plain_mat_host[idx_N + idx_M * mat_N] * real_mes_host[idx_N + idx_K * mat_N];
    void* plain_mat_device = nullptr;
    check(ckks_malloc(&plain_mat_device, plain_mat_host.size() * 4), "malloc W");
    check(ckks_memcpy_h2d(plain_mat_device, plain_mat_host.data(), plain_mat_host.size() * 4), "h2d W");

    const int decomp_num = N / PCMM_N1;
    std::vector<MLWECiphertext*> mlwe_cipher_decomposed;
    for (int i = 0; i < decomp_num; i++) mlwe_cipher_decomposed.push_back(new MLWECiphertext(PCMM_N1, q_ringpack_count - 1, q_ringpack_count - 1, mlwe_rank, precision));
    Plaintext plain_m1_coeffs_encode(N, L, target_level, slots, precision), m1_dec(N, L, target_level, slots, precision), m2_dec(N, L, target_level, slots, precision);
    MLWEPlaintext mlwe_dec(PCMM_N1, q_ringpack_count - 1, q_ringpack_count - 1, precision);
    Ciphertext c1(N, L, L, slots, precision), c2(N, L, L, slots, precision);
    double* real_msg_dec = device_doubles(std::vector<double>(N, 0.0));
    double* mlwe_msg_dec = device_doubles(std::vector<double>(PCMM_N1, 0.0));

    context.encode_coeffs(real_msg1, plain_m1_coeffs_encode);
    scheme.encryptMsg(c1, plain_m1_coeffs_encode);
    pcmm_scheme.rlweCipherDecompose(c1, mlwe_cipher_decomposed, decomp_num, 0);

    double worst = 0, mean = 0;
    for (int i = 0; i < 4; i++) {                                                            // the program's commented-out check (:143-151)
        pcmm_scheme.mlweDecrypt(*mlwe_cipher_decomposed[i], mlwe_sk, mlwe_dec);
        pcmm_context.decodeCoeffs(mlwe_dec, mlwe_msg_dec);
        std::vector<double> got = host_doubles(mlwe_msg_dec, PCMM_N1), want(PCMM_N1);
        for (int n = 0; n < PCMM_N1; n++) want[n] = real_mes_host[i + n * mlwe_rank];
        precision_bits(got, want, worst, mean);
        EXPECT(worst > 30, "MLWE sample decrypts to the strided coefficients of the message");
    }
    scheme.decryptMsg(m1_dec, sk, c1);
    context.decode_coeffs(m1_dec, real_msg_dec);
    precision_bits(host_doubles(real_msg_dec, N), real_mes_host, worst, mean);
    printf("decrypt(encrypt(m)): worst %.1f bits, mean %.1f bits\n", worst, mean);
    EXPECT(worst > 30, "coeff message_dec2 == message");

    pcmm_scheme.PPMM((float*)plain_mat_device, mlwe_cipher_decomposed, mat_M, mat_N, PCMM_N1, decomp_num);
    pcmm_scheme.mlweCipherPacking(c2, mlwe_cipher_decomposed, decomp_num, 0);
    scheme.decryptMsg(m2_dec, sk, c2);
    context.decode_coeffs(m2_dec, real_msg_dec);
    std::vector<double> real_values_computed = host_doubles(real_msg_dec, N);
    precision_bits(real_values_computed, plain_gemm_host, worst, mean, true);      // the table the reference prints (:195-196)
    printf("repacking decrypt vs plain gemm: worst %.1f bits, mean %.1f bits (scale 2^%.1f)\n", worst, mean, (double)std::log2((double)c2.scale));
    double biggest = 0;
    for (double v : plain_gemm_host) biggest = std::max(biggest, std::fabs(v));
    EXPECT(biggest > 0.02 && worst > 20, "PPMM + mlweCipherPacking decrypts to W times the message (GetPrecisionStats > 20 bits)");

    for (MLWECiphertext* m : mlwe_cipher_decomposed) delete m;
    ckks_free(plain_mat_device);
    ckks_free(real_msg1);
    ckks_free(real_msg_dec);
    ckks_free(mlwe_msg_dec);
    return failures;
}

int main() {
    setvbuf(stdout, nullptr, _IONBF, 0);
    const int failed = run();
    printf(failed ? "FAILED: %d check(s)\n" : "the reference's PCMM test flow passed\n", failed);
    fflush(stdout);
    _exit(failed ? 1 : 0);          // skip the exit handlers of the HIP runtime (their order at process exit is not defined)
}
