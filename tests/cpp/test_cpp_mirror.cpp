// Parity test of the C++ host mirror (include/ckks_llm_amd.hpp) in the style of the reference's own test programs
// (test_rlwe_decomp.cu, ntt_throughput.cu): build objects, call the member functions, compare - but against the CPU
// oracle, bit for bit, and with assertions instead of prints.  Needs a GPU.  Exit code 0 = all checks passed.
#include <cstdio>
#include <cstdlib>
#include <cmath>
#include <cstring>
#include <algorithm>
#include <unistd.h>
#include <random>
#include <vector>

#include "../../include/ckks_llm_amd.hpp"
#include "../../oracle/ckks_oracle.h"

using namespace ckks_llm_amd;

static int failures = 0;
#define EXPECT(cond, what)                                                      \
    do {                                                                        \
        if (!(cond)) { printf("FAIL %s (line %d)\n", what, __LINE__); failures++; } \
        else printf("ok   %s\n", what);                                         \
    } while (0)

static std::vector<uint64_tt> uniform_limbs(std::mt19937_64& rng, const std::vector<uint64_tt>& primes, int polys, long N) {
    std::vector<uint64_tt> v((size_t)polys * primes.size() * N);
    for (int y = 0; y < polys; y++)
        for (size_t j = 0; j < primes.size(); j++)
            for (long i = 0; i < N; i++) v[((size_t)y * primes.size() + j) * N + i] = rng() % primes[j];
    return v;
}
static void upload(uint64_tt* dev, const std::vector<uint64_tt>& h) { check(ckks_memcpy_h2d(dev, h.data(), h.size() * 8), "h2d"); }
static std::vector<uint64_tt> download(const uint64_tt* dev, size_t words) {
    std::vector<uint64_tt> h(words);
    check(ckks_memcpy_d2h(h.data(), dev, words * 8), "d2h");
    return h;
}

static int run() {
    // the four largest primes below 2^36 that are 1 mod 2^13 (N = 2^12), as in BASELINE config 1
    const std::vector<uint64_tt> q = {0xffffee001ull, 0xffffc4001ull, 0xffffbe001ull, 0xffffba001ull};
    const int logN = 12;
    const long N = 1l << logN;
    std::mt19937_64 rng(7);

    Context_23 context(logN, {}, q);
    orc_ctx* orc = orc_ctx_create(logN, nullptr, 0, q.data(), (int)q.size(), nullptr, 0, 0);
    Scheme_23 scheme(context);

    // ---- ToNTTInplace / FromNTTInplace on a ciphertext (2 polys x 4 limbs), reference addressing ----
    Ciphertext ct((int)N, context.L, context.L, (int)(N / 2), (long double)(1ll << 40));
    std::vector<uint64_tt> h = uniform_limbs(rng, q, 2, N), want = h;
    upload(ct.cipher_device, h);
    context.ToNTTInplace(ct.cipher_device, 0, context.K, 2, context.L + 1, context.L + 1);
    orc_ntt_fwd(orc, want.data(), 0, 0, 2, (int)q.size(), (int)q.size());
    EXPECT(download(ct.cipher_device, h.size()) == want, "ToNTTInplace == oracle");
    context.FromNTTInplace(ct.cipher_device, 0, context.K, 2, context.L + 1, context.L + 1);
    EXPECT(download(ct.cipher_device, h.size()) == h, "FromNTTInplace(ToNTTInplace(x)) == x");

    // ---- the reference's own constructor: Context_23(logN, logslots, h, sigma) picks the compiled-in set (Params.cuh:11-30) ----
    {
        Context_23 ref13(13, 12);
        EXPECT(ref13.q_num == 5 && ref13.p_num == 1 && ref13.t_num == 3 && ref13.gamma == 3 && ref13.slots == 4096 &&
               ref13.qVec[0] == 0x4001b00001ull && ref13.pVec[0] == 0x10a19000001ull && ref13.tVec[2] == 0xfffffffff6a0001ull &&
               ref13.precision == (1l << 36) && ref13.h == 64 && ref13.dnum == 5,
               "Context_23(13, 12) holds the reference's logN = 13 set");
        const long n13 = ref13.N;
        orc_ctx* o13 = orc_ctx_create(13, ref13.pVec.data(), 1, ref13.qVec.data(), 5, ref13.tVec.data(), 3, 3);
        std::vector<uint64_tt> all = ref13.pVec;
        all.insert(all.end(), ref13.qVec.begin(), ref13.qVec.end());
        all.insert(all.end(), ref13.tVec.begin(), ref13.tVec.end());
        std::vector<uint64_tt> x = uniform_limbs(rng, all, 1, n13), w = x;
        uint64_tt* d = device_alloc_words(x.size());
        upload(d, x);
        ref13.ToNTTInplace(d, 0, 0, 1, (int)all.size(), (int)all.size());           // all nine primes in pqt order
        orc_ntt_fwd(o13, w.data(), 0, 0, 1, (int)all.size(), (int)all.size());
        EXPECT(download(d, x.size()) == w, "ToNTTInplace over [P | Q | T] of the logN = 13 set == oracle");
        device_release(d);
        orc_ctx_destroy(o13);
        bool bad_h = false, bad_n = false;
        try { Context_23 c(13, 12, 100); } catch (const std::invalid_argument&) { bad_h = true; }
        try { Context_23 c(12, 11); } catch (const std::invalid_argument&) { bad_n = true; }
        EXPECT(bad_h && bad_n, "Hamming weight other than 64 / 192 and an unknown logN throw std::invalid_argument");
    }

    // ---- rescaleAndEqual: level L -> L-1 against the oracle, then std::invalid_argument at level 0 ----
    upload(ct.cipher_device, want);                       // NTT-domain content
    std::vector<uint64_tt> want_rs = want;
    orc_rescale(orc, want_rs.data(), context.L);
    scheme.rescaleAndEqual(ct);
    EXPECT(download(ct.cipher_device, h.size()) == want_rs && ct.l == context.L - 1, "rescaleAndEqual == oracle, level drops");
    Ciphertext ct0((int)N, context.L, 0, (int)(N / 2), 1.0L);
    bool threw = false;
    try { scheme.rescaleAndEqual(ct0); } catch (const std::invalid_argument&) { threw = true; }
    EXPECT(threw, "rescaleAndEqual on level 0 throws std::invalid_argument");

    // ---- rlweCipherDecompose + PPMM (N1 = 128, rank 32: N = N1 * rank), two ring-pack primes ----
    const int N1 = 128, rank = 32, mlwe_num = 16, M = 16;
    const std::vector<uint64_tt> q_rp = {q[0], q[1]};
    PCMM_Context pcmm_context(N1, rank, {}, q_rp, context);
    PCMM_Scheme pcmm_scheme(pcmm_context, scheme);
    orc_pcmm* orc_p = orc_pcmm_create(orc, N1, rank, nullptr, 0, q_rp.data(), 2);
    Ciphertext rlwe((int)N, context.L, 1, (int)(N / 2), (long double)(1ll << 36));     // level 1: primes q0, q1
    std::vector<uint64_tt> rl = uniform_limbs(rng, q, 2, N);
    upload(rlwe.cipher_device, rl);
    std::vector<MLWECiphertext*> mlwe;
    for (int i = 0; i < mlwe_num; i++) mlwe.push_back(new MLWECiphertext(N1, 1, 1, rank, rlwe.scale));
    pcmm_scheme.rlweCipherDecompose(rlwe, mlwe, mlwe_num, 0);
    // oracle: iNTT of the level-1 limbs, gather
    std::vector<uint64_tt> rl_coeff = rl;
    orc_ntt_inv(orc, rl_coeff.data(), 0, 0, 2, 2, (int)q.size());
    const size_t mlwe_words = (size_t)2 * (rank + 1) * N1;
    std::vector<std::vector<uint64_tt>> om(mlwe_num, std::vector<uint64_tt>(mlwe_words));
    std::vector<uint64_tt*> omp(mlwe_num);
    for (int i = 0; i < mlwe_num; i++) omp[i] = om[i].data();
    orc_rlwe_decompose(orc_p, rl_coeff.data(), omp.data(), mlwe_num, 1);
    bool same = true;
    for (int i = 0; i < mlwe_num; i++) same = same && download(mlwe[i]->cipher_device, mlwe_words) == om[i];
    EXPECT(same, "rlweCipherDecompose == oracle");
    EXPECT(download(rlwe.cipher_device, rl.size()) == rl, "rlweCipherDecompose leaves the RLWE ciphertext in NTT form");

    std::vector<float> W((size_t)M * mlwe_num);
    std::normal_distribution<float> nd(0.f, 0.02f);
    for (float& w : W) w = nd(rng);
    void* Wd = nullptr;
    check(ckks_malloc(&Wd, W.size() * 4), "malloc W");
    check(ckks_memcpy_h2d(Wd, W.data(), W.size() * 4), "h2d W");
    const long double scale0 = mlwe[0]->scale;
    const long scaler = (long)((long double)q_rp[1] * (long double)(1ll << 49) / scale0);
    const size_t C = (size_t)(rank + 1) * N1;
    std::vector<uint64_tt> oout((size_t)M * 2 * C);
    std::vector<const uint64_tt*> ocp(mlwe_num);
    for (int i = 0; i < mlwe_num; i++) ocp[i] = om[i].data();
    orc_ppmm(orc_p, W.data(), ocp.data(), oout.data(), M, mlwe_num, 2, (double)scaler, 0, (long)C);
    pcmm_scheme.PPMM((float*)Wd, mlwe, M, mlwe_num, N1, mlwe_num);
    EXPECT(pcmm_scheme.last_scaler == scaler, "PPMM scaler = q_ringpack[1] * 2^49 / scale");
    same = true;
    for (int i = 0; i < M; i++) {
        std::vector<uint64_tt> row = download(mlwe[i]->cipher_device, C);
        same = same && std::memcmp(row.data(), oout.data() + (size_t)i * 2 * C, C * 8) == 0;
    }
    EXPECT(same, "PPMM rows copied back == oracle (first modulus, fused rescale)");
    EXPECT(download(pcmm_scheme.ppmm_output, oout.size()) == oout, "PPMM output buffer == oracle (all moduli)");
    const long double want_scale = scale0 * scaler / (long double)q_rp[1];
    EXPECT(mlwe[0]->scale == want_scale, "PPMM updates the scale as the reference");
    // shape errors: message and no work, as the reference
    std::vector<uint64_tt> before = download(mlwe[0]->cipher_device, C);
    pcmm_scheme.PPMM((float*)Wd, mlwe, M, mlwe_num, N1 + 1, mlwe_num);
    pcmm_scheme.PPMM((float*)Wd, mlwe, M, mlwe_num - 1, N1, mlwe_num);
    EXPECT(download(mlwe[0]->cipher_device, C) == before, "PPMM shape errors do no work");

    // mlweCipherPacking without repacking keys: std::invalid_argument, as a missing key in the reference (KeySwitch_23.cuh:198-201)
    threw = false;
    try { pcmm_scheme.mlweCipherPacking(rlwe, mlwe, mlwe_num, 0); } catch (const std::invalid_argument&) { threw = true; }
    EXPECT(threw, "mlweCipherPacking without keys throws std::invalid_argument");

    // ---- SecretKey, addEncKey, encode_coeffs, encryptMsg, decryptMsg, decode_coeffs: the context's stream is Salsa20 under its
    //      key (set to zero here; a fresh context holds random bytes) with nonces 1, 2, 3 for the three draws, so the oracle can follow word for word ----
    {
        const int h = 64, L1 = context.L + 1;
        const uint8_t zero_key[32] = {0};
        for (int i = 0; i < 32; i++) context.rng_key[i] = 0;       // a fixed key, as a program that must repeat a run sets it
        context.rng_nonce = 0;
        SecretKey sk(context, h);
        std::vector<uint8_t> r1(5 * h), r2(8 * N * L1 + 4 * N), r3(9 * N);
        orc_salsa20_stream(r1.data(), r1.size(), zero_key, 1);
        orc_salsa20_stream(r2.data(), r2.size(), zero_key, 2);
        orc_salsa20_stream(r3.data(), r3.size(), zero_key, 3);
        std::vector<uint64_tt> o_sx((size_t)N * L1), o_pk((size_t)2 * N * L1), o_mx((size_t)N * L1), o_ct((size_t)2 * N * L1, 0), o_dec((size_t)N * L1);
        orc_keygen_secret(orc, o_sx.data(), r1.data(), h);
        EXPECT(download(sk.sx_device, o_sx.size()) == o_sx, "SecretKey == oracle");
        scheme.addEncKey(sk);
        orc_keygen_public(orc, o_pk.data(), o_sx.data(), r2.data(), r2.data() + 8 * N * L1);
        EXPECT(download(scheme.publicKey->cipher_device, o_pk.size()) == o_pk, "addEncKey == oracle");
        std::vector<double> vals(N);
        std::uniform_real_distribution<double> ud(-3.0, 3.0);
        for (double& v : vals) v = ud(rng);
        void* vd = nullptr;
        check(ckks_malloc(&vd, N * 8), "malloc vals");
        check(ckks_memcpy_h2d(vd, vals.data(), N * 8), "h2d vals");
        Plaintext msg((int)N, context.L, 2, (int)(N / 2), (long double)(1ll << 40));
        context.encode_coeffs((const double*)vd, msg);
        orc_encode_coeffs(orc, o_mx.data(), vals.data(), 1l << 40, 2);
        EXPECT(download(msg.mx_device, (size_t)3 * N) == std::vector<uint64_tt>(o_mx.begin(), o_mx.begin() + 3 * N), "encode_coeffs == oracle");
        Ciphertext enc((int)N, context.L, context.L, (int)(N / 2), 1.0L);
        check(ckks_memset(enc.cipher_device, 0, o_ct.size() * 8), "memset");
        scheme.encryptMsg(enc, msg);
        orc_encrypt(orc, o_ct.data(), o_mx.data(), o_pk.data(), r3.data(), 2);
        EXPECT(download(enc.cipher_device, o_ct.size()) == o_ct && enc.l == 2 && enc.scale == msg.scale, "encryptMsg == oracle, level and scale follow");
        Plaintext dec((int)N, context.L, context.L, 1, 1.0L);
        scheme.decryptMsg(dec, sk, enc);
        orc_decrypt(orc, o_dec.data(), o_ct.data(), o_sx.data(), 2);
        EXPECT(download(dec.mx_device, o_dec.size()) == o_dec && dec.l == 2 && dec.slots == (int)(N / 2), "decryptMsg == oracle");
        context.decode_coeffs(dec, (double*)vd);
        std::vector<double> back(N);
        check(ckks_memcpy_d2h(back.data(), vd, N * 8), "d2h vals");
        double worst = 0;
        for (long i = 0; i < N; i++) worst = std::max(worst, std::fabs(back[i] - vals[i]));
        EXPECT(worst > 0 && worst <= 19.0 * (N + h + 2) / (double)(1ll << 40), "decode_coeffs(decrypt(encrypt(encode(x)))) = x up to the encryption noise");
        Scheme_23 bare(context);
        threw = false;
        try { bare.encryptZero(enc, 1, 1); } catch (const std::invalid_argument&) { threw = true; }
        EXPECT(threw, "encryptZero without a public key throws std::invalid_argument");
        ckks_free(vd);
    }

    // ---- the reference's logN = 13 parameter set (5 q, 1 p, 3 t, gamma 3; Params.cuh) at N = 2^10: keys in the T basis,
    //      mult_23, leftRotate_23, conjugate_23 against the oracle, word for word on the same stream ----
    {
        const std::vector<uint64_tt> q13 = {0x4001b00001ull, 0xfff9c0001ull, 0xfff8e0001ull, 0xfff840001ull, 0xfff700001ull};
        const std::vector<uint64_tt> p13 = {0x10a19000001ull};
        const std::vector<uint64_tt> t13 = {0xffffffffffc0001ull, 0xfffffffff840001ull, 0xfffffffff6a0001ull};
        const int lg = 10, h = 64;
        const long n = 1l << lg;
        Context_23 c2(lg, p13, q13, t13, 3);
        for (int i = 0; i < 32; i++) c2.rng_key[i] = 0;        // fixed key: the oracle follows the same stream
        orc_ctx* o2 = orc_ctx_create(lg, p13.data(), 1, q13.data(), 5, t13.data(), 3, 3);
        const int K = c2.K, L1 = c2.L + 1, KL = K + L1;
        const size_t keyw = (size_t)2 * c2.dnum * c2.Ri_blockNum * c2.t_num * n;
        const size_t na = (size_t)c2.dnum * 8 * n * KL, ne = (size_t)c2.dnum * 4 * n;
        const uint8_t zero_key[32] = {0};
        auto stream = [&](size_t bytes, uint64_t nonce) { std::vector<uint8_t> r(bytes); orc_salsa20_stream(r.data(), bytes, zero_key, nonce); return r; };
        Scheme_23 s2(c2);
        SecretKey sk(c2, h);                                   // nonce 1
        s2.addEncKey(sk);                                      // nonce 2
        s2.addMultKey_23(sk);                                  // nonce 3
        s2.addConjKey_23(sk);                                  // nonce 4
        s2.addLeftRotKey_23(sk, 7);                            // nonce 5
        std::vector<uint64_tt> o_sx((size_t)n * KL), o_pk((size_t)2 * n * L1), o_ss((size_t)n * KL), o_key(keyw);
        std::vector<uint8_t> r = stream(5 * h, 1);
        orc_keygen_secret(o2, o_sx.data(), r.data(), h);
        r = stream(8 * n * L1 + 4 * n, 2);
        orc_keygen_public(o2, o_pk.data(), o_sx.data(), r.data(), r.data() + 8 * n * L1);
        r = stream(na + ne, 3);
        orc_poly_op(o2, 0, o_ss.data(), o_sx.data(), o_sx.data(), 0, K, K, K, L1);
        orc_keygen_switch_23(o2, o_key.data(), o_sx.data(), o_ss.data(), r.data(), r.data() + na);
        EXPECT(download(s2.rlk_23->cipher_device, keyw) == o_key, "addMultKey_23 == oracle");
        std::vector<uint64_tt> o_rlk = o_key;
        r = stream(na + ne, 4);
        orc_conjugate_ntt(o2, o_ss.data(), o_sx.data(), 0, K, L1);
        orc_keygen_switch_23(o2, o_key.data(), o_sx.data(), o_ss.data(), r.data(), r.data() + na);
        EXPECT(download(s2.ConjKey_23->cipher_device, keyw) == o_key, "addConjKey_23 == oracle");
        std::vector<uint64_tt> o_conj = o_key;
        r = stream(na + ne, 5);
        orc_automorph_ntt(o2, o_ss.data(), o_sx.data(), orc_rot_group(o2, 7), 0, 0, KL);
        orc_keygen_switch_23(o2, o_key.data(), o_ss.data(), o_sx.data() + (size_t)n * K, r.data(), r.data() + na);
        EXPECT(download(s2.rotKey_vec_23[7]->cipher_device, keyw) == o_key, "addLeftRotKey_23 == oracle");
        // two ciphertexts (nonces 6, 7), then the three operations at the top level
        Plaintext m1((int)n, c2.L, c2.L, (int)(n / 2), (long double)(1 << 20)), m2((int)n, c2.L, c2.L, (int)(n / 2), (long double)(1 << 20));
        std::vector<uint64_tt> o_m1 = uniform_limbs(rng, q13, 1, n), o_m2 = uniform_limbs(rng, q13, 1, n);
        upload(m1.mx_device, o_m1);
        upload(m2.mx_device, o_m2);
        Ciphertext e1((int)n, c2.L, c2.L, 1, 1.0L), e2((int)n, c2.L, c2.L, 1, 1.0L), res((int)n, c2.L, c2.L, 1, 1.0L);
        s2.encryptMsg(e1, m1);
        s2.encryptMsg(e2, m2);
        std::vector<uint64_tt> o_c1((size_t)2 * n * L1), o_c2((size_t)2 * n * L1), o_res((size_t)2 * n * L1);
        r = stream(9 * n, 6);
        orc_encrypt(o2, o_c1.data(), o_m1.data(), o_pk.data(), r.data(), c2.L);
        r = stream(9 * n, 7);
        orc_encrypt(o2, o_c2.data(), o_m2.data(), o_pk.data(), r.data(), c2.L);
        EXPECT(download(e1.cipher_device, o_c1.size()) == o_c1 && download(e2.cipher_device, o_c2.size()) == o_c2, "two encryptions == oracle");
        s2.mult_23(res, e1, e2);
        orc_mult_23(o2, o_res.data(), o_c1.data(), o_c2.data(), o_rlk.data(), c2.L);
        EXPECT(download(res.cipher_device, o_res.size()) == o_res && res.scale == e1.scale * e2.scale, "mult_23 == oracle");
        s2.leftRotate_23(res, e1, 7);
        orc_rotate_23(o2, o_res.data(), o_c1.data(), o_key.data(), 7, c2.L);
        EXPECT(download(res.cipher_device, o_res.size()) == o_res, "leftRotate_23 == oracle");
        s2.conjugate_23(res, e1);
        orc_conjugate_23(o2, o_res.data(), o_c1.data(), o_conj.data(), c2.L);
        EXPECT(download(res.cipher_device, o_res.size()) == o_res, "conjugate_23 == oracle");
        threw = false;
        try { s2.leftRotate_23(res, e1, 8); } catch (const std::invalid_argument&) { threw = true; }
        EXPECT(threw, "leftRotate_23 without its key throws std::invalid_argument");
        Ciphertext lvl0((int)n, c2.L, 0, 1, 1.0L);
        threw = false;
        try { s2.mult_23(res, e1, lvl0); } catch (const std::invalid_argument&) { threw = true; }
        EXPECT(threw, "mult_23 on level 0 throws std::invalid_argument");
        // one baby-step / giant-step level of the slot <-> coefficient transforms through EncodingMatrix::EvalLevel, with the
        // rotation key generated above and random plaintexts over T, against the oracle's level on the same words
        {
            const int T = c2.t_num, b = 2, g = 2, numRotations = 3;
            std::vector<PlaintextT*> A;
            std::vector<std::vector<uint64_tt>> A_host;
            for (int i = 0; i < b * g; i++) {
                A.push_back(new PlaintextT((int)n, T, 1.0L));
                A_host.push_back(uniform_limbs(rng, t13, 1, n));
                upload(A.back()->mx_device, A_host.back());
            }
            const std::vector<int> rot_in = {0, 7}, rot_out = {0, 7};
            std::vector<const uint64_tt*> o_plain = {A_host[0].data(), A_host[1].data(), A_host[2].data(), nullptr};
            const int o_acc[2] = {2, 1};
            const uint64_tt* o_in_keys[2] = {nullptr, o_key.data()};
            const uint64_tt* o_out_keys[2] = {nullptr, o_key.data()};
            std::vector<uint64_tt> o_lvl = o_c1;
            orc_ntt_inv(o2, o_lvl.data(), 0, K, 2, L1, L1);
            orc_bsgs_level_23(o2, o_lvl.data(), c2.L, o_plain.data(), o_acc, rot_in.data(), o_in_keys, rot_out.data(), o_out_keys, b, g);
            orc_rescale_coeff(o2, o_lvl.data(), c2.L);
            Ciphertext lvl(e1);
            c2.FromNTTInplace(lvl.cipher_device, 0, K, 2, L1, L1);
            EncodingMatrix em(s2);
            em.EvalLevel(A, lvl, rot_in, rot_out, b, g, numRotations);
            std::vector<uint64_tt> got = download(lvl.cipher_device, o_lvl.size());
            bool same = lvl.l == c2.L - 1;
            for (int z = 0; z < 2 && same; z++)
                for (size_t w = 0; w < (size_t)n * (L1 - 1); w++)
                    if (got[(size_t)z * n * L1 + w] != o_lvl[(size_t)z * n * L1 + w]) { same = false; break; }
            EXPECT(same, "EncodingMatrix::EvalLevel (hoisted rotations + rescale) == oracle");
            threw = false;
            try { em.EvalLevel(A, lvl, {0, 9}, rot_out, b, g, numRotations); } catch (const std::invalid_argument&) { threw = true; }
            EXPECT(threw, "EvalLevel without a rotation key throws std::invalid_argument");
            for (PlaintextT* a : A) delete a;
        }
        orc_ctx_destroy(o2);
    }

    // ---- the layer step without 8-byte samples in between: packedBegin + rlweCipherDecomposePacked + PPMMPacked must leave what
    //      rlweCipherDecompose + PPMM leave (N = 2^13, N1 = 128, rank 64, two 36-bit ring-pack primes, 64 samples) ----
    {
        const std::vector<uint64_tt> q2 = {0xffff00001ull, 0xfff9c0001ull};
        const int lg = 13, n1 = 128;
        const long n = 1l << lg;
        const int rk = (int)(n / n1), rows_m = 32;
        Context_23 c3(lg, {}, q2);
        Scheme_23 s3(c3);
        PCMM_Context pc3(n1, rk, {}, q2, c3);
        PCMM_Scheme ps3(pc3, s3);
        Ciphertext ct3((int)n, c3.L, c3.L, 1, (long double)(1ll << 59));   // PPMM scaler = q1 * 2^49 / scale = about 2^26
        upload(ct3.cipher_device, uniform_limbs(rng, q2, 2, n));
        std::vector<float> W3((size_t)rows_m * rk);
        std::normal_distribution<float> nd3(0.f, 0.02f);
        for (float& w : W3) w = nd3(rng);
        void* W3d = nullptr;
        check(ckks_malloc(&W3d, W3.size() * 4), "malloc W3");
        check(ckks_memcpy_h2d(W3d, W3.data(), W3.size() * 4), "h2d W3");
        std::vector<MLWECiphertext*> smp;
        for (int i = 0; i < rk; i++) smp.push_back(new MLWECiphertext(n1, 1, 1, rk, ct3.scale));
        ps3.rlweCipherDecompose(ct3, smp, rk, 0);
        ps3.PPMM((float*)W3d, smp, rows_m, rk, n1, rk);
        const size_t words = (size_t)rows_m * 2 * (size_t)n1 * (rk + 1);
        std::vector<uint64_tt> two_step = download(ps3.ppmm_output, words);
        const long double scale_after = smp[0]->scale;
        std::vector<MLWECiphertext*> rows3;
        for (int i = 0; i < rows_m; i++) rows3.push_back(new MLWECiphertext(n1, 1, 1, rk, 1.0L));
        ps3.packedBegin(rk);
        ps3.rlweCipherDecomposePacked(ct3, rk, 0);
        ps3.PPMMPacked((float*)W3d, rows3, rows_m);
        EXPECT(download(ps3.ppmm_output, words) == two_step && pc3.info("last_path") == 1, "packed gather + PPMMPacked == rlweCipherDecompose + PPMM (MFMA kernel)");
        EXPECT(download(rows3[5]->cipher_device, (size_t)n1 * (rk + 1)) == download(smp[5]->cipher_device, (size_t)n1 * (rk + 1)) && rows3[5]->scale == scale_after,
               "PPMMPacked leaves the rows and the scale as PPMM does");
        for (MLWECiphertext* m : smp) delete m;
        for (MLWECiphertext* m : rows3) delete m;
        ckks_free(W3d);
    }

    for (MLWECiphertext* m : mlwe) delete m;
    ckks_free(Wd);
    orc_pcmm_destroy(orc_p);
    orc_ctx_destroy(orc);
    return failures;
}

int main() {
    setvbuf(stdout, nullptr, _IONBF, 0);
    const int failed = run();          // every device object is released when run() returns
    printf(failed ? "FAILED: %d check(s)\n" : "all C++ mirror checks passed\n", failed);
    fflush(stdout);
    // leave without running the exit handlers of the HIP runtime and of the oracle's OpenMP runtime: their relative order
    // at process exit is not defined and has crashed once after all checks had passed
    _exit(failed ? 1 : 0);
}
