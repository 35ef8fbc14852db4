// The linear layers of the reference's BERT shell on encrypted activations, at the reference's ring (N = 2^16, N1 = 128 tokens,
// rank 512, ring-pack primes [p0 | q0, q1]): weights come from a `model.safetensors` in the directory given as argv[1] through the
// Bert_model_weights mirror; every layer (768 x 768 with two and with three input ciphertexts, 3072 x 768, 768 x 3072) is run
// through the Bert mirror, decrypted and compared with the plain product in double, as the reference's test programs compare
// (GetPrecisionStats, precision.cuh:104).  Prints one "tensor <name> <bytes> <position-weighted word sum>" line per loaded tensor so that the caller
// can compare the device copies with what it wrote.  Needs a GPU.  Exit code 0 = passed.
#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <random>
#include <unistd.h>
#include <vector>

#include "../../include/ckks_llm_amd_bert.hpp"

using namespace ckks_llm_amd;

static int failures = 0;
#define EXPECT(cond, what)                                                      \
    do {                                                                        \
        if (!(cond)) { printf("FAIL %s (line %d)\n", what, __LINE__); failures++; } \
        else printf("ok   %s\n", what);                                         \
    } while (0)

// position-weighted sum of the 32-bit words modulo 2^64
static uint64_t weighted_sum(const float* p, size_t n) {
    uint64_t h = 0;
    for (size_t i = 0; i < n; i++) {
        uint32_t w;
        memcpy(&w, p + i, 4);
        h += (uint64_t)(i + 1) * w;
    }
    return h;
}
static std::vector<float> host_floats(const float* d, size_t n) {
    std::vector<float> h(n);
    check(ckks_memcpy_d2h(h.data(), d, n * 4), "d2h");
    return h;
}

struct Harness {
    Context_23& context;
    Scheme_23& scheme;
    SecretKey& sk;
    int N, L, N1, rank;
    long double in_scale;
    double* d_vals = nullptr;

    // ciphertext whose coefficient n * rank + j * (rank / extract) is X[n][first + j], j < count (the coefficient packing the gather reads)
    Ciphertext* encrypt_part(const std::vector<double>& X, int features, int first, int count, int extract) {
        std::vector<double> coeffs((size_t)N, 0.0);
        const int gap = rank / extract;
        for (int n = 0; n < N1; n++)
            for (int j = 0; j < count; j++) coeffs[(size_t)n * rank + (size_t)j * gap] = X[(size_t)n * features + first + j];
        check(ckks_memcpy_h2d(d_vals, coeffs.data(), 8 * (size_t)N), "h2d");
        Plaintext msg(N, L, L, N / 2, in_scale);
        context.encode_coeffs(d_vals, msg);
        Ciphertext* ct = new Ciphertext(N, L, L, N / 2, in_scale);
        scheme.encryptMsg(*ct, msg);
        return ct;
    }
    // worst |error| of the rows first .. first + count - 1 of Y (tokens x rows) held by a packed ciphertext
    double worst_error(Ciphertext& ct, const std::vector<double>& Y, int rows, int first, int count) {
        Plaintext dec(N, L, 0, N / 2, 1);
        scheme.decryptMsg(dec, sk, ct);
        context.decode_coeffs(dec, d_vals);
        std::vector<double> got((size_t)N);
        check(ckks_memcpy_d2h(got.data(), d_vals, 8 * (size_t)N), "d2h");
        const int gap = rank / count;
        double worst = 0;
        for (int n = 0; n < N1; n++)
            for (int j = 0; j < count; j++)
                worst = std::max(worst, std::fabs(got[(size_t)n * rank + (size_t)j * gap] - Y[(size_t)n * rows + first + j]));
        return worst;
    }
};

// Y[n][m] = sum_f W[m][f] X[n][f]
static std::vector<double> plain_product(const std::vector<float>& W, const std::vector<double>& X, int tokens, int M, int F) {
    std::vector<double> Y((size_t)tokens * M, 0.0);
    for (int n = 0; n < tokens; n++)
        for (int m = 0; m < M; m++) {
            double s = 0;
            for (int f = 0; f < F; f++) s += (double)W[(size_t)m * F + f] * X[(size_t)n * F + f];
            Y[(size_t)n * M + m] = s;
        }
    return Y;
}

static int run(const std::string& catalog) {
    const std::vector<uint64_tt> q = {0xffff00001ull, 0xfff9c0001ull}, p = {0x1ffffe0001ull};
    const int logN = 16, PCMM_N1 = 128;
    Context_23 context(logN, p, q);
    for (int i = 0; i < 32; i++) context.rng_key[i] = (uint8_t)(7 * i + 1);
    Scheme_23 scheme(context);
    const int N = (int)context.N, L = context.L, mlwe_rank = N / PCMM_N1;
    SecretKey sk(context, 192);
    PCMM_Context pcmm_context(PCMM_N1, mlwe_rank, p, q, context);
    PCMM_Scheme pcmm_scheme(pcmm_context, scheme);
    MLWESecretKey mlwe_sk(PCMM_N1, pcmm_context.ringpack_pq_count - 1, mlwe_rank);
    pcmm_scheme.convertMLWESKfromRLWESK(mlwe_sk, sk);
    scheme.addEncKey(sk);
    pcmm_scheme.addRepakcingKey(mlwe_sk, sk);
    pcmm_scheme.ppmm_target_scale = (long double)(1ll << 26);          // 36-bit ring-pack primes: product rows at scale 2^26

    {
        Bert_model_weights nothing("/nonexistent-directory/");
        EXPECT(!nothing.opened && nothing.loaded.empty(), "a missing model file is reported, nothing is loaded");
    }
    Bert bert(catalog, context, scheme, pcmm_scheme, sk);
    EXPECT(bert.model_weights.opened, "model.safetensors opened");
    {
        // device copies of everything that was loaded, for the caller to compare
        Bert_model_weights& w = bert.model_weights;
        std::vector<std::pair<std::string, float*>> all = {
            {"bert.embeddings.LayerNorm.beta", w.embeddings_LayerNorm_beta},
            {"bert.embeddings.LayerNorm.gamma", w.embeddings_LayerNorm_gamma},
            {"bert.pooler.dense.bias", w.pooler_dense_bias},
            {"cls.predictions.bias", w.cls_predictions_bias},
            {"bert.encoder.layer.0.attention.self.query.weight", w.attention_self_query_weight[0]},
            {"bert.encoder.layer.0.attention.self.key.weight", w.attention_self_key_weight[0]},
            {"bert.encoder.layer.0.attention.self.value.weight", w.attention_self_value_weight[0]},
            {"bert.encoder.layer.0.attention.output.dense.weight", w.attention_output_dense_weight[0]},
            {"bert.encoder.layer.0.attention.output.dense.bias", w.attention_output_dense_bias[0]},
            {"bert.encoder.layer.0.intermediate.dense.weight", w.intermediate_dense_weight[0]},
            {"bert.encoder.layer.0.output.dense.weight", w.output_dense_weight[0]},
            {"bert.encoder.layer.0.output.dense.bias", w.output_dense_bias[0]},
            {"bert.encoder.layer.1.output.dense.bias", w.output_dense_bias[1]},
            {"bert.encoder.layer.11.output.dense.bias", w.output_dense_bias[11]},
            {"cls.seq_relationship.bias", w.cls_seq_relationship_bias},
            {"cls.seq_relationship.weight", w.cls_seq_relationship_weight},
        };
        for (auto& [name, ptr] : all) {
            size_t bytes = 0;
            for (auto& [lname, lbytes] : w.loaded) if (lname == name) bytes = lbytes;
            if (!ptr) { printf("tensor %s absent\n", name.c_str()); continue; }
            std::vector<float> h = host_floats(ptr, bytes / 4);
            printf("tensor %s %zu %016llx\n", name.c_str(), bytes, (unsigned long long)weighted_sum(h.data(), bytes / 4));
        }
        printf("loaded %zu missing %zu\n", w.loaded.size(), w.missing.size());
    }
    EXPECT(bert.packed_gather, "36-bit ring-pack primes select the gather into the operand planes");

    Harness hs{context, scheme, sk, N, L, PCMM_N1, mlwe_rank, (long double)(1ll << 33)};
    void* dv = nullptr;
    check(ckks_malloc(&dv, 8 * (size_t)N), "malloc");
    hs.d_vals = static_cast<double*>(dv);
    std::mt19937_64 rng(5);
    std::normal_distribution<double> act(0.0, 1.0);
    const int tokens = PCMM_N1;
    const double bound = std::ldexp(1.0, -10);

    for (int variant = 0; variant < 2; variant++) {
        bert.packed_gather = variant == 0;
        const char* how = variant == 0 ? "gather into operand planes" : "rlweCipherDecompose + PPMM";
        // ---- 768 x 768, two input ciphertexts of 512 samples (do_s2c = 0), query weight of layer 0 ----
        {
            std::vector<double> X((size_t)tokens * 768);
            for (double& v : X) v = act(rng);
            std::vector<float> W = host_floats(bert.model_weights.attention_self_query_weight[0], 768 * 768);
            std::vector<double> Y = plain_product(W, X, tokens, 768, 768);
            std::vector<Ciphertext*> in = {hs.encrypt_part(X, 768, 0, 512, 512), hs.encrypt_part(X, 768, 512, 256, 512)};
            std::vector<Ciphertext*> out = {new Ciphertext(N, L, 0, N / 2, 1), new Ciphertext(N, L, 0, N / 2, 1), new Ciphertext(N, L, 0, N / 2, 1)};
            bert.PCMM_Boot_768_768(bert.model_weights.attention_self_query_weight[0], in, out, L, 0);      // Bert.h:62
            double worst = 0;
            for (int j = 0; j < 3; j++) worst = std::max(worst, hs.worst_error(*out[j], Y, 768, 256 * j, 256));
            printf("768 x 768, 2 inputs (%s): worst error 2^%.1f, output scale 2^%.1f\n", how, std::log2(worst), (double)std::log2((double)out[0]->scale));
            EXPECT(worst < bound, "PCMM_768_768 (two input ciphertexts) decrypts to W x");
            for (Ciphertext* c : in) delete c;
            for (Ciphertext* c : out) delete c;
        }
        // ---- intermediate: 3072 x 768 ----
        std::vector<double> H;
        {
            std::vector<double> X((size_t)tokens * 768);
            for (double& v : X) v = act(rng);
            std::vector<float> W = host_floats(bert.model_weights.intermediate_dense_weight[0], 3072 * 768);
            std::vector<double> Y = plain_product(W, X, tokens, 3072, 768);
            std::vector<Ciphertext*> O = {hs.encrypt_part(X, 768, 0, 512, 512), nullptr, hs.encrypt_part(X, 768, 512, 256, 256)};
            std::vector<Ciphertext*> res(12, nullptr);
            for (int i = 0; i < 6; i++) res[2 * i] = new Ciphertext(N, L, 0, N / 2, 1);
            bert.intermediate(O, 0, res);
            double worst = 0;
            for (int i = 0; i < 6; i++) worst = std::max(worst, hs.worst_error(*res[2 * i], Y, 3072, 512 * i, 512));
            printf("intermediate 3072 x 768 (%s): worst error 2^%.1f\n", how, std::log2(worst));
            EXPECT(worst < bound, "intermediate decrypts to W x");
            H = Y;
            delete O[0]; delete O[2];
            for (Ciphertext* c : res) delete c;
        }
        if (variant == 1) break;          // the call-for-call variant: the first layer and the one with more rows than samples
        // ---- 768 x 768, three input ciphertexts of 256 samples (do_s2c = 1), through mul_W_QKV ----
        {
            std::vector<double> X((size_t)tokens * 768);
            for (double& v : X) v = act(rng);
            std::vector<Ciphertext*> in = {hs.encrypt_part(X, 768, 0, 256, 256), hs.encrypt_part(X, 768, 256, 256, 256), hs.encrypt_part(X, 768, 512, 256, 256)};
            std::vector<Ciphertext*> Q, K, V;
            for (int j = 0; j < 3; j++) { Q.push_back(new Ciphertext(N, L, 0, N / 2, 1)); K.push_back(new Ciphertext(N, L, 0, N / 2, 1)); V.push_back(new Ciphertext(N, L, 0, N / 2, 1)); }
            bert.mul_W_QKV(in, bert.model_weights, Q, K, V, 0);                    // the reference's signature (Bert.h:51)
            float* weights[3] = {bert.model_weights.attention_self_query_weight[0], bert.model_weights.attention_self_key_weight[0], bert.model_weights.attention_self_value_weight[0]};
            std::vector<Ciphertext*>* res[3] = {&Q, &K, &V};
            double worst = 0;
            for (int w = 0; w < 3; w++) {
                std::vector<double> Y = plain_product(host_floats(weights[w], 768 * 768), X, tokens, 768, 768);
                for (int j = 0; j < 3; j++) worst = std::max(worst, hs.worst_error(*(*res[w])[j], Y, 768, 256 * j, 256));
            }
            printf("mul_W_QKV, 3 inputs: worst error 2^%.1f\n", std::log2(worst));
            EXPECT(worst < bound, "mul_W_QKV decrypts to W_q x, W_k x, W_v x");
            for (Ciphertext* c : in) delete c;
            for (int w = 0; w < 3; w++) for (Ciphertext* c : *res[w]) delete c;
        }
        // ---- attn_output(O, layer) as Bert.h:59 declares it: the dense product in place, three ciphertexts of 256 samples ----
        {
            std::vector<double> X((size_t)tokens * 768);
            for (double& v : X) v = act(rng);
            std::vector<Ciphertext*> O = {hs.encrypt_part(X, 768, 0, 256, 256), hs.encrypt_part(X, 768, 256, 256, 256), hs.encrypt_part(X, 768, 512, 256, 256)};
            bert.attn_output(O, 0);
            std::vector<double> Y = plain_product(host_floats(bert.model_weights.attention_output_dense_weight[0], 768 * 768), X, tokens, 768, 768);
            double worst = 0;
            for (int j = 0; j < 3; j++) worst = std::max(worst, hs.worst_error(*O[j], Y, 768, 256 * j, 256));
            printf("attn_output in place: worst error 2^%.1f\n", std::log2(worst));
            EXPECT(worst < bound, "attn_output(O, layer) leaves W_o x in O");
            for (Ciphertext* c : O) delete c;
        }
        // ---- layer_output: 768 x 3072 on the previous product (scaled to unit size) ----
        {
            std::vector<double> X = H;
            for (double& v : X) v *= 1.5;
            std::vector<float> W = host_floats(bert.model_weights.output_dense_weight[0], 768 * 3072);
            std::vector<double> Y = plain_product(W, X, tokens, 768, 3072);
            std::vector<Ciphertext*> O(12, nullptr);
            for (int i = 0; i < 6; i++) O[2 * i] = hs.encrypt_part(X, 3072, 512 * i, 512, 512);
            std::vector<Ciphertext*> layer_res;
            bert.layer_output(O, 0, layer_res);                                   // Bert.h:61
            const double worst = std::max(hs.worst_error(*O[0], Y, 768, 0, 512), hs.worst_error(*O[2], Y, 768, 512, 256));
            printf("layer_output 768 x 3072: worst error 2^%.1f\n", std::log2(worst));
            EXPECT(worst < bound, "layer_output decrypts to W x");
            for (Ciphertext* c : O) delete c;
        }
    }
    ckks_free(dv);
    return failures;
}

int main(int argc, char** argv) {
    setvbuf(stdout, nullptr, _IONBF, 0);
    if (argc < 2) { printf("usage: %s <directory with model.safetensors>/\n", argv[0]); return 2; }
    int failed = 1;
    try {
        failed = run(argv[1]);
    } catch (const std::exception& e) {
        printf("FAIL exception: %s\n", e.what());
    }
    printf(failed ? "FAILED: %d check(s)\n" : "the BERT linear layers passed\n", failed);
    fflush(stdout);
    _exit(failed ? 1 : 0);          // skip the exit handlers of the HIP runtime (their order at process exit is not defined)
}
