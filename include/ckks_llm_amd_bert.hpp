// C++ host mirror of the reference's BERT layer shell for the plaintext-matrix products (src/bert/Bert.h:15-66, Bert.cuh) and of
// its weight loader (src/bert/Load_bert.cuh:11-348), on top of the mirror classes of ckks_llm_amd.hpp.
//
// What is here: Bert_model_weights (the tensors of a BERT-base `model.safetensors` as fp32 device arrays, same member names), and
// the PCMM part of every linear layer of Bert: gather of the input ciphertexts into MLWE samples, PPMM with the layer's weight,
// ring packing of the product rows into the output ciphertexts - the calls of
//   Bert::PCMM_Boot_768_768  (Bert.cuh:404-425, 471, 480, 489),
//   Bert::intermediate       (Bert.cuh:249-257),
//   Bert::layer_output       (Bert.cuh:296-302)
// in the reference's order and with its sample counts and offsets.
// What is not here: the slot <-> coefficient conversions, the EvalMod bootstrapping and the non-linear layers that the reference
// runs between these calls (EncodingMatrix, Bootstrapper, Attention); ciphertexts enter and leave in coefficient packing.
#pragma once
#include <fcntl.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cstdio>
#include <cstdlib>
#include <string>
#include <utility>
#include <vector>

#include "ckks_llm_amd.hpp"

namespace ckks_llm_amd {

// Bert_model_weights (Load_bert.cuh:11-348).  File format: 8 bytes little-endian header length, a JSON header that maps a tensor
// name to {"dtype", "shape", "data_offsets":[begin,end]}, then the tensor bytes; offsets count from the end of the header.
// Differences from the reference, on purpose: a tensor name is looked up with its quotes (the reference matches the bare name as
// a substring, Load_bert.cuh:317), offsets are checked against the file size, a tensor that is not F32 is refused, the device
// memory is released by the destructor, and `missing` lists what the file did not hold.
class Bert_model_weights {
public:
    float* embeddings_LayerNorm_beta = nullptr;                  // [768]
    float* embeddings_LayerNorm_gamma = nullptr;                 // [768]
    float* embeddings_position_embeddings_weight = nullptr;      // [512,768]
    float* embeddings_token_type_embeddings_weight = nullptr;    // [2,768]
    float* embeddings_word_embeddings_weight = nullptr;          // [30522,768]

    float* attention_output_LayerNorm_beta[12] = {};
    float* attention_output_LayerNorm_gamma[12] = {};
    float* attention_output_dense_bias[12] = {};
    float* attention_output_dense_weight[12] = {};
    float* attention_self_key_bias[12] = {};
    float* attention_self_key_weight[12] = {};
    float* attention_self_query_bias[12] = {};
    float* attention_self_query_weight[12] = {};
    float* attention_self_value_bias[12] = {};
    float* attention_self_value_weight[12] = {};
    float* intermediate_dense_bias[12] = {};
    float* intermediate_dense_weight[12] = {};
    float* output_LayerNorm_beta[12] = {};
    float* output_LayerNorm_gamma[12] = {};
    float* output_dense_bias[12] = {};
    float* output_dense_weight[12] = {};

    float* pooler_dense_bias = nullptr;
    float* pooler_dense_weight = nullptr;
    float* cls_predictions_bias = nullptr;
    float* cls_predictions_transform_LayerNorm_beta = nullptr;
    float* cls_predictions_transform_LayerNorm_gamma = nullptr;
    float* cls_predictions_transform_dense_bias = nullptr;
    float* cls_predictions_transform_dense_weight = nullptr;
    float* cls_seq_relationship_bias = nullptr;
    float* cls_seq_relationship_weight = nullptr;

    int num_layers = 12;
    bool opened = false;                                         // the file was found and its header read
    std::vector<std::string> missing;                            // tensor names the header does not hold (or holds unusably)
    std::vector<std::pair<std::string, size_t>> loaded;          // tensor name, bytes

    explicit Bert_model_weights(std::string model_catalog) {
        const std::string fname = model_catalog + "model.safetensors";          // Load_bert.cuh:50
        const int fd = open(fname.c_str(), O_RDONLY);
        if (fd < 0) { std::cout << "Failed to open model file: " << fname << std::endl; return; }
        struct stat st;
        uint64_t header_size = 0;
        if (fstat(fd, &st) != 0 || pread(fd, &header_size, 8, 0) != 8 || header_size + 8 > (uint64_t)st.st_size) {
            std::cout << "Failed to read header size from: " << fname << std::endl;
            close(fd);
            return;
        }
        std::string header(header_size, '\0');
        if (pread(fd, &header[0], header_size, 8) != (ssize_t)header_size) {
            std::cout << "Failed to read header from: " << fname << std::endl;
            close(fd);
            return;
        }
        opened = true;
        const uint64_t data_begin = 8 + header_size, data_bytes = (uint64_t)st.st_size - data_begin;

        std::vector<std::pair<std::string, float**>> want = {
            {"bert.embeddings.LayerNorm.beta", &embeddings_LayerNorm_beta},
            {"bert.embeddings.LayerNorm.gamma", &embeddings_LayerNorm_gamma},
            {"bert.embeddings.position_embeddings.weight", &embeddings_position_embeddings_weight},
            {"bert.embeddings.token_type_embeddings.weight", &embeddings_token_type_embeddings_weight},
            {"bert.embeddings.word_embeddings.weight", &embeddings_word_embeddings_weight},
            {"bert.pooler.dense.bias", &pooler_dense_bias},
            {"bert.pooler.dense.weight", &pooler_dense_weight},
            {"cls.predictions.bias", &cls_predictions_bias},
            {"cls.predictions.transform.LayerNorm.beta", &cls_predictions_transform_LayerNorm_beta},
            {"cls.predictions.transform.LayerNorm.gamma", &cls_predictions_transform_LayerNorm_gamma},
            {"cls.predictions.transform.dense.bias", &cls_predictions_transform_dense_bias},
            {"cls.predictions.transform.dense.weight", &cls_predictions_transform_dense_weight},
            {"cls.seq_relationship.bias", &cls_seq_relationship_bias},
            {"cls.seq_relationship.weight", &cls_seq_relationship_weight},
        };
        for (int i = 0; i < num_layers; i++) {                                   // Load_bert.cuh:172-270
            const std::string layer_prefix = "bert.encoder.layer." + std::to_string(i) + ".";
            want.push_back({layer_prefix + "attention.output.LayerNorm.beta", &attention_output_LayerNorm_beta[i]});
            want.push_back({layer_prefix + "attention.output.LayerNorm.gamma", &attention_output_LayerNorm_gamma[i]});
            want.push_back({layer_prefix + "attention.output.dense.bias", &attention_output_dense_bias[i]});
            want.push_back({layer_prefix + "attention.output.dense.weight", &attention_output_dense_weight[i]});
            want.push_back({layer_prefix + "attention.self.key.bias", &attention_self_key_bias[i]});
            want.push_back({layer_prefix + "attention.self.key.weight", &attention_self_key_weight[i]});
            want.push_back({layer_prefix + "attention.self.query.bias", &attention_self_query_bias[i]});
            want.push_back({layer_prefix + "attention.self.query.weight", &attention_self_query_weight[i]});
            want.push_back({layer_prefix + "attention.self.value.bias", &attention_self_value_bias[i]});
            want.push_back({layer_prefix + "attention.self.value.weight", &attention_self_value_weight[i]});
            want.push_back({layer_prefix + "intermediate.dense.bias", &intermediate_dense_bias[i]});
            want.push_back({layer_prefix + "intermediate.dense.weight", &intermediate_dense_weight[i]});
            want.push_back({layer_prefix + "output.LayerNorm.beta", &output_LayerNorm_beta[i]});
            want.push_back({layer_prefix + "output.LayerNorm.gamma", &output_LayerNorm_gamma[i]});
            want.push_back({layer_prefix + "output.dense.bias", &output_dense_bias[i]});
            want.push_back({layer_prefix + "output.dense.weight", &output_dense_weight[i]});
        }
        std::vector<char> staging;
        for (auto& [name, slot] : want) {
            int64_t begin = 0, end = 0;
            if (!parseKeyFromString(header, name, begin, end) || begin < 0 || end < begin || (uint64_t)end > data_bytes || (end - begin) % 4) {
                missing.push_back(name);
                continue;
            }
            const size_t bytes = (size_t)(end - begin);
            staging.resize(bytes ? bytes : 1);
            if (pread(fd, staging.data(), bytes, (off_t)(data_begin + begin)) != (ssize_t)bytes) { missing.push_back(name); continue; }
            load_tensor(staging.data(), *slot, bytes);
            loaded.push_back({name, bytes});
        }
        close(fd);
    }
    Bert_model_weights(const Bert_model_weights&) = delete;
    Bert_model_weights& operator=(const Bert_model_weights&) = delete;
    ~Bert_model_weights() {
        if (owned.empty()) return;
        ckks_sync();
        for (float* p : owned) ckks_free(p);
    }

    // Load_bert.cuh:297-306: device array of read_size bytes filled from the host bytes
    void load_tensor(const char* host_bytes, float*& weight, size_t read_size) {
        void* p = nullptr;
        check(ckks_malloc(&p, read_size ? read_size : 4), "Bert_model_weights: device memory");
        check(ckks_memcpy_h2d(p, host_bytes, read_size), "Bert_model_weights: upload");
        weight = static_cast<float*>(p);
        owned.push_back(weight);
    }

    // Load_bert.cuh:315-343: the two numbers of the tensor's "data_offsets".  The entry of a tensor is the JSON object that
    // follows its quoted name; entries hold no nested objects, so it ends at the next closing brace.
    bool parseKeyFromString(const std::string& input, const std::string& targetKey, int64_t& offset1Out, int64_t& offset2Out) {
        const std::string quoted = "\"" + targetKey + "\"";
        // a tensor's entry is its quoted name followed by a colon and an opening brace; the same text elsewhere (a key inside an
        // entry, a metadata string) is passed over
        size_t keyPos = input.find(quoted);
        for (; keyPos != std::string::npos; keyPos = input.find(quoted, keyPos + 1)) {
            size_t at = input.find_first_not_of(" \t\r\n", keyPos + quoted.size());
            if (at == std::string::npos || input[at] != ':') continue;
            at = input.find_first_not_of(" \t\r\n", at + 1);
            if (at != std::string::npos && input[at] == '{') break;
        }
        if (keyPos == std::string::npos) return false;
        const size_t entryEnd = input.find('}', keyPos);
        const size_t dtypePos = input.find("\"dtype\"", keyPos);
        if (dtypePos != std::string::npos && dtypePos < entryEnd) {
            const size_t v = input.find('"', input.find(':', dtypePos));
            if (v == std::string::npos || input.compare(v, 5, "\"F32\"") != 0) return false;
        }
        const size_t offPos = input.find("\"data_offsets\"", keyPos);
        if (offPos == std::string::npos || offPos > entryEnd) return false;
        const size_t open = input.find('[', offPos), comma = input.find(',', open), closeb = input.find(']', open);
        if (open == std::string::npos || comma == std::string::npos || closeb == std::string::npos || comma > closeb) return false;
        char* stop = nullptr;
        const std::string first = input.substr(open + 1, comma - open - 1), second = input.substr(comma + 1, closeb - comma - 1);
        offset1Out = std::strtoll(first.c_str(), &stop, 10);
        if (stop == first.c_str()) return false;
        offset2Out = std::strtoll(second.c_str(), &stop, 10);
        return stop != second.c_str();
    }

    // the device arrays this object allocated, in the order of `loaded`
    const std::vector<float*>& tensors() const { return owned; }

private:
    std::vector<float*> owned;
};

// Bert (Bert.h:15-66), the part on the PCMM path.  The reference's constructor also takes SchemeAlgo, Attention and Bootstrapper
// (Bert.cuh:8-9); they serve the steps that are not here.
class Bert {
public:
    Context_23& context;
    Scheme_23& scheme;
    SecretKey& sk;
    Bert_model_weights model_weights;
    PCMM_Scheme& pcmm_scheme;
    std::vector<MLWECiphertext*> mlwe_cipher_buffer;
    int PCMM_N1 = 128;
    int q_ringpack_count;
    int mlwe_rank;
    int mat_M = 768, mat_N = 768;
    int N;
    int L;
    // true: the gather writes PPMM's operand planes directly (ring-pack primes that fit five balanced digits, i.e. just below 2^39); false: rlweCipherDecompose into
    // mlwe_cipher_buffer and PPMM, call for call as the reference
    bool packed_gather;

    // decomp_num MLWE ciphertexts are kept for the samples and product rows of a layer (Bert.cuh:26-30: 3072)
    Bert(std::string model_catalog, Context_23& context, Scheme_23& scheme, PCMM_Scheme& pcmm_scheme, SecretKey& sk, int decomp_num = 3072)
        : context(context), scheme(scheme), sk(sk), model_weights(model_catalog), pcmm_scheme(pcmm_scheme) {
        N = (int)context.N;
        L = context.L;
        PCMM_N1 = pcmm_scheme.pcmm_context.N1;
        q_ringpack_count = pcmm_scheme.pcmm_context.ringpack_q_count;
        mlwe_rank = N / PCMM_N1;                                                                       // Bert.cuh:24
        if (mlwe_rank != pcmm_scheme.pcmm_context.mlwe_rank) throw std::invalid_argument("Bert: the PCMM context's rank is not N / N1");
        packed_gather = true;
        for (uint64_tt q : pcmm_scheme.pcmm_context.q_ringpack) packed_gather = packed_gather && q - 1 <= 0x7f7f7f7f7full;      // five balanced residue digits
        for (int i = 0; i < decomp_num; i++)
            mlwe_cipher_buffer.push_back(new MLWECiphertext(PCMM_N1, q_ringpack_count - 1, q_ringpack_count - 1, mlwe_rank, 0));
        // the model's tensors were uploaded by this object and are not written again: their digit planes are kept between calls
        // (a caller that does overwrite one says so: pcmm_scheme.pcmm_context.weights_changed)
        for (size_t i = 0; i < model_weights.tensors().size() && i < model_weights.loaded.size(); i++)
            if (model_weights.loaded[i].second) pcmm_scheme.pcmm_context.weights_static(model_weights.tensors()[i], model_weights.loaded[i].second);
    }
    Bert(const Bert&) = delete;
    ~Bert() {
        for (size_t i = 0; i < model_weights.tensors().size() && i < model_weights.loaded.size(); i++)
            if (model_weights.loaded[i].second) pcmm_weights_static(pcmm_scheme.pcmm_context.handle, model_weights.tensors()[i], model_weights.loaded[i].second, 0);
        for (MLWECiphertext* m : mlwe_cipher_buffer) delete m;
    }

    // one input or output of a linear layer: `count` MLWE samples of a ciphertext at sample positions `offset`.. ; for an input,
    // `extract` >= count is the number of samples the gather addresses (it fixes the stride rank / extract between them)
    struct Part {
        Ciphertext* cipher;
        int count, offset, extract;
    };
    // gather -> PPMM (mat_M x mat_N) -> ring packing
    void linear(float* plain_mat, int M, int Nin, const std::vector<Part>& in, const std::vector<Part>& out) {
        if ((size_t)M > mlwe_cipher_buffer.size() || (size_t)Nin > mlwe_cipher_buffer.size()) throw std::invalid_argument("Bert: layer larger than mlwe_cipher_buffer");
        if (packed_gather) {
            pcmm_scheme.packedBegin(Nin);
            for (const Part& p : in) pcmm_scheme.rlweCipherDecomposePacked(*p.cipher, p.extract, p.offset, p.count);
            pcmm_scheme.PPMMPacked(plain_mat, mlwe_cipher_buffer, M);
        } else {
            for (const Part& p : in) {
                if ((size_t)(p.offset + p.extract) > mlwe_cipher_buffer.size()) throw std::invalid_argument("Bert: gather beyond mlwe_cipher_buffer");
                pcmm_scheme.rlweCipherDecompose(*p.cipher, mlwe_cipher_buffer, p.extract, p.offset);
                for (int i = 0; i < p.extract; i++) mlwe_cipher_buffer[p.offset + i]->scale = p.cipher->scale;
            }
            pcmm_scheme.PPMM(plain_mat, mlwe_cipher_buffer, M, Nin, PCMM_N1, Nin);
            // PPMM hands back the first min(M, Nin) product rows (PPMM_kernel.cuh:345-348); the layer needs all M
            const size_t C = (size_t)PCMM_N1 * (mlwe_rank + 1);
            for (int i = Nin; i < M; i++) {
                mlwe_cipher_buffer[i]->scale = mlwe_cipher_buffer[0]->scale;
                check(ckks_memcpy_d2d(mlwe_cipher_buffer[i]->cipher_device, pcmm_scheme.ppmm_output + (size_t)i * C * q_ringpack_count, sizeof(uint64_tt) * C),
                      "Bert: product row");
            }
        }
        for (const Part& p : out) pcmm_scheme.mlweCipherPacking(*p.cipher, mlwe_cipher_buffer, p.count, p.offset);
    }

    // The PCMM calls of Bert::PCMM_Boot_768_768 (Bert.cuh:379-498).  do_s2c = 0: two input ciphertexts with 512 samples each, of
    // which the product takes the first 768 (:416-417, 425); do_s2c = 1: three input ciphertexts with 256 samples each (:404, 408,
    // 412; the slot-to-coefficient conversion in front of each gather is the caller's).  Three output ciphertexts of 256 rows
    // (:471, 480, 489).
    void PCMM_768_768(float* plain_mat, std::vector<Ciphertext*>& rlwe_cipher, std::vector<Ciphertext*>& res_cipher, int do_s2c) {
        std::vector<Part> in;
        if (do_s2c == 1) in = {{rlwe_cipher[0], 256, 0, 256}, {rlwe_cipher[1], 256, 256, 256}, {rlwe_cipher[2], 256, 512, 256}};
        else in = {{rlwe_cipher[0], 512, 0, 512}, {rlwe_cipher[1], 256, 512, 512}};
        linear(plain_mat, 768, 768, in, {{res_cipher[0], 256, 0, 0}, {res_cipher[1], 256, 256, 0}, {res_cipher[2], 256, 512, 0}});
    }
    // ---- the reference's own member signatures (Bert.h:51, 59-63), so that code written against Bert.h compiles.  What they do not
    //      carry out of the reference's bodies is listed at each member. ----
    // Bert::PCMM_Boot_768_768 (Bert.h:62, Bert.cuh:379-498).  target_level is the level the reference raises the packed result to
    // before its coefficient-to-slot conversion and EvalMod (:472-497); that stage is outside this library, so the argument is
    // accepted and not used: the results stay at level 0 in coefficient packing.
    void PCMM_Boot_768_768(float* plain_mat, std::vector<Ciphertext*>& rlwe_cipher, std::vector<Ciphertext*>& res_cipher, int target_level, int do_s2c) {
        (void)target_level;
        PCMM_768_768(plain_mat, rlwe_cipher, res_cipher, do_s2c);
    }
    // Bert.h:63: the reference keeps a second copy of the member for its test program
    void test_PCMM_Boot_768_768(float* plain_mat, std::vector<Ciphertext*>& rlwe_cipher, std::vector<Ciphertext*>& res_cipher, int target_level, int do_s2c) {
        PCMM_Boot_768_768(plain_mat, rlwe_cipher, res_cipher, target_level, do_s2c);
    }
    // Bert::mul_W_QKV (Bert.h:51, Bert.cuh:155-169): the three products on the weights handed in, three input ciphertexts of 256
    // samples (do_s2c = 1, as the reference calls it).  The bias additions of :158-168 act on slot-packed plaintexts after the
    // bootstrapping and are not part of this library.
    void mul_W_QKV(std::vector<Ciphertext*>& X, Bert_model_weights& weights, std::vector<Ciphertext*>& resQ, std::vector<Ciphertext*>& resK,
                   std::vector<Ciphertext*>& resV, int layer) {
        PCMM_Boot_768_768(weights.attention_self_query_weight[layer], X, resQ, X[0]->L - 2, 1);
        PCMM_Boot_768_768(weights.attention_self_key_weight[layer], X, resK, X[0]->L - 2, 1);
        PCMM_Boot_768_768(weights.attention_self_value_weight[layer], X, resV, 18, 1);
    }
    // Bert::attn_output (Bert.h:59, Bert.cuh:204-211): the dense product in place, O -> O; the LayerNorm behind it is not part of this library
    void attn_output(std::vector<Ciphertext*>& O, int layer) {
        PCMM_Boot_768_768(model_weights.attention_output_dense_weight[layer], O, O, O[0]->L, 1);
    }
    // Bert::layer_output (Bert.h:61, Bert.cuh:290-302).  layer_res is not touched: the reference's body does not use it either (every
    // line that names it is commented out, Bert.cuh:333, 349-353).
    void layer_output(std::vector<Ciphertext*>& O, int layer, std::vector<Ciphertext*>& layer_res) {
        (void)layer_res;
        layer_output(O, layer);
    }

    // ---- the same calls with the choices the reference hard-wires left to the caller ----
    // Bert::mul_W_QKV (Bert.cuh:155-169)
    void mul_W_QKV(std::vector<Ciphertext*>& X, std::vector<Ciphertext*>& resQ, std::vector<Ciphertext*>& resK, std::vector<Ciphertext*>& resV,
                   int layer, int do_s2c = 1) {
        PCMM_768_768(model_weights.attention_self_query_weight[layer], X, resQ, do_s2c);
        PCMM_768_768(model_weights.attention_self_key_weight[layer], X, resK, do_s2c);
        PCMM_768_768(model_weights.attention_self_value_weight[layer], X, resV, do_s2c);
    }
    // Bert::attn_output (Bert.cuh:204-211)
    void attn_output(std::vector<Ciphertext*>& O, std::vector<Ciphertext*>& res, int layer, int do_s2c = 1) {
        PCMM_768_768(model_weights.attention_output_dense_weight[layer], O, res, do_s2c);
    }
    // Bert::intermediate (Bert.cuh:249-257): 512 samples of O[0] and 256 of O[2]; 3072 x 768; rows 512 i .. into res[2 i]
    void intermediate(std::vector<Ciphertext*>& O, int layer, std::vector<Ciphertext*>& res) {
        std::vector<Part> out;
        for (int i = 0; i < 3072 / 512; i++) out.push_back({res[2 * i], 512, i * 512, 0});
        linear(model_weights.intermediate_dense_weight[layer], 3072, 768, {{O[0], 512, 0, 512}, {O[2], 256, 512, 256}}, out);
    }
    // Bert::layer_output (Bert.cuh:290-302): 512 samples of each O[2 i]; 768 x 3072; rows 0..511 into O[0], 512..767 into O[2]
    void layer_output(std::vector<Ciphertext*>& O, int layer) {
        std::vector<Part> in;
        for (int i = 0; i < 3072 / 512; i++) in.push_back({O[2 * i], 512, i * 512, 512});
        linear(model_weights.output_dense_weight[layer], 768, 3072, in, {{O[0], 512, 0, 0}, {O[2], 256, 512, 0}});
    }
};

}  // namespace ckks_llm_amd
