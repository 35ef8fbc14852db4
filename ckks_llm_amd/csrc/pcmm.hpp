// Internal types shared by the PCMM launchers and kernels.
#pragma once
#include <utility>
#include <vector>

#include "context.hpp"

struct pcmm_ctx {
    ckks_ctx* ctx = nullptr;
    int N1 = 0, rank = 0, np = 0, nq = 0;
    std::vector<uint64_t> pq;
    ckks::PrimeConst* d_pq = nullptr;        // ring-pack primes [p_ringpack | q_ringpack]
    uint64_t** d_ptrs = nullptr;             // device copy of the caller's MLWE pointer table (PCMM_Scheme.cuh:16-18)
    int ptr_cap = 0;
    int8_t* d_Bdig = nullptr;                // residue digit planes [prime][K step][digit][column][64]
    size_t Bdig_cap = 0;
    uint64_t* d_zero = nullptr;              // zero rows the K padding of the row-pointer table points to
    size_t zero_cap = 0;
    int packed_K = 0, packed_mods = 0;       // shape the residue digit planes were opened for by pcmm_packed_begin (0: not open)
    int last_path = -1, last_DW = 0, last_DC = 0;   // what the last PPMM call ran: 1 = MFMA kernel, 0 = generic kernel
    int last_slices = 0;                     // plaintext digit slices of the last MFMA call (1: one launch with the fused rescale)
    uint64_t* d_slices = nullptr;            // outputs of the plaintext slices above the first, [slice - 1][M][mod_num][C]
    size_t slices_cap = 0;
    unsigned long long last_absmax = 0;
    ckks_ctx* small = nullptr;               // tables of the size-N1 transform over the ring-pack primes, built on first use
    uint64_t* d_small_tw = nullptr;          // tables of the size-N1 transform when N1 < 256: [prime][forward | inverse][N1]
    uint64_t small_n_inv[8] = {};            // N1^-1 modulo each ring-pack prime (N1 < 256)
    unsigned long long* d_absmax = nullptr;  // |A| maximum word, followed by the per-call constant table (PPMM_CONST_WORDS)
    unsigned long long* h_absmax = nullptr;  // pinned host word the maximum is copied to, and the event behind that copy
    hipEvent_t ev_absmax = nullptr;
    // Prepared plaintext matrices (only while the caller has switched the cache on: pcmm_set_weight_cache).  The first PPMM call
    // with a given (device pointer, shape, scaler) quantises the matrix, measures |A|max (the one host round trip) and splits it
    // into digit planes; later calls with the same key reuse the planes and issue no host synchronisation at all.
    struct Weights {
        const float* W = nullptr;
        int M = 0, Kin = 0;
        double scaler = 0;
        unsigned long long absmax = 0;
        long long* d_A = nullptr;            // kept when the generic kernel runs this matrix
        int8_t* d_Adig = nullptr;            // kept when the MFMA kernel runs it: `planes` planes of Mpad x Kpad
        int planes = 0;
        size_t bytes = 0;
        uint64_t stamp = 0;
    };
    std::vector<Weights> weights;
    bool weights_cached = false;
    bool gather_plain = false, ppmm_generic = false, ppmm_no_tail = false;      // test / tuning switches (pcmm_set_option)
    std::vector<std::pair<uintptr_t, size_t>> static_ranges;    // device address ranges whose matrices the caller has declared static
    // work space of the calls that keep nothing: the quantised matrix and its digit planes of the call in flight
    long long* d_workA = nullptr;
    size_t workA_cap = 0;
    int8_t* d_workAdig = nullptr;
    size_t workAdig_cap = 0;
    hipStream_t work_stream = nullptr;
    bool work_stream_known = false;
    size_t weights_bytes = 0;
    uint64_t weights_clock = 0;
    // last row-pointer table and epilogue constants sent to the device (resent only when they change), and the pinned staging
    // area they travel through, so that the copies need no stream synchronisation
    std::vector<const uint64_t*> tab_sent;
    int cst_mods = 0;
    void* pin = nullptr;
    size_t pin_cap = 0;
    hipEvent_t pin_ev = nullptr;
    uint64_t** d_ptrs_slot(int count);       // the device table, grown to `count` entries (nullptr: out of memory)
};

namespace ckks {

// per-call constants of the PPMM epilogue, one row of PPMM_MAX_MODS words each:
//   [0] q_last^-1 mod q_i   [1] its Shoup word   [2] 2^32 mod q_i   [3] 2^64 mod q_i   [4] q_last^-1 mod q_i
//   rows 2..4 are balanced representatives stored as IEEE double bit patterns (FP64 epilogue)
constexpr int PPMM_MAX_MODS = 64;
constexpr int PPMM_CONST_ROWS = 5;
constexpr int PPMM_CONST_WORDS = PPMM_MAX_MODS * PPMM_CONST_ROWS;

struct PpmmArgs {
    const long long* A;           // [M][Kin]
    const int8_t* Adig;           // [DW][Mpad][Kpad]
    const u64* const* mlwe;       // Kin pointers (nullptr when strided)
    const u64* mlwe_base;         // strided operand
    long mlwe_stride;             // words between consecutive MLWE ciphertexts
    u64* out;
    const PrimeConst* pq;         // ring-pack primes, q part starts at np
    const u64* consts;            // PPMM_CONST_WORDS words, see above
    long C;
    int M, Kin, Mpad, Kpad, mod_num, np;
    int raw_all;                  // MFMA kernel: store every modulus' residue as it is (no fused rescale); the caller combines slices
    int no_tail = 0;              // MFMA kernel: run the remainder column panels whole instead of as jobs by prime (tuning switch)
};

size_t ppmm_bdig_bytes(const PpmmArgs& a, int DC);
int launch_ppmm_mfma_impl(hipStream_t stream, const PpmmArgs& a, int DW, int DC, int8_t* bdig, bool pack);
int launch_ppmm_pack(hipStream_t stream, const PpmmArgs& a, int DC, int8_t* bdig);

}  // namespace ckks
