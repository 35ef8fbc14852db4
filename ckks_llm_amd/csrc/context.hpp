// Internal definition of the context handle shared by the kernels' launchers.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <string>
#include <vector>

#include "../../include/ckks_hip.h"
#include "modarith.hpp"

namespace ckks {

// per-prime constants in device memory, indexed in pqt order
struct PrimeConst {
    u64 q, mu_hi, mu_lo;
    u64 n_inv, n_inv_s;          // N^-1 and its Shoup word
    u64 w1n, w1n_s;              // psiinv_table[1] (which already carries N^-1, Utils.cuh:200) and its Shoup word
    double qd, qinv_d;           // (double)q and 1/q for the FP64 back end
    double n_inv_d, w1n_d;       // balanced representatives of n_inv, w1n as doubles
    int f64_ok;                  // prime small enough for the FP64 back end
    int pad;
};

// one block of an exact RNS conversion (BasisConv.cuh:18-58): nsrc source primes -> ntgt target primes
constexpr int CONV_MAX_SRC = 16;
constexpr int CONV_MAX_TGT = 32;
struct ConvBlock {
    int nsrc, ntgt;
    short src_prime[CONV_MAX_SRC], src_limb[CONV_MAX_SRC];
    short tgt_prime[CONV_MAX_TGT], tgt_limb[CONV_MAX_TGT];
    u64 hatinv[CONV_MAX_SRC], hatinv_s[CONV_MAX_SRC];   // (D/d_j)^-1 mod d_j
    u64 hat[CONV_MAX_TGT][CONV_MAX_SRC];                // (D/d_j) mod r_k
    u64 dmod[CONV_MAX_TGT];                             // D mod r_k
    u64 add_in[CONV_MAX_SRC];                           // added to the input residue before scaling (T -> PQ centring)
    u64 sub_out[CONV_MAX_TGT];                          // subtracted from the output residue (T -> PQ centring)
    short copy_prime[CONV_MAX_SRC], copy_limb[CONV_MAX_SRC];  // ncopy source limbs passed through unchanged
    int ncopy;
    int f64_ok;                                         // every prime of the block is below 2^41: all FP64 tables below are filled
    int split_ok;                                       // every TARGET prime is below 2^50: hat_d, hat31_d and dmod_d are filled
    double hatinv_d[CONV_MAX_SRC];                      // balanced representatives as doubles
    double hat_d[CONV_MAX_TGT][CONV_MAX_SRC];
    double hat31_d[CONV_MAX_TGT][CONV_MAX_SRC];         // (D/d_j) 2^31 mod r_k: the factor of the upper part of a scaled residue split at bit 31
    double dmod_d[CONV_MAX_TGT];
};

struct ConvPlan {          // blocks of one map at one level, contiguous in device memory
    int first = 0, count = 0;
    bool f64_ok = false;   // all blocks can take the FP64 kernel
    bool split_ok = false; // all blocks can take the kernel that scales in integers and sums in FP64
    int max_tgt = 0;       // largest number of targets of a block
};

}  // namespace ckks

struct ckks_ctx {
    int logN = 0, p_num = 0, q_num = 0, t_num = 0, gamma = 0, L = 0, K = 0, dnum = 0;
    int Ri_blockNum = 0, Qj_blockNum = 0, nprimes = 0;
    long N = 0;
    hipStream_t stream = nullptr;
    hipEvent_t ev0 = nullptr, ev1 = nullptr, ev_mid = nullptr;
    std::vector<hipEvent_t> ev_marks;          // ckks_timer_mark: created on first use, destroyed with the context
    bool ev_mid_armed = false;           // record ev_mid between the two passes of the next NTT (per-kernel timing)

    // host copies (reference names, reference layouts) for ckks_ctx_table and for launch-time decisions
    std::vector<uint64_t> pqt, mu_hi, mu_lo, psi, psiinv, n_inv, n_inv_shoup, halfTmodpqti;
    std::vector<uint64_t> psi_table, psiinv_table;                       // [prime][N]
    std::vector<uint64_t> pHatVecModq, pHatInvVecModp, PModqt, PinvModq;
    std::vector<uint64_t> RiHatInv, RiHatModT, Rimodti;
    std::vector<uint64_t> QjHatInv, QjHatModT, Qjmodti;
    std::vector<uint64_t> THatInv, THatModRi, Tmodpqi;
    std::vector<uint64_t> qiInvModql;
    std::vector<int> f64_ok;

    // device tables
    ckks::PrimeConst* d_primes = nullptr;
    ckks::PrimeConst* d_primes_modup = nullptr;     // [level][prime]: d_primes with the digit's (D/q_i)^-1 folded in the same way
    ckks::PrimeConst* d_primes_moddown = nullptr;   // d_primes with (P/p_i)^-1 folded into the inverse transform's final constants of p_i
    ulonglong2* d_tw_fwd = nullptr;       // [prime][N] (w, shoup(w)), index = reference psi_table index
    ulonglong2* d_tw_inv = nullptr;       // [prime][N] from psiinv_table
    double* d_twd_fwd = nullptr;          // [prime][N] balanced doubles, FP64 back end (0 entries for large primes)
    double* d_twd_inv = nullptr;
    ckks::ConvBlock* d_conv = nullptr;    // all conversion blocks
    std::vector<ckks::ConvPlan> plan_pq_to_t, plan_qj_to_t, plan_t_to_pq, plan_hybrid, plan_hybrid_all;   // indexed by level l
    // ModDown / rescale constants on device
    uint64_t* d_pHatVecModq = nullptr;    // [L+1][K]
    uint64_t* d_pHatInvVecModp = nullptr; // [K] then [K] Shoup words
    uint64_t* d_PinvModq = nullptr;       // [L+1] then [L+1] Shoup words
    uint64_t* d_qiInvModql = nullptr;     // triangular (+ Shoup words after)
    size_t qiInv_count = 0;

    int arith_mode = 0;                   // 0: automatic (FP64 where valid), 1: force integer back end
    unsigned res_backwards = 0;           // resident transform: direction in which the next launch walks its rounds (alternates)
    int ntt_mode = 0;                     // 0: automatic, 1: two launches per transform, 2: chained one-launch transform, 3: one workgroup per limb,
                                          // 4: paired one-launch transform at every batch size, 5: the same with a limb's tiles spread over the XCDs
    int cu_count = 256;
    void* d_ntt_mid = nullptr;            // compact inter-pass buffer of the two-launch transform, grown on demand
    size_t ntt_mid_cap = 0;
    int device = 0;                       // the device that was current when the context was created
    struct DecodeTab { int level, words; void* dev; };
    std::vector<DecodeTab> decode_tabs;   // CRT tables of decode_coeffs, one per level, built on first use
    int chain_skew = 0, chain_spin = -1;  // chained transform: limbs a chain's first pass runs ahead of its second (0: default), poll limit of a wait (-1: default)
    void* d_ntt_pair = nullptr;           // completion words of the paired (one-launch, small-batch) transform, one per 128-byte line
    unsigned pair_resident_blocks[6] = {}; // workgroups of each one-launch kernel that fit the chip at once (occupancy x compute units), by PAIR_KIND_*
    // test / tuning switches (ckks_ctx_set_option): the fused key-switch, rescale and ring-packing launches off; the key switch's
    // last steps as separate launches; conversions into primes below 2^50 in 128-bit integers; the second launch of a transform
    // takes the limbs in forward order; limbs per trip through the inter-pass buffer (0: all)
    bool ks_split = false, ks_back_split = false, conv_int = false, ntt_no_reverse = false, pair_no_steal = false;
    int ntt_chunk = 0;
    unsigned* h_pair_fail = nullptr;      // pinned host word that a paired transform raises when one of its waits ran out
    void* d_ntt_chain = nullptr;          // completion words of the chained (one-launch) transform, allocated on its first use; zero between transforms
};

namespace ckks {
void set_error(const std::string& s);
int hip_fail(hipError_t e, const char* what);
#define CKKS_HIP_TRY(expr)                                   \
    do {                                                     \
        hipError_t _e = (expr);                              \
        if (_e != hipSuccess) return ckks::hip_fail(_e, #expr); \
    } while (0)

// launchers (ntt.hip, basisconv.hip)
// chained (one-launch) transform: tiles left to its finishing launch so far, and the host view of its slot order (for tests)
int ntt_chain_deferred(ckks_ctx* c, long* tiles);
// 1 once a paired (one-launch) transform of the context has given up a wait: its output is incomplete and the context unusable
enum { PAIR_KIND_F64 = 0, PAIR_KIND_WIDE, PAIR_KIND_INT, PAIR_KIND_RESCALE, PAIR_KIND_RESCALE_WIDE, PAIR_KIND_KS_BACK };
int ntt_pair_failed(const ckks_ctx* c);
int ntt_pair_deferred(ckks_ctx* c, long* tiles, bool stolen = false);        // second-pass tiles that paired launches have left to their limb's last workgroup (synchronises)
int ntt_extra_forms();                                  // 1 if the library was built with launch forms 2 and 3
int ntt_pair_init(ckks_ctx* c);
void ntt_chain_slot(unsigned s, unsigned tiles, unsigned skew, unsigned* second, unsigned* k, unsigned* tile);
unsigned ntt_chain_slots(unsigned kmax, unsigned tiles, unsigned skew);
// Address, on the current device, of the file-scope inter-pass area of the transform that allocates nothing (looked up once per
// device), its capacity in limbs, and that transform (N = 2^16 with the 5-byte inter-pass form, or any ring in place).
int ntt_noalloc_init(char** ptr_out);
int ntt_noalloc_max_limbs();
int launch_ntt_noalloc(ckks_ctx* c, uint64_t* dev, int start_poly_idx, int start_mod_idx, int poly_num, int mod_num, int poly_mod_len,
                       bool inverse);
// Resident transform (ntt_resident.hip): whether it takes a call of `limbs` limbs, and its launch (FP64 back end, primes below 2^36).
struct NttArgs;
bool ntt_resident_applies(const ckks_ctx* c, int limbs);
int ntt_resident_round(const ckks_ctx* c);              // limbs per round: one per workgroup of its grid
// transforms the first `count` of the call's `limbs` limbs (limb order of the two-launch form)
int launch_ntt_resident(ckks_ctx* c, const NttArgs& args, int limbs, int count, bool inverse);
int launch_ntt(ckks_ctx* c, uint64_t* dev, int start_poly_idx, int start_mod_idx, int poly_num, int mod_num,
               int poly_mod_len, long batch_stride_limbs, int batch, bool inverse);
// Hybrid key switch up to the inverse transform of the two sums, in five launches (four where the input's transform runs as one
// paired launch; with `out` given the whole switch is five) where the separate steps take nine:
//   inverse transform of the input (two passes; the second leaves the residues scaled for the exact conversion, in `work`),
//   the conversion's quotient estimate per digit and coefficient, the conversion inside the first pass of every digit limb's
//   forward transform, the row passes of both transforms around the inner product with the key, the last pass of the sums' inverse
//   transform.  in_ntt: l + 1 limbs of a polynomial of q_num limbs, NTT domain, left untouched; work: at least l + 2 limbs;
//   sums: two polynomials of poly_mod_len limbs, coefficient domain on return, their first p_num limbs multiplied by (P/p_i)^-1 mod p_i
//   (ready for launch_ks_moddown_fused(..., pre_scaled = true)).  *done = false where it does not apply (nothing launched).
// With `out` and `finished` given the call may also finish the switch (the last pass of the sums' inverse transform, the ModDown
// and the results' forward transform, written to two polynomials of out_poly_mod_len limbs): then *finished = true and `sums`
// holds the special-prime limbs only.
int launch_hybrid_front_fused(ckks_ctx* c, const uint64_t* in_ntt, uint64_t* work, uint64_t* sums, const uint64_t* key, int l, bool* done,
                              uint64_t* out = nullptr, int out_poly_mod_len = 0, bool* finished = nullptr);
// Rescale after the inverse transform of limb l (cipher: [2][L+1] limbs, inv: q_l^-1 mod q_i for i < l): the reduction of limb l
// modulo each remaining prime, its forward transform and the final subtraction and scaling in two launches; *done = false where
// it does not apply.
int launch_rescale_fused(ckks_ctx* c, uint64_t* cipher, int l, const uint64_t* inv, bool* done);
// End of a key switch (ModDown of two extended polynomials, forward transform of the results) with the ModDown inside the first
// pass of the transform; *done = false where it does not apply (the caller then runs the separate steps).  With addend set, limb
// i of result z leaves as its sum with addend[(z * addend_poly_stride + i) * N ...] (NTT domain, canonical).
int launch_ks_moddown_fused(ckks_ctx* c, uint64_t* out, const uint64_t* in, long in_z_stride, int l, int out_poly_mod_len, bool pre_scaled,
                            bool* done, const uint64_t* addend = nullptr, long addend_poly_stride = 0);
// ckks_keyswitch_23 with the option of adding addend (as above) to the result inside the last launch; *added tells whether it was.
int keyswitch_23_add(ckks_ctx* c, uint64_t* out, uint64_t* d2, const uint64_t* swk, int l, uint64_t* up, uint64_t* ext, uint64_t* buf,
                     const uint64_t* addend, long addend_poly_stride, bool* added);
// Key switch through the T basis: external product of the digits `up` (NTT domain over T) with the key `swk` and inverse transform
// of the sums into `ext` (coefficient domain on return), the product and the first pass of the transform in one launch;
// *done = false where it does not apply (nothing launched: the caller runs the separate steps).
int launch_ext_product_inverse_fused(ckks_ctx* c, uint64_t* ext, const uint64_t* up, const uint64_t* swk, int l, bool* done);
// Forward transform whose first pass reads its input from MLWE samples (the embedding of the ring packing) instead of dev:
// coefficient pos of polynomial y = coefficient pos >> logk of row y of sample (pos mod 2^logk) >> loggap, zero where pos mod 2^logk
// is no multiple of 2^loggap; on the limbs of prime start_mod_idx the value is lifted around zero from q0 to p0.
// mlwe: DEVICE table of sample pointers, each [(k+1)][n1] words of one modulus.
struct NttEmbedSource {
    const uint64_t* const* mlwe;
    uint64_t p0, q0;
    int logk, loggap, n1;
};
int launch_ntt_embedded(ckks_ctx* c, uint64_t* dev, int start_poly_idx, int start_mod_idx, int poly_num, int mod_num, int poly_mod_len,
                        const NttEmbedSource& src);
// Ring packing up to the inner product with the repacking keys: first pass of the forward transform of the `rank` embedded
// polynomials (two limbs each, modulo primes prime0 and prime0 + 1, gathered from the samples), then their row pass and the
// products with the keys in one launch, then the sum over chunks.  work: 2 * rank limbs of scratch; acc: [z][limb][N] sums in
// the NTT domain.  *done = false where it does not apply (the caller then runs the separate steps).
int launch_repack_front_fused(ckks_ctx* c, uint64_t* work, uint64_t* acc, const uint64_t* keys, int rank, int prime0,
                              const NttEmbedSource& src, bool* done);
}  // namespace ckks

// Device memory [lo, lo + bytes) was freed or overwritten through the library's own plumbing: every ring-pack handle forgets the
// plaintext matrices it had prepared from there (pcmm.hip).
void pcmm_forget_weights(const void* lo, size_t bytes, bool freed = false);
