/*
 * CPU oracle for the CKKS arithmetic hot path (RNS negacyclic NTT, RNS basis
 * conversion / key switching, ring-packed plaintext x ciphertext matrix product).
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  It is a plain, single-threaded
 * (optionally OpenMP) restatement of the arithmetic of haozetao/ckks_llm, written
 * from the reference's sources read as text; every function cites the reference
 * file:line it follows.  Only tests/, __graft_entry__.smoke() and bench.py's
 * cpu_baseline leg may load it.  The shipped library never links or calls it.
 *
 * All polynomial data are host arrays of uint64_t in the reference's limb-major
 * layout: limb = N consecutive words of one polynomial modulo one prime.
 * Prime index space ("pqt order"): [p_0..p_{K-1} | q_0..q_L | t_0..t_{tnum-1}]
 * (Context_23.cuh:63-113).
 *
 * Pinning status of each group of functions (what fixes it besides this file):
 *   modmath / Shoup / Barrett      brute force against __uint128_t %            (tests/test_oracle_modmath.py)
 *   root / table generation        psi^N = -1, table inverse identities, sympy  (tests/test_oracle_tables.py)
 *   NTT / iNTT                     closed form NTT(X^k), negacyclic schoolbook
 *                                  convolution, the reference notebook's KAT in
 *                                  Z_65537[x]/(x^32+1)                          (tests/test_oracle_ntt.py)
 *   base conversions, ModDown      exact big-integer CRT in Python              (tests/test_oracle_basisconv.py)
 *   external / inner product       Python big-int brute force                   (tests/test_oracle_basisconv.py)
 *   RLWE->MLWE gather              ring identity at N=32 against negacyclic
 *                                  algebra in Python                            (tests/test_oracle_pcmm.py)
 *   PPMM                           Python big-int brute force + fused-rescale
 *                                  closed form                                  (tests/test_oracle_pcmm.py)
 *   Salsa20 stream                 ECRYPT known-answer vectors                  (tests/test_oracle_scheme.py)
 *   samplers                       scipy's normal tail for the Gaussian steps,
 *                                  exact probabilities, hand-worked words       (tests/test_oracle_scheme.py)
 *   keys, encryption, decryption   decrypt identities with Python negacyclic
 *                                  algebra (a*s + b = m + small noise)          (tests/test_oracle_scheme.py)
 *   coefficient encode / decode    Python big-integer CRT and exact rationals   (tests/test_oracle_scheme.py)
 *   NTT-domain automorphisms       coefficient-domain substitution X -> X^g     (tests/test_oracle_keys.py)
 *   MLWE secret, repacking keys,   s_i[n] = s[i + n*rank]; a*s + b = p0*iota(s_i) + small e; MLWE decryption of the
 *   MLWE decryption                gather = the RLWE message at the gathered positions; whole pipeline decrypts to
 *                                  W times the message with generated keys     (tests/test_oracle_pcmm.py)
 *   switching keys, mult / rotate  decrypt identities: product of messages,
 *   / conjugate                    m(X^(5^r)), m(X^-1), within a noise bound   (tests/test_oracle_keys.py)
 */
#pragma once
#include <stdint.h>
#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct orc_ctx orc_ctx;
typedef struct orc_pcmm orc_pcmm;

/* ---- scalar modmath: Utils.cuh:14-53, uint128.cuh:143-212 ---- */
uint64_t orc_mulmod(uint64_t a, uint64_t b, uint64_t q);
uint64_t orc_powmod(uint64_t a, uint64_t e, uint64_t q);
uint64_t orc_invmod(uint64_t a, uint64_t q);
uint64_t orc_xshoup(uint64_t x, uint64_t q);
uint64_t orc_mulmod_shoup(uint64_t a, uint64_t b, uint64_t b_shoup, uint64_t q);
void     orc_barrett_mu(uint64_t q, uint64_t* mu_hi, uint64_t* mu_lo);
uint64_t orc_barrett128(uint64_t a_hi, uint64_t a_lo, uint64_t q, uint64_t mu_hi, uint64_t mu_lo);
uint64_t orc_barrett64(uint64_t a, uint64_t q, uint64_t mu_hi);
/* ---- roots and tables: Utils.cuh:63-109,125-132,190-210 ---- */
uint64_t orc_find_primitive_root(uint64_t q);
uint64_t orc_find_mth_root(uint64_t M, uint64_t q);
uint32_t orc_bitrev(uint32_t x, int bits);
void orc_fill_psi_tables(uint64_t psi, uint64_t q, uint32_t n, uint64_t* psi_tab, uint64_t* psiinv_tab,
                         uint64_t* psi_shoup, uint64_t* psiinv_shoup);
/* ---- stand-alone transforms on one limb (table-driven; python/ntt.ipynb cell 2 loop shape) ---- */
void orc_ntt_limb(uint64_t* a, uint32_t n, uint64_t q, const uint64_t* psi_tab);
void orc_intt_limb(uint64_t* a, uint32_t n, uint64_t q, const uint64_t* psiinv_tab_with_ninv, uint64_t n_inv);
/* schoolbook negacyclic product, Utils.cuh:255-285 */
void orc_negacyclic_mul(const uint64_t* a, const uint64_t* b, uint64_t* c, uint32_t n, uint64_t q);

/* ---- context: Context_23.cuh:12-472 ---- */
orc_ctx* orc_ctx_create(int logN, const uint64_t* p, int p_num, const uint64_t* q, int q_num,
                        const uint64_t* t, int t_num, int gamma);
void orc_ctx_destroy(orc_ctx*);
/* copies a named constant table (flattened in the reference's device layout) ; returns element count or -1 */
long orc_ctx_get(const orc_ctx*, const char* name, uint64_t* out, long cap);
int  orc_ctx_info(const orc_ctx*, const char* name);

/* Context_23.cuh:847-930 addressing: limb (poly y, mod j) at a + (y*poly_mod_len + start_poly_idx + j)*N,
 * prime index start_mod_idx + j. */
int orc_ntt_fwd(const orc_ctx*, uint64_t* a, int start_poly_idx, int start_mod_idx, int poly_num, int mod_num, int poly_mod_len);
int orc_ntt_inv(const orc_ctx*, uint64_t* a, int start_poly_idx, int start_mod_idx, int poly_num, int mod_num, int poly_mod_len);
int orc_ntt_fwd_ext(const orc_ctx*, uint64_t* a, int start_poly_idx, int start_mod_idx, int poly_num, int mod_num,
                    int poly_mod_len, int cipher_mod_num, int batch_size);
int orc_ntt_inv_ext(const orc_ctx*, uint64_t* a, int start_poly_idx, int start_mod_idx, int poly_num, int mod_num,
                    int poly_mod_len, int cipher_mod_num, int batch_size);

/* BasisConv.cuh */
int orc_modup_pq_to_t(const orc_ctx*, uint64_t* out, const uint64_t* in, int l, int batch);
int orc_modup_qj_to_t(const orc_ctx*, uint64_t* out, const uint64_t* in, int l, int batch);
int orc_modup_t_to_pql(const orc_ctx*, uint64_t* buf, const uint64_t* in, int l, int batch);
int orc_moddown_pql_to_ql(const orc_ctx*, uint64_t* out, const uint64_t* buf, int l, int batch);
/* ExternalProduct.cuh:7-97 */
int orc_external_product_t(const orc_ctx*, uint64_t* out, const uint64_t* c_T, const uint64_t* swk_T, int l);
int orc_external_product_t_swk_reuse(const orc_ctx*, uint64_t* out, const uint64_t* c_T, const uint64_t* swk_T, int l, int batch_size);
/* Scheme_23.cuh:321-385 ; cipher = [a: L+1 limbs | b: L+1 limbs], NTT domain, level l -> l-1 */
int orc_rescale(const orc_ctx*, uint64_t* cipher, int l);
/* KeySwitch_23.cuh:216-231 (steps 2..9 of mult_23 without the tensor product):
 * d2 (NTT domain, q_num limbs, level l) -> out = [a: q_num limbs | b: q_num limbs] (NTT domain). */
int orc_keyswitch_23(const orc_ctx*, uint64_t* out, const uint64_t* d2, const uint64_t* swk_T, int l);

/* textbook hybrid key switch over [P | Q_l] (BASELINE config 3); alpha = p_num primes per digit.
 * digits_out: [dnum_l][p_num+q_num] limbs, coefficient domain in/out. */
int orc_hybrid_modup(const orc_ctx*, uint64_t* digits_out, const uint64_t* in, int l);
int orc_hybrid_inner_product(const orc_ctx*, uint64_t* out, const uint64_t* digits, const uint64_t* evk, int l);
int orc_hybrid_moddown(const orc_ctx*, uint64_t* out, const uint64_t* in, int l);
int orc_hybrid_keyswitch(const orc_ctx*, uint64_t* out, const uint64_t* in_ntt, const uint64_t* evk, int l);

/* ---- ring-packed PCMM: pcmm/PCMM_Context.cuh, PCMM_Scheme.cuh:50-125, PPMM_kernel.cuh ---- */
orc_pcmm* orc_pcmm_create(const orc_ctx*, int N1, int rank, const uint64_t* p_ringpack, int np,
                          const uint64_t* q_ringpack, int nq);
void orc_pcmm_destroy(orc_pcmm*);
/* rlwe = [a: L+1 limbs | b: L+1 limbs] in COEFFICIENT domain (the caller does the iNTT / NTT around it);
 * mlwe[m] -> buffer of mlwe_L1 * (rank+1) * N1 words. */
int orc_rlwe_decompose(const orc_pcmm*, const uint64_t* rlwe, uint64_t* const* mlwe, int mlwe_num, int l);
/* W: row-major [M][Kin] fp32. mlwe[n]: [mod][rank+1][N1]. out: [M][mod_num][(rank+1)*N1].
 * col_begin/col_count restrict the computed column range (for timing a panel); pass 0,(rank+1)*N1 for all. */
int orc_ppmm(const orc_pcmm*, const float* W, const uint64_t* const* mlwe, uint64_t* out, int M, int Kin,
             int mod_num, double scaler, long col_begin, long col_count);

/* PCMM_Scheme::mlweCipherPacking (PCMM_Scheme.cuh:361-425): mlwe_num MLWE ciphertexts [(nq-1)][(rank+1)][N1] (coefficient
 * domain) -> one RLWE ciphertext [a | b] (L+1 limbs each, limbs 0..nq-2 written, NTT domain) with rank repacking keys
 * (key i at keys + i*N*mod_num*2 = [a | b], mod_num = np+nq-1 limbs, NTT domain).  One special prime, two ring-pack moduli. */
int orc_mlwe_pack(const orc_pcmm*, uint64_t* rlwe_out, const uint64_t* const* mlwe, int mlwe_num, const uint64_t* keys);

/* PCMM_Context::ToNTTInplace / FromNTTInplace (PCMM_Context.cuh:243-273): size-N1 transforms over the ring-pack primes,
 * layout [mod_batch_size][mod_num][poly_num][N1], prime pq_ringpack[start_mod_idx + j]. */
int orc_pcmm_ntt(const orc_pcmm*, uint64_t* data, int poly_num, int mod_num, int start_mod_idx, int mod_batch_size, int inverse);

/* ---- randomness, samplers, pointwise arithmetic, keys, encryption, coefficient encoding ---- */
void orc_salsa20_stream(uint8_t* out, size_t n, const uint8_t key[32], uint64_t nonce);
void orc_gauss_thresholds(uint32_t thr[19]);
int orc_sample_uniform(const orc_ctx*, const uint8_t* random, uint64_t* out, int idx_out, int idx_mod, int mod_num);
int orc_sample_gaussian(const orc_ctx*, const uint8_t* random, uint64_t* out, int idx_out, int idx_mod, int mod_num);
int orc_sample_zo(const orc_ctx*, const uint8_t* random, uint64_t* out, double probability, int idx_out, int idx_mod, int mod_num);
int orc_sample_hwt(const orc_ctx*, const uint8_t* random, uint64_t* out, int h, int idx_out, int idx_mod, int mod_num);
int orc_poly_op(const orc_ctx*, int op, uint64_t* c, const uint64_t* a, const uint64_t* b, int idx_c, int idx_a, int idx_b,
                int idx_mod, int mod_num);
int orc_keygen_secret(const orc_ctx*, uint64_t* sx, const uint8_t* random, int h);
int orc_keygen_public(const orc_ctx*, uint64_t* pk, const uint64_t* sx, const uint8_t* random_a, const uint8_t* random_e);
int orc_encrypt(const orc_ctx*, uint64_t* cipher, const uint64_t* mx, const uint64_t* pk, const uint8_t* random, int l);
int orc_decrypt(const orc_ctx*, uint64_t* mx, const uint64_t* cipher, const uint64_t* sx, int l);
int orc_encode_coeffs(const orc_ctx*, uint64_t* mx, const double* vals, long scale, int l);

/* ---- automorphisms, switching keys in the T basis, homomorphic multiply / rotate / conjugate ---- */
uint64_t orc_rot_group(const orc_ctx*, long idx);
int orc_automorph_ntt(const orc_ctx*, uint64_t* out, const uint64_t* in, uint64_t pow, int idx_out, int idx_in, int mod_num);
int orc_conjugate_ntt(const orc_ctx*, uint64_t* out, const uint64_t* in, int idx_out, int idx_in, int mod_num);
int orc_keygen_switch_23(const orc_ctx*, uint64_t* swk, const uint64_t* s_to, const uint64_t* s_from, const uint8_t* random_a,
                         const uint8_t* random_e);
int orc_mult_23(const orc_ctx*, uint64_t* out, const uint64_t* c1, const uint64_t* c2, const uint64_t* rlk, int l);
int orc_rotate_23(const orc_ctx*, uint64_t* out, const uint64_t* cipher, const uint64_t* rotkey, long rot, int l);
int orc_conjugate_23(const orc_ctx*, uint64_t* out, const uint64_t* cipher, const uint64_t* conjkey, int l);
/* hoisted rotations of the slot <-> coefficient transforms (Bootstrapping_C2S_S2C_impl.cuh) */
int orc_cipher_mul_p(const orc_ctx*, uint64_t* out, const uint64_t* cipher, int l);
int orc_cipher_add_t(const orc_ctx*, uint64_t* a, const uint64_t* b, int blocks);
int orc_rescale_coeff(const orc_ctx*, uint64_t* cipher, int l);
int orc_giant_rotate_mult_plain_t(const orc_ctx*, uint64_t* bs_cipher_T, const uint64_t* PQ_to_T, const uint64_t* modUp_QjtoT,
                                  const uint64_t* const* rotKeys, const int* rotSlots, const uint64_t* const* plaintextT, const int* accNum,
                                  int bs, int gs, int l);
int orc_baby_rotate(const orc_ctx*, uint64_t* output, const uint64_t* modUp_QjtoT, const uint64_t* input, int rotNum,
                    const uint64_t* const* rotKeys, const int* rotSlots, int l);
int orc_bsgs_level_23(const orc_ctx*, uint64_t* cipher, int l, const uint64_t* const* plaintextT, const int* accNum, const int* rot_in,
                      const uint64_t* const* rot_in_keys, const int* rot_out, const uint64_t* const* rot_out_keys, int bs, int gs);

/* ---- MLWE secret key, repacking keys, MLWE decryption ---- */
int orc_pcmm_convert_mlwe_sk(const orc_pcmm*, uint64_t* mlwe_sk, const uint64_t* rlwe_sk);
int orc_pcmm_add_repacking_key(const orc_pcmm*, uint64_t* keys, const uint64_t* mlwe_sk, const uint64_t* rlwe_sk, const uint8_t* random);
int orc_pcmm_mlwe_decrypt(const orc_pcmm*, uint64_t* plain, const uint64_t* cipher, const uint64_t* mlwe_sk, int l);
int orc_pcmm_decode_coeffs(const orc_pcmm*, double* vals, const uint64_t* plain, long long scaler, int l);

int orc_max_threads(void);

#ifdef __cplusplus
}
#endif
