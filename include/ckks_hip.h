/*
 * C ABI of the MI355X (gfx950) implementation of the CKKS arithmetic hot path:
 * batched RNS negacyclic NTT / iNTT, RNS basis conversion for key switching, and the ring-packed
 * plaintext x ciphertext matrix product (PPMM).
 *
 * The reference (haozetao/ckks_llm) has no FFI layer: its boundary for this path is a set of C++ member
 * functions compiled into the caller.  Each entry point below replaces one of them and cites it; argument
 * order and meaning follow the reference.  All polynomial pointers are DEVICE pointers to uint64_t in the
 * reference's limb-major layout (limb = N consecutive words of one polynomial modulo one prime); prime
 * indices are in "pqt order" [p_0..p_{K-1} | q_0..q_L | t_0..t_{tnum-1}] (Context_23.cuh:63-113).
 *
 * Every function returns 0 on success or a negative CKKS_E_* code; ckks_last_error() gives the text.
 * A handle owns its device tables (the reference keeps them in process-global __constant__ symbols, so it can
 * hold one context per process; here any number of contexts may coexist).  Work is issued on the stream set
 * with ckks_set_stream (default: the null stream); calls on one handle from several host threads must be
 * serialised by the caller, as in the reference.
 */
#ifndef CKKS_HIP_H
#define CKKS_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CKKS_OK 0
#define CKKS_E_INVALID (-1)   /* bad argument (level, shape, unsupported size) */
#define CKKS_E_HIP (-2)       /* a HIP runtime call failed */
#define CKKS_E_NOMEM (-3)
#define CKKS_E_STATE (-4)     /* e.g. missing key / level-0 operand: the C++ shell maps it to std::invalid_argument */
#define CKKS_E_UNAVAILABLE (-5) /* a code path that this build has switched off, or a device-side wait that ran out */

typedef struct ckks_ctx ckks_ctx;
typedef struct pcmm_ctx pcmm_ctx;

const char* ckks_last_error(void);
const char* ckks_version(void);

/* ---- device memory and stream plumbing (cudaMalloc / cudaMemcpy / cudaDeviceSynchronize of the reference) ---- */
int ckks_malloc(void** dev_ptr, size_t bytes);
int ckks_free(void* dev_ptr);
int ckks_memcpy_h2d(void* dst_dev, const void* src_host, size_t bytes);
int ckks_memcpy_d2h(void* dst_host, const void* src_dev, size_t bytes);
int ckks_memcpy_d2d(void* dst_dev, const void* src_dev, size_t bytes);
int ckks_memset(void* dst_dev, int value, size_t bytes);
int ckks_sync(void);
int ckks_device_count(int* count);
/* HIP-event timing on the context's stream (replaces CUDATimer, TimeUtils.cuh:10-35) */
int ckks_timer_start(ckks_ctx* ctx);
int ckks_timer_stop(ckks_ctx* ctx, float* elapsed_ms);
/* Marks between launches queued back to back: ckks_timer_mark records event `slot` (0 .. 4095) on the context's stream and
 * returns at once; ckks_timer_between waits for mark slot_b and gives the time from mark slot_a to it.  A measurement aid with
 * no counterpart in the reference (its CUDATimer brackets one region). */
int ckks_timer_mark(ckks_ctx* ctx, int slot);
int ckks_timer_between(ckks_ctx* ctx, int slot_a, int slot_b, float* elapsed_ms);

/* ---- context: Context_23::Context_23 + getPrimeCKKS + preComputeOnCPU + copyMemoryToGPU
 *      (Context_23.cuh:12-472, 475-701; Params.cuh).  Primes are passed explicitly; gamma is the block width of
 *      the [P|Q] -> T conversion (Params.cuh "gamma").  t_num may be 0 (no auxiliary basis), p_num may be 0. ---- */
int ckks_ctx_create(ckks_ctx** out, int logN, const uint64_t* p, int p_num, const uint64_t* q, int q_num,
                    const uint64_t* t, int t_num, int gamma);
int ckks_ctx_destroy(ckks_ctx* ctx);
int ckks_set_stream(ckks_ctx* ctx, void* hip_stream);
/* scalar facts: "N","logN","p_num","q_num","t_num","gamma","dnum","Ri_blockNum","Qj_blockNum","arith_mode","ntt_mode";
 * "ntt_mid_bytes": size of the inter-pass buffer that the ordinary transforms have grown so far;
 * "ntt_pair_deferred_tiles" (synchronises): second-pass tiles that paired transforms have left to the last workgroup of their limb;
 * "ntt_pair_resident_blocks" / "ntt_pair_resident_blocks_int": workgroups of the paired transform kernel (FP64 / integer back end) that the chip
 * holds at once; "ntt_pair_stolen_tiles" (synchronises): first-pass tiles taken over from workgroups that had not started; "ntt_extra_forms": 1 if
 * modes 2 and 3 are built in;
 * "ntt_chain_deferred_tiles" (synchronises): second-pass tiles that chained transforms have left to their finishing launch;
 * "ntt_resident_round": limbs that one round of the resident transform takes (one per compute unit; 0 where it never applies) */
int ckks_ctx_info(const ckks_ctx* ctx, const char* name, long* value);
/* 0 (default): FP64 butterflies for primes < 2^41, integer butterflies otherwise; 1: integer butterflies everywhere.
 * Both give the same residues; the switch exists for testing and tuning. */
int ckks_ctx_set_arith_mode(ckks_ctx* ctx, int mode);
/* How a transform is launched.  0 (default): chosen by the library; 1: two launches, one per pass, data in place between
 * them; 2: chained - both passes in one launch, the second pass of a limb following its first pass on the same XCD so that
 * the limb stays in that XCD's L2 in between (N >= 2^15; other rings take two launches), plus a small finishing launch;
 * 3: one workgroup carries a limb through both passes (N >= 2^15); 4: paired - both passes in one launch of one workgroup per
 * (limb, tile), which waits between its two tiles until the limb's first pass is complete (N = 2^16, up to 4096 limbs; mode 0
 * takes this form for batches of up to 128 limbs, where it is faster than two launches); 5: as 4 with the tiles of a limb spread
 * over all XCDs (what mode 0 does above 40 limbs); 6: resident - one persistent workgroup per compute unit carries whole limbs
 * through both passes in its registers, so that a limb crosses HBM once in and once out (N = 2^16, primes below 2^36, at least one
 * limb per compute unit; mode 0 takes it there too, for the whole rounds of a batch).  All give the same residues.  Modes 2 and 3
 * exist only in a library built with CKKS_NTT_EXTRA_FORMS (they lose to two launches at every size; the default build leaves
 * them out and runs two launches where they are asked for).  The paired form completes whatever part of its grid the chip holds
 * at once and in whatever order its workgroups start: a workgroup that waits too long takes over the tiles of workgroups that have
 * not started, and what it leaves undone the last workgroup of the limb completes.
 * No counterpart in the reference (its transforms are always two launches, Context_23.cuh:847-889). */
int ckks_ctx_set_ntt_mode(ckks_ctx* ctx, int mode);
/* Synchronises the context's stream and returns what HIP reports for the launches so far.  Plays the part of the reference's
 * cudaDeviceSynchronize + cudaGetLastError checks (Utils.cuh CUDA_CHECK). */
int ckks_ctx_check(ckks_ctx* ctx);
/* Test / tuning hook of the chained transform (mode 2).  skew: limbs that a chain's first pass runs ahead of its second pass
 * (0 = default); spin_max: polls that a second-pass workgroup spends waiting for its limb's first pass before it leaves its tile
 * to the finishing launch (-1 = default; 0 sends every tile there).  Results do not depend on either.  spin_max also bounds
 * the waits of the paired transform (modes 0, 4, 5): 0 makes every workgroup take over what it can at once and leave its second
 * pass to the last workgroup of its limb ("ntt_pair_deferred_tiles" of ckks_ctx_info counts those), with the same results.
 * The one wait that can still fail is in the last launch of the fused hybrid key switch (its ModDown workgroups wait for the
 * special-prime workgroups of the same grid, which the launcher only uses while the whole grid fits the chip): should it run
 * out, ckks_ctx_check and every later call on the context return CKKS_E_UNAVAILABLE. */
int ckks_ctx_set_ntt_chain(ckks_ctx* ctx, int skew, int spin_max);
/* Test / tuning switches of a context, by name (value 0 = off, the default).  Results do not depend on any of them.
 *   "ks_split"        the hybrid key switch, the rescale and the ring packing run their stages as separate launches
 *   "ks_back_split"   the hybrid key switch runs its last three steps as separate launches
 *   "conv_int"        basis conversions into primes below 2^50 accumulate in 128-bit integers instead of FP64
 *   "ntt_no_reverse"  the second launch of a two-launch transform takes the limbs in forward order
 *   "ntt_chunk"       value = limbs per trip through the inter-pass buffer of a two-launch transform (0: the whole batch) */
int ckks_ctx_set_option(ckks_ctx* ctx, const char* name, long value);
/* Order of work of the chained transform, for tests: slot `slot` of a chain of `tiles` workgroups per pass -> pass (0 / 1),
 * index k of the limb within the chain and tile; ckks_ntt_chain_slots = slots of a chain of kmax limbs.  Pure host functions. */
int ckks_ntt_chain_slot(unsigned slot, unsigned tiles, unsigned skew, unsigned* second, unsigned* k, unsigned* tile);
unsigned ckks_ntt_chain_slots(unsigned kmax, unsigned tiles, unsigned skew);
/* host copy of a constant table, flattened in the reference's device layout (names as in ckks_oracle.h /
 * Context_23.h: "pqt","psi","psi_table","psiinv_table","RiHatInv","QjHatModT",...). *count receives the length. */
int ckks_ctx_table(const ckks_ctx* ctx, const char* name, uint64_t* host_out, size_t cap, size_t* count);

/* ---- NTT: Context_23::ToNTTInplace / FromNTTInplace (Context_23.cuh:847-889; kernels ntt_60bit.cuh:421-901).
 * Limb (y, j), y < poly_num, j < mod_num, lives at dev + (y*poly_mod_len + start_poly_idx + j)*N and is
 * transformed modulo prime start_mod_idx + j.  Forward: natural -> bit-reversed order; inverse: bit-reversed ->
 * natural order, scaled by N^-1.  Outputs are fully reduced. ---- */
int ckks_ntt_fwd(ckks_ctx* ctx, uint64_t* dev, int start_poly_idx, int start_mod_idx, int poly_num, int mod_num,
                 int poly_mod_len);
int ckks_ntt_inv(ckks_ctx* ctx, uint64_t* dev, int start_poly_idx, int start_mod_idx, int poly_num, int mod_num,
                 int poly_mod_len);
/* Context_23::ToNTTInplace_for_externalProduct / FromNTTInplace_for_externalProduct (Context_23.cuh:891-930):
 * same, repeated batch_size times with a stride of cipher_mod_num limbs. */
int ckks_ntt_fwd_ext(ckks_ctx* ctx, uint64_t* dev, int start_poly_idx, int start_mod_idx, int poly_num, int mod_num,
                     int poly_mod_len, int cipher_mod_num, int batch_size);
int ckks_ntt_inv_ext(ckks_ctx* ctx, uint64_t* dev, int start_poly_idx, int start_mod_idx, int poly_num, int mod_num,
                     int poly_mod_len, int cipher_mod_num, int batch_size);

/* The same transform as ckks_ntt_fwd (inverse = 0) / ckks_ntt_inv (inverse != 0), for callers that cannot allocate device
 * memory: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference.
 * The ordinary entry points keep the data between the two launches of a transform at N = 2^16 in a buffer that they allocate
 * and grow on demand; this one keeps it in a fixed device array inside the library (ckks_ntt_noalloc_max_limbs() limbs of
 * 320 KiB = 20 MiB per GPU, held until the process ends) and calls no allocating routine.  poly_num * mod_num above that limit
 * returns CKKS_E_INVALID.  All calls on one GPU share the array: calls that overlap on one GPU (two streams, two host threads)
 * race.  The call runs as two launches whatever launch form the context is set to and changes nothing in the context, so it
 * may run beside other host threads' calls on the same context (on data of their own).  The context must have been created on
 * the current device.  Results are those of ckks_ntt_fwd / ckks_ntt_inv. */
int ckks_ntt_noalloc(ckks_ctx* ctx, uint64_t* dev, int start_poly_idx, int start_mod_idx, int poly_num, int mod_num,
                     int poly_mod_len, int inverse);
int ckks_ntt_noalloc_max_limbs(void);

/* Measurement aid of the benchmark (no counterpart in the reference): int8 multiply-accumulates per second that a loop of
 * v_mfma_i32_16x16x64_i8 on registers alone reaches on the current device, two workgroups of 512 lanes per compute unit, timed
 * with HIP events on `stream` (NULL: the default stream).  The ceiling that the PPMM contraction is set against beside the
 * published peak. */
int ckks_measure_mfma_i8_peak(void* stream, double* macs_per_s);

/* One transform with HIP-event timing of its two kernel launches (strided pass and row pass; the forward transform
 * runs the strided pass first, the inverse the row pass first).  Replaces the cudaEvent pairs of ntt_throughput.cu:51-60. */
int ckks_ntt_timed(ckks_ctx* ctx, uint64_t* dev, int start_poly_idx, int start_mod_idx, int poly_num, int mod_num,
                   int poly_mod_len, int inverse, float* first_pass_ms, float* second_pass_ms);

/* ---- basis conversion: Context_23::modUpPQtoT_23 / modUpQjtoT_23 / modUpTtoPQl_23 / modDownPQltoQl_23
 *      (BasisConv.cuh:61-77, 161-179, 243-254, 328-347; strides as indexed at :25,:52,:110,:142,:201,:239,:304,:325) ---- */
int ckks_modup_pq_to_t(ckks_ctx* ctx, uint64_t* out, const uint64_t* in, int l, int batch_size);
int ckks_modup_qj_to_t(ckks_ctx* ctx, uint64_t* out, const uint64_t* in, int l, int batch_size);
int ckks_modup_t_to_pql(ckks_ctx* ctx, uint64_t* buf, const uint64_t* in, int l, int batch_size);
int ckks_moddown_pql_to_ql(ckks_ctx* ctx, uint64_t* out, const uint64_t* buf, int l, int batch_size);
/* Context_23::external_product_T (ExternalProduct.cuh:85-97); swk laid out as Key_decomp (Key_decomp.cuh:19-24) */
int ckks_external_product_t(ckks_ctx* ctx, uint64_t* out, const uint64_t* c_T, const uint64_t* swk_T, int l);
/* Context_23::external_product_T_swk_reuse (Context_23.h:62, ExternalProduct.cuh:103-162): one switching key against batch_size
 * (1 .. 8) digit sets.  Set it of c_T starts Qj_blockNum * t_num limbs behind set it - 1 (the layout modUpQjtoT_23 writes for a
 * batch); out holds 2 * batch_size polynomials of Ri_blockNum * t_num limbs: polynomials 2 it and 2 it + 1 are the pair of set it. */
int ckks_external_product_t_swk_reuse(ckks_ctx* ctx, uint64_t* out, const uint64_t* c_T, const uint64_t* swk_T, int l, int batch_size);
/* Scheme_23::rescaleAndEqual (Scheme_23.cuh:369-385): cipher = [a: L+1 limbs | b: L+1 limbs], level l -> l-1.
 * scratch: 2*(L+1)*N words (Scheme_23::rescale_buffer). */
int ckks_rescale(ckks_ctx* ctx, uint64_t* cipher, uint64_t* scratch, int l);
/* steps 2..9 of Scheme_23::mult_23 (KeySwitch_23.cuh:219-231): d2 (NTT domain, L+1 limbs, overwritten with its
 * coefficient form) -> out = [a | b] (NTT domain).  Scratch buffers are the reference's
 * modUp_QjtoT_temp (N*t_num*Qj_blockNum), exProduct_T_temp and modUp_TtoQj_buffer (N*t_num*Ri_blockNum*2 each). */
int ckks_keyswitch_23(ckks_ctx* ctx, uint64_t* out, uint64_t* d2, const uint64_t* swk_T, int l,
                      uint64_t* modUp_QjtoT_temp, uint64_t* exProduct_T_temp, uint64_t* modUp_TtoQj_buffer);

/* ---- textbook hybrid key switch over [P | Q_l] with alpha = p_num primes per digit.  No counterpart in the
 * reference (its switch goes through T); built from the reference's exact-conversion recipe (BasisConv.cuh:18-58)
 * and ModDown (BasisConv.cuh:286-326).  digits: [ceil((l+1)/p_num)][p_num+q_num] limbs;
 * evk: [2][ceil(q_num/p_num)][p_num+q_num] limbs (NTT domain); ip/in_pq: [2][p_num+q_num] limbs; out: [2][q_num]. ---- */
int ckks_hybrid_modup(ckks_ctx* ctx, uint64_t* digits, const uint64_t* in_coeff, int l);
int ckks_hybrid_inner_product(ckks_ctx* ctx, uint64_t* ip, const uint64_t* digits_ntt, const uint64_t* evk, int l);
int ckks_hybrid_moddown(ckks_ctx* ctx, uint64_t* out, const uint64_t* in_pq_coeff, int l);
/* whole switch: in_ntt (q_num limbs, NTT domain; on return either overwritten with its coefficient form or left as it was,
 * depending on the kernels the ring size and primes admit) -> out [2][q_num] NTT domain.
 * scratch: (ceil((l+1)/p_num) + 2) * (p_num+q_num) * N words. */
int ckks_hybrid_keyswitch(ckks_ctx* ctx, uint64_t* out, uint64_t* in_ntt, const uint64_t* evk, int l, uint64_t* scratch);

/* ---- randomness, samplers, pointwise arithmetic, keys, encryption, coefficient encoding (the client side of the path) ---- */
/* RNG::generateRandom_device (RNG.cuh:18-56; kernel VecCrypt, RNG_impl.cuh:72-176): n_bytes of the Salsa20/20 key stream of
 * (32-byte key, 64-bit nonce), block counter from 0, written to dev.  The reference draws key and nonce from rand() and leaves
 * the cipher's four diagonal words at zero (RNG_impl.cuh:37 is never written); here they are Salsa20's constants, so the output
 * is the published cipher's stream.  A trailing partial block is truncated (the reference stops at floor(n/64) blocks). */
int ckks_random_bytes(ckks_ctx* ctx, uint8_t* dev, size_t n_bytes, const uint8_t* key32, uint64_t nonce);
/* Sampler::uniformSampler_xq / gaussianSampler_xq / ZOSampler / HWTSampler (Sampler.cuh:17-41; conversions Sampler_impl.cuh:13-113).
 * random: device bytes (8 per value and limb for uniform; 4 per coefficient for gaussian; 1 per coefficient for ZO; 4*h + h for
 * HWT), out: limbs idx_out.. of a device polynomial, primes idx_mod.. in pqt order.  Uniform, ZO and HWT give the reference's
 * values for the same bytes; HWT zeroes the limbs first, lets the later word win when two name one position (a race in the
 * reference), and keeps the reference's output offset idx_out + idx_mod.  The Gaussian (sigma 3.2, |value| <= 19) is the
 * reference's step function of the 32-bit word with the steps placed by integer thresholds instead of float arithmetic. */
int ckks_sample_uniform(ckks_ctx* ctx, const uint8_t* random, uint64_t* out, int idx_out, int idx_mod, int mod_num);
int ckks_sample_gaussian(ckks_ctx* ctx, const uint8_t* random, uint64_t* out, int idx_out, int idx_mod, int mod_num);
int ckks_sample_zo(ckks_ctx* ctx, const uint8_t* random, uint64_t* out, double probability, int idx_out, int idx_mod, int mod_num);
int ckks_sample_hwt(ckks_ctx* ctx, const uint8_t* random, uint64_t* out, int h, int idx_out, int idx_mod, int mod_num);
/* barrett_batch_3param_device, poly_add_3param_batch_device, poly_sub_3param_batch_device (poly_arithmetic.cuh:101-105, 423-427,
 * 481-485): c[idx_c + t] = a[idx_a + t] (*, +, -) b[idx_b + t] modulo prime idx_mod + t, t < mod_num; c may alias a or b
 * (which gives barrett_batch_device, poly_add_batch_device, poly_sub_batch_device and poly_sub2_batch_device, :37-41, 395-399, 467-478). */
int ckks_poly_mul(ckks_ctx* ctx, uint64_t* c, const uint64_t* a, const uint64_t* b, int idx_c, int idx_a, int idx_b, int idx_mod, int mod_num);
int ckks_poly_add(ckks_ctx* ctx, uint64_t* c, const uint64_t* a, const uint64_t* b, int idx_c, int idx_a, int idx_b, int idx_mod, int mod_num);
int ckks_poly_sub(ckks_ctx* ctx, uint64_t* c, const uint64_t* a, const uint64_t* b, int idx_c, int idx_a, int idx_b, int idx_mod, int mod_num);
/* SecretKey::SecretKey (SecretKey.cuh:18-31): sx = K+L+1 limbs over [P | Q], NTT domain, from 5*h random bytes */
int ckks_keygen_secret(ckks_ctx* ctx, uint64_t* sx, const uint8_t* random, int h);
/* Scheme_23::addEncKey (Scheme_23.cuh:54-80): pk = [a: L+1 limbs | b: L+1 limbs] = (a, e - a*s) over Q, NTT domain;
 * random_a: 8*N*(L+1) bytes, random_e: 4*N bytes */
int ckks_keygen_public(ckks_ctx* ctx, uint64_t* pk, const uint64_t* sx, const uint8_t* random_a, const uint8_t* random_e);
/* Scheme_23::encryptZero + encryptMsg (Scheme_23.cuh:82-112): cipher = [a: L+1 limbs | b: L+1 limbs], limbs 0..l written:
 * a = v*pk.a + e0, b = v*pk.b + e1 + m.  random: 9*N bytes = N (v) | 4*N (e0) | 4*N (e1), the reference's in_enc layout;
 * mx: plaintext limbs in the NTT domain, or NULL for encryptZero; scratch: (l+1)*N words (Scheme_23::vx_enc). */
int ckks_encrypt(ckks_ctx* ctx, uint64_t* cipher, const uint64_t* mx, const uint64_t* pk, const uint8_t* random, uint64_t* scratch, int l);
/* Scheme_23::decryptMsg (Scheme_23.cuh:114-127): mx = a*s + b on limbs 0..l, limbs l+1..L zeroed */
int ckks_decrypt(ckks_ctx* ctx, uint64_t* mx, const uint64_t* cipher, const uint64_t* sx, int l);
/* Context_23::encode_coeffs (Encoder.cuh:67-96): coefficient i = (long)(vals[i] * scale) modulo q_0..q_l, then NTT; vals: N device
 * doubles.  The reference stores q + data for negative data, which is the residue whenever |data| < q; the residue is taken here. */
int ckks_encode_coeffs(ckks_ctx* ctx, uint64_t* mx, const double* vals, long scale, int l);
/* Context_23::decode_coeffs (Encoder.cuh:113-186): iNTT of limbs 0..l (on a copy in scratch, (l+1)*N words), CRT of every
 * coefficient j*gap and N/2 + j*gap (gap = N/2/slots, j < slots) to the centred integer modulo q_0..q_l, as a double divided by
 * scale; other coefficients 0; is_bitrev writes to the bit-reversed index and multiplies by 256 (:171-173).  The reference does
 * the CRT on the host with NTL::ZZ; here it runs on the device (mixed-radix digits, multi-word Horner, correctly rounded
 * conversion), vals: N device doubles. */
int ckks_decode_coeffs(ckks_ctx* ctx, double* vals, const uint64_t* mx, uint64_t* scratch, double scale, int slots, int is_bitrev, int l);

/* ---- switching keys in the T basis and the operations built on the key switch ---- */
/* Context_23::rotGroups (Context_23.cuh:648-659): 5^idx mod 2N */
int ckks_rot_group(const ckks_ctx* ctx, long idx, uint64_t* value);
/* sk_and_poly_LeftRot_ntt_double / sk_and_poly_LeftRot_inv (poly_arithmetic.cuh:581-660): the NTT-domain slot permutation
 * out[j] = in[i] with 2*bitrev(j)+1 = pow * (2*bitrev(i)+1) mod 2N (the reference passes pow = rotGroups[N/2 - rot] or
 * rotGroups[rot]), on limbs idx_in.. -> idx_out..; in the coefficient domain this is X -> X^(pow^-1).  Not in place. */
int ckks_poly_automorph_ntt(ckks_ctx* ctx, uint64_t* out, const uint64_t* in, uint64_t pow, int idx_out, int idx_in, int mod_num);
/* sk_and_poly_conjugate (poly_arithmetic.cuh:666-680): out[i] = in[N-1-i], i.e. X -> X^-1.  Not in place. */
int ckks_poly_conjugate_ntt(ckks_ctx* ctx, uint64_t* out, const uint64_t* in, int idx_out, int idx_in, int mod_num);
/* the body shared by Scheme_23::addMultKey_23 / addConjKey_23 / addLeftRotKey_23 (KeySwitch_23.cuh:36-64, 85-113, 136-165):
 * swk (Key_decomp layout, [2][dnum][Ri_blockNum * t_num] limbs, NTT domain over T) switches from the secret s_from to the secret
 * s_to.  s_to: K+L+1 limbs over [P | Q]; s_from: L+1 limbs over Q (s^2 for the multiplication key, the reversed s for the
 * conjugation key, s itself for a rotation key whose s_to is the permuted s); both NTT domain.
 * random_a: dnum * 8*N*(K+L+1) bytes, random_e: dnum * 4*N bytes; scratch: (K+L+1)*N words. */
int ckks_keygen_switch_23(ckks_ctx* ctx, uint64_t* swk, const uint64_t* s_to, const uint64_t* s_from, const uint8_t* random_a,
                          const uint8_t* random_e, uint64_t* scratch);
/* Scheme_23::mult_23 (KeySwitch_23.cuh:192-236): out = c1 * c2 relinearised with rlk, limbs 0..l of [a: L+1 | b: L+1].
 * work: 3*(L+1)*N words (the reference's axbx1_mul, axax_mul, bxbx_mul); the other three as in ckks_keyswitch_23.
 * Level 0 or a null key: CKKS_E_STATE (std::invalid_argument in the reference, :194-201). */
int ckks_mult_23(ckks_ctx* ctx, uint64_t* out, const uint64_t* c1, const uint64_t* c2, const uint64_t* rlk, int l, uint64_t* work,
                 uint64_t* modUp_QjtoT_temp, uint64_t* exProduct_T_temp, uint64_t* modUp_TtoQj_buffer);
/* Scheme_23::leftRotate_23 (KeySwitch_23.cuh:556-586): out = cipher rotated left by rot slots (decrypts to m(X^(5^rot))).
 * work: 3*(L+1)*N words (a copy of a, and the reference's cipher_temp_pool).  out != cipher. */
int ckks_rotate_23(ckks_ctx* ctx, uint64_t* out, const uint64_t* cipher, const uint64_t* rotkey, long rot, int l, uint64_t* work,
                   uint64_t* modUp_QjtoT_temp, uint64_t* exProduct_T_temp, uint64_t* modUp_TtoQj_buffer);
/* Scheme_23::conjugate_23 (KeySwitch_23.cuh:433-468): decrypts to m(X^-1).  work: (L+1)*N words.  out != cipher. */
int ckks_conjugate_23(ckks_ctx* ctx, uint64_t* out, const uint64_t* cipher, const uint64_t* conjkey, int l, uint64_t* work,
                      uint64_t* modUp_QjtoT_temp, uint64_t* exProduct_T_temp, uint64_t* modUp_TtoQj_buffer);

/* ---- hoisted rotations of the slot <-> coefficient transforms (baby-step / giant-step in the T basis) ---- */
/* cipher_mul_P_batch as the transforms call it (poly_arithmetic.cuh:863-887; Bootstrapping_C2S_S2C_impl.cuh:270): cipher is a pair of
 * L+1 limbs (coefficient or NTT domain), out a pair of K+L+1 limbs over [P | Q]: special limbs zero, limb K+i = c_i * P mod q_i for
 * i <= l, limbs above l untouched. */
int ckks_cipher_mul_p(ckks_ctx* ctx, uint64_t* out, const uint64_t* cipher, int l);
/* cipher_add_T_batch_device (poly_arithmetic.cuh:143-153, 409-413): a += b on `blocks` groups of t_num limbs modulo the T primes. */
int ckks_cipher_add_t(ckks_ctx* ctx, uint64_t* a, const uint64_t* b, int blocks);
/* Scheme_23::rescaleAndEqual_noNTT (Scheme_23.cuh:321-337, 427-440): rescale of a coefficient-domain pair from level l to l-1 in
 * place; limb l is left as it is.  Level 0 is refused. */
int ckks_rescale_coeff(ckks_ctx* ctx, uint64_t* cipher, int l);
/* EncodingMatrix::Giant_Rotate_And_Mult_PlaintT (Bootstrapping_C2S_S2C_impl.cuh:7-152).  PQ_to_T = P * (a, b) in the T basis, NTT
 * domain, [a | b][Ri_blockNum][t_num] limbs; modUp_QjtoT = the digits of a in T, NTT domain, [digit][t_num]; rotKeys_host[j], j < gs:
 * device pointer to the rotation key of rotSlots_host[j] slots ([a | b][dnum][Ri_blockNum][t_num]) or NULL for "no rotation";
 * plaintextT_host[i * gs + j]: device pointer to t_num limbs of the plaintext (T basis, NTT domain) of baby step i < bs and
 * rotation j, read for j < accNum_host[i].  bs_cipher_T[i] = sum_j plaintext(i, j) * rot_j(cipher) as pairs
 * [bs][a | b][Ri_blockNum][t_num]; blocks at and above ceil((K+l+1)/gamma) are untouched.  The reference instantiates
 * (gs, bs) = (16, 4), (16, 2), (8, 2); here 1 <= gs <= 16, 1 <= bs <= 8.  All four tables are host arrays. */
int ckks_giant_rotate_mult_plain_t(ckks_ctx* ctx, uint64_t* bs_cipher_T, const uint64_t* PQ_to_T, const uint64_t* modUp_QjtoT,
                                   const uint64_t* const* rotKeys_host, const int* rotSlots_host, const uint64_t* const* plaintextT_host,
                                   const int* accNum_host, int bs, int gs, int l);
/* EncodingMatrix::Baby_Rotate (Bootstrapping_C2S_S2C_impl.cuh:154-228): output (a pair in T, NTT domain) += the pair `input`
 * rotated with each of the rotNum <= 16 keys given (NULL entries are skipped); modUp_QjtoT holds the digits of input's a part
 * after its ModDown.  output != input. */
int ckks_baby_rotate(ckks_ctx* ctx, uint64_t* output, const uint64_t* modUp_QjtoT, const uint64_t* input, int rotNum,
                     const uint64_t* const* rotKeys_host, const int* rotSlots_host, int l);
/* One level of EncodingMatrix::EvalCoeffsToSlots / EvalSlotsToCoeffs (Bootstrapping_C2S_S2C_impl.cuh:254-382, 531-625) up to, not
 * including, its rescale: cipher (pair of L+1 limbs, COEFFICIENT domain, level l) becomes, in place,
 * sum_{i<bs} rot_out[i]( sum_{j<accNum[i]} plaintext(i, j) * rot_in[j](cipher) ); a rotation by 0 slots needs no key, rot_out[0] is
 * not applied (as in the reference).  A missing key for a non-zero rotation returns CKKS_E_STATE.
 * scratch: ckks_bsgs_scratch_words(ctx, bs) words. */
int ckks_bsgs_scratch_words(const ckks_ctx* ctx, int bs, size_t* words);
int ckks_bsgs_level_23(ckks_ctx* ctx, uint64_t* cipher, int l, const uint64_t* const* plaintextT_host, const int* accNum_host,
                       const int* rot_in_host, const uint64_t* const* rot_in_keys_host, const int* rot_out_host,
                       const uint64_t* const* rot_out_keys_host, int bs, int gs, uint64_t* scratch);

/* ---- ring-packed PCMM ---- */
/* PCMM_Context::PCMM_Context (PCMM_Context.cuh:7-57) */
int pcmm_ctx_create(pcmm_ctx** out, ckks_ctx* ctx, int N1, int mlwe_rank, const uint64_t* p_ringpack, int p_count,
                    const uint64_t* q_ringpack, int q_count);
int pcmm_ctx_destroy(pcmm_ctx* h);
/* PCMM_Context::ToNTTInplace / FromNTTInplace (PCMM_Context.cuh:243-273; kernels smallntt_60bit.cuh:7-152): negacyclic transforms
 * of size N1 over the ring-pack primes, data = [mod_batch_size][mod_num][poly_num][N1], limb (z, j, y) modulo
 * pq_ringpack[start_mod_idx + j].  start_poly_idx is carried for the signature only (the reference's kernels ignore it).
 * The reference runs N1 = 256 only and silently does nothing otherwise; here every power of two N1 >= 2
 * runs (N1 < 256, such as the BERT layer's 128, through a wave-per-polynomial LDS kernel). */
int pcmm_ntt_fwd(pcmm_ctx* h, uint64_t* data, int poly_num, int mod_num, int start_poly_idx, int start_mod_idx, int mod_batch_size);
int pcmm_ntt_inv(pcmm_ctx* h, uint64_t* data, int poly_num, int mod_num, int start_poly_idx, int start_mod_idx, int mod_batch_size);
/* "N1", "mlwe_rank", and facts about the last PPMM call: "last_path" (1 = int8 MFMA kernel, 0 = generic 128-bit kernel),
 * "last_DW" / "last_DC" (base-256 digits of the plaintext matrix / of the residues), "last_slices" (three-digit slices the
 * plaintext matrix was cut into on the matrix cores, 1 = one launch), "last_absmax" (max |A|). */
int pcmm_info(const pcmm_ctx* h, const char* name, long* value);
/* the gather kernel of PCMM_Scheme::rlweCipherDecompose (PCMM_Scheme.cuh:50-88,115-119): rlwe = [a | b] with
 * L+1 limbs each, COEFFICIENT domain; mlwe_ptrs_host: mlwe_num device pointers, each [(l+1)][(rank+1)][N1]. */
int pcmm_rlwe_decompose(pcmm_ctx* h, const uint64_t* rlwe, uint64_t* const* mlwe_ptrs_host, int mlwe_num, int l);
/* PCMM_Scheme::rlweCipherDecompose (PCMM_Scheme.cuh:90-125): iNTT, gather, NTT back; rlwe in NTT domain. */
int pcmm_rlwe_decompose_ntt(pcmm_ctx* h, uint64_t* rlwe, uint64_t* const* mlwe_ptrs_host, int mlwe_num, int l);
/* PCMM_Scheme::mlweCipherPacking (PCMM_Scheme.cuh:361-425; kernels :262-340): packs mlwe_num MLWE ciphertexts (the rows PPMM
 * leaves behind: one modulus, [(rank+1)][N1] words each, coefficient domain, mlwe_num divides rank) into one RLWE ciphertext
 * rlwe_out = [a: L+1 limbs | b: L+1 limbs], of which limb 0 of both polynomials is written, NTT domain, level 0.
 * repacking_keys: rank keys over the primes [p0 | q0] (p0 = the context's last special prime = the ring-pack special prime,
 * q0 = the first ring-pack modulus), key i at keys + i*4*N = [a mod p0 | a mod q0 | b mod p0 | b mod q0], NTT domain
 * (PCMM_Scheme::addRepakcingKey, :152-224).  embed_scratch: (rank+1)*2*N words (PCMM_Scheme::embeded_mlwe_buffer, :12);
 * mult_scratch: 4*N words (the reference borrows Scheme_23::modUp_TtoQj_buffer, :394).
 * The reference's embedding is only meaningful for one special prime and two ring-pack moduli; other contexts get CKKS_E_INVALID. */
int pcmm_mlwe_pack(pcmm_ctx* h, uint64_t* rlwe_out, const uint64_t* const* mlwe_ptrs_host, int mlwe_num,
                   const uint64_t* repacking_keys, uint64_t* embed_scratch, uint64_t* mult_scratch);
/* PCMM_Scheme::convertMLWESKfromRLWESK (PCMM_Scheme.cuh:23-48; ringDown_kernel, ringSwitch.cuh:7-19): mlwe_sk =
 * [p_count + q_count moduli][rank][N1], small polynomial i = the coefficients i + n*rank of the RLWE secret, NTT domain (size N1).
 * rlwe_sk (K+L+1 limbs, NTT domain) is transformed back and forth in place as in the reference and ends unchanged.
 * The two copies of the reference are kept as they are: RLWE limbs 0.. to key moduli 0.., then RLWE limbs K.. to key moduli
 * p_count.. (so modulus slot 0 holds the secret modulo the FIRST special prime; nothing reads it).  N1 a multiple of 64. */
int pcmm_convert_mlwe_sk(pcmm_ctx* h, uint64_t* mlwe_sk, uint64_t* rlwe_sk);
/* PCMM_Scheme::addRepakcingKey (PCMM_Scheme.cuh:126-224): rank keys over the context primes [last p_count special primes |
 * q_0 .. q_{q_count-2}], key i at keys + i*2*m*N = [a: m limbs | b: m limbs], m = p_count + q_count - 1, NTT domain,
 * b = -a*s + p0 * iota(s_i) + e - the layout pcmm_mlwe_pack reads.  Randomness: key i draws 4*N bytes (e) then 8*N*m bytes (a)
 * from the Salsa20 stream of (key32, nonce + i).  scratch: (m + 1)*N words.  mlwe_sk is taken to the coefficient domain and
 * back on ALL its moduli (the reference brings back all but the last, :182).  b starts from zero (the reference writes the
 * embedded secret into fresh cudaMalloc memory).  N1 a multiple of 64. */
int pcmm_add_repacking_key(pcmm_ctx* h, uint64_t* keys, uint64_t* mlwe_sk, const uint64_t* rlwe_sk, const uint8_t* key32, uint64_t nonce,
                           uint64_t* scratch);
/* PCMM_Scheme::mlweDecrypt (PCMM_Scheme.cuh:531-576): plain[mod][n] = b + sum_i a_i * s_i for moduli 0..l of the sample, in the
 * size-N1 NTT domain (where the reference leaves it); the sample is transformed in place and back.  Any rank (the reference
 * instantiates 256 and 512).  N1 a multiple of 64. */
int pcmm_mlwe_decrypt(pcmm_ctx* h, uint64_t* plain, uint64_t* mlwe_cipher, const uint64_t* mlwe_sk, int l);
/* PCMM_Context::decodeCoeffs (PCMM_Context.cuh:149-178): inverse transform of a copy (scratch: (l+1)*N1 words), then the centred
 * residue modulo the first ring-pack modulus divided by scaler; vals: N1 device doubles. */
int pcmm_decode_coeffs(pcmm_ctx* h, double* vals, const uint64_t* plain, uint64_t* scratch, long long scaler, int l);
/* PCMM_Scheme::PPMM device part (PPMM_kernel.cuh:93-252, launch :294-340):
 * out[m][mod][c] = fused-rescaled sum_n trunc(W[m][n]*scaler) * mlwe[n][mod][c] mod q_mod, for mod_num ring-pack
 * primes (the reference fixes mod_num = 2), c < (rank+1)*N1.  W: device fp32 row-major [M][Kin];
 * mlwe_ptrs_host: Kin device pointers; out: device [M][mod_num][(rank+1)*N1].
 * Runs on the int8 matrix cores when (rank+1)*N1 is a multiple of 64, the rows are 16-byte aligned and the operands fit balanced
 * base-256 digits: residues in 5 digits (primes up to 0x7f7f7f7f80, i.e. the 36-bit sets) or in 7 digits (primes below 2^50, i.e.
 * the reference's own 49-bit ring-pack primes), and |trunc(W*scaler)| below the smallest prime.  One launch takes a plaintext
 * matrix of up to 4 digits (3 with the 7-digit residues); wider ones, such as the 46-bit entries that the reference's scaler
 * q1 * 2^49 / scale gives, run as two or three launches over slices of three digits and a combining pass, with the same result.
 * Anything else takes a one-output-per-lane kernel with 128-bit accumulation (pcmm_info "last_path" tells which ran). */
int pcmm_ppmm(pcmm_ctx* h, const float* W_dev, const uint64_t* const* mlwe_ptrs_host, uint64_t* out_dev, int M,
              int Kin, int mod_num, double scaler);
/* same contraction with the MLWE operands in one contiguous device array [Kin][mod_num][(rank+1)*N1] */
int pcmm_ppmm_strided(pcmm_ctx* h, const float* W_dev, const uint64_t* mlwe_dev, uint64_t* out_dev, int M, int Kin,
                      int mod_num, double scaler);
/* Prepared plaintext matrices (no counterpart in the reference, which quantises W inside every call, PPMM_kernel.cuh:148).
 * By default every PPMM call reads W afresh, as the reference does: it quantises the matrix, measures |A|max (one stream
 * synchronisation) and splits it into digit planes in work space of the handle, so a call always multiplies by what W_dev
 * holds when it is made, whoever wrote it.
 * pcmm_weights_static(h, W_dev, bytes, 1) declares the device memory [W_dev, W_dev + bytes) static: the caller's promise that a
 * weight matrix in it changes only through this library's own copies (ckks_memcpy_h2d / _d2d, ckks_memset, ckks_free - the last
 * also ends the declaration) or is announced with pcmm_weights_changed(h, W_dev) (W_dev = NULL: every matrix).
 * pcmm_set_weight_cache(h, 1) makes the same promise for every matrix the handle is given.  The planes of a static
 * (W_dev, M, Kin, scaler) are kept after the first call (at most 4 GiB per handle, least recently used first out) and later
 * calls with the same four values enqueue their kernels and return without waiting for the stream.  A writer the library does
 * not see (the caller's own kernel, hipMemcpy, an allocator that hands the same address to another matrix) makes such a call
 * multiply by the OLD weights: that is why nothing is kept unless the caller asks for it.
 * pcmm_weights_static(.., 0) and pcmm_set_weight_cache(h, 0) take the promise back and drop what was kept under it. */
int pcmm_weights_static(pcmm_ctx* h, const float* W_dev, size_t bytes, int is_static);
int pcmm_set_weight_cache(pcmm_ctx* h, int enabled);
/* Test / tuning switches of a ring-pack handle, by name (value 0 = off, the default; results do not depend on them):
 * "gather_plain" (rlweCipherDecompose with the one-lane-per-word gather), "ppmm_generic" (PPMM on the generic 128-bit kernel),
 * "ppmm_no_tail" (PPMM runs the remainder column panels whole instead of as jobs by prime). */
int pcmm_set_option(pcmm_ctx* h, const char* name, long value);
int pcmm_weights_changed(pcmm_ctx* h, const float* W_dev);

/* ---- the gather writing PPMM's operand directly.  No counterpart in the reference, where rlweCipherDecompose materialises every
 * MLWE sample as 8-byte words that PPMM reads back (PCMM_Scheme.cuh:90-125, PPMM_kernel.cuh:254-349); in a layer the two always
 * follow each other (Bert.cuh:411-424), so the samples can go straight into the int8 digit planes the MFMA kernel reads
 * (5 bytes per residue).  Results are bit-identical to pcmm_rlwe_decompose_ntt followed by pcmm_ppmm.
 *   pcmm_packed_begin(h, Kin, mod_num)      opens the planes for Kin samples (a multiple of 64) over mod_num moduli
 *   pcmm_rlwe_decompose_packed(...)         the first `take` of the mlwe_num samples that rlweCipherDecompose extracts from one RLWE
 *                                           ciphertext (mlwe_num divides the rank; level l = mod_num - 1; NTT domain, restored) become
 *                                           samples sample_offset .. sample_offset + take - 1 (take, sample_offset: multiples of 64)
 *   pcmm_ppmm_packed(h, W, out, M, scaler)  the contraction over the Kin samples; out as pcmm_ppmm
 * A call of pcmm_ppmm / pcmm_ppmm_strided reuses the same work space and closes the planes (CKKS_E_STATE afterwards). ---- */
int pcmm_packed_begin(pcmm_ctx* h, int Kin, int mod_num);
int pcmm_rlwe_decompose_packed(pcmm_ctx* h, uint64_t* rlwe, int sample_offset, int mlwe_num, int take, int l);
int pcmm_ppmm_packed(pcmm_ctx* h, const float* W_dev, uint64_t* out_dev, int M, double scaler);

#ifdef __cplusplus
}
#endif
#endif /* CKKS_HIP_H */
