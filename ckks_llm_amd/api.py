"""Host-side mirror of the reference's interface for the hot path (names, argument order and error behaviour of
Context_23 / PCMM_Context / PCMM_Scheme), calling the HIP library through its C ABI.

Polynomial arguments are DeviceBuffer objects or raw device addresses (ints, e.g. torch.Tensor.data_ptr()).
"""
import os
import ctypes as C

import numpy as np

from ._lib import load_library, u64p, vp


class CkksError(RuntimeError):
    pass


def _check(rc, what):
    if rc != 0:
        msg = load_library().ckks_last_error().decode()
        if rc == -4:
            raise ValueError(msg or what)          # std::invalid_argument of the reference (KeySwitch_23.cuh:194-201)
        raise CkksError("%s failed (%d): %s" % (what, rc, msg))


def _addr(x):
    if isinstance(x, DeviceBuffer):
        return x.ptr
    if hasattr(x, "data_ptr"):
        return x.data_ptr()
    return int(x)


def _arr(v):
    return np.ascontiguousarray(np.array(list(v), dtype=np.uint64))


class DeviceBuffer:
    """Owns one device allocation (the cudaMalloc'd member of Ciphertext / Plaintext / Key_decomp / MLWECiphertext,
    Ciphertext.cuh:26-31,88-99)."""

    def __init__(self, nbytes):
        self.L_ = load_library()
        self.nbytes = int(nbytes)
        p = vp()
        _check(self.L_.ckks_malloc(C.byref(p), max(self.nbytes, 8)), "ckks_malloc")
        self.ptr = p.value

    @classmethod
    def from_numpy(cls, a):
        a = np.ascontiguousarray(a)
        b = cls(a.nbytes)
        b.upload(a)
        return b

    def upload(self, a):
        a = np.ascontiguousarray(a)
        assert a.nbytes <= self.nbytes
        _check(self.L_.ckks_memcpy_h2d(self.ptr, a.ctypes.data, a.nbytes), "ckks_memcpy_h2d")

    def download(self, dtype=np.uint64, count=None, offset_bytes=0):
        item = np.dtype(dtype).itemsize
        if count is None:
            count = (self.nbytes - offset_bytes) // item
        out = np.empty(count, dtype=dtype)
        _check(self.L_.ckks_memcpy_d2h(out.ctypes.data, self.ptr + offset_bytes, out.nbytes), "ckks_memcpy_d2h")
        return out

    def zero(self):
        _check(self.L_.ckks_memset(self.ptr, 0, self.nbytes), "ckks_memset")

    def free(self):
        if self.ptr:
            self.L_.ckks_sync()
            self.L_.ckks_free(self.ptr)
            self.ptr = 0

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Context_23:
    """Context_23 (Context_23.h:19-279) for the hot path.  `Context_23(logN, p, q, t, gamma)` takes explicit prime lists;
    `Context_23(logN, logslots, h=64, sigma=3.2)` is the reference's own constructor (Context_23.h:21), which selects the
    parameter set compiled in for logN = 13..16 (Params.cuh:11-170) and accepts a secret Hamming weight of 64 or 192 only."""

    def __init__(self, logN, p, q=None, t=(), gamma=0):
        self.logslots, self.h_weight, self.sigma, self.precision = logN - 1, 64, 3.2, 0
        if isinstance(p, int):                                               # (logN, logslots, h, sigma)
            from .params import REF_PARAMS
            self.logslots = p
            self.h_weight = 64 if q is None else q
            self.sigma = 3.2 if isinstance(t, tuple) else t
            if self.h_weight not in (64, 192):
                raise ValueError("hamming weight error!")                    # Params.cuh:228
            if logN not in REF_PARAMS:
                raise ValueError("Context_23: the reference holds parameter sets for logN = 13, 14, 15 and 16 only")
            r = REF_PARAMS[logN]
            p, q, t, gamma = r["p"], r["q"], r["t"], r["gamma"]
            self.precision = 1 << 36 if logN < 15 else 1 << 49               # Params.cuh:15, 36, 58, 85
        self.slots = 1 << self.logslots
        self.L_ = load_library()
        self.logN, self.N = logN, 1 << logN
        self.pVec, self.qVec, self.tVec = list(p), list(q), list(t)
        self.p_num, self.q_num, self.t_num, self.gamma = len(self.pVec), len(self.qVec), len(self.tVec), gamma
        self.K, self.L = self.p_num, self.q_num - 1
        pa, qa, ta = _arr(p), _arr(q), _arr(t)
        h = vp()
        _check(self.L_.ckks_ctx_create(C.byref(h), logN, pa.ctypes.data_as(u64p), len(pa), qa.ctypes.data_as(u64p), len(qa),
                                       ta.ctypes.data_as(u64p), len(ta), gamma), "ckks_ctx_create")
        self.h = h.value
        self.dnum = self.info("dnum")
        self.Ri_blockNum = self.info("Ri_blockNum")
        self.Qj_blockNum = self.info("Qj_blockNum")

    def __del__(self):
        try:
            if self.h:
                self.L_.ckks_ctx_destroy(self.h)
                self.h = None
        except Exception:
            pass

    def info(self, name):
        v = C.c_long()
        _check(self.L_.ckks_ctx_info(self.h, name.encode(), C.byref(v)), "ckks_ctx_info")
        return v.value

    def table(self, name):
        n = C.c_size_t()
        _check(self.L_.ckks_ctx_table(self.h, name.encode(), None, 0, C.byref(n)), "ckks_ctx_table")
        out = np.zeros(n.value, dtype=np.uint64)
        _check(self.L_.ckks_ctx_table(self.h, name.encode(), out.ctypes.data_as(u64p), n.value, None), "ckks_ctx_table")
        return out

    def set_arith_mode(self, mode):
        _check(self.L_.ckks_ctx_set_arith_mode(self.h, mode), "ckks_ctx_set_arith_mode")

    def set_ntt_mode(self, mode):
        """0: automatic, 1: two launches per transform (data in place between them), 2: chained one-launch transform
        (N >= 2^15), 3: one workgroup per limb (N >= 2^15), 4: paired one-launch transform (N = 2^16; what mode 0 takes for
        batches of up to 128 limbs), 5: as 4 with a limb's tiles spread over all XCDs (mode 0 above 40 limbs).  All give the same residues."""
        _check(self.L_.ckks_ctx_set_ntt_mode(self.h, mode), "ckks_ctx_set_ntt_mode")

    def set_option(self, name, value=1):
        """Test / tuning switch by name: ks_split, ks_back_split, conv_int, ntt_no_reverse, ntt_chunk (see ckks_hip.h)."""
        _check(self.L_.ckks_ctx_set_option(self.h, name.encode(), int(value)), "ckks_ctx_set_option")

    def set_ntt_chain(self, skew=0, spin_max=-1):
        """Tuning / test hook of the chained transform (ntt_mode 2); spin_max = 0 sends every second-pass tile to the finishing launch."""
        _check(self.L_.ckks_ctx_set_ntt_chain(self.h, skew, spin_max), "ckks_ctx_set_ntt_chain")

    def check(self):
        """Synchronise the context's stream; raises if HIP reports an error for the launches so far."""
        _check(self.L_.ckks_ctx_check(self.h), "ckks_ctx_check")

    def set_stream(self, stream_handle):
        _check(self.L_.ckks_set_stream(self.h, stream_handle), "ckks_set_stream")

    def sync(self):
        _check(self.L_.ckks_sync(), "ckks_sync")

    def timer_mark(self, slot):
        """Record mark `slot` (0 .. 4095) on the context's stream; returns at once."""
        _check(self.L_.ckks_timer_mark(self.h, slot), "ckks_timer_mark")

    def timer_between(self, slot_a, slot_b):
        """Milliseconds from mark slot_a to mark slot_b (waits for slot_b)."""
        ms = C.c_float()
        _check(self.L_.ckks_timer_between(self.h, slot_a, slot_b, C.byref(ms)), "ckks_timer_between")
        return ms.value

    def timer_start(self):
        _check(self.L_.ckks_timer_start(self.h), "ckks_timer_start")

    def timer_stop(self):
        ms = C.c_float()
        _check(self.L_.ckks_timer_stop(self.h, C.byref(ms)), "ckks_timer_stop")
        return ms.value

    # -- Context_23.h:42-45
    def ToNTTInplace(self, device_a, start_poly_idx, start_mod_idx, poly_num, mod_num, poly_mod_len):
        _check(self.L_.ckks_ntt_fwd(self.h, _addr(device_a), start_poly_idx, start_mod_idx, poly_num, mod_num, poly_mod_len), "ckks_ntt_fwd")

    def FromNTTInplace(self, device_a, start_poly_idx, start_mod_idx, poly_num, mod_num, poly_mod_len):
        _check(self.L_.ckks_ntt_inv(self.h, _addr(device_a), start_poly_idx, start_mod_idx, poly_num, mod_num, poly_mod_len), "ckks_ntt_inv")

    def ntt_noalloc(self, device_a, start_poly_idx, start_mod_idx, poly_num, mod_num, poly_mod_len, inverse):
        """ToNTTInplace / FromNTTInplace without any device allocation (fixed inter-pass area inside the library;
        at most ntt_noalloc_max_limbs() limbs per call)."""
        _check(self.L_.ckks_ntt_noalloc(self.h, _addr(device_a), start_poly_idx, start_mod_idx, poly_num, mod_num, poly_mod_len,
                                        1 if inverse else 0), "ckks_ntt_noalloc")

    def ntt_noalloc_max_limbs(self):
        return int(self.L_.ckks_ntt_noalloc_max_limbs())

    def ntt_timed(self, device_a, start_poly_idx, start_mod_idx, poly_num, mod_num, poly_mod_len, inverse):
        """One transform; returns the HIP-event durations (ms) of its two kernel launches."""
        a, b = C.c_float(), C.c_float()
        _check(self.L_.ckks_ntt_timed(self.h, _addr(device_a), start_poly_idx, start_mod_idx, poly_num, mod_num, poly_mod_len,
                                      1 if inverse else 0, C.byref(a), C.byref(b)), "ckks_ntt_timed")
        return a.value, b.value

    def ToNTTInplace_for_externalProduct(self, device_a, start_poly_idx, start_mod_idx, poly_num, mod_num, poly_mod_len,
                                         cipher_mod_num, batch_size):
        _check(self.L_.ckks_ntt_fwd_ext(self.h, _addr(device_a), start_poly_idx, start_mod_idx, poly_num, mod_num, poly_mod_len,
                                        cipher_mod_num, batch_size), "ckks_ntt_fwd_ext")

    def FromNTTInplace_for_externalProduct(self, device_a, start_poly_idx, start_mod_idx, poly_num, mod_num, poly_mod_len,
                                           cipher_mod_num, batch_size):
        _check(self.L_.ckks_ntt_inv_ext(self.h, _addr(device_a), start_poly_idx, start_mod_idx, poly_num, mod_num, poly_mod_len,
                                        cipher_mod_num, batch_size), "ckks_ntt_inv_ext")

    # -- Context_23.h:54-61
    def modUpPQtoT_23(self, output, input, l, batch_size):
        _check(self.L_.ckks_modup_pq_to_t(self.h, _addr(output), _addr(input), l, batch_size), "ckks_modup_pq_to_t")

    def modUpQjtoT_23(self, output, input, l, batch_size):
        _check(self.L_.ckks_modup_qj_to_t(self.h, _addr(output), _addr(input), l, batch_size), "ckks_modup_qj_to_t")

    def modUpTtoPQl_23(self, modUp_TtoQj_buffer, exProduct_T_temp, l, batch_size):
        _check(self.L_.ckks_modup_t_to_pql(self.h, _addr(modUp_TtoQj_buffer), _addr(exProduct_T_temp), l, batch_size), "ckks_modup_t_to_pql")

    def modDownPQltoQl_23(self, output, modUp_TtoQj_buffer, l, batch_size):
        _check(self.L_.ckks_moddown_pql_to_ql(self.h, _addr(output), _addr(modUp_TtoQj_buffer), l, batch_size), "ckks_moddown_pql_to_ql")

    def external_product_T(self, output, cipher_modUp_QjtoT, swk_modUp_RitoT, l):
        _check(self.L_.ckks_external_product_t(self.h, _addr(output), _addr(cipher_modUp_QjtoT), _addr(swk_modUp_RitoT), l), "ckks_external_product_t")

    def external_product_T_swk_reuse(self, output, cipher_modUp_QjtoT, swk_modUp_RitoT, l, batch_size):
        """Context_23.h:62, ExternalProduct.cuh:151-162: one key against batch_size digit sets."""
        _check(self.L_.ckks_external_product_t_swk_reuse(self.h, _addr(output), _addr(cipher_modUp_QjtoT), _addr(swk_modUp_RitoT), l, batch_size),
               "ckks_external_product_t_swk_reuse")

    def rescaleAndEqual(self, cipher, scratch, l):
        _check(self.L_.ckks_rescale(self.h, _addr(cipher), _addr(scratch), l), "ckks_rescale")

    def keyswitch_23(self, out, d2, swk, l, modUp_QjtoT_temp, exProduct_T_temp, modUp_TtoQj_buffer):
        _check(self.L_.ckks_keyswitch_23(self.h, _addr(out), _addr(d2), _addr(swk), l, _addr(modUp_QjtoT_temp),
                                         _addr(exProduct_T_temp), _addr(modUp_TtoQj_buffer)), "ckks_keyswitch_23")

    # -- textbook hybrid key switch (no reference counterpart)
    def hybrid_modup(self, digits, in_coeff, l):
        _check(self.L_.ckks_hybrid_modup(self.h, _addr(digits), _addr(in_coeff), l), "ckks_hybrid_modup")

    def hybrid_inner_product(self, ip, digits_ntt, evk, l):
        _check(self.L_.ckks_hybrid_inner_product(self.h, _addr(ip), _addr(digits_ntt), _addr(evk), l), "ckks_hybrid_inner_product")

    def hybrid_moddown(self, out, in_pq, l):
        _check(self.L_.ckks_hybrid_moddown(self.h, _addr(out), _addr(in_pq), l), "ckks_hybrid_moddown")

    def hybrid_keyswitch(self, out, in_ntt, evk, l, scratch):
        _check(self.L_.ckks_hybrid_keyswitch(self.h, _addr(out), _addr(in_ntt), _addr(evk), l, _addr(scratch)), "ckks_hybrid_keyswitch")


    # -- RNG::generateRandom_device (RNG.cuh:18), Sampler (Sampler.cuh:17-41), pointwise arithmetic (poly_arithmetic.cuh)
    def generateRandom_device(self, a, n, key, nonce):
        """n bytes of the Salsa20/20 stream of (32-byte key, 64-bit nonce).  The reference draws key and nonce from rand();
        here the caller names them, so a run can be repeated."""
        key = bytes(key)
        if len(key) != 32:
            raise ValueError("generateRandom_device: the key has 32 bytes")
        _check(self.L_.ckks_random_bytes(self.h, _addr(a), n, key, nonce), "ckks_random_bytes")

    def uniformSampler_xq(self, random, out, idx_out, idx_mod, mod_num):
        _check(self.L_.ckks_sample_uniform(self.h, _addr(random), _addr(out), idx_out, idx_mod, mod_num), "ckks_sample_uniform")

    def gaussianSampler_xq(self, random, out, idx_out, idx_mod, mod_num):
        _check(self.L_.ckks_sample_gaussian(self.h, _addr(random), _addr(out), idx_out, idx_mod, mod_num), "ckks_sample_gaussian")

    def ZOSampler(self, random, out, probability, idx_out, idx_mod, mod_num):
        _check(self.L_.ckks_sample_zo(self.h, _addr(random), _addr(out), probability, idx_out, idx_mod, mod_num), "ckks_sample_zo")

    def HWTSampler(self, random, out, h, idx_out, idx_mod, mod_num):
        _check(self.L_.ckks_sample_hwt(self.h, _addr(random), _addr(out), h, idx_out, idx_mod, mod_num), "ckks_sample_hwt")

    def barrett_batch_3param_device(self, c, a, b, idx_c, idx_a, idx_b, idx_mod, mod_num):
        _check(self.L_.ckks_poly_mul(self.h, _addr(c), _addr(a), _addr(b), idx_c, idx_a, idx_b, idx_mod, mod_num), "ckks_poly_mul")

    def poly_add_3param_batch_device(self, c, a, b, idx_c, idx_a, idx_b, idx_mod, mod_num):
        _check(self.L_.ckks_poly_add(self.h, _addr(c), _addr(a), _addr(b), idx_c, idx_a, idx_b, idx_mod, mod_num), "ckks_poly_add")

    def poly_sub_3param_batch_device(self, c, a, b, idx_c, idx_a, idx_b, idx_mod, mod_num):
        _check(self.L_.ckks_poly_sub(self.h, _addr(c), _addr(a), _addr(b), idx_c, idx_a, idx_b, idx_mod, mod_num), "ckks_poly_sub")

    # -- rotGroups (Context_23.cuh:648-659) and the NTT-domain permutations (poly_arithmetic.cuh:581-680)
    def rotGroups(self, idx):
        v = C.c_uint64()
        _check(self.L_.ckks_rot_group(self.h, idx, C.byref(v)), "ckks_rot_group")
        return v.value

    def sk_and_poly_LeftRot_ntt(self, device_a, device_b, rot_num, idx_a, idx_b, mod_num):
        """a[perm(i)] = b[i] with the exponent rotGroups[N/2 - rot_num] (poly_arithmetic.cuh:581-596): X -> X^(5^rot_num)."""
        _check(self.L_.ckks_poly_automorph_ntt(self.h, _addr(device_a), _addr(device_b), self.rotGroups(self.N // 2 - rot_num),
                                               idx_a, idx_b, mod_num), "ckks_poly_automorph_ntt")

    def sk_and_poly_LeftRot_inv(self, device_a, device_b, rot_num, idx_a, idx_b, mod_num):
        """The same with the exponent rotGroups[rot_num] (poly_arithmetic.cuh:639-660): X -> X^(5^-rot_num)."""
        _check(self.L_.ckks_poly_automorph_ntt(self.h, _addr(device_a), _addr(device_b), self.rotGroups(rot_num), idx_a, idx_b, mod_num),
               "ckks_poly_automorph_ntt")

    def sk_and_poly_conjugate(self, device_a, device_b, idx_a, idx_b, mod_num):
        _check(self.L_.ckks_poly_conjugate_ntt(self.h, _addr(device_a), _addr(device_b), idx_a, idx_b, mod_num), "ckks_poly_conjugate_ntt")

    # -- Context_23::encode_coeffs / decode_coeffs (Encoder.cuh:83-96, 113-186)
    def encode_coeffs(self, vals, msg):
        """vals: N device doubles; msg: Plaintext (level msg.l, integer scale msg.scale)."""
        _check(self.L_.ckks_encode_coeffs(self.h, _addr(msg.mx_device), _addr(vals), int(msg.scale), msg.l), "ckks_encode_coeffs")

    def decode_coeffs(self, msg, vals, is_bitRev=False):
        """vals: N device doubles (written)."""
        scratch = DeviceBuffer(8 * self.N * (msg.l + 1))
        _check(self.L_.ckks_decode_coeffs(self.h, _addr(vals), _addr(msg.mx_device), scratch.ptr, float(msg.scale), msg.slots,
                                          1 if is_bitRev else 0, msg.l), "ckks_decode_coeffs")
        scratch.free()


class Plaintext:
    """Plaintext (Plaintext.cuh:6-76): one device buffer of L+1 limbs, level l, slots, scale."""

    def __init__(self, N, L, l, slots, scale):
        if l > L:
            raise ValueError("new Plaintext error!")
        self.N, self.L, self.l, self.slots, self.scale = N, L, l, slots, scale
        self.mx_device = DeviceBuffer(8 * N * (L + 1))


class Ciphertext:
    """Ciphertext (Ciphertext.cuh:6-99): one device buffer [a: L+1 limbs | b: L+1 limbs]."""

    def __init__(self, N, L, l, slots, scale):
        self.N, self.L, self.l, self.slots, self.scale = N, L, l, slots, scale
        self.cipher_device = DeviceBuffer(8 * N * (L + 1) * 2)
        self.ax_device = self.cipher_device.ptr
        self.bx_device = self.cipher_device.ptr + 8 * N * (L + 1)


class SecretKey:
    """SecretKey (SecretKey.cuh:9-31): sparse ternary secret of Hamming weight <= h over [P | Q], NTT domain, sampled from
    5*h bytes of the context's stream under (key, nonce).  h = None takes the context's Hamming weight, as the reference's
    SecretKey(context) does (SecretKey.cuh:20-29).  key = None (the default) draws 32 bytes from the operating system, so two
    processes never share a secret; a fixed key is for runs that must repeat (the parity tests)."""

    def __init__(self, context, h=None, key=None, nonce=0):
        key = os.urandom(32) if key is None else bytes(key)
        if h is None:
            h = context.h_weight
        self.N, self.L, self.K = context.N, context.L, context.K
        self.sx_device = DeviceBuffer(8 * self.N * (self.K + self.L + 1))
        rnd = DeviceBuffer(5 * h + 64)
        context.generateRandom_device(rnd, 5 * h, key, nonce)
        _check(context.L_.ckks_keygen_secret(context.h, self.sx_device.ptr, rnd.ptr, h), "ckks_keygen_secret")
        rnd.free()


class Key:
    """Key (Key.cuh:5-24): [a | b], (L+1+K)*dnum limbs each."""

    def __init__(self, N, L, K, dnum):
        self.N, self.L, self.K, self.dnum = N, L, K, dnum
        self.cipher_device = DeviceBuffer(8 * N * (L + 1 + K) * dnum * 2)
        self.ax_device = self.cipher_device.ptr
        self.bx_device = self.cipher_device.ptr + 8 * N * (L + 1 + K) * dnum


class Key_decomp:
    """Key_decomp (Key_decomp.cuh:5-24): a switching key in the T basis, [a | b] with dnum * Ri_blockNum * t_num limbs each."""

    def __init__(self, N, dnum, t_num, Ri_blockNum):
        self.N, self.dnum, self.t_num, self.Ri_blockNum = N, dnum, t_num, Ri_blockNum
        self.cipher_device = DeviceBuffer(8 * N * dnum * t_num * Ri_blockNum * 2)
        self.ax_device = self.cipher_device.ptr
        self.bx_device = self.cipher_device.ptr + 8 * N * dnum * t_num * Ri_blockNum


class Scheme_23:
    """The members of Scheme_23 on this path (Scheme_23.h:113-182): addEncKey, encryptZero, encryptMsg, decryptMsg,
    rescaleAndEqual, addMultKey_23, addConjKey_23, addLeftRotKey_23, mult_23, leftRotate_23, conjugate_23.
    Randomness is the context's Salsa20 stream under this object's key with a nonce that counts calls; key = None (the
    default) draws the key from the operating system, a fixed key makes a run repeatable."""

    def __init__(self, context, key=None):
        self.context = context
        self.key = os.urandom(32) if key is None else bytes(key)
        self.nonce = 1
        N, L = context.N, context.L
        self.publicKey = None
        self.in_enc = DeviceBuffer(9 * N)                                   # Scheme_23.cuh:38-39
        self.vx_enc = DeviceBuffer(8 * N * (L + 1))
        self.rescale_buffer = DeviceBuffer(8 * N * (L + 1) * 2)
        self.rlk_23 = None
        self.ConjKey_23 = None
        self.rotKey_vec_23 = {}
        if context.t_num:                                                   # Scheme_23::mallocMemory (Scheme_23.cuh:7-51)
            T, RB, K = context.t_num, context.Ri_blockNum, context.K
            self.sxsx = DeviceBuffer(8 * N * (K + L + 1))
            self.temp_mul = DeviceBuffer(8 * N * (K + L + 1))
            self.mul_work = DeviceBuffer(8 * N * (L + 1) * 3)               # axbx1_mul, axax_mul, bxbx_mul
            self.modUp_QjtoT_temp = DeviceBuffer(8 * N * T * context.Qj_blockNum)
            self.exProduct_T_temp = DeviceBuffer(8 * N * T * RB * 2)
            self.modUp_TtoQj_buffer = DeviceBuffer(8 * N * T * RB * 2)

    def _switch_key(self, s_to, s_from):
        c = self.context
        N, KL = c.N, c.K + c.L + 1
        key = Key_decomp(N, c.dnum, c.t_num, c.Ri_blockNum)
        na, ne = c.dnum * 8 * N * KL, c.dnum * 4 * N
        rnd = DeviceBuffer(na + ne)                                         # KeySwitch_23.cuh:36-37
        c.generateRandom_device(rnd, na + ne, self.key, self._next_nonce())
        _check(c.L_.ckks_keygen_switch_23(c.h, key.cipher_device.ptr, _addr(s_to), _addr(s_from), rnd.ptr, rnd.ptr + na,
                                          self.temp_mul.ptr), "ckks_keygen_switch_23")
        rnd.free()
        return key

    def addMultKey_23(self, secretKey):
        """KeySwitch_23.cuh:21-65: the key that switches s^2 to s."""
        if self.rlk_23 is not None:
            return
        c = self.context
        c.barrett_batch_3param_device(self.sxsx, secretKey.sx_device, secretKey.sx_device, 0, c.K, c.K, c.K, c.L + 1)
        self.rlk_23 = self._switch_key(secretKey.sx_device, self.sxsx)

    def addConjKey_23(self, secretKey):
        """KeySwitch_23.cuh:69-114: the key that switches the reversed secret to s."""
        if self.ConjKey_23 is not None:
            return
        c = self.context
        c.sk_and_poly_conjugate(self.sxsx, secretKey.sx_device, 0, c.K, c.L + 1)
        self.ConjKey_23 = self._switch_key(secretKey.sx_device, self.sxsx)

    def addLeftRotKey_23(self, secretKey, rot_num):
        """KeySwitch_23.cuh:119-165: the key that switches s to s(X^(5^-rot_num))."""
        if rot_num in self.rotKey_vec_23:
            return
        c = self.context
        c.sk_and_poly_LeftRot_inv(self.sxsx, secretKey.sx_device, rot_num, 0, 0, c.K + c.L + 1)
        self.rotKey_vec_23[rot_num] = self._switch_key(self.sxsx, secretKey.sx_device.ptr + 8 * c.N * c.K)

    def _ks_buffers(self):
        return self.mul_work.ptr, self.modUp_QjtoT_temp.ptr, self.exProduct_T_temp.ptr, self.modUp_TtoQj_buffer.ptr

    def mult_23(self, cipher_res, cipher1, cipher2):
        """KeySwitch_23.cuh:192-236; level 0 or a missing key raise ValueError (std::invalid_argument there)."""
        c = self.context
        l = min(cipher1.l, cipher2.l)
        key = self.rlk_23.cipher_device.ptr if self.rlk_23 is not None else None
        if l != 0 and key is None:
            raise ValueError("rotKey_23 not exists")
        _check(c.L_.ckks_mult_23(c.h, cipher_res.cipher_device.ptr, cipher1.cipher_device.ptr, cipher2.cipher_device.ptr, key, l,
                                 *self._ks_buffers()), "ckks_mult_23")
        cipher_res.l, cipher_res.scale = l, cipher1.scale * cipher2.scale

    def leftRotate_23(self, cipher_res, cipher, rotSlots):
        """KeySwitch_23.cuh:556-586."""
        c = self.context
        if rotSlots not in self.rotKey_vec_23:
            raise ValueError("rotKey_23 not exists")
        _check(c.L_.ckks_rotate_23(c.h, cipher_res.cipher_device.ptr, cipher.cipher_device.ptr,
                                   self.rotKey_vec_23[rotSlots].cipher_device.ptr, rotSlots, cipher.l, *self._ks_buffers()), "ckks_rotate_23")
        cipher_res.l, cipher_res.scale, cipher_res.slots = cipher.l, cipher.scale, cipher.slots

    def rescaleAndEqual_noNTT(self, cipher):
        """Scheme_23.cuh:427-440: rescale of a coefficient-domain ciphertext."""
        c = self.context
        _check(c.L_.ckks_rescale_coeff(c.h, cipher.cipher_device.ptr, cipher.l), "ckks_rescale_coeff")
        cipher.scale = cipher.scale / c.qVec[cipher.l]
        cipher.l -= 1

    def conjugate_23(self, cipher_res, cipher):
        """KeySwitch_23.cuh:433-468."""
        c = self.context
        if self.ConjKey_23 is None:
            raise ValueError("conjKey_23 not exists")
        _check(c.L_.ckks_conjugate_23(c.h, cipher_res.cipher_device.ptr, cipher.cipher_device.ptr, self.ConjKey_23.cipher_device.ptr,
                                      cipher.l, *self._ks_buffers()), "ckks_conjugate_23")
        cipher_res.l, cipher_res.scale, cipher_res.slots = cipher.l, cipher.scale, cipher.slots

    # ---- the in-place and derived forms of the members above: host composition over the same entry points, same words ----
    def _temp(self, like):
        c = self.context
        t = getattr(self, "_cipher_temp", None)
        if t is None:
            t = self._cipher_temp = Ciphertext(c.N, c.L, like.l, like.slots, like.scale)
        return t

    def _copy_back(self, dst, src):
        c = self.context
        _check(c.L_.ckks_memcpy_d2d(dst.cipher_device.ptr, src.cipher_device.ptr, 8 * c.N * (c.L + 1) * 2), "ckks_memcpy_d2d")
        dst.l, dst.scale = src.l, src.scale

    def multAndEqual_23(self, cipher1, cipher2):
        """KeySwitch_23.cuh:238-282."""
        t = self._temp(cipher1)
        self.mult_23(t, cipher1, cipher2)
        self._copy_back(cipher1, t)

    def square(self, cipher1, cipher2):
        """KeySwitch_23.cuh:346-388: cipher1 = cipher2^2 (2ab, a^2, b^2 are the tensor of cipher2 with itself)."""
        self.mult_23(cipher1, cipher2, cipher2)

    def squareAndEqual(self, cipher):
        """KeySwitch_23.cuh:390-430."""
        t = self._temp(cipher)
        self.mult_23(t, cipher, cipher)
        self._copy_back(cipher, t)

    def conjugateAndEqual_23(self, cipher):
        """KeySwitch_23.cuh:473-506."""
        t = self._temp(cipher)
        self.conjugate_23(t, cipher)
        self._copy_back(cipher, t)

    def leftRotateAndEqual_23(self, cipher, rotSlots):
        """KeySwitch_23.cuh:509-553."""
        t = self._temp(cipher)
        self.leftRotate_23(t, cipher, rotSlots)
        self._copy_back(cipher, t)

    def rightRotateAndEqual_23(self, cipher, rotSlots):
        """KeySwitch_23.cuh:618-622: a right rotation by 2^rotSlots slots as the left rotation by N/2 - 2^rotSlots."""
        self.leftRotateAndEqual_23(cipher, self.context.N // 2 - (1 << rotSlots))

    def leftRotateAddSelf_23(self, cipher, rotSlots):
        """KeySwitch_23.cuh:583-616: cipher += cipher rotated left by rotSlots."""
        t = self._temp(cipher)
        self.leftRotate_23(t, cipher, rotSlots)
        self.addAndEqual(cipher, t)

    def add(self, cipher_res, cipher1, cipher2):
        """Scheme_23.cuh:130-141."""
        c = self.context
        l = min(cipher1.l, cipher2.l)
        for z in range(2):
            o = z * (c.L + 1)
            c.poly_add_3param_batch_device(cipher_res.cipher_device, cipher1.cipher_device, cipher2.cipher_device, o, o, o, c.K, l + 1)
        cipher_res.l, cipher_res.scale = l, cipher1.scale

    def addAndEqual(self, cipher1, cipher2):
        """Scheme_23.cuh:143-152."""
        scale = cipher1.scale
        self.add(cipher1, cipher1, cipher2)
        cipher1.scale = scale

    def sub(self, cipher_res, cipher1, cipher2):
        """Scheme_23.cuh:268-280 (the result keeps cipher1's level, as there)."""
        c = self.context
        l = min(cipher1.l, cipher2.l)
        for z in range(2):
            o = z * (c.L + 1)
            c.poly_sub_3param_batch_device(cipher_res.cipher_device, cipher1.cipher_device, cipher2.cipher_device, o, o, o, c.K, l + 1)
        cipher_res.l, cipher_res.scale = cipher1.l, cipher1.scale

    def subAndEqual(self, cipher1, cipher2):
        """Scheme_23.cuh:282-292."""
        l = min(cipher1.l, cipher2.l)
        self.sub(cipher1, cipher1, cipher2)
        cipher1.l = l

    def rescaleToAndEqual(self, cipher, level):
        """Scheme_23.cuh:407-425: to the coefficient domain, one coefficient-domain rescale per level, back."""
        c = self.context
        c.FromNTTInplace(cipher.cipher_device, 0, c.K, 2, cipher.l + 1, c.L + 1)
        while cipher.l > level:
            self.rescaleAndEqual_noNTT(cipher)
        c.ToNTTInplace(cipher.cipher_device, 0, c.K, 2, cipher.l + 1, c.L + 1)

    def _next_nonce(self):
        self.nonce += 1
        return self.nonce

    def addEncKey(self, secretKey):
        c = self.context
        N, L = c.N, c.L
        self.publicKey = Key(N, L, 0, 1)
        rnd = DeviceBuffer(8 * N * (L + 1) + 4 * N)
        c.generateRandom_device(rnd, rnd.nbytes, self.key, self._next_nonce())
        _check(c.L_.ckks_keygen_public(c.h, self.publicKey.cipher_device.ptr, secretKey.sx_device.ptr, rnd.ptr,
                                       rnd.ptr + 8 * N * (L + 1)), "ckks_keygen_public")
        rnd.free()

    def _encrypt(self, cipher, mx, l):
        if self.publicKey is None:
            raise ValueError("encryptMsg: no encryption key (addEncKey)")
        c = self.context
        c.generateRandom_device(self.in_enc, 9 * c.N, self.key, self._next_nonce())
        _check(c.L_.ckks_encrypt(c.h, cipher.cipher_device.ptr, mx, self.publicKey.cipher_device.ptr, self.in_enc.ptr,
                                 self.vx_enc.ptr, l), "ckks_encrypt")

    def encryptZero(self, cipher, l, slots):
        cipher.l, cipher.slots = l, slots
        self._encrypt(cipher, None, l)

    def encryptMsg(self, cipher, message):
        cipher.l, cipher.scale, cipher.slots = message.l, message.scale, message.slots
        self._encrypt(cipher, message.mx_device.ptr, message.l)

    def decryptMsg(self, plain, secretKey, cipher):
        c = self.context
        plain.l, plain.scale, plain.slots = cipher.l, cipher.scale, cipher.slots
        _check(c.L_.ckks_decrypt(c.h, plain.mx_device.ptr, cipher.cipher_device.ptr, secretKey.sx_device.ptr, cipher.l), "ckks_decrypt")

    def rescaleAndEqual(self, cipher):
        """Scheme_23.cuh:369-385: divides by q_l, level l -> l-1, scale /= q_l."""
        c = self.context
        c.rescaleAndEqual(cipher.cipher_device, self.rescale_buffer, cipher.l)
        cipher.scale = cipher.scale / c.qVec[cipher.l]
        cipher.l -= 1


class PCMM_Context:
    """PCMM_Context (pcmm/PCMM_Context.h:14-90)."""

    def __init__(self, N1, mlwe_rank, p_ringpack, q_ringpack, context):
        self.L_ = load_library()
        self.context, self.N1, self.mlwe_rank = context, N1, mlwe_rank
        self.p_ringpack, self.q_ringpack = list(p_ringpack), list(q_ringpack)
        self.ringpack_p_count, self.ringpack_q_count = len(self.p_ringpack), len(self.q_ringpack)
        self.ringpack_pq_count = self.ringpack_p_count + self.ringpack_q_count
        self.pq_ringpack = self.p_ringpack + self.q_ringpack
        pa, qa = _arr(p_ringpack), _arr(q_ringpack)
        h = vp()
        _check(self.L_.pcmm_ctx_create(C.byref(h), context.h, N1, mlwe_rank, pa.ctypes.data_as(u64p), len(pa),
                                       qa.ctypes.data_as(u64p), len(qa)), "pcmm_ctx_create")
        self.h = h.value

    def info(self, name):
        v = C.c_long()
        _check(self.L_.pcmm_info(self.h, name.encode(), C.byref(v)), "pcmm_info")
        return v.value

    def set_option(self, name, value=1):
        """Test / tuning switch by name: gather_plain, ppmm_generic, ppmm_no_tail (see ckks_hip.h)."""
        _check(self.L_.pcmm_set_option(self.h, name.encode(), int(value)), "pcmm_set_option")

    def weights_static(self, plain_mat, nbytes=None, is_static=True):
        """Declare a weight matrix static (it changes only through this library's copies): its digit planes are kept between PPMM
        calls.  By default every call reads its matrix afresh, as the reference does (PPMM_kernel.cuh:148)."""
        n = nbytes if nbytes is not None else plain_mat.nbytes
        _check(self.L_.pcmm_weights_static(self.h, _addr(plain_mat), n, int(bool(is_static))), "pcmm_weights_static")

    def set_weight_cache(self, enabled):
        """Declare every plaintext matrix given to this context static (True), or take that back (False, the default)."""
        _check(self.L_.pcmm_set_weight_cache(self.h, int(bool(enabled))), "pcmm_set_weight_cache")

    def weights_changed(self, plain_mat=None):
        """Say that a weight matrix was overwritten in place (None: all of them): its digit planes are built again."""
        _check(self.L_.pcmm_weights_changed(self.h, _addr(plain_mat) if plain_mat is not None else None), "pcmm_weights_changed")

    # -- PCMM_Context.h: size-N1 transforms over the ring-pack primes, data = [mod_batch_size][mod_num][poly_num][N1]
    def decodeCoeffs(self, msg, vals):
        """PCMM_Context.cuh:165-178: vals = N1 device doubles."""
        scratch = DeviceBuffer(8 * self.N1 * (msg.l + 1))
        _check(self.L_.pcmm_decode_coeffs(self.h, _addr(vals), _addr(msg.mx_device), scratch.ptr, int(msg.scale), msg.l), "pcmm_decode_coeffs")
        scratch.free()

    def ToNTTInplace(self, data, poly_num, mod_num, start_poly_idx, start_mod_idx, mod_batch_size):
        _check(self.L_.pcmm_ntt_fwd(self.h, _addr(data), poly_num, mod_num, start_poly_idx, start_mod_idx, mod_batch_size), "pcmm_ntt_fwd")

    def FromNTTInplace(self, data, poly_num, mod_num, start_poly_idx, start_mod_idx, mod_batch_size):
        _check(self.L_.pcmm_ntt_inv(self.h, _addr(data), poly_num, mod_num, start_poly_idx, start_mod_idx, mod_batch_size), "pcmm_ntt_inv")

    def __del__(self):
        try:
            if self.h:
                self.L_.pcmm_ctx_destroy(self.h)
                self.h = None
        except Exception:
            pass


class PlaintextT:
    """PlaintextT (bootstrapping/Bootstrapping_encoding.h): a plaintext over the T primes, NTT domain, t_num limbs, as the slot <->
    coefficient transforms multiply it into rotated ciphertexts."""

    def __init__(self, N, t_num, scale=1.0):
        self.N, self.t_num, self.scale = N, t_num, scale
        self.mx_device = DeviceBuffer(8 * N * t_num)


def _addr_or_null(x):
    if x is None:
        return None
    return _addr(x.cipher_device if hasattr(x, "cipher_device") else x.mx_device if hasattr(x, "mx_device") else x)


def _ptr_table(items):
    T = C.c_void_p * max(len(items), 1)
    return T(*[_addr_or_null(x) for x in items])


def _int_table(vals):
    T = C.c_int * max(len(vals), 1)
    return T(*[int(v) for v in vals])


class EncodingMatrix:
    """The hoisted baby-step / giant-step part of EncodingMatrix (Bootstrapping_C2S_S2C_impl.cuh): Giant_Rotate_And_Mult_PlaintT,
    Baby_Rotate, and one level of EvalCoeffsToSlots / EvalSlotsToCoeffs around them.  The plaintext diagonals and the rotation
    tables of a level (A[s], rot_in[s], rot_out[s]) come from the caller; their generation belongs to the bootstrapping set-up and
    is not part of this library."""

    def __init__(self, scheme):
        self.scheme = scheme
        self._scratch = None

    def Giant_Rotate_And_Mult_PlaintT(self, bs_cipher_T, PQ_to_T_temp, modUp_QjtoT_temp, rotKey_pointer, rotSlots_vec, plaintextT_pointer,
                                      accNum_vec, bs, gs, l):
        c = self.scheme.context
        _check(c.L_.ckks_giant_rotate_mult_plain_t(c.h, _addr(bs_cipher_T), _addr(PQ_to_T_temp), _addr(modUp_QjtoT_temp), _ptr_table(rotKey_pointer),
                                                   _int_table(rotSlots_vec), _ptr_table(plaintextT_pointer), _int_table(accNum_vec), bs, gs, l),
               "Giant_Rotate_And_Mult_PlaintT")

    def Baby_Rotate(self, output, modUp_QjtoT_temp, input, rotNum_here, rotKey_pointer, rotSlots_vec, l):
        c = self.scheme.context
        _check(c.L_.ckks_baby_rotate(c.h, _addr(output), _addr(modUp_QjtoT_temp), _addr(input), rotNum_here, _ptr_table(rotKey_pointer),
                                     _int_table(rotSlots_vec), l), "Baby_Rotate")

    def EvalLevel(self, A_s, cipher, rot_in, rot_out, b, g, numRotations, rescale=True):
        """One pass of the level loop (Bootstrapping_C2S_S2C_impl.cuh:254-382): cipher is in the COEFFICIENT domain and stays there.
        A_s[G + j] is the plaintext of baby step G / g and rotation j; index numRotations has none (:290-300).  Keys are taken from
        scheme.rotKey_vec_23; a missing one raises ValueError as the reference's key switches do."""
        sch, c = self.scheme, self.scheme.context
        plain, acc = [None] * (b * g), [0] * b
        for i in range(b):
            for j in range(g):
                if i * g + j != numRotations and i * g + j < len(A_s):
                    plain[i * g + j] = A_s[i * g + j]
                    acc[i] += 1
        key = lambda r: sch.rotKey_vec_23.get(r) if r else None
        words = C.c_size_t(0)
        _check(c.L_.ckks_bsgs_scratch_words(c.h, b, C.byref(words)), "ckks_bsgs_scratch_words")
        if self._scratch is None or self._scratch.nbytes < 8 * words.value:
            self._scratch = DeviceBuffer(8 * words.value)
        _check(c.L_.ckks_bsgs_level_23(c.h, _addr(cipher.cipher_device), cipher.l, _ptr_table(plain), _int_table(acc), _int_table(rot_in),
                                       _ptr_table([key(r) for r in rot_in]), _int_table(rot_out), _ptr_table([key(r) for r in rot_out]), b, g,
                                       self._scratch.ptr), "EvalLevel")
        cipher.scale = cipher.scale * A_s[0].scale
        if rescale:
            self.scheme.rescaleAndEqual_noNTT(cipher)


class MLWESecretKey:
    """MLWESecretKey (pcmm/MLWESecretKey.cuh:6-52): [L+1 moduli][k polynomials][N1]."""

    def __init__(self, N1, L, k):
        self.N1, self.L, self.k = N1, L, k
        self.sx_device = DeviceBuffer(8 * N1 * k * (L + 1))


class MLWEPlaintext:
    """MLWEPlaintext (pcmm/MLWEPlaintext.cuh:7-60): [L+1 moduli][N1]."""

    def __init__(self, N1, L, l, scale):
        self.N1, self.L, self.l, self.scale = N1, L, l, scale
        self.mx_device = DeviceBuffer(8 * N1 * (L + 1))


class MLWECiphertext:
    """MLWECiphertext (pcmm/MLWECiphertext.cuh): [L+1 moduli][a_0 .. a_{k-1}, b][N1] words, level l, scale."""

    def __init__(self, N1, L, l, k, scale):
        self.N1, self.L, self.l, self.k, self.scale = N1, L, l, k, scale
        self.cipher_device = DeviceBuffer(8 * N1 * (k + 1) * (L + 1))


class PCMM_Scheme:
    """PCMM_Scheme (pcmm/PCMM_Scheme.h:12-48): convertMLWESKfromRLWESK, addRepakcingKey, rlweCipherDecompose, PPMM,
    mlweCipherPacking, mlweDecrypt."""

    def __init__(self, pcmm_context, key=None):
        """key: 32 bytes of the random stream of the repacking keys; None (the default) draws them from the operating system."""
        self.L_ = load_library()
        self.pcmm_context = pcmm_context
        self.repackingKeys = None
        self.key, self.nonce = (os.urandom(32) if key is None else bytes(key)), 1 << 32
        self.ppmm_output = None                       # the reference's ppmm_output buffer (PCMM_Scheme.h), grown on demand
        self.ppmm_target_scale = float(1 << 49)       # PPMM_kernel.cuh:283 fixes 2^49, which suits its 50- to 60-bit ring-pack primes
        self.last_scaler = 0

    def convertMLWESKfromRLWESK(self, mlwe_sk, rlwe_sk):
        """PCMM_Scheme.cuh:23-48."""
        _check(self.L_.pcmm_convert_mlwe_sk(self.pcmm_context.h, _addr(mlwe_sk.sx_device), _addr(rlwe_sk.sx_device)), "pcmm_convert_mlwe_sk")

    def addRepakcingKey(self, mlwe_sk, rlwe_sk):
        """PCMM_Scheme.cuh:126-224; the keys stay in self.repackingKeys (one device buffer, key i at i*2*m*N words)."""
        pc = self.pcmm_context
        if self.repackingKeys is not None:
            return                                                           # "repacking keys already generated!" (:152-155)
        N = pc.context.N
        m = pc.ringpack_p_count + pc.ringpack_q_count - 1
        keys = DeviceBuffer(8 * N * m * 2 * pc.mlwe_rank)
        scratch = DeviceBuffer(8 * N * (m + 1))
        _check(self.L_.pcmm_add_repacking_key(pc.h, keys.ptr, _addr(mlwe_sk.sx_device), _addr(rlwe_sk.sx_device), self.key, self.nonce,
                                              scratch.ptr), "pcmm_add_repacking_key")
        self.nonce += pc.mlwe_rank
        scratch.free()
        self.repackingKeys = keys

    def mlweDecrypt(self, mlwe_cipher, mlwe_sk, mlwe_plain, l):
        """PCMM_Scheme.cuh:557-576; mlwe_cipher: device buffer of one sample."""
        _check(self.L_.pcmm_mlwe_decrypt(self.pcmm_context.h, _addr(mlwe_plain.mx_device), _addr(mlwe_cipher), _addr(mlwe_sk.sx_device), l),
               "pcmm_mlwe_decrypt")
        mlwe_plain.l = l

    @staticmethod
    def _ptrs(bufs):
        T = vp * len(bufs)
        return T(*[_addr(b) for b in bufs])

    def rlweCipherDecompose(self, rlwe_cipher, mlwe_cipher_decomposed, mlwe_num, offset, l, coeff_domain=False):
        """PCMM_Scheme.cuh:90-125.  rlwe_cipher: [a | b] device buffer at level l; coeff_domain=True runs the gather only."""
        bufs = mlwe_cipher_decomposed[offset:offset + mlwe_num]
        f = self.L_.pcmm_rlwe_decompose if coeff_domain else self.L_.pcmm_rlwe_decompose_ntt
        _check(f(self.pcmm_context.h, _addr(rlwe_cipher), self._ptrs(bufs), mlwe_num, l), "pcmm_rlwe_decompose")

    def mlweCipherPacking(self, rlwe_cipher, mlwe_cipher_decomposed, mlwe_num, offset, repacking_keys, embeded_mlwe_buffer,
                          mult_key_output):
        """PCMM_Scheme.cuh:361-425.  rlwe_cipher: [a | b] device buffer (limb 0 of both polynomials is written, NTT domain);
        repacking_keys: rank keys [a | b] over [p0 | q0] in one device buffer; the two scratch buffers are the reference's
        embeded_mlwe_buffer ((rank+1)*2*N words) and the 4*N words it borrows from the scheme for the key product."""
        bufs = mlwe_cipher_decomposed[offset:offset + mlwe_num]
        _check(self.L_.pcmm_mlwe_pack(self.pcmm_context.h, _addr(rlwe_cipher), self._ptrs(bufs), mlwe_num, _addr(repacking_keys),
                                      _addr(embeded_mlwe_buffer), _addr(mult_key_output)), "pcmm_mlwe_pack")

    def PPMM(self, plain_mat, mlwe_cipher_decomposed, *args):
        """Two forms.  The reference's (PCMM_Scheme.h, PPMM_kernel.cuh:254-349): PPMM(plain_mat, mlwe_cipher_decomposed, mat_M, mat_N, mat_K,
        mlwe_num) on MLWECiphertext objects - the scaler is (long)(q_ringpack[1] * 2^49 / scale) (:283-284), all ring-pack moduli take
        part, row i of the product (first modulus) is copied back into mlwe_cipher_decomposed[i] for i < min(mat_M, mlwe_num) and its
        scale becomes scale * scaler / q_ringpack[1] (:345-348).  And the device part alone: PPMM(plain_mat, buffers, out, mat_M, mat_N,
        mat_K, mlwe_num, mod_num, scaler).  Shape errors are reported the way the reference does: a message and no work
        (PPMM_kernel.cuh:256-263), here as ValueError."""
        if len(args) == 4:
            return self._PPMM_reference(plain_mat, mlwe_cipher_decomposed, *args)
        out, mat_M, mat_N, mat_K, mlwe_num, mod_num, scaler = args
        if mat_K != self.pcmm_context.N1:
            raise ValueError("matrix K should be equal to N1!")
        if mat_N != mlwe_num:
            raise ValueError("matrix N should be equal to mlwe number!")
        _check(self.L_.pcmm_ppmm(self.pcmm_context.h, _addr(plain_mat), self._ptrs(mlwe_cipher_decomposed[:mlwe_num]), _addr(out),
                                 mat_M, mat_N, mod_num, float(scaler)), "pcmm_ppmm")

    def _PPMM_reference(self, plain_mat, mlwe, mat_M, mat_N, mat_K, mlwe_num):
        pc = self.pcmm_context
        if mat_K != pc.N1:
            raise ValueError("matrix K should be equal to N1!")
        if mat_N != mlwe_num:
            raise ValueError("matrix N should be equal to mlwe number!")
        mods, C = pc.ringpack_q_count, (pc.mlwe_rank + 1) * pc.N1
        if self.ppmm_output is None or self.ppmm_output.nbytes < 8 * mat_M * mods * C:
            self.ppmm_output = DeviceBuffer(8 * mat_M * mods * C)
        scaler = int(pc.q_ringpack[1] * self.ppmm_target_scale / mlwe[0].scale)                 # PPMM_kernel.cuh:283-284
        self.last_scaler = scaler
        _check(self.L_.pcmm_ppmm(pc.h, _addr(plain_mat), self._ptrs([m.cipher_device for m in mlwe[:mlwe_num]]), _addr(self.ppmm_output),
                                 mat_M, mat_N, mods, float(scaler)), "pcmm_ppmm")
        for i in range(min(mat_M, mlwe_num)):                                                    # :345-348
            mlwe[i].scale = mlwe[i].scale * scaler / pc.q_ringpack[1]
            _check(self.L_.ckks_memcpy_d2d(mlwe[i].cipher_device.ptr, self.ppmm_output.ptr + 8 * i * C * mods, 8 * C), "ckks_memcpy_d2d")

    # -- the gather writing PPMM's operand directly (no counterpart in the reference: its layer runs rlweCipherDecompose and PPMM back
    #    to back through 8-byte MLWE samples, Bert.cuh:411-424)
    def packed_begin(self, mat_N, mod_num):
        _check(self.L_.pcmm_packed_begin(self.pcmm_context.h, mat_N, mod_num), "pcmm_packed_begin")

    def rlweCipherDecompose_packed(self, rlwe_cipher, mlwe_num, offset, l, take=None):
        """The first `take` (default: all) of the mlwe_num samples of one RLWE ciphertext (NTT domain, level l) become samples
        offset .. offset + take - 1 of the opened operand."""
        _check(self.L_.pcmm_rlwe_decompose_packed(self.pcmm_context.h, _addr(rlwe_cipher), offset, mlwe_num, mlwe_num if take is None else take, l),
               "pcmm_rlwe_decompose_packed")

    def PPMM_packed(self, plain_mat, out, mat_M, scaler):
        _check(self.L_.pcmm_ppmm_packed(self.pcmm_context.h, _addr(plain_mat), _addr(out), mat_M, float(scaler)), "pcmm_ppmm_packed")

    def PPMM_strided(self, plain_mat, mlwe_all, out, mat_M, mat_N, mod_num, scaler):
        _check(self.L_.pcmm_ppmm_strided(self.pcmm_context.h, _addr(plain_mat), _addr(mlwe_all), _addr(out), mat_M, mat_N,
                                         mod_num, float(scaler)), "pcmm_ppmm_strided")


class Bert_model_weights:
    """Bert_model_weights (src/bert/Load_bert.cuh:11-348): the fp32 tensors of a BERT-base `model.safetensors` as device buffers
    under the reference's member names (per-layer members are lists of 12).  File format: 8 bytes little-endian header length, a
    JSON header {name: {"dtype", "shape", "data_offsets": [begin, end]}}, then the tensor bytes.  A tensor that is absent, not
    F32 or out of the file's range stays None and is listed in `missing`."""

    GLOBAL = {
        "embeddings_LayerNorm_beta": "bert.embeddings.LayerNorm.beta", "embeddings_LayerNorm_gamma": "bert.embeddings.LayerNorm.gamma",
        "embeddings_position_embeddings_weight": "bert.embeddings.position_embeddings.weight",
        "embeddings_token_type_embeddings_weight": "bert.embeddings.token_type_embeddings.weight",
        "embeddings_word_embeddings_weight": "bert.embeddings.word_embeddings.weight",
        "pooler_dense_bias": "bert.pooler.dense.bias", "pooler_dense_weight": "bert.pooler.dense.weight",
        "cls_predictions_bias": "cls.predictions.bias",
        "cls_predictions_transform_LayerNorm_beta": "cls.predictions.transform.LayerNorm.beta",
        "cls_predictions_transform_LayerNorm_gamma": "cls.predictions.transform.LayerNorm.gamma",
        "cls_predictions_transform_dense_bias": "cls.predictions.transform.dense.bias",
        "cls_predictions_transform_dense_weight": "cls.predictions.transform.dense.weight",
        "cls_seq_relationship_bias": "cls.seq_relationship.bias", "cls_seq_relationship_weight": "cls.seq_relationship.weight",
    }
    LAYER = ["attention.output.LayerNorm.beta", "attention.output.LayerNorm.gamma", "attention.output.dense.bias",
             "attention.output.dense.weight", "attention.self.key.bias", "attention.self.key.weight", "attention.self.query.bias",
             "attention.self.query.weight", "attention.self.value.bias", "attention.self.value.weight", "intermediate.dense.bias",
             "intermediate.dense.weight", "output.LayerNorm.beta", "output.LayerNorm.gamma", "output.dense.bias", "output.dense.weight"]

    def __init__(self, model_catalog):
        import json
        import os
        self.num_layers = 12
        self.opened, self.missing, self.loaded = False, [], []
        for member in self.GLOBAL:
            setattr(self, member, None)
        for leaf in self.LAYER:
            setattr(self, leaf.replace(".", "_"), [None] * self.num_layers)
        fname = model_catalog + "model.safetensors"                       # Load_bert.cuh:50
        if not os.path.exists(fname):
            print("Failed to open model file: " + fname)
            return
        with open(fname, "rb") as f:
            head = f.read(8)
            size = os.path.getsize(fname)
            n = int.from_bytes(head, "little") if len(head) == 8 else -1
            if n < 0 or 8 + n > size:
                print("Failed to read header size from: " + fname)
                return
            header = json.loads(f.read(n))
            self.opened = True
            data_bytes = size - 8 - n

            def load(name):
                e = header.get(name)
                if not isinstance(e, dict) or e.get("dtype") != "F32":
                    self.missing.append(name)
                    return None
                begin, end = e["data_offsets"]
                if begin < 0 or end < begin or end > data_bytes or (end - begin) % 4:
                    self.missing.append(name)
                    return None
                f.seek(8 + n + begin)
                buf = DeviceBuffer.from_numpy(np.frombuffer(f.read(end - begin), dtype=np.float32))
                self.loaded.append((name, end - begin))
                return buf

            for member, name in self.GLOBAL.items():
                setattr(self, member, load(name))
            for i in range(self.num_layers):
                for leaf in self.LAYER:
                    getattr(self, leaf.replace(".", "_"))[i] = load("bert.encoder.layer.%d.%s" % (i, leaf))

    def buffers(self):
        """Every device buffer that was loaded."""
        out = [getattr(self, m) for m in self.GLOBAL]
        for leaf in self.LAYER:
            out += getattr(self, leaf.replace(".", "_"))
        return [b for b in out if b is not None]


class Bert:
    """The PCMM calls of the linear layers of Bert (src/bert/Bert.h:15-66; Bert.cuh:155-169, 204-211, 249-257, 296-302, 404-489):
    gather of the input ciphertexts into MLWE samples, PPMM with the layer's weight, ring packing of the product rows, with the
    reference's sample counts and offsets.  Ciphertexts enter and leave in coefficient packing; the slot <-> coefficient
    conversions, EvalMod and the non-linear layers that the reference runs in between are not part of this library.
    The gather writes PPMM's operand planes directly, which needs ring-pack primes below 2^39."""

    def __init__(self, model_catalog, context, scheme, pcmm_scheme, sk, target_scale=float(1 << 49)):
        self.context, self.scheme, self.pcmm_scheme, self.sk = context, scheme, pcmm_scheme, sk
        self.model_weights = Bert_model_weights(model_catalog)
        pc = pcmm_scheme.pcmm_context
        self.PCMM_N1, self.mlwe_rank, self.q_ringpack_count = pc.N1, pc.mlwe_rank, pc.ringpack_q_count
        self.N, self.L = context.N, context.L
        if self.mlwe_rank * self.PCMM_N1 != self.N:
            raise ValueError("Bert: the PCMM context's rank is not N / N1")
        self.target_scale = target_scale                                  # the reference fixes 2^49 (PPMM_kernel.cuh:283)
        self.ppmm_output = None
        self.embeded_mlwe_buffer = DeviceBuffer(8 * (self.mlwe_rank + 1) * 2 * self.N)
        self.mult_key_output = DeviceBuffer(8 * 4 * self.N)
        # the model's tensors were uploaded by this object and are not written again: their digit planes are kept between calls
        for buf in self.model_weights.buffers():
            pc.weights_static(buf)

    def linear(self, plain_mat, M, Nin, parts_in, parts_out):
        """parts_in: (ciphertext, count, offset, extract); parts_out: (ciphertext, count, offset)."""
        ps, pc = self.pcmm_scheme, self.pcmm_scheme.pcmm_context
        mods, C = self.q_ringpack_count, (self.mlwe_rank + 1) * self.PCMM_N1
        if self.ppmm_output is None or self.ppmm_output.nbytes < 8 * M * mods * C:
            self.ppmm_output = DeviceBuffer(8 * M * mods * C)
        in_scale = parts_in[0][0].scale
        scaler = float(int(pc.q_ringpack[1] * self.target_scale / in_scale))        # PPMM_kernel.cuh:283-284
        ps.packed_begin(Nin, mods)
        for ct, count, offset, extract in parts_in:
            ps.rlweCipherDecompose_packed(ct.cipher_device, extract, offset, ct.l, take=count)
        ps.PPMM_packed(plain_mat, self.ppmm_output, M, scaler)
        rows = [self.ppmm_output.ptr + 8 * m * mods * C for m in range(M)]          # row m, first modulus
        for ct, count, offset in parts_out:
            ps.mlweCipherPacking(ct.cipher_device, rows, count, offset, ps.repackingKeys, self.embeded_mlwe_buffer, self.mult_key_output)
            ct.l, ct.scale = 0, in_scale * scaler / pc.q_ringpack[1]

    def PCMM_768_768(self, plain_mat, rlwe_cipher, res_cipher, do_s2c):
        """do_s2c = 0: two inputs of 512 samples, the first 768 multiplied (Bert.cuh:416-417, 425); 1: three of 256 (:404-412)."""
        if do_s2c == 1:
            parts = [(rlwe_cipher[0], 256, 0, 256), (rlwe_cipher[1], 256, 256, 256), (rlwe_cipher[2], 256, 512, 256)]
        else:
            parts = [(rlwe_cipher[0], 512, 0, 512), (rlwe_cipher[1], 256, 512, 512)]
        self.linear(plain_mat, 768, 768, parts, [(res_cipher[0], 256, 0), (res_cipher[1], 256, 256), (res_cipher[2], 256, 512)])

    def PCMM_Boot_768_768(self, plain_mat, rlwe_cipher, res_cipher, target_level, do_s2c):
        """Bert.h:62 (Bert.cuh:379-498).  target_level is the level the reference raises the packed result to before its
        coefficient-to-slot conversion and EvalMod (:472-497), a stage outside this library: accepted and not used."""
        self.PCMM_768_768(plain_mat, rlwe_cipher, res_cipher, do_s2c)

    test_PCMM_Boot_768_768 = PCMM_Boot_768_768                         # Bert.h:63

    def mul_W_QKV(self, X, *args):
        """Bert.h:51: mul_W_QKV(X, model_weights, resQ, resK, resV, layer), three inputs of 256 samples (do_s2c = 1) as the
        reference calls it (Bert.cuh:155-169; its bias additions on slot-packed plaintexts are not part of this library).
        Also mul_W_QKV(X, resQ, resK, resV, layer, do_s2c=1) on the object's own weights."""
        if isinstance(args[0], Bert_model_weights):
            w, resQ, resK, resV, layer = args
            do_s2c = 1
        else:
            w = self.model_weights
            resQ, resK, resV, layer = args[:4]
            do_s2c = args[4] if len(args) > 4 else 1
        self.PCMM_768_768(w.attention_self_query_weight[layer], X, resQ, do_s2c)
        self.PCMM_768_768(w.attention_self_key_weight[layer], X, resK, do_s2c)
        self.PCMM_768_768(w.attention_self_value_weight[layer], X, resV, do_s2c)

    def attn_output(self, O, *args):
        """Bert.h:59: attn_output(O, layer), the dense product in place (Bert.cuh:204-211).  Also attn_output(O, res, layer, do_s2c=1)."""
        if isinstance(args[0], int):
            res, layer, do_s2c = O, args[0], 1
        else:
            res, layer = args[:2]
            do_s2c = args[2] if len(args) > 2 else 1
        self.PCMM_768_768(self.model_weights.attention_output_dense_weight[layer], O, res, do_s2c)

    def intermediate(self, O, layer, res):
        """Bert.cuh:249-257: 512 samples of O[0] and 256 of O[2]; 3072 x 768; rows 512 i .. into res[2 i]."""
        self.linear(self.model_weights.intermediate_dense_weight[layer], 3072, 768, [(O[0], 512, 0, 512), (O[2], 256, 512, 256)],
                    [(res[2 * i], 512, 512 * i) for i in range(6)])

    def layer_output(self, O, layer, layer_res=None):
        """Bert.h:61, Bert.cuh:290-302: 512 samples of each O[2 i]; 768 x 3072; rows 0..511 into O[0], 512..767 into O[2].
        layer_res is not touched: the reference's body does not use it either (Bert.cuh:333, 349-353 are commented out)."""
        self.linear(self.model_weights.output_dense_weight[layer], 768, 3072, [(O[2 * i], 512, 512 * i, 512) for i in range(6)],
                    [(O[0], 512, 0), (O[2], 256, 512)])
