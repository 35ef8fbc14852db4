"""ctypes binding of the CPU oracle (oracle/libckks_oracle.so).

Test infrastructure: imported by tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg only.
"""
import ctypes as C
import os
import subprocess
import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libckks_oracle.so")
u64 = C.c_uint64
P64 = C.POINTER(C.c_uint64)
P8 = C.POINTER(C.c_uint8)


def build(force=False):
    if force or not os.path.exists(_SO):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "libckks_oracle.so"])
    return _SO


def _ptr(a):
    assert a.dtype == np.uint64 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(P64)


def _bytes(a):
    assert a.dtype == np.uint8 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(P8)


def salsa20_stream(n, key, nonce):
    """n bytes of the Salsa20/20 key stream of (32-byte key, 64-bit nonce), block counter from 0 (RNG.cuh:18-56)."""
    out = np.zeros(n, dtype=np.uint8)
    k = np.frombuffer(bytes(key), dtype=np.uint8).copy()
    assert k.size == 32
    lib().orc_salsa20_stream(_bytes(out), n, _bytes(k), nonce)
    return out


def gauss_thresholds():
    out = np.zeros(19, dtype=np.uint32)
    lib().orc_gauss_thresholds(out.ctypes.data_as(C.POINTER(C.c_uint32)))
    return out


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(_SO)
        i, d, l = C.c_int, C.c_double, C.c_long
        vp = C.c_void_p
        sig = {
            "orc_mulmod": (u64, [u64, u64, u64]), "orc_powmod": (u64, [u64, u64, u64]),
            "orc_invmod": (u64, [u64, u64]), "orc_xshoup": (u64, [u64, u64]),
            "orc_mulmod_shoup": (u64, [u64, u64, u64, u64]),
            "orc_barrett_mu": (None, [u64, P64, P64]),
            "orc_barrett128": (u64, [u64, u64, u64, u64, u64]), "orc_barrett64": (u64, [u64, u64, u64]),
            "orc_find_primitive_root": (u64, [u64]), "orc_find_mth_root": (u64, [u64, u64]),
            "orc_bitrev": (C.c_uint32, [C.c_uint32, i]),
            "orc_fill_psi_tables": (None, [u64, u64, C.c_uint32, P64, P64, P64, P64]),
            "orc_ntt_limb": (None, [P64, C.c_uint32, u64, P64]),
            "orc_intt_limb": (None, [P64, C.c_uint32, u64, P64, u64]),
            "orc_negacyclic_mul": (None, [P64, P64, P64, C.c_uint32, u64]),
            "orc_ctx_create": (vp, [i, P64, i, P64, i, P64, i, i]), "orc_ctx_destroy": (None, [vp]),
            "orc_ctx_get": (l, [vp, C.c_char_p, P64, l]), "orc_ctx_info": (i, [vp, C.c_char_p]),
            "orc_ntt_fwd": (i, [vp, P64, i, i, i, i, i]), "orc_ntt_inv": (i, [vp, P64, i, i, i, i, i]),
            "orc_ntt_fwd_ext": (i, [vp, P64, i, i, i, i, i, i, i]), "orc_ntt_inv_ext": (i, [vp, P64, i, i, i, i, i, i, i]),
            "orc_modup_pq_to_t": (i, [vp, P64, P64, i, i]), "orc_modup_qj_to_t": (i, [vp, P64, P64, i, i]),
            "orc_modup_t_to_pql": (i, [vp, P64, P64, i, i]), "orc_moddown_pql_to_ql": (i, [vp, P64, P64, i, i]),
            "orc_external_product_t": (i, [vp, P64, P64, P64, i]), "orc_external_product_t_swk_reuse": (i, [vp, P64, P64, P64, i, i]), "orc_rescale": (i, [vp, P64, i]),
            "orc_keyswitch_23": (i, [vp, P64, P64, P64, i]),
            "orc_hybrid_modup": (i, [vp, P64, P64, i]), "orc_hybrid_inner_product": (i, [vp, P64, P64, P64, i]),
            "orc_hybrid_moddown": (i, [vp, P64, P64, i]), "orc_hybrid_keyswitch": (i, [vp, P64, P64, P64, i]),
            "orc_pcmm_create": (vp, [vp, i, i, P64, i, P64, i]), "orc_pcmm_destroy": (None, [vp]),
            "orc_rlwe_decompose": (i, [vp, P64, C.POINTER(P64), i, i]),
            "orc_ppmm": (i, [vp, C.POINTER(C.c_float), C.POINTER(P64), P64, i, i, i, d, l, l]),
            "orc_mlwe_pack": (i, [vp, P64, C.POINTER(P64), i, P64]),
            "orc_pcmm_ntt": (i, [vp, P64, i, i, i, i, i]),
            "orc_salsa20_stream": (None, [P8, C.c_size_t, P8, u64]),
            "orc_gauss_thresholds": (None, [C.POINTER(C.c_uint32)]),
            "orc_sample_uniform": (i, [vp, P8, P64, i, i, i]), "orc_sample_gaussian": (i, [vp, P8, P64, i, i, i]),
            "orc_sample_zo": (i, [vp, P8, P64, d, i, i, i]), "orc_sample_hwt": (i, [vp, P8, P64, i, i, i, i]),
            "orc_poly_op": (i, [vp, i, P64, P64, P64, i, i, i, i, i]),
            "orc_keygen_secret": (i, [vp, P64, P8, i]), "orc_keygen_public": (i, [vp, P64, P64, P8, P8]),
            "orc_encrypt": (i, [vp, P64, P64, P64, P8, i]), "orc_decrypt": (i, [vp, P64, P64, P64, i]),
            "orc_encode_coeffs": (i, [vp, P64, C.POINTER(C.c_double), l, i]),
            "orc_rot_group": (u64, [vp, l]),
            "orc_automorph_ntt": (i, [vp, P64, P64, u64, i, i, i]), "orc_conjugate_ntt": (i, [vp, P64, P64, i, i, i]),
            "orc_keygen_switch_23": (i, [vp, P64, P64, P64, P8, P8]),
            "orc_mult_23": (i, [vp, P64, P64, P64, P64, i]), "orc_rotate_23": (i, [vp, P64, P64, P64, l, i]),
            "orc_conjugate_23": (i, [vp, P64, P64, P64, i]),
            "orc_cipher_mul_p": (i, [vp, P64, P64, i]), "orc_cipher_add_t": (i, [vp, P64, P64, i]), "orc_rescale_coeff": (i, [vp, P64, i]),
            "orc_giant_rotate_mult_plain_t": (i, [vp, P64, P64, P64, C.POINTER(P64), C.POINTER(i), C.POINTER(P64), C.POINTER(i), i, i, i]),
            "orc_baby_rotate": (i, [vp, P64, P64, P64, i, C.POINTER(P64), C.POINTER(i), i]),
            "orc_bsgs_level_23": (i, [vp, P64, i, C.POINTER(P64), C.POINTER(i), C.POINTER(i), C.POINTER(P64), C.POINTER(i), C.POINTER(P64), i, i]),
            "orc_pcmm_convert_mlwe_sk": (i, [vp, P64, P64]), "orc_pcmm_add_repacking_key": (i, [vp, P64, P64, P64, P8]),
            "orc_pcmm_mlwe_decrypt": (i, [vp, P64, P64, P64, i]),
            "orc_pcmm_decode_coeffs": (i, [vp, C.POINTER(C.c_double), P64, C.c_longlong, i]),
            "orc_max_threads": (i, []),
        }
        for name, (res, args) in sig.items():
            f = getattr(L, name)
            f.restype = res
            f.argtypes = args
        _lib = L
    return _lib


def _arr(v):
    return np.ascontiguousarray(np.array(list(v), dtype=np.uint64))


class OracleContext:
    """Mirror of Context_23 (Context_23.h:19-279) on host arrays, with explicit prime lists."""

    def __init__(self, logN, p, q, t=(), gamma=0):
        self.L_ = lib()
        self.logN, self.N = logN, 1 << logN
        self.p, self.q, self.t = list(p), list(q), list(t)
        self.p_num, self.q_num, self.t_num, self.gamma = len(self.p), len(self.q), len(self.t), gamma
        pa, qa, ta = _arr(p), _arr(q), _arr(t)
        self.h = self.L_.orc_ctx_create(logN, _ptr(pa), len(pa), _ptr(qa), len(qa), _ptr(ta), len(ta), gamma)
        self.K, self.L = self.p_num, self.q_num - 1
        self.dnum = self.info("dnum")
        self.Ri_blockNum = self.info("Ri_blockNum")
        self.Qj_blockNum = self.info("Qj_blockNum")

    def __del__(self):
        try:
            self.L_.orc_ctx_destroy(self.h)
        except Exception:
            pass

    def info(self, name):
        return self.L_.orc_ctx_info(self.h, name.encode())

    def table(self, name):
        n = self.L_.orc_ctx_get(self.h, name.encode(), None, 0)
        if n < 0:
            raise KeyError(name)
        out = np.zeros(n, dtype=np.uint64)
        self.L_.orc_ctx_get(self.h, name.encode(), _ptr(out), n)
        return out

    def _ck(self, rc):
        if rc != 0:
            raise ValueError("oracle call failed: %d" % rc)

    def ToNTTInplace(self, a, start_poly_idx, start_mod_idx, poly_num, mod_num, poly_mod_len):
        self._ck(self.L_.orc_ntt_fwd(self.h, _ptr(a), start_poly_idx, start_mod_idx, poly_num, mod_num, poly_mod_len))

    def FromNTTInplace(self, a, start_poly_idx, start_mod_idx, poly_num, mod_num, poly_mod_len):
        self._ck(self.L_.orc_ntt_inv(self.h, _ptr(a), start_poly_idx, start_mod_idx, poly_num, mod_num, poly_mod_len))

    def ToNTTInplace_for_externalProduct(self, a, sp, sm, pn, mn, pml, cmn, bs):
        self._ck(self.L_.orc_ntt_fwd_ext(self.h, _ptr(a), sp, sm, pn, mn, pml, cmn, bs))

    def FromNTTInplace_for_externalProduct(self, a, sp, sm, pn, mn, pml, cmn, bs):
        self._ck(self.L_.orc_ntt_inv_ext(self.h, _ptr(a), sp, sm, pn, mn, pml, cmn, bs))

    def modUpPQtoT_23(self, out, inp, l, batch):
        self._ck(self.L_.orc_modup_pq_to_t(self.h, _ptr(out), _ptr(inp), l, batch))

    def modUpQjtoT_23(self, out, inp, l, batch):
        self._ck(self.L_.orc_modup_qj_to_t(self.h, _ptr(out), _ptr(inp), l, batch))

    def modUpTtoPQl_23(self, buf, inp, l, batch):
        self._ck(self.L_.orc_modup_t_to_pql(self.h, _ptr(buf), _ptr(inp), l, batch))

    def modDownPQltoQl_23(self, out, buf, l, batch):
        self._ck(self.L_.orc_moddown_pql_to_ql(self.h, _ptr(out), _ptr(buf), l, batch))

    def external_product_T(self, out, cT, swk, l):
        self._ck(self.L_.orc_external_product_t(self.h, _ptr(out), _ptr(cT), _ptr(swk), l))

    def external_product_T_swk_reuse(self, out, cT, swk, l, batch_size):
        self._ck(self.L_.orc_external_product_t_swk_reuse(self.h, _ptr(out), _ptr(cT), _ptr(swk), l, batch_size))

    def rescaleAndEqual(self, cipher, l):
        self._ck(self.L_.orc_rescale(self.h, _ptr(cipher), l))

    def keyswitch_23(self, out, d2, swk, l):
        self._ck(self.L_.orc_keyswitch_23(self.h, _ptr(out), _ptr(d2), _ptr(swk), l))

    def hybrid_modup(self, digits, inp, l):
        self._ck(self.L_.orc_hybrid_modup(self.h, _ptr(digits), _ptr(inp), l))

    def hybrid_inner_product(self, out, digits, evk, l):
        self._ck(self.L_.orc_hybrid_inner_product(self.h, _ptr(out), _ptr(digits), _ptr(evk), l))

    def hybrid_moddown(self, out, inp, l):
        self._ck(self.L_.orc_hybrid_moddown(self.h, _ptr(out), _ptr(inp), l))

    def hybrid_keyswitch(self, out, in_ntt, evk, l):
        self._ck(self.L_.orc_hybrid_keyswitch(self.h, _ptr(out), _ptr(in_ntt), _ptr(evk), l))

    # ---- samplers (Sampler.cuh:17-54), pointwise arithmetic (poly_arithmetic.cuh), keys and encryption (Scheme_23.cuh:54-127) ----
    def uniformSampler_xq(self, random, out, idx_out, idx_mod, mod_num):
        self._ck(self.L_.orc_sample_uniform(self.h, _bytes(random), _ptr(out), idx_out, idx_mod, mod_num))

    def gaussianSampler_xq(self, random, out, idx_out, idx_mod, mod_num):
        self._ck(self.L_.orc_sample_gaussian(self.h, _bytes(random), _ptr(out), idx_out, idx_mod, mod_num))

    def ZOSampler(self, random, out, probability, idx_out, idx_mod, mod_num):
        self._ck(self.L_.orc_sample_zo(self.h, _bytes(random), _ptr(out), probability, idx_out, idx_mod, mod_num))

    def HWTSampler(self, random, out, h, idx_out, idx_mod, mod_num):
        self._ck(self.L_.orc_sample_hwt(self.h, _bytes(random), _ptr(out), h, idx_out, idx_mod, mod_num))

    def poly_op(self, op, c, a, b, idx_c, idx_a, idx_b, idx_mod, mod_num):
        """op 0: c = a*b (barrett_batch_3param_device), 1: c = a+b (poly_add_3param_batch_device), 2: c = a-b."""
        self._ck(self.L_.orc_poly_op(self.h, op, _ptr(c), _ptr(a), _ptr(b), idx_c, idx_a, idx_b, idx_mod, mod_num))

    def keygen_secret(self, sx, random, h):
        self._ck(self.L_.orc_keygen_secret(self.h, _ptr(sx), _bytes(random), h))

    def keygen_public(self, pk, sx, random_a, random_e):
        self._ck(self.L_.orc_keygen_public(self.h, _ptr(pk), _ptr(sx), _bytes(random_a), _bytes(random_e)))

    def encrypt(self, cipher, mx, pk, random, l):
        self._ck(self.L_.orc_encrypt(self.h, _ptr(cipher), None if mx is None else _ptr(mx), _ptr(pk), _bytes(random), l))

    def decrypt(self, mx, cipher, sx, l):
        self._ck(self.L_.orc_decrypt(self.h, _ptr(mx), _ptr(cipher), _ptr(sx), l))

    def encode_coeffs(self, mx, vals, scale, l):
        assert vals.dtype == np.float64 and vals.size == self.N
        self._ck(self.L_.orc_encode_coeffs(self.h, _ptr(mx), vals.ctypes.data_as(C.POINTER(C.c_double)), int(scale), l))

    # ---- automorphisms, switching keys in the T basis, homomorphic multiply / rotate / conjugate (KeySwitch_23.cuh) ----
    def rot_group(self, idx):
        return int(self.L_.orc_rot_group(self.h, idx))

    def automorph_ntt(self, out, inp, pow_, idx_out, idx_in, mod_num):
        self._ck(self.L_.orc_automorph_ntt(self.h, _ptr(out), _ptr(inp), pow_, idx_out, idx_in, mod_num))

    def conjugate_ntt(self, out, inp, idx_out, idx_in, mod_num):
        self._ck(self.L_.orc_conjugate_ntt(self.h, _ptr(out), _ptr(inp), idx_out, idx_in, mod_num))

    def keygen_switch_23(self, swk, s_to, s_from, random_a, random_e):
        self._ck(self.L_.orc_keygen_switch_23(self.h, _ptr(swk), _ptr(s_to), _ptr(s_from), _bytes(random_a), _bytes(random_e)))

    def mult_23(self, out, c1, c2, rlk, l):
        rc = self.L_.orc_mult_23(self.h, _ptr(out), _ptr(c1), _ptr(c2), _ptr(rlk), l)
        if rc == -4:
            raise ValueError("Ciphertexts are on level 0")
        self._ck(rc)

    def leftRotate_23(self, out, cipher, rotkey, rot, l):
        self._ck(self.L_.orc_rotate_23(self.h, _ptr(out), _ptr(cipher), _ptr(rotkey), rot, l))

    def conjugate_23(self, out, cipher, conjkey, l):
        self._ck(self.L_.orc_conjugate_23(self.h, _ptr(out), _ptr(cipher), _ptr(conjkey), l))

    # hoisted rotations of the slot <-> coefficient transforms (Bootstrapping_C2S_S2C_impl.cuh); a missing key / plaintext is None
    @staticmethod
    def _ptr_table(arrs):
        T = P64 * max(len(arrs), 1)
        return T(*[(_ptr(a) if a is not None else P64()) for a in arrs])

    @staticmethod
    def _int_table(vals):
        T = C.c_int * max(len(vals), 1)
        return T(*[int(v) for v in vals])

    def cipher_mul_P(self, out, cipher, l):
        self._ck(self.L_.orc_cipher_mul_p(self.h, _ptr(out), _ptr(cipher), l))

    def cipher_add_T(self, a, b, blocks):
        self._ck(self.L_.orc_cipher_add_t(self.h, _ptr(a), _ptr(b), blocks))

    def rescaleAndEqual_noNTT(self, cipher, l):
        self._ck(self.L_.orc_rescale_coeff(self.h, _ptr(cipher), l))

    def Giant_Rotate_And_Mult_PlaintT(self, bs_cipher_T, PQ_to_T, modUp_QjtoT, rotKeys, rotSlots, plaintextT, accNum, bs, gs, l):
        self._ck(self.L_.orc_giant_rotate_mult_plain_t(self.h, _ptr(bs_cipher_T), _ptr(PQ_to_T), _ptr(modUp_QjtoT), self._ptr_table(rotKeys),
                                                       self._int_table(rotSlots), self._ptr_table(plaintextT), self._int_table(accNum), bs, gs, l))

    def Baby_Rotate(self, output, modUp_QjtoT, inp, rotKeys, rotSlots, l):
        self._ck(self.L_.orc_baby_rotate(self.h, _ptr(output), _ptr(modUp_QjtoT), _ptr(inp), len(rotKeys), self._ptr_table(rotKeys),
                                         self._int_table(rotSlots), l))

    def bsgs_level_23(self, cipher, l, plaintextT, accNum, rot_in, rot_in_keys, rot_out, rot_out_keys, bs, gs):
        self._ck(self.L_.orc_bsgs_level_23(self.h, _ptr(cipher), l, self._ptr_table(plaintextT), self._int_table(accNum), self._int_table(rot_in),
                                           self._ptr_table(rot_in_keys), self._int_table(rot_out), self._ptr_table(rot_out_keys), bs, gs))

    def decode_coeffs(self, mx, scale, slots, l, is_bitrev=False):
        """Context_23::decode_coeffs (Encoder.cuh:113-186): iNTT of limbs 0..l, CRT to the centred integer modulo q_0..q_l
        (Python integers for NTL::ZZ), divided by the scale; only coefficients j*gap and N/2 + j*gap, j < slots, are
        produced (the rest stay 0); with is_bitrev the value goes to the bit-reversed index times 256 (:171-173)."""
        from fractions import Fraction
        N, K = self.N, self.K
        buf = np.array(mx[: (l + 1) * N], dtype=np.uint64, copy=True)
        full = np.zeros((self.L + 1) * N, dtype=np.uint64)
        full[: (l + 1) * N] = buf
        self.FromNTTInplace(full, 0, K, 1, l + 1, self.L + 1)
        qs = [int(v) for v in self.q[: l + 1]]
        Q = 1
        for q in qs:
            Q *= q
        rec = [(Q // q) * pow(Q // q, -1, q) for q in qs]
        out = np.zeros(N, dtype=np.float64)
        gap = (N // 2) // slots
        sc = Fraction(scale)
        logN = self.logN
        for j in range(slots):
            for idx in (j * gap, N // 2 + j * gap):
                x = sum(int(full[k * N + idx]) * rec[k] for k in range(l + 1)) % Q
                c = x if x <= Q // 2 else x - Q
                v = float(Fraction(c) / sc)
                if is_bitrev:
                    out[int(format(idx, "0%db" % logN)[::-1], 2)] = v * 256
                else:
                    out[idx] = v
        return out


class OraclePCMM:
    """Mirror of PCMM_Context + the PPMM / rlweCipherDecompose members of PCMM_Scheme on host arrays."""

    def __init__(self, ctx, N1, rank, p_ringpack, q_ringpack):
        self.ctx, self.N1, self.rank = ctx, N1, rank
        self.p_ringpack, self.q_ringpack = list(p_ringpack), list(q_ringpack)
        pa, qa = _arr(p_ringpack), _arr(q_ringpack)
        self.L_ = lib()
        self.h = self.L_.orc_pcmm_create(ctx.h, N1, rank, _ptr(pa), len(pa), _ptr(qa), len(qa))

    def __del__(self):
        try:
            self.L_.orc_pcmm_destroy(self.h)
        except Exception:
            pass

    def _ptrs(self, arrs):
        T = P64 * len(arrs)
        return T(*[_ptr(a) for a in arrs])

    def rlweCipherDecompose(self, rlwe_coeff, mlwe, l):
        rc = self.L_.orc_rlwe_decompose(self.h, _ptr(rlwe_coeff), self._ptrs(mlwe), len(mlwe), l)
        if rc:
            raise ValueError("orc_rlwe_decompose: %d" % rc)

    def ToNTTInplace(self, data, poly_num, mod_num, start_poly_idx, start_mod_idx, mod_batch_size):
        """PCMM_Context.cuh:243-258 on a host array [mod_batch_size][mod_num][poly_num][N1]."""
        if self.L_.orc_pcmm_ntt(self.h, _ptr(data), poly_num, mod_num, start_mod_idx, mod_batch_size, 0):
            raise ValueError("orc_pcmm_ntt")

    def FromNTTInplace(self, data, poly_num, mod_num, start_poly_idx, start_mod_idx, mod_batch_size):
        if self.L_.orc_pcmm_ntt(self.h, _ptr(data), poly_num, mod_num, start_mod_idx, mod_batch_size, 1):
            raise ValueError("orc_pcmm_ntt")

    def mlweCipherPacking(self, rlwe_out, mlwe, keys):
        """PCMM_Scheme.cuh:361-425 on host arrays: mlwe list of [(nq-1)][(rank+1)][N1] coefficient-domain arrays, keys
        [rank][2][mod_num][N] (NTT domain); writes limbs 0..nq-2 of both polynomials of rlwe_out ([2][L+1][N], NTT domain)."""
        rc = self.L_.orc_mlwe_pack(self.h, _ptr(rlwe_out), self._ptrs(mlwe), len(mlwe), _ptr(keys))
        if rc:
            raise ValueError("orc_mlwe_pack: %d" % rc)

    def convertMLWESKfromRLWESK(self, mlwe_sk, rlwe_sk):
        self.ctx._ck(self.L_.orc_pcmm_convert_mlwe_sk(self.h, _ptr(mlwe_sk), _ptr(rlwe_sk)))

    def addRepakcingKey(self, keys, mlwe_sk, rlwe_sk, random):
        self.ctx._ck(self.L_.orc_pcmm_add_repacking_key(self.h, _ptr(keys), _ptr(mlwe_sk), _ptr(rlwe_sk), _bytes(random)))

    def mlweDecrypt(self, plain, cipher, mlwe_sk, l):
        self.ctx._ck(self.L_.orc_pcmm_mlwe_decrypt(self.h, _ptr(plain), _ptr(cipher), _ptr(mlwe_sk), l))

    def decodeCoeffs(self, plain, scaler, l):
        out = np.zeros(self.N1, dtype=np.float64)
        self.ctx._ck(self.L_.orc_pcmm_decode_coeffs(self.h, out.ctypes.data_as(C.POINTER(C.c_double)), _ptr(plain), int(scaler), l))
        return out

    def PPMM(self, W, mlwe, out, M, Kin, mod_num, scaler, col_begin=0, col_count=None):
        C_ = (self.rank + 1) * self.N1
        if col_count is None:
            col_count = C_
        assert W.dtype == np.float32 and W.flags["C_CONTIGUOUS"]
        rc = self.L_.orc_ppmm(self.h, W.ctypes.data_as(C.POINTER(C.c_float)), self._ptrs(mlwe), _ptr(out), M, Kin,
                              mod_num, float(scaler), col_begin, col_count)
        if rc:
            raise ValueError("orc_ppmm: %d" % rc)
