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


def build(force=False):
    if force or not os.path.exists(_SO):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "libckks_oracle.so"])
    return _SO


def _ptr(a):
    assert a.dtype == np.uint64 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(P64)


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
            "orc_external_product_t": (i, [vp, P64, P64, P64, i]), "orc_rescale": (i, [vp, P64, i]),
            "orc_keyswitch_23": (i, [vp, P64, P64, P64, i]),
            "orc_hybrid_modup": (i, [vp, P64, P64, i]), "orc_hybrid_inner_product": (i, [vp, P64, P64, P64, i]),
            "orc_hybrid_moddown": (i, [vp, P64, P64, i]), "orc_hybrid_keyswitch": (i, [vp, P64, P64, P64, i]),
            "orc_pcmm_create": (vp, [vp, i, i, P64, i, P64, i]), "orc_pcmm_destroy": (None, [vp]),
            "orc_rlwe_decompose": (i, [vp, P64, C.POINTER(P64), i, i]),
            "orc_ppmm": (i, [vp, C.POINTER(C.c_float), C.POINTER(P64), P64, i, i, i, d, l, l]),
            "orc_mlwe_pack": (i, [vp, P64, C.POINTER(P64), i, P64]),
            "orc_pcmm_ntt": (i, [vp, P64, i, i, i, i, i]),
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

    def PPMM(self, W, mlwe, out, M, Kin, mod_num, scaler, col_begin=0, col_count=None):
        C_ = (self.rank + 1) * self.N1
        if col_count is None:
            col_count = C_
        assert W.dtype == np.float32 and W.flags["C_CONTIGUOUS"]
        rc = self.L_.orc_ppmm(self.h, W.ctypes.data_as(C.POINTER(C.c_float)), self._ptrs(mlwe), _ptr(out), M, Kin,
                              mod_num, float(scaler), col_begin, col_count)
        if rc:
            raise ValueError("orc_ppmm: %d" % rc)
