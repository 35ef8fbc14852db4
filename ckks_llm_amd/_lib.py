"""ctypes loader of the HIP library.  Fails loudly when the library is missing: there is no fallback path."""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libckks_hip.so")
CSRC = os.path.join(_HERE, "csrc")


class LibraryMissing(RuntimeError):
    pass


def build_library(force=True, jobs=8):
    """Compiles every HIP source for gfx950 (hipcc cross-compiles without a GPU)."""
    import subprocess
    cmd = ["make", "-C", CSRC, "-j%d" % jobs]
    if force:
        cmd.append("-B")
    subprocess.check_call(cmd)
    return LIB_PATH


_lib = None
u64p = C.POINTER(C.c_uint64)
vp = C.c_void_p


def _declare(L):
    i, l, d, sz = C.c_int, C.c_long, C.c_double, C.c_size_t
    S = {
        "ckks_last_error": (C.c_char_p, []), "ckks_version": (C.c_char_p, []),
        "ckks_malloc": (i, [C.POINTER(vp), sz]), "ckks_free": (i, [vp]),
        "ckks_memcpy_h2d": (i, [vp, vp, sz]), "ckks_memcpy_d2h": (i, [vp, vp, sz]), "ckks_memcpy_d2d": (i, [vp, vp, sz]),
        "ckks_memset": (i, [vp, i, sz]), "ckks_sync": (i, []), "ckks_device_count": (i, [C.POINTER(i)]),
        "ckks_measure_mfma_i8_peak": (i, [vp, C.POINTER(d)]),
        "ckks_timer_start": (i, [vp]), "ckks_timer_stop": (i, [vp, C.POINTER(C.c_float)]),
        "ckks_timer_mark": (i, [vp, i]), "ckks_timer_between": (i, [vp, i, i, C.POINTER(C.c_float)]),
        "ckks_ctx_create": (i, [C.POINTER(vp), i, u64p, i, u64p, i, u64p, i, i]), "ckks_ctx_destroy": (i, [vp]),
        "ckks_set_stream": (i, [vp, vp]), "ckks_ctx_info": (i, [vp, C.c_char_p, C.POINTER(l)]),
        "ckks_ctx_set_arith_mode": (i, [vp, i]), "ckks_ctx_set_ntt_mode": (i, [vp, i]), "ckks_ctx_check": (i, [vp]), "ckks_ctx_set_ntt_chain": (i, [vp, i, i]),
        "ckks_ctx_set_option": (i, [vp, C.c_char_p, l]), "pcmm_set_option": (i, [vp, C.c_char_p, l]),
        "ckks_ctx_table": (i, [vp, C.c_char_p, u64p, sz, C.POINTER(sz)]),
        "ckks_ntt_fwd": (i, [vp, vp, i, i, i, i, i]), "ckks_ntt_inv": (i, [vp, vp, i, i, i, i, i]),
        "ckks_ntt_timed": (i, [vp, vp, i, i, i, i, i, i, C.POINTER(C.c_float), C.POINTER(C.c_float)]),
        "ckks_ntt_chain_slot": (i, [C.c_uint, C.c_uint, C.c_uint, C.POINTER(C.c_uint), C.POINTER(C.c_uint), C.POINTER(C.c_uint)]),
        "ckks_ntt_chain_slots": (C.c_uint, [C.c_uint, C.c_uint, C.c_uint]),
        "ckks_ntt_noalloc": (i, [vp, vp, i, i, i, i, i, i]), "ckks_ntt_noalloc_max_limbs": (i, []),
        "ckks_ntt_fwd_ext": (i, [vp, vp, i, i, i, i, i, i, i]), "ckks_ntt_inv_ext": (i, [vp, vp, i, i, i, i, i, i, i]),
        "ckks_modup_pq_to_t": (i, [vp, vp, vp, i, i]), "ckks_modup_qj_to_t": (i, [vp, vp, vp, i, i]),
        "ckks_modup_t_to_pql": (i, [vp, vp, vp, i, i]), "ckks_moddown_pql_to_ql": (i, [vp, vp, vp, i, i]),
        "ckks_external_product_t": (i, [vp, vp, vp, vp, i]), "ckks_external_product_t_swk_reuse": (i, [vp, vp, vp, vp, i, i]), "ckks_rescale": (i, [vp, vp, vp, i]),
        "ckks_keyswitch_23": (i, [vp, vp, vp, vp, i, vp, vp, vp]),
        "ckks_hybrid_modup": (i, [vp, vp, vp, i]), "ckks_hybrid_inner_product": (i, [vp, vp, vp, vp, i]),
        "ckks_hybrid_moddown": (i, [vp, vp, vp, i]), "ckks_hybrid_keyswitch": (i, [vp, vp, vp, vp, i, vp]),
        "ckks_random_bytes": (i, [vp, vp, sz, C.c_char_p, C.c_uint64]),
        "ckks_sample_uniform": (i, [vp, vp, vp, i, i, i]), "ckks_sample_gaussian": (i, [vp, vp, vp, i, i, i]),
        "ckks_sample_zo": (i, [vp, vp, vp, d, i, i, i]), "ckks_sample_hwt": (i, [vp, vp, vp, i, i, i, i]),
        "ckks_poly_mul": (i, [vp, vp, vp, vp, i, i, i, i, i]), "ckks_poly_add": (i, [vp, vp, vp, vp, i, i, i, i, i]),
        "ckks_poly_sub": (i, [vp, vp, vp, vp, i, i, i, i, i]),
        "ckks_keygen_secret": (i, [vp, vp, vp, i]), "ckks_keygen_public": (i, [vp, vp, vp, vp, vp]),
        "ckks_encrypt": (i, [vp, vp, vp, vp, vp, vp, i]), "ckks_decrypt": (i, [vp, vp, vp, vp, i]),
        "ckks_encode_coeffs": (i, [vp, vp, vp, l, i]), "ckks_decode_coeffs": (i, [vp, vp, vp, vp, d, i, i, i]),
        "ckks_rot_group": (i, [vp, l, u64p]),
        "ckks_poly_automorph_ntt": (i, [vp, vp, vp, C.c_uint64, i, i, i]), "ckks_poly_conjugate_ntt": (i, [vp, vp, vp, i, i, i]),
        "ckks_keygen_switch_23": (i, [vp, vp, vp, vp, vp, vp, vp]),
        "ckks_mult_23": (i, [vp, vp, vp, vp, vp, i, vp, vp, vp, vp]),
        "ckks_rotate_23": (i, [vp, vp, vp, vp, l, i, vp, vp, vp, vp]),
        "ckks_conjugate_23": (i, [vp, vp, vp, vp, i, vp, vp, vp, vp]),
        "ckks_cipher_mul_p": (i, [vp, vp, vp, i]), "ckks_cipher_add_t": (i, [vp, vp, vp, i]), "ckks_rescale_coeff": (i, [vp, vp, i]),
        "ckks_giant_rotate_mult_plain_t": (i, [vp, vp, vp, vp, C.POINTER(vp), C.POINTER(i), C.POINTER(vp), C.POINTER(i), i, i, i]),
        "ckks_baby_rotate": (i, [vp, vp, vp, vp, i, C.POINTER(vp), C.POINTER(i), i]),
        "ckks_bsgs_scratch_words": (i, [vp, i, C.POINTER(sz)]),
        "ckks_bsgs_level_23": (i, [vp, vp, i, C.POINTER(vp), C.POINTER(i), C.POINTER(i), C.POINTER(vp), C.POINTER(i), C.POINTER(vp), i, i, vp]),
        "pcmm_ctx_create": (i, [C.POINTER(vp), vp, i, i, u64p, i, u64p, i]), "pcmm_ctx_destroy": (i, [vp]),
        "pcmm_info": (i, [vp, C.c_char_p, C.POINTER(l)]),
        "pcmm_rlwe_decompose": (i, [vp, vp, C.POINTER(vp), i, i]),
        "pcmm_rlwe_decompose_ntt": (i, [vp, vp, C.POINTER(vp), i, i]),
        "pcmm_mlwe_pack": (i, [vp, vp, C.POINTER(vp), i, vp, vp, vp]),
        "pcmm_ntt_fwd": (i, [vp, vp, i, i, i, i, i]), "pcmm_ntt_inv": (i, [vp, vp, i, i, i, i, i]),
        "pcmm_convert_mlwe_sk": (i, [vp, vp, vp]),
        "pcmm_add_repacking_key": (i, [vp, vp, vp, vp, C.c_char_p, C.c_uint64, vp]),
        "pcmm_mlwe_decrypt": (i, [vp, vp, vp, vp, i]),
        "pcmm_decode_coeffs": (i, [vp, vp, vp, vp, C.c_longlong, i]),
        "pcmm_packed_begin": (i, [vp, i, i]), "pcmm_rlwe_decompose_packed": (i, [vp, vp, i, i, i, i]),
        "pcmm_ppmm_packed": (i, [vp, vp, vp, i, d]),
        "pcmm_ppmm": (i, [vp, vp, C.POINTER(vp), vp, i, i, i, d]),
        "pcmm_ppmm_strided": (i, [vp, vp, vp, vp, i, i, i, d]),
        "pcmm_set_weight_cache": (i, [vp, i]), "pcmm_weights_static": (i, [vp, vp, sz, i]),
        "pcmm_weights_changed": (i, [vp, vp]),
    }
    missing = []
    for name, (res, args) in S.items():
        try:
            f = getattr(L, name)
        except AttributeError:
            missing.append(name)
            continue
        f.restype, f.argtypes = res, args
    return missing


EXPORTS = None


def load_library():
    """Returns the loaded library; raises LibraryMissing if it was not built (run __graft_entry__.build())."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise LibraryMissing("HIP library not built: %s (run `python -c 'import __graft_entry__ as g; g.build()'`)" % LIB_PATH)
        L = C.CDLL(LIB_PATH)
        missing = _declare(L)
        if missing:
            raise LibraryMissing("libckks_hip.so lacks symbols: %s" % ", ".join(missing))
        _lib = L
    return _lib
