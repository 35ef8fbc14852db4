"""MI355X (gfx950) implementation of the CKKS arithmetic hot path of haozetao/ckks_llm:
batched RNS NTT/iNTT, RNS basis conversion for key switching, ring-packed PPMM.

The compute lives in hand-written HIP kernels behind a C ABI (include/ckks_hip.h, built to
ckks_llm_amd/lib/libckks_hip.so).  This package is the thin host-side mirror of the reference's
Context_23 / PCMM_Context / PCMM_Scheme interface for that path; it has no CPU fallback.
"""
from ._lib import load_library, LibraryMissing  # noqa: F401
from .api import (Context_23, PCMM_Context, PCMM_Scheme, DeviceBuffer, CkksError, Scheme_23, SecretKey, Key,  # noqa: F401
                  Plaintext, Ciphertext, Key_decomp, MLWESecretKey, MLWEPlaintext, MLWECiphertext, PlaintextT, EncodingMatrix, Bert_model_weights, Bert)
from .precision import GetPrecisionStats, PrecisionStats, Stats  # noqa: F401
