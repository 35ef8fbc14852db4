"""GPU parity of the C++ host mirror (include/ckks_llm_amd.hpp): runs the test program built from tests/cpp, which calls
the mirror's member functions the way the reference's test programs call the reference's and compares every result with
the CPU oracle bit for bit."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))


def test_cpp_mirror_program_passes():
    exe = os.path.join(HERE, "cpp", "test_cpp_mirror.bin")
    assert os.path.exists(exe), "tests/cpp/test_cpp_mirror.bin is not built (run __graft_entry__.build())"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=100)
    print(r.stdout[-3000:], r.stderr[-2000:])
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-2000:]
    assert "all C++ mirror checks passed" in r.stdout


def test_reference_pcmm_test_program_flow_passes():
    """tests/cpp/test_rlwe_decomp_flow.cpp: the reference's test_rlwe_decomp.cu replayed against the mirror (no oracle involved:
    its check is the program's own comparison with the plain matrix product)."""
    exe = os.path.join(HERE, "cpp", "test_rlwe_decomp_flow.bin")
    assert os.path.exists(exe), "tests/cpp/test_rlwe_decomp_flow.bin is not built (run __graft_entry__.build())"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=100)
    print(r.stdout[-3000:], r.stderr[-2000:])
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-2000:]
    assert "the reference's PCMM test flow passed" in r.stdout


def test_bert_linear_layers_with_safetensors_weights(tmp_path):
    """tests/cpp/test_bert_layer.cpp: a BERT-base `model.safetensors` (layer 0's linear weights at their real shapes, random values,
    written here with the safetensors package - an independent writer of the format) is loaded by the Bert_model_weights mirror and
    the four linear layers of the Bert mirror run on encrypted activations at N = 2^16.  Here: the device copies of the tensors
    equal what was written (position-weighted word sums), names that merely contain a wanted name are not picked up, and a tensor
    that is not fp32 is refused; the program itself checks the decrypted layer outputs against the plain products."""
    import numpy as np
    from safetensors.numpy import save_file
    rng = np.random.default_rng(11)
    pre = "bert.encoder.layer.0."
    shapes = {
        "bert.embeddings.LayerNorm.beta": (768,), "bert.embeddings.LayerNorm.gamma": (768,), "bert.pooler.dense.bias": (768,),
        "cls.predictions.bias": (30522,),
        pre + "attention.self.query.weight": (768, 768), pre + "attention.self.key.weight": (768, 768),
        pre + "attention.self.value.weight": (768, 768), pre + "attention.output.dense.weight": (768, 768),
        pre + "attention.output.dense.bias": (768,), pre + "intermediate.dense.weight": (3072, 768),
        pre + "output.dense.weight": (768, 3072), pre + "output.dense.bias": (768,),
        "bert.encoder.layer.1.output.dense.bias": (768,), "bert.encoder.layer.11.output.dense.bias": (768,),
    }
    tensors = {name: rng.normal(0, 0.02, shape).astype(np.float32) for name, shape in shapes.items()}
    decoys = {
        "a." + pre + "output.dense.bias": np.full(768, 7, np.float32),                 # a wanted name with something in front
        pre + "output.dense.bias.extra": np.full(768, 9, np.float32),                  # ... and with something behind
        "bert.encoder.layer.1.output.dense.bias_v2": np.full(16, 3, np.float32),
        "cls.seq_relationship.bias": np.zeros(2, np.float16),                          # wanted, but not fp32: refused
        "cls.seq_relationship.weight": np.zeros((2, 768), np.int32),                   # wanted, 4-byte words, but not fp32 either
    }
    save_file({**decoys, **tensors}, str(tmp_path / "model.safetensors"), metadata={"format": "pt"})

    def weighted_sum(a):
        w = np.ascontiguousarray(a).view(np.uint32).reshape(-1).astype(np.uint64)
        with np.errstate(over="ignore"):
            return int((w * np.arange(1, w.size + 1, dtype=np.uint64)).sum(dtype=np.uint64))

    exe = os.path.join(HERE, "cpp", "test_bert_layer.bin")
    assert os.path.exists(exe), "tests/cpp/test_bert_layer.bin is not built (run __graft_entry__.build())"
    r = subprocess.run([exe, str(tmp_path) + "/"], capture_output=True, text=True, timeout=280)
    print(r.stdout[-6000:], r.stderr[-2000:])
    assert r.returncode == 0, r.stdout[-6000:] + r.stderr[-2000:]
    assert "the BERT linear layers passed" in r.stdout
    seen = {}
    for line in r.stdout.splitlines():
        f = line.split()
        if f and f[0] == "tensor":
            seen[f[1]] = None if f[2] == "absent" else (int(f[2]), int(f[3], 16))
    for name, a in tensors.items():
        assert seen[name] == (a.nbytes, weighted_sum(a)), name
    assert seen["cls.seq_relationship.bias"] is None and seen["cls.seq_relationship.weight"] is None
    assert "loaded %d missing %d" % (len(tensors), 14 + 16 * 12 - len(tensors)) in r.stdout
