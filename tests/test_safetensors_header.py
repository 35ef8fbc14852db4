"""The safetensors header parser of the C++ Bert_model_weights mirror (include/ckks_llm_amd_bert.hpp, after Load_bert.cuh:315-343)
against files written by the safetensors package and read back with Python's json: same offsets for every fp32 tensor, nothing
for names that are absent, only contained in another name, or not fp32.  No GPU involved."""
import json
import os
import struct
import subprocess

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
EXE = os.path.join(HERE, "cpp", "test_safetensors_header.bin")


def offsets_by_json(path):
    raw = open(path, "rb").read()
    n = struct.unpack("<Q", raw[:8])[0]
    return {k: v for k, v in json.loads(raw[8:8 + n]).items() if k != "__metadata__"}


@pytest.mark.parametrize("with_metadata", [False, True])
def test_offsets_match_json(tmp_path, with_metadata):
    from safetensors.numpy import save_file
    assert os.path.exists(EXE), "tests/cpp/test_safetensors_header.bin is not built (run __graft_entry__.build())"
    rng = np.random.default_rng(3)
    names = ["bert.embeddings.LayerNorm.beta", "bert.pooler.dense.weight", "cls.predictions.bias"]
    for layer in (0, 1, 10, 11):
        for leaf in ("attention.output.dense.weight", "output.dense.weight", "output.dense.bias", "attention.self.query.weight"):
            names.append("bert.encoder.layer.%d.%s" % (layer, leaf))
    tensors = {n: rng.normal(size=rng.integers(1, 40, rng.integers(1, 3))).astype(np.float32) for n in names}
    tensors["x.bert.encoder.layer.1.output.dense.bias"] = np.ones(5, np.float32)
    tensors["bert.encoder.layer.1.output.dense.bias.more"] = np.ones(6, np.float32)
    tensors["cls.seq_relationship.bias"] = np.ones(2, np.float16)
    tensors["cls.seq_relationship.weight"] = np.ones(4, np.int32)
    tensors["empty"] = np.zeros((0,), np.float32)
    path = str(tmp_path / "model.safetensors")
    save_file(tensors, path, metadata={"format": "pt", "note": "data_offsets"} if with_metadata else None)
    want = offsets_by_json(path)
    ask = list(tensors) + ["bert.encoder.layer.1", "output.dense.bias", "absent", "dtype", "format"]
    out = subprocess.run([EXE, path] + ask, capture_output=True, text=True, timeout=30)
    assert out.returncode == 0, out.stdout + out.stderr
    got = {}
    for line in out.stdout.splitlines():
        f = line.split()
        if len(f) >= 2 and f[0] in ask:
            got[f[0]] = None if f[1] == "none" else [int(f[1]), int(f[2])]
    for name in ask:
        entry = want.get(name)
        expect = entry["data_offsets"] if entry is not None and entry["dtype"] == "F32" else None
        assert got[name] == expect, name
