"""Committed golden vectors (tests/golden/vectors.json, made by tests/golden/make_vectors.py
without the oracle or the product) against the oracle on the host and the HIP path on the GPU."""

import json
from pathlib import Path

import numpy as np
import pytest

from golden.make_vectors import lcg_bytes

VEC = json.loads((Path(__file__).parent / "golden" / "vectors.json").read_text())


# (fixture key, source field, destination field, oracle function, MXP_CAST_* code, source dtype, destination dtype)
_CASTS = [("cast_f32_f16", "f32_bits", "f16_bits", "cast_f32_f16_bits", 4),
          ("cast_f16_f32", "f16_bits", "f32_bits", "cast_f16_f32_bits", 3),
          ("cast_bf16_f32", "bf16_bits", "f32_bits", "cast_bf16_f32_bits", 2),
          ("cast_f8e4m3_bf16", "f8_bits", "bf16_bits", "cast_f8e4m3_bf16_bits", 5),
          ("cast_f16_bf16", "f16_bits", "bf16_bits", None, 6), ("cast_bf16_f16", "bf16_bits", "f16_bits", None, 7)]
_DTYPES = {4: ("F32", "F16"), 3: ("F16", "F32"), 2: ("BF16", "F32"), 5: ("F8_E4M3", "BF16"), 6: ("F16", "BF16"), 7: ("BF16", "F16")}
_NP = {"f32_bits": np.uint32, "f16_bits": np.uint16, "bf16_bits": np.uint16, "f8_bits": np.uint8}


def test_oracle_matches_golden_vectors(oracle, oracle_c):
    for v in VEC["checksum"]:
        raw = lcg_bytes(v["seed"], v["n"])
        if v["hex"] is not None:
            assert raw.hex() == v["hex"]
        assert oracle.safe_checksum_bytes(raw) == v["checksum"]
        assert oracle_c.checksum32(np.frombuffer(raw, dtype=np.uint8)) == v["checksum"]
    for v in VEC["digest"]:
        raw = lcg_bytes(v["seed"], v["n"])
        sc = [x & ((1 << 64) - 1) for x in oracle.tensor_digest_scalars(raw)]
        assert [str(x) for x in sc] == v["scalars"]
        assert oracle.tensor_digest_bytes(raw) == v["digest"]
    bits = np.array(VEC["cast"]["f32_bits"], dtype=np.uint32)
    want = np.array(VEC["cast"]["bf16_bits"], dtype=np.uint16)
    assert np.array_equal(oracle.cast_f32_bf16_bits(bits), want)
    assert np.array_equal(oracle_c.cast_f32_bf16(bits), want)
    for key, src_k, dst_k, fn, code in _CASTS:
        src = np.array(VEC[key][src_k], dtype=_NP[src_k])
        want = np.array(VEC[key][dst_k], dtype=_NP[dst_k])
        if fn is None:  # the recoding pairs are compositions in the oracle
            got = oracle.cast_tensor(oracle.OTensor.from_array(src, _DTYPES[code][0]), _DTYPES[code][1]).data.reshape(-1).view("<u2")
        else:
            got = getattr(oracle, fn)(src)
        assert np.array_equal(got, want), key
        assert np.array_equal(oracle_c.cast(code, src), want), key


@pytest.mark.gpu
def test_hip_path_matches_golden_vectors(gpu_engine):
    import torch

    def dev(raw):
        return torch.from_numpy(np.frombuffer(raw, dtype=np.uint8).copy()).cuda() if raw else \
            torch.empty(0, dtype=torch.uint8, device="cuda")

    bufs = [dev(lcg_bytes(v["seed"], v["n"])) for v in VEC["checksum"]]
    assert gpu_engine.checksum32(bufs) == [v["checksum"] for v in VEC["checksum"]]
    assert gpu_engine.digest(bufs) == [v["digest"] for v in VEC["digest"]]
    bits = np.array(VEC["cast"]["f32_bits"], dtype=np.uint32)
    want = np.array(VEC["cast"]["bf16_bits"], dtype=np.uint16)
    src = torch.from_numpy(bits.view(np.uint8).copy()).cuda()
    dst = torch.zeros(bits.size * 2, dtype=torch.uint8, device="cuda")
    gpu_engine.cast_f32_bf16(src, dst, bits.size)
    assert np.array_equal(dst.cpu().numpy().view(np.uint16), want)
    for key, src_k, dst_k, _fn, code in _CASTS:
        src = np.array(VEC[key][src_k], dtype=_NP[src_k])
        want = np.array(VEC[key][dst_k], dtype=_NP[dst_k])
        d_src = torch.from_numpy(src.view(np.uint8).copy()).cuda()
        d_dst = torch.zeros(want.nbytes, dtype=torch.uint8, device="cuda")
        gpu_engine.cast(d_src, d_dst, src.size, *_DTYPES[code])
        assert np.array_equal(d_dst.cpu().numpy().view(want.dtype), want), key
