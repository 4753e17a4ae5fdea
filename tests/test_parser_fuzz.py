"""Property tests of the safetensors parser (csrc/mxp_ckpt.cpp): whatever bytes a file holds,
opening it either succeeds with self-consistent entries or fails with a classified error
(gds_loader.py:254-262 are the reference's rejection rules) - never a crash, never an entry
that points outside the file."""

import json
import struct

import pytest
from hypothesis import HealthCheck, given, settings
from hypothesis import strategies as st

from modelexpress_amd._lib import ERR_FORMAT, ERR_IO, ERR_UNSUPPORTED, MxpError
from modelexpress_amd.engine import Checkpoint

DTYPES = ["F64", "F32", "F16", "BF16", "F8_E4M3", "F8_E5M2", "I64", "I32", "I16", "I8", "U8", "BOOL", "F4", "", "bf16"]
SIZES = {"F64": 8, "F32": 4, "F16": 2, "BF16": 2, "F8_E4M3": 1, "F8_E5M2": 1, "I64": 8, "I32": 4, "I16": 2, "I8": 1, "U8": 1, "BOOL": 1}

entry = st.fixed_dictionaries({
    "dtype": st.sampled_from(DTYPES),
    "shape": st.lists(st.integers(-1, 70), max_size=5),
    "data_offsets": st.one_of(st.lists(st.integers(-5, 5000), min_size=0, max_size=3),
                              st.tuples(st.integers(0, 400), st.integers(0, 400)).map(list)),
})
header = st.dictionaries(st.text(st.characters(min_codepoint=32, max_codepoint=0x24F), max_size=12), entry, max_size=6)


def _check(path):
    try:
        ck = Checkpoint(str(path))
    except MxpError as e:
        assert e.code in (ERR_FORMAT, ERR_IO, ERR_UNSUPPORTED), e
        return None
    size = path.stat().st_size
    for t in ck.tensors():
        n = SIZES[t.dtype]
        for d in t.shape:
            n *= d
        assert t.nbytes == n and t.file_offset >= 8 and t.file_offset + t.nbytes <= size, t
    ck.close()
    return True


@settings(max_examples=300, deadline=None, suppress_health_check=[HealthCheck.function_scoped_fixture])
@given(hdr=header, blob=st.integers(0, 600), pad=st.integers(0, 9), meta=st.booleans())
def test_structured_headers_never_escape_the_file(tmp_path, hdr, blob, pad, meta):
    body = dict(hdr)
    if meta:
        body["__metadata__"] = {"format": "pt"}
    raw = json.dumps(body).encode() + b" " * pad
    p = tmp_path / "model.safetensors"
    p.write_bytes(struct.pack("<Q", len(raw)) + raw + b"\x5a" * blob)
    _check(p)


@settings(max_examples=300, deadline=None, suppress_health_check=[HealthCheck.function_scoped_fixture])
@given(data=st.binary(max_size=300), claimed=st.one_of(st.none(), st.integers(0, 2 ** 64 - 1)))
def test_arbitrary_bytes_are_classified(tmp_path, data, claimed):
    p = tmp_path / "model.safetensors"
    p.write_bytes((struct.pack("<Q", claimed) if claimed is not None else b"") + data)
    _check(p)


@settings(max_examples=150, deadline=None, suppress_health_check=[HealthCheck.function_scoped_fixture])
@given(cut=st.integers(0, 400), flip=st.integers(0, 399), bit=st.integers(0, 7))
def test_truncations_and_bit_flips_of_a_good_file(tmp_path, cut, flip, bit):
    good = {"a.weight": {"dtype": "BF16", "shape": [4, 8], "data_offsets": [0, 64]},
            "b.bias": {"dtype": "F32", "shape": [8], "data_offsets": [64, 96]}, "__metadata__": {"k": "v"}}
    raw = json.dumps(good).encode()
    blob = bytearray(struct.pack("<Q", len(raw)) + raw + bytes(96))
    p = tmp_path / "model.safetensors"
    p.write_bytes(bytes(blob))
    assert _check(p)
    blob[flip % len(blob)] ^= 1 << bit
    p.write_bytes(bytes(blob[: max(0, len(blob) - cut)]))
    _check(p)
