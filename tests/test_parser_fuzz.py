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


def _write(path, header: dict, blob: int):
    raw = json.dumps(header).encode()
    path.write_bytes(struct.pack("<Q", len(raw)) + raw + bytes(blob))


def test_shape_products_that_wrap_are_rejected(tmp_path):
    """[2^32, 2^32] multiplies to 0 mod 2^64: it must not pass for an empty tensor."""
    p = tmp_path / "model.safetensors"
    _write(p, {"w": {"dtype": "U8", "shape": [1 << 32, 1 << 32], "data_offsets": [0, 0]}}, 16)
    with pytest.raises(MxpError) as e:
        Checkpoint(str(p))
    assert e.value.code == ERR_FORMAT and "overflows" in e.value.message
    _write(p, {"w": {"dtype": "F64", "shape": [1 << 61], "data_offsets": [0, 0]}}, 16)  # numel fits, bytes do not
    with pytest.raises(MxpError) as e:
        Checkpoint(str(p))
    assert e.value.code == ERR_FORMAT and "overflows" in e.value.message


def test_parameter_sizes_that_wrap_are_rejected(tmp_path):
    from modelexpress_amd._lib import ERR_ARG
    from modelexpress_amd.engine import PlacementPlan

    p = tmp_path / "model.safetensors"
    _write(p, {"w": {"dtype": "U8", "shape": [4], "data_offsets": [0, 4]}}, 4)
    with Checkpoint(str(p)) as ck:
        for shape in ((1 << 32, 1 << 32), (1 << 62,)):
            with pytest.raises(MxpError) as e:
                PlacementPlan(ck, [_Spec("w", "U8", shape)])
            assert e.value.code == ERR_ARG and "overflows" in e.value.message


class _Spec:
    """A parameter row whose byte count Python does not pre-compute."""

    def __init__(self, name, dtype, shape):
        self.name, self.dtype, self.shape = name, dtype, shape


def test_overlapping_tensors_are_rejected(tmp_path):
    p = tmp_path / "model.safetensors"
    _write(p, {"a": {"dtype": "U8", "shape": [8], "data_offsets": [0, 8]},
               "b": {"dtype": "U8", "shape": [8], "data_offsets": [4, 12]}}, 12)
    with pytest.raises(MxpError) as e:
        Checkpoint(str(p))
    assert e.value.code == ERR_FORMAT and "overlap" in e.value.message
    # empty tensors share an offset with their neighbour without sharing bytes
    _write(p, {"a": {"dtype": "U8", "shape": [8], "data_offsets": [0, 8]},
               "e": {"dtype": "F32", "shape": [0, 4], "data_offsets": [4, 4]},
               "b": {"dtype": "U8", "shape": [4], "data_offsets": [8, 12]}}, 12)
    with Checkpoint(str(p)) as ck:
        assert len(ck) == 3


def test_index_names_missing_from_their_shard_fail_the_open(tmp_path):
    """gds_loader.py:297-313 looks every indexed name up in its shard's header: a missing one is an
    error there (KeyError), not a silently shorter checkpoint."""
    _write(tmp_path / "s0.safetensors", {"a": {"dtype": "U8", "shape": [4], "data_offsets": [0, 4]}}, 4)
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps(
        {"weight_map": {"a": "s0.safetensors", "ghost": "s0.safetensors"}}))
    with pytest.raises(MxpError) as e:
        Checkpoint(str(tmp_path))
    assert e.value.code == ERR_FORMAT and "ghost" in e.value.message
