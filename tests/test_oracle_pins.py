"""Pins the CPU oracle (oracle/) before anything is compared against it.

Every check here is independent of the oracle's own code path: vectors asserted by the
reference's tests (cited per test, paths under modelexpress_client/python/tests/),
closed forms, brute force from the defining formula, or a third-party library the
reference itself calls (hashlib.blake2b, torch's CPU cast, the safetensors reader).
"""

import hashlib
import json
import struct

import numpy as np
import pytest
import torch

K = 2654435761
M32 = 0xFFFFFFFF


# ---------------------------------------------------------------- safe_checksum ------
def test_checksum_hand_values(oracle):
    # [1,255]: 1*1 + 255*(K+1) mod 2^32, worked by hand = 0x9942384f
    assert (1 * 1 + 255 * ((K + 1) & M32)) & M32 == 0x9942384F
    assert oracle.safe_checksum_bytes(bytes([1, 255])) == "9942384f"
    assert oracle.safe_checksum_bytes(bytes([255, 1])) == format((255 + ((K + 1) & M32)) & M32, "08x")
    assert oracle.safe_checksum_bytes(b"") == "00000000"
    assert oracle.safe_checksum_bytes(bytes([7])) == "00000007"  # weight of index 0 is 1


def test_checksum_constant_buffer_closed_form(oracle, oracle_c):
    # all bytes = c: c * (K * n(n-1)/2 + n) mod 2^32
    for c, n in [(1, 10), (255, 4097), (17, 100003), (128, 1 << 20)]:
        want = (c * (K * (n * (n - 1) // 2) + n)) & M32
        buf = np.full(n, c, dtype=np.uint8)
        assert oracle.safe_checksum_bytes(buf) == format(want, "08x")
        assert oracle_c.checksum32(buf) == format(want, "08x")


def test_checksum_bigint_brute_force_matches_vectorised_and_c(oracle, oracle_c):
    rng = np.random.default_rng(1)
    for n in [1, 2, 3, 15, 16, 17, 255, 1024, 4095]:
        buf = rng.integers(0, 256, n, dtype=np.uint8)
        want = oracle.safe_checksum_bigint(buf.tobytes())
        assert oracle.safe_checksum_bytes(buf) == want
        assert oracle_c.checksum32(buf) == want


def test_checksum_properties_from_reference_tests(oracle):
    # tests/test_tensor_utils.py:255-284: 8 hex chars; order and compensating changes matter
    f = oracle.safe_checksum_bytes
    assert len(f(bytes(range(32)))) == 8 and int(f(bytes(range(32))), 16) >= 0
    assert f(bytes([1, 255])) != f(bytes([255, 1]))
    assert f(bytes([10, 20, 30])) != f(bytes([11, 19, 30]))
    assert f(np.arange(10, dtype=np.float32).tobytes()) == f(np.arange(10, dtype=np.float32).tobytes())


def test_checksum_index_wraps_mod_2_32(oracle_c):
    # position 2^32 + j weighs the same as position j: (i*K+1) mod 2^32 depends on i mod 2^32
    rng = np.random.default_rng(2)
    buf = rng.integers(0, 256, 1000, dtype=np.uint8)
    assert oracle_c.checksum32(buf, first_index=(1 << 32) + 5) == oracle_c.checksum32(buf, first_index=5)
    # and splitting a buffer adds up
    whole = int(oracle_c.checksum32(buf), 16)
    parts = int(oracle_c.checksum32(buf[:333]), 16) + int(oracle_c.checksum32(buf[333:], first_index=333), 16)
    assert whole == parts & M32


def test_checksum_reference_literal_mode(oracle):
    # tensor_utils.py:38-44: only 1-D, (1,N) and 0-dim inputs yield a value upstream
    OT = oracle.OTensor
    a = np.arange(8, dtype=np.float32)
    flat = oracle.safe_checksum(OT.from_array(a, "F32"), reference_literal=True)
    assert oracle.safe_checksum(OT.from_array(a.reshape(1, 8), "F32"), reference_literal=True) == flat
    assert oracle.safe_checksum(OT.from_array(a.reshape(4, 2), "F32"), reference_literal=True).startswith("err:")
    assert oracle.safe_checksum(OT.from_array(a.reshape(4, 2), "F32")) == flat  # flat-byte definition


# ---------------------------------------------------------------- tensor_digest ------
def _digest_of_scalars(scalars):
    h = hashlib.blake2b(digest_size=16)
    for v in scalars:
        h.update((v & ((1 << 64) - 1)).to_bytes(8, "little"))
    return h.hexdigest()


def test_digest_scalars_closed_form_arange(oracle, oracle_c):
    # int32 arange(8192): 8 rows of 1024; row r sums to 1024*(1024 r) + 1023*1024/2
    a = np.arange(8192, dtype=np.int32)
    rows = [1024 * 1024 * r + 1023 * 1024 // 2 for r in range(8)]
    want = [8192 * 4, sum(rows), sum(rs * (r + 1) for r, rs in enumerate(rows))]
    assert oracle.tensor_digest_scalars(a.tobytes()) == want
    sc = oracle_c.digest_scalars(a)
    assert [sc[0], sc[1], sc[2]] == want and sc[3:] == [0, 0, 0, 0]
    assert oracle.tensor_digest_bytes(a.tobytes()) == _digest_of_scalars(want)


def test_digest_scalars_tail_and_ragged(oracle, oracle_c):
    # int16[1031] = 2062 bytes: 515 whole words (no full row) + 2 ragged bytes
    a = (np.arange(1031, dtype=np.int32) - 500).astype(np.int16)
    raw = a.tobytes()
    words = np.frombuffer(raw[:2060], dtype="<i4").astype(object)
    want = [2062, int(sum(words)), int(sum(int(w) * (k + 1) for k, w in enumerate(words))), raw[2060] + raw[2061], 2]
    want = [v & ((1 << 64) - 1) for v in want]
    got = [v & ((1 << 64) - 1) for v in oracle.tensor_digest_scalars(raw)]
    assert got == want
    sc = oracle_c.digest_scalars(a)
    assert [sc[0], sc[3], sc[4], sc[5], sc[6]] == want
    # negative words: signed interpretation matters
    neg = np.full(2048, -1, dtype=np.int32)
    assert oracle.tensor_digest_scalars(neg.tobytes()) == [8192, -2048, -1024 * 1 - 1024 * 2]


def test_digest_invariants_from_reference_tests(oracle):
    OT = oracle.OTensor
    d = oracle.tensor_digest
    # tests/test_reshard_refit_verify.py:43-52
    x = np.random.default_rng(0).standard_normal((64, 48)).astype(np.float32)
    assert d(OT.from_array(x, "F32")) == d(OT.from_array(x.copy(), "F32"))
    y = x.copy()
    y[7, 3] += 1
    assert d(OT.from_array(x, "F32")) != d(OT.from_array(y, "F32"))
    # :55-67 swapping two whole 1024-word rows keeps the plain sum, changes the digest
    a = np.arange(8192, dtype=np.int32)
    b = a.copy()
    b[0:1024], b[1024:2048] = a[1024:2048], a[0:1024]
    assert a.sum() == b.sum()
    assert d(OT.from_array(a, "I32")) != d(OT.from_array(b, "I32"))
    # :70-79 ragged tail
    t = np.arange(1031, dtype=np.int16)
    u = t.copy()
    u[-1] += 1
    assert d(OT.from_array(t, "I16")) != d(OT.from_array(u, "I16"))
    # :82-85 strided view == contiguous copy;  :88-108 odd-offset view == clone
    big = OT.from_array(np.arange(4096, dtype=np.uint16).reshape(64, 64), "BF16")
    view = big.narrow(1, 3, 17)
    assert d(view) == d(OT(np.ascontiguousarray(view.data), "BF16"))
    flat = OT.from_array(np.arange(5000, dtype=np.uint16), "BF16")
    assert d(flat.narrow(0, 1409, 2000)) == d(OT(flat.data[1409:3409].copy(), "BF16"))
    assert len(d(flat)) == 32


def test_shard_region_from_reference_tests(oracle):
    # tests/test_reshard_refit_verify.py:135-171
    OT = oracle.OTensor
    full = np.arange(24, dtype=np.float32).reshape(4, 6)
    region = oracle.shard_region(OT.from_array(full.reshape(-1), "F32"), (4, 6), (1, 2), (2, 3))
    assert region.tobytes() == np.ascontiguousarray(full[1:3, 2:5]).tobytes()
    assert oracle.tensor_digest(region) == oracle.tensor_digest(OT.from_array(np.ascontiguousarray(full[1:3, 2:5]), "F32"))
    with pytest.raises(ValueError, match="rank mismatch"):
        oracle.shard_region(OT.from_array(full.reshape(-1), "F32"), (4, 6), (1,), (2, 3))


def test_product_blake2b_matches_hashlib(mxp):
    from modelexpress_amd.engine import digest_from_scalars

    for n, sc in [(5, [5, 0, 0, 9, 9, 3, 1]), (4096, [4096, 11, 22, 0, 0, 0, 0]),
                  (4 * 1024 * 3 + 7, [4 * 1024 * 3 + 7, (1 << 64) - 5, 12345, 77, 88, 600, 3]), (0, [0] * 7)]:
        body_words = n // 4
        rows = body_words // 1024
        lst = [sc[0]]
        if rows:
            lst += sc[1:3]
        if body_words - rows * 1024:
            lst += sc[3:5]
        if n % 4:
            lst += [sc[5], n % 4]
        assert digest_from_scalars(sc) == _digest_of_scalars(lst)


# ---------------------------------------------------------------- cast ---------------
def _torch_bf16_bits(u32: np.ndarray) -> np.ndarray:
    t = torch.from_numpy(u32.astype(np.int64).astype(np.uint32).view(np.int32).copy()).view(torch.float32)
    return t.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)


def test_cast_hand_values(oracle, oracle_c):
    src = np.array([0x00000001, 0x00007FFF, 0x00008000, 0x00008001, 0x00018000, 0x7F7FFFFF, 0x3F808000, 0x3F818000,
                    0x7F800000, 0xFF800000, 0x80000000, 0xFF7FFFFF], dtype=np.uint32)
    want = np.array([0x0000, 0x0000, 0x0000, 0x0001, 0x0002, 0x7F80, 0x3F80, 0x3F82, 0x7F80, 0xFF80, 0x8000, 0xFF80],
                    dtype=np.uint16)
    assert np.array_equal(oracle.cast_f32_bf16_bits(src), want)
    assert np.array_equal(oracle_c.cast_f32_bf16(src), want)


def test_cast_matches_torch_cpu_on_every_rounding_class(oracle, oracle_c):
    hi = np.arange(1 << 16, dtype=np.uint32) << 16
    lows = np.array([0x0000, 0x0001, 0x7FFF, 0x8000, 0x8001, 0xFFFF, 0x1234, 0xC000], dtype=np.uint32)
    u = (hi[:, None] | lows[None, :]).reshape(-1)
    is_nan = (u & 0x7FFFFFFF) > 0x7F800000
    ref = _torch_bf16_bits(u)
    got = oracle.cast_f32_bf16_bits(u)
    assert np.array_equal(got[~is_nan], ref[~is_nan])
    # every NaN stays a NaN in both; torch's image depends on the host ISA, ours is a parameter
    assert np.all((ref[is_nan] & 0x7FFF) > 0x7F80)
    assert np.all(got[is_nan] == 0x7FC0)
    torch_nan = int(ref[is_nan][0])
    if np.all(ref[is_nan] == torch_nan):
        assert np.array_equal(oracle.cast_f32_bf16_bits(u, nan_bits=torch_nan), ref)
        assert np.array_equal(oracle_c.cast_f32_bf16(u, nan_bits=torch_nan), ref)
    rnd = np.random.default_rng(3).integers(0, 1 << 32, 1 << 20, dtype=np.uint64).astype(np.uint32)
    ok = (rnd & 0x7FFFFFFF) <= 0x7F800000
    assert np.array_equal(oracle.cast_f32_bf16_bits(rnd)[ok], _torch_bf16_bits(rnd)[ok])
    assert np.array_equal(oracle_c.cast_f32_bf16(rnd), oracle.cast_f32_bf16_bits(rnd))


def _torch_convert(bits: np.ndarray, src: str, dst: str) -> np.ndarray:
    st = {"F32": (torch.float32, np.int32), "BF16": (torch.bfloat16, np.int16), "F16": (torch.float16, np.int16)}
    ut = {"F32": np.uint32, "BF16": np.uint16, "F16": np.uint16}
    t = torch.from_numpy(bits.view(st[src][1]).copy()).view(st[src][0]).to(st[dst][0])
    return t.view(torch.int32 if dst == "F32" else torch.int16).numpy().view(ut[dst])


def test_widening_casts_match_torch_on_every_pattern(oracle, oracle_c):
    # refit/reshard/receiver.py:962-969: recv (fp32) .copy_(staging (bf16)); torch is the library the reference calls
    h = np.arange(1 << 16, dtype=np.uint16)
    assert np.array_equal(oracle.cast_bf16_f32_bits(h), _torch_convert(h, "BF16", "F32"))
    assert np.array_equal(oracle.cast_f16_f32_bits(h), _torch_convert(h, "F16", "F32"))
    assert np.array_equal(oracle_c.cast(2, h), oracle.cast_bf16_f32_bits(h))
    assert np.array_equal(oracle_c.cast(3, h), oracle.cast_f16_f32_bits(h))
    # hand values: 1.0, -2.0, smallest subnormal half (2^-24), largest subnormal, inf, a signalling NaN made quiet
    hv = np.array([0x3C00, 0xC000, 0x0001, 0x03FF, 0x7C00, 0x7C01], dtype=np.uint16)
    assert oracle.cast_f16_f32_bits(hv).tolist() == [0x3F800000, 0xC0000000, 0x33800000, 0x387FC000, 0x7F800000, 0x7FC02000]
    assert oracle.cast_bf16_f32_bits(np.array([0x3F80, 0x7FC1], dtype=np.uint16)).tolist() == [0x3F800000, 0x7FC10000]
    # exactness: widening then narrowing is the identity on every non-NaN pattern
    not_nan16 = (h & 0x7FFF) <= 0x7C00
    assert np.array_equal(oracle.cast_f32_f16_bits(oracle.cast_f16_f32_bits(h))[not_nan16], h[not_nan16])
    not_nan_bf = (h & 0x7FFF) <= 0x7F80
    assert np.array_equal(oracle.cast_f32_bf16_bits(oracle.cast_bf16_f32_bits(h))[not_nan_bf], h[not_nan_bf])


def test_fp8_e4m3_to_bf16_matches_torch_on_every_code(oracle, oracle_c):
    # engines/vllm/refit/receiver.py:258-261: w_uk.permute(1, 2, 0).to(out_dtype) with an fp8 kv_b_proj
    codes = np.arange(256, dtype=np.uint8)
    ref = torch.from_numpy(codes.copy()).view(torch.float8_e4m3fn).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(oracle.cast_f8e4m3_bf16_bits(codes), ref)
    assert np.array_equal(oracle_c.cast(5, codes), ref)
    # hand values: 1.0 (0x38), -448 (largest), 2^-9 (smallest subnormal), 2^-6 (smallest normal), NaN of either sign
    hv = np.array([0x38, 0xFE, 0x01, 0x08, 0x7F, 0xFF], dtype=np.uint8)
    assert oracle.cast_f8e4m3_bf16_bits(hv).tolist() == [0x3F80, 0xC3E0, 0x3B00, 0x3C80, 0x7FC0, 0x7FC0]


def test_fp16_bf16_recoding_matches_torch_on_every_pattern(oracle, oracle_c):
    # destination.copy_(source) between the two 16-bit formats (installer.py:419-424) goes through fp32
    h = np.arange(1 << 16, dtype=np.uint16)
    OT = oracle.OTensor
    a = oracle.cast_tensor(OT.from_array(h, "F16"), "BF16").data.reshape(-1).view("<u2")
    b = oracle.cast_tensor(OT.from_array(h, "BF16"), "F16").data.reshape(-1).view("<u2")
    assert np.array_equal(a, _torch_convert(h, "F16", "BF16"))  # torch's NaN image here is 0x7FC0, the default
    assert np.array_equal(b, _torch_convert(h, "BF16", "F16"))
    assert np.array_equal(oracle_c.cast(6, h), a) and np.array_equal(oracle_c.cast(7, h), b)
    # hand values: fp16 1.0 -> bf16 1.0; fp16 65504 -> bf16 0x4780 (rounds up to 65536); bf16 1e5 -> fp16 inf
    assert oracle.cast_tensor(OT.from_array(np.array([0x3C00, 0x7BFF], dtype=np.uint16), "F16"), "BF16").data.reshape(-1).view("<u2").tolist() == [0x3F80, 0x4780]
    assert oracle.cast_tensor(OT.from_array(np.array([0x47C3], dtype=np.uint16), "BF16"), "F16").data.reshape(-1).view("<u2").tolist() == [0x7C00]


def test_f32_to_f16_matches_torch_and_numpy(oracle, oracle_c):
    hi = np.arange(1 << 16, dtype=np.uint32) << 16
    lows = np.array([0, 1, 0x0FFF, 0x1000, 0x1001, 0x1FFF, 0x2000, 0x2FFF, 0x3000, 0x7FFF, 0x8000, 0x8001, 0xFFFF],
                    dtype=np.uint32)
    u = (hi[:, None] | lows[None, :]).reshape(-1)
    u = np.concatenate([u, np.random.default_rng(4).integers(0, 1 << 32, 1 << 21, dtype=np.uint64).astype(np.uint32)])
    got = oracle.cast_f32_f16_bits(u)
    assert np.array_equal(got, _torch_convert(u, "F32", "F16"))  # NaN payload rule included
    not_nan = (u & 0x7FFFFFFF) <= 0x7F800000
    with np.errstate(over="ignore"):
        assert np.array_equal(got[not_nan], u.view(np.float32).astype(np.float16).view(np.uint16)[not_nan])
    assert np.array_equal(oracle_c.cast(4, u), got)
    # hand values: 1.0; 65504 (max half); 65520 -> inf (tie to even overflows); 2^-25 -> 0 (tie to even);
    # just above 2^-25 -> smallest subnormal; 2^-14 (smallest normal); -0.0
    hv = np.array([0x3F800000, 0x477FE000, 0x477FF000, 0x33000000, 0x33000001, 0x38800000, 0x80000000], dtype=np.uint32)
    assert oracle.cast_f32_f16_bits(hv).tolist() == [0x3C00, 0x7BFF, 0x7C00, 0x0000, 0x0001, 0x0400, 0x8000]


# ---------------------------------------------------------------- paired_runs --------
def test_paired_runs_reference_vectors(oracle):
    # tests/test_reshard_refit_slice_plan.py:54-65: narrow(1,0,4) of (4,8) into (4,4)
    runs = list(oracle.paired_runs([(0, 4), (0, 4)], (0, 0), [8, 1], (0, 0), [4, 1]))
    assert [r[0] for r in runs] == [0, 8, 16, 24]
    assert [r[1] for r in runs] == [0, 4, 8, 12]
    assert all(r[2] == 4 for r in runs)
    # :82-96 two column-half shards fanning into (4,8)
    left = list(oracle.paired_runs([(0, 4), (0, 4)], (0, 0), [4, 1], (0, 0), [8, 1]))
    right = list(oracle.paired_runs([(0, 4), (4, 8)], (0, 4), [4, 1], (0, 0), [8, 1]))
    assert [r[1] for r in left] == [0, 8, 16, 24]
    assert [r[1] for r in right] == [4, 12, 20, 28]
    # fully contiguous overlap: one run
    assert list(oracle.paired_runs([(2, 4), (0, 8)], (0, 0), [8, 1], (2, 0), [8, 1])) == [(16, 0, 16)]


@pytest.mark.parametrize("tp_size,tp_rank,expected_bytes,expected_segments", [(2, 1, 272, 3), (4, 2, 144, 10)])
def test_paired_runs_megatron_target_vectors(oracle, tp_size, tp_rank, expected_bytes, expected_segments):
    """tests/test_reshard_megatron.py:30-113: bf16 sources published by two trainer ranks - expert_fc1 (16, 8)
    split on rows, expert_fc2 (8, 16) split on columns, a replicated norm (8,) - pulled by a TP rank that owns
    rows / columns / everything.  The reference expects 272 bytes in 3 segments (TP 2, rank 1) and 144 bytes in
    10 segments (TP 4, rank 2): every (destination box x source shard) intersection decomposed into runs."""
    sources = {"expert_fc1": ((16, 8), [((0, 0), (8, 8)), ((8, 0), (8, 8))]),
               "expert_fc2": ((8, 16), [((0, 0), (8, 8)), ((0, 8), (8, 8))]),
               "norm": ((8,), [((0,), (8,))])}
    wanted = {"expert_fc1": 0, "expert_fc2": 1, "norm": None}  # the axis the destination rank owns a slice of
    n_bytes = n_segments = 0
    for name, (shape, shards) in sources.items():
        axis = wanted[name]
        dst_box = [(0, n) for n in shape]
        if axis is not None:
            per = shape[axis] // tp_size
            dst_box[axis] = (tp_rank * per, (tp_rank + 1) * per)
        dst_shape = [hi - lo for lo, hi in dst_box]
        for off, sshape in shards:
            src_box = [(o, o + n) for o, n in zip(off, sshape)]
            overlap = oracle.intersect(dst_box, src_box)
            if overlap is None:
                continue
            for _s, _d, run in oracle.paired_runs(overlap, off, oracle.row_major_strides(sshape), [lo for lo, _ in dst_box],
                                                  oracle.row_major_strides(dst_shape)):
                n_bytes += run * 2
                n_segments += 1
    assert (n_bytes, n_segments) == (expected_bytes, expected_segments)


def test_paired_runs_brute_force(oracle):
    rng = np.random.default_rng(4)
    for _ in range(50):
        shape = tuple(int(v) for v in rng.integers(1, 6, 3))
        lo = [int(rng.integers(0, s)) for s in shape]
        hi = [int(rng.integers(l + 1, s + 1)) for l, s in zip(lo, shape)]
        src = np.arange(np.prod(shape)).reshape(shape)
        box = tuple(slice(l, h) for l, h in zip(lo, hi))
        dst_shape = tuple(h - l for l, h in zip(lo, hi))
        dst = np.full(int(np.prod(dst_shape)), -1)
        for s_off, d_off, n in oracle.paired_runs(list(zip(lo, hi)), (0, 0, 0), oracle.row_major_strides(shape), lo,
                                                  oracle.row_major_strides(dst_shape)):
            dst[d_off : d_off + n] = src.reshape(-1)[s_off : s_off + n]
        assert np.array_equal(dst.reshape(dst_shape), src[box])


# ---------------------------------------------------------------- parse --------------
def _write_st(path, entries, blobs, metadata=True, pad=0):
    header = dict(entries)
    if metadata:
        header["__metadata__"] = {"format": "pt"}
    body = json.dumps(header).encode() + b" " * pad
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(body)) + body + blobs)


def test_parse_hand_built_header(oracle, tmp_path):
    # shape of tests/test_gds_loader.py:126-149: two tensors, offsets relative to the data section
    p = tmp_path / "m.safetensors"
    _write_st(p, {"a": {"dtype": "F32", "shape": [2, 2], "data_offsets": [0, 16]},
                  "b": {"dtype": "F16", "shape": [4], "data_offsets": [16, 24]}}, bytes(range(24)), pad=3)
    info = oracle.parse_safetensors_header(str(p))
    with open(p, "rb") as f:
        hl = struct.unpack("<Q", f.read(8))[0]
    assert set(info) == {"a", "b"}
    assert info["a"] == {"file_offset": 8 + hl, "size": 16, "dtype": "F32", "shape": [2, 2]}
    assert info["b"]["file_offset"] == 8 + hl + 16 and info["b"]["size"] == 8


def test_parse_matches_safetensors_library(oracle, tmp_path):
    from safetensors.torch import save_file
    from safetensors import safe_open

    tensors = {"w": torch.arange(24, dtype=torch.float32).reshape(4, 6), "h": torch.ones(5, dtype=torch.bfloat16),
               "q": torch.arange(6, dtype=torch.uint8).view(torch.float8_e4m3fn).reshape(2, 3),
               "s": torch.tensor(3.0)}
    p = tmp_path / "model.safetensors"
    save_file(tensors, str(p))
    got = dict(oracle.load_checkpoint(str(tmp_path)))
    with safe_open(str(p), "pt") as f:
        assert set(f.keys()) == set(got)
        for k in f.keys():
            t = f.get_tensor(k)
            assert got[k].shape == tuple(t.shape)
            assert got[k].tobytes() == t.contiguous().reshape(-1).view(torch.uint8).numpy().tobytes()
    assert got["q"].dtype == "F8_E4M3" and got["s"].shape == ()


def test_parse_errors_and_resolution_order(oracle, tmp_path):
    short = tmp_path / "short.safetensors"
    short.write_bytes(b"\x01\x02\x03")
    with pytest.raises(RuntimeError, match="Invalid safetensors file"):  # gds_loader.py:254-255
        oracle.parse_safetensors_header(str(short))
    big = tmp_path / "big.safetensors"
    big.write_bytes(struct.pack("<Q", 100 * 1024 * 1024 + 1) + b"{}")
    with pytest.raises(RuntimeError, match="header too large"):  # :259-262
        oracle.parse_safetensors_header(str(big))
    d = tmp_path / "model"
    d.mkdir()
    with pytest.raises(FileNotFoundError):
        oracle.resolve_safetensors_files(str(d))
    e = {"x": {"dtype": "U8", "shape": [4], "data_offsets": [0, 4]}}
    _write_st(d / "b.safetensors", e, b"abcd")
    _write_st(d / "a.safetensors", {"y": e["x"]}, b"efgh")
    assert [k.rsplit("/", 1)[1] for k in oracle.resolve_safetensors_files(str(d))] == ["a.safetensors", "b.safetensors"]
    _write_st(d / "model.safetensors", {"z": e["x"]}, b"ijkl")
    assert list(oracle.resolve_safetensors_files(str(d)).values()) == [["z"]]
    (d / "model.safetensors.index.json").write_text(json.dumps({"weight_map": {"x": "b.safetensors", "y": "a.safetensors"}}))
    assert {k.rsplit("/", 1)[1]: v for k, v in oracle.resolve_safetensors_files(str(d)).items()} == {
        "b.safetensors": ["x"], "a.safetensors": ["y"]}
    (d / "model.safetensors.index.json").write_text(json.dumps({"weight_map": {}}))
    with pytest.raises(RuntimeError, match="Empty weight_map"):
        oracle.resolve_safetensors_files(str(d))


# ---------------------------------------------------------------- permuted copies ----
def test_permute_copy_reference_vectors(oracle):
    # tests/test_reshard_refit_slice_plan.py:155-197: transpose, 3-D permute, narrow+transpose
    OT = oracle.OTensor
    src = torch.arange(12, dtype=torch.float32).reshape(3, 4)
    got = oracle.permute_copy(OT.from_array(src.numpy(), "F32"), (1, 0))
    assert got.tobytes() == src.transpose(0, 1).contiguous().numpy().tobytes() and got.shape == (4, 3)
    src = torch.arange(24, dtype=torch.float32).reshape(2, 3, 4)
    got = oracle.permute_copy(OT.from_array(src.numpy(), "F32"), (2, 0, 1))
    assert got.tobytes() == src.permute(2, 0, 1).contiguous().numpy().tobytes() and got.shape == (4, 2, 3)
    src = torch.arange(20, dtype=torch.float32).reshape(4, 5)
    got = oracle.permute_copy(OT.from_array(src.numpy(), "F32").narrow(0, 1, 2), (1, 0))
    assert got.tobytes() == src.narrow(0, 1, 2).transpose(0, 1).contiguous().numpy().tobytes()


def test_mla_absorbed_weights_match_torch(oracle):
    # engines/vllm/refit/receiver.py:244-261 restated with torch ops as the reference composes them
    H, nope, v, L = 4, 6, 5, 7
    w = torch.arange(H * (nope + v) * L, dtype=torch.float32).reshape(H * (nope + v), L)
    view = w.view(H, nope + v, -1)
    w_uk, w_uv = view.split([nope, v], dim=1)
    uv, ukt = oracle.mla_absorbed_weights(oracle.OTensor.from_array(w.numpy(), "F32"), H, nope, v)
    assert uv.shape == (v, H, L) and ukt.shape == (nope, L, H)
    assert uv.tobytes() == w_uv.transpose(0, 1).contiguous().numpy().tobytes()
    assert ukt.tobytes() == w_uk.permute(1, 2, 0).contiguous().numpy().tobytes()
