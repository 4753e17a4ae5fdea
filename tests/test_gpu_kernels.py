"""Stand-alone device operators against the CPU oracle, through the C ABI."""

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _dev(arr: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(arr).view(np.uint8).reshape(-1).copy()).cuda()


SIZES = [0, 1, 3, 4, 15, 16, 17, 255, 4096, 4097, 65536, 65537, 8192 * 3 + 5, 1 << 20, (1 << 22) + 12345]


def test_checksum32_matches_oracle(gpu_engine, oracle, oracle_c):
    rng = np.random.default_rng(10)
    bufs = [rng.integers(0, 256, n, dtype=np.uint8) for n in SIZES]
    dev = [_dev(b) if b.size else torch.empty(0, dtype=torch.uint8, device="cuda") for b in bufs]
    got = gpu_engine.checksum32(dev)
    for b, g in zip(bufs, got):
        assert g == oracle_c.checksum32(b), b.size
    assert got[3] == oracle.safe_checksum_bigint(bufs[3].tobytes())
    assert got[8] == oracle.safe_checksum_bytes(bufs[8])


def test_checksum32_unaligned_views(gpu_engine, oracle_c):
    rng = np.random.default_rng(11)
    base = rng.integers(0, 256, 70000, dtype=np.uint8)
    d = _dev(base)
    for off, n in [(1, 1000), (2, 4096), (3, 65000), (4, 8192), (8, 33333), (13, 16), (16, 50000)]:
        got = gpu_engine.checksum32([d[off: off + n]])[0]
        assert got == oracle_c.checksum32(base[off: off + n]), (off, n)


def test_checksum32_constant_closed_form(gpu_engine):
    K = 2654435761
    n = (1 << 24) + 7
    d = torch.full((n,), 3, dtype=torch.uint8, device="cuda")
    want = (3 * (K * (n * (n - 1) // 2) + n)) & 0xFFFFFFFF
    assert gpu_engine.checksum32([d])[0] == format(want, "08x")


def test_digest_matches_oracle(gpu_engine, oracle, oracle_c):
    rng = np.random.default_rng(12)
    sizes = [0, 1, 3, 4, 7, 4095, 4096, 4097, 4099, 65536, 65536 + 4096 * 3 + 9, 16 * 4096, 17 * 4096 + 2, 1 << 21]
    bufs = [rng.integers(0, 256, n, dtype=np.uint8) for n in sizes]
    dev = [_dev(b) if b.size else torch.empty(0, dtype=torch.uint8, device="cuda") for b in bufs]
    hexes, scalars = gpu_engine.digest(dev, with_scalars=True)
    for b, h, sc in zip(bufs, hexes, scalars):
        assert sc == oracle_c.digest_scalars(b), b.size
        assert h == oracle.tensor_digest_bytes(b.tobytes()), b.size


def test_verify_plan_repeats_match_one_shot_calls(gpu_engine, oracle, oracle_c):
    """Buffers lowered once (the reference caches its descriptor lists, refit/reshard/receiver.py:787-801):
    every run must give what the one-shot calls and the oracle give, also after the bytes changed and
    on another stream; the accumulators a run leaves behind must not leak into the next."""
    rng = np.random.default_rng(15)
    sizes = [0, 1, 3, 16, 4097, 65536 + 4096 * 3 + 9, 17 * 4096 + 2, (1 << 21) + 5]
    bufs = [rng.integers(0, 256, n, dtype=np.uint8) for n in sizes]
    base = torch.from_numpy(np.concatenate([np.zeros(3, np.uint8)] + bufs)).cuda()  # views at odd offsets
    dev, pos = [], 3
    for b in bufs:
        dev.append(base[pos: pos + b.size])
        pos += b.size
    plan = gpu_engine.verify_plan(dev)
    side = torch.cuda.Stream()
    for rep in range(3):
        want_c = [oracle_c.checksum32(b) for b in bufs]
        want_d = [oracle.tensor_digest_bytes(b.tobytes()) for b in bufs]
        stream = side.cuda_stream if rep == 1 else 0
        torch.cuda.synchronize()
        assert plan.checksums(stream=stream) == want_c == gpu_engine.checksum32(dev)
        assert plan.digests(stream=stream) == want_d == gpu_engine.digest(dev)
        for b, d in zip(bufs, dev):  # new bytes at the same addresses
            if b.size:
                b[b.size // 2] ^= 0x5A
                d[b.size // 2] ^= 0x5A
    plan.close()
    empty = gpu_engine.verify_plan([])
    assert empty.checksums() == [] and empty.digests() == []


def test_batches_too_large_for_accumulator_copies_take_the_plain_layout(gpu_engine, oracle_c):
    """Accumulators are kept in 64 copies up to 16,384 of them and in one copy beyond (csrc/mxp_device.h, make_fan):
    both sides of that limit, through the one-shot calls and a verify plan, repeated; one large buffer among the
    small ones gives many workgroups adding to one accumulator."""
    rng = np.random.default_rng(23)
    for n in (16384, 16385, 20000):
        sizes = rng.integers(0, 200, n)
        sizes[n // 2] = 3 * (1 << 20) + 7
        data = rng.integers(0, 256, int(sizes.sum()), dtype=np.uint8)
        base = torch.from_numpy(data).cuda()
        offs = np.concatenate(([0], np.cumsum(sizes)))
        dev = [base[int(offs[k]): int(offs[k + 1])] for k in range(n)]
        probe = list(range(0, n, 997)) + [n // 2, n - 1]
        want = {k: oracle_c.checksum32(data[int(offs[k]): int(offs[k + 1])]) for k in probe}
        got = gpu_engine.checksum32(dev)
        assert all(got[k] == want[k] for k in probe), n
        plan = gpu_engine.verify_plan(dev)
        for _ in range(2):
            assert plan.checksums() == got, n
        assert plan.digests() == gpu_engine.digest(dev), n
        plan.close()


def test_digest_reference_invariants_on_device(gpu_engine, oracle):
    a = np.arange(8192, dtype=np.int32)
    b = a.copy()
    b[0:1024], b[1024:2048] = a[1024:2048], a[0:1024]
    da, db = gpu_engine.digest([_dev(a), _dev(b)])
    assert da != db and da == oracle.tensor_digest_bytes(a.tobytes())
    # offset independence, including a 2-byte-aligned start (bf16 view at an odd element)
    flat = np.arange(20000, dtype=np.uint16)
    d = _dev(flat)
    view = d[2 * 1409: 2 * 1409 + 2 * 9000]
    assert gpu_engine.digest([view])[0] == oracle.tensor_digest_bytes(flat[1409: 1409 + 9000].tobytes())
    neg = np.full(4096, -1, dtype=np.int32)
    assert gpu_engine.digest([_dev(neg)])[0] == oracle.tensor_digest_bytes(neg.tobytes())


def test_cast_f32_bf16_matches_oracle(gpu_engine, oracle, oracle_c):
    rng = np.random.default_rng(13)
    hi = np.arange(1 << 16, dtype=np.uint32) << 16
    lows = np.array([0x0000, 0x0001, 0x7FFF, 0x8000, 0x8001, 0xFFFF], dtype=np.uint32)
    classes = (hi[:, None] | lows[None, :]).reshape(-1)
    rnd = rng.integers(0, 1 << 32, (1 << 20) + 3, dtype=np.uint64).astype(np.uint32)
    for src in (classes, rnd, rnd[:1], rnd[:7], rnd[:8], rnd[:4099]):
        s = _dev(src)
        d = torch.zeros(src.size * 2 + 16, dtype=torch.uint8, device="cuda")
        csum = gpu_engine.cast_f32_bf16(s, d, src.size)
        got = d[: src.size * 2].cpu().numpy().view(np.uint16)
        want = oracle.cast_f32_bf16_bits(src)
        assert np.array_equal(got, want)
        assert np.array_equal(got, oracle_c.cast_f32_bf16(src))
        assert csum == oracle_c.checksum32(want)
        assert int(d[src.size * 2:].sum()) == 0  # nothing written past the end


@pytest.mark.parametrize("src_dtype,dst_dtype", [("BF16", "F32"), ("F16", "F32"), ("F32", "F16"), ("F8_E4M3", "BF16"),
                                                 ("F16", "BF16"), ("BF16", "F16")])
def test_cast_pairs_match_oracle(gpu_engine, oracle, oracle_c, src_dtype, dst_dtype):
    """The other conversions of dest.copy_(src) (refit/reshard/receiver.py:962-969): every 16-bit
    pattern for the widening ones, every rounding class for fp32 -> fp16, odd sizes and offsets."""
    rng = np.random.default_rng(14)
    code = oracle.CAST_CODES[(src_dtype, dst_dtype)]
    if src_dtype == "F32":
        hi = np.arange(1 << 16, dtype=np.uint32) << 16
        lows = np.array([0, 1, 0x0FFF, 0x1000, 0x1001, 0x1FFF, 0x2000, 0x3000, 0xFFFF], dtype=np.uint32)
        full = np.concatenate([(hi[:, None] | lows[None, :]).reshape(-1),
                               rng.integers(0, 1 << 32, (1 << 20) + 3, dtype=np.uint64).astype(np.uint32)])
        fn, se, de = oracle.cast_f32_f16_bits, 4, 2
    elif src_dtype == "F8_E4M3":
        full = np.concatenate([np.arange(256, dtype=np.uint8), rng.integers(0, 256, (1 << 20) + 5, dtype=np.uint8)])
        fn, se, de = oracle.cast_f8e4m3_bf16_bits, 1, 2
    elif dst_dtype != "F32":  # between the two 16-bit formats, through fp32
        full = np.concatenate([np.arange(1 << 16, dtype=np.uint16), rng.integers(0, 1 << 16, (1 << 20) + 5, dtype=np.uint16)])
        if src_dtype == "F16":
            fn = lambda u: oracle.cast_f32_bf16_bits(oracle.cast_f16_f32_bits(u))  # noqa: E731
        else:
            fn = lambda u: oracle.cast_f32_f16_bits(oracle.cast_bf16_f32_bits(u))  # noqa: E731
        se, de = 2, 2
    else:
        full = np.concatenate([np.arange(1 << 16, dtype=np.uint16), rng.integers(0, 1 << 16, (1 << 20) + 5, dtype=np.uint16)])
        fn, se, de = (oracle.cast_bf16_f32_bits if src_dtype == "BF16" else oracle.cast_f16_f32_bits), 2, 4
    dev = _dev(full)
    for off, n in ((0, full.size), (0, 1), (1, 7), (3, 8), (5, 4099), (2, 65536 + 11)):
        src = full[off: off + n]
        d = torch.zeros(n * de + 16, dtype=torch.uint8, device="cuda")
        csum = gpu_engine.cast(dev.view(torch.uint8)[off * se:], d, n, src_dtype, dst_dtype)
        want = fn(src)
        got = d[: n * de].cpu().numpy().view(want.dtype)
        assert np.array_equal(got, want), (off, n)
        assert np.array_equal(oracle_c.cast(code, src), want)
        assert csum == oracle_c.checksum32(want.view(np.uint8))
        assert int(d[n * de:].sum()) == 0  # nothing written past the end
    with pytest.raises(ValueError):
        gpu_engine.cast(dev, dev, 1, "BF16", "I32")


def test_cast_nan_image_is_a_parameter(mxp, oracle):
    from modelexpress_amd.engine import PlacementEngine

    eng = PlacementEngine(0, nan_bits=0xFFFF)
    src = np.array([0x7FC00001, 0xFFFFFFFF, 0x7F800001, 0x3F800000], dtype=np.uint32)
    d = torch.zeros(16, dtype=torch.uint8, device="cuda")
    eng.cast_f32_bf16(_dev(src), d, 4)
    assert d[:8].cpu().numpy().view(np.uint16).tolist() == [0xFFFF, 0xFFFF, 0xFFFF, 0x3F80]
    ref = torch.from_numpy(src.view(np.float32).copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert ref[3] == 0x3F80 and all((int(v) & 0x7FFF) > 0x7F80 for v in ref[:3])
    # the same image through the wide path (eight elements per lane), a converting transpose and fp16 -> bf16
    big = np.tile(src, 4096)
    d = torch.zeros(big.size * 2, dtype=torch.uint8, device="cuda")
    eng.cast_f32_bf16(_dev(big), d, big.size)
    assert np.array_equal(d.cpu().numpy().view(np.uint16), np.tile(np.array([0xFFFF, 0xFFFF, 0xFFFF, 0x3F80], dtype=np.uint16), 4096))
    m = big.reshape(128, 128)
    d = torch.zeros(m.size * 2, dtype=torch.uint8, device="cuda")
    eng.copy_view(_dev(m), d, (128, 128), 2, src_strides=(1, 128), cast=oracle.CAST_CODES[("F32", "BF16")], checksum=False)
    assert np.array_equal(d.cpu().numpy().view(np.uint16).reshape(128, 128), oracle.cast_f32_bf16_bits(m, 0xFFFF).astype(np.uint16).T)
    h = np.tile(np.array([0x7C01, 0xFE00, 0x3C00, 0x7C00], dtype=np.uint16), 4096)
    d = torch.zeros(h.size * 2, dtype=torch.uint8, device="cuda")
    eng.cast(_dev(h), d, h.size, "F16", "BF16")
    assert np.array_equal(d.cpu().numpy().view(np.uint16), np.tile(np.array([0xFFFF, 0xFFFF, 0x3F80, 0x7F80], dtype=np.uint16), 4096))
    eng.close()


_TORCH = {"F32": (torch.float32, np.uint32), "BF16": (torch.bfloat16, np.uint16), "F16": (torch.float16, np.uint16),
          "F8_E4M3": (torch.float8_e4m3fn, np.uint8)}


@pytest.mark.parametrize("src_dtype,dst_dtype", [("F32", "BF16"), ("BF16", "F32"), ("F16", "F32"), ("F32", "F16"),
                                                 ("F8_E4M3", "BF16"), ("F16", "BF16"), ("BF16", "F16")])
def test_default_conversions_equal_torch_on_this_device(gpu_engine, src_dtype, dst_dtype):
    """What the reference runs for a dtype-converting copy is ``recv.copy_(staging)`` on the DEVICE
    (refit/reshard/receiver.py:964-971, fsdp/adapter.py:203-206), so the images this library produces
    with default options - NaNs of every sign and payload included - are compared bit for bit with
    ``torch.Tensor.to`` run on this very GPU.  (torch's CPU kernels may disagree about NaNs with the
    device ones: fp32 -> bf16 gives 0xFFFF on AVX-512 hosts and 0x7FC0 on the device.)"""
    rng = np.random.default_rng(21)
    t_src, np_src = _TORCH[src_dtype]
    t_dst, np_dst = _TORCH[dst_dtype]
    bits = np.dtype(np_src).itemsize * 8
    if bits == 32:
        nan_exp = np.uint32(0x7F800000)
        payload = rng.integers(1, 1 << 23, 4096, dtype=np.uint64).astype(np.uint32)
        sign = (rng.integers(0, 2, 4096, dtype=np.uint64).astype(np.uint32) << 31)
        nans = nan_exp | payload | sign
        special = np.array([0x7FC00000, 0xFFC00000, 0x7F800001, 0xFF800001, 0x7FFFFFFF, 0xFFFFFFFF, 0x7F800000, 0xFF800000,
                            0x00000001, 0x807FFFFF, 0x7F7FFFFF, 0x3F808000, 0x3F818000, 0x477FE000, 0x477FF000, 0x33000000],
                           dtype=np.uint32)
        src = np.concatenate([special, nans, rng.integers(0, 1 << 32, 1 << 16, dtype=np.uint64).astype(np.uint32)])
    elif bits == 16:
        src = np.arange(1 << 16, dtype=np.uint16)  # every pattern, every NaN among them
    else:
        src = np.arange(256, dtype=np.uint8)
    dev_src = torch.from_numpy(src.copy()).cuda()
    want = dev_src.view(t_src).to(t_dst).contiguous().view(torch.uint8).cpu().numpy().view(np_dst)
    out = torch.zeros(src.size * np.dtype(np_dst).itemsize, dtype=torch.uint8, device="cuda")
    gpu_engine.cast(dev_src.view(torch.uint8), out, src.size, src_dtype, dst_dtype, checksum=False)
    got = out.cpu().numpy().view(np_dst)
    bad = np.flatnonzero(got != want)
    assert bad.size == 0, [(hex(int(src[i])), hex(int(got[i])), hex(int(want[i]))) for i in bad[:8]]


def test_nan_image_of_the_host_can_be_probed_and_asked_for(mxp):
    """A caller that wants the CPU path's bytes instead (torch CPU maps every fp32 NaN to one image that
    depends on the host's vector ISA) probes that image and passes it as ``nan_bits``."""
    from modelexpress_amd.engine import PlacementEngine

    probed = int(torch.tensor([float("nan")]).to(torch.bfloat16).view(torch.int16).item()) & 0xFFFF
    assert (probed & 0x7FFF) > 0x7F80
    rng = np.random.default_rng(22)
    nans = (np.uint32(0x7F800000) | rng.integers(1, 1 << 23, 2048, dtype=np.uint64).astype(np.uint32)
            | (rng.integers(0, 2, 2048, dtype=np.uint64).astype(np.uint32) << 31))
    src = np.concatenate([nans, rng.integers(0, 1 << 32, 1 << 14, dtype=np.uint64).astype(np.uint32)])
    want = torch.from_numpy(src.view(np.float32).copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    if not np.all(want[:2048] == probed):
        pytest.skip("torch CPU on this host does not map every NaN to one image")
    eng = PlacementEngine(0, nan_bits=probed)
    out = torch.zeros(src.size * 2, dtype=torch.uint8, device="cuda")
    eng.cast_f32_bf16(_dev(src), out, src.size)
    assert np.array_equal(out.cpu().numpy().view(np.uint16), want)
    eng.close()


@pytest.mark.parametrize("rows,row_bytes,src_pitch,dst_pitch,src_off", [
    (4096, 1024, 8192, 1024, 1024 * 3),      # o_proj TP=8 column slice
    (512, 3584, 28672, 3584, 3584 * 5),      # down_proj TP=8 column slice
    (56, 64, 512, 64, 64 * 2),               # fp8 scale-tile column slice
    (7, 13, 29, 17, 3),                      # byte-granular
    (33, 20, 44, 24, 4),                     # dword-granular
    (1, 100001, 100001, 100001, 0),          # contiguous odd size
    (3, 70000, 140000, 70000, 16),           # rows wider than one tile row
])
def test_gather2d_matches_oracle(gpu_engine, oracle_c, rows, row_bytes, src_pitch, dst_pitch, src_off):
    rng = np.random.default_rng(14)
    src = rng.integers(0, 256, src_off + rows * src_pitch + 64, dtype=np.uint8)
    want = np.full(rows * dst_pitch + 32, 0xEE, dtype=np.uint8)
    for r in range(rows):
        want[r * dst_pitch: r * dst_pitch + row_bytes] = src[src_off + r * src_pitch: src_off + r * src_pitch + row_bytes]
    s = _dev(src)
    d = torch.full((want.size,), 0xEE, dtype=torch.uint8, device="cuda")
    csum = gpu_engine.gather2d(s[src_off:], src_pitch, d, dst_pitch, rows, row_bytes)
    assert np.array_equal(d.cpu().numpy(), want)
    acc = 0
    for r in range(rows):
        acc += int(oracle_c.checksum32(want[r * dst_pitch: r * dst_pitch + row_bytes], first_index=r * dst_pitch), 16)
    assert csum == format(acc & 0xFFFFFFFF, "08x")


def test_place_boxes_mixed_batch(gpu_engine, oracle, oracle_c):
    rng = np.random.default_rng(15)
    src_a = rng.integers(0, 256, 64 * 512, dtype=np.uint8)           # (64, 512) bytes, take cols 128..255
    src_f = rng.integers(0, 1 << 32, 4096, dtype=np.uint64).astype(np.uint32)  # fp32 bits, cast 1000 elements
    src_c = rng.integers(0, 256, 5000, dtype=np.uint8)
    da, df, dc = _dev(src_a), _dev(src_f), _dev(src_c)
    out = torch.zeros(64 * 128 + 2048 + 5008, dtype=torch.uint8, device="cuda")
    o_a, o_f, o_c = 0, 64 * 128, 64 * 128 + 2048
    boxes = [
        {"src": da[128:], "dst": out[o_a:], "src_pitch": 512, "dst_pitch": 128, "rows": 64, "row_bytes": 128,
         "csum_index": 0, "csum_group": 0},
        {"src": df[4 * 8:], "dst": out[o_f:], "rows": 1, "row_bytes": 2000, "cast": 1, "csum_index": 0, "csum_group": 1},
        {"src": dc[3:], "dst": out[o_c:], "rows": 1, "row_bytes": 4990, "csum_index": 10, "csum_group": 2},
    ]
    sums = gpu_engine.place_boxes(boxes, 3)
    got = out.cpu().numpy()
    want_a = np.ascontiguousarray(src_a.reshape(64, 512)[:, 128:256])
    want_f = oracle.cast_f32_bf16_bits(src_f[8:1008]).view(np.uint8)
    want_c = src_c[3:4993]
    assert got[o_a:o_a + want_a.size].tobytes() == want_a.tobytes()
    assert got[o_f:o_f + 2000].tobytes() == want_f.tobytes()
    assert got[o_c:o_c + 4990].tobytes() == want_c.tobytes()
    assert sums[0] == oracle_c.checksum32(want_a)
    assert sums[1] == oracle_c.checksum32(want_f)
    assert sums[2] == oracle_c.checksum32(want_c, first_index=10)


def test_shard_region_matches_oracle(gpu_engine, oracle):
    # refit/reshard/verify.py:158-183 and tests/test_reshard_refit_verify.py:135-171
    OT = oracle.OTensor
    full = np.arange(24, dtype=np.float32).reshape(4, 6)
    d = _dev(full)
    buf, csum = gpu_engine.shard_region(d, (4, 6), (1, 2), (2, 3), 4)
    want = oracle.shard_region(OT.from_array(full.reshape(-1), "F32"), (4, 6), (1, 2), (2, 3))
    assert buf.cpu().numpy().tobytes() == want.tobytes() == np.ascontiguousarray(full[1:3, 2:5]).tobytes()
    assert csum == oracle.safe_checksum(want)
    assert gpu_engine.digest([buf])[0] == oracle.tensor_digest(want)
    with pytest.raises(ValueError, match="rank mismatch"):
        gpu_engine.shard_region(d, (4, 6), (1,), (2, 3), 4)
    rng = np.random.default_rng(16)
    big = rng.integers(0, 1 << 16, (6, 40, 96), dtype=np.uint16)
    db = _dev(big)
    for off, shp in [((1, 8, 0), (4, 16, 96)), ((0, 0, 32), (6, 40, 48)), ((2, 3, 5), (3, 30, 7)), ((0, 0, 0), (6, 40, 96))]:
        buf, csum = gpu_engine.shard_region(db, big.shape, off, shp, 2)
        want = oracle.shard_region(OT.from_array(big.reshape(-1), "BF16"), big.shape, off, shp)
        assert buf.cpu().numpy().tobytes() == want.tobytes(), (off, shp)
        assert csum == oracle.safe_checksum(want)


@pytest.mark.parametrize("shape,perm,es", [
    ((3, 4), (1, 0), 4),                 # test_reshard_refit_slice_plan.py:155-167
    ((2, 3, 4), (2, 0, 1), 4),           # :170-183
    ((64, 64), (1, 0), 2),
    ((130, 67), (1, 0), 2),              # ragged tiles, element-wise edges
    ((257, 129), (1, 0), 1),
    ((100, 72), (1, 0), 8),
    ((5, 96, 80), (0, 2, 1), 2),         # batched transposes
    ((16, 128, 512), (1, 2, 0), 2),      # W_UK_T shape of one TP=8 rank: [heads, nope, lora] -> [nope, lora, heads]
    ((16, 128, 512), (1, 0, 2), 2),      # W_UV: keeps the innermost dim -> row gather
    ((7, 5, 6, 9), (3, 1, 0, 2), 4),     # 4-D
    ((6, 1, 33), (2, 1, 0), 2),          # unit dim dropped
    ((1000,), (0,), 2),
    ((256, 384), (1, 0), 1),             # whole sub-tiles only, every element size
    ((1024, 192), (1, 0), 2),
    ((192, 96), (1, 0), 4),
    ((128, 48), (1, 0), 8),
    ((200, 300), (1, 0), 1),             # ragged in both directions
    ((600, 200), (1, 0), 2),             # ragged, 16-byte accesses on both sides
    ((600, 201), (1, 0), 2),             # source rows not 16-byte aligned
    ((601, 200), (1, 0), 2),             # destination rows not 16-byte aligned
    ((3, 520, 136), (0, 2, 1), 4),
    ((16, 1024), (1, 0), 2),             # destination rows shorter than a sub-tile
    ((1024, 16), (1, 0), 2),             # source rows shorter than a sub-tile
    ((2, 3, 70, 130), (1, 3, 0, 2), 2),  # two batch dimensions, transposed inner pair
])
def test_permute_copy_matches_oracle(gpu_engine, oracle, oracle_c, shape, perm, es):
    rng = np.random.default_rng(17)
    n = int(np.prod(shape))
    raw = rng.integers(0, 256, n * es, dtype=np.uint8)
    dtype = {1: "U8", 2: "BF16", 4: "F32", 8: "I64"}[es]
    src = oracle.OTensor(raw.reshape(tuple(shape) + (es,)), dtype)
    want = oracle.permute_copy(src, perm)
    d = torch.full((n * es + 16,), 0xEE, dtype=torch.uint8, device="cuda")
    csum = gpu_engine.permute_copy(_dev(raw), d, shape, perm, es)
    assert d[: n * es].cpu().numpy().tobytes() == want.tobytes()
    assert int((d[n * es:] != 0xEE).sum()) == 0
    assert csum == oracle_c.checksum32(np.frombuffer(want.tobytes(), dtype=np.uint8))


@pytest.mark.parametrize("seed", range(10))
def test_permute_copy_random(gpu_engine, oracle, oracle_c, seed):
    """Random shapes, permutations and element sizes against the element-enumerating oracle."""
    rng = np.random.default_rng(900 + seed)
    nd = int(rng.integers(2, 5))
    es = int(rng.choice([1, 2, 4, 8]))
    shape = tuple(int(x) for x in rng.integers(1, {2: 700, 3: 90, 4: 30}[nd], nd))
    perm = tuple(int(x) for x in rng.permutation(nd))
    n = int(np.prod(shape))
    raw = rng.integers(0, 256, n * es, dtype=np.uint8)
    src = oracle.OTensor(raw.reshape(shape + (es,)), {1: "U8", 2: "BF16", 4: "F32", 8: "I64"}[es])
    want = oracle.permute_copy(src, perm)
    d = torch.full((n * es + 16,), 0xEE, dtype=torch.uint8, device="cuda")
    csum = gpu_engine.permute_copy(_dev(raw), d, shape, perm, es)
    assert d[: n * es].cpu().numpy().tobytes() == want.tobytes(), (shape, perm, es)
    assert int((d[n * es:] != 0xEE).sum()) == 0
    assert csum == oracle_c.checksum32(np.frombuffer(want.tobytes(), dtype=np.uint8))


_SRC_WORD = {"F32": np.uint32, "BF16": np.uint16, "F16": np.uint16, "F8_E4M3": np.uint8}
_DST_WORD = {"F32": np.uint32, "BF16": np.uint16, "F16": np.uint16}


@pytest.mark.parametrize("src_dtype,dst_dtype", [("F32", "BF16"), ("BF16", "F32"), ("F16", "F32"), ("F32", "F16"),
                                                 ("F8_E4M3", "BF16"), ("F16", "BF16"), ("BF16", "F16")])
def test_converting_transposes_match_oracle(gpu_engine, oracle, oracle_c, src_dtype, dst_dtype):
    """``dest.copy_(src.t())`` across dtypes (refit/reshard/receiver.py:962-969 on a transposed view;
    engines/vllm/refit/receiver.py:258-261): one pass, bit-exact against convert-then-transpose on the
    host, over every 16-bit pattern (every rounding class for fp32 sources), ragged edges, strided and
    unaligned sides, batches, with the checksum of the destination bytes."""
    rng = np.random.default_rng(77)
    code = oracle.CAST_CODES[(src_dtype, dst_dtype)]
    sw, dw = _SRC_WORD[src_dtype], _DST_WORD[dst_dtype]
    se, de = np.dtype(sw).itemsize, np.dtype(dw).itemsize

    def patterns(n):
        if src_dtype == "F32":
            hi = rng.integers(0, 1 << 16, n, dtype=np.uint32) << 16
            lows = np.array([0, 1, 0x0FFF, 0x1000, 0x1001, 0x1FFF, 0x2000, 0x3000, 0x7FFF, 0x8000, 0x8001, 0xFFFF], dtype=np.uint32)
            out = hi | lows[rng.integers(0, lows.size, n)]
            out[: min(n, 1 << 16)] = (np.arange(min(n, 1 << 16), dtype=np.uint32) << 16) | lows[np.arange(min(n, 1 << 16)) % lows.size]
            return out
        out = rng.integers(0, 1 << (8 * se), n, dtype=np.uint64).astype(sw)
        k = min(n, 1 << (8 * se))
        out[:k] = np.arange(k, dtype=sw)
        return out

    # (batch, rows, cols, source row pitch, destination row pitch, source offset, destination offset), in elements:
    # dst[b, c, r] = convert(src[b, r, c])
    cases = [(1, 512, 512, 512, 512, 0, 0),      # whole tiles, every pattern
             (1, 130, 70, 70, 130, 0, 0),        # ragged both ways
             (1, 130, 70, 75, 131, 3, 5),        # odd pitches and offsets: no 16-byte access is aligned
             (3, 65, 257, 264, 72, 8, 8),        # batch, aligned pitches, ragged extents
             (1, 1, 300, 300, 1, 0, 0),          # degenerate: a single source row
             (2, 7, 5, 5, 7, 1, 0)]
    for (nb, r, c, sp, dp, so, do) in cases:
        raw = patterns(so + nb * r * sp + 16)
        src = raw[so: so + nb * r * sp].reshape(nb, r, sp)[:, :, :c]
        conv = oracle_c.cast(code, np.ascontiguousarray(src).reshape(-1)).reshape(nb, r, c)
        dst_elems = do + nb * c * dp + 16
        want = np.full(dst_elems, 0xEEEE if de == 2 else 0xEEEEEEEE, dtype=dw)
        want[do: do + nb * c * dp].reshape(nb, c, dp)[:, :, :r] = conv.transpose(0, 2, 1)
        d = torch.from_numpy(np.full(dst_elems * de, 0xEE, dtype=np.uint8)).cuda()
        dev = _dev(raw.view(np.uint8))
        csum = gpu_engine.copy_view(dev[so * se:], d[do * de:], (nb, c, r), de, src_strides=(r * sp, 1, sp),
                                    dst_strides=(c * dp, dp, 1), cast=code)
        got = d.cpu().numpy().view(dw)
        assert np.array_equal(got, want), (src_dtype, dst_dtype, nb, r, c, sp, dp, so, do)
        # the checksum is over the destination view's bytes, positions counted from its first element
        region = want[do: do + nb * c * dp].copy()
        mask = np.zeros(nb * c * dp, dtype=bool)
        mask.reshape(nb, c, dp)[:, :, :r] = True
        pos = np.flatnonzero(np.repeat(mask, de))
        b = region.view(np.uint8)[pos].astype(np.uint64)
        ref = int((b * ((pos.astype(np.uint64) * np.uint64(2654435761) + np.uint64(1)) & np.uint64(0xFFFFFFFF))).sum() & np.uint64(0xFFFFFFFF))
        assert int(csum, 16) == ref, (src_dtype, dst_dtype, nb, r, c)


_PANEL_PAIRS = [("U8", "U8"), ("BF16", "BF16"), ("F32", "F32"), ("F32", "BF16"), ("BF16", "F32"), ("F16", "F32"), ("F32", "F16"),
                ("F8_E4M3", "BF16"), ("F16", "BF16"), ("BF16", "F16")]
_WORD = {"U8": np.uint8, "F32": np.uint32, "BF16": np.uint16, "F16": np.uint16, "F8_E4M3": np.uint8}


def _panel_cases(se, de):
    """(batch dims, rows r = destination innermost, columns c, source row pitch, destination row pitch) in elements,
    chosen so that the transposes take the staged-tile ("panel") form: whole tiles, 16-byte aligned, and either short
    abutting destination rows or long pitches on both sides."""
    cases = [((3,), 128, 1024 // se, 1024 // se, 128),         # destination rows abut: one tile = one contiguous block
             ((2, 3), 16, 2048 // se, 2048 // se + 16 // se, 16),   # very short rows, two batch dimensions, padded source pitch
             ((1,), 1024 // de, 512, 512, 1024 // de),         # the longest rows of that branch (1 KiB)
             ((600,), 32, 256 // se, 256 // se, 32)]           # many small tiles: enough for full-size workgroups
    if se == 2 and de == 2:
        cases.append(((1,), 1024, 512, 16384, 16384))          # 32 KiB pitches on both sides
    if se == 2 and de == 4:
        cases.append(((2,), 512, 512, 8192, 8192))             # widening: 16 KiB source pitch, 32 KiB destination pitch
    return cases


@pytest.mark.parametrize("src_dtype,dst_dtype", _PANEL_PAIRS)
def test_staged_tile_transposes_match_oracle(gpu_engine, oracle, oracle_c, src_dtype, dst_dtype):
    """The transposes that run as whole staged tiles (a workgroup's read burst, a barrier, a write burst; no edge
    handling in the kernel): every element type and conversion, single launches with their checksum and batched
    launches (mxp_copy_views), against convert-then-transpose on the host."""
    rng = np.random.default_rng(78)
    code = 0 if src_dtype == dst_dtype else oracle.CAST_CODES[(src_dtype, dst_dtype)]
    sw, dw = _WORD[src_dtype], _WORD[dst_dtype]
    se, de = np.dtype(sw).itemsize, np.dtype(dw).itemsize
    fill = {1: 0xEE, 2: 0xEEEE, 4: 0xEEEEEEEE}[de]
    batch_views, batch_wants = [], []
    for (bdims, r, c, sp, dp) in _panel_cases(se, de):
        nb = int(np.prod(bdims))
        raw = rng.integers(0, 1 << (8 * se), nb * r * sp, dtype=np.uint64).astype(sw)
        k = min(raw.size, 1 << 16)
        raw[:k] = np.arange(k, dtype=np.uint64).astype(sw) if se < 4 else (np.arange(k, dtype=np.uint32) << 16) | 0x8000
        src = raw.reshape(nb, r, sp)[:, :, :c]
        conv = src if code == 0 else oracle_c.cast(code, np.ascontiguousarray(src).reshape(-1)).reshape(nb, r, c)
        want = np.full(nb * c * dp, fill, dtype=dw)
        want.reshape(nb, c, dp)[:, :, :r] = conv.transpose(0, 2, 1)
        d = torch.from_numpy(np.full(want.size * de, 0xEE, dtype=np.uint8)).cuda()
        dev = _dev(raw.view(np.uint8))
        # batch dimensions outermost, then (c, r): dst[b..., c, r] = convert(src[b..., r, c])
        shape = tuple(bdims) + (c, r)
        b_src = [int(np.prod(bdims[i + 1:])) * r * sp for i in range(len(bdims))]
        b_dst = [int(np.prod(bdims[i + 1:])) * c * dp for i in range(len(bdims))]
        view = dict(src=dev, dst=d, shape=shape, elem_size=de, src_strides=tuple(b_src) + (1, sp), dst_strides=tuple(b_dst) + (dp, 1), cast=code)
        kind, tile_rows, tile_row_bytes = gpu_engine.describe_views([view])[0]
        assert kind == "staged_tile" and r % tile_rows == 0 and (c * se) % tile_row_bytes == 0, (kind, tile_rows, tile_row_bytes, bdims, r, c)
        csum = gpu_engine.copy_view(dev, d, shape, de, src_strides=view["src_strides"], dst_strides=view["dst_strides"], cast=code)
        got = d.cpu().numpy().view(dw)
        assert np.array_equal(got, want), (src_dtype, dst_dtype, bdims, r, c, sp, dp)
        mask = np.zeros(nb * c * dp, dtype=bool)
        mask.reshape(nb, c, dp)[:, :, :r] = True
        pos = np.flatnonzero(np.repeat(mask, de))
        b = want.view(np.uint8)[pos].astype(np.uint64)
        ref = int((b * ((pos.astype(np.uint64) * np.uint64(2654435761) + np.uint64(1)) & np.uint64(0xFFFFFFFF))).sum() & np.uint64(0xFFFFFFFF))
        assert int(csum, 16) == ref, (src_dtype, dst_dtype, bdims, r, c)
        d2 = torch.from_numpy(np.full(want.size * de, 0xEE, dtype=np.uint8)).cuda()
        batch_views.append(dict(view, dst=d2))
        batch_wants.append((d2, want))
    # the same views again as one call: transposes that share a tile shape go out as one launch - with one descriptor
    # for all when they are alike (the first view twice), each with its own otherwise (its first two batches alone)
    first, (_d, want0) = batch_views[0], batch_wants[0]
    part = torch.from_numpy(np.full(want0.size * de, 0xEE, dtype=np.uint8)).cuda()
    shorter = dict(first, dst=part, shape=(2,) + tuple(first["shape"][1:]))
    gpu_engine.copy_views(batch_views + [dict(first), shorter])
    for d2, want in batch_wants:
        assert np.array_equal(d2.cpu().numpy().view(want.dtype), want), (src_dtype, dst_dtype, want.size)
    per_batch = want0.size // 3
    got = part.cpu().numpy().view(dw)
    assert np.array_equal(got[: 2 * per_batch], want0[: 2 * per_batch]) and np.all(got[2 * per_batch:] == fill)


def test_staged_tile_uniform_batch_longer_than_one_argument_block(gpu_engine):
    """230 transposes of one shape in one mxp_copy_views call: their pointers travel as kernel arguments, 96 items to
    a launch, so the call is three launches; every item must land in its own destination and nowhere else."""
    rng = np.random.default_rng(79)
    n_items, nb, r, c = 230, 4, 128, 256     # per item: [4, 128, 256] bf16 -> [4, 256, 128]
    raw = rng.integers(0, 1 << 16, (n_items, nb, r, c), dtype=np.uint16)
    src = _dev(raw.reshape(-1).view(np.uint8))
    dst = torch.from_numpy(np.full(raw.size * 2 + 4096, 0xEE, dtype=np.uint8)).cuda()
    per = nb * r * c * 2
    order = rng.permutation(n_items)           # item k writes the order[k]-th slot of the destination
    views = [dict(src=src[k * per:(k + 1) * per], dst=dst[int(order[k]) * per:(int(order[k]) + 1) * per], shape=(nb, c, r), elem_size=2,
                  src_strides=(r * c, 1, c), dst_strides=(c * r, r, 1)) for k in range(n_items)]
    kinds = gpu_engine.describe_views(views)
    assert all(kind == "staged_tile" for kind, _r, _b in kinds), kinds[0]
    gpu_engine.copy_views(views)
    got = dst.cpu().numpy()
    assert np.all(got[n_items * per:] == 0xEE)
    got = got[: n_items * per].view(np.uint16).reshape(n_items, nb, c, r)
    assert np.array_equal(got[order], raw.transpose(0, 1, 3, 2))


def _random_layout(rng, shape):
    """Strides (in elements) of a view of `shape` inside a padded buffer whose dimensions are stored in a random order."""
    order = list(rng.permutation(len(shape)))  # storage order, outermost first
    strides = [0] * len(shape)
    run = 1
    for d in reversed(order):
        strides[d] = run
        run *= shape[d] + int(rng.integers(0, 3)) * int(rng.integers(0, 2))  # sometimes padded
    return strides, run


@pytest.mark.parametrize("seed", range(24))
def test_copy_view_random_layouts_and_conversions(gpu_engine, oracle, oracle_c, seed):
    """``dst.as_strided(shape, ds).copy_(src.as_strided(shape, ss))`` for random shapes, storage orders,
    paddings, offsets and conversions (refit/reshard/types.py:57-71 executed on the device): whichever
    route a view takes - row boxes, the transpose, element runs - the bytes equal numpy's strided copy
    of the host-converted source, and nothing outside the view is written."""
    rng = np.random.default_rng(4000 + seed)
    pairs = [None] + list(oracle.CAST_CODES)
    pair = pairs[seed % len(pairs)]
    if pair is None:
        es = int(rng.choice([1, 2, 4, 8]))
        sw = dw = {1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}[es]
        code = 0
    else:
        sw, dw, code = _SRC_WORD[pair[0]], _DST_WORD[pair[1]], oracle.CAST_CODES[pair]
    se, de = np.dtype(sw).itemsize, np.dtype(dw).itemsize
    nd = int(rng.integers(1, 5))
    shape = [int(x) for x in rng.integers(1, {1: 5000, 2: 300, 3: 60, 4: 20}[nd], nd)]
    ss, s_span = _random_layout(rng, shape)
    ds, d_span = _random_layout(rng, shape)
    so, do = int(rng.integers(0, 9)), int(rng.integers(0, 9))
    raw = rng.integers(0, 1 << 63, so + s_span + 8, dtype=np.uint64).astype(sw)
    view = np.lib.stride_tricks.as_strided(raw[so:], shape, [x * se for x in ss])
    conv = view.copy() if code == 0 else oracle_c.cast(code, np.ascontiguousarray(view).reshape(-1)).reshape(shape)
    fill = np.array(0xEEEEEEEEEEEEEEEE, dtype=np.uint64).astype(dw)
    want = np.full(do + d_span + 8, fill, dtype=dw)
    np.lib.stride_tricks.as_strided(want[do:], shape, [x * de for x in ds])[...] = conv
    d = torch.from_numpy(np.full(want.size * de, 0xEE, dtype=np.uint8)).cuda()
    dev = _dev(raw.view(np.uint8))
    gpu_engine.copy_view(dev[so * se:], d[do * de:], shape, de, src_strides=ss, dst_strides=ds, cast=code, checksum=False)
    assert np.array_equal(d.cpu().numpy().view(dw), want), (pair, shape, ss, ds, so, do)


def test_mla_absorbed_weights_on_device(gpu_engine, oracle, oracle_c):
    # engines/vllm/refit/receiver.py:244-261 on a strided view of kv_b_proj (no intermediate copy)
    H, nope, v, L, es = 16, 128, 128, 512, 2
    rng = np.random.default_rng(18)
    raw = rng.integers(0, 256, H * (nope + v) * L * es, dtype=np.uint8)
    kv_b = oracle.OTensor(raw.reshape(H * (nope + v), L, es), "BF16")
    want_uv, want_ukt = oracle.mla_absorbed_weights(kv_b, H, nope, v)
    d = _dev(raw)
    strides = ((nope + v) * L, L, 1)
    uv = torch.zeros(v * H * L * es, dtype=torch.uint8, device="cuda")
    ukt = torch.zeros(nope * L * H * es, dtype=torch.uint8, device="cuda")
    c_uv = gpu_engine.permute_copy(d[nope * L * es:], uv, (H, v, L), (1, 0, 2), es, src_strides=strides)
    c_ukt = gpu_engine.permute_copy(d, ukt, (H, nope, L), (1, 2, 0), es, src_strides=strides)
    assert uv.cpu().numpy().tobytes() == want_uv.tobytes()
    assert ukt.cpu().numpy().tobytes() == want_ukt.tobytes()
    assert c_uv == oracle.safe_checksum(want_uv) and c_ukt == oracle.safe_checksum(want_ukt)


@pytest.mark.parametrize("seed", range(12))
def test_place_boxes_random_batches(gpu_engine, oracle, oracle_c, seed):
    """Random batches of pitched boxes with every alignment class (16 / 8 / 4 / 2 / 1 byte
    units), copies and casts mixed, rows from 1 to thousands, wide rows split by columns."""
    rng = np.random.default_rng(500 + seed)
    src = rng.integers(0, 256, 6 << 20, dtype=np.uint8)
    f32 = src.view(np.uint32)
    d_src = _dev(src)
    out_size = 8 << 20
    want = np.full(out_size, 0xEE, dtype=np.uint8)
    boxes, sums_want, cursor = [], [], 0
    for g in range(int(rng.integers(1, 9))):
        cast = int(rng.choice([0, 0, 0, 1, 2, 3, 4, 5, 6, 7]))  # MXP_CAST_* code
        narrow, widen = cast in (1, 4), cast in (2, 3, 5)
        align = int(rng.choice([1, 2, 4, 8, 16])) if not cast else int(rng.choice([4, 8, 16]) if cast in (2, 3) else rng.choice([2, 4, 8, 16]))
        rows = int(rng.choice([1, 1, 2, 7, 64, 513, 3000]))
        row_bytes = int(rng.integers(1, 40)) * align if rng.integers(0, 4) else int(rng.integers(1, 5)) * 20000 // align * align
        row_bytes = max(align, row_bytes - row_bytes % (4 if cast in (2, 3) else 2 if cast else 1))
        src_row = row_bytes * 2 if narrow else row_bytes // 2 if widen else row_bytes
        src_align = align * 2 if narrow else align // 2 if widen else align
        dst_pitch = row_bytes + int(rng.integers(0, 4)) * align
        src_pitch = src_row + int(rng.integers(0, 5)) * src_align
        if rows * max(dst_pitch, 1) > (1 << 20) or rows * src_pitch > (4 << 20):
            rows = max(1, min((1 << 20) // dst_pitch, (4 << 20) // src_pitch))
        src_off = int(rng.integers(0, 64)) * (4 if narrow else 2 if cast in (2, 3, 6, 7) else 1)
        src_off -= src_off % (min(src_align, 16) if cast else min(align, 16))
        dst_off = (cursor + 15) // 16 * 16
        if rows == 1 and not cast and align < 16 and rng.integers(0, 2):
            dst_off += align  # a byte/dword-granular start inside the buffer
        csum = 0
        for r in range(rows):
            s = src[src_off + r * src_pitch: src_off + r * src_pitch + src_row]
            if cast == 1:
                s = oracle.cast_f32_bf16_bits(s.view(np.uint32)).view(np.uint8)
            elif cast == 4:
                s = oracle.cast_f32_f16_bits(s.view(np.uint32)).view(np.uint8)
            elif cast == 2:
                s = oracle.cast_bf16_f32_bits(s.view(np.uint16)).view(np.uint8)
            elif cast == 3:
                s = oracle.cast_f16_f32_bits(s.view(np.uint16)).view(np.uint8)
            elif cast == 5:
                s = oracle.cast_f8e4m3_bf16_bits(s).view(np.uint8)
            elif cast == 6:
                s = oracle.cast_f32_bf16_bits(oracle.cast_f16_f32_bits(s.view(np.uint16))).view(np.uint8)
            elif cast == 7:
                s = oracle.cast_f32_f16_bits(oracle.cast_bf16_f32_bits(s.view(np.uint16))).view(np.uint8)
            want[dst_off + r * dst_pitch: dst_off + r * dst_pitch + row_bytes] = s
            csum += int(oracle_c.checksum32(s, first_index=1000 + r * dst_pitch), 16)
        sums_want.append(format(csum & 0xFFFFFFFF, "08x"))
        boxes.append({"src": d_src.data_ptr() + src_off, "dst": dst_off, "src_pitch": src_pitch, "dst_pitch": dst_pitch,
                      "rows": rows, "row_bytes": row_bytes, "csum_index": 1000, "csum_group": g, "cast": cast})
        cursor = dst_off + rows * dst_pitch + 64
        assert cursor < out_size
    out = torch.full((out_size,), 0xEE, dtype=torch.uint8, device="cuda")
    for b in boxes:
        b["dst"] = out.data_ptr() + b["dst"]
    sums = gpu_engine.place_boxes(boxes, len(boxes))
    assert np.array_equal(out.cpu().numpy(), want)
    assert sums == sums_want


@pytest.mark.gpu
@pytest.mark.parametrize("cast", [0, 1, 2, 4, 5, 7])
@pytest.mark.parametrize("row_bytes,src_extra,dst_pitched", [(1024, 7, False), (256, 1, True), (4096, 3, False), (16, 0, False)])
def test_column_slices_out_of_power_of_two_pitches(gpu_engine, oracle, oracle_c, cast, row_bytes, src_extra, dst_pitched):
    """Row gathers out of power-of-two flavoured pitches, whole batches of rows plus a ragged rest: the
    o_proj slice of installer.py:292-317 (4096 rows of 1 KiB out of 8 KiB) and its like, also through
    every kind of conversion, with a column offset and a pitched destination.  Bytes and checksums
    against the oracle."""
    rng = np.random.default_rng(cast * 131 + row_bytes)
    narrow, widen = cast in (1, 4), cast in (2, 3, 5)
    src_row = row_bytes * 2 if narrow else row_bytes // 2 if widen else row_bytes
    units = row_bytes // (8 if narrow else 16)
    tile_rows = 8192 // units
    rows = 3 * tile_rows + tile_rows // 2 + 5  # three whole tiles and a ragged rest
    src_pitch = (src_row + 2047) // 2048 * 2048 + 2048 * src_extra
    dst_pitch = (row_bytes + 2047) // 2048 * 2048 + 2048 if dst_pitched else row_bytes
    col = 3 * src_row if 4 * src_row <= src_pitch else 0
    src = rng.integers(0, 256, rows * src_pitch, dtype=np.uint8)
    if cast in (1, 4):  # a few NaNs, infinities and denormals among the fp32 inputs
        w = src.view(np.uint32)
        w[:: 977] = 0x7FC12345
        w[5:: 1201] = 0xFF800000
        w[7:: 1409] = 0x00000123
    want = np.full(rows * dst_pitch + 64, 0xEE, dtype=np.uint8)
    conv = {0: lambda s: s,
            1: lambda s: oracle.cast_f32_bf16_bits(s.view(np.uint32)).view(np.uint8),
            2: lambda s: oracle.cast_bf16_f32_bits(s.view(np.uint16)).view(np.uint8),
            4: lambda s: oracle.cast_f32_f16_bits(s.view(np.uint32)).view(np.uint8),
            5: lambda s: oracle.cast_f8e4m3_bf16_bits(s).view(np.uint8),
            7: lambda s: oracle.cast_f32_f16_bits(oracle.cast_bf16_f32_bits(s.view(np.uint16))).view(np.uint8)}[cast]
    csum = 0
    for r in range(rows):
        piece = conv(src[r * src_pitch + col: r * src_pitch + col + src_row])
        want[32 + r * dst_pitch: 32 + r * dst_pitch + row_bytes] = piece
        csum += int(oracle_c.checksum32(piece, first_index=77 + r * dst_pitch), 16)
    d_src = _dev(src)
    out = torch.full((want.size,), 0xEE, dtype=torch.uint8, device="cuda")
    sums = gpu_engine.place_boxes([{"src": d_src.data_ptr() + col, "dst": out.data_ptr() + 32, "src_pitch": src_pitch, "dst_pitch": dst_pitch,
                                    "rows": rows, "row_bytes": row_bytes, "csum_index": 77, "csum_group": 0, "cast": cast}], 1)
    assert np.array_equal(out.cpu().numpy(), want)
    assert sums == [format(csum & 0xFFFFFFFF, "08x")]


@pytest.mark.gpu
@pytest.mark.parametrize("rows,row_bytes,pitch,col", [(4096, 8192, None, 0), (8192, 1024, 8192, 3072), (2341, 3584, 28672, 10752),
                                                      (100000, 64, 512, 192), (7, 16, 48, 32)])
def test_bare_gather_probe_moves_what_the_placement_kernel_moves(gpu_engine, mxp, rows, row_bytes, pitch, col):
    """``mxp_measure_gather`` times a bare kernel on an access shape; before it reports a rate it checks
    its own output against the placement kernel's gather of the same rows (it fails with MXP_ERR_STATE
    otherwise), so a positive figure here means the probe moved the right bytes."""
    rate = gpu_engine.measure_gather(rows, row_bytes, pitch, col, repeats=2)
    assert rate > 0
    if row_bytes % 32 == 0 and pitch is not None:  # the same source rows read as fp32 and stored as bf16
        assert gpu_engine.measure_gather(rows, row_bytes // 2, pitch, col, repeats=2, cast=1) > 0
    elif pitch is None:
        assert gpu_engine.measure_gather(rows, row_bytes // 2, None, 0, repeats=2, cast=1) > 0
    with pytest.raises(mxp.MxpError):
        gpu_engine.measure_gather(16, 24, 64)  # rows that are not a multiple of 16 bytes
    with pytest.raises(mxp.MxpError):
        gpu_engine.measure_gather(16, 64, 96, 48)  # the column runs past the pitch


@pytest.mark.gpu
def test_operator_calls_back_to_back_on_two_streams_keep_their_own_tables(gpu_engine):
    """Stand-alone operator calls take their descriptor tables from two staging arenas in turn and do not
    wait for each other's kernels: sixty calls of changing shapes, alternating between two streams with
    nothing synchronised in between, must each move exactly their own rows (a table overwritten under a
    running launch, or read before its upload, would show up as rows from another call's geometry)."""
    rng = np.random.default_rng(99)
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    src = torch.from_numpy(rng.integers(0, 256, 80 << 20, dtype=np.uint8)).cuda()
    torch.cuda.synchronize()
    calls = []
    for k in range(60):
        rows = int(rng.choice([1, 3, 64, 500, 2048]))
        row_bytes = int(rng.choice([16, 48, 1024, 3584, 8192]))
        pitch = row_bytes + 16 * int(rng.integers(0, 9)) if rows > 1 else row_bytes
        first = 16 * int(rng.integers(0, 1000))
        big = k % 7 == 0  # some calls long enough for the next ones to be issued while they run
        if big:
            rows, row_bytes, pitch = 8192, 4096, 8192
        assert first + (rows - 1) * pitch + row_bytes <= src.numel()  # the library is handed raw addresses: bounds are the caller's
        out = torch.full((rows * row_bytes,), 0xEE, dtype=torch.uint8, device="cuda")
        st = streams[k % 2]
        with torch.cuda.stream(st):
            if k % 3 == 2 and row_bytes % 2 == 0 and rows > 1:  # a transposed view: the other launch path and its own table
                n_el = row_bytes // 2
                gpu_engine.copy_view(src[first:], out, (n_el, rows), 2, src_strides=(1, pitch // 2), stream=st.cuda_stream, checksum=False)
                calls.append(("t", first, rows, n_el, pitch, out))
            else:
                gpu_engine.copy_view(src[first:], out, (rows, row_bytes), 1, src_strides=(pitch, 1), stream=st.cuda_stream, checksum=False)
                calls.append(("g", first, rows, row_bytes, pitch, out))
    torch.cuda.synchronize()
    host = src.cpu().numpy()
    for kind, first, rows, width, pitch, out in calls:
        got = out.cpu().numpy()
        if kind == "g":
            want = np.lib.stride_tricks.as_strided(host[first:], (rows, width), (pitch, 1)).reshape(-1)
        else:
            want = np.lib.stride_tricks.as_strided(host[first:].view(np.uint16), (width, rows), (2, pitch)).reshape(-1).view(np.uint8)
        assert np.array_equal(got, want), (kind, first, rows, width, pitch)

