"""CPU oracle for the weight-placement path.  TEST INFRASTRUCTURE ONLY.

A plain numpy / pure-Python restatement of the reference's algorithm for every stage
of the path, each function citing the reference file:line it follows
(paths relative to modelexpress_client/python/ in ai-dynamo/modelexpress v0.5.0).
Nothing in the product (the ``modelexpress_amd`` package or libmxplace.so) imports,
links or executes this module: only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` do, and only as the checker.

Tensor representation.  numpy has no bfloat16 / float8, and every stage except the
cast only moves bytes, so a tensor is held as a ``uint8`` array of shape
``(*shape, itemsize)`` next to its safetensors dtype string (class ``OTensor``).
``narrow`` on a logical axis is then ordinary numpy slicing, and an in-place view
assignment has exactly the semantics of ``torch.Tensor.copy_`` into a view.

How each function is pinned (no function here is "parity unpinned"):
  parse_safetensors_header / resolve_safetensors_files
      the public safetensors byte format, cross-checked against the installed
      third-party ``safetensors`` reader; the hand-built header of the reference's
      tests/test_gds_loader.py:126-149; error cases of gds_loader.py:254-262.
  MdlOracle (TP slice, fused, premerged, expert, scales)
      the reference's own vectors: tests/test_mdl_tp.py:28-81,
      tests/test_mdl_fp8.py:31-169,202-228,279-434; closed forms ``np.concatenate`` of
      ``x[r*n:(r+1)*n]`` slices.
  paired_runs        tests/test_reshard_refit_slice_plan.py:54-65,82-96 + element brute force.
  cast_f32_bf16      torch CPU ``.to(torch.bfloat16)`` (third-party library present in the
                     image) on every exponent/rounding class; hand values.
  safe_checksum      hand-computed values, the closed form for constant buffers,
                     a big-integer brute force written straight from the formula,
                     the inequalities of tests/test_tensor_utils.py:255-284.
  tensor_digest      hashlib.blake2b (the library the reference calls), arithmetic-series
                     closed forms for the scalars, the invariants of
                     tests/test_reshard_refit_verify.py:43-171.
"""

from __future__ import annotations

import hashlib
import itertools
import json
import os
import struct
from collections import defaultdict
from dataclasses import dataclass
from pathlib import Path

import numpy as np

# --------------------------------------------------------------------------------------
# dtypes (gds_loader.py:36-49)
# --------------------------------------------------------------------------------------
DTYPE_SIZE = {
    "F64": 8, "F32": 4, "F16": 2, "BF16": 2, "F8_E4M3": 1, "F8_E5M2": 1,
    "I64": 8, "I32": 4, "I16": 2, "I8": 1, "U8": 1, "BOOL": 1,
}
FP8_DTYPES = ("F8_E4M3", "F8_E5M2")


@dataclass
class OTensor:
    """A tensor as raw bytes: ``data`` is uint8 with shape ``(*shape, itemsize)``."""

    data: np.ndarray
    dtype: str

    @property
    def shape(self) -> tuple:
        return tuple(self.data.shape[:-1])

    @property
    def ndim(self) -> int:
        return self.data.ndim - 1

    def numel(self) -> int:
        return int(np.prod(self.shape, dtype=np.int64)) if self.shape else 1

    def narrow(self, axis: int, start: int, size: int) -> "OTensor":
        idx = [slice(None)] * self.data.ndim
        idx[axis] = slice(start, start + size)
        return OTensor(self.data[tuple(idx)], self.dtype)

    def tobytes(self) -> bytes:
        return np.ascontiguousarray(self.data).tobytes()

    @staticmethod
    def zeros(shape, dtype: str) -> "OTensor":
        return OTensor(np.zeros(tuple(shape) + (DTYPE_SIZE[dtype],), dtype=np.uint8), dtype)

    @staticmethod
    def from_array(arr: np.ndarray, dtype: str) -> "OTensor":
        """Wrap a typed numpy array (float32, uint16 bit patterns, uint8 ...)."""
        arr = np.ascontiguousarray(arr)
        if arr.dtype.itemsize != DTYPE_SIZE[dtype]:
            raise ValueError(f"{arr.dtype} does not match {dtype}")
        return OTensor(arr.view(np.uint8).reshape(arr.shape + (arr.dtype.itemsize,)), dtype)

    @staticmethod
    def from_bytes(raw, shape, dtype: str) -> "OTensor":
        a = np.frombuffer(raw, dtype=np.uint8)
        return OTensor(a.reshape(tuple(shape) + (DTYPE_SIZE[dtype],)), dtype)


def _reshape_view(a: np.ndarray, shape) -> np.ndarray:
    """Reshape that is guaranteed to alias ``a`` (raises instead of copying)."""
    v = a.view()
    v.shape = shape
    return v


# --------------------------------------------------------------------------------------
# a1: safetensors parse (gds_loader.py:189-282)
# --------------------------------------------------------------------------------------
def parse_safetensors_header(file_path: str) -> dict:
    """gds_loader.py:245-282: ``{name: {file_offset, size, dtype, shape}}``."""
    with open(file_path, "rb") as f:
        raw = f.read(8)
        if len(raw) < 8:
            raise RuntimeError(f"Invalid safetensors file: {file_path}")
        (header_size,) = struct.unpack("<Q", raw)
        if header_size > 100 * 1024 * 1024:
            raise RuntimeError(f"Safetensors header too large ({header_size} bytes): {file_path}")
        header_bytes = f.read(header_size)
    header = json.loads(header_bytes)
    data_start = 8 + header_size
    out = {}
    for name, info in header.items():
        if name == "__metadata__":
            continue
        b, e = info["data_offsets"]
        out[name] = {"file_offset": data_start + b, "size": e - b, "dtype": info["dtype"], "shape": info["shape"]}
    return out


def resolve_safetensors_files(model_path: str) -> dict:
    """gds_loader.py:189-243: ``{file: [tensor names]}``, index -> single file -> glob."""
    model_dir = Path(model_path)
    index_path = model_dir / "model.safetensors.index.json"
    if index_path.exists():
        with open(index_path) as f:
            weight_map = json.load(f).get("weight_map", {})
        if not weight_map:
            raise RuntimeError(f"Empty weight_map in {index_path}")
        files = defaultdict(list)
        for tensor_name, filename in weight_map.items():
            files[str(model_dir / filename)].append(tensor_name)
        return dict(files)
    single = model_dir / "model.safetensors"
    if single.exists():
        return {str(single): list(parse_safetensors_header(str(single)).keys())}
    st_files = sorted(model_dir.glob("*.safetensors"))
    if not st_files:
        raise FileNotFoundError(f"No .safetensors files found in {model_path}")
    return {str(p): list(parse_safetensors_header(str(p)).keys()) for p in st_files}


def load_checkpoint(model_path: str, mmap: bool = True) -> list:
    """a2: every tensor of the checkpoint as ``(name, OTensor)``, files in resolution
    order and tensors by ascending file offset (gds_loader.py:297-300,327-328:
    ``raw.view(dtype).reshape(shape)``)."""
    out = []
    if os.path.isfile(model_path):
        file_map = {model_path: list(parse_safetensors_header(model_path).keys())}
    else:
        file_map = resolve_safetensors_files(model_path)
    for file_path, names in file_map.items():
        info = parse_safetensors_header(file_path)
        wanted = [n for n in names if n in info]
        wanted.sort(key=lambda n: info[n]["file_offset"])
        raw = np.memmap(file_path, dtype=np.uint8, mode="r") if mmap else np.fromfile(file_path, dtype=np.uint8)
        for n in wanted:
            i = info[n]
            if i["dtype"] not in DTYPE_SIZE:
                raise RuntimeError(f"Unsupported safetensors dtype '{i['dtype']}' for tensor '{n}'")
            if i["file_offset"] + i["size"] > raw.shape[0]:
                raise RuntimeError(f"read past end of file for tensor '{n}'")
            seg = raw[i["file_offset"] : i["file_offset"] + i["size"]]
            out.append((n, OTensor(seg.reshape(tuple(i["shape"]) + (DTYPE_SIZE[i["dtype"]],)), i["dtype"])))
    return out


# --------------------------------------------------------------------------------------
# a9: fp32 -> bf16 (torch copy_ at modelexpress_rl/train/engines/fsdp/adapter.py:203-206,
# refit/reshard/receiver.py:964-971).  Round to nearest even on the bit pattern; every
# NaN maps to one image.  c10's scalar conversion gives 0x7FC0; torch's AVX-512 CPU
# kernel gives 0xFFFF -- the image is a parameter so either can be checked.
# --------------------------------------------------------------------------------------
def cast_f32_bf16_bits(u32: np.ndarray, nan_bits: int = 0x7FC0) -> np.ndarray:
    u = u32.astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    is_nan = (u & 0x7FFFFFFF) > 0x7F800000
    return np.where(is_nan, np.uint16(nan_bits), r)


def cast_tensor_f32_bf16(t: OTensor, nan_bits: int = 0x7FC0) -> OTensor:
    if t.dtype != "F32":
        raise ValueError("cast source must be F32")
    u32 = np.ascontiguousarray(t.data).view("<u4").reshape(t.shape)
    return OTensor.from_array(cast_f32_bf16_bits(u32, nan_bits).astype("<u2"), "BF16")


# The receive side of the same path converts the other way: "Cast the served bf16 staging
# into the (fp32) receive buffer - a torch op" (refit/reshard/receiver.py:962-969), and a
# half-precision engine takes fp32 trainer weights as fp16.  Conversion codes, shared with
# the product's write records: 1 fp32->bf16, 2 bf16->fp32, 3 fp16->fp32, 4 fp32->fp16,
# 5 fp8-e4m3 -> bf16 (the ``.to(out_dtype)`` of the MLA absorbed weights when ``kv_b_proj`` is
# stored in fp8: engines/vllm/refit/receiver.py:258-261).
# 6 fp16 -> bf16 and 7 bf16 -> fp16 go through fp32, as torch's copy_ does between the two 16-bit formats.
CAST_CODES = {("F32", "BF16"): 1, ("BF16", "F32"): 2, ("F16", "F32"): 3, ("F32", "F16"): 4, ("F8_E4M3", "BF16"): 5,
              ("F16", "BF16"): 6, ("BF16", "F16"): 7}


def cast_bf16_f32_bits(u16: np.ndarray) -> np.ndarray:
    """Exact: bf16 is the upper half of the fp32 pattern (NaN payloads are kept)."""
    return u16.astype(np.uint32) << np.uint32(16)


_F16_TOP_BIT = np.array([0] + [int(m).bit_length() - 1 for m in range(1, 1024)], dtype=np.uint32)


def cast_f16_f32_bits(u16: np.ndarray) -> np.ndarray:
    """Exact widening.  Subnormal halves are renormalised; a NaN keeps its payload and is
    made quiet (what hardware converters and torch's CPU path produce)."""
    h = u16.astype(np.uint32)
    sign = (h & 0x8000) << 16
    e = (h >> 10) & 0x1F
    m = h & 0x3FF
    normal = sign | ((e + 112) << 23) | (m << 13)
    top = _F16_TOP_BIT[m]
    sub = np.where(m == 0, sign, sign | ((top + 103) << 23) | ((m << (23 - top)) & 0x7FFFFF))
    special = sign | 0x7F800000 | (m << 13) | np.where(m != 0, np.uint32(0x400000), np.uint32(0))
    return np.where(e == 31, special, np.where(e == 0, sub, normal)).astype(np.uint32)


def cast_f32_f16_bits(u32: np.ndarray) -> np.ndarray:
    """fp32 -> fp16, round to nearest even; overflow goes to infinity, values below half
    the smallest subnormal to (signed) zero; a NaN keeps the top ten payload bits and is made
    quiet (the hardware converters' rule, which torch's CPU path follows)."""
    u = u32.astype(np.uint64)
    sign = (u >> 16) & 0x8000
    a = u & 0x7FFFFFFF
    # normal half range: re-bias the exponent, round the 13 dropped bits to nearest even
    r = (a - 0x38000000) & 0xFFFFFFFF
    hn = np.minimum((r + 0xFFF + ((r >> 13) & 1)) >> 13, 0x7C00)
    # subnormal half: shift the 24-bit significand right, round to nearest even
    e = a >> 23
    m = (a & 0x7FFFFF) | 0x800000
    shift = np.minimum(126 - np.minimum(e, 126), 25).astype(np.uint64)
    q = m >> shift
    rem = m & ((np.uint64(1) << shift) - 1)
    half = np.uint64(1) << (shift - 1)
    hs = q + ((rem > half) | ((rem == half) & ((q & 1) == 1)))
    out = np.where(a >= 0x38800000, hn, hs)
    out = np.where(a > 0x7F800000, 0x7E00 | ((a >> 13) & 0x3FF), out)
    return (sign | out).astype(np.uint16)


_F8_TOP_BIT = np.array([0, 0, 1, 1, 2, 2, 2, 2], dtype=np.uint16)


def cast_f8e4m3_bf16_bits(u8: np.ndarray) -> np.ndarray:
    """Exact: e4m3fn (bias 7, no infinities, 0x7F / 0xFF = NaN) into bf16.  Subnormals
    (m * 2^-9) are renormalised; both NaN codes become 0x7FC0, as torch's conversion does."""
    c = u8.astype(np.uint16)
    sign = (c & 0x80) << 8
    e = (c >> 3) & 0xF
    m = c & 7
    top = _F8_TOP_BIT[m]
    sub = np.where(m == 0, sign, sign | ((top + 118) << 7) | ((m << (7 - top)) & 0x7F))
    normal = sign | ((e + 120) << 7) | (m << 4)
    out = np.where(e == 0, sub, normal)
    return np.where((e == 15) & (m == 7), np.uint16(0x7FC0), out).astype(np.uint16)


def cast_tensor(t: OTensor, dst_dtype: str, nan_bits: int = 0x7FC0) -> OTensor:
    """dtype conversion of ``dest.copy_(src)`` for the supported pairs."""
    code = CAST_CODES.get((t.dtype, dst_dtype))
    if code is None:
        raise ValueError(f"no conversion from {t.dtype} to {dst_dtype}")
    src = np.ascontiguousarray(t.data)
    if code == 1:
        return cast_tensor_f32_bf16(t, nan_bits)
    if code == 4:
        return OTensor.from_array(cast_f32_f16_bits(src.view("<u4").reshape(t.shape)).astype("<u2"), "F16")
    if code == 5:
        return OTensor.from_array(cast_f8e4m3_bf16_bits(src.view("u1").reshape(t.shape)).astype("<u2"), "BF16")
    if code == 6:
        u = cast_f32_bf16_bits(cast_f16_f32_bits(src.view("<u2").reshape(t.shape)), nan_bits)
        return OTensor.from_array(u.astype("<u2"), "BF16")
    if code == 7:
        u = cast_f32_f16_bits(cast_bf16_f32_bits(src.view("<u2").reshape(t.shape)))
        return OTensor.from_array(u.astype("<u2"), "F16")
    fn = cast_bf16_f32_bits if code == 2 else cast_f16_f32_bits
    return OTensor.from_array(fn(src.view("<u2").reshape(t.shape)).astype("<u4"), "F32")


# --------------------------------------------------------------------------------------
# a10: safe_checksum (tensor_utils.py:27-44) over the row-major flat byte stream
# --------------------------------------------------------------------------------------
KNUTH = 2654435761


def safe_checksum_bytes(raw) -> str:
    """Vectorised form: sum_i b_i * ((i*K + 1) mod 2^32) mod 2^32, as 8 hex digits."""
    b = np.frombuffer(raw, dtype=np.uint8) if not isinstance(raw, np.ndarray) else raw.reshape(-1)
    total = 0
    step = 1 << 22
    for lo in range(0, b.shape[0], step):
        blk = b[lo : lo + step].astype(np.uint64)
        idx = np.arange(lo, lo + blk.shape[0], dtype=np.uint64)
        w = (idx * np.uint64(KNUTH) + np.uint64(1)) & np.uint64(0xFFFFFFFF)
        total = (total + int(((blk * w) & np.uint64(0xFFFFFFFF)).sum(dtype=np.uint64))) & 0xFFFFFFFF
    return format(total, "08x")


def safe_checksum_bigint(raw: bytes) -> str:
    """The formula of tensor_utils.py:39-42 in unbounded Python integers (small inputs)."""
    total = 0
    for i, byte in enumerate(bytes(raw)):
        weight = (i * KNUTH + 1) & 0xFFFFFFFF
        total += (byte * weight) & 0xFFFFFFFF
    return format(total & 0xFFFFFFFF, "08x")


def safe_checksum(t: OTensor, reference_literal: bool = False) -> str:
    """Checksum of the tensor's row-major bytes.

    With ``reference_literal`` the outcome of the reference's op sequence is reproduced
    for shapes where it does not produce a value: its uint8 view keeps the leading dims
    while the weight vector is 1-D (tensor_utils.py:38-41), so for a tensor with two or
    more dims and a leading dim other than 1 the multiply cannot broadcast and the
    function returns an ``err:`` string (tensor_utils.py:43-44).
    """
    if reference_literal and t.ndim >= 2 and any(int(d) != 1 for d in t.shape[:-1]):
        return "err:shape"
    return safe_checksum_bytes(t.tobytes())


# --------------------------------------------------------------------------------------
# a11: tensor_digest / shard_region (refit/reshard/verify.py:57-183)
# --------------------------------------------------------------------------------------
ROW_WORDS = 1024  # verify.py:57
U64 = (1 << 64) - 1


def tensor_digest_scalars(raw) -> list:
    """verify.py:112-150: the ordered scalar list that gets hashed."""
    b = np.frombuffer(raw, dtype=np.uint8) if not isinstance(raw, np.ndarray) else np.ascontiguousarray(raw).reshape(-1)
    n = int(b.shape[0])
    body = n - (n % 4)
    words = np.frombuffer(b[:body].tobytes(), dtype="<i4")
    rows = words.shape[0] // ROW_WORDS
    scalars = [n]
    if rows:
        row_sums = words[: rows * ROW_WORDS].reshape(rows, ROW_WORDS).sum(axis=1, dtype=np.int64)
        weights = np.arange(1, rows + 1, dtype=np.int64)
        scalars.append(int(row_sums.sum(dtype=np.int64)))
        with np.errstate(over="ignore"):
            scalars.append(int((row_sums * weights).sum(dtype=np.int64)))
    tail = words[rows * ROW_WORDS :]
    if tail.shape[0]:
        t64 = tail.astype(np.int64)
        scalars.append(int(t64.sum(dtype=np.int64)))
        scalars.append(int((t64 * np.arange(1, t64.shape[0] + 1, dtype=np.int64)).sum(dtype=np.int64)))
    if n % 4:
        scalars.append(int(b[body:].astype(np.int64).sum()))
        scalars.append(n % 4)
    return scalars


def tensor_digest_bytes(raw) -> str:
    h = hashlib.blake2b(digest_size=16)  # verify.py:152-155
    for value in tensor_digest_scalars(raw):
        h.update((value & U64).to_bytes(8, "little"))
    return h.hexdigest()


def tensor_digest(t: OTensor) -> str:
    """Digest of the tensor's contiguous bytes; a strided or offset view digests as its
    contiguous copy (verify.py:95-111)."""
    return tensor_digest_bytes(t.tobytes())


def shard_region(full: OTensor, global_shape, shard_offset, shape) -> OTensor:
    """verify.py:158-183."""
    if not len(global_shape) == len(shard_offset) == len(shape):
        raise ValueError(
            f"rank mismatch: global_shape {tuple(global_shape)}, shard_offset "
            f"{tuple(shard_offset)} and shape {tuple(shape)} must have equal rank"
        )
    itemsize = full.data.shape[-1]
    view = OTensor(np.ascontiguousarray(full.data).reshape(tuple(global_shape) + (itemsize,)), full.dtype)
    for axis, (start, extent) in enumerate(zip(shard_offset, shape)):
        view = view.narrow(axis, int(start), int(extent))
    return OTensor(np.ascontiguousarray(view.data), full.dtype)


# --------------------------------------------------------------------------------------
# a12: run decomposition (refit/reshard/slice_plan.py:86-90,248-294)
# --------------------------------------------------------------------------------------
def row_major_strides(shape) -> list:
    strides = [1] * len(shape)
    for d in range(len(shape) - 2, -1, -1):
        strides[d] = strides[d + 1] * shape[d + 1]
    return strides


def intersect(box_a, box_b):
    out = []
    for (a0, a1), (b0, b1) in zip(box_a, box_b):
        lo, hi = max(a0, b0), min(a1, b1)
        if lo >= hi:
            return None
        out.append((lo, hi))
    return out


def paired_runs(overlap, src_origin, src_strides, dst_origin, dst_strides):
    """slice_plan.py:259-294: ``(src_elem_off, dst_elem_off, run_len)`` triples."""
    ndim = len(overlap)
    sizes = [hi - lo for lo, hi in overlap]
    src_start = [lo - o for (lo, _), o in zip(overlap, src_origin)]
    dst_start = [lo - o for (lo, _), o in zip(overlap, dst_origin)]
    run_len = 1
    p = ndim
    while p - 1 >= 0 and src_strides[p - 1] == run_len and dst_strides[p - 1] == run_len:
        run_len *= sizes[p - 1]
        p -= 1
    src_base = sum(src_start[d] * src_strides[d] for d in range(ndim))
    dst_base = sum(dst_start[d] * dst_strides[d] for d in range(ndim))
    if p == 0:
        yield src_base, dst_base, run_len
        return
    for idx in itertools.product(*[range(sizes[d]) for d in range(p)]):
        yield (
            src_base + sum(idx[d] * src_strides[d] for d in range(p)),
            dst_base + sum(idx[d] * dst_strides[d] for d in range(p)),
            run_len,
        )


# --------------------------------------------------------------------------------------
# permuted copies: ``dest.copy_(src.permute(...))`` -- the MLA absorbed weights
# W_UV = w_uv.transpose(0, 1), W_UK_T = w_uk.permute(1, 2, 0)
# (engines/vllm/refit/receiver.py:244-261) and permuted box views (slice_plan.py:166-220)
# --------------------------------------------------------------------------------------
def permute_copy(t: OTensor, perm) -> OTensor:
    """Contiguous copy of ``t.permute(perm)``; the element-byte axis stays last."""
    axes = tuple(int(p) for p in perm) + (t.data.ndim - 1,)
    return OTensor(np.ascontiguousarray(np.transpose(t.data, axes)), t.dtype)


def mla_absorbed_weights(kv_b_proj: OTensor, num_heads: int, qk_nope: int, v_head: int) -> tuple:
    """receiver.py:244-261: view [H, nope+v, L], split on dim 1, then W_UV = w_uv.transpose(0,1)
    -> [v, H, L] and W_UK_T = w_uk.permute(1,2,0) -> [nope, L, H]."""
    es = kv_b_proj.data.shape[-1]
    v3 = _reshape_view(np.ascontiguousarray(kv_b_proj.data), (num_heads, qk_nope + v_head, -1, es))
    w_uk = OTensor(v3[:, :qk_nope], kv_b_proj.dtype)
    w_uv = OTensor(v3[:, qk_nope:], kv_b_proj.dtype)
    return permute_copy(w_uv, (1, 0, 2)), permute_copy(w_uk, (1, 2, 0))


# --------------------------------------------------------------------------------------
# trainer-native layouts (modelexpress_rl/train/engines/megatron/aliases.py)
# --------------------------------------------------------------------------------------
def megatron_qkv_split(fused: OTensor, q_heads: int, kv_heads: int, head_dim: int) -> tuple:
    """Whole q, k, v from a by-KV-group interleaved fused tensor (aliases.py:206-263: per
    group its query rows, then one K head, then one V head)."""
    q_rows = (q_heads // kv_heads) * head_dim
    group_rows = q_rows + 2 * head_dim
    q, k, v = [], [], []
    for g in range(kv_heads):
        lo = g * group_rows
        q.append(fused.data[lo : lo + q_rows])
        k.append(fused.data[lo + q_rows : lo + q_rows + head_dim])
        v.append(fused.data[lo + q_rows + head_dim : lo + group_rows])
    return tuple(OTensor(np.concatenate(parts), fused.dtype) for parts in (q, k, v))


def assemble_virtual(full_shape, dtype: str, shards) -> OTensor:
    """A full tensor assembled from shards ``(source OTensor, source_offset, shard_offset,
    shape)``: what a receiver builds when it stages a whole logical tensor from its
    publishers (refit/reshard/transfer_plan.py:134-189) before re-slicing it."""
    out = OTensor.zeros(full_shape, dtype)
    hit = np.zeros(tuple(full_shape), dtype=np.int32)
    for src, src_off, shard_off, shape in shards:
        s_idx = tuple(slice(o, o + n) for o, n in zip(src_off, shape))
        d_idx = tuple(slice(o, o + n) for o, n in zip(shard_off, shape))
        out.data[d_idx] = src.data[s_idx]
        hit[d_idx] += 1
    if not np.all(hit == 1):
        raise CoverageError("virtual tensor shards leave gaps or overlap")
    return out


# --------------------------------------------------------------------------------------
# a4-a8: destination map and writes (engines/vllm/refit/installer.py)
# --------------------------------------------------------------------------------------
STACKED_GROUPS = (  # installer.py:72-78
    ("qkv_proj", "q_proj", 0),
    ("qkv_proj", "k_proj", 1),
    ("qkv_proj", "v_proj", 2),
    ("gate_up_proj", "gate_proj", 0),
    ("gate_up_proj", "up_proj", 1),
)
SCALE_NAME_ALIASES = (("weight_scale_inv", "weight_scale"), ("input_scale", "activation_scale"))  # :80-83


class CoverageError(RuntimeError):
    pass


class MdlOracle:
    """Destination-map loader over numpy buffers, following installer.py:86-843.

    ``params``: ``{name: OTensor}`` -- the rank's (local) parameters, written in place.
    ``stacked_params_mapping``: list of ``(fused_suffix, member_suffix)`` in pack order or
    None for the built-in groups.  ``expert_mapping``: rows
    ``(param_prefix, weight_prefix, expert_id, shard)``.  ``expert_local``: callable
    ``(fused_param_name, global_id) -> local id``; return ``None`` for "translation
    failed" and a negative id for "not local".
    """

    def __init__(self, params, tp_size=1, tp_rank=0, stacked_params_mapping=None, expert_mapping=None,
                 expert_local=None, allow_cast=False, nan_bits=0x7FC0):
        self.params = params
        self.tp_size = tp_size
        self.tp_rank = tp_rank
        self.stacked_params_mapping = stacked_params_mapping
        self.expert_mapping = expert_mapping
        self.expert_local = expert_local
        self.allow_cast = allow_cast
        self.nan_bits = nan_bits
        self.direct, self.fused, self.premerged, self.expert = {}, {}, {}, {}
        self.covered = set()
        self.skipped = []

    # ---- shape rules ----
    def tp_local_tensor(self, tensor: OTensor, expected_shape):  # installer.py:292-317
        expected_shape = tuple(expected_shape)
        if tensor.shape == expected_shape:
            return tensor
        if self.tp_size <= 1 or tensor.ndim != len(expected_shape):
            return None
        candidates = []
        for axis, (loaded, expected) in enumerate(zip(tensor.shape, expected_shape)):
            if int(loaded) != int(expected) * self.tp_size:
                continue
            if all(d == axis or int(tensor.shape[d]) == int(expected_shape[d]) for d in range(tensor.ndim)):
                candidates.append(axis)
        if len(candidates) != 1:
            return None
        axis = candidates[0]
        local = int(expected_shape[axis])
        return tensor.narrow(axis, self.tp_rank * local, local)

    def tp_shape_compatible(self, loaded_shape, expected_shape) -> bool:  # installer.py:319-339
        loaded_shape, expected_shape = tuple(loaded_shape), tuple(expected_shape)
        if loaded_shape == expected_shape:
            return True
        if self.tp_size <= 1 or len(loaded_shape) != len(expected_shape):
            return False
        mism = [i for i, (l, e) in enumerate(zip(loaded_shape, expected_shape)) if int(l) != int(e)]
        return len(mism) == 1 and int(loaded_shape[mism[0]]) == int(expected_shape[mism[0]]) * self.tp_size

    # ---- name rules ----
    @staticmethod
    def is_scale_name(name: str) -> bool:  # installer.py:440-449
        return name.endswith(("weight_scale", "weight_scale_inv", "input_scale", "activation_scale"))

    @staticmethod
    def param_candidates(name: str) -> tuple:  # installer.py:451-459
        cands = [name]
        for left, right in SCALE_NAME_ALIASES:
            if left in name:
                cands.append(name.replace(left, right))
            if right in name:
                cands.append(name.replace(right, left))
        return tuple(dict.fromkeys(cands))

    def find_param(self, name: str):  # installer.py:461-468
        for cand in self.param_candidates(name):
            p = self.params.get(cand)
            if p is not None:
                return cand, p
        return None

    def stacked_groups(self) -> tuple:  # installer.py:773-797
        groups = []
        if self.stacked_params_mapping:
            seen = {}
            for entry in self.stacked_params_mapping:
                fused = str(entry[0]).lstrip(".")
                member = str(entry[1]).lstrip(".")
                if not fused or not member or fused == member:
                    continue
                order = seen.get(fused, 0)
                seen[fused] = order + 1
                groups.append((fused, member, order))
        return tuple(groups) if groups else STACKED_GROUPS

    # ---- classification (installer.py:470-564) ----
    def extend_dest_map(self, weights) -> None:
        name_to_shape = {
            n: t.shape for n, t in weights if n not in self.direct and n not in self.fused and n not in self.expert
        }
        if not name_to_shape:
            return
        expert_lookup = {}
        for p_suf, w_suf, eid, shard in self.expert_mapping or ():
            expert_lookup[w_suf] = (p_suf, int(eid), shard)
        stacked = self.stacked_groups()
        counts = {}
        for fused_suf, _m, _o in stacked:
            counts[fused_suf] = counts.get(fused_suf, 0) + 1
        premerge_suffixes = {s: n for s, n in counts.items() if n == 2}  # installer.py:618-627
        groups = {}
        for hf_name, shape in name_to_shape.items():
            pm = self._premerged_destination(hf_name, shape, premerge_suffixes)
            if pm is not None:
                dest, parts, pname = pm
                self.premerged[hf_name] = (dest, parts)
                self.covered.add(pname)
                continue
            direct = self.find_param(hf_name)
            if direct is not None and self.tp_shape_compatible(shape, direct[1].shape):
                self.direct[hf_name] = direct[1]
                self.covered.add(direct[0])
                continue
            if ".experts." in hf_name and expert_lookup:
                res = self._resolve_expert(hf_name, shape, expert_lookup)
                if res == "skip":
                    self.skipped.append(hf_name)
                    self.direct[hf_name] = None  # marked: deliberately not placed
                    continue
                if res is not None:
                    self.expert[hf_name] = res[0]
                    self.covered.add(res[1])
                    continue
            for fused_suf, member_suf, order in stacked:
                if member_suf + "." in hf_name or hf_name.endswith(member_suf + ".weight"):
                    fused = self.find_param(hf_name.replace(member_suf, fused_suf))
                    if fused is None:
                        continue
                    groups.setdefault(fused[0], []).append((order, hf_name, shape))
                    break
        for fused_name, members in groups.items():
            members.sort(key=lambda m: m[0])
            dests = self._fused_destinations(self.params[fused_name], members)
            if dests is None:
                continue
            self.fused.update(dests)
            self.covered.add(fused_name)

    def _fused_destinations(self, fused_param: OTensor, members):  # installer.py:566-616
        data = fused_param
        if all(not shape for _o, _n, shape in members):
            if data.numel() == 1:
                flat = OTensor(_reshape_view(data.data, (1, -1)), data.dtype)
                return {name: OTensor(flat.data[0], data.dtype) for _o, name, _s in members}
            if data.numel() == len(members):
                flat = OTensor(_reshape_view(data.data, (len(members), -1)), data.dtype)
                return {name: OTensor(flat.data[i], data.dtype) for i, (_o, name, _s) in enumerate(members)}
            return None
        if not members or any(len(shape) != data.ndim for _o, _n, shape in members):
            return None
        candidates = []
        for axis in range(data.ndim):
            if not all(
                all(d == axis or int(shape[d]) == int(data.shape[d]) for d in range(data.ndim))
                for _o, _n, shape in members
            ):
                continue
            total = sum(int(shape[axis]) for _o, _n, shape in members)
            if total == int(data.shape[axis]):
                candidates.append((axis, 1))
            elif (
                self.tp_size > 1
                and total == int(data.shape[axis]) * self.tp_size
                and all(int(shape[axis]) % self.tp_size == 0 for _o, _n, shape in members)
            ):
                candidates.append((axis, self.tp_size))
        if not candidates:
            return None
        axis, divisor = candidates[0]
        offset, out = 0, {}
        for _o, name, shape in members:
            size = int(shape[axis]) // divisor
            out[name] = data.narrow(axis, offset, size)
            offset += size
        return out

    def _premerged_destination(self, hf_name, src_shape, premerge_suffixes):  # installer.py:629-668
        if self.tp_size <= 1 or not src_shape:
            return None
        if not any(hf_name.endswith(suf + ".weight") or (suf + ".") in hf_name for suf in premerge_suffixes):
            return None
        found = self.find_param(hf_name)
        if found is None:
            return None
        pname, param = found
        if param.ndim < 1 or len(src_shape) != param.ndim:
            return None
        parts = 2
        dest0, src0 = int(param.shape[0]), int(src_shape[0])
        if src0 != dest0 * self.tp_size:
            return None
        if dest0 % parts != 0 or src0 % (parts * self.tp_size) != 0:
            return None
        if any(int(src_shape[d]) != int(param.shape[d]) for d in range(1, param.ndim)):
            return None
        return param, parts, pname

    def _premerged_writes(self, dest: OTensor, parts: int, source: OTensor):  # installer.py:670-693
        src0, dst0 = int(source.shape[0]), int(dest.shape[0])
        if src0 % parts != 0 or dst0 % parts != 0:
            return None
        part_src, part_dst = src0 // parts, dst0 // parts
        if part_src != part_dst * self.tp_size:
            return None
        return [
            (dest.narrow(0, p * part_dst, part_dst), source.narrow(0, p * part_src + self.tp_rank * part_dst, part_dst))
            for p in range(parts)
        ]

    def _resolve_expert(self, hf_name, hf_shape, expert_lookup):  # installer.py:695-754
        for w_suf, (p_suf, eid, shard) in expert_lookup.items():
            if w_suf not in hf_name:
                continue
            fused = self.find_param(hf_name.replace(w_suf, p_suf))
            if fused is None:
                return None
            fused_name, fp = fused
            if fp.ndim < 1:
                return None
            local = eid if self.expert_local is None else self.expert_local(fused_name, eid)
            if local is None:
                return None
            if local < 0:
                return "skip"  # not local to this rank (expert parallelism)
            if local >= int(fp.shape[0]):
                return None
            expert_data = OTensor(fp.data[local], fp.dtype)
            if shard == "w2":
                return (expert_data, fused_name) if self.tp_shape_compatible(hf_shape, expert_data.shape) else None
            if not hf_shape:
                if expert_data.numel() == 1:
                    return OTensor(_reshape_view(expert_data.data, (-1,)), fp.dtype), fused_name
                if expert_data.numel() == 2:
                    index = 0 if shard == "w1" else 1
                    return OTensor(_reshape_view(expert_data.data, (2, -1))[index], fp.dtype), fused_name
                return None
            if len(hf_shape) != expert_data.ndim:
                return None
            if shard in ("w1", "w3") and int(expert_data.shape[0]) % 2 == 0:
                local_size = int(expert_data.shape[0]) // 2
                dest = expert_data.narrow(0, 0 if shard == "w1" else local_size, local_size)
                if self.tp_shape_compatible(hf_shape, dest.shape):
                    return dest, fused_name
            for axis in range(expert_data.ndim):
                if not all(d == axis or int(hf_shape[d]) == int(expert_data.shape[d]) for d in range(expert_data.ndim)):
                    continue
                source, dest = int(hf_shape[axis]), int(expert_data.shape[axis])
                if dest == source * 2:
                    local_size = source
                elif self.tp_size > 1 and dest * self.tp_size == source * 2:
                    local_size = dest // 2
                else:
                    continue
                return expert_data.narrow(axis, 0 if shard == "w1" else local_size, local_size), fused_name
        return None

    # ---- resolution and writes (installer.py:341-437) ----
    def _resolve_write(self, hf_name, tensor):
        for kind, table in (("fused", self.fused), ("expert", self.expert)):
            d = table.get(hf_name)
            if d is not None:
                local = self.tp_local_tensor(tensor, d.shape)
                return None if local is None else (kind, d, local)
        p = self.direct.get(hf_name)
        if p is not None:
            local = self.tp_local_tensor(tensor, p.shape)
            if local is not None:
                return "direct", p, local
        return None

    def _copy(self, dest: OTensor, src: OTensor) -> None:
        if src.dtype == dest.dtype:
            dest.data[...] = src.data
        elif (src.dtype, dest.dtype) in CAST_CODES and self.allow_cast:
            dest.data[...] = cast_tensor(src, dest.dtype, self.nan_bits).data
        else:
            raise RuntimeError(f"no conversion from {src.dtype} to {dest.dtype}")

    def resolve(self, weights, strict_params: bool = True) -> list:
        """Classify and resolve every write, check coverage; nothing is copied
        (installer.py:366-410 with the coverage rule of :219-251 applied to every
        parameter).  Returns ``[(kind, dest_view, src_view)]``."""
        weights = list(weights)
        self.extend_dest_map(weights)
        writes, unmapped = [], []
        for hf_name, tensor in weights:
            if hf_name in self.direct and self.direct[hf_name] is None:
                continue
            pm = self.premerged.get(hf_name)
            if pm is not None:
                sub = self._premerged_writes(pm[0], pm[1], tensor)
                if sub is None:
                    unmapped.append(hf_name)
                else:
                    writes.extend(("fused", d, s) for d, s in sub)
                continue
            resolved = self._resolve_write(hf_name, tensor)
            if resolved is None:
                unmapped.append(hf_name)
            else:
                writes.append(resolved)
        if unmapped:
            raise CoverageError(f"unmapped checkpoint tensors={unmapped[:10]}")
        required = set(self.params) if strict_params else {
            n for n, p in self.params.items() if p.dtype in FP8_DTYPES or self.is_scale_name(n)
        }
        missing = sorted(required - self.covered)
        if missing:
            raise CoverageError(f"uncovered local parameters={missing[:10]}")
        return writes

    def load_weights(self, weights, strict_params: bool = True) -> dict:
        """Resolve everything, then copy (installer.py:419-424)."""
        writes = self.resolve(weights, strict_params)
        counts = {"direct": 0, "fused": 0, "expert": 0}
        for kind, dest, src in writes:
            self._copy(dest, src)
            counts[kind] += 1
        return counts
