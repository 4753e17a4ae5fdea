"""The whole placement path on host cores, composed from the oracle's parts.  TEST AND
BASELINE INFRASTRUCTURE ONLY: bench.py times this as the CPU baseline ("port" of the
reference's CPU path: safetensors parse -> narrow().contiguous() -> copy_ into fused /
stacked views -> dtype cast -> checksum); the product never calls it.

Planning is the numpy restatement (oracle.MdlOracle); the byte work is the C part
(mxp_oracle.c: orc_run_writes) spread over host threads, one pass per write with the
checksum taken from the bytes just written.
"""

from __future__ import annotations

import itertools
import time

import numpy as np

from . import cbind
from . import oracle as O


def _boxes(dst: np.ndarray, src: np.ndarray, cast: bool):
    """Pitched byte boxes of ``dst[...] = src`` for two uint8 views of equal logical shape
    (last axis = element bytes; for a cast the source elements are 4 bytes, the
    destination's 2)."""
    shape = list(dst.shape[:-1])
    ds, ss = list(dst.strides[:-1]), list(src.strides[:-1])
    de, se = dst.shape[-1], src.shape[-1]
    dims = [(n, a, b) for n, a, b in zip(shape, ds, ss) if n != 1]
    run_d, run_s = de, se
    while dims and dims[-1][1] == run_d and dims[-1][2] == run_s:
        n = dims.pop()[0]
        run_d *= n
        run_s *= n
    if not dims:
        yield 0, 0, 1, run_d, run_d, run_s
        return
    rows, dp, sp = dims.pop()
    for idx in itertools.product(*[range(n) for n, _a, _b in dims]):
        d_off = sum(i * a for i, (_n, a, _b) in zip(idx, dims))
        s_off = sum(i * b for i, (_n, _a, b) in zip(idx, dims))
        yield d_off, s_off, rows, run_d, dp, sp


def run(ckpt_dir: str, rank_params: list, *, tp_size=1, tp_rank=0, stacked=None, expert_mapping=None,
        expert_local=None, allow_cast=False, nan_bits=0x7FC0, threads=1, repeats=1, only_tensors=None) -> dict:
    """Parse, plan and place one rank on the CPU.  ``rank_params`` is ``[(name, dtype, shape)]``.
    Returns timings, the placed buffers and their checksums."""
    lib = cbind.load()
    t0 = time.perf_counter()
    weights = O.load_checkpoint(ckpt_dir, mmap=True)
    if only_tensors is not None:  # a bounded sample: the checkpoint tensors that feed ``rank_params``
        weights = [(n, t) for n, t in weights if n in only_tensors]
    t_parse = time.perf_counter() - t0
    params = {n: O.OTensor.zeros(shape, dtype) for n, dtype, shape in rank_params}
    index = {n: i for i, (n, _d, _s) in enumerate(rank_params)}
    base_addr = {n: p.data.ctypes.data for n, p in params.items()}
    owner = {}
    for n, p in params.items():
        owner[id(p.data)] = n
    t0 = time.perf_counter()
    m = O.MdlOracle(params, tp_size, tp_rank, stacked, expert_mapping, expert_local, allow_cast=allow_cast,
                    nan_bits=nan_bits)
    writes = m.resolve(weights)
    recs = []
    placed = 0
    for _kind, dest, src in writes:
        cast = O.CAST_CODES[(src.dtype, dest.dtype)] if src.dtype != dest.dtype else 0
        se, de = src.data.shape[-1], dest.data.shape[-1]
        base = dest.data
        while base.base is not None and isinstance(base.base, np.ndarray):
            base = base.base
        pname = owner[id(base)]
        d0 = dest.data.ctypes.data
        s0 = src.data.ctypes.data
        for d_off, s_off, rows, row_bytes, dp, sp in _boxes(dest.data, src.data, cast):
            placed += rows * row_bytes
            # Pieces of at most ~4 MiB, so one large tensor does not serialise the thread pool.
            if rows == 1:
                step = 4 << 20
                for lo in range(0, row_bytes, step):
                    n = min(step, row_bytes - lo)
                    recs.append(cbind.OrcWrite(src=s0 + s_off + lo * se // de, dst=d0 + d_off + lo, src_pitch=0,
                                               dst_pitch=0, rows=1, row_bytes=n,
                                               dst_index=d0 + d_off + lo - base_addr[pname], param=index[pname],
                                               cast=int(cast)))
            else:
                step = max(1, (4 << 20) // row_bytes)
                for lo in range(0, rows, step):
                    n = min(step, rows - lo)
                    recs.append(cbind.OrcWrite(src=s0 + s_off + lo * sp, dst=d0 + d_off + lo * dp, src_pitch=sp,
                                               dst_pitch=dp, rows=n, row_bytes=row_bytes,
                                               dst_index=d0 + d_off + lo * dp - base_addr[pname], param=index[pname],
                                               cast=int(cast)))
    t_plan = time.perf_counter() - t0
    best = None
    sums = None
    for _ in range(max(1, repeats)):
        t0 = time.perf_counter()
        sums = lib.run_writes(recs, len(rank_params), threads, nan_bits)
        dt = time.perf_counter() - t0
        best = dt if best is None else min(best, dt)
    return {"parse_s": t_parse, "plan_s": t_plan, "place_s": best, "placed_bytes": placed, "n_writes": len(recs),
            "params": params, "checksums": dict(zip([n for n, _d, _s in rank_params], sums)), "threads": threads}


def run_faithful_sample(ckpt_dir: str, names: list, tp_size: int, tp_rank: int, threads: int) -> dict:
    """The reference's own op sequence on torch CPU tensors, for a handful of tensors:
    ``narrow(axis, r*n, n).contiguous()`` (installer.py:317), ``dest.copy_(src)``
    (installer.py:419-424) and ``safe_checksum`` exactly as written -- int64 ``arange`` of one
    entry per byte, int64 products, masked sum (tensor_utils.py:36-42) -- applied to the
    flattened tensor (the 1-D case, the only one in which the reference returns a value).
    Returns bytes processed and seconds; used only to report how the literal formulation
    compares with the one-pass C form."""
    import warnings

    import torch

    # the memory-mapped checkpoint is read-only and only ever read here
    warnings.filterwarnings("ignore", message="The given NumPy array is not writable")
    torch.set_num_threads(threads)
    weights = dict(O.load_checkpoint(ckpt_dir, mmap=True))
    placed = 0
    t0 = time.perf_counter()
    sums = {}
    for name, axis in names:
        src = weights[name]
        t = torch.from_numpy(np.ascontiguousarray(src.data).reshape(src.shape + (src.data.shape[-1],)))
        local = t.shape[axis] // tp_size
        shard = t.narrow(axis, tp_rank * local, local).contiguous()
        dest = torch.empty_like(shard)
        dest.copy_(shard)
        flat = dest.reshape(-1)
        idx = torch.arange(flat.numel(), dtype=torch.int64)
        w = (idx * 2654435761 + 1) & 0xFFFFFFFF
        mixed = (flat.to(torch.int64) * w) & 0xFFFFFFFF
        sums[name] = format(mixed.sum().item() & 0xFFFFFFFF, "08x")
        placed += flat.numel()
    return {"seconds": time.perf_counter() - t0, "placed_bytes": placed, "checksums": sums}
