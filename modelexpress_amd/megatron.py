"""Trainer-native (Megatron) layouts as virtual tensors for the placement planner.

Megatron stores attention as one fused ``linear_qkv`` tensor laid out one block per KV
group -- that group's query rows, then its K head, then its V head -- so q, k and v rows
interleave; and the gated MLP as ``[gate; up]``.  The reference turns those into
Hugging Face named aliases made of row bands
(modelexpress_rl/train/engines/megatron/aliases.py:116-168 for gate/up, :206-350 for QKV).
Here the same bands become ``VirtualTensor`` shards, so the planner slices, fuses and
casts them like any checkpoint tensor and the device never sees the interleave.
"""

from __future__ import annotations

from typing import Iterator, Sequence

from .engine import VirtualTensor

Q, K, V = 0, 1, 2


def qkv_bands(head_dim: int, q_heads: int, kv_heads: int) -> Iterator[tuple]:
    """``(projection, start_row_in_fused, rows, start_row_in_projection)`` in fused row order
    (aliases.py:247-263)."""
    if head_dim < 1 or q_heads < 1 or kv_heads < 1 or q_heads % kv_heads:
        raise ValueError("invalid global Q/KV head geometry")
    q_rows = (q_heads // kv_heads) * head_dim
    group_rows = q_rows + 2 * head_dim
    for g in range(kv_heads):
        start = g * group_rows
        yield Q, start, q_rows, g * q_rows
        yield K, start + q_rows, head_dim, g * head_dim
        yield V, start + q_rows + head_dim, head_dim, g * head_dim


def qkv_virtuals(sources: Sequence[tuple], hf_names: Sequence[str], hidden: int, *, head_dim: int, q_heads: int,
                 kv_heads: int) -> list:
    """Virtual q/k/v tensors over fused QKV sources.

    ``sources`` rows are ``(tensor_name, row_lo, row_hi)``: each checkpoint tensor holds the
    fused rows ``[row_lo, row_hi)`` (one row for an unsharded tensor, one per trainer TP rank
    otherwise).  Every source row interval is intersected with every band
    (aliases.py:291-350); a source that owns no K or V rows simply matches no such band.
    """
    if len(hf_names) != 3:
        raise ValueError("QKV aliasing requires q/k/v names")
    total_rows = kv_heads * ((q_heads // kv_heads) * head_dim + 2 * head_dim)
    dest_rows = (q_heads * head_dim, kv_heads * head_dim, kv_heads * head_dim)
    shards = ([], [], [])
    for name, lo, hi in sources:
        if not 0 <= lo < hi <= total_rows:
            raise ValueError(f"{name}: inconsistent QKV source row interval")
        mapped = 0
        for proj, start, rows, dest_start in qkv_bands(head_dim, q_heads, kv_heads):
            a, b = max(lo, start), min(hi, start + rows)
            if a >= b:
                continue
            shards[proj].append((name, (a - lo, 0), (dest_start + a - start, 0), (b - a, hidden)))
            mapped += b - a
        if mapped != hi - lo:
            raise ValueError(f"{name}: QKV interval mapping covered {mapped} of {hi - lo} source rows")
    return [VirtualTensor(n, (r, hidden), tuple(s)) for n, r, s in zip(hf_names, dest_rows, shards) if s]


def gated_virtuals(sources: Sequence[tuple], hf_names: Sequence[str], trailing: Sequence[int], *, global_rows: int,
                   order: str = "gate_then_up") -> list:
    """Virtual gate / up tensors over ``[gate; up]`` sources split on axis 0.

    ``sources`` rows are ``(tensor_name, rank, n_ranks)``: the tensor holds rank ``rank``'s
    local ``[gate_local; up_local]`` rows (aliases.py:116-168; the storage order must be
    stated, it cannot be detected from the bytes)."""
    if order != "gate_then_up":
        raise ValueError("fused gate/up aliasing requires order == 'gate_then_up'")
    if len(hf_names) != 2 or global_rows % 2:
        raise ValueError("gated tensor requires gate/up names and an even global extent")
    half_global = global_rows // 2
    zeros = tuple(0 for _ in trailing)
    shards = ([], [])
    for name, rank, n_ranks in sources:
        if half_global % n_ranks:
            raise ValueError(f"{name}: fused gate/up extent must split evenly over the source ranks")
        half = half_global // n_ranks
        for part in (0, 1):
            shards[part].append((name, (part * half,) + zeros, (rank * half,) + zeros, (half,) + tuple(trailing)))
    return [VirtualTensor(n, (half_global,) + tuple(trailing), tuple(s)) for n, s in zip(hf_names, shards)]
