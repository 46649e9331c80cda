"""Varlen chunk tables: same results as ``prepare_lens`` / ``prepare_chunk_indices`` /
``prepare_chunk_offsets`` of fla/ops/utils/index.py:41-43,156-172.

The tables are tiny integer arrays; they are built on the HOST from ``cu_seqlens_cpu`` when
the caller supplies it (no device sync), otherwise from one device-to-host copy of
``cu_seqlens``, and then uploaded.  Results are memoised by tensor identity and version (an in-place
update of ``cu_seqlens`` recomputes); ``cu_seqlens_cpu``, when given, must mirror ``cu_seqlens``: it is
the copy that is checked and the tables are built from, while the kernels index with the device tensor."""
from __future__ import annotations

import torch

from fla_hip.utils import tensor_cache


def prepare_lens(cu_seqlens: torch.Tensor) -> torch.Tensor:
    return cu_seqlens[1:] - cu_seqlens[:-1]


@tensor_cache
def _host_cu(cu_seqlens: torch.Tensor, cu_seqlens_cpu: torch.Tensor | None = None) -> torch.Tensor:
    """The boundaries as int64 on the host (one device-to-host copy per ``cu_seqlens`` tensor, none with ``cu_seqlens_cpu``)."""
    src = cu_seqlens_cpu if cu_seqlens_cpu is not None else cu_seqlens
    return src.detach().to('cpu', torch.int64)


def _host_lens(cu_seqlens: torch.Tensor, cu_seqlens_cpu: torch.Tensor | None) -> torch.Tensor:
    src = _host_cu(cu_seqlens, cu_seqlens_cpu)
    return src[1:] - src[:-1]


@tensor_cache
def _cu_summary(cu_seqlens: torch.Tensor, cu_seqlens_cpu: torch.Tensor | None = None) -> tuple:
    src = _host_cu(cu_seqlens, cu_seqlens_cpu)
    if src.dim() != 1 or src.numel() < 2:
        return (tuple(src.shape),)
    shown = src.tolist() if src.numel() <= 16 else [int(src[0]), '...', int(src[-1])]
    return int(src[0]), int(src[-1]), not bool((src[1:] < src[:-1]).any()), shown


def check_cu_seqlens(cu_seqlens: torch.Tensor, total_tokens: int, cu_seqlens_cpu: torch.Tensor | None = None) -> None:
    """The kernels take token positions from ``cu_seqlens`` as they are: boundaries that decrease, start below zero or end
    beyond the packed tensor would send them out of bounds.  Checked on the host copy the chunk tables are built from
    (memoised per tensor, like the tables)."""
    summary = _cu_summary(cu_seqlens, cu_seqlens_cpu)
    if len(summary) == 1:
        raise ValueError(f'cu_seqlens must hold N + 1 >= 2 boundaries, got shape {summary[0]}')
    first, last, monotone, shown = summary
    if first < 0 or not monotone or last > total_tokens:
        raise ValueError(f'cu_seqlens must be non-decreasing within [0, {total_tokens}] (the packed length), got {shown}')


def cu_bounds(cu_seqlens: torch.Tensor, cu_seqlens_cpu: torch.Tensor | None = None) -> tuple[int, int]:
    """First and last boundary (tokens outside [first, last) belong to no sequence); from the memoised host summary."""
    summary = _cu_summary(cu_seqlens, cu_seqlens_cpu)
    return summary[0], summary[1]


def max_seq_len(cu_seqlens: torch.Tensor, cu_seqlens_cpu: torch.Tensor | None = None) -> int:
    """Length of the longest packed sequence (host copy, memoised)."""
    lens = _host_lens(cu_seqlens, cu_seqlens_cpu)
    return int(lens.max()) if lens.numel() else 0


@tensor_cache
def prepare_chunk_indices(cu_seqlens: torch.Tensor, chunk_size: int,
                          cu_seqlens_cpu: torch.Tensor | None = None) -> torch.Tensor:
    """[num_chunks, 2] rows (sequence id, chunk id inside that sequence), packed order;
    dtype and device of ``cu_seqlens``."""
    counts = (_host_lens(cu_seqlens, cu_seqlens_cpu) + (chunk_size - 1)) // chunk_size
    seq_id = torch.repeat_interleave(torch.arange(counts.numel(), dtype=torch.int64), counts)
    first = torch.cumsum(counts, 0) - counts                    # first packed chunk of each sequence
    within = torch.arange(seq_id.numel(), dtype=torch.int64) - first[seq_id]
    return torch.stack([seq_id, within], 1).to(device=cu_seqlens.device, dtype=cu_seqlens.dtype)


@tensor_cache
def prepare_chunk_offsets(cu_seqlens: torch.Tensor, chunk_size: int,
                          cu_seqlens_cpu: torch.Tensor | None = None) -> torch.Tensor:
    """[N+1] exclusive prefix sum of the number of chunks per sequence."""
    counts = (_host_lens(cu_seqlens, cu_seqlens_cpu) + (chunk_size - 1)) // chunk_size
    out = torch.zeros(counts.numel() + 1, dtype=torch.int64)
    out[1:] = torch.cumsum(counts, 0)
    return out.to(device=cu_seqlens.device, dtype=cu_seqlens.dtype)


@tensor_cache
def prepare_scan_tables(cu_seqlens: torch.Tensor, chunk_size: int,
                        cu_seqlens_cpu: torch.Tensor | None = None) -> torch.Tensor:
    """``prepare_chunk_offsets`` ([N+1]) followed by [N] sequence ids sorted by decreasing length:
    the order in which the sequential kernel hands sequences to the CUs (longest first, so that
    no CU is left with a long sequence at the end).  One tensor, one upload."""
    lens = _host_lens(cu_seqlens, cu_seqlens_cpu)
    counts = (lens + (chunk_size - 1)) // chunk_size
    out = torch.zeros(2 * counts.numel() + 1, dtype=torch.int64)
    out[1:counts.numel() + 1] = torch.cumsum(counts, 0)
    out[counts.numel() + 1:] = torch.argsort(counts, descending=True, stable=True)
    return out.to(device=cu_seqlens.device, dtype=cu_seqlens.dtype)
