"""Parallel-K policy of the quantized matmul (python/hidet/graph/ops/quant/resolve.py:23-100).

The reference rewrites the generic operator into `symmetric_quant_matmul_f16_i8(..., parallel_k_parts=k).sum(0)`
with k chosen by `hidet.option.parallel_k`.  Here the kernel sums its K parts itself, so the rule only picks
the hint that is handed to the library: 0 means "let the library plan for MI355X".
"""
from typing import Union

import torch

from hidet_amd import option

# The reference estimates 80 SMs x 5 resident blocks (resolve.py:46); here the streaming kernel runs one round of one
# 8-wave workgroup per CU, and the library sizes its own plan for the CUs of the device it launches on (at most 256,
# a full MI355X).
MAX_CONCURRENT_BLOCKS = 256


def estimate_concurrent_blocks(device=None) -> int:
    """Workgroups the streaming kernel keeps in flight on `device`: one per CU, at most 256 (what the library's plan uses)."""
    if not torch.cuda.is_available():
        return MAX_CONCURRENT_BLOCKS
    return min(MAX_CONCURRENT_BLOCKS, int(torch.cuda.get_device_properties(device).multi_processor_count))
SEARCH_CANDIDATES = [1, 2, 3, 4, 5, 6, 8, 10, 12, 16]  # resolve.py:54


def _cdiv(a: int, b: int) -> int:
    return -(-a // b)


def reference_k_parts(parallel_k: Union[str, int], batch_size: int, m_size: int, n_size: int, k_size: int,
                      concurrent_blocks: int = 80 * 5) -> int:
    """The reference's formula, verbatim in behaviour (resolve.py:42-48, 95-96)."""
    if isinstance(parallel_k, str):
        if parallel_k == 'default':
            estimate_blocks = batch_size * _cdiv(m_size, 64) * _cdiv(n_size, 64)
            return min(_cdiv(concurrent_blocks, estimate_blocks), _cdiv(k_size, 64))
        if parallel_k == 'disabled':
            return 1
        raise ValueError('invalid parallel_k: {}'.format(parallel_k))
    if isinstance(parallel_k, int):
        return min(max(parallel_k, 1), 32)
    raise ValueError('invalid parallel_k: {}'.format(parallel_k))


def resolve_parallel_k_parts(parallel_k: Union[str, int], a: torch.Tensor, b: torch.Tensor) -> int:
    """Hint passed to the library for `symmetric_quant_matmul`.

    'disabled' (the reference's default) and 'default' leave the split to the library's own plan, which is
    sized for the CUs of the device (`estimate_concurrent_blocks`); an integer is passed through clamped to [1, 32] as in the reference; 'search' times the
    reference's candidate list on the GPU and keeps the fastest.
    """
    if isinstance(parallel_k, str):
        if parallel_k in ('disabled', 'default'):
            return 0
        if parallel_k == 'search':
            return search_k_parts(a, b)
        raise ValueError('invalid parallel_k: {}'.format(parallel_k))
    if isinstance(parallel_k, int):
        return min(max(parallel_k, 1), 32)
    raise ValueError('invalid parallel_k: {}'.format(parallel_k))


_SEARCH_CACHE = {}


def search_k_parts(a: torch.Tensor, b: torch.Tensor) -> int:
    from .matmul import run_w8a16

    key = (tuple(a.shape), tuple(b.shape))
    if key in _SEARCH_CACHE:
        return _SEARCH_CACHE[key]
    scale = torch.ones(b.shape[1], dtype=torch.float16, device=b.device)
    best, best_ms = 0, float('inf')
    for cand in [0] + SEARCH_CANDIDATES:
        for _ in range(3):
            run_w8a16(a, b, scale, cand)
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(20):
            run_w8a16(a, b, scale, cand)
        stop.record()
        stop.synchronize()
        ms = start.elapsed_time(stop) / 20
        if ms < best_ms:
            best, best_ms = cand, ms
    _SEARCH_CACHE[key] = best
    return best
