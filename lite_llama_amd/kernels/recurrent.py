"""Recurrent sequence mixers over ragged steps (csrc/seq_mix.hip): fixed-size fp32 state per (sequence slot, head), carried
from step to step -- the counterpart, for layers without a growing cache, of the attention kernels next door."""

from __future__ import annotations

import torch

from .. import _lib as L


def gated_linear_scan_supported(dk: int, dv: int) -> bool:
    return bool(L.lib().ll_gated_linear_scan_supported(dk, dv))


@torch.no_grad()
def gated_linear_scan(qfv: torch.Tensor, heads: int, dk: int, dv: int, f_bias, lower, norm_weight, eps: float, step,
                      state: torch.Tensor) -> torch.Tensor:
    """HGRN2-style gated linear attention.  ``qfv [n, 2 heads dk + heads dv]`` = the fused projection rows
    ``[q_raw | f_raw | v]``; per head ``f = lower + (1 - lower) sigmoid(f_raw + f_bias)``,
    ``S <- diag(f) S + (1 - f) v^T``, ``o = S^T silu(q_raw)``, then ``o`` RMS-normed over ``dv`` with ``norm_weight``.
    ``state [slots, heads, dk, dv]`` fp32: a sequence whose run starts at position 0 starts from zeros (whatever an earlier
    owner of the slot left), every run leaves its final state.  Returns ``[n, heads dv]`` in the storage dtype."""
    L.require_cuda(qfv, f_bias, lower, norm_weight, state)
    n = qfv.shape[0]
    dt = qfv.dtype
    if qfv.dim() != 2 or qfv.stride(1) != 1 or qfv.shape[1] < 2 * heads * dk + heads * dv:
        raise ValueError("gated_linear_scan: qfv rows hold [q | f | v]")
    if state.dtype != torch.float32 or not state.is_contiguous() or tuple(state.shape[1:]) != (heads, dk, dv):
        raise ValueError("gated_linear_scan: state is contiguous fp32 [slots, heads, dk, dv]")
    for t, size in ((f_bias, heads * dk), (lower, heads * dk), (norm_weight, dv)):
        if t.dtype != dt or t.numel() != size or not t.is_contiguous():
            raise ValueError("gated_linear_scan: gate bias / lower bound [heads dk] and norm weight [dv] in the rows' dtype")
    if step.num_tokens != n:
        raise ValueError("gated_linear_scan: the step describes another number of tokens")
    if not gated_linear_scan_supported(dk, dv):
        raise ValueError(f"gated_linear_scan: head geometry {dk} x {dv} is not served (dv <= 256, <= 128 state rows per thread)")
    out = torch.empty(n, heads * dv, dtype=dt, device=qfv.device)
    # the wide form (a workgroup per 16 state columns; o through an fp32 scratch, then the norm) needs a scratch; the library
    # picks the form (runs of several tokens, or batches too small to fill the chip with a workgroup per (sequence, head))
    scratch = torch.empty(n, heads * dv, dtype=torch.float32, device=qfv.device) if dk <= 256 else None
    es = qfv.element_size()
    base = qfv.data_ptr()
    L.check(L.lib().ll_gated_linear_scan(
        base, base + heads * dk * es, base + 2 * heads * dk * es, qfv.stride(0), f_bias.data_ptr(), lower.data_ptr(),
        norm_weight.data_ptr(), float(eps), out.data_ptr(), step.num_seqs, heads, dk, dv, step.seq_start.data_ptr(),
        step.seq_first_pos.data_ptr(), step.seq_slot.data_ptr(), state.data_ptr(), n, step.longest_run, L.ptr(scratch),
        L.dtype_code(dt), L.stream_ptr()),
        "gated_linear_scan")
    return out


@torch.no_grad()
def mingru_scan(zxg: torch.Tensor, width: int, z_bias, x_bias, step, state: torch.Tensor) -> torch.Tensor:
    """minGRU over a ragged step.  ``zxg [n, >= 3 width]`` = fused projection rows ``[z_raw | x_raw | g_raw]``; per channel
    ``z = sigmoid(z_raw + z_bias)``, ``u = x_raw + x_bias``, candidate ``u + 1/2`` where ``u >= 0`` and ``sigmoid(u)`` below,
    ``S <- (1 - z) S + z candidate``; returns ``S * silu(g_raw)`` ``[n, width]`` in the storage dtype.  ``state
    [slots, width]`` fp32: a sequence whose run starts at position 0 starts from zeros, every run leaves its final state."""
    L.require_cuda(zxg, z_bias, x_bias, state)
    n, dt = zxg.shape[0], zxg.dtype
    if zxg.dim() != 2 or zxg.stride(1) != 1 or zxg.shape[1] < 3 * width:
        raise ValueError("mingru_scan: rows hold [z | x | g]")
    if state.dtype != torch.float32 or not state.is_contiguous() or state.dim() != 2 or state.shape[1] != width:
        raise ValueError("mingru_scan: state is contiguous fp32 [slots, width]")
    for b in (z_bias, x_bias):
        if b is not None and (b.dtype != dt or b.numel() != width or not b.is_contiguous()):
            raise ValueError("mingru_scan: biases are [width] in the rows' dtype")
    if step.num_tokens != n:
        raise ValueError("mingru_scan: the step describes another number of tokens")
    out = torch.empty(n, width, dtype=dt, device=zxg.device)
    es, base = zxg.element_size(), zxg.data_ptr()
    # long runs: chunks of a run are walked side by side (chunk maps, entering states, the chunks again) over an fp32 scratch
    floats = int(L.lib().ll_mingru_scan_scratch_floats(step.num_seqs, width, step.longest_run))
    scratch = torch.empty(floats, dtype=torch.float32, device=zxg.device) if floats else None
    L.check(L.lib().ll_mingru_scan(base, base + width * es, base + 2 * width * es, zxg.stride(0), L.ptr(z_bias), L.ptr(x_bias),
                                   out.data_ptr(), step.num_seqs, width, step.seq_start.data_ptr(), step.seq_first_pos.data_ptr(),
                                   step.seq_slot.data_ptr(), state.data_ptr(), step.longest_run, L.ptr(scratch), L.dtype_code(dt),
                                   L.stream_ptr()), "mingru_scan")
    return out
