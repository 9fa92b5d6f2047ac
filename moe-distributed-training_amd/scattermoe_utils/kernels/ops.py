"""Kernel-level operators of the expert-MLP path, with the reference's names and argument order.

Reference-owned (scattermoe_utils/kernels/ops.py): ``scatter2scatter_lora`` (:156-212), ``group_bwd_AB`` (:220-255).
scattermoe-owned, imported by the reference (megablocks_utils/config_utils.py:116, tests/test_scattermoe.py:3,
scattermoe_utils/parallel_linear_lora.py:87,98): ``flatten_and_sort``, ``padded_block_indices``,
``scatter2scatter``, ``group``, ``group_bwd_W``.

Every function validates shapes like the reference (asserts), allocates outputs with torch and enqueues HIP
kernels of libmoe_hip.so on the current stream.  Nothing is computed on the host.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from ... import _lib
from ..._lib import lib, check, dtype_code, is64, ptr, require_gpu, stream_ptr, workspace

BLOCK_M = 128  # rows per padded block, as in the reference (ops.py:6)


def _strides3(t: Optional[torch.Tensor]):
    return (0, 0, 0) if t is None else tuple(t.stride())


def expert_offsets_from_sorted(sorted_expert_idxs: torch.Tensor, num_experts: int) -> torch.Tensor:
    """Inclusive running count per expert (what the reference passes as ``expert_offsets``, ops.py:315-319)."""
    dev = require_gpu(sorted_expert_idxs)
    sei = sorted_expert_idxs.contiguous()
    out = torch.empty(num_experts, dtype=sei.dtype, device=dev)
    check(lib.moe_expert_offsets(ptr(sei), is64(sei), sei.numel(), num_experts, ptr(out), is64(out), stream_ptr(dev)),
          "moe_expert_offsets")
    return out


MAX_EXPERTS = 4096  # largest expert count the counting sort takes


def flatten_and_sort(expert_idxs: torch.Tensor, num_experts: Optional[int] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """(sorted_expert_idxs, sorted_scattered_idxs): stable ascending sort of the flattened (token-major) expert
    assignments -- the tuple megablocks_utils/config_utils.py:131-132 feeds to the kernels.  Like the ``torch.sort`` it
    stands in for, the sorted ids keep the input's dtype, the positions are int64, and nothing synchronises with the
    host (so the call can be captured into a graph).  The function it replaces has no expert-count argument: without
    ``num_experts`` the sort runs with the largest count it supports, ``MAX_EXPERTS``, which costs a few microseconds
    more than the exact count.

    Ids outside ``[0, num_experts)`` (``[0, MAX_EXPERTS)`` without the argument) take no part in the sorted order: the
    valid assignments fill the front of both outputs and every entry behind them reads ``-1`` (never uninitialised
    memory), so ``(sorted_expert_idxs < 0).any()`` tells a caller that ids were out of range.  An expert count above
    ``MAX_EXPERTS`` is refused (``RuntimeError``, from the library's status) before anything is enqueued."""
    dev = require_gpu(expert_idxs)
    flat = expert_idxs.reshape(-1).contiguous()
    if flat.dtype not in (torch.int32, torch.int64):
        flat = flat.to(torch.int64)
    E = MAX_EXPERTS if num_experts is None else int(num_experts)
    sei, ssi = _sort(flat, E, want_meta=False, sentinel=True)[:2]
    return sei, ssi if ssi.dtype == torch.int64 else ssi.long()


def _sort(flat: torch.Tensor, E: int, want_meta: bool = True, block_m: int = BLOCK_M, sentinel: bool = False):
    """Stable counting sort on the device. Returns (sei, ssi, counts, offsets, padded_blocks_buf, num_padded, inv).
    ``sentinel``: entries that no valid id lands on (ids outside [0, E) are left out of the order) read -1."""
    dev = flat.device
    R = flat.numel()
    sei = torch.full_like(flat, -1) if sentinel else torch.empty_like(flat)
    ssi = torch.full_like(flat, -1) if sentinel else torch.empty_like(flat)
    counts = torch.empty(E, dtype=flat.dtype, device=dev) if want_meta else None
    offsets = torch.empty(E, dtype=flat.dtype, device=dev) if want_meta else None
    cap = R // block_m + E
    pbi = torch.empty(cap, dtype=flat.dtype, device=dev) if want_meta else None
    npad = torch.empty(1, dtype=torch.int32, device=dev) if want_meta else None
    inv = torch.empty(R, dtype=torch.int32, device=dev) if want_meta else None
    wsb = lib.moe_sort_workspace_bytes(R, E)
    ws = workspace(wsb, dev)
    check(lib.moe_sort_by_expert(ptr(flat), is64(flat), R, E, block_m, ptr(sei), ptr(ssi), is64(flat), ptr(counts),
                                 ptr(offsets), ptr(pbi), cap, ptr(npad), ptr(inv), ptr(ws), ws.numel(), stream_ptr(dev)),
          "moe_sort_by_expert")
    return sei, ssi, counts, offsets, pbi, npad, inv


def padded_block_indices(sorted_experts_idxs: torch.Tensor, k: int, N_BLOCK_SIZE: int = BLOCK_M):
    """(padded_block_idxs, expert_offsets) -- semantics of scattermoe_utils/kernels/ops.py:39-51; ``k`` is the number
    of experts (call sites config_utils.py:116-118, tests/test_scattermoe.py:161-163)."""
    dev = require_gpu(sorted_experts_idxs)
    sei = sorted_experts_idxs.contiguous()
    if sei.dtype not in (torch.int32, torch.int64):
        sei = sei.to(torch.int64)
    R = sei.numel()
    offsets = torch.empty(k, dtype=torch.int64, device=dev)
    st = stream_ptr(dev)
    check(lib.moe_expert_offsets(ptr(sei), is64(sei), R, k, ptr(offsets), 1, st), "moe_expert_offsets")
    cap = R // N_BLOCK_SIZE + k
    blocks = torch.empty(cap, dtype=torch.int64, device=dev)
    npad = torch.empty(1, dtype=torch.int32, device=dev)
    check(lib.moe_padded_block_indices(ptr(offsets), 1, k, N_BLOCK_SIZE, ptr(blocks), 1, cap, ptr(npad), st),
          "moe_padded_block_indices")
    n = int(npad.item())  # data-dependent length: one host read, as the reference's torch ops imply
    return blocks[:n], offsets


def _scatter2scatter(X, W, A, B, lora_alp, sorted_expert_idxs, sorted_scattered_idxs, k, x_grouped, y_grouped, out,
                     expert_offsets=None):
    dev = require_gpu(X, W, A, B, sorted_expert_idxs, sorted_scattered_idxs)
    assert sorted_scattered_idxs.size(0) == sorted_expert_idxs.size(0)
    assert sorted_scattered_idxs.size(0) == X.size(0) * k
    assert X.dim() == 2 and W.dim() == 3 and X.size(1) == W.size(1), "X and W have inconsistent inner dims."
    assert W.dtype == X.dtype, "X and W must share a dtype"
    rank = 0
    scaling = 0.0
    if A is not None:
        assert W.size(1) == A.size(1), "A has incorrect input size."
        assert W.size(2) == B.size(2), "B has incorrect output size."
        assert A.size(2) == B.size(1), "A and B have inconsistent inner dims."
        assert A.dtype == X.dtype and B.dtype == X.dtype
        rank = A.size(2)
        scaling = float(lora_alp) / rank
    E, K, N = W.shape
    L = sorted_expert_idxs.size(0)
    if out is None:
        O = torch.empty((L, N), device=dev, dtype=X.dtype)
    else:
        assert out.size(0) == L and out.size(1) == N
        O = out
    if L == 0:
        return O
    ssi = sorted_scattered_idxs.contiguous()
    if expert_offsets is None:
        expert_offsets = expert_offsets_from_sorted(sorted_expert_idxs, E)
    eo = expert_offsets.contiguous()
    sa, sb = _strides3(A), _strides3(B)
    wsb = lib.moe_scatter2scatter_workspace_bytes(L, E, K, N, rank)
    ws = workspace(wsb, dev)
    check(lib.moe_scatter2scatter(
        ptr(X), X.stride(0), X.stride(1), ptr(W), W.stride(0), W.stride(1), W.stride(2),
        ptr(A), sa[0], sa[1], sa[2], ptr(B), sb[0], sb[1], sb[2], rank, scaling,
        ptr(O), O.stride(0), O.stride(1), ptr(ssi), is64(ssi), ptr(eo), is64(eo), E, L, K, N, k,
        int(bool(x_grouped)), int(bool(y_grouped)), dtype_code(X), ptr(ws), ws.numel(), stream_ptr(dev)),
        "moe_scatter2scatter")
    return O


def scatter2scatter_lora(X, W, A, B, lora_alp, sorted_expert_idxs, sorted_scattered_idxs, k, padded_block_idxs,
                         x_grouped=False, y_grouped=False, out=None):
    """Y = X (W + (lora_alp / r) A B) over ragged expert groups (reference ops.py:156-212).  ``padded_block_idxs`` is
    accepted for signature compatibility; the kernels derive their own row tiles from the expert boundaries."""
    assert A is not None and B is not None
    return _scatter2scatter(X, W, A, B, lora_alp, sorted_expert_idxs, sorted_scattered_idxs, k, x_grouped, y_grouped, out)


def scatter2scatter(X, W, sorted_expert_idxs, sorted_scattered_idxs, k, padded_block_idxs=None, x_grouped=False,
                    y_grouped=False, out=None):
    """The adapter-free sibling from scattermoe (selected at megablocks_utils/config_utils.py:124-125)."""
    return _scatter2scatter(X, W, None, None, 0.0, sorted_expert_idxs, sorted_scattered_idxs, k, x_grouped, y_grouped, out)


def group(A, sorted_expert_idxs, coeff=None, fan_out=1, out=None):
    """out[i] = A[idx[i] // fan_out] * coeff[idx[i]] -- scattermoe.kernels.ops.group as called at
    scattermoe_utils/parallel_linear_lora.py:87-91,98 (the second argument receives sorted_scattered_idxs)."""
    dev = require_gpu(A, sorted_expert_idxs, coeff)
    idx = sorted_expert_idxs.contiguous()
    L, K = idx.size(0), A.size(1)
    assert A.dim() == 2 and A.stride(1) == 1
    if out is None:
        Y = torch.empty((L, K), dtype=A.dtype, device=dev)
    else:
        assert out.size(0) == L and out.size(1) == K and out.stride(1) == 1
        Y = out
    cdt = 0
    if coeff is not None:
        coeff = coeff.contiguous()
        cdt = dtype_code(coeff)
    check(lib.moe_group_rows(ptr(A), A.stride(0), ptr(Y), Y.stride(0), ptr(idx), is64(idx), fan_out, ptr(coeff), cdt,
                             L, K, dtype_code(A), stream_ptr(dev)), "moe_group_rows")
    return Y


def group_bwd_AB(DY, X, A, B, scaling, expert_offsets, E):
    """(DA (E,K,r), DB (E,r,N)) = (s X^T DY B^T, s A^T X^T DY) per expert group, zero for empty groups (reference
    ops.py:220-255 and the definition at :284-289).  Full reductions over N and K."""
    dev = require_gpu(DY, X, A, B, expert_offsets)
    assert A.size(2) == B.size(1), "A and B have inconsistent inner dims."
    assert DY.size(0) == X.size(0) and X.size(1) == A.size(1) and DY.size(1) == B.size(2)
    R, K, N, r = X.size(0), X.size(1), DY.size(1), A.size(2)
    DA = torch.empty((E, K, r), device=dev, dtype=DY.dtype)
    DB = torch.empty((E, r, N), device=dev, dtype=DY.dtype)
    eo = expert_offsets.contiguous()
    dt = dtype_code(DY)
    wsb = lib.moe_group_bwd_ab_workspace_bytes(R, E, K, N, r, dt)
    ws = workspace(wsb, dev)
    check(lib.moe_group_bwd_ab(
        ptr(DY), DY.stride(0), DY.stride(1), ptr(X), X.stride(0), X.stride(1),
        ptr(A), A.stride(0), A.stride(1), A.stride(2), ptr(B), B.stride(0), B.stride(1), B.stride(2), r, float(scaling),
        ptr(DA), DA.stride(0), DA.stride(1), DA.stride(2), ptr(DB), DB.stride(0), DB.stride(1), DB.stride(2),
        ptr(eo), is64(eo), E, R, K, N, dt, ptr(ws), ws.numel(), stream_ptr(dev)), "moe_group_bwd_ab")
    return DA, DB


def group_bwd_W(DY, X, expert_offsets, E):
    """DW[e] = X_e^T DY_e (scattermoe.kernels.ops.group_bwd_W; full fine-tuning path)."""
    dev = require_gpu(DY, X, expert_offsets)
    assert X.size(0) == DY.size(0) and X.dtype == DY.dtype
    R, K, N = X.size(0), X.size(1), DY.size(1)
    DW = torch.empty((E, K, N), device=dev, dtype=DY.dtype)
    eo = expert_offsets.contiguous()
    check(lib.moe_group_bwd_w(ptr(DY), DY.stride(0), DY.stride(1), ptr(X), X.stride(0), X.stride(1), ptr(DW),
                              DW.stride(0), DW.stride(1), DW.stride(2), ptr(eo), is64(eo), E, R, K, N, dtype_code(DY),
                              stream_ptr(dev)), "moe_group_bwd_w")
    return DW


def combine(y, gates, inv=None, k=None, out=None, extra_coef=None, extra_rows=None):
    """out[t] = sum_j gates[t,j] * y[row(t,j)] -- the gates bmm of parallel_linear_lora.py:30-35 (inv=None: y rows
    are token-major) or megablocks' ops.scatter (inv = position of assignment (t,j) in grouped order)."""
    dev = require_gpu(y, gates, inv)
    if gates is not None:
        T, kk = gates.shape
        gates = gates.contiguous()
    else:
        kk = k
        T = y.size(0) // kk
    N = y.size(1)
    O = torch.empty((T, N), dtype=y.dtype, device=dev) if out is None else out
    ne = 0 if extra_coef is None else extra_coef.size(1)
    check(lib.moe_combine(ptr(y), y.stride(0), ptr(O), O.stride(0), ptr(gates), 0 if gates is None else dtype_code(gates),
                          ptr(inv), kk, T, N, dtype_code(y), ptr(extra_coef), ptr(extra_rows),
                          0 if extra_rows is None else extra_rows.stride(0), ne, stream_ptr(dev)), "moe_combine")
    return O


def combine_dgates(y, dout, k, gates_dtype, inv=None):
    """d_gates[t,j] = <y[row(t,j)], dout[t]> (parallel_linear_lora.py:70-72)."""
    dev = require_gpu(y, dout, inv)
    T = dout.size(0)
    dg = torch.empty((T, k), dtype=gates_dtype, device=dev)
    check(lib.moe_combine_dgates(ptr(y), y.stride(0), ptr(dout), dout.stride(0), ptr(dg), dtype_code(dg), ptr(inv), k, T,
                                 y.size(1), dtype_code(y), stream_ptr(dev)), "moe_combine_dgates")
    return dg


def swiglu(gate, up):
    dev = require_gpu(gate, up)
    gate, up = gate.contiguous(), up.contiguous()
    h = torch.empty_like(gate)
    check(lib.moe_swiglu(ptr(gate), ptr(up), ptr(h), gate.numel(), dtype_code(gate), stream_ptr(dev)), "moe_swiglu")
    return h


def swiglu_bwd(gate, up, dh):
    dev = require_gpu(gate, up, dh)
    gate, up, dh = gate.contiguous(), up.contiguous(), dh.contiguous()
    dg, du = torch.empty_like(gate), torch.empty_like(up)
    check(lib.moe_swiglu_bwd(ptr(gate), ptr(up), ptr(dh), ptr(dg), ptr(du), gate.numel(), dtype_code(gate), stream_ptr(dev)),
          "moe_swiglu_bwd")
    return dg, du
