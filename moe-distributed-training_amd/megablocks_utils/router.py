"""Top-k router of the MoE layer: softmax over expert logits, top-k, L1 renormalisation -- the patched
``LearnedRouter.forward`` of the reference (megablocks_utils/config_utils.py:255-280), followed by the integer
pipeline megablocks runs next (stable sort by expert, histogram, running sum).  Softmax is computed in fp32 from
fp32-accumulated logits (as transformers' MixtralTopKRouter does), not in the activation dtype."""
from __future__ import annotations

from typing import NamedTuple, Optional

import torch

from .._lib import lib, check, dtype_code, ptr, require_gpu, stream_ptr, workspace
from ..scattermoe_utils.kernels import ops


class Routing(NamedTuple):
    logits: torch.Tensor          # (T, E) fp32
    scores: torch.Tensor          # (T, E) fp32 softmax
    weights: torch.Tensor         # (T, k) fp32, renormalised
    indices: torch.Tensor         # (T, k) int32
    sorted_expert_idxs: torch.Tensor     # (T*k,) int32   ("bin_ids")
    sorted_scattered_idxs: torch.Tensor  # (T*k,) int32   ("indices")
    tokens_per_expert: torch.Tensor      # (E,) int32
    expert_offsets: torch.Tensor         # (E,) int32 inclusive ("bins")
    inverse: torch.Tensor                # (T*k,) int32: sorted position of assignment t*k+j


def router_logits(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    dev = require_gpu(x, weight)
    x2 = x.reshape(-1, x.shape[-1])
    if x2.stride(-1) != 1:
        x2 = x2.contiguous()
    w = weight if weight.stride(-1) == 1 else weight.contiguous()
    assert w.dtype == x2.dtype and w.size(1) == x2.size(1)
    T, d = x2.shape
    E = w.size(0)
    logits = torch.empty((T, E), dtype=torch.float32, device=dev)
    check(lib.moe_router_logits(ptr(x2), x2.stride(0), ptr(w), w.stride(0), dtype_code(x2), ptr(logits), T, d, E,
                                stream_ptr(dev)), "moe_router_logits")
    return logits


def router_topk(logits: torch.Tensor, top_k: int, normalize: bool = True):
    """fp32 logits (T,E) -> (scores (T,E), weights (T,k), indices (T,k) int32)."""
    dev = require_gpu(logits)
    logits = logits.contiguous().float()
    T, E = logits.shape
    scores = torch.empty_like(logits)
    w = torch.empty((T, top_k), dtype=torch.float32, device=dev)
    idx = torch.empty((T, top_k), dtype=torch.int32, device=dev)
    check(lib.moe_router_topk(ptr(logits), ptr(scores), ptr(w), ptr(idx), T, E, top_k, int(bool(normalize)),
                              stream_ptr(dev)), "moe_router_topk")
    return scores, w, idx


def router_forward(x: torch.Tensor, weight: torch.Tensor, top_k: int, normalize: bool = True):
    """x (T, d), router weight (E, d) -> (logits (T,E) fp32, scores (T,E), weights (T,k), indices (T,k) int32): the
    logits GEMV, the softmax and the top-k of config_utils.py:262-270 in one library call."""
    dev = require_gpu(x, weight)
    x2 = x.reshape(-1, x.shape[-1])
    if x2.stride(-1) != 1:
        x2 = x2.contiguous()
    w = weight if weight.stride(-1) == 1 else weight.contiguous()
    assert w.dtype == x2.dtype and w.size(1) == x2.size(1)
    T, d = x2.shape
    E = w.size(0)
    assert 1 <= top_k <= E
    logits = torch.empty((T, E), dtype=torch.float32, device=dev)
    scores = torch.empty_like(logits)
    tw = torch.empty((T, top_k), dtype=torch.float32, device=dev)
    idx = torch.empty((T, top_k), dtype=torch.int32, device=dev)
    check(lib.moe_router_forward(ptr(x2), x2.stride(0), ptr(w), w.stride(0), dtype_code(x2), ptr(logits), ptr(scores),
                                 ptr(tw), ptr(idx), T, d, E, top_k, int(bool(normalize)), stream_ptr(dev)),
          "moe_router_forward")
    return logits, scores, tw, idx


def router_topk_bwd(d_weights, weights, indices, scores, normalize: bool = True):
    dev = require_gpu(d_weights, weights, indices, scores)
    T, E = scores.shape
    k = weights.size(1)
    dl = torch.empty_like(scores)
    dw = d_weights.contiguous().float()
    check(lib.moe_router_topk_bwd(ptr(dw), ptr(weights), ptr(indices), ptr(scores), ptr(dl), T, E, k,
                                  int(bool(normalize)), stream_ptr(dev)), "moe_router_topk_bwd")
    return dl


def router_input_grad(dlogits: torch.Tensor, weight: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """dx = dlogits @ weight from the fp32 dlogits (fp32 accumulate, one rounding to ``dtype``)."""
    dev = require_gpu(dlogits, weight)
    dl = dlogits.contiguous().float()
    w = weight if weight.stride(-1) == 1 else weight.contiguous()
    if w.dtype != dtype:
        w = w.to(dtype)
    T, E = dl.shape
    d = w.size(1)
    out = torch.empty((T, d), dtype=dtype, device=dev)
    check(lib.moe_combine(0, 0, ptr(out), out.stride(0), 0, 0, 0, 0, T, d, dtype_code(out), ptr(dl), ptr(w), w.stride(0), E,
                          stream_ptr(dev)), "moe_combine (router input gradient)")
    return out


def router_weight_grad(x2: torch.Tensor, dlogits: torch.Tensor) -> torch.Tensor:
    """dWg = dlogits^T @ x2 from the fp32 dlogits (fp32 accumulate in a fixed order, one rounding to x2's dtype)."""
    dev = require_gpu(x2, dlogits)
    dl = dlogits.contiguous().float()
    if x2.stride(-1) != 1:
        x2 = x2.contiguous()
    T, d = x2.shape
    E = dl.size(1)
    out = torch.empty((E, d), dtype=x2.dtype, device=dev)
    ws = workspace(lib.moe_router_weight_grad_workspace_bytes(T, d, E), dev)
    check(lib.moe_router_weight_grad(ptr(x2), x2.stride(0), ptr(dl), ptr(out), out.stride(0), T, d, E, dtype_code(x2), ptr(ws),
                                     ws.numel(), stream_ptr(dev)), "moe_router_weight_grad")
    return out


class _RouterFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x2, weight, top_k, normalize):
        _, scores, w, idx = router_forward(x2, weight, top_k, normalize)
        ctx.save_for_backward(x2, weight, scores, w, idx)
        ctx.normalize = normalize
        ctx.mark_non_differentiable(idx)
        return scores, w, idx

    @staticmethod
    def backward(ctx, d_scores, d_w, _d_idx):
        x2, weight, scores, w, idx = ctx.saved_tensors
        dl = router_topk_bwd(d_w, w, idx, scores, ctx.normalize)
        if d_scores is not None:
            # softmax backward for a gradient that reaches the full score matrix (e.g. an auxiliary loss)
            ds = d_scores.float()
            dl = dl + scores * (ds - (ds * scores).sum(-1, keepdim=True))
        dx = router_input_grad(dl, weight, x2.dtype) if ctx.needs_input_grad[0] else None
        dwg = router_weight_grad(x2, dl) if ctx.needs_input_grad[1] else None
        return dx, dwg, None, None


class _LogitsFn(torch.autograd.Function):
    """fp32 router logits with autograd, for the router variants that put something between the linear layer and the
    softmax."""
    @staticmethod
    def forward(ctx, x2, weight):
        ctx.save_for_backward(x2, weight)
        return router_logits(x2, weight)

    @staticmethod
    def backward(ctx, dl):
        x2, weight = ctx.saved_tensors
        return (router_input_grad(dl, weight, x2.dtype) if ctx.needs_input_grad[0] else None,
                router_weight_grad(x2, dl) if ctx.needs_input_grad[1] else None)


class _TopkFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits, top_k, normalize):
        scores, w, idx = router_topk(logits, top_k, normalize)
        ctx.save_for_backward(scores, w, idx)
        ctx.normalize = normalize
        ctx.mark_non_differentiable(idx)
        return scores, w, idx

    @staticmethod
    def backward(ctx, d_scores, d_w, _d_idx):
        scores, w, idx = ctx.saved_tensors
        dl = router_topk_bwd(torch.zeros_like(w) if d_w is None else d_w, w, idx, scores, ctx.normalize)
        if d_scores is not None:
            ds = d_scores.float()
            dl = dl + scores * (ds - (ds * scores).sum(-1, keepdim=True))
        return dl, None, None


def jitter(x: torch.Tensor, eps: float) -> torch.Tensor:
    """Multiplicative input noise of the router, uniform in [1 - eps, 1 + eps) (config_utils.py:256-257 calls the
    router's own ``jitter``)."""
    low, high = 1.0 - eps, 1.0 + eps
    return low + torch.rand(x.size(), dtype=x.dtype, device=x.device) * (high - low)


def forward_router(x: torch.Tensor, weight: torch.Tensor, top_k: int, moe_normalize_expert_weights=1,
                   bias: Optional[torch.Tensor] = None, moe_jitter_eps: Optional[float] = None, training: bool = False,
                   uniform_expert_assignment: bool = False):
    """(scores, expert_weights, expert_indices) as the reference's router returns them (config_utils.py:255-280), with
    its switches: input jitter while training (:256-257), a bias on the linear layer (:259-262), division of the
    selected scores by their p-norm, p = ``moe_normalize_expert_weights`` (:264-270), and the uniform assignment that
    replaces the indices by 0, 1, .., E-1, 0, .. in flat order (:272-279).  scores / expert_weights are fp32;
    expert_indices int64 like torch.topk's.  Without bias and with p in {None, 1} this is one fused library call."""
    x2 = x.reshape(-1, x.shape[-1])
    if training and moe_jitter_eps is not None:
        x2 = x2 * jitter(x2, float(moe_jitter_eps))
    p = moe_normalize_expert_weights
    p = None if p in (None, False, 0) else (1 if p is True else p)
    if bias is None and p in (None, 1):
        scores, w, idx = _RouterFn.apply(x2, weight, top_k, p == 1)
    else:
        logits = _LogitsFn.apply(x2, weight)
        if bias is not None:
            logits = logits + bias.float()
        scores, w, idx = _TopkFn.apply(logits, top_k, p == 1)
        if p not in (None, 1):
            w = w / torch.norm(w, p=float(p), dim=-1, keepdim=True)
    idx = idx.long()
    if uniform_expert_assignment:
        idx = torch.remainder(torch.arange(idx.numel(), dtype=idx.dtype, device=idx.device), weight.size(0)).view(idx.shape)
    return scores, w, idx


def sort_assignments(expert_indices: torch.Tensor, num_experts: int):
    """Stable sort by expert + histogram + inclusive running sum + inverse permutation, no host synchronisation."""
    flat = expert_indices.reshape(-1).contiguous()
    sei, ssi, counts, offsets, _pbi, _npad, inv = ops._sort(flat, num_experts, want_meta=True)
    return sei, ssi, counts, offsets, inv


def route_and_sort(x: torch.Tensor, weight: torch.Tensor, top_k: int, normalize: bool = True) -> Routing:
    """Router forward and the expert-grouped order in one call, all on the device (no grad tracking)."""
    with torch.no_grad():
        logits, scores, w, idx = router_forward(x, weight, top_k, normalize)
        sei, ssi, counts, offsets, inv = sort_assignments(idx, weight.size(0))
    return Routing(logits, scores, w, idx, sei, ssi, counts, offsets, inv)
