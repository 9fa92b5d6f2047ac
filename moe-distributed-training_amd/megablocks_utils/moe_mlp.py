"""The expert-MLP caller of the MoE layer: w1 / w3 grouped GEMMs, SiLU * mul, w2 grouped GEMM, weighted combine.

Follows ``scattermoe_permute_and_compute`` of the reference (megablocks_utils/config_utils.py:99-185) and the weight
views it builds (``get_mlp_weights`` :28-35, ``get_mlp_weights_lora`` :37-61).  For bf16 tensors of Mixtral-like
shape the three projections run as two fused launches (dual-weight GEMM with SwiGLU epilogue, then w2) through
``moe_mlp_fwd`` / ``moe_mlp_bwd`` of libmoe_hip.so; everything else goes through the same three
``parallel_linear(_lora)`` calls the reference makes, which use the generic HIP kernels.
"""
from __future__ import annotations

import ctypes
from typing import NamedTuple, Optional, Tuple

import torch
import torch.nn as nn

from .._lib import lib, check, dtype_code, is64, ptr, require_gpu, stream_ptr, workspace
from ..scattermoe_utils.kernels import ops
from ..scattermoe_utils.parallel_experts import parallel_linear
from ..scattermoe_utils.parallel_linear_lora import parallel_linear_lora
from . import router as _router


# ---------------------------------------------------------------------------------------------------------------
# weight views (reference config_utils.py:28-61)
# ---------------------------------------------------------------------------------------------------------------
def resolve_dtensor(t):
    """The local shard of a DTensor parameter, anything else unchanged (config_utils.py:32,58-59 strip the DTensor
    wrapper the same way before the kernels see the weights)."""
    return t.to_local() if hasattr(t, "to_local") else t


def get_mlp_weights(w: torch.Tensor, ffn_hidden_size: int, hidden_size: int, name: str = "w1") -> torch.Tensor:
    """Storage (E*ffn, hidden) -> the (E, K, N) view the kernels take: w1/w3 (E, hidden, ffn) K-contiguous,
    w2 (E, ffn, hidden) N-contiguous."""
    w = resolve_dtensor(w).view(-1, ffn_hidden_size, hidden_size)
    return w.permute(0, 2, 1) if name in ("w1", "w3") else w


def get_mlp_weights_lora(w: torch.Tensor, lora_A: torch.Tensor, lora_B: torch.Tensor, r: int,
                         ffn_hidden_size: int, hidden_size: int, name: str = "w1"):
    """Adapter storage of the reference (lora_A.weight kept transposed as (E*hidden, r), lora_B.weight (E*ffn, r),
    megablocks_utils/peft_utils.py:37-38,68-70) -> (W, A (E,K,r), B (E,r,N)) views, swapped for w2 (:51-56)."""
    W = get_mlp_weights(w, ffn_hidden_size, hidden_size, name)
    A = resolve_dtensor(lora_A).view(-1, hidden_size, r)
    B = resolve_dtensor(lora_B).view(-1, ffn_hidden_size, r).permute(0, 2, 1)
    if name == "w2":
        A, B = B.permute(0, 2, 1), A.permute(0, 2, 1)
    return W, A, B


class LoraViews(NamedTuple):
    a1: torch.Tensor
    b1: torch.Tensor
    a3: torch.Tensor
    b3: torch.Tensor
    a2: torch.Tensor
    b2: torch.Tensor


def _fast_path_ok(x, w1, w2, w3, lora: Optional[LoraViews]) -> bool:
    if x.dtype not in (torch.bfloat16, torch.float16) or w1.dtype != x.dtype:
        return False
    if lora is not None and any(t.dtype != x.dtype for t in lora):
        return False
    E, f, d = w1.shape
    if d % 64 or f % 64 or x.stride(-1) != 1 or x.stride(0) % 8:
        return False
    if not (w1.is_contiguous() and w2.is_contiguous() and w3.is_contiguous()):
        return False
    if lora is not None and lora.a1.size(2) > 128:   # the fused launches take an adapter as up to eight 16-wide rank chunks
        return False
    # gathered activation rows and one expert's matrix are addressed with 32-bit byte offsets (the same check the library
    # makes before it enqueues anything); the number of rows is otherwise not limited
    if (x.size(0) * x.stride(0) + d) * 2 >= 1 << 32 or (f * d + d) * 2 >= 1 << 32:
        return False
    return True


def _lora_arrays(tensors):
    ptrs = (ctypes.c_void_p * 6)(*[t.data_ptr() for t in tensors])
    strides = (ctypes.c_int64 * 18)(*[s for t in tensors for s in t.stride()])
    return ptrs, strides


class _SwiGLU(torch.autograd.Function):
    @staticmethod
    def forward(ctx, gate, up):
        ctx.save_for_backward(gate, up)
        return ops.swiglu(gate, up)

    @staticmethod
    def backward(ctx, dh):
        gate, up = ctx.saved_tensors
        return ops.swiglu_bwd(gate, up, dh)


def _mlp_fwd(x, w1, w3, w2, lora, scaling, ssi, offsets, fan_out, y_grouped, save_gate_up=True):
    dev = x.device
    E, f, d = w1.shape
    R = ssi.numel()
    rank = 0 if lora is None else lora.a1.size(2)
    gate = torch.empty((R, f), dtype=x.dtype, device=dev) if save_gate_up else None
    up = torch.empty((R, f), dtype=x.dtype, device=dev) if save_gate_up else None
    h = torch.empty((R, f), dtype=x.dtype, device=dev)
    y = torch.empty((R, d), dtype=x.dtype, device=dev)
    saved = workspace(lib.moe_mlp_saved_bytes(R, rank), dev)
    ws = workspace(lib.moe_mlp_workspace_bytes(R, E, d, f, rank), dev)
    lp, ls = (None, None) if lora is None else _lora_arrays(lora)
    check(lib.moe_mlp_fwd(ptr(x), x.stride(0), ptr(w1), ptr(w3), ptr(w2), lp, ls, rank, scaling, ptr(gate), ptr(up),
                          ptr(h), ptr(y), y.stride(0), ptr(ssi), is64(ssi), ptr(offsets), is64(offsets), E, R, d, f,
                          fan_out, int(y_grouped), dtype_code(x), ptr(saved), ptr(ws), ws.numel(), stream_ptr(dev)), "moe_mlp_fwd")
    return gate, up, h, y, saved


def _mlp_bwd(dy, dy_grouped, dy_fan_out, row_scale, x, w1, w3, w2, lora, scaling, gate, up, h, saved, ssi, offsets,
             fan_out, dx_grouped):
    dev = x.device
    E, f, d = w1.shape
    R = ssi.numel()
    rank = 0 if lora is None else lora.a1.size(2)
    dgate = torch.empty_like(gate)
    dup = torch.empty_like(up)
    dx_rows = torch.empty((R, d), dtype=x.dtype, device=dev)
    ws = workspace(lib.moe_mlp_workspace_bytes(R, E, d, f, rank), dev)
    grads = None
    lp = ls = gp = gs = None
    if lora is not None:
        grads = tuple(torch.empty_like(t) for t in lora)
        lp, ls = _lora_arrays(lora)
        gp, gs = _lora_arrays(grads)
    check(lib.moe_mlp_bwd(ptr(dy), dy.stride(0), int(dy_grouped), dy_fan_out, ptr(row_scale), ptr(x), x.stride(0),
                          ptr(w1), ptr(w3), ptr(w2), lp, ls, gp, gs, rank, scaling, ptr(gate), ptr(up), ptr(h),
                          ptr(dgate), ptr(dup), ptr(dx_rows), dx_rows.stride(0), int(dx_grouped), ptr(ssi), is64(ssi),
                          ptr(offsets), is64(offsets), E, R, d, f, fan_out, dtype_code(x), ptr(saved), ptr(ws), ws.numel(),
                          stream_ptr(dev)), "moe_mlp_bwd")
    return dx_rows, grads, dgate, dup


def _base_weight_grads(needs, x, dy, dy_grouped, dy_fan_out, coeff, dgate, dup, h, ssi, offsets, fan_out, E):
    """Gradients of the stored (E, f, d) expert weights (full fine-tuning; the reference gets them from
    scattermoe's group_bwd_W in ParallelLinear.backward): dW2[e] = h_e^T dy_e, dW1[e] = dgate_e^T x_e,
    dW3[e] = dup_e^T x_e over each expert's grouped rows -- already in the storage orientation, no transposes.
    `needs` = (w1, w3, w2) flags; `coeff` the per-assignment gate weights folded into dy (or None)."""
    d_w1 = d_w3 = d_w2 = None
    if needs[0] or needs[1]:
        x_g = ops.group(x, ssi, fan_out=fan_out)
        if needs[0]:
            d_w1 = ops.group_bwd_W(x_g, dgate, offsets, E)
        if needs[1]:
            d_w3 = ops.group_bwd_W(x_g, dup, offsets, E)
    if needs[2]:
        dy_g = dy if dy_grouped else ops.group(dy, ssi, coeff=coeff, fan_out=dy_fan_out)
        d_w2 = ops.group_bwd_W(dy_g, h, offsets, E)
    return d_w1, d_w3, d_w2


class FusedExpertMLP(torch.autograd.Function):
    """silu(x W1^T) * (x W3^T) -> W2 over ragged expert groups, with adapters, optional gate-weighted combine."""

    @staticmethod
    def forward(ctx, x, w1, w3, w2, a1, b1, a3, b3, a2, b2, lora_alpha, gates, ssi, offsets, fan_out, grouped_out):
        lora = None if a1 is None else LoraViews(a1, b1, a3, b3, a2, b2)
        scaling = 0.0 if lora is None else float(lora_alpha) / a1.size(2)
        y_grouped = bool(grouped_out) and gates is None
        gate, up, h, y, saved = _mlp_fwd(x, w1, w3, w2, lora, scaling, ssi, offsets, fan_out, y_grouped)
        out = y if gates is None else ops.combine(y, gates)
        ctx.save_for_backward(x, w1, w3, w2, a1, b1, a3, b3, a2, b2, gates, ssi, offsets, gate, up, h, saved,
                              y if gates is not None else None)
        ctx.cfg = (scaling, fan_out, y_grouped)
        return out

    @staticmethod
    def backward(ctx, dout):
        (x, w1, w3, w2, a1, b1, a3, b3, a2, b2, gates, ssi, offsets, gate, up, h, saved, y) = ctx.saved_tensors
        scaling, fan_out, y_grouped = ctx.cfg
        lora = None if a1 is None else LoraViews(a1, b1, a3, b3, a2, b2)
        dout = dout.contiguous()
        d_gates = row_scale = None
        if gates is not None:
            k = gates.size(1)
            d_gates = ops.combine_dgates(y, dout, k, gates.dtype)
            row_scale = ops.group(gates.reshape(-1, 1).float(), ssi)          # gate of each sorted position
            dy_grouped, dy_fan = False, k
        else:
            dy_grouped, dy_fan = y_grouped, 1
        dx_rows, grads, dgate, dup = _mlp_bwd(dout, dy_grouped, dy_fan, row_scale, x, w1, w3, w2, lora, scaling, gate, up,
                                              h, saved, ssi, offsets, fan_out, False)
        d_x = dx_rows if fan_out == 1 else ops.combine(dx_rows, None, k=fan_out)
        g = grads if grads is not None else (None,) * 6
        d_w = (None, None, None)
        if any(ctx.needs_input_grad[1:4]):
            d_w = _base_weight_grads(ctx.needs_input_grad[1:4], x, dout, dy_grouped, dy_fan,
                                     None if gates is None else gates.reshape(-1), dgate, dup, h, ssi, offsets, fan_out,
                                     w1.size(0))
        return (d_x,) + tuple(d_w) + tuple(g) + (None, d_gates, None, None, None, None)


def fused_expert_mlp(x, w1, w2, w3, k, sorted_scattered_idxs, expert_offsets, lora: Optional[LoraViews] = None,
                     lora_alpha: float = 1.0, gates: Optional[torch.Tensor] = None, grouped_out: bool = False):
    """Expert MLP on expert-grouped assignments.  x (rows, d); w1, w2, w3 (E, f, d) in the reference's storage
    layout; ``k`` = fan-out of x rows (top_k, or 1 for pre-dispatched rows).  With ``gates`` (T, k) the k expert
    rows of each token are combined and (T, d) is returned; otherwise one row per assignment, in grouped order
    when ``grouped_out`` else at its flat position."""
    require_gpu(x, w1, w2, w3, sorted_scattered_idxs, expert_offsets)
    lt = (None,) * 6 if lora is None else tuple(lora)
    if not _fast_path_ok(x, w1, w2, w3, lora):
        raise RuntimeError("fused_expert_mlp needs bf16, contiguous (E,f,d) weights, d and f multiples of 64 and rank <= 128; "
                           "use scattermoe_permute_and_compute for other cases")
    return FusedExpertMLP.apply(x, w1, w3, w2, *lt, lora_alpha, gates, sorted_scattered_idxs.contiguous(),
                                expert_offsets.contiguous(), k, grouped_out)


def scattermoe_permute_and_compute(x, w1, w2, w3, ffn_hidden_size, hidden_size, top_k, bin_ids, indices, num_experts,
                                   lora_pointers=None, moe_expert_model_parallelism=True, expert_offsets=None,
                                   lora_views: Optional[LoraViews] = None, lora_alpha: float = 1.0):
    """Functional form of the reference caller (config_utils.py:99-185).

    x (rows, hidden); w1, w2, w3 storage (E*ffn, hidden); ``bin_ids`` / ``indices`` = sorted expert ids and sorted
    flat positions; ``lora_pointers[name] = (A.weight, B.weight, r, alpha, hidden, ffn)`` as peft_utils.py:127-132
    (or ``lora_views`` / ``lora_alpha``: the six factor views already in (E, K, r) / (E, r, N) form).
    Expert-parallel mode treats x as pre-dispatched rows (fan-out 1) and scatters the output back to ``indices``;
    otherwise the fan-out is top_k and the output stays in grouped order (the caller's ops.scatter combines it)."""
    with torch.no_grad():
        if expert_offsets is None:
            expert_offsets = ops.expert_offsets_from_sorted(bin_ids, num_experts)
    fan = 1 if moe_expert_model_parallelism else top_k
    grouped_out = not moe_expert_model_parallelism
    W = {n: w.view(-1, ffn_hidden_size, hidden_size) for n, w in (("w1", w1), ("w2", w2), ("w3", w3))}
    lora = None
    alpha = 1.0
    if lora_pointers is not None:
        v = {}
        for n in ("w1", "w2", "w3"):
            A, B, r, alpha, hs, fs = lora_pointers[n]
            _, v["a" + n[1]], v["b" + n[1]] = get_mlp_weights_lora(W[n], A, B, r, fs, hs, n)
        lora = LoraViews(v["a1"], v["b1"], v["a3"], v["b3"], v["a2"], v["b2"])
    elif lora_views is not None:
        lora, alpha = lora_views, lora_alpha
    if _fast_path_ok(x, W["w1"], W["w2"], W["w3"], lora):
        return fused_expert_mlp(x, W["w1"], W["w2"], W["w3"], fan, indices, expert_offsets, lora, alpha, None, grouped_out)
    # generic route: the reference's three calls (:127-166)
    def proj(inp, name, kk, gin, gout):
        Wv = get_mlp_weights(W[name], ffn_hidden_size, hidden_size, name)
        if lora is None:
            return parallel_linear(inp, Wv, kk, bin_ids, indices, None, expert_offsets, None, gin, gout)
        a, b = getattr(lora, "a" + name[1]), getattr(lora, "b" + name[1])
        return parallel_linear_lora(inp, Wv, a, b, a.size(2), alpha, kk, bin_ids, indices, None, expert_offsets, None,
                                    gin, gout)
    h1 = proj(x, "w1", fan, False, True)
    h3 = proj(x, "w3", fan, False, True)
    h = _SwiGLU.apply(h1, h3)
    return proj(h, "w2", 1, True, grouped_out)


# ---------------------------------------------------------------------------------------------------------------
# whole layer: router -> sort -> expert MLP -> weighted combine, one autograd node
# ---------------------------------------------------------------------------------------------------------------
class MoELayerFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, wg, w1, w3, w2, a1, b1, a3, b3, a2, b2, lora_alpha, top_k, normalize):
        lora = None if a1 is None else LoraViews(a1, b1, a3, b3, a2, b2)
        scaling = 0.0 if lora is None else float(lora_alpha) / a1.size(2)
        rt = _router.route_and_sort(x, wg, top_k, normalize)
        gate, up, h, y, saved = _mlp_fwd(x, w1, w3, w2, lora, scaling, rt.sorted_scattered_idxs, rt.expert_offsets,
                                         top_k, False)
        out = ops.combine(y, rt.weights)
        ctx.save_for_backward(x, wg, w1, w3, w2, a1, b1, a3, b3, a2, b2, rt.scores, rt.weights, rt.indices,
                              rt.sorted_scattered_idxs, rt.expert_offsets, gate, up, h, y, saved)
        ctx.cfg = (scaling, top_k, normalize)
        ctx.mark_non_differentiable(rt.indices)
        ctx.set_materialize_grads(False)   # an unused expert_weights output must not cost a zero-fill per step
        return out, rt.weights, rt.indices

    @staticmethod
    def backward(ctx, dout, _dw, _di):
        (x, wg, w1, w3, w2, a1, b1, a3, b3, a2, b2, scores, weights, indices, ssi, offsets, gate, up, h, y,
         saved) = ctx.saved_tensors
        scaling, k, normalize = ctx.cfg
        lora = None if a1 is None else LoraViews(a1, b1, a3, b3, a2, b2)
        dout = torch.zeros_like(x) if dout is None else dout.contiguous()
        d_gates = ops.combine_dgates(y, dout, k, torch.float32)
        if _dw is not None:   # the caller also used the returned expert weights (e.g. in an auxiliary loss)
            d_gates = d_gates + _dw.to(d_gates.dtype)
        dlogits = _router.router_topk_bwd(d_gates, weights, indices, scores, normalize)
        row_scale = ops.group(weights.reshape(-1, 1), ssi)
        dx_rows, grads, dgate, dup = _mlp_bwd(dout, False, k, row_scale, x, w1, w3, w2, lora, scaling, gate, up, h, saved,
                                              ssi, offsets, k, False)
        d_w = (None, None, None)
        if any(ctx.needs_input_grad[2:5]):
            d_w = _base_weight_grads(ctx.needs_input_grad[2:5], x, dout, False, k, weights.reshape(-1), dgate, dup, h, ssi,
                                     offsets, k, w1.size(0))
        # fan-out sum of the k expert rows of each token plus the router's contribution dlogits @ wg, one pass
        d_x = ops.combine(dx_rows, None, k=k, extra_coef=dlogits, extra_rows=wg if wg.stride(-1) == 1 else wg.contiguous())
        d_wg = _router.router_weight_grad(x, dlogits) if ctx.needs_input_grad[1] else None
        g = grads if grads is not None else (None,) * 6
        return (d_x, d_wg) + tuple(d_w) + tuple(g) + (None, None, None)


def moe_layer_forward(x, wg, w1, w2, w3, top_k=2, lora: Optional[LoraViews] = None, lora_alpha: float = 1.0,
                      normalize: bool = True):
    """x (T, d) bf16 -> (out (T, d), expert_weights (T, k) fp32, expert_indices (T, k) int32).
    wg (E, d) router weight; w1, w2, w3 (E, f, d) expert weights in the reference's storage layout."""
    require_gpu(x, wg, w1, w2, w3)
    if x.size(0) == 0:   # an empty batch routes nothing: empty outputs, and backward leaves every parameter's grad unset
        return (x.clone(), torch.zeros((0, top_k), dtype=torch.float32, device=x.device),
                torch.zeros((0, top_k), dtype=torch.int32, device=x.device))
    if not _fast_path_ok(x, w1, w2, w3, lora):
        scores, ew, ei = _router.forward_router(x, wg, top_k, normalize)
        sei, ssi, counts, offsets, inv = _router.sort_assignments(ei.int(), w1.size(0))
        E, f, d = w1.shape
        y = scattermoe_permute_and_compute(x, w1.reshape(E * f, d), w2.reshape(E * f, d), w3.reshape(E * f, d), f, d,
                                           top_k, sei, ssi, E, None, moe_expert_model_parallelism=False,
                                           expert_offsets=offsets, lora_views=lora, lora_alpha=lora_alpha)
        out = _GatherCombine.apply(y, ew, inv, ssi)
        return out, ew, ei.int()
    lt = (None,) * 6 if lora is None else tuple(lora)
    return MoELayerFn.apply(x, wg, w1, w3, w2, *lt, lora_alpha, top_k, normalize)


class _GatherCombine(torch.autograd.Function):
    """out[t] = sum_j w[t,j] * y_grouped[inv[t*k+j]]  (megablocks ops.scatter, config_utils.py:251)."""

    @staticmethod
    def forward(ctx, y, w, inv, ssi):
        ctx.save_for_backward(y, w, inv, ssi)
        return ops.combine(y, w, inv=inv)

    @staticmethod
    def backward(ctx, dout):
        y, w, inv, ssi = ctx.saved_tensors
        dout = dout.contiguous()
        k = w.size(1)
        d_w = ops.combine_dgates(y, dout, k, w.dtype, inv=inv)
        # dy_grouped[i] = w[pos_i] * dout[pos_i // k]; pos, the inverse of inv, is the sort's own sorted_scattered_idxs
        d_y = ops.group(dout, ssi, coeff=w.reshape(-1), fan_out=k)
        return d_y, d_w, None, None


class ScatterMoEBlock(nn.Module):
    """Drop-in for a Mixtral sparse-MoE block built the way the reference builds it: router weight (E, d), expert
    weights w1, w2, w3 stored (E*f, d) (megablocks_utils/sparse_mlp2.py:22-36, HF w2 transposed on load,
    shard_moe_utils.py:153-157), optional LoRA factors stored as peft_utils.py:37-38,68-70 does.  Returns
    ``(hidden, None)`` like the patched ParallelMLP.forward (config_utils.py:75-92); with ``bias=True`` the block owns an
    output bias (megablocks' ``ParallelMLP.bias``) and follows that method's bias branch (config_utils.py:80-84):
    ``(hidden, bias)`` when ``return_bias`` is set, otherwise the single tensor ``hidden + bias``."""

    def __init__(self, hidden_size, ffn_hidden_size, num_experts, top_k=2, lora_r=0, lora_alpha=16.0,
                 dtype=torch.bfloat16, device=None, bias=False, return_bias=False):
        super().__init__()
        self.return_bias = return_bias
        self.bias = nn.Parameter(torch.zeros(hidden_size, dtype=dtype, device=device)) if bias else None
        self.hidden_size, self.ffn_hidden_size = hidden_size, ffn_hidden_size
        self.num_experts, self.top_k, self.lora_r, self.lora_alpha = num_experts, top_k, lora_r, lora_alpha
        kw = dict(dtype=dtype, device=device)
        self.router = nn.Parameter(torch.empty(num_experts, hidden_size, **kw))
        self.w1 = nn.Parameter(torch.empty(num_experts * ffn_hidden_size, hidden_size, **kw))
        self.w2 = nn.Parameter(torch.empty(num_experts * ffn_hidden_size, hidden_size, **kw))
        self.w3 = nn.Parameter(torch.empty(num_experts * ffn_hidden_size, hidden_size, **kw))
        for p in (self.router, self.w1, self.w2, self.w3):
            nn.init.normal_(p, std=0.02)
        if lora_r > 0:
            for n in ("w1", "w2", "w3"):
                a = nn.Parameter(torch.empty(num_experts * hidden_size, lora_r, **kw))
                b = nn.Parameter(torch.zeros(num_experts * ffn_hidden_size, lora_r, **kw))
                nn.init.normal_(a, std=0.02)
                self.register_parameter(f"lora_A_{n}", a)
                self.register_parameter(f"lora_B_{n}", b)
            for p in (self.router, self.w1, self.w2, self.w3) + (() if self.bias is None else (self.bias,)):
                p.requires_grad_(False)

    def lora_views(self) -> Optional[LoraViews]:
        if self.lora_r == 0:
            return None
        v = {}
        for n in ("w1", "w2", "w3"):
            _, a, b = get_mlp_weights_lora(getattr(self, n), getattr(self, f"lora_A_{n}"), getattr(self, f"lora_B_{n}"),
                                           self.lora_r, self.ffn_hidden_size, self.hidden_size, n)
            v["a" + n[1]], v["b" + n[1]] = a, b
        return LoraViews(v["a1"], v["b1"], v["a3"], v["b3"], v["a2"], v["b2"])

    def forward(self, hidden_states: torch.Tensor):
        shape = hidden_states.shape
        x = hidden_states.reshape(-1, shape[-1])
        E, f, d = self.num_experts, self.ffn_hidden_size, self.hidden_size
        out, _, _ = moe_layer_forward(x, self.router, self.w1.view(E, f, d), self.w2.view(E, f, d),
                                      self.w3.view(E, f, d), self.top_k, self.lora_views(), self.lora_alpha)
        out = out.view(shape)
        if self.bias is not None:
            if self.return_bias:
                return out, self.bias
            return out + self.bias
        return out, None
