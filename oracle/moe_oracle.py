"""TEST INFRASTRUCTURE ONLY -- CPU restatement (PyTorch fp32/fp64, per-expert loops) of the dropless
MoE expert-MLP path.  Only tests, the smoke check and the CPU-baseline leg of the benchmark may
import this module; the shipped package never does.

Every function is a restatement from the definition, written for clarity, not speed, and cites the
reference lines whose behaviour it follows.  Deliberate deviations from the reference's kernels:

* ``group_bwd_AB`` implements the mathematical definition (full reduction over N for dA and over K
  for dB).  The reference Triton kernel only does that when K <= 128 and N <= 128
  (scattermoe_utils/kernels/ops.py:399-405 store per-block partial sums with a plain store).
* LoRA interim ``s * (x @ A)`` is kept in the working precision here; the reference rounds it to
  the storage dtype per 32-wide K chunk (ops.py:139-141), an artefact of its tiling.
* ``parallel_linear_lora`` returns ``d_gates`` in the ``gates`` slot (the reference returns 15
  values for 14 inputs, parallel_linear_lora.py:136-149).

Pins (tests/test_oracle_*.py): the index fixture and shapes of tests/test_scattermoe.py:84-85,114-120;
the docstring example of ops.py:45-49; transformers' MixtralSparseMoeBlock / MixtralTopKRouter as an
independent library restatement of the block; torch.autograd.gradcheck in fp64; brute-force loops.
The router's optional switches (``router_with_options``): bias, p-norm and jitter are pinned by the library
routines they consist of (F.linear, torch.norm, a product); the uniform expert assignment (megablocks'
published ``_uniform_expert_assignment``, called at config_utils.py:272-279: experts 0..E-1 handed out in turn over the
flattened assignments, ``arange % E``) by that closed form (tests/test_oracle_routing.py).
"""
from __future__ import annotations

import ctypes
import os
from typing import Optional, Tuple

import numpy as np
import torch
import torch.nn.functional as F

_HERE = os.path.dirname(os.path.abspath(__file__))
_CLIB = None


def routing_clib() -> ctypes.CDLL:
    """The C restatement of the integer pipeline (oracle/routing_oracle.c), built by `make -C oracle`."""
    global _CLIB
    if _CLIB is None:
        path = os.path.join(_HERE, "liboracle_routing.so")
        if not os.path.exists(path):
            raise RuntimeError(f"{path} is missing: run `make -C oracle` (or __graft_entry__.build())")
        lib = ctypes.CDLL(path)
        lib.oracle_topk_renorm.restype = ctypes.c_int
        lib.oracle_sort_by_expert.restype = ctypes.c_int
        lib.oracle_padded_block_indices.restype = ctypes.c_int64
        _CLIB = lib
    return _CLIB


def _p(a: np.ndarray):
    return a.ctypes.data_as(ctypes.c_void_p)


# ----------------------------------------------------------------------------------------------
# A1 router: megablocks_utils/config_utils.py:255-280 (softmax -> top-k -> L1 renorm); fp32 as in
# transformers' MixtralTopKRouter.forward (softmax in float, topk, divide by sum).
# ----------------------------------------------------------------------------------------------
def router_from_logits(logits: torch.Tensor, k: int, renorm: bool = True):
    """logits (T,E) -> (scores (T,E) fp32, weights (T,k) fp32, indices (T,k) int64)."""
    scores = torch.softmax(logits.float(), dim=-1)
    w, idx = torch.topk(scores, k, dim=-1)
    if renorm:
        w = w / w.sum(dim=-1, keepdim=True)       # == w / torch.norm(w, p=1): scores are positive
    return scores, w, idx


def router(x: torch.Tensor, wg: torch.Tensor, k: int, renorm: bool = True):
    """x (T,d), wg (E,d): config_utils.py:262 (F.linear then softmax)."""
    logits = F.linear(x.float(), wg.float())
    return (logits,) + router_from_logits(logits, k, renorm)


def router_with_options(x: torch.Tensor, wg: torch.Tensor, k: int, p=1, bias: Optional[torch.Tensor] = None,
                        jitter: Optional[torch.Tensor] = None, uniform_expert_assignment: bool = False):
    """The patched router with every switch it has (config_utils.py:255-280): input jitter `x * jitter` (:256-257, the
    factor is passed in), linear layer with optional bias (:259-262), softmax, top-k (:263), division by the p-norm of
    the selected scores when p is set (:264-270), and the uniform assignment that replaces the indices by
    0, 1, .., E-1, 0, 1, .. in flat order (:272-279; megablocks' `_uniform_expert_assignment`, whose source is not part
    of the reference tree: restated from its name and use, parity unpinned).
    Returns (scores (T,E), weights (T,k), indices (T,k) int64), fp32."""
    xf = x.float() if jitter is None else x.float() * jitter.float()
    logits = F.linear(xf, wg.float(), None if bias is None else bias.float())
    scores = torch.softmax(logits, dim=-1)
    w, idx = torch.topk(scores, k, dim=-1)
    if p:
        w = w / torch.norm(w, p=float(p), dim=-1, keepdim=True)
    if uniform_expert_assignment:
        idx = torch.remainder(torch.arange(idx.numel(), dtype=idx.dtype), wg.size(0)).view(idx.shape)
    return scores, w, idx


def topk_renorm_c(scores: np.ndarray, k: int, renorm: bool = True):
    """Same selection through the C restatement (ties -> lower expert index)."""
    scores = np.ascontiguousarray(scores, dtype=np.float32)
    T, E = scores.shape
    idx = np.empty((T, k), dtype=np.int32)
    w = np.empty((T, k), dtype=np.float32)
    rc = routing_clib().oracle_topk_renorm(_p(scores), ctypes.c_int64(T), E, k, int(renorm), _p(idx), _p(w))
    assert rc == 0
    return w, idx


# ----------------------------------------------------------------------------------------------
# A2 flatten_and_sort (+ histogram / cumsum): call sites config_utils.py:131-132; stable order is
# what megablocks' radix sort and the reference test fixture (tests/test_scattermoe.py:84-85) give.
# ----------------------------------------------------------------------------------------------
def flatten_and_sort(expert_idxs: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    flat = expert_idxs.flatten()
    sorted_expert_idxs, sorted_scattered_idxs = torch.sort(flat, stable=True)
    return sorted_expert_idxs, sorted_scattered_idxs


def sort_by_expert_c(expert_idxs: np.ndarray, E: int):
    """C counting sort: returns dict(sorted_expert, sorted_pos, counts, offsets, inv)."""
    flat = np.ascontiguousarray(expert_idxs, dtype=np.int32).reshape(-1)
    R = flat.shape[0]
    out = dict(sorted_expert=np.empty(R, np.int32), sorted_pos=np.empty(R, np.int32),
               counts=np.empty(E, np.int32), offsets=np.empty(E, np.int32), inv=np.empty(R, np.int32))
    rc = routing_clib().oracle_sort_by_expert(_p(flat), ctypes.c_int64(R), E, _p(out["sorted_expert"]),
                                              _p(out["sorted_pos"]), _p(out["counts"]), _p(out["offsets"]),
                                              _p(out["inv"]))
    assert rc == 0
    return out


# ----------------------------------------------------------------------------------------------
# A3 padded_block_indices: semantics at scattermoe_utils/kernels/ops.py:39-51, consumers ops.py:56,
# ops.py:315-319; called at config_utils.py:114-118 and tests/test_scattermoe.py:161-163.
# ----------------------------------------------------------------------------------------------
def padded_block_indices(sorted_experts_idxs: torch.Tensor, k: int, N_BLOCK_SIZE: int = 128):
    """k is the number of experts (the reference's argument name). Returns int64 tensors."""
    counts = torch.bincount(sorted_experts_idxs.long(), minlength=k)[:k]
    ends = torch.cumsum(counts, 0)
    starts = ends - counts
    blocks = []
    for e in range(k):
        c = int(counts[e])
        for j in range((c + N_BLOCK_SIZE - 1) // N_BLOCK_SIZE):
            blocks.append(int(starts[e]) + j * N_BLOCK_SIZE)
    return torch.tensor(blocks, dtype=torch.int64), ends.to(torch.int64)


def padded_block_indices_c(sorted_experts_idxs: np.ndarray, E: int, block: int = 128):
    sei = np.ascontiguousarray(sorted_experts_idxs, dtype=np.int32)
    R = sei.shape[0]
    cap = R // block + E + 1
    blocks = np.empty(cap, np.int32)
    offsets = np.empty(E, np.int32)
    nb = routing_clib().oracle_padded_block_indices(_p(sei), ctypes.c_int64(R), E, block, _p(blocks),
                                                    ctypes.c_int64(cap), _p(offsets))
    assert nb >= 0
    return blocks[:nb].copy(), offsets


# ----------------------------------------------------------------------------------------------
# A4 scatter2scatter(_lora): scattermoe_utils/kernels/ops.py:37-150 (row/expert/mask semantics
# :56-83, math :131-141, masked store :149-150), wrapper :156-212.
# ----------------------------------------------------------------------------------------------
def scatter2scatter_lora(X, W, A, B, lora_alp, sorted_expert_idxs, sorted_scattered_idxs, k,
                         padded_block_idxs=None, x_grouped=False, y_grouped=False, out=None):
    """Y[out_row(i)] = X[in_row(i)] @ (W[e_i] + (lora_alp / r) * A[e_i] @ B[e_i]) for every sorted
    position i; in_row = i if x_grouped else ssi[i] // k; out_row = i if y_grouped else ssi[i].
    A/B may be None (plain scatter2scatter).  Computation in X's dtype promoted to at least fp32."""
    sei = sorted_expert_idxs.long()
    ssi = sorted_scattered_idxs.long()
    L = sei.shape[0]
    assert ssi.shape[0] == L
    E, K, N = W.shape
    ct = torch.float64 if X.dtype == torch.float64 else torch.float32
    Y = torch.zeros((L, N), dtype=ct) if out is None else out
    pos = torch.arange(L)
    in_rows = pos if x_grouped else ssi // k
    out_rows = pos if y_grouped else ssi
    for e in range(E):
        sel = sei == e
        if not bool(sel.any()):
            continue
        xe = X[in_rows[sel]].to(ct)
        ye = xe @ W[e].to(ct)
        if A is not None:
            s = lora_alp / A.shape[2]
            ye = ye + ((xe @ A[e].to(ct)) * s) @ B[e].to(ct)
        Y[out_rows[sel]] = ye.to(Y.dtype)
    return Y


# ----------------------------------------------------------------------------------------------
# scattermoe.kernels.ops.group: call sites scattermoe_utils/parallel_linear_lora.py:87-91,98
# out[i] = src[ssi[i] // fan_out] * coeff[ssi[i]]
# ----------------------------------------------------------------------------------------------
def group(A, sorted_scattered_idxs, coeff=None, fan_out=1):
    ssi = sorted_scattered_idxs.long()
    out = A[ssi // fan_out]
    if coeff is not None:
        out = out * coeff.flatten()[ssi][:, None]
    return out


# ----------------------------------------------------------------------------------------------
# A7 group_bwd_AB: definition at scattermoe_utils/kernels/ops.py:284-289 (dA = s X^T dY B^T,
# dB = s A^T X^T dY), group bounds :315-319, zero for empty experts :224-225,:344.
# ----------------------------------------------------------------------------------------------
def group_bwd_AB(DY, X, A, B, scaling, expert_offsets, E):
    ct = torch.float64 if X.dtype == torch.float64 else torch.float32
    K, r, N = X.shape[-1], A.shape[2], DY.shape[-1]
    DA = torch.zeros((E, K, r), dtype=ct)
    DB = torch.zeros((E, r, N), dtype=ct)
    start = 0
    for e in range(E):
        end = int(expert_offsets[e])
        if end > start:
            xe, dye = X[start:end].to(ct), DY[start:end].to(ct)
            DA[e] = scaling * (xe.T @ (dye @ B[e].to(ct).T))
            DB[e] = scaling * ((xe @ A[e].to(ct)).T @ dye)
        start = end
    return DA, DB


def group_bwd_W(DY, X, expert_offsets, E):
    """scattermoe.kernels.ops.group_bwd_W (selected at config_utils.py:124-125): dW[e] = X_e^T dY_e."""
    ct = torch.float64 if X.dtype == torch.float64 else torch.float32
    DW = torch.zeros((E, X.shape[-1], DY.shape[-1]), dtype=ct)
    start = 0
    for e in range(E):
        end = int(expert_offsets[e])
        if end > start:
            DW[e] = X[start:end].to(ct).T @ DY[start:end].to(ct)
        start = end
    return DW


# ----------------------------------------------------------------------------------------------
# A5/A8 parallel_linear(_lora) written with differentiable torch ops so torch.autograd supplies
# dX, dA, dB, dW, d_gates: scattermoe_utils/parallel_linear_lora.py:13-53 (forward incl. the gates
# bmm :30-35), :56-149 (backward it must agree with).
# ----------------------------------------------------------------------------------------------
def parallel_linear_lora(inputs, expert_weights, expert_lora_A, expert_lora_B, lora_r, lora_alp, k,
                         sorted_expert_idxs, sorted_scattered_idxs, padded_block_idxs=None,
                         expert_offsets=None, gates=None, grouped_in=False, grouped_out=False):
    sei = sorted_expert_idxs.long()
    ssi = sorted_scattered_idxs.long()
    L = sei.shape[0]
    E, K, N = expert_weights.shape
    pos = torch.arange(L)
    in_rows = pos if grouped_in else ssi // k
    xg = inputs[in_rows]                                        # (L,K) in sorted order
    ys = []
    bounds = torch.searchsorted(sei, torch.arange(E + 1))
    for e in range(E):
        lo, hi = int(bounds[e]), int(bounds[e + 1])
        xe = xg[lo:hi]
        ye = xe @ expert_weights[e]
        if expert_lora_A is not None:
            s = lora_alp / expert_lora_A.shape[2]
            ye = ye + ((xe @ expert_lora_A[e]) * s) @ expert_lora_B[e]
        ys.append(ye)
    yg = torch.cat(ys, 0)                                       # grouped order
    if grouped_out:
        out = yg
    else:
        out = torch.zeros_like(yg).index_copy(0, ssi, yg)       # out[ssi[i]] = yg[i]
    if gates is not None:
        out = (gates[:, :, None] * out.view(gates.shape[0], gates.shape[1], N)).sum(1)
    return out


# ----------------------------------------------------------------------------------------------
# A11 weighted combine (megablocks ops.scatter at config_utils.py:251):
# out[t] = sum_j w[t,j] * y_grouped[inv[t*k+j]]
# ----------------------------------------------------------------------------------------------
def combine(y_grouped, sorted_scattered_idxs, weights, T, k):
    ssi = sorted_scattered_idxs.long()
    scattered = torch.zeros_like(y_grouped).index_copy(0, ssi, y_grouped)
    return (weights.reshape(T, k, 1).to(y_grouped.dtype) * scattered.view(T, k, -1)).sum(1)


# ----------------------------------------------------------------------------------------------
# A10 whole block: router (config_utils.py:255-280) + w1, w3, silu*mul, w2 of
# scattermoe_permute_and_compute (config_utils.py:127-166) + weighted combine (:251), in the
# per-expert-loop + index_add_ form of the HF MixtralSparseMoeBlock.  Weights in the reference's
# storage layout: w1, w2, w3 each (E, f, d) (sparse_mlp2.py:22-36 viewed as config_utils.py:31);
# LoRA: lora[name] = (A (E,K,r), B (E,r,N)) in the views of config_utils.py:48-56.
# ----------------------------------------------------------------------------------------------
def moe_block(x, wg, w1, w2, w3, k=2, lora=None, lora_alpha=32.0, renorm=True, routing=None):
    """x (T,d). Returns (out (T,d), aux dict).  `routing` = (weights (T,k), idx (T,k)) overrides the router."""
    T, d = x.shape
    E = w1.shape[0]
    if routing is None:
        logits, scores, gw, idx = router(x, wg, k, renorm)
    else:
        gw, idx = routing
        logits = scores = None
    out = torch.zeros_like(x)
    for e in range(E):
        tok, slot = torch.where(idx == e)
        if tok.numel() == 0:
            continue
        xe = x[tok]
        W1, W3, W2 = w1[e].T, w3[e].T, w2[e]                    # (d,f), (d,f), (f,d)
        h1, h3 = xe @ W1, xe @ W3
        if lora is not None:
            (A1, B1), (A3, B3) = lora["w1"], lora["w3"]
            s = lora_alpha / A1.shape[2]
            h1 = h1 + ((xe @ A1[e]) * s) @ B1[e]
            h3 = h3 + ((xe @ A3[e]) * s) @ B3[e]
        h = F.silu(h1) * h3
        y = h @ W2
        if lora is not None:
            A2, B2 = lora["w2"]
            y = y + ((h @ A2[e]) * (lora_alpha / A2.shape[2])) @ B2[e]
        out = out.index_add(0, tok, y * gw[tok, slot][:, None].to(y.dtype))
    return out, dict(logits=logits, scores=scores, weights=gw, indices=idx)
