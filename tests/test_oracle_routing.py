"""Pins the integer/routing part of the CPU oracle (C restatement + torch restatement) against the reference's own
fixture, the documented example, library routines and brute force.  Runs without a GPU."""
import numpy as np
import pytest
import torch
from hypothesis import given, settings, strategies as st


def _golden():
    import json, os
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_known_answers.json")) as fh:
        return json.load(fh)


def test_reference_index_fixture(oracle):
    # tests/test_scattermoe.py:84-85 of the reference hard-codes the two sorted vectors for 10 tokens, 2 experts, k=1;
    # they are the stable sort of the assignment vector stored beside them
    fx = _golden()["index_fixture"]
    expert_idxs = np.array(fx["implied"]["expert_idxs"])
    out = oracle.sort_by_expert_c(expert_idxs, fx["implied"]["num_experts"])
    assert out["sorted_expert"].tolist() == fx["held"]["sorted_expert_idxs"]
    assert out["sorted_pos"].tolist() == fx["held"]["sorted_scattered_idxs"]
    sei, ssi = oracle.flatten_and_sort(torch.tensor(expert_idxs))
    assert sei.tolist() == fx["held"]["sorted_expert_idxs"] and ssi.tolist() == fx["held"]["sorted_scattered_idxs"]
    # no other assignment of 10 tokens to 2 experts sorts to the held vectors: the held order fixes every position
    inv = np.empty(10, dtype=np.int64)
    inv[np.array(fx["held"]["sorted_scattered_idxs"])] = np.array(fx["held"]["sorted_expert_idxs"])
    assert inv.tolist() == fx["implied"]["expert_idxs"]
    # padded_block_indices(sorted_expert_idxs, 2) as the reference test calls it (:161-163)
    pb, eo = oracle.padded_block_indices(sei, 2)
    assert pb.tolist() == fx["implied"]["padded_block_idxs"] and eo.tolist() == fx["implied"]["expert_offsets"]
    pbc, eoc = oracle.padded_block_indices_c(sei.numpy(), 2)
    assert pbc.tolist() == fx["implied"]["padded_block_idxs"] and eoc.tolist() == fx["implied"]["expert_offsets"]


def test_documented_block_example(oracle):
    # scattermoe_utils/kernels/ops.py:45-49: 300 rows of expert 0 then expert 1 -> [0, 128, 256, 300, 428, ...]
    fx = _golden()["documented_block_example"]
    n0, n1 = fx["held"]["rows_of_expert_0"], fx["implied"]["rows_of_expert_1_used_here"]
    sei = torch.tensor([0] * n0 + [1] * n1)
    pb, eo = oracle.padded_block_indices(sei, 2, fx["held"]["block_m"])
    assert pb.tolist()[:5] == fx["held"]["block_start_idx_prefix"]
    assert pb.tolist() == fx["implied"]["padded_block_idxs"] and eo.tolist() == fx["implied"]["expert_offsets"]
    pbc, eoc = oracle.padded_block_indices_c(sei.numpy(), 2)
    assert pbc.tolist() == fx["implied"]["padded_block_idxs"] and eoc.tolist() == fx["implied"]["expert_offsets"]


@pytest.mark.parametrize("counts", [[0, 5, 0], [128, 128], [129, 0, 1], [0, 0, 0, 7], [256], [1] * 9])
def test_block_edge_cases(oracle, counts):
    sei = torch.tensor([e for e, c in enumerate(counts) for _ in range(c)], dtype=torch.int64)
    pb, eo = oracle.padded_block_indices(sei, len(counts))
    exp, start = [], 0
    for c in counts:
        exp += [start + 128 * j for j in range(-(-c // 128))]
        start += c
    assert pb.tolist() == exp and eo.tolist() == np.cumsum(counts).tolist()
    pbc, eoc = oracle.padded_block_indices_c(sei.numpy(), len(counts))
    assert pbc.tolist() == exp and eoc.tolist() == np.cumsum(counts).tolist()


@settings(max_examples=60, deadline=None)
@given(st.integers(1, 12), st.integers(0, 700), st.integers(0, 2 ** 31 - 1), st.sampled_from([1, 4, 128]))
def test_sort_properties(oracle, E, R, seed, block):
    rng = np.random.default_rng(seed)
    idx = rng.integers(0, E, size=R)
    out = oracle.sort_by_expert_c(idx, E)
    order = np.argsort(idx, kind="stable")
    assert np.array_equal(out["sorted_pos"], order)
    assert np.array_equal(out["sorted_expert"], idx[order])
    assert np.array_equal(out["counts"], np.bincount(idx, minlength=E))
    assert np.array_equal(out["offsets"], np.cumsum(np.bincount(idx, minlength=E)))
    assert np.array_equal(out["inv"][out["sorted_pos"]], np.arange(R))
    sei_t, ssi_t = oracle.flatten_and_sort(torch.from_numpy(idx))
    assert np.array_equal(ssi_t.numpy(), order)
    pbc, eoc = oracle.padded_block_indices_c(out["sorted_expert"], E, block)
    # brute force: a block starts at every row whose distance from its group's start is a multiple of `block`
    starts = np.concatenate([[0], np.cumsum(np.bincount(idx, minlength=E))[:-1]])
    brute = [i for i in range(R) if (i - starts[out["sorted_expert"][i]]) % block == 0]
    assert pbc.tolist() == brute
    if block == 128:
        pbt, eot = oracle.padded_block_indices(sei_t, E)
        assert pbt.tolist() == brute and eot.tolist() == eoc.tolist()


def test_topk_against_library_router(oracle):
    # independent statement of the same routing rule: transformers' Mixtral router (softmax in fp32, topk, renorm)
    from transformers.models.mixtral.modeling_mixtral import MixtralTopKRouter
    from transformers import MixtralConfig
    cfg = MixtralConfig(hidden_size=64, intermediate_size=128, num_local_experts=8, num_experts_per_tok=2,
                        num_hidden_layers=1, num_attention_heads=4, num_key_value_heads=4, vocab_size=32)
    torch.manual_seed(0)
    router = MixtralTopKRouter(cfg)
    with torch.no_grad():
        router.weight.normal_(0, 0.5)
    x = torch.randn(300, 64)
    with torch.no_grad():
        res = router(x)
    # (router_logits | probs, scores, indices) depending on the library version: take the last two
    lib_w, lib_idx = res[-2], res[-1]
    logits, scores, w, idx = oracle.router(x, router.weight.detach(), 2)
    assert torch.equal(idx, lib_idx)
    assert torch.allclose(w, lib_w.float(), atol=1e-6)
    # C restatement on the oracle's own scores: identical indices, weights to fp32 rounding
    wc, ic = oracle.topk_renorm_c(scores.numpy(), 2)
    assert np.array_equal(ic, idx.numpy())
    assert np.allclose(wc, w.numpy(), atol=1e-6)
    # invariants
    assert torch.allclose(w.sum(-1), torch.ones(300), atol=1e-6)
    assert (idx[:, 0] != idx[:, 1]).all() and (scores.gather(1, idx)[:, 0] >= scores.gather(1, idx)[:, 1]).all()


def test_topk_ties_and_bruteforce(oracle):
    s = np.array([[0.25, 0.25, 0.25, 0.25], [0.1, 0.4, 0.4, 0.1], [0.7, 0.1, 0.1, 0.1]], dtype=np.float32)
    w, i = oracle.topk_renorm_c(s, 2)
    assert i.tolist() == [[0, 1], [1, 2], [0, 1]]          # ties go to the lower expert id
    assert np.allclose(w, [[0.5, 0.5], [0.5, 0.5], [0.875, 0.125]])
    rng = np.random.default_rng(1)
    s = rng.random((200, 6)).astype(np.float32)
    w, i = oracle.topk_renorm_c(s, 3, renorm=False)
    order = np.argsort(-s, axis=1, kind="stable")[:, :3]
    assert np.array_equal(i, order) and np.allclose(w, np.take_along_axis(s, order, 1))


def test_router_switches_reduce_to_library_routines(oracle):
    """`router_with_options` against what fixes each switch: p=1 / p=None reproduce the plain router (itself pinned by
    transformers' MixtralTopKRouter above), p=2 leaves unit 2-norm weights in the same order, a bias equals an extra
    input column of ones whose weight is the bias, jitter is a product on the input, and the uniform assignment hands
    out experts 0..E-1 in turn (its only specification is the call site, config_utils.py:272-279)."""
    g = torch.Generator().manual_seed(3)
    x, wg, b = torch.randn(40, 24, generator=g), torch.randn(6, 24, generator=g), torch.randn(6, generator=g)
    _, s, w, i = oracle.router(x, wg, 2, True)
    s1, w1, i1 = oracle.router_with_options(x, wg, 2, 1)
    assert torch.equal(i, i1) and torch.allclose(w, w1) and torch.allclose(s, s1)
    _, _, w0, _ = oracle.router(x, wg, 2, False)
    assert torch.allclose(oracle.router_with_options(x, wg, 2, None)[1], w0)
    s2, w2, i2 = oracle.router_with_options(x, wg, 2, 2)
    assert torch.equal(i2, i) and torch.allclose((w2 ** 2).sum(-1), torch.ones(40)) and torch.allclose(w2 / w2.sum(-1, keepdim=True), w)
    sb, wb, ib = oracle.router_with_options(x, wg, 2, 1, bias=b)
    _, s_aug, w_aug, i_aug = oracle.router(torch.cat([x, torch.ones(40, 1)], 1), torch.cat([wg, b[:, None]], 1), 2, True)
    assert torch.equal(ib, i_aug) and torch.allclose(sb, s_aug, atol=1e-6) and torch.allclose(wb, w_aug, atol=1e-6)
    noise = 0.9 + 0.2 * torch.rand(40, 24, generator=g)
    sj, wj, ij = oracle.router_with_options(x, wg, 2, 1, jitter=noise)
    _, s_n, w_n, i_n = oracle.router(x * noise, wg, 2, True)
    assert torch.equal(ij, i_n) and torch.allclose(sj, s_n) and torch.allclose(wj, w_n)
    _, wu, iu = oracle.router_with_options(x, wg, 2, 1, uniform_expert_assignment=True)
    assert iu.flatten().tolist() == [j % 6 for j in range(80)] and torch.allclose(wu, w)


def test_c_restatement_is_clean_under_asan_and_ubsan():
    """The C restatement built with the host AddressSanitizer / UndefinedBehaviorSanitizer (`make -C oracle asan`) works
    through exact-size buffers over edge sizes (no rows, one expert, block-size boundaries, skewed groups, ties in the
    top-k) without a report and with every answer meeting its definition."""
    import os, subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run(["make", "-B", "-C", os.path.join(root, "oracle"), "asan"], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    assert "sanitizer run clean" in r.stdout and "ERROR" not in r.stderr and "runtime error" not in r.stderr
