"""HIP router + integer pipeline against the oracle: indices, sorted order, histogram, offsets and block table
must match bit for bit; softmax values to fp32 rounding."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _mods():
    import moe_distributed_training_amd as moe
    from moe_distributed_training_amd.megablocks_utils import router
    from moe_distributed_training_amd.scattermoe_utils.kernels import ops
    return moe, router, ops


@pytest.mark.parametrize("T,E,k", [(1, 1, 1), (7, 4, 2), (1000, 8, 2), (4096, 8, 2), (3000, 64, 4), (513, 3, 3)])
def test_topk_from_logits_bit_exact(dev, oracle, T, E, k):
    _, router, _ = _mods()
    torch.manual_seed(T + E)
    logits = torch.randn(T, E) * 1.3
    s, w, i = router.router_topk(logits.to(dev), k)
    so, wo, io = oracle.router_from_logits(logits, k)
    assert torch.equal(i.cpu().long(), io)
    assert torch.allclose(s.cpu(), so, atol=2e-7) and torch.allclose(w.cpu(), wo, atol=5e-7)
    # the C restatement fed the device's own softmax reproduces the device selection exactly
    wc, ic = oracle.topk_renorm_c(s.cpu().numpy(), k)
    assert np.array_equal(ic, i.cpu().numpy()) and np.allclose(wc, w.cpu().numpy(), atol=1e-7)


def test_topk_ties_lower_index(dev):
    _, router, _ = _mods()
    logits = torch.zeros(5, 6)
    logits[1, 4] = logits[1, 2] = 3.0
    _, w, i = router.router_topk(logits.to(dev), 2)
    assert i.cpu().tolist() == [[0, 1], [2, 4], [0, 1], [0, 1], [0, 1]]
    assert torch.allclose(w.cpu(), torch.full((5, 2), 0.5))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("T,d,E", [(4096, 4096, 8), (257, 100, 5), (33, 1032, 11)])
def test_router_end_to_end(dev, oracle, dtype, T, d, E):
    """x -> logits -> (weights, indices): logits within fp32 summation-order noise; indices identical to the fp32
    oracle on these seeded inputs (no token whose 2nd/3rd score gap is at the noise level)."""
    moe, router, _ = _mods()
    torch.manual_seed(0)
    x = torch.randn(T, d).to(dtype)
    wg = (torch.randn(E, d) * 0.02).to(dtype)
    k = min(2, E)
    logits = router.router_logits(x.to(dev), wg.to(dev))
    lo, so, wo, io = oracle.router(x, wg, k)
    assert torch.allclose(logits.cpu(), lo, atol=2e-5, rtol=1e-5)
    scores, w, idx = moe.forward_router(x.to(dev), wg.to(dev), k)
    assert idx.dtype == torch.int64
    srt = torch.sort(so, dim=-1, descending=True).values
    margin = (srt[:, k - 1] - srt[:, k]).abs().min() if E > k else torch.tensor(1.0)
    assert margin > 1e-6, "test data has a near tie; pick another seed"
    assert torch.equal(idx.cpu(), io)
    assert torch.allclose(w.cpu(), wo, atol=1e-5)
    # the one-call form: two launches give the same bits as the two calls; the single fused launch (<= 8 experts of a
    # 2-byte type, hidden size a multiple of 32) sums its logits on the matrix cores in another order -- fp32 rounding
    # apart, the same indices, and exactly the softmax / top-k of ITS logits
    l2, s2, w2, i2 = router.router_forward(x.to(dev), wg.to(dev), k)
    s1, w1, i1 = router.router_topk(l2, k)
    assert torch.equal(s2, s1) and torch.equal(w2, w1) and torch.equal(i2, i1)
    if dtype == torch.float32 or E > 8 or d % 32 != 0:
        assert torch.equal(l2, logits)
    else:
        assert torch.allclose(l2.cpu(), lo, atol=2e-5, rtol=1e-5) and torch.equal(i2.cpu().long(), io)


def test_router_forward_ragged_token_count(dev, oracle):
    """Token counts that do not fill the fused kernel's 16-token workgroups or 4-token waves."""
    _, router, _ = _mods()
    for T in (1, 3, 17, 63):
        torch.manual_seed(T)
        x = torch.randn(T, 256).bfloat16(); wg = (torch.randn(8, 256) * 0.05).bfloat16()
        l, s, w, i = router.router_forward(x.to(dev), wg.to(dev), 2)
        lo, so, wo, io = oracle.router(x, wg, 2)
        assert torch.allclose(l.cpu(), lo, atol=2e-5, rtol=1e-5) and torch.equal(i.cpu().long(), io)
        assert torch.allclose(s.cpu(), so, atol=1e-6) and torch.allclose(w.cpu(), wo, atol=1e-5)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,d,E,k", [(5, 32, 1, 1), (40, 96, 3, 2), (100, 544, 8, 2), (16, 8192, 8, 8), (1000, 1024, 7, 3)])
def test_router_matrix_core_kernel_shapes(dev, oracle, dtype, T, d, E, k):
    """The one-launch router (logits on the matrix cores) at hidden sizes that leave some of its eight waves without a
    K step (32, 96), that split unevenly over them (544 = 17 steps), with fewer than 8 experts (the unused rows of the
    weight operand must enter as zeros) and with token counts that do not fill its 16-token workgroups."""
    _, router, _ = _mods()
    torch.manual_seed(T + d + E)
    x = torch.randn(T, d).to(dtype)
    wg = (torch.randn(E, d) * 0.05).to(dtype)
    l, s, w, i = router.router_forward(x.to(dev), wg.to(dev), k)
    lo, so, wo, io = oracle.router(x, wg, k)
    srt = torch.sort(so, dim=-1, descending=True).values
    if E > k:
        assert (srt[:, k - 1] - srt[:, k]).abs().min() > 1e-6, "test data has a near tie; pick another seed"
    assert torch.allclose(l.cpu(), lo, atol=3e-5, rtol=1e-5)
    assert torch.equal(i.cpu().long(), io)
    assert torch.allclose(s.cpu(), so, atol=1e-6) and torch.allclose(w.cpu(), wo, atol=1e-5)


def test_reference_known_answers_on_the_device(dev):
    """The vectors the reference's own test holds (tests/test_scattermoe.py:84-85) and its documented block-table
    example (scattermoe_utils/kernels/ops.py:45-49), from the committed fixture, through the HIP path."""
    import json, os
    import moe_distributed_training_amd as moe
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_known_answers.json")) as fh:
        g = json.load(fh)
    fx = g["index_fixture"]
    for idt in (torch.int32, torch.int64):
        e = torch.tensor(fx["implied"]["expert_idxs"], dtype=idt, device=dev).view(-1, 1)
        sei, ssi = moe.flatten_and_sort(e)
        assert sei.cpu().tolist() == fx["held"]["sorted_expert_idxs"]
        assert ssi.cpu().tolist() == fx["held"]["sorted_scattered_idxs"]
        pb, eo = moe.padded_block_indices(sei, fx["implied"]["num_experts"])
        assert pb.cpu().tolist() == fx["implied"]["padded_block_idxs"] and eo.cpu().tolist() == fx["implied"]["expert_offsets"]
    ex = g["documented_block_example"]
    sei = torch.tensor([0] * ex["held"]["rows_of_expert_0"] + [1] * ex["implied"]["rows_of_expert_1_used_here"], device=dev)
    pb, eo = moe.padded_block_indices(sei, 2, ex["held"]["block_m"])
    assert pb.cpu().tolist() == ex["implied"]["padded_block_idxs"] and eo.cpu().tolist() == ex["implied"]["expert_offsets"]


@pytest.mark.parametrize("idt", [torch.int32, torch.int64])
@pytest.mark.parametrize("R,E", [(0, 4), (1, 1), (10, 2), (8192, 8), (32768, 8), (5000, 64), (70000, 300), (16384, 8), (16385, 8),
                                 (300, 65), (1023, 3)])
def test_sort_bit_exact(dev, oracle, idt, R, E):
    _, router, ops = _mods()
    rng = np.random.default_rng(R + E)
    p = rng.random(E) ** 3 + 1e-3                                   # ragged, some experts nearly empty
    if E > 3:
        p[1] = 0.0                                                  # one expert with no rows at all
    idx = rng.choice(E, size=R, p=p / p.sum()).astype(np.int64)
    exp = oracle.sort_by_expert_c(idx, E)
    t = torch.from_numpy(idx).to(idt).to(dev)
    sei, ssi, counts, offs, inv = router.sort_assignments(t, E)
    assert sei.dtype == idt and ssi.dtype == idt
    assert np.array_equal(sei.cpu().numpy(), exp["sorted_expert"])
    assert np.array_equal(ssi.cpu().numpy(), exp["sorted_pos"])
    assert np.array_equal(counts.cpu().numpy(), exp["counts"])
    assert np.array_equal(offs.cpu().numpy(), exp["offsets"])
    assert np.array_equal(inv.cpu().numpy(), exp["inv"])
    if R > 0:
        pb, eo = ops.padded_block_indices(sei, E)
        pbo, eoo = oracle.padded_block_indices_c(exp["sorted_expert"], E)
        assert pb.dtype == torch.int64 and np.array_equal(pb.cpu().numpy(), pbo) and np.array_equal(eo.cpu().numpy(), eoo)
        # scattermoe's flatten_and_sort on the (T,k)-shaped tensor
        s2, p2 = ops.flatten_and_sort(t.view(-1, 1) if R % 2 else t.view(-1, 2))
        assert np.array_equal(s2.cpu().numpy(), exp["sorted_expert"]) and np.array_equal(p2.cpu().numpy(), exp["sorted_pos"])
        assert s2.dtype == idt and p2.dtype == torch.int64          # as torch.sort: values keep the dtype, positions are int64
        s3, p3 = ops.flatten_and_sort(t, num_experts=E)
        assert torch.equal(s3, s2) and torch.equal(p3, p2)


def test_flatten_and_sort_never_synchronises(dev):
    """The drop-in flatten_and_sort (no expert-count argument, like the torch.sort it replaces) reads nothing back to the
    host: it can be captured into a graph, and replays follow the captured buffer's new contents."""
    _, _, ops = _mods()
    t = torch.randint(0, 8, (4096, 2), device=dev)
    ops.flatten_and_sort(t)                       # first call outside capture (module / attribute set-up)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        ops.flatten_and_sort(t)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        sei, ssi = ops.flatten_and_sort(t)
    for seed in range(3):
        t.copy_(torch.randint(0, 8, (4096, 2), generator=torch.Generator().manual_seed(seed)))
        graph.replay()
        torch.cuda.synchronize()
        want_e, want_p = torch.sort(t.flatten().cpu(), stable=True)
        assert torch.equal(sei.cpu(), want_e) and torch.equal(ssi.cpu(), want_p)


def test_flatten_and_sort_marks_ids_out_of_range(dev):
    """Ids the counting sort cannot place (negative, or at / above the expert count -- 4096 without the argument) take no
    part in the order: the valid entries come first, stably sorted, and everything behind them reads -1 in both outputs,
    never uninitialised memory; more experts than the sort takes is an error before anything is enqueued."""
    _, _, ops = _mods()
    g = torch.Generator().manual_seed(5)
    for n_exp, limit in ((None, ops.MAX_EXPERTS), (8, 8)):
        t = torch.randint(0, limit, (3001,), generator=g)
        bad = torch.randperm(3001, generator=g)[:37]
        t[bad[:20]] = limit + torch.arange(20)       # too large
        t[bad[20:]] = -1 - torch.arange(17)          # negative
        for dt in (torch.int32, torch.int64):
            sei, ssi = ops.flatten_and_sort(t.to(dt).to(dev), num_experts=n_exp)
            keep = (t >= 0) & (t < limit)
            want_e, order = torch.sort(t[keep], stable=True)
            want_p = torch.where(keep)[0][order]
            n = int(keep.sum())
            assert torch.equal(sei.cpu()[:n].long(), want_e) and torch.equal(ssi.cpu()[:n], want_p)
            assert bool((sei.cpu()[n:] == -1).all()) and bool((ssi.cpu()[n:] == -1).all()) and sei.numel() - n == 37
    with pytest.raises(RuntimeError, match="bad argument"):
        ops.flatten_and_sort(torch.zeros(16, dtype=torch.int64, device=dev), num_experts=ops.MAX_EXPERTS + 1)


def test_sort_is_deterministic(dev):
    _, router, _ = _mods()
    t = torch.randint(0, 8, (32768,), device=dev, dtype=torch.int32)
    a = router.sort_assignments(t, 8)
    b = router.sort_assignments(t, 8)
    assert all(torch.equal(u, v) for u, v in zip(a, b))


def test_router_backward_matches_autograd(dev, oracle):
    _, router, _ = _mods()
    torch.manual_seed(3)
    T, d, E, k = 300, 64, 8, 2
    x = torch.randn(T, d); wg = torch.randn(E, d) * 0.3
    xo = x.clone().requires_grad_(True); wo = wg.clone().requires_grad_(True)
    _, _, w_o, _ = oracle.router(xo, wo, k)
    g = torch.randn(T, k)
    (w_o * g).sum().backward()
    xg = x.to(dev).requires_grad_(True); wgg = wg.to(dev).requires_grad_(True)
    _, w, _ = router.forward_router(xg, wgg, k)
    (w * g.to(dev)).sum().backward()
    assert torch.allclose(xg.grad.cpu(), xo.grad, atol=1e-5, rtol=1e-4)
    assert torch.allclose(wgg.grad.cpu(), wo.grad, atol=1e-5, rtol=1e-4)


@pytest.mark.parametrize("dtype,T,d,E", [(torch.float32, 1000, 260, 8), (torch.float32, 130, 77, 19), (torch.bfloat16, 4096, 4096, 8),
                                         (torch.bfloat16, 333, 200, 3), (torch.float16, 65, 72, 16)])
def test_router_gradients_from_fp32_dlogits(dev, dtype, T, d, E):
    """dWg = dlogits^T x and dx = dlogits Wg computed by the library from the fp32 dlogits (several token chunks, a
    partial last chunk, expert counts off the register block, widths off the 16-byte vectors): fp32 inputs to 1e-5,
    2-byte inputs to one rounding of the result (the coefficients are never rounded to the activation dtype)."""
    _, router, _ = _mods()
    g = torch.Generator().manual_seed(T + d)
    x = torch.randn(T, d, generator=g).to(dtype)
    wg = (torch.randn(E, d, generator=g) * 0.3).to(dtype)
    dl = torch.randn(T, E, generator=g) * 0.01
    dwg = router.router_weight_grad(x.to(dev), dl.to(dev))
    dx = router.router_input_grad(dl.to(dev), wg.to(dev), dtype)
    ref_w = (dl.double().t() @ x.double()).float()
    ref_x = (dl.double() @ wg.double()).float()
    assert dwg.dtype == dtype and dx.dtype == dtype and dwg.shape == (E, d) and dx.shape == (T, d)
    tol = 1e-5 if dtype == torch.float32 else (2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -10)
    assert float((dwg.float().cpu() - ref_w).abs().max() / ref_w.abs().max()) < tol
    assert float((dx.float().cpu() - ref_x).abs().max() / ref_x.abs().max()) < tol
    assert torch.equal(dwg, router.router_weight_grad(x.to(dev), dl.to(dev)))      # fixed summation order


@pytest.mark.parametrize("case", ["bias", "p2", "bias_p2_k1", "no_norm", "jitter", "uniform"])
def test_forward_router_switches(dev, oracle, case):
    """The router's optional switches (input jitter, bias, p-norm division, uniform assignment) against the oracle's
    restatement of config_utils.py:255-280, forward and backward."""
    moe, router, _ = _mods()
    T, d, E = 300, 256, 8
    k = 1 if case.endswith("k1") else 2
    g = torch.Generator().manual_seed(7)
    x = torch.randn(T, d, generator=g).bfloat16()
    wg = (torch.randn(E, d, generator=g) * 0.2).bfloat16()
    bias = torch.randn(E, generator=g).bfloat16() if "bias" in case else None
    p = 2 if "p2" in case else (None if case == "no_norm" else 1)
    c_w, c_s = torch.randn(T, k, generator=g), torch.randn(T, E, generator=g)
    xd, wd = x.to(dev).requires_grad_(True), wg.to(dev).requires_grad_(True)
    bd = None if bias is None else bias.to(dev).requires_grad_(True)
    noise = None
    if case == "jitter":
        torch.manual_seed(11)
        scores, w, idx = router.forward_router(xd, wd, k, p, bd, moe_jitter_eps=0.1, training=True)
        torch.manual_seed(11)
        noise = router.jitter(xd.detach(), 0.1)
        assert float(noise.min()) >= 0.89 and float(noise.max()) <= 1.11 and float(noise.float().std()) > 0.03
        noise = noise.cpu()
        # not training: no jitter
        s0, _, _ = router.forward_router(xd, wd, k, p, bd, moe_jitter_eps=0.1, training=False)
        assert torch.allclose(s0.cpu(), oracle.router_with_options(x, wg, k, p)[0], atol=2e-6)
    else:
        scores, w, idx = router.forward_router(xd, wd, k, p, bd, uniform_expert_assignment=(case == "uniform"))
    xo, wo = x.float().requires_grad_(True), wg.float().requires_grad_(True)
    bo = None if bias is None else bias.float().requires_grad_(True)
    # the product multiplies in the activation dtype (x * jitter(x), as the reference does)
    xin = xo if noise is None else (x * noise).float() + (xo - xo.detach()) * noise.float()
    rs, rw, ri = oracle.router_with_options(xin, wo, k, p, bo, None, case == "uniform")
    assert idx.dtype == torch.int64 and torch.equal(idx.cpu(), ri)
    if case == "uniform":
        assert torch.equal(idx.cpu().flatten(), torch.arange(T * k) % E)
    assert torch.allclose(scores.cpu(), rs, atol=2e-6) and torch.allclose(w.cpu(), rw, atol=2e-6, rtol=1e-5)
    ((w * c_w.to(dev)).sum() + (scores * c_s.to(dev)).sum()).backward()
    ((rw * c_w).sum() + (rs * c_s).sum()).backward()
    rel = lambda a, b: float((a.float().cpu() - b).abs().max() / b.abs().max())
    assert rel(xd.grad, xo.grad) < 1e-2 and rel(wd.grad, wo.grad) < 1e-2
    if bias is not None:
        assert rel(bd.grad, bo.grad) < 1e-2
