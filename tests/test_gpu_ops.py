"""Operator-level parity of the HIP path (called through the C ABI by the Python mirror of the reference's plugin
surface) against the CPU oracle.  Tolerances: fp32 1e-5 relative to the output scale; bf16 max rel err 1e-2
(fp32 accumulate), the bar the path's specification states."""
import pytest
import torch

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 2e-5, torch.bfloat16: 1e-2, torch.float16: 2e-3}


from _metrics import rel, rel_per_expert


def check_expert_grads(got, want, tol, what=""):
    """Gradients whose first dimension is the expert: every expert's slice against its own scale (a one-row group must
    meet the bound on its own), max and RMS."""
    mx, rms = rel_per_expert(got, want, with_rms=True)
    assert mx < tol and rms < tol, f"{what}: per-expert max rel err {mx:.4g}, rms rel err {rms:.4g}"


def _ops():
    from moe_distributed_training_amd.scattermoe_utils.kernels import ops
    return ops


def _routing(oracle, T, E, k, seed=0, skew=False):
    g = torch.Generator().manual_seed(seed)
    logits = torch.randn(T, E, generator=g)
    if skew:
        logits[:, 0] += 3.0
        logits[:, -1] -= 6.0
    idx = torch.topk(logits, k, dim=-1).indices
    sei, ssi = oracle.flatten_and_sort(idx)
    eo = torch.bincount(sei, minlength=E).cumsum(0)
    return idx, sei, ssi, eo


CASES = [
    # dtype, T, E, k, K, N, r
    (torch.float32, 10, 2, 1, 128, 16, 16),      # the reference's own test shape
    (torch.float32, 300, 4, 2, 100, 36, 4),
    (torch.float16, 300, 4, 2, 64, 40, 8),       # fp16 on the matrix cores
    (torch.bfloat16, 300, 4, 2, 72, 40, 8),      # K not a multiple of 64: a partial last K tile, masked loads
    (torch.float16, 700, 8, 2, 200, 264, 16),    # fp16, three whole K tiles and a partial one, N tail, adapters
    (torch.bfloat16, 500, 4, 2, 1096, 512, 24),  # split K with a partial last tile, two adapter slabs
    (torch.bfloat16, 300, 4, 2, 40, 64, 8),      # K below one K tile -> generic kernels
    (torch.bfloat16, 1000, 8, 2, 256, 512, 16),
    (torch.bfloat16, 1500, 8, 2, 512, 264, 16),  # N tail inside a 256-wide tile
    (torch.bfloat16, 700, 3, 2, 1024, 256, 4),   # rank < 16 zero padded
    (torch.bfloat16, 2500, 8, 2, 128, 1280, 16),
    (torch.bfloat16, 600, 4, 2, 2048, 512, 16),  # few tiles, deep K: every tile is cut 4 ways along K
    (torch.bfloat16, 400, 4, 2, 256, 512, 32),   # rank above 16: the adapter enters as two 16-wide slabs
    (torch.bfloat16, 400, 4, 2, 256, 512, 64),   # four slabs in two MFMA steps
    (torch.bfloat16, 400, 4, 2, 256, 512, 40),   # three slabs, the last one partly filled
    (torch.bfloat16, 400, 4, 2, 256, 512, 96),   # a rank above 64: six slabs at a fixed stride, two per step in a loop
    (torch.float16, 400, 4, 2, 264, 256, 136),   # nine slabs (the last half empty), fp16, and a partial last K tile
    (torch.bfloat16, 1200, 96, 4, 256, 512, 16), # more than 64 experts (serial group lookup), top-4, every tile ragged
    (torch.bfloat16, 500, 4, 2, 64, 512, 16),    # a single K tile: the adapter slabs' LDS image is requested before the loop
    (torch.bfloat16, 500, 4, 2, 192, 300, 16),   # three K tiles: ... by the first trip through the loop
]


@pytest.mark.parametrize("layout", ["k_contiguous", "n_contiguous"])
@pytest.mark.parametrize("dtype,T,E,k,K,N,r", CASES)
def test_scatter2scatter_all_row_mappings(dev, oracle, layout, dtype, T, E, k, K, N, r):
    ops = _ops()
    torch.manual_seed(1)
    _, sei, ssi, eo = _routing(oracle, T, E, k, skew=True)
    W = (torch.randn(E, N, K) * 0.05).to(dtype).permute(0, 2, 1) if layout == "k_contiguous" else (torch.randn(E, K, N) * 0.05).to(dtype)
    A = (torch.randn(E, K, r) * 0.05).to(dtype)
    B = (torch.randn(E, r, N) * 0.05).to(dtype)
    seid, ssid = sei.to(dev), ssi.int().to(dev)            # mixed index widths on purpose
    # which kernel a shape takes: 2-byte types with K >= 64 and K, N multiples of 8 run on the matrix cores (one grouped
    # GEMM launch per call), everything else on the generic kernels
    from moe_distributed_training_amd._lib import lib
    on_matrix_cores = dtype != torch.float32 and K >= 64 and K % 8 == 0 and N % 8 == 0
    for xg, yg in [(False, True), (False, False), (True, False), (True, True)]:
        X = torch.randn(T * k if xg else T, K).to(dtype)
        kk = 1 if xg else k
        s_in = ssi if not xg else ssi
        n0 = lib.moe_gemm_debug_launch_count()
        y = ops.scatter2scatter_lora(X.to(dev), W.to(dev), A.to(dev), B.to(dev), 32.0, seid, ssid, kk, None, xg, yg)
        assert lib.moe_gemm_debug_launch_count() - n0 == int(on_matrix_cores)
        yo = oracle.scatter2scatter_lora(X, W, A, B, 32.0, sei, s_in, kk, None, xg, yg)
        assert rel(y, yo) < TOL[dtype], (xg, yg)
        y2 = ops.scatter2scatter(X.to(dev), W.to(dev), seid, ssid, kk, None, xg, yg)
        assert lib.moe_gemm_debug_launch_count() - n0 == 2 * int(on_matrix_cores)
        yo2 = oracle.scatter2scatter_lora(X, W, None, None, 0.0, sei, s_in, kk, None, xg, yg)
        assert rel(y2, yo2) < TOL[dtype], (xg, yg)


@pytest.mark.parametrize("T,E,k,K,N,layout", [(600, 4, 2, 2048, 512, "k_contiguous"), (600, 4, 2, 2048, 512, "n_contiguous"),
                                              (4096, 8, 2, 14336, 4096, "n_contiguous")])
def test_k_split_exchange_is_stable_over_many_launches(dev, oracle, T, E, k, K, N, layout):
    """Tiles of the last, partial round are cut 2 or 4 ways along K; the parts exchange fp32 partials through memory
    that crosses the XCDs' separate L2 caches and a counter.  A stale read there would be a silent, intermittent wrong
    sum: 2000 launches of the same problem (a small one where every tile is split, and the h W2 product at the Mixtral
    shape) must all be bitwise equal to the first, which itself meets the oracle; stops at the first mismatch."""
    ops = _ops()
    torch.manual_seed(21)
    _, sei, ssi, eo = _routing(oracle, T, E, k, seed=21)
    L = T * k
    g = torch.Generator(device=dev).manual_seed(22)
    X = torch.randn(L, K, generator=g, device=dev).bfloat16()
    W = (torch.randn(E, N, K, generator=g, device=dev) * 0.05).bfloat16().permute(0, 2, 1) if layout == "k_contiguous" else \
        (torch.randn(E, K, N, generator=g, device=dev) * 0.05).bfloat16()
    seid, ssid = sei.to(dev), ssi.int().to(dev)
    plan, _ = _plan(dev, torch.bincount(sei, minlength=E).tolist(), K, N, False)
    assert (plan[:, 0] == 1).any() and (plan[plan[:, 0] == 1][:, 6] > 1).any(), "the case must have K-split tiles"
    first = ops.scatter2scatter(X, W, seid, ssid, 1, None, True, True)
    if L * K * N <= 2e10:
        ref = oracle.scatter2scatter_lora(X.float().cpu(), W.float().cpu(), None, None, 0.0, sei, ssi, 1, None, True, True)
        assert rel(first, ref) < 1e-2
    out = torch.empty_like(first)
    bad = torch.zeros((), dtype=torch.int32, device=dev)
    launches, check_every = 2000, 100
    for i in range(launches):
        ops.scatter2scatter(X, W, seid, ssid, 1, None, True, True, out=out)
        bad += (out != first).any().int()
        if (i + 1) % check_every == 0:
            assert int(bad.item()) == 0, f"a launch among {i + 2 - check_every}..{i + 1} differs from the first"


@pytest.mark.slow
@pytest.mark.parametrize("case", ["grouped_out_above_2GiB", "scattered_out_above_2GiB", "grouped_in_above_4GiB"])
def test_scatter2scatter_beyond_32_bit_spans(dev, case):
    """Tensors larger than a 32-bit byte offset reaches: a grouped output above 2 GiB (tiles addressed from their own
    first row), a scattered output above 2 GiB (64-bit row addresses) and a grouped input above 4 GiB.  Rows from the
    first tile, the last tile and around the 2 / 4 GiB marks against per-row fp32 products."""
    ops = _ops()
    g = torch.Generator(device=dev).manual_seed(31)
    E = 4
    if case == "grouped_in_above_4GiB":
        R, K, N = 140000, 16384, 64
    else:
        R, K, N = 70000, 64, 16384
    counts = [R // 2 - 777, 0, R // 4 + 500, R - (R // 2 - 777) - (R // 4 + 500)]
    eo = torch.tensor(counts).cumsum(0)
    sei = torch.repeat_interleave(torch.arange(E), torch.tensor(counts)).to(dev)
    scattered = case == "scattered_out_above_2GiB"
    ssi = (torch.randperm(R, generator=torch.Generator().manual_seed(32)) if scattered else torch.arange(R)).to(dev)
    X = torch.randn(R, K, generator=g, device=dev).bfloat16()
    W = (torch.randn(E, K, N, generator=g, device=dev) * 0.05).bfloat16()
    assert max(X.numel(), R * N) * 2 > (1 << 31)
    y = ops.scatter2scatter(X, W, sei, ssi, 1, None, True, not scattered)
    torch.cuda.synchronize()
    mark = (1 << 31) // (2 * N) if case != "grouped_in_above_4GiB" else (1 << 32) // (2 * K)
    rows = sorted(set(list(range(0, 300)) + list(range(R - 300, R)) + list(range(mark - 300, mark + 300)) +
                      [int(v) for v in eo.tolist() if 0 < v < R] + [int(v) - 1 for v in eo.tolist() if v > 0]))
    m = torch.tensor(rows, device=dev)
    e_of = sei[m]
    ref = torch.bmm(X[m].float().unsqueeze(1), W.float()[e_of]).squeeze(1)
    got = y[ssi[m] if scattered else m].float()
    assert float((got - ref).abs().max() / ref.abs().max()) < 1e-2
    if scattered:   # every output row was written exactly once: a permutation of the grouped result
        yg = ops.scatter2scatter(X, W, sei, ssi, 1, None, True, True)
        assert torch.equal(y[ssi], yg)


def test_scatter2scatter_out_argument_and_empty(dev, oracle):
    ops = _ops()
    torch.manual_seed(2)
    T, E, k, K, N = 64, 4, 2, 64, 64
    _, sei, ssi, eo = _routing(oracle, T, E, k)
    X = torch.randn(T, K).bfloat16(); W = (torch.randn(E, K, N) * 0.1).bfloat16()
    out = torch.zeros(T * k, N, dtype=torch.bfloat16, device=dev)
    y = ops.scatter2scatter(X.to(dev), W.to(dev), sei.to(dev), ssi.to(dev), k, None, False, True, out=out)
    assert y.data_ptr() == out.data_ptr()
    assert rel(out, oracle.scatter2scatter_lora(X, W, None, None, 0, sei, ssi, k, None, False, True)) < 1e-2
    with pytest.raises(AssertionError):
        ops.scatter2scatter(X.to(dev), W.to(dev), sei.to(dev), ssi.to(dev), 1, None, False, True)   # rows(X)*k mismatch
    e = torch.empty(0, dtype=torch.int64, device=dev)
    y0 = ops.scatter2scatter(X[:0].to(dev), W.to(dev), e, e, k)
    assert y0.shape == (0, N)


@pytest.mark.parametrize("counts,K,N", [
    ([301, 0, 77, 1, 513], 256, 512),        # ragged groups: empty, one row, not a multiple of the 64-row step
    ([64, 128, 192], 512, 256),              # whole steps only
    ([130, 5, 0, 260], 264, 136),            # K and N not multiples of the 256 tile: edge columns are masked
    ([1000, 3000], 768, 2304),               # several panels of n tiles, long contraction
])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_group_bwd_w_matrix_cores(dev, oracle, counts, K, N, dtype):
    """bf16 / fp16 DW[e] = X_e^T DY_e (scattermoe group_bwd_W, full fine-tuning) against the fp32 per-expert matmul; rows of
    the next group must not leak into a group's last, partial contraction step, an empty group gives zeros."""
    ops = _ops()
    torch.manual_seed(11)
    E = len(counts)
    eo = torch.tensor(counts).cumsum(0)
    R = int(eo[-1])
    X = torch.randn(R, K).to(dtype); DY = (torch.randn(R, N) * 0.25).to(dtype)
    ref = oracle.group_bwd_W(DY, X, eo, E)
    for offs in (eo.to(dev), eo.int().to(dev)):
        dW = ops.group_bwd_W(DY.to(dev), X.to(dev), offs, E)
        assert dW.shape == (E, K, N) and dW.dtype == dtype
        for e in range(E):
            if counts[e] == 0:
                assert float(dW[e].abs().max()) == 0.0
            else:
                assert rel(dW[e], ref[e]) < TOL[dtype]
    if dtype != torch.bfloat16:
        return
    # row-strided operands (column slices of wider buffers) take the same kernel
    Xw = torch.randn(R, K + 64).bfloat16().to(dev); DYw = torch.randn(R, N + 8).bfloat16().to(dev)
    dW = ops.group_bwd_W(DYw[:, 8:], Xw[:, 64:], eo.to(dev), E)
    check_expert_grads(dW, oracle.group_bwd_W(DYw[:, 8:].cpu(), Xw[:, 64:].cpu(), eo, E), TOL[torch.bfloat16], "dW strided")


def test_group_bwd_w_mixtral_shape(dev, oracle):
    """Full size of one Mixtral projection (R=8192 rows in 8 ragged groups, K=4096, N=14336): every expert's matrix
    against the fp32 per-expert matmul on the host."""
    ops = _ops()
    g = torch.Generator(device=dev).manual_seed(5)
    counts = [1100, 950, 1030, 1200, 900, 1012, 1000, 1000]
    eo = torch.tensor(counts).cumsum(0)
    X = torch.randn(8192, 4096, generator=g, device=dev).bfloat16()
    DY = torch.randn(8192, 14336, generator=g, device=dev).bfloat16()
    dW = ops.group_bwd_W(DY, X, eo.to(dev), 8)
    torch.cuda.synchronize()
    torch.set_num_threads(16)
    Xc, DYc = X.float().cpu(), DY.float().cpu()
    start = 0
    for e, c in enumerate(counts):
        ref = Xc[start:start + c].T @ DYc[start:start + c]
        assert rel(dW[e], ref) < TOL[torch.bfloat16], f"expert {e}"
        start += c


@pytest.mark.parametrize("dtype,K,N,r", [(torch.float32, 150, 140, 4), (torch.bfloat16, 256, 512, 16), (torch.bfloat16, 256, 512, 64),
                                         (torch.bfloat16, 4096, 1024, 16), (torch.bfloat16, 96, 160, 8),
                                         (torch.float16, 130, 70, 16), (torch.float16, 256, 512, 16), (torch.float16, 512, 288, 48)])
def test_group_bwd_ab_full_reduction(dev, oracle, dtype, K, N, r):
    """K and N above 128 on purpose: every N tile must contribute to dA and every K tile to dB."""
    ops = _ops()
    torch.manual_seed(3)
    E = 5
    counts = torch.tensor([301, 0, 77, 1, 513])
    eo = counts.cumsum(0)
    R = int(eo[-1])
    X = torch.randn(R, K).to(dtype); DY = torch.randn(R, N).to(dtype)
    A = (torch.randn(E, K, r) * 0.1).to(dtype); B = (torch.randn(E, r, N) * 0.1).to(dtype)
    dA, dB = ops.group_bwd_AB(DY.to(dev), X.to(dev), A.to(dev), B.to(dev), 2.0, eo.to(dev), E)
    dAo, dBo = oracle.group_bwd_AB(DY, X, A, B, 2.0, eo, E)
    assert dA.shape == (E, K, r) and dB.shape == (E, r, N) and dA.dtype == dtype
    check_expert_grads(dA, dAo, TOL[dtype] * 1.5, "dA"); check_expert_grads(dB, dBo, TOL[dtype] * 1.5, "dB")
    assert float(dA[1].abs().max()) == 0.0 and float(dB[1].abs().max()) == 0.0
    dW = ops.group_bwd_W(DY.to(dev), X.to(dev), eo.int().to(dev), E)
    check_expert_grads(dW, oracle.group_bwd_W(DY, X, eo, E), TOL[dtype] * 1.5, "dW")
    # strided adapter views (the w2 arrangement of the reference: both factors permuted)
    A2 = (torch.randn(E, r, K) * 0.1).to(dtype).permute(0, 2, 1); B2 = (torch.randn(E, N, r) * 0.1).to(dtype).permute(0, 2, 1)
    dA2, dB2 = ops.group_bwd_AB(DY.to(dev), X.to(dev), A2.to(dev), B2.to(dev), 0.5, eo.to(dev), E)
    dAo2, dBo2 = oracle.group_bwd_AB(DY, X, A2, B2, 0.5, eo, E)
    check_expert_grads(dA2, dAo2, TOL[dtype] * 1.5, "dA strided"); check_expert_grads(dB2, dBo2, TOL[dtype] * 1.5, "dB strided")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_group_and_combine(dev, oracle, dtype):
    ops = _ops()
    torch.manual_seed(4)
    T, E, k, N = 257, 6, 2, 200
    _, sei, ssi, eo = _routing(oracle, T, E, k)
    src = torch.randn(T, N).to(dtype); coeff = torch.rand(T * k).to(dtype)
    g = ops.group(src.to(dev), ssi.to(dev), coeff=coeff.to(dev), fan_out=k)
    assert rel(g, oracle.group(src.float(), ssi, coeff.float(), k)) < TOL[dtype]
    g1 = ops.group(src.to(dev), ssi.to(dev), fan_out=k)
    assert torch.equal(g1.cpu(), src[ssi // k])
    yg = torch.randn(T * k, N).to(dtype); w = torch.rand(T, k)
    inv = torch.empty(T * k, dtype=torch.int32); inv[ssi] = torch.arange(T * k, dtype=torch.int32)
    out = ops.combine(yg.to(dev), w.to(dev), inv=inv.to(dev))
    assert rel(out, oracle.combine(yg.float(), ssi, w, T, k)) < TOL[dtype]
    dout = torch.randn(T, N).to(dtype)
    dg = ops.combine_dgates(yg.to(dev), dout.to(dev), k, torch.float32, inv=inv.to(dev))
    ref = (yg.float()[inv.long()].view(T, k, N) * dout.float()[:, None, :]).sum(-1)
    assert rel(dg, ref) < TOL[dtype]


def _run_parallel_linear(dev, oracle, dtype, T, E, k, K, N, r, gates, gin, gout, lora=True, seed=5):
    import moe_distributed_training_amd as moe
    torch.manual_seed(seed)
    _, sei, ssi, eo = _routing(oracle, T, E, k, seed)
    L = T * k
    X = torch.randn(L if gin else T, K).to(dtype)
    W = (torch.randn(E, N, K) * 0.05).to(dtype).permute(0, 2, 1)
    A = (torch.randn(E, K, r) * 0.05).to(dtype); B = (torch.randn(E, r, N) * 0.05).to(dtype)
    G = torch.rand(T, k).to(dtype) if gates else None
    kk = 1 if gin else k
    rows_out = T if gates else L
    dY = torch.randn(rows_out, N).to(dtype)
    f32 = lambda t: None if t is None else t.detach().float().clone().requires_grad_(True)
    Xo, Wo, Ao, Bo, Go = f32(X), f32(W), f32(A), f32(B), f32(G)
    yo = oracle.parallel_linear_lora(Xo, Wo, Ao if lora else None, Bo if lora else None, r, 32.0, kk, sei, ssi, None, eo,
                                     Go, gin, gout)
    yo.backward(dY.float())
    d = lambda t: None if t is None else t.detach().to(dev).requires_grad_(True)
    Xd, Wd, Ad, Bd, Gd = d(X), d(W), d(A), d(B), d(G)
    pb, eod = moe.padded_block_indices(sei.to(dev), E)
    if lora:
        y = moe.parallel_linear_lora(Xd, Wd, Ad, Bd, r, 32.0, kk, sei.to(dev), ssi.to(dev), pb, eod, Gd, gin, gout)
    else:
        y = moe.parallel_linear(Xd, Wd, kk, sei.to(dev), ssi.to(dev), pb, eod, Gd, gin, gout)
    y.backward(dY.to(dev))
    tol = TOL[dtype] * 1.5
    assert rel(y, yo) < tol
    assert rel(Xd.grad, Xo.grad) < tol
    if lora:
        check_expert_grads(Ad.grad, Ao.grad, tol, "dA"); check_expert_grads(Bd.grad, Bo.grad, tol, "dB")
        assert Wd.grad is None                                   # base weights are frozen on the LoRA path
    else:
        check_expert_grads(Wd.grad, Wo.grad, tol, "dW")
    if gates:
        assert rel(Gd.grad, Go.grad) < tol


@pytest.mark.parametrize("dtype,K,N,r", [(torch.float32, 128, 16, 16), (torch.bfloat16, 256, 384, 16), (torch.bfloat16, 200, 136, 16),
                                         (torch.bfloat16, 256, 384, 32), (torch.float16, 256, 384, 16)])
@pytest.mark.parametrize("gates,gin,gout", [(False, False, True), (False, True, False), (True, False, False), (False, False, False), (False, True, True)])
def test_parallel_linear_lora_autograd(dev, oracle, dtype, K, N, r, gates, gin, gout):
    _run_parallel_linear(dev, oracle, dtype, 333, 4, 2, K, N, r, gates, gin, gout)


@pytest.mark.parametrize("gates,gin,gout", [(False, False, True), (True, False, False), (False, True, False)])
def test_parallel_linear_plain_autograd_with_dw(dev, oracle, gates, gin, gout):
    _run_parallel_linear(dev, oracle, torch.bfloat16, 333, 4, 2, 256, 128, 16, gates, gin, gout, lora=False)
    _run_parallel_linear(dev, oracle, torch.float32, 100, 3, 2, 50, 30, 16, gates, gin, gout, lora=False)


def test_reference_test_case(dev, oracle):
    """tests/test_scattermoe.py of the reference: E=2, 128 -> 16, r=16, alpha=32, 10 rows, k=1, scattered in, grouped
    out, loss = out.norm(); output and dB compared at atol=1e-2 (here also dA and dX)."""
    import moe_distributed_training_amd as moe
    torch.manual_seed(42)
    X = torch.randn(10, 128)
    sei = torch.tensor([0, 0, 0, 0, 1, 1, 1, 1, 1, 1]); ssi = torch.tensor([4, 6, 8, 9, 0, 1, 2, 3, 5, 7])
    lin = [torch.nn.Linear(128, 16, bias=False) for _ in range(2)]
    W = torch.stack([l.weight.detach().T for l in lin])
    A = torch.randn(2, 128, 16) * 0.02; B = torch.randn(2, 16, 16) * 0.02
    Ao, Bo, Xo = A.clone().requires_grad_(True), B.clone().requires_grad_(True), X.clone().requires_grad_(True)
    out = torch.cat([Xo[ssi[sei == i]] @ (W[i] + 2.0 * Ao[i] @ Bo[i]) for i in range(2)])     # ExpertModel loop + LoRA
    out.norm().backward()
    Xd, Ad, Bd = X.to(dev).requires_grad_(True), A.to(dev).requires_grad_(True), B.to(dev).requires_grad_(True)
    pb, eo = moe.padded_block_indices(sei.to(dev), 2)
    out2 = moe.parallel_linear_lora(Xd, W.to(dev), Ad, Bd, 16, 32, 1, sei.to(dev), ssi.to(dev), pb, eo,
                                    grouped_in=False, grouped_out=True)
    out2.norm().backward()
    assert torch.allclose(out, out2.cpu(), atol=1e-2)
    assert torch.allclose(Bo.grad, Bd.grad.cpu(), atol=1e-2) and torch.allclose(Ao.grad, Ad.grad.cpu(), atol=1e-2)
    assert torch.allclose(out, out2.cpu(), atol=1e-5) and torch.allclose(Bo.grad, Bd.grad.cpu(), atol=1e-5)
    assert torch.allclose(Xo.grad, Xd.grad.cpu(), atol=1e-5)


def test_parallel_experts_module(dev, oracle):
    import moe_distributed_training_amd as moe
    torch.manual_seed(6)
    T, E, k, K, N = 128, 4, 2, 64, 128
    m = moe.ParallelExperts(E, K, N, device=dev, dtype=torch.bfloat16)
    assert m.weight.shape == (E, N, K)
    _, sei, ssi, eo = _routing(oracle, T, E, k)
    X = torch.randn(T, K).bfloat16()
    y = m(X.to(dev), k, sei.to(dev), ssi.to(dev), None, eo.to(dev), grouped_out=True)
    yo = oracle.scatter2scatter_lora(X, m.weight.detach().cpu().permute(0, 2, 1), None, None, 0, sei, ssi, k, None, False, True)
    assert rel(y, yo) < 1e-2


def _plan(dev, counts, K, N, pair, nseg=1):
    from moe_distributed_training_amd._lib import lib, check, ptr, stream_ptr
    E = len(counts)
    R = int(sum(counts))
    eo = torch.tensor(counts, dtype=torch.int64).cumsum(0).to(dev)
    blocks = lib.moe_gemm_debug_plan_blocks(R, E, N, int(pair))
    out = torch.full((blocks, 9), -7, dtype=torch.int32, device=dev)
    check(lib.moe_gemm_debug_plan(ptr(eo), 1, E, R, K, N, int(pair), nseg, ptr(out), stream_ptr(dev)), "moe_gemm_debug_plan")
    return out.cpu().numpy(), blocks


@pytest.mark.parametrize("case", range(24))
def test_grouped_gemm_tile_plan_covers_every_tile_once(dev, case):
    """The work items the grouped GEMM's workgroups decode for themselves, for seeded group sizes (even, ragged, skewed,
    empty groups, few and many rounds of tiles, both tile widths): every output tile appears exactly once, either whole
    or as K parts 0..n-1 with consecutive exchange slots and one counter, and slots and counters are unique and within
    the exchange area's size."""
    import random
    rng = random.Random(500 + case)
    E = rng.choice([1, 2, 3, 8, 8, 8, 17, 64])
    kind = rng.choice(["even", "ragged", "skewed", "tiny"])
    R = rng.choice([300, 2000, 8192, 8192, 20000])
    if kind == "even":
        counts = [R // E] * E
    elif kind == "ragged":
        counts = [max(0, int(R / E * (1 + 0.15 * rng.uniform(-1, 1)))) for _ in range(E)]
    elif kind == "skewed":
        w = [1.0 / (i + 1) ** 1.2 for i in range(E)]
        counts = [int(R * x / sum(w)) for x in w]
        rng.shuffle(counts)
    else:
        counts = [rng.choice([0, 0, 1, 5, 40, 130, 257]) for _ in range(E)]
    if sum(counts) == 0:
        counts[0] = 3
    K = rng.choice([512, 4096, 14336])
    N = rng.choice([256, 4096, 14336, 1000])
    pair = rng.choice([False, True])
    nseg = 1 if pair else rng.choice([1, 2])
    plan, blocks = _plan(dev, counts, K, N, pair, nseg)
    ncu = torch.cuda.get_device_properties(dev).multi_processor_count // 8 * 8
    bn = 128 if pair else 256
    ntn = (N + bn - 1) // bn
    expected = {}
    start = 0
    for e, c in enumerate(counts):
        for ntile in range(ntn):
            for r0 in range(start, start + c, 256):
                expected[(e, ntile, r0)] = min(r0 + 256, start + c)
        start += c
    tiles_ub = (sum(counts) // 256 + E) * ((N + 255) // 256)
    slots_cap = min(4 * tiles_ub, ncu)
    seen = {}
    for b in range(blocks):
        valid, e, ntile, r0, r1, part, nparts, slot, counter = (int(v) for v in plan[b])
        assert valid in (0, 1), f"block {b} wrote nothing"
        if not valid:
            continue
        key = (e, ntile, r0)
        assert key in expected and expected[key] == r1, (case, key, r1)
        assert nparts in (1, 2, 4) and 0 <= part < nparts
        seen.setdefault(key, []).append((part, nparts, slot, counter))
    assert set(seen) == set(expected), (case, len(seen), len(expected))
    used_slots, used_counters = set(), set()
    for key, items in seen.items():
        nparts = items[0][1]
        assert len(items) == nparts and sorted(i[0] for i in items) == list(range(nparts)), (case, key, items)
        if nparts > 1:
            assert max_split_ok(pair), "the pair kernel never splits"
            first = min(i[2] for i in items)
            assert all(i[2] == first + i[0] and i[1] == nparts and i[3] == items[0][3] for i in items), (case, key, items)
            for i in items:
                assert 0 <= i[2] < slots_cap and i[2] not in used_slots
                used_slots.add(i[2])
            assert 0 <= items[0][3] < ncu and items[0][3] not in used_counters
            used_counters.add(items[0][3])


def max_split_ok(pair):
    return not pair

