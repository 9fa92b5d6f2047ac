"""moe_sort_by_expert_static -- the entry point that allocates nothing (its per-chunk histograms live in a static
device array of the library) -- gives bit-identical results to moe_sort_by_expert, on two calls in a row, the second
with a smaller input, so stale contents of the shared array from the first call would show."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _run(lib, static, flat, E, block_m=128):
    from moe_distributed_training_amd._lib import ptr, is64, check, stream_ptr, workspace
    dev = flat.device
    R = flat.numel()
    cap = R // block_m + E
    out = {
        "sei": torch.full_like(flat, -7), "ssi": torch.full_like(flat, -7),
        "counts": torch.full((E,), -7, dtype=flat.dtype, device=dev),
        "offsets": torch.full((E,), -7, dtype=flat.dtype, device=dev),
        "pbi": torch.full((cap,), -7, dtype=flat.dtype, device=dev),
        "npad": torch.full((1,), -7, dtype=torch.int32, device=dev),
        "inv": torch.full((R,), -7, dtype=torch.int32, device=dev),
    }
    args = (ptr(flat), is64(flat), R, E, block_m, ptr(out["sei"]), ptr(out["ssi"]), is64(flat), ptr(out["counts"]),
            ptr(out["offsets"]), ptr(out["pbi"]), cap, ptr(out["npad"]), ptr(out["inv"]))
    if static:
        check(lib.moe_sort_by_expert_static(*args, stream_ptr(dev)), "moe_sort_by_expert_static")
    else:
        ws = workspace(lib.moe_sort_workspace_bytes(R, E), dev)
        check(lib.moe_sort_by_expert(*args, ptr(ws), ws.numel(), stream_ptr(dev)), "moe_sort_by_expert")
    torch.cuda.synchronize()
    n = int(out["npad"].item())
    out["pbi"] = out["pbi"][:n]
    return out


@pytest.mark.parametrize("dtype", [torch.int32, torch.int64])
def test_static_sort_matches_workspace_sort_twice(dev, oracle, dtype):
    from moe_distributed_training_amd._lib import lib
    g = torch.Generator().manual_seed(11)
    # first a large ragged batch (many chunks), then a much smaller one with another expert count
    for R, E in ((70001, 8), (1537, 5), (0, 3)):
        flat = torch.randint(0, E, (R,), generator=g).to(dtype).to(dev)
        print(f"static sort case R={R} E={E} {dtype}", flush=True)
        a = _run(lib, True, flat, E)
        b = _run(lib, False, flat, E)
        for key in a:
            assert torch.equal(a[key], b[key]), f"{key} differs (R={R}, E={E})"
        if R:
            # and against the CPU checker, so that both being wrong the same way would show
            sei, ssi = oracle.flatten_and_sort(flat.cpu().long())
            assert torch.equal(a["sei"].cpu().long(), sei) and torch.equal(a["ssi"].cpu().long(), ssi)


def test_static_sort_rejects_sizes_beyond_its_array(dev):
    from moe_distributed_training_amd._lib import lib
    cap = lib.moe_sort_static_max_bytes()
    assert cap == 1 << 20
    E = 4096
    R = 512 * (cap // 4 // E) + 1   # one chunk too many for E = 4096
    assert lib.moe_sort_workspace_bytes(R, E) > cap
    one = torch.zeros(1, dtype=torch.int32, device=dev)
    # rejected on the host before anything is enqueued or dereferenced
    rc = lib.moe_sort_by_expert_static(one.data_ptr(), 0, R, E, 128, one.data_ptr(), one.data_ptr(), 0, None, None, None, 0,
                                       None, None, None)
    assert rc == -3
