"""The C-ABI library loads without a GPU, exports every symbol include/moe_hip.h declares with the signature the
Python binding assumes, and rejects bad arguments before touching the device."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _header_decls():
    hdr = open(os.path.join(ROOT, "include", "moe_hip.h")).read()
    hdr = re.sub(r"/\*.*?\*/", "", hdr, flags=re.S)
    decls = {}
    for m in re.finditer(r"\b(moe_\w+)\s*\(([^;{]*?)\)\s*;", hdr, flags=re.S):
        args = m.group(2).strip()
        codes = ""
        for a in ([] if args == "void" else [a.strip() for a in args.split(",")]):
            codes += "p" if "*" in a else "l" if a.startswith("int64_t") else "z" if a.startswith("size_t") else \
                "f" if a.startswith("float") else "i"
        decls[m.group(1)] = codes
    return decls


def test_library_exports_every_declared_symbol():
    from moe_distributed_training_amd import _lib
    decls = _header_decls()
    assert len(decls) >= 25
    raw = ctypes.CDLL(_lib.LIB_PATH)
    for name in decls:
        assert hasattr(raw, name), f"libmoe_hip.so does not export {name}"
    assert set(decls) == set(_lib._SIGNATURES), set(decls) ^ set(_lib._SIGNATURES)
    for name, codes in decls.items():
        assert _lib._SIGNATURES[name][1] == codes, f"binding of {name} disagrees with the header"
    assert _lib.lib.moe_hip_abi_version() == _lib.ABI_VERSION == int(re.search(r"#define\s+MOE_HIP_ABI_VERSION\s+(\d+)", open(os.path.join(ROOT, "include", "moe_hip.h")).read()).group(1))


def test_bad_arguments_are_rejected_on_the_host():
    from moe_distributed_training_amd._lib import lib
    assert lib.moe_hip_strerror(0) == b"ok" and lib.moe_hip_strerror(-3) == b"workspace too small"
    # null pointers / inconsistent sizes: status -1 and nothing is launched
    assert lib.moe_router_topk(None, None, None, None, 4, 8, 2, 1, None) == -1
    assert lib.moe_router_topk(1, 1, 1, 1, 4, 8, 9, 1, None) == -1          # k > E
    assert lib.moe_scatter2scatter(None, 1, 1, None, 1, 1, 1, None, 0, 0, 0, None, 0, 0, 0, 0, 0.0, None, 1, 1, None, 0,
                                   None, 0, 4, 8, 16, 16, 1, 0, 0, 0, None, 0, None) == -1
    assert lib.moe_group_bwd_ab(None, 1, 1, None, 1, 1, None, 1, 1, 1, None, 1, 1, 1, 4, 1.0, None, 1, 1, 1, None, 1, 1, 1,
                                None, 0, 2, 8, 16, 16, 0, None, 0, None) == -1
    assert lib.moe_mlp_fwd(None, 1, None, None, None, None, None, 0, 0.0, None, None, None, None, 1, None, 0, None, 0, 2,
                           8, 64, 64, 1, 0, 0, None, None, 0, None) == -1
    assert lib.moe_sort_workspace_bytes(8192, 8) >= 4 * 8 * 4
    # the sort's status path: more experts than the counting sort takes (4096) is refused before anything is enqueued
    # (16: non-null stand-ins that are never dereferenced); this is what flatten_and_sort's RuntimeError comes from
    assert lib.moe_sort_by_expert(16, 0, 8, 4097, 128, 16, 16, 0, None, None, None, 0, None, None, 16, 1 << 20, None) == -1
    assert lib.moe_sort_by_expert_static(16, 0, 8, 4097, 128, 16, 16, 0, None, None, None, 0, None, None, None) == -1
    assert lib.moe_mlp_workspace_bytes(8192, 8, 4096, 14336, 16) > 0


def test_cpu_tensors_fail_loudly():
    import pytest
    import torch
    import moe_distributed_training_amd as moe
    with pytest.raises(RuntimeError, match="GPU only"):
        moe.flatten_and_sort(torch.tensor([1, 0, 1]))
    with pytest.raises(RuntimeError, match="GPU only"):
        moe.forward_router(torch.randn(4, 8), torch.randn(2, 8), 1)


def test_size_limits_are_checked_before_anything_is_enqueued():
    """The fused entry points address gathered activation rows and one expert's matrix with 32-bit byte offsets; sizes
    beyond that are refused on the host with MOE_ERR_UNSUPPORTED (status codes only: nothing is dereferenced), while the
    number of rows alone never is (grouped tiles are addressed from their own first row)."""
    from moe_distributed_training_amd._lib import lib
    one = 16   # non-null, 16-byte aligned stand-ins: rejected before any use

    def fwd(R, d, f, fan_out):
        return lib.moe_mlp_fwd(one, d, one, one, one, None, None, 0, 0.0, one, one, one, one, d, one, 0, one, 0, 8,
                               R, d, f, fan_out, 0, 0, None, None, 0, None)
    # a gathered x of 4 GiB or more: T * ldx * 2 bytes
    assert fwd(2 * 600000, 4096, 14336, 2) == -2
    # one expert's matrix of 4 GiB or more
    assert fwd(8192, 65536, 32768, 2) == -2
    # many rows alone are fine: the call gets as far as the workspace check (status -3), i.e. past the size checks
    assert fwd(2 * 200000, 4096, 14336, 2) == -3
    assert lib.moe_mlp_workspace_bytes(400000, 8, 4096, 14336, 16) > 0


def test_fused_layer_rank_limit_is_checked_on_the_host():
    """The fused layer takes an adapter as up to eight chunks of 16 rank columns: rank 128 gets past the shape checks (as
    far as the workspace check), rank 129 is refused with MOE_ERR_UNSUPPORTED before anything is enqueued; the sizes of
    the saved interims and of the workspace grow with the number of chunks."""
    import ctypes
    from moe_distributed_training_amd._lib import lib
    one = 16   # non-null, 16-byte aligned stand-ins: never dereferenced
    lora = (ctypes.c_void_p * 6)(*([one] * 6))
    strides = (ctypes.c_int64 * 18)(*([1] * 18))

    def fwd(rank):
        return lib.moe_mlp_fwd(one, 4096, one, one, one, lora, strides, rank, 1.0, one, one, one, one, 4096, one, 0, one, 0,
                               8, 8192, 4096, 14336, 2, 0, 0, one, None, 0, None)
    assert fwd(128) == -3 and fwd(72) == -3 and fwd(16) == -3
    assert fwd(129) == -2 and fwd(256) == -2
    saved = [lib.moe_mlp_saved_bytes(8192, r) for r in (16, 17, 32, 33, 128)]
    assert saved[1] == saved[2] == 2 * saved[0] and saved[3] == 3 * saved[0] and saved[4] == 8 * saved[0]
    ws = [lib.moe_mlp_workspace_bytes(8192, 8, 4096, 14336, r) for r in (0, 16, 32, 64, 128)]
    assert ws == sorted(ws) and len(set(ws)) == 5
