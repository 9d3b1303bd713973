"""The split decode attention through the entry point that allocates nothing
(`llms_attention_decode_noalloc`: its partial results go through a fixed array the library owns),
called through ctypes and checked against the entry point that takes a caller's workspace: two
calls in a row on the same GPU, the second with a smaller input, so that what the first call left
in the array lies under and beside what the second one uses."""

import ctypes

import pytest
import torch

from kernel_helpers import attention_reference, make_paged

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
c_void_p, c_int, c_float = ctypes.c_void_p, ctypes.c_int, ctypes.c_float


def rnd(*shape, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed))


def decode_case(nh, nkv, d, bs, lens, seed):
    """Every request brings its last token; returns the kernel's operands on the device and the plain result."""
    dtype = torch.bfloat16
    qs = [rnd(s, nh, d, seed=seed + 3 * b).to(dtype) for b, s in enumerate(lens)]
    ks = [rnd(s, nkv, d, seed=seed + 3 * b + 1).to(dtype) for b, s in enumerate(lens)]
    vs = [rnd(s, nkv, d, seed=seed + 3 * b + 2).to(dtype) for b, s in enumerate(lens)]
    k_pool, v_pool, tables = make_paged(ks, vs, bs, dtype, seed=seed)
    q = torch.cat([qs[b][-1:].reshape(1, nh * d) for b in range(len(lens))]).contiguous().to(DEV)
    ref = torch.cat([attention_reference(qs[b], ks[b], vs[b], [lens[b] - 1]) for b in range(len(lens))])
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)  # noqa: E731
    return dict(q=q, k_pool=k_pool.to(DEV), v_pool=v_pool.to(DEV), tables=tables.to(DEV),
                cu=i32(list(range(len(lens) + 1))), ctx=i32(lens), n=len(lens), nh=nh, nkv=nkv, d=d, bs=bs), ref


def new_out(case):
    return torch.full((case["n"], case["nh"] * case["d"]), float("nan"), dtype=torch.bfloat16, device=DEV)


def call_noalloc(lib, case, num_splits, waves, out):
    n, nh, d = case["n"], case["nh"], case["d"]
    ptr = lambda t: c_void_p(t.data_ptr())  # noqa: E731
    stream = c_void_p(torch.cuda.current_stream().cuda_stream)
    status = lib.llms_attention_decode_noalloc(
        ptr(out), c_int(out.stride(0)), ptr(case["q"]), c_int(case["q"].stride(0)), ptr(case["k_pool"]),
        ptr(case["v_pool"]), ptr(case["tables"]), c_void_p(0), c_int(case["tables"].shape[1]), ptr(case["cu"]),
        ptr(case["ctx"]), c_int(0), c_int(n), c_int(0), c_int(n), c_int(nh), c_int(case["nkv"]), c_int(d),
        c_int(case["bs"]), c_int(0), c_float(d ** -0.5), c_int(num_splits), c_int(waves), stream)
    return status, out


def call_with_workspace(ops, case, num_splits, waves):
    n, nh, d = case["n"], case["nh"], case["d"]
    out = new_out(case)
    ops.attention_mfma(out, case["q"], case["k_pool"], case["v_pool"], case["tables"], case["cu"], case["ctx"],
                       0, n, 1, 0, n, nh, case["nkv"], d, case["bs"], 0, None, split_waves=True,
                       num_splits=num_splits, waves=waves)
    return out


def test_decode_attention_without_allocation_matches_the_workspace_entry_point():
    from llmserve.ops import library as ops

    lib = ops.load("attention_mfma")
    big, big_ref = decode_case(32, 4, 64, 16, [600, 31, 257, 1, 90, 333], seed=5)
    small, small_ref = decode_case(8, 2, 128, 8, [150, 40], seed=9)
    out_big, out_small = new_out(big), new_out(small)
    # A first call outside the measurement: it loads the library's code object onto the device (which places the
    # fixed array) and asks for the array's address; callers under graph capture make it before they capture.
    warm, _ = decode_case(4, 2, 32, 8, [9], seed=2)
    assert call_noalloc(lib, warm, 2, 4, new_out(warm))[0] == 0
    # Neither of the two calls takes memory from the device: the free memory of the whole device (which a hipMalloc
    # behind torch's back would lower as well) and torch's own counters stay as they are.
    torch.cuda.synchronize()
    free_before, _total = torch.cuda.mem_get_info()
    reserved_before, allocated_before = torch.cuda.memory_reserved(), torch.cuda.memory_allocated()
    status_big, got_big = call_noalloc(lib, big, 5, 8, out_big)
    status_small, got_small = call_noalloc(lib, small, 3, 4, out_small)  # right behind it, over what the first call left
    torch.cuda.synchronize()
    assert status_big == 0 and status_small == 0
    assert torch.cuda.mem_get_info()[0] == free_before
    assert torch.cuda.memory_reserved() == reserved_before and torch.cuda.memory_allocated() == allocated_before
    for case, got, ref, splits, waves in ((big, got_big, big_ref, 5, 8), (small, got_small, small_ref, 3, 4)):
        want = call_with_workspace(ops, case, splits, waves)
        assert torch.isfinite(got.float()).all()
        assert torch.equal(got, want), "the two entry points run the same kernels in the same order"
        err = (got.float().cpu() - ref).abs().max()
        assert err <= max(1e-3, float(ref.abs().max())) * 2.0 ** -7


def test_decode_attention_without_allocation_refuses_what_does_not_fit():
    from llmserve.ops import library as ops

    lib = ops.load("attention_mfma")
    case, _ = decode_case(32, 4, 64, 16, [20, 20], seed=1)
    # 2 rows x 32 heads x 600 splits x 66 floats > 8 MiB: refused before anything is launched
    status, out = call_noalloc(lib, case, 600, 8, new_out(case))
    torch.cuda.synchronize()
    assert status == 1 and out.float().isnan().all()
    status, _ = call_noalloc(lib, case, 1, 8, new_out(case))  # one split needs no scratch and belongs to the other entry point
    assert status == 1
