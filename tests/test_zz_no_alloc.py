"""The argmax entry point that allocates nothing (``tie_argmax_static``), called through ctypes.

Its candidates between the two stages live in a static device array instead of a workspace, so the
test checks what that changes: two calls in a row, the second on a smaller input (fewer and shorter
rows, so that stale candidates of the first call lie beside the new ones), each against the
existing ``tie_argmax`` with a workspace; the size limit; and that no device memory is allocated.
"""

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

MAX_ROWS = 1024
TOO_LARGE = -2


def _library():
    from tie_amd import kernels
    return kernels._lib("elementwise")


def _reference(lib, logits):
    R, V = logits.shape
    out = torch.full((R,), -7, dtype=torch.int32, device=logits.device)
    mx = torch.zeros(R, dtype=torch.float32, device=logits.device)
    part_v = torch.empty(R * 64, dtype=torch.float32, device=logits.device)
    part_i = torch.empty(R * 64, dtype=torch.int32, device=logits.device)
    stream = torch.cuda.current_stream().cuda_stream
    assert lib.tie_argmax(logits.data_ptr(), out.data_ptr(), mx.data_ptr(), part_v.data_ptr(), part_i.data_ptr(),
                          R, V, stream) == 0
    return out, mx


def _static(lib, logits, out, mx):
    R, V = logits.shape
    stream = torch.cuda.current_stream().cuda_stream
    return lib.tie_argmax_static(ctypes.c_void_p(logits.data_ptr()), ctypes.c_void_p(out.data_ptr()),
                                 ctypes.c_void_p(mx.data_ptr()), R, V, ctypes.c_void_p(stream))


def test_two_calls_in_a_row_match_the_workspace_argmax_and_allocate_nothing():
    lib = _library()
    dev = torch.device("cuda:0")
    gen = torch.Generator(device="cpu").manual_seed(5)
    big = torch.randn(37, 5003, generator=gen).to(dev)
    big[3, 4999] = 50.0                      # a maximum in the last, short slice of a row
    big[9, 17] = float("nan")                # a NaN row reports -1
    big[11, 100] = big[11, 4000] = 40.0      # a tie goes to the lower index
    small = torch.randn(5, 129, generator=gen).to(dev)
    small[4, 128] = 30.0
    outs = [torch.full((t.shape[0],), -7, dtype=torch.int32, device=dev) for t in (big, small)]
    maxes = [torch.zeros(t.shape[0], dtype=torch.float32, device=dev) for t in (big, small)]
    want = [_reference(lib, t) for t in (big, small)]
    torch.cuda.synchronize()

    before = torch.cuda.memory_stats(dev)["allocation.all.allocated"], torch.cuda.mem_get_info(dev)[0]
    for t, o, m in zip((big, small), outs, maxes):          # back to back on one stream, nothing in between
        assert _static(lib, t, o, m) == 0
    torch.cuda.synchronize()
    after = torch.cuda.memory_stats(dev)["allocation.all.allocated"], torch.cuda.mem_get_info(dev)[0]
    assert after[0] == before[0], "the entry point went through torch's allocator"
    assert after[1] >= before[1], "free device memory shrank during the calls"

    for (w_out, w_max), o, m in zip(want, outs, maxes):
        assert torch.equal(o.cpu(), w_out.cpu())
        got, ref = m.cpu(), w_max.cpu()
        assert torch.equal(torch.isnan(got), torch.isnan(ref)) and torch.equal(got[~torch.isnan(got)], ref[~torch.isnan(ref)])
    assert outs[0][3].item() == 4999 and outs[0][9].item() == -1 and outs[0][11].item() == 100
    assert outs[1][4].item() == 128


def test_the_python_wrapper_and_the_row_limit():
    from tie_amd import kernels
    from tie_amd.errors import InvalidArgument

    lib = _library()
    dev = torch.device("cuda:0")
    full = torch.randn(MAX_ROWS, 70, device=dev)
    out = torch.empty(MAX_ROWS, dtype=torch.int32, device=dev)
    kernels.argmax_rows_static(full, out)                    # the largest size it takes
    assert torch.equal(out.cpu().long(), full.cpu().argmax(dim=1))
    over = torch.randn(MAX_ROWS + 1, 70, device=dev)
    out2 = torch.full((MAX_ROWS + 1,), -7, dtype=torch.int32, device=dev)
    mx2 = torch.zeros(MAX_ROWS + 1, dtype=torch.float32, device=dev)
    assert _static(lib, over, out2, mx2) == TOO_LARGE
    torch.cuda.synchronize()
    assert bool((out2 == -7).all()), "a refused call must launch nothing"
    with pytest.raises(InvalidArgument, match="at most 1024 rows"):
        kernels.argmax_rows_static(over, out2)
