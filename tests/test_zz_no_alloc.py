"""The argmax entry point that allocates nothing (`lle_argmax_rows_static`, its partial
results in a buffer inside the library's device image), called through ctypes as a C caller
would, against the entry point with caller-provided workspaces.  Two calls in a row on the
same buffer, the second with a smaller input; the size limit is refused with its own code."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

MAX_ROWS = 256
TOO_SMALL = 100001


def entry_points():
    from litellmengine_amd.csrc import build

    lib = build.load_library("sampling")
    static = lib.lle_argmax_rows_static
    static.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    static.restype = ctypes.c_int
    return lib, static


def test_static_argmax_equals_workspace_argmax_twice_in_a_row():
    from litellmengine_amd.csrc.ops import default_ops

    ops = default_ops()
    lib, static = entry_points()
    dev = torch.device("cuda", torch.cuda.current_device())
    g = torch.Generator(device="cpu").manual_seed(5)
    stream = torch.cuda.current_stream().cuda_stream
    # The library's code and its static array come to the device with its first launch; after that
    # a call may not change what the device has free (torch's own counters cannot see a hipMalloc
    # made inside the library: hipMemGetInfo, through mem_get_info, can).
    warm = torch.zeros((2, 4099), device=dev)
    assert static(warm.data_ptr(), torch.empty(2, dtype=torch.int32, device=dev).data_ptr(), 2, 4099, stream) == 0
    torch.cuda.synchronize()
    # the second call is smaller in both directions: what the first left in the buffer must not show
    for rows, vocab in ((37, 151936), (5, 4099), (MAX_ROWS, 2048 * 3 + 17), (1, 7)):
        logits = torch.randn((rows, vocab), generator=g).to(dev)
        logits[0, vocab // 2] = logits[0, vocab - 1] = 50.0  # a tie: the first maximum wins
        want = ops.argmax(logits)
        out = torch.full((rows,), -7, dtype=torch.int32, device=dev)
        torch.cuda.synchronize()
        before, free_before = torch.cuda.memory_allocated(dev), torch.cuda.mem_get_info(dev)[0]
        code = static(logits.data_ptr(), out.data_ptr(), rows, vocab, stream)
        assert code == 0, lib.lle_error_string(code).decode()
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated(dev) == before
        assert torch.cuda.mem_get_info(dev)[0] == free_before, "the call took device memory"
        assert torch.equal(out, want), (rows, vocab)
        assert out[0].item() == vocab // 2
        assert torch.equal(out.cpu().long(), logits.cpu().argmax(dim=1))


def test_static_argmax_refuses_more_rows_than_its_buffer_holds():
    lib, static = entry_points()
    dev = torch.device("cuda", torch.cuda.current_device())
    logits = torch.zeros((MAX_ROWS + 1, 64), dtype=torch.float32, device=dev)
    out = torch.full((MAX_ROWS + 1,), -7, dtype=torch.int32, device=dev)
    code = static(logits.data_ptr(), out.data_ptr(), MAX_ROWS + 1, 64, torch.cuda.current_stream().cuda_stream)
    assert code == TOO_SMALL
    assert b"at most 256 rows" in lib.lle_error_string(code)
    torch.cuda.synchronize()
    assert (out == -7).all()  # nothing was launched
