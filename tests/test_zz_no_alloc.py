"""The sampling entry point that allocates nothing (``tl_sample_static``), called through ``ctypes``
as a caller without the package would: against ``tl_sample`` (which takes the caller's scratch
buffer) on two calls in a row, the second with a smaller input, then the refusal of too many rows.
"""
import ctypes
from ctypes import c_int, c_void_p

import pytest
import torch

pytestmark = pytest.mark.gpu

MAX_ROWS = 256       # TL_SAMPLE_STATIC_MAX_ROWS of csrc/sampling.h


def _library():
    from torchlet_amd.kernels import build

    lib = ctypes.CDLL(str(build.build("sampling")))
    lib.tl_last_error.restype = ctypes.c_char_p
    return lib


def _ptr(t):
    return c_void_p(t.data_ptr()) if t is not None else c_void_p(0)


def _both(lib, logits, temperature, keys):
    """Tokens of the entry point with the caller's scratch and of the one with the library's own."""
    rows, vocab = logits.shape
    stream = c_void_p(torch.cuda.current_stream().cuda_stream)
    chunks = lib.tl_sample_chunks(c_int(vocab))
    scratch = torch.empty((2, rows, chunks), dtype=torch.int32, device=logits.device)
    want = torch.full((rows,), -1, dtype=torch.int32, device=logits.device)
    got = torch.full((rows,), -2, dtype=torch.int32, device=logits.device)
    rc = lib.tl_sample(_ptr(logits), c_int(rows), c_int(vocab), c_int(logits.stride(0)), _ptr(temperature), _ptr(keys),
                       _ptr(want), _ptr(scratch), stream)
    assert rc == 0, lib.tl_last_error().decode()
    static = lambda: lib.tl_sample_static(_ptr(logits), c_int(rows), c_int(vocab), c_int(logits.stride(0)), _ptr(temperature),
                                          _ptr(keys), _ptr(got), stream)
    rc = static()           # (the first call on a device asks for the array's address and loads the kernels)
    assert rc == 0, lib.tl_last_error().decode()
    torch.cuda.synchronize()
    # Free memory of the device itself, not the count of torch's allocator (which a hipMalloc inside the
    # library would not move): with torch's allocator idle, a call must leave it where it was.
    free_before, _ = torch.cuda.mem_get_info()
    held_before = torch.cuda.memory_reserved()
    got.fill_(-2)
    torch.cuda.synchronize()
    rc = static()
    assert rc == 0, lib.tl_last_error().decode()
    torch.cuda.synchronize()
    assert torch.cuda.memory_reserved() == held_before, "torch's own allocator moved: the measurement below would not be the library's"
    assert torch.cuda.mem_get_info()[0] == free_before, "tl_sample_static changed the device's free memory"
    return want.tolist(), got.tolist()


def test_the_measurement_of_free_device_memory_sees_an_allocation_that_torch_does_not_count():
    """What the check above relies on: memory taken from the device behind torch's back (here through the HIP runtime
    directly, as a ``hipMalloc`` inside the library would be) lowers ``mem_get_info`` and leaves torch's count alone."""
    torch.cuda.synchronize()
    # the HIP runtime this process already runs on (the copy torch loaded), not a second one
    loaded = {line.split()[-1] for line in open("/proc/self/maps") if "libamdhip64" in line}
    assert len(loaded) == 1, loaded
    hip = ctypes.CDLL(loaded.pop())
    free_before, counted = torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated()
    ptr = c_void_p()
    assert hip.hipMalloc(ctypes.byref(ptr), ctypes.c_size_t(64 << 20)) == 0
    try:
        assert torch.cuda.mem_get_info()[0] <= free_before - (64 << 20) and torch.cuda.memory_allocated() == counted
    finally:
        assert hip.hipFree(ptr) == 0


def test_sampling_without_allocation_matches_the_entry_point_with_scratch():
    lib = _library()
    g = torch.Generator().manual_seed(11)
    # first call: many rows of a wide vocabulary (the most chunks), greedy and temperature rows mixed
    rows, vocab = 37, 152064
    logits = torch.randn((rows, vocab), generator=g).cuda()
    logits[3, 777] = logits[3, 150000] = 50.0                      # a tie: the lower index wins
    temperature = torch.tensor([0.0 if i % 3 == 0 else 0.5 + 0.1 * i for i in range(rows)]).cuda()
    keys = torch.randint(-2**31, 2**31 - 1, (rows,), generator=g, dtype=torch.int64).to(torch.int32).cuda()
    want, got = _both(lib, logits, temperature, keys)
    assert got == want
    assert got[3] == 777 and got[0] == int(logits[0].argmax())
    assert len(set(got)) > rows // 2                               # draws, not one constant
    # second call, smaller in rows and in vocabulary (fewer chunks, another row pitch inside the array):
    # what the first call left there must not show
    rows2, vocab2 = 5, 3001
    logits2 = torch.randn((rows2, vocab2), generator=g).cuda()
    want2, got2 = _both(lib, logits2, None, None)
    assert got2 == want2 == logits2.argmax(dim=1).tolist()
    # a view with a row stride, at the largest row count
    wide = torch.randn((MAX_ROWS, 1500), generator=g).cuda()
    want3, got3 = _both(lib, wide[:, :1201], None, None)
    assert got3 == want3 == wide[:, :1201].argmax(dim=1).tolist()


def test_sampling_without_allocation_refuses_what_its_array_cannot_hold():
    lib = _library()
    logits = torch.zeros((MAX_ROWS + 1, 64), device="cuda")
    out = torch.zeros((MAX_ROWS + 1,), dtype=torch.int32, device="cuda")
    stream = c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = lib.tl_sample_static(_ptr(logits), c_int(MAX_ROWS + 1), c_int(64), c_int(64), c_void_p(0), c_void_p(0), _ptr(out), stream)
    assert rc != 0 and b"256" in lib.tl_last_error()
    torch.cuda.synchronize()
