"""The streaming-probe library (libmhc_probe.so, csrc/stream_probe.hip): every mode moves the bytes it
says it moves, and arguments that do not fit a mode are refused on the host before any launch."""
import ctypes
import os

import pytest
import torch

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HIP_ERROR_INVALID_VALUE = 1


def _probe():
    fn = ctypes.CDLL(os.path.join(ROOT, "mhc.cu_amd", "mhc", "libmhc_probe.so")).mhc_stream_probe
    fn.restype = ctypes.c_int
    fn.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.c_void_p,
                   ctypes.c_void_p]
    return fn


def test_modes_move_what_they_say():
    fn = _probe()
    n = 1 << 20  # int32 words: 4 MiB, plus a ragged tail of 16-byte words
    n += 12
    src = torch.arange(n, dtype=torch.int32, device="cuda")
    sink = torch.zeros(1, dtype=torch.int32, device="cuda")
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for mode in (1, 4):  # copies
        for blocks in (0, 7, 4096):
            dst = torch.full_like(src, -1)
            assert fn(mode, src.data_ptr(), dst.data_ptr(), n * 4, blocks, None, st) == 0
            torch.cuda.synchronize()
            assert torch.equal(dst, src), (mode, blocks)
    for mode in (2, 5):  # fills with the bit pattern of 1.0f
        dst = torch.zeros(n, dtype=torch.float32, device="cuda")
        assert fn(mode, None, dst.data_ptr(), n * 4, 64, None, st) == 0
        torch.cuda.synchronize()
        assert bool((dst == 1.0).all()), mode
    for mode in (0, 3):  # read-only: leaves everything as it was
        assert fn(mode, src.data_ptr(), None, n * 4, 0, sink.data_ptr(), st) == 0
        torch.cuda.synchronize()
        assert int(sink.item()) == 0
    assert fn(6, None, None, 0, 2048, None, st) == 0  # the empty launch takes no memory at all
    torch.cuda.synchronize()


def test_bad_arguments_are_refused_before_any_launch():
    fn = _probe()
    buf = torch.zeros(1024, dtype=torch.int32, device="cuda")
    p, st = buf.data_ptr(), None
    bad = [(0, None, None, 4096, 0, p), (0, p, None, 4096, 0, None), (1, p, None, 4096, 0, None),
           (2, None, None, 4096, 0, None), (1, p, p + 4, 4096 - 16, 0, None), (1, p, p, 4090, 0, None),
           (1, p, p, 0, 0, None), (7, p, p, 4096, 8, p), (10, p, None, 4096, 8, p), (-1, p, p, 4096, 0, p),
           (1, p, p, 4096, -3, None), (1, p, p, 4096, (1 << 20) + 1, None)]
    for mode, s, d, nbytes, blocks, sink in bad:
        assert fn(mode, s, d, nbytes, blocks, sink, st) == HIP_ERROR_INVALID_VALUE, (mode, nbytes, blocks)
    torch.cuda.synchronize()
    assert int(buf.abs().sum().item()) == 0
