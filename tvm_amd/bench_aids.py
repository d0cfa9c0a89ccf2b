"""Python face of libtvmkv_bench.so: the measurement aids of bench.py (include/tvmkv_bench.h).  They are
not part of the drop-in library and have no counterpart in the reference."""
import ctypes

import torch

from ._lib import KVError, bench_lib
from .kernels import _p, _stream


def _check(rc, what):
    if rc != 0:
        raise KVError(rc, f"{what} failed with code {rc}")


def stream_read(src, sink):
    """Plain streaming read of the whole tensor (bandwidth calibration)."""
    _check(bench_lib().tvmkvb_stream_read(_p(src), src.numel() * src.element_size(), _p(sink), _stream()), "stream_read")


def stream_read_nt(src, sink):
    """stream_read with non-temporal loads."""
    _check(bench_lib().tvmkvb_stream_read_nt(_p(src), src.numel() * src.element_size(), _p(sink), _stream()),
           "stream_read_nt")


def stream_copy(src, dst):
    """Plain copy of the whole tensor (bandwidth calibration, counter scaling)."""
    _check(bench_lib().tvmkvb_stream_copy(_p(src), _p(dst), src.numel() * src.element_size(), _stream()), "stream_copy")


def mfma_loop(operands, out, iters):
    """Matrix-core calibration loop: operands (256, 16) fp16, out (workgroups, 256) fp32."""
    assert operands.dtype == torch.float16 and operands.numel() == 256 * 16
    assert out.dtype == torch.float32 and out.shape[1] == 256
    _check(bench_lib().tvmkvb_mfma_loop(_p(operands), _p(out), int(iters), out.shape[0], _stream()), "mfma_loop")


class ClockSampler:
    """Shader clock while the body of the `with` block runs on the current stream: one wave on a second
    stream (default priority) reads the shader-cycle counter and the 100 MHz counter until the block has
    finished (or `max_seconds` have passed, whichever comes first).  `mhz` holds the result afterwards."""

    def __init__(self, max_seconds=5.0):
        self.max_ticks = int(min(max_seconds, 10.0) * 1e8)
        self.stream = torch.cuda.Stream()
        self.flag = torch.zeros(1, dtype=torch.int32).pin_memory()
        self.out = torch.zeros(2, dtype=torch.int64, device="cuda")
        self.mhz = None

    def __enter__(self):
        self.flag[0] = 0
        torch.cuda.synchronize()
        _check(bench_lib().tvmkvb_clock_sampler(ctypes.c_void_p(self.flag.data_ptr()), self.max_ticks, _p(self.out),
                                                ctypes.c_void_p(self.stream.cuda_stream)), "clock_sampler")
        return self

    def __exit__(self, *exc):
        torch.cuda.current_stream().synchronize()
        self.flag[0] = 1  # the sampler sees it within one sleep period and ends
        self.stream.synchronize()
        cycles, ticks = (int(x) for x in self.out.cpu())
        self.mhz = cycles / max(ticks, 1) * 100.0
        return False
