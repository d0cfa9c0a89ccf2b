"""Python face of libtvmkv_bench.so: the measurement aids of bench.py (include/tvmkv_bench.h).  They are
not part of the drop-in library and have no counterpart in the reference."""
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
