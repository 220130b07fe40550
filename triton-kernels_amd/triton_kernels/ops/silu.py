"""triton_silu(x_ptr, b_ptr, xnumel): b = x * sigmoid(x) (ops/silu.py:5-13 of the reference)."""
from triton_kernels import _native as nv
from triton_kernels.ops._launch import HipOp


def _silu(x_ptr, b_ptr, xnumel=None):
    dev = nv.require_gpu(x_ptr, b_ptr)
    n = x_ptr.numel() if xnumel is None else int(xnumel)
    assert x_ptr.is_contiguous() and b_ptr.is_contiguous() and x_ptr.dtype == b_ptr.dtype
    assert n <= x_ptr.numel() and n <= b_ptr.numel()
    with nv.on_device(dev):
        rc = nv.lib().flux_silu(x_ptr.data_ptr(), b_ptr.data_ptr(), n, nv.dtype_code(x_ptr), nv.stream_ptr(dev))
    nv.check(rc, "flux_silu")
    return b_ptr


triton_silu = HipOp(_silu, "triton_silu")
