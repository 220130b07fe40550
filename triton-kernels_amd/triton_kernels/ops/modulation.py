"""adaLN helpers that read shift / scale / gate straight out of the [B, 6*hid] (or [B, 3*hid])
Modulation projection (ops/modulation.py:5-44 of the reference).

Argument names follow the reference even where they mislead: `batch_size` is the number of elements
per batch entry (L * hid), `head_size` is the hidden size, `modulation_size` the row stride of the
modulation tensor.
"""
from triton_kernels import _native as nv
from triton_kernels.ops._launch import HipOp


def _dims(x, batch_size, head_size):
    total = x.numel()
    per_batch, hid = int(batch_size), int(head_size)
    assert per_batch % hid == 0 and total % per_batch == 0
    return total // per_batch, per_batch // hid, hid


def _scale_shift(x_ptr, modulation_ptr, output_ptr, batch_size, head_size, modulation_size, is_mod1):
    """output = (1 + scale) * x + shift with (shift, scale) = modulation chunks (0, 1) if is_mod1 else (3, 4)."""
    dev = nv.require_gpu(x_ptr, modulation_ptr, output_ptr)
    assert x_ptr.is_contiguous() and output_ptr.is_contiguous() and modulation_ptr.stride(-1) == 1
    assert x_ptr.dtype == modulation_ptr.dtype == output_ptr.dtype
    B, L, hid = _dims(x_ptr, batch_size, head_size)
    with nv.on_device(dev):
        rc = nv.lib().flux_modulation_scale_shift(
            x_ptr.data_ptr(), modulation_ptr.data_ptr(), output_ptr.data_ptr(), B, L, hid, int(modulation_size),
            1 if is_mod1 else 0, nv.dtype_code(x_ptr), nv.stream_ptr(dev))
    nv.check(rc, "flux_modulation_scale_shift")
    return output_ptr


def _gate_proj(img_ptr, mod_ptr, proj_ptr, output_ptr, batch_size, head_size, modulation_size):
    """output = img + gate * proj with gate = modulation chunk 2, products kept in fp32."""
    dev = nv.require_gpu(img_ptr, mod_ptr, proj_ptr, output_ptr)
    assert img_ptr.is_contiguous() and proj_ptr.is_contiguous() and output_ptr.is_contiguous()
    assert img_ptr.dtype == mod_ptr.dtype == proj_ptr.dtype == output_ptr.dtype and mod_ptr.stride(-1) == 1
    B, L, hid = _dims(img_ptr, batch_size, head_size)
    gate_ptr = mod_ptr.data_ptr() + 2 * hid * mod_ptr.element_size()
    with nv.on_device(dev):
        rc = nv.lib().flux_gate_residual(
            img_ptr.data_ptr(), gate_ptr, proj_ptr.data_ptr(), output_ptr.data_ptr(), B, L, hid, int(modulation_size),
            0, nv.dtype_code(img_ptr), nv.stream_ptr(dev))
    nv.check(rc, "flux_gate_residual")
    return output_ptr


triton_modulation_scale_shift = HipOp(_scale_shift, "triton_modulation_scale_shift")
triton_modulation_gate_proj = HipOp(_gate_proj, "triton_modulation_gate_proj")
