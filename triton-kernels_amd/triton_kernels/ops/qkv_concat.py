"""triton_qkv_concat: split the txt and img qkv projections into heads and concatenate them along
the sequence, txt first (ops/qkv_concat.py:5-60 of the reference).

Inputs  txt_qkv [B, Lt, 3*hidden], img_qkv [B, Li, 3*hidden]  (rows may be strided)
Outputs q, k, v each contiguous [B, H, Lt+Li, D] with hidden = H*D. Pure data movement, bit-exact.
The stride arguments of the reference signature are accepted and checked against the tensors.
"""
from triton_kernels import _native as nv
from triton_kernels.ops._launch import HipOp


def _qkv_concat(txt_qkv, img_qkv, out_q_ptr, out_k_ptr, out_v_ptr,
                seq_len, num_heads, head_dim, hidden_dim, seq_txt_len,
                stride_txt_a=None, stride_txt_b=None, stride_img_a=None, stride_img_b=None,
                stride_output_a=None, stride_output_b=None, stride_output_c=None):
    dev = nv.require_gpu(txt_qkv, img_qkv, out_q_ptr, out_k_ptr, out_v_ptr)
    H, D, hid, L, Lt = int(num_heads), int(head_dim), int(hidden_dim), int(seq_len), int(seq_txt_len)
    Li = L - Lt
    assert hid == H * D
    B = img_qkv.shape[0]
    assert img_qkv.shape == (B, Li, 3 * hid) and img_qkv.stride(2) == 1
    if Lt:
        assert txt_qkv.shape == (B, Lt, 3 * hid) and txt_qkv.stride(2) == 1 and txt_qkv.dtype == img_qkv.dtype
    for given, actual in ((stride_txt_a, txt_qkv.stride(0) if Lt else None), (stride_txt_b, txt_qkv.stride(1) if Lt else None),
                          (stride_img_a, img_qkv.stride(0)), (stride_img_b, img_qkv.stride(1)),
                          (stride_output_a, H * L * D), (stride_output_b, L * D), (stride_output_c, D)):
        assert given is None or actual is None or int(given) == actual, "stride argument disagrees with the tensor"
    a = nv.QkvPrepArgs()
    esz = img_qkv.element_size()
    for i, (name, out) in enumerate((("q", out_q_ptr), ("k", out_k_ptr), ("v", out_v_ptr))):
        assert out.is_contiguous() and out.numel() == B * H * L * D and out.dtype == img_qkv.dtype
        setattr(a, f"{name}_img", nv.Src4(img_qkv.data_ptr() + i * hid * esz, img_qkv.stride(0), D, img_qkv.stride(1)))
        if Lt:
            setattr(a, f"{name}_txt", nv.Src4(txt_qkv.data_ptr() + i * hid * esz, txt_qkv.stride(0), D, txt_qkv.stride(1)))
        setattr(a, f"{name}_out", out.data_ptr())
    a.B, a.H, a.Lt, a.Li, a.D = B, H, Lt, Li, D
    a.dtype = a.scale_dtype = nv.dtype_code(img_qkv)
    a.eps = 0.0
    with nv.on_device(dev):
        rc = nv.lib().flux_qkv_prep(nv.byref(a), nv.stream_ptr(dev))
    nv.check(rc, "flux_qkv_prep")
    return out_q_ptr, out_k_ptr, out_v_ptr


triton_qkv_concat = HipOp(_qkv_concat, "triton_qkv_concat")
