"""triton_linear: out = a @ b + c with c broadcast along rows (ops/linear.py:5-71 of the reference,
an inductor matmul template with a bias suffix). b is addressed through (stride_bk, stride_bn); for
an nn.Linear weight W[N, K] that is W.T, i.e. stride_bk = 1 and stride_bn = K, which is the layout
the MFMA kernel wants. Any other layout is copied into it first."""
import torch

from triton_kernels.kernels.linear import linear_into
from triton_kernels.ops._launch import HipOp


def _linear(a_ptr, b_ptr, c_ptr, out_ptr, M, N, K, stride_am, stride_ak, stride_bk, stride_bn):
    M, N, K = int(M), int(N), int(K)
    a = torch.as_strided(a_ptr, (M, K), (int(stride_am), int(stride_ak)))
    w = torch.as_strided(b_ptr, (N, K), (int(stride_bn), int(stride_bk)))  # W[n, k] = b[k, n]
    out = out_ptr.view(-1)[: M * N].view(M, N)
    linear_into(a, w, c_ptr, out=out)
    return out_ptr


triton_linear = HipOp(_linear, "triton_linear")
