"""Call convention shim for the raw `ops` kernels.

In the reference these are bare @triton.jit kernels (no launcher, no importer), so the only thing
their callers can rely on is the name, the positional argument order and the launch spelling
`kernel[grid](*args, XBLOCK=...)`. A HipOp accepts that spelling as well as a plain call; grid and
the block-size keywords carry no information for the HIP kernels and are ignored. Pointer arguments
are torch tensors on the GPU.
"""
from __future__ import annotations

_IGNORED_KW = {
    "XBLOCK", "BLOCK_M", "BLOCK_N", "BLOCK_K", "GROUP_M", "EVEN_K", "ALLOW_TF32", "ACC_TYPE",
    "B_PROLOGUE_CAST_TYPE", "num_warps", "num_stages", "num_ctas",
}


class HipOp:
    def __init__(self, fn, name: str):
        self._fn = fn
        self.__name__ = name
        self.__doc__ = fn.__doc__

    def __call__(self, *args, **kw):
        kw = {k: v for k, v in kw.items() if k not in _IGNORED_KW}
        return self._fn(*args, **kw)

    def __getitem__(self, grid):
        return self.__call__

    def __repr__(self):
        return f"<HipOp {self.__name__}>"
