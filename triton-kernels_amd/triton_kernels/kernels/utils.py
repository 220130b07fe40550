"""Launch-shape helper kept for API compatibility with kernels/utils.py:4-19 of the reference.

The HIP row-wise kernels pick their own lanes-per-row / vectors-per-lane plan on the C side; this
function only reports the equivalent (padded row length, waves) pair and enforces the same limit.
"""
from triton_kernels._native import MAX_ROW


def _next_pow2(n: int) -> int:
    return 1 if n <= 1 else 1 << (int(n) - 1).bit_length()


def calculate_settings(n: int):
    width = _next_pow2(n)
    if width > MAX_ROW:
        raise RuntimeError(f"Cannot launch a row-wise kernel: n = {n} exceeds the maximum row length {MAX_ROW}.")
    waves = 4
    for threshold, w in ((32768, 32), (8192, 16), (2048, 8)):
        if width >= threshold:
            waves = w
            break
    return width, waves
