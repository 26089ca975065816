"""Hadamard tables and plans for the online rotation (host side).

Selection rule and table data follow `get_hadK` and the `get_had<K>` tables of the reference
(mxmoe/quant/hadamard_utils.py:5-59, 162-4379); the tables live bit-packed in data/had_tables.npz.
"""
from __future__ import annotations

from functools import lru_cache
from pathlib import Path

import numpy as np
import torch

_HAD_FILE = Path(__file__).resolve().parent / "data" / "had_tables.npz"
_HAD_ORDER = (176, 172, 156, 140, 108, 60, 52, 36, 28, 40, 20, 12)  # test order of get_hadK


def is_pow2(n: int) -> bool:
    return n > 0 and (n & (n - 1)) == 0


@lru_cache(maxsize=None)
def had_table(k: int) -> np.ndarray:
    bits = np.unpackbits(np.load(_HAD_FILE)[f"had{k}"])[: k * k].reshape(k, k)
    return (1 - 2 * bits.astype(np.int8)).astype(np.int8)


def get_hadK(n: int):
    """(H_K or None, K): first K in the reference's order dividing n with n / K a power of two."""
    for k in _HAD_ORDER:
        if n % k == 0:
            if not is_pow2(n // k):
                raise ValueError(f"n = {n}: n / {k} is not a power of two")
            return had_table(k), k
    if not is_pow2(n):
        raise ValueError(f"n = {n} is neither a power of two nor (known Hadamard order) x (power of two)")
    return None, 1


@lru_cache(maxsize=None)
def had_plan(n: int):
    """(K, f, B) with H_K = S_f kron B, S_f Sylvester of the largest power of two f for which that holds."""
    hk, k = get_hadK(n)
    if k == 1:
        return 1, 1, None
    f = 1
    while k % (2 * f) == 0:
        g = 2 * f
        b = k // g
        blk = hk[:b, :b]
        if not all(np.array_equal(hk[i * b:(i + 1) * b, j * b:(j + 1) * b], ((-1) ** bin(i & j).count("1")) * blk) for i in range(g) for j in range(g)):
            break
        f = g
    kb = k // f
    return k, f, hk[:kb, :kb].astype(np.float32).copy()


_sign_cache: dict = {}


def device_signs(n: int, device) -> tuple[int, int, torch.Tensor | None]:
    """(K, f, B as a device float tensor or None) for row length n, cached per device."""
    k, f, b = had_plan(n)
    if b is None:
        return k, f, None
    key = (k, str(device))
    if key not in _sign_cache:
        _sign_cache[key] = torch.from_numpy(b).to(device).contiguous()
    return k, f, _sign_cache[key]
