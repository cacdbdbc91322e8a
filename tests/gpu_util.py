"""Helpers shared by the GPU parity tests: moving oracle arrays (float32, or bf16 bit
patterns in uint16) to the device and back without any arithmetic on the way."""
from __future__ import annotations

import numpy as np
import torch


def to_dev(a: np.ndarray, offset_elems: int = 0) -> torch.Tensor:
    """numpy -> device tensor.  uint16 arrays are bf16 bit patterns.  With offset_elems > 0 the
    tensor is a view that starts that many elements into a larger allocation, so that its
    address is only naturally aligned."""
    if a.dtype == np.uint16:
        t = torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)
    elif a.dtype == np.float16:
        t = torch.from_numpy(a.copy())
    else:
        t = torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32).copy())
    if offset_elems:
        slab = torch.empty(t.numel() + offset_elems + 16, dtype=t.dtype, device="cuda")
        view = slab[offset_elems:offset_elems + t.numel()]
        view.copy_(t)
        return view
    return t.cuda()


def to_host(t: torch.Tensor) -> np.ndarray:
    """device tensor -> numpy (bf16 comes back as uint16 bit patterns)."""
    t = t.detach().cpu().contiguous()
    if t.dtype == torch.bfloat16:
        return t.view(torch.int16).numpy().view(np.uint16).copy()
    return t.numpy().copy()


def bits(a: np.ndarray) -> np.ndarray:
    a = np.ascontiguousarray(a)
    return a.view(np.uint32) if a.dtype == np.float32 else a.view(np.uint16)


def assert_bit_equal(got: np.ndarray, want: np.ndarray, what: str = "") -> None:
    assert got.dtype == want.dtype and got.shape == want.shape, (what, got.dtype, want.dtype, got.shape, want.shape)
    gb, wb = bits(got), bits(want)
    if np.array_equal(gb, wb):
        return
    # NaNs may differ in payload only
    if got.dtype in (np.float32, np.float16):
        both_nan = np.isnan(got) & np.isnan(want)
    else:
        both_nan = ((gb & 0x7FFF) > 0x7F80) & ((wb & 0x7FFF) > 0x7F80)
    bad = (gb != wb) & ~both_nan
    if bad.any():
        i = int(np.flatnonzero(bad)[0])
        raise AssertionError(f"{what}: {int(bad.sum())} of {bad.size} elements differ; first at {i}: "
                             f"got {got[i]!r} ({gb[i]:#x}) want {want[i]!r} ({wb[i]:#x})")


def _ordered(a: np.ndarray) -> np.ndarray:
    """Bit patterns mapped to integers that are ordered like the values (float32 or bf16 in uint16)."""
    a = np.ascontiguousarray(a)
    if a.dtype == np.float32:
        u = a.view(np.uint32).astype(np.int64)
        return np.where(u & 0x80000000, 0x80000000 - u, u)
    u = a.astype(np.int64)
    return np.where(u & 0x8000, 0x8000 - u, u)


def assert_within_ulps(got: np.ndarray, want: np.ndarray, ulps: int, rel: float = 0.0, what: str = "") -> int:
    """Every element within `ulps` units in the last place of its dtype (float32, or bf16 held as uint16), or --
    when rel > 0, float32 only -- within rel * |want|.  Returns the largest distance seen, in ulps."""
    assert got.dtype == want.dtype and got.shape == want.shape, (what, got.dtype, want.dtype)
    d = np.abs(_ordered(got) - _ordered(want))
    bad = d > ulps
    if rel > 0.0 and got.dtype == np.float32 and bad.any():
        bad &= np.abs(got.astype(np.float64) - want.astype(np.float64)) > rel * np.abs(want.astype(np.float64))
    if bad.any():
        i = int(np.flatnonzero(bad)[0])
        raise AssertionError(f"{what}: {int(bad.sum())} of {bad.size} elements are more than {ulps} ulp apart; "
                             f"first at {i}: got {got[i]!r} want {want[i]!r} ({int(d[i])} ulp)")
    return int(d.max()) if d.size else 0
