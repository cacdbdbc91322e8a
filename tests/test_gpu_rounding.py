"""Write-back rounding on the device, exhaustively where it is cheap: float32 -> bf16 / f16 through
the first accumulation pass (acc = astype(g)) against the oracle's round-to-nearest-even and torch's
CPU conversion, for every tie pattern, subnormals, infinities and NaN."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import mxopt_oracle as O
from gpu_util import to_dev, to_host

F = np.float32


def special_values():
    rng = np.random.default_rng(3)
    ties = ((np.arange(65536, dtype=np.uint32) << 16) | 0x8000).view(F)              # exact halves
    near = ((np.arange(65536, dtype=np.uint32) << 16) | 0x7FFF).view(F)              # just below
    above = ((np.arange(65536, dtype=np.uint32) << 16) | 0x8001).view(F)             # just above
    sub = (rng.normal(0, 1, 4096) * 1e-39).astype(F)                                 # float32 subnormals
    misc = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 3.3895314e38, -3.3895314e38, 3.4028235e38, 65504.0, 65520.0,
                     6e-8, 1e-8], dtype=F)
    return np.concatenate([ties, near, above, sub, misc, rng.normal(0, 1, 100000).astype(F)])


@pytest.mark.parametrize("offset", [0, 1])
def test_bf16_write_back_is_round_to_nearest_even(offset):
    import torch
    import mxopt as mx
    x = special_values()
    ctx = mx.default_context()
    src = to_dev(x, offset)
    dst = torch.empty(x.size + 8, dtype=torch.bfloat16, device="cuda")[offset:offset + x.size]
    ctx.accumulate(ctx.table([mx.TensorSpec(g=src, g_out=dst)]), first=True)
    got = to_host(dst)
    want = O.f32_to_bf16(x)
    nan = np.isnan(x)
    assert np.array_equal(got[~nan], want[~nan])
    assert (((got[nan] & 0x7FFF) > 0x7F80)).all()                   # NaN stays NaN
    ref = torch.tensor(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got[~nan], ref[~nan])


def test_f16_write_back_is_round_to_nearest_even():
    import torch
    import mxopt as mx
    x = special_values()
    x = x[np.isfinite(x)]
    ctx = mx.default_context()
    src = to_dev(x)
    dst = torch.empty(x.size, dtype=torch.float16, device="cuda")
    ctx.accumulate(ctx.table([mx.TensorSpec(g=src, g_out=dst)]), first=True)
    got = dst.cpu().numpy()
    with np.errstate(over="ignore"):
        want = x.astype(np.float16)                                # NumPy converts with RNE
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
