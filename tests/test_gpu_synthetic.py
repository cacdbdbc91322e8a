"""The device side of the synthetic-data generator against the oracle's statement of it, bit for bit:
every distribution, every dtype, ragged sizes, unaligned buffers, slices that start in the middle."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import mxopt_oracle as O
from gpu_util import assert_bit_equal, to_host


@pytest.mark.parametrize("dist,a,b", [(O.SYNTH_NORMAL, 1e-3, 0.0), (O.SYNTH_NORMAL_OUTLIERS, 1e-3, 100.0),
                                      (O.SYNTH_UNIFORM, 0.9, 1.1), (O.SYNTH_NORMAL, 0.02, 0.0),
                                      (O.SYNTH_GAUSSIAN, 1e-3, 0.0), (O.SYNTH_GAUSSIAN_OUTLIERS, 0.02, 100.0)])
@pytest.mark.parametrize("dt", ["f32", "bf16", "f16"])
def test_device_fill_equals_the_oracle(dist, a, b, dt):
    import torch
    import mxopt as mx
    ctx = mx.default_context()
    tdt = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}[dt]
    for n, offset, first in ((0, 0, 0), (1, 0, 0), (1000003, 0, 0), (70001, 3, 2 ** 33 + 5), (4096, 1, 12345)):
        seed = mx.synthetic_key(0x5EED0001, 5, 2, 1, n)
        assert seed == O.synthetic_key(0x5EED0001, 5, 2, 1, n)
        buf = torch.full((n + 16,), 7.0, dtype=tdt, device="cuda")
        view = buf[offset:offset + n]
        ctx.fill_synthetic(view, seed, dist, a, b, first_index=first)
        assert_bit_equal(to_host(view), O.synthetic(n, dt, seed, dist, a, b, first_index=first), f"{dt} n={n}")
        assert (buf[:offset] == 7.0).all() and (buf[offset + n:] == 7.0).all()      # nothing outside the view


def test_full_size_inputs_can_be_checked_slice_by_slice():
    """A 622 M element tensor (the largest of the 8B list) filled on the device; seeded slices regenerated on
    the host."""
    import torch
    import mxopt as mx
    ctx = mx.default_context()
    n = 622_329_856
    t = torch.empty(n, dtype=torch.bfloat16, device="cuda")
    seed = mx.synthetic_key(0x5EED0001, 5, 0, 3, 0)
    ctx.fill_synthetic(t, seed, mx.SYNTH_NORMAL, 1e-3)
    rng = np.random.default_rng(0)
    for start in [0, n - 5000] + [int(s) for s in rng.integers(0, n - 5000, 12)]:
        assert_bit_equal(to_host(t[start:start + 5000]), O.synthetic(5000, "bf16", seed, O.SYNTH_NORMAL, 1e-3, first_index=start),
                         f"slice at {start}")
    std = float(t.float().std())
    assert abs(std - 1e-3) < 2e-5
