"""mxopt_hbm_spread_begin / _end: all free device memory is taken in blocks, part of it released at
once, the rest when the window closes; nothing may be left behind and results do not depend on it."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import mxopt_oracle as O
from gpu_util import assert_bit_equal, to_dev, to_host

F = np.float32


def test_spread_window_gives_memory_back_and_changes_no_result():
    import torch
    import mxopt as mx
    ctx = mx.Context()
    torch.cuda.empty_cache()
    free0, total = torch.cuda.mem_get_info()
    rng = np.random.default_rng(3)
    n = 1 << 20
    p, g = rng.normal(0, 0.02, n).astype(F), rng.normal(0, 1e-3, n).astype(F)
    with ctx.hbm_spread(block_bytes=256 << 20, keep_one_in=2):
        inside, _ = torch.cuda.mem_get_info()
        # about half of what was free is held by the window, the other half can be allocated
        assert 0.35 * free0 < inside < 0.65 * free0
        dp, dg = to_dev(p), to_dev(g)
        dm, dv = torch.zeros(n, device="cuda"), torch.zeros(n, device="cuda")
    after, _ = torch.cuda.mem_get_info()
    assert after > free0 - (1 << 30)                      # everything but the four small tensors is back
    t = ctx.table([mx.TensorSpec(p=dp, p_out=dp, g=dg, m=dm, v=dv)])
    ctx.adam(t, mx.adam_hp(1e-3, 0.9, 0.999, 1e-8, 0.01))
    ref = O.AdamW(1e-3, 0.9, 0.999, 1e-8, 0.01)
    assert_bit_equal(to_host(dp), ref.update_single("w", p, g), "parameters allocated inside the window")
    t.close()
    with pytest.raises(mx.InvalidArg, match="at least 2 MiB"):
        with ctx.hbm_spread(block_bytes=4096):
            pass
    with pytest.raises(mx.InvalidArg, match="keep_one_in >= 2"):
        with ctx.hbm_spread(keep_one_in=1):
            pass
    with pytest.raises(mx.InvalidArg, match="too small for this much free memory"):
        with ctx.hbm_spread(block_bytes=2 << 20):
            pass
    assert torch.cuda.mem_get_info()[0] > free0 - (1 << 30)
    ctx.close()
