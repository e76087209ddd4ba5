"""GPU parity: greedy selection over the full vocabulary vs the oracle (tokens bit-exact)."""
import numpy as np
import pytest

import util
from util import oracle, p

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("V", [248320, 32768, 4096, 1000])
def test_greedy_and_argmax_rows(orn, ctx, V):
    rng = np.random.default_rng(V)
    rows = 4
    x = util.bf16_normal(rng, (rows, V), 1.0)   # unit-variance logits: many bf16 ties near the top
    x[1] = util.f32_to_bf16(np.round(util.bf16_to_f32(x[1]) * 2) / 2)  # heavy ties
    x[2, :] = x[2, 0]                            # everything tied -> token 0
    want = np.empty(rows, np.uint32); wl = np.empty(rows, np.uint16); wraw = np.empty(rows, np.uint32)
    oracle().orc_greedy_rows(p(x), rows, V, p(want), p(wl))
    oracle().orc_argmax_rows(p(x), rows, V, p(wraw))
    dx, dt, dl = ctx.to_device(x), ctx.alloc(rows * 4), ctx.alloc(rows * 2)
    ctx.greedy_rows(dx, rows, V, dt, dl)
    assert np.array_equal(dl.download(np.uint16, (rows,)), wl)
    assert np.array_equal(dt.download(np.uint32, (rows,)), want)
    ctx.argmax_rows(dx, rows, V, dt)
    assert np.array_equal(dt.download(np.uint32, (rows,)), wraw)
    assert want[2] == 0 and wraw[2] == 0
    for b in (dx, dt, dl): b.free()
