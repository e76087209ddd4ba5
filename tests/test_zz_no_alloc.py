"""GPU: the entry point that allocates nothing (ornith_greedy_rows_noalloc) gives the same
tokens and logsumexp bits as ornith_greedy_rows, on two calls in a row (the second over a
smaller input, so whatever the first left in the fixed scratch array must not matter), and
rejects sizes beyond its fixed array."""
import numpy as np
import pytest

import util

pytestmark = pytest.mark.gpu


def _both(ctx, x):
    rows, V = x.shape
    dx = ctx.to_device(x)
    dt, dl = ctx.alloc(rows * 4).zero(), ctx.alloc(rows * 2).zero()
    ctx.greedy_rows(dx, rows, V, dt, dl)
    want_t, want_l = dt.download(np.uint32, (rows,)), dl.download(np.uint16, (rows,))
    dt.zero(); dl.zero()
    ctx.greedy_rows_noalloc(dx, rows, V, dt, dl)
    got_t, got_l = dt.download(np.uint32, (rows,)), dl.download(np.uint16, (rows,))
    for b in (dx, dt, dl):
        b.free()
    return (want_t, want_l), (got_t, got_l)


def test_noalloc_greedy_rows_equals_greedy_rows_twice(orn, ctx):
    rng = np.random.default_rng(11)
    for rows, V in ((8, 248320), (3, 5000)):          # second call: fewer rows, fewer chunks
        x = util.bf16_normal(rng, (rows, V), 1.0)
        x[0] = util.f32_to_bf16(np.round(util.bf16_to_f32(x[0]) * 2) / 2)   # heavy ties
        (wt, wl), (gt, gl) = _both(ctx, x)
        assert np.array_equal(gt, wt), (rows, V, gt, wt)
        assert np.array_equal(gl, wl), (rows, V)
        # and the oracle agrees with both
        ot, ol = np.empty(rows, np.uint32), np.empty(rows, np.uint16)
        util.oracle().orc_greedy_rows(util.p(x), rows, V, util.p(ot), util.p(ol))
        assert np.array_equal(gt, ot) and np.array_equal(gl, ol)


def test_noalloc_rejects_sizes_beyond_its_array(orn, ctx):
    d = ctx.alloc(1024)
    for rows, V in ((9, 1000), (1, 262145), (0, 10)):
        with pytest.raises(orn.OrnithError, match="greedy_rows_noalloc"):
            ctx.greedy_rows_noalloc(d, rows, V, d, None)
    d.free()
