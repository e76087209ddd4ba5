"""The machine probes behind `bench.py --ceiling` (csrc/probe.hip) run and report sane values.
They have no oracle: what is checked is that every entry point launches, that bounded waits end,
and that what they store has the stated meaning."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _ok(orn, rc, what):
    assert rc == 0, f"{what}: {orn.lib().ornith_last_error().decode()}"


def test_probes_run_and_store_what_they_say(orn, ctx):
    lib = orn.lib()
    sink = ctx.alloc(256)
    # launches that do nothing, from the stream and from a graph
    _ok(orn, lib.ornith_probe_empty(ctx.h, 64, 256, 1, 10), "probe_empty")
    ms = C.c_float(-1.0)
    _ok(orn, lib.ornith_probe_empty_graph(ctx.h, 64, 256, 0, 10, C.byref(ms)), "probe_empty_graph")
    assert 0.0 < ms.value < 50.0
    # stream-only launches and a long read over a small buffer
    buf = ctx.alloc(8 << 20)
    buf.zero()
    _ok(orn, lib.ornith_probe_stream(ctx.h, buf.ptr, C.c_size_t(8 << 20), 64, 4, C.c_size_t(1024), sink.ptr, 5), "probe_stream")
    _ok(orn, lib.ornith_probe_read(ctx.h, buf.ptr, C.c_size_t(8 << 20), sink.ptr), "probe_read")
    assert lib.ornith_probe_stream(ctx.h, buf.ptr, C.c_size_t(1 << 20), 4096, 16, C.c_size_t(1024), sink.ptr, 1) != 0   # does not fit
    # die ids
    n = 256
    xo = ctx.alloc(n * 4)
    _ok(orn, lib.ornith_probe_xcc(ctx.h, n, xo.ptr), "probe_xcc")
    ids = xo.download(np.uint32, (n,))
    assert ids.max() < 8 and len(np.unique(ids)) == 8
    # a word between workgroups: seen with agent-scope loads; the plain-load poll runs out (bounded) and says so
    flag, out4 = ctx.alloc(4096), ctx.alloc(64)
    flag.zero()
    _ok(orn, lib.ornith_probe_handoff(ctx.h, flag.ptr, out4.ptr, 0, 1, 0), "probe_handoff")
    o = out4.download(np.int64, (4,))
    assert o[1] > o[0] > 0 and 0 <= o[2] < 8 and 0 <= o[3] < 8
    _ok(orn, lib.ornith_probe_handoff(ctx.h, C.c_void_p(flag.ptr.value + 256), out4.ptr, 0, 8, 2), "probe_handoff")
    ctx.sync()
    # one vector instruction at a time
    lib.ornith_probe_valu_name.restype = C.c_char_p
    dx = ctx.to_device(np.array([1e-3, 2e-3, 3e-3, 4e-3], np.float32))
    dp = ctx.to_device(np.full(4, 0x47000007, np.uint32))
    dout = ctx.alloc(8 * 256 * 4)
    assert lib.ornith_probe_valu_count() >= 10
    for op in range(lib.ornith_probe_valu_count()):
        assert lib.ornith_probe_valu_name(op).startswith(b"v_")
        _ok(orn, lib.ornith_probe_valu(ctx.h, op, 8, 16, dx.ptr, dp.ptr, dout.ptr), "probe_valu")
    assert lib.ornith_probe_valu(ctx.h, lib.ornith_probe_valu_count(), 8, 16, dx.ptr, dp.ptr, dout.ptr) != 0
    # kernel arguments: the four stamps of a workgroup do not go backwards, in either form
    didx = ctx.to_device(np.array([3], np.uint32))
    ddata = ctx.alloc(64 << 10)
    ddata.zero()
    dst = ctx.alloc(32 * 32)
    for flat in (0, 1):
        _ok(orn, lib.ornith_probe_kernarg(ctx.h, flat, 32, didx.ptr, ddata.ptr, dst.ptr), "probe_kernarg")
        st = dst.download(np.int64, (32, 4))
        assert np.all(np.diff(st, axis=1) >= 0) and np.all(st[:, 0] > 0), flat
    for b in (sink, buf, xo, flag, out4, dx, dp, dout, didx, ddata, dst):
        b.free()
