"""lv_kernel_attention_static: the attention entry point that allocates nothing (its rotation table, partial sums and
split counters live in a fixed work area every device holds) against lv_kernel_attention, through the C-ABI.

Two calls in a row on the same context, the second with a smaller input: the work area keeps the first call's contents,
so stale table rows, partial sums or counters would show in the second result.  Both entry points run the same attention
kernel over tables computed from the same fp32 angles (one on the host, one on the device, cos/sin in double rounded to
fp32), so the outputs are compared at the floating-point bar of the other attention tests (2e-5 of the largest output)
and, beside that, against the CPU checker.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _case(lva, orc, ctx, heads, rot, backlog, pos, batch, seed):
    dim = heads * rot
    rng = np.random.default_rng(seed)
    n_rows = pos + batch
    kc = np.zeros((backlog, dim), dtype=np.uint16)
    vc = np.zeros((backlog, dim), dtype=np.uint16)
    kc[:n_rows] = (rng.standard_normal((n_rows, dim)) * 0.7).astype(np.float16).view(np.uint16)
    vc[:n_rows] = rng.standard_normal((n_rows, dim)).astype(np.float16).view(np.uint16)
    kc[n_rows:] = np.float16(9.0).view(np.uint16)
    vc[n_rows:] = np.float16(-7.0).view(np.uint16)
    q = (rng.standard_normal((batch, dim)) * 0.7).astype(np.float32)
    dk, dv, dq = ctx.to_device(kc), ctx.to_device(vc), ctx.to_device(q)
    d_ref, d_new = ctx.alloc(batch * dim * 4), ctx.alloc(batch * dim * 4)
    lva.check(ctx.lib.lv_kernel_attention(ctx.h, d_ref, dk, dv, dq, pos, backlog, heads, rot, batch))
    ref = ctx.to_host(d_ref, (batch, dim), np.float32)
    lva.check(ctx.lib.lv_kernel_attention_static(ctx.h, d_new, dk, dv, dq, pos, backlog, heads, rot, batch))
    got = ctx.to_host(d_new, (batch, dim), np.float32)
    want = orc.attention(kc, vc, q, pos, heads, rot)
    for p in (dk, dv, dq, d_ref, d_new):
        ctx.free(p)
    tol = 2e-5 * max(1.0, float(np.max(np.abs(want))))
    assert np.max(np.abs(got - ref)) < tol
    assert np.max(np.abs(got - want)) < tol


def test_static_attention_two_calls_in_a_row(lva, orc, ctx):
    # large first (32 heads of 128, 2048 rows: the whole rotation table, 32 splits per head), then smaller in every
    # dimension (other head size, fewer heads, shorter cache, a batch of 3)
    _case(lva, orc, ctx, heads=32, rot=128, backlog=2048, pos=2047, batch=1, seed=71)
    _case(lva, orc, ctx, heads=4, rot=64, backlog=256, pos=130, batch=3, seed=72)
    # and a larger one again after the small one
    _case(lva, orc, ctx, heads=40, rot=128, backlog=512, pos=300, batch=1, seed=73)


def _free_device_bytes():
    """hipMemGetInfo of the runtime the library is linked against (already loaded into this process)"""
    import ctypes as C
    hip = C.CDLL("libamdhip64.so")
    free, total = C.c_size_t(), C.c_size_t()
    assert hip.hipMemGetInfo(C.byref(free), C.byref(total)) == 0
    return free.value


def test_static_attention_leaves_device_memory_as_it_was(lva, ctx):
    """what the entry point is for: calls that allocate nothing.  Free device memory (hipMemGetInfo) is read before and after
    calls of three different sizes, each the first of its size on this context (so a workspace that grew with the input, as
    lv_kernel_attention's does, would show), and is the same to the byte."""
    rng = np.random.default_rng(5)
    bufs = []
    for heads, rot, backlog, pos, batch in ((32, 128, 2048, 2047, 1), (8, 64, 1024, 1000, 4), (40, 128, 1024, 700, 2)):
        dim = heads * rot
        kc = (rng.standard_normal((backlog, dim)) * 0.5).astype(np.float16).view(np.uint16)
        q = rng.standard_normal((batch, dim)).astype(np.float32)
        bufs.append((ctx.to_device(kc), ctx.to_device(kc), ctx.to_device(q), ctx.alloc(batch * dim * 4), pos, backlog, heads, rot, batch))
    ctx.sync()
    before = _free_device_bytes()
    for dk, dv, dq, dout, pos, backlog, heads, rot, batch in bufs:
        lva.check(ctx.lib.lv_kernel_attention_static(ctx.h, dout, dk, dv, dq, pos, backlog, heads, rot, batch))
        ctx.sync()
        assert _free_device_bytes() == before
    for dk, dv, dq, dout, *_ in bufs:
        for p in (dk, dv, dq, dout):
            ctx.free(p)


def test_static_attention_rejects_sizes_beyond_the_work_area(lva, ctx):
    lib = ctx.lib
    p = lva.C.c_void_p(256)          # never dereferenced: the call is refused on its sizes
    assert lib.lv_kernel_attention_static(ctx.h, p, p, p, p, 0, 4096, 32, 128, 1) == -5       # rotation table
    assert b"static work area" in lib.lv_last_error()
    assert lib.lv_kernel_attention_static(ctx.h, p, p, p, p, 0, 2048, 64, 128, 1) == -5       # partial sums
    assert lib.lv_kernel_attention_static(ctx.h, p, p, p, p, 0, 64, 64, 32, 5) == -5          # counters
    assert lib.lv_kernel_attention_static(ctx.h, p, p, p, p, 0, 64, 4, 48, 1) == -1           # head size
