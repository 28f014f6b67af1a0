"""Parity of every HIP kernel against the CPU checker, through the C-ABI (include/llava_hip.h).

Tolerances: dequantisation and the fp16 cache append are bit-exact.  Floating-point kernels reduce in a
different order than the shaders' trees, so they are compared with an fp32 reassociation bound:
|got - want| <= 1e-5 * sum_k |w_k x_k| (a few hundred ulps of the largest partial sum), far inside the
1e-2 abs / 1e-3 rel budget the logits have.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _abs_dot_bound(orc, blocks, ftype, rows, cols, x):
    w = orc.dequant(blocks, ftype, rows * cols).reshape(rows, cols).astype(np.float64)
    return np.abs(w) @ np.abs(x.astype(np.float64)).T  # [rows][batch]


@pytest.mark.parametrize("ftype_name", ["q4_0", "q8_0"])
@pytest.mark.parametrize("rows,cols", [(8, 32), (64, 4096), (40, 11008), (24, 5120), (16, 13824), (100, 96), (33, 2048 + 64)])
def test_dequant_bit_exact(lva, orc, ctx, ftype_name, rows, cols):
    ftype = lva.LV_Q4_0 if ftype_name == "q4_0" else lva.LV_Q8_0
    blocks = lva.synth_quant(ftype, rows, cols, seed=11)
    # adversarial scales: zero, subnormal, largest normal, negative, and every code value somewhere
    stride = 18 if ftype == lva.LV_Q4_0 else 34
    b = blocks.reshape(-1, stride)
    special = np.array([0x0000, 0x0001, 0x03FF, 0x0400, 0x7BFF, 0x8001, 0xBC00, 0x3C00], dtype=np.uint16)
    n_sp = min(len(special), b.shape[0])
    b[:n_sp, 0:2] = special[:n_sp].view(np.uint8).reshape(-1, 2)
    b[-1, 2:] = (np.arange(stride - 2) * 17 % 256).astype(np.uint8)
    m = ctx.matrix(blocks, ftype, rows, cols)
    dst = ctx.alloc(rows * cols * 4)
    lva.check(ctx.lib.lv_kernel_dequant(ctx.h, m, 0, rows, dst))
    got = ctx.to_host(dst, (rows * cols,), np.float32)
    want = orc.dequant(blocks, ftype, rows * cols)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # a row window
    if rows > 3:
        lva.check(ctx.lib.lv_kernel_dequant(ctx.h, m, 2, 1, dst))
        got1 = ctx.to_host(dst, (cols,), np.float32)
        assert np.array_equal(got1.view(np.uint32), want.reshape(rows, cols)[2].view(np.uint32))
    ctx.free(dst)
    ctx.matrix_free(m)


@pytest.mark.parametrize("ftype_name", ["q4_0", "q8_0"])
@pytest.mark.parametrize("rows,cols,batch", [
    (64, 4096, 1), (40, 11008, 1), (48, 5120, 1), (24, 13824, 1), (37, 96, 3), (8, 32, 2), (19, 2048 + 64, 1), (256, 256, 1),
    # 2048 rows and more: the streaming kernel (256 workgroups, x in LDS); ragged row counts, 1..12 column slabs per
    # row (24576 columns is the widest row the library accepts)
    (2048, 32, 1), (2049, 2048 + 64, 2), (4096, 4096, 1), (2500, 11008, 1), (2051, 13824, 3), (2048, 24576, 1),
    # the decode shapes the isolated-kernel figures are quoted on, whole: down projection (with accumulate = the fused
    # residual add) and output matrix of the 7B model, and the 13B down projection
    (4096, 11008, 1), (32000, 4096, 1), (5120, 13824, 1),
])
@pytest.mark.parametrize("accumulate", [False, True])
def test_gemv_matches_oracle(lva, orc, ctx, ftype_name, rows, cols, batch, accumulate):
    ftype = lva.LV_Q4_0 if ftype_name == "q4_0" else lva.LV_Q8_0
    blocks = lva.synth_quant(ftype, rows, cols, seed=21)
    x = lva.synth_normal(batch, cols, seed=22)
    prev = lva.synth_normal(batch, rows, seed=23)
    m = ctx.matrix(blocks, ftype, rows, cols)
    dx = ctx.to_device(x)
    dout = ctx.to_device(prev)
    lva.check(ctx.lib.lv_kernel_gemv(ctx.h, dout, m, dx, batch, int(accumulate)))
    got = ctx.to_host(dout, (batch, rows), np.float32)
    want = orc.gemv(blocks, ftype, rows, cols, x, out=prev if accumulate else None, accumulate=accumulate)
    bound = 1e-5 * _abs_dot_bound(orc, blocks, ftype, rows, cols, x).T + 1e-7
    ratio = float(np.max(np.abs(got.astype(np.float64) - want) / bound))
    assert ratio <= 1.0, ratio
    for p in (dx, dout):
        ctx.free(p)
    ctx.matrix_free(m)


@pytest.mark.parametrize("ftype_name", ["q4_0", "q8_0"])
@pytest.mark.parametrize("rows,cols,batch", [(96, 4096, 1), (64, 5120, 1), (50, 256, 2), (11008, 4096, 1), (2077, 5120, 2), (2048, 96, 1)])
def test_gemv_silu_matches_oracle(lva, orc, ctx, ftype_name, rows, cols, batch):
    ftype = lva.LV_Q4_0 if ftype_name == "q4_0" else lva.LV_Q8_0
    w3 = lva.synth_quant(ftype, rows, cols, seed=31, tensor_id=3)
    w1 = lva.synth_quant(ftype, rows, cols, seed=31, tensor_id=1)
    x = lva.synth_normal(batch, cols, seed=32)
    m3, m1 = ctx.matrix(w3, ftype, rows, cols), ctx.matrix(w1, ftype, rows, cols)
    dx, dout = ctx.to_device(x), ctx.alloc(batch * rows * 4)
    lva.check(ctx.lib.lv_kernel_gemv_silu(ctx.h, dout, m3, m1, dx, batch))
    got = ctx.to_host(dout, (batch, rows), np.float32)
    want = orc.gemv_silu(w3, w1, ftype, rows, cols, x)
    # error of a product of two dot products: |r2| d1 + 1.1 |r1| d2 (silu' <= 1.1), d = 1e-5 * sum |w x|
    r1 = orc.gemv(w3, ftype, rows, cols, x).astype(np.float64)
    r2 = orc.gemv(w1, ftype, rows, cols, x).astype(np.float64)
    d1 = 1e-5 * _abs_dot_bound(orc, w3, ftype, rows, cols, x).T
    d2 = 1e-5 * _abs_dot_bound(orc, w1, ftype, rows, cols, x).T
    bound = np.abs(r2) * d1 + 1.1 * np.abs(r1) * d2 + 1e-6
    ratio = float(np.max(np.abs(got.astype(np.float64) - want) / bound))
    assert ratio <= 1.0, ratio
    for p in (dx, dout):
        ctx.free(p)
    ctx.matrix_free(m3)
    ctx.matrix_free(m1)


@pytest.mark.parametrize("dim,batch", [(4096, 1), (5120, 1), (256, 3), (96, 2)])
def test_normalize_matches_oracle(lva, orc, ctx, dim, batch):
    x = lva.synth_normal(batch, dim, seed=41) + np.float32(0.75)  # non-zero mean: centred variance matters
    w = lva.synth_normal(1, dim, seed=42, sigma=0.02)[0]
    dx, dw, dout = ctx.to_device(x), ctx.to_device(w), ctx.alloc(batch * dim * 4)
    lva.check(ctx.lib.lv_kernel_normalize(ctx.h, dout, dx, dw, dim, batch))
    got = ctx.to_host(dout, (batch, dim), np.float32)
    want = orc.normalize(x, w)
    assert np.max(np.abs(got - want)) <= 2e-6 * np.max(np.abs(want)) + 1e-9
    for p in (dx, dw, dout):
        ctx.free(p)


@pytest.mark.parametrize("dim,batch,pos,backlog", [(4096, 1, 0, 128), (4096, 1, 127, 128), (256, 5, 3, 16), (5120, 2, 100, 256)])
def test_kv_append_bit_exact(lva, orc, ctx, dim, batch, pos, backlog):
    rows = lva.synth_normal(batch, dim, seed=51, sigma=3.0)
    rows[0, :8] = [0.0, -0.0, 65504.0, 65520.0, 1e-8, 5.9604645e-8, 2.9802322e-8, -70000.0]  # edges of fp16
    rows[0, 8:12] = np.array([0x3F801000, 0x3F803000, 0x3F801001, 0x387FC000], dtype=np.uint32).view(np.float32)  # ties
    cache_host = np.full((backlog, dim), 0x1234, dtype=np.uint16)
    dcache, drows = ctx.to_device(cache_host), ctx.to_device(rows)
    lva.check(ctx.lib.lv_kernel_kv_append(ctx.h, dcache, drows, pos, dim, batch, backlog))
    got = ctx.to_host(dcache, (backlog, dim), np.uint16)
    want = orc.kv_append(cache_host.copy(), rows, pos)
    assert np.array_equal(got, want)
    with np.errstate(over="ignore"):
        assert np.array_equal(got[pos:pos + batch], rows.astype(np.float16).view(np.uint16))
    for p in (dcache, drows):
        ctx.free(p)


@pytest.mark.parametrize("heads,rot,backlog,pos,batch", [
    (32, 128, 128, 0, 1), (32, 128, 128, 40, 1), (32, 128, 128, 127, 1), (4, 64, 128, 77, 1), (16, 32, 64, 63, 1),
    (40, 128, 256, 200, 1), (32, 128, 512, 511, 1), (4, 64, 128, 10, 4), (2, 128, 256, 250, 3),
    # 16 rows and more: the kernels of a prompt batch (16-bit matrix-core products of split operands)
    # (the oracle's tree sums want a power-of-two backlog, as the shaders do)
    (4, 128, 256, 37, 100), (8, 64, 256, 0, 150), (5, 32, 128, 3, 120), (3, 128, 64, 0, 16), (2, 128, 512, 283, 17),
    (2, 64, 32, 5, 20), (40, 128, 512, 0, 512),
])
def test_attention_matches_oracle(lva, orc, ctx, heads, rot, backlog, pos, batch):
    dim = heads * rot
    rng = np.random.default_rng(61)
    n_rows = pos + batch
    kc = np.zeros((backlog, dim), dtype=np.uint16)
    vc = np.zeros((backlog, dim), dtype=np.uint16)
    kc[:n_rows] = (rng.standard_normal((n_rows, dim)) * 0.7).astype(np.float16).view(np.uint16)
    vc[:n_rows] = rng.standard_normal((n_rows, dim)).astype(np.float16).view(np.uint16)
    # rows past the written ones hold junk that must be ignored (a rewound session leaves such rows behind)
    kc[n_rows:] = np.float16(9.0).view(np.uint16)
    vc[n_rows:] = np.float16(-7.0).view(np.uint16)
    q = (rng.standard_normal((batch, dim)) * 0.7).astype(np.float32)
    dk, dv, dq, dout = ctx.to_device(kc), ctx.to_device(vc), ctx.to_device(q), ctx.alloc(batch * dim * 4)
    for _ in range(2):  # twice: the split counters must come back to zero
        lva.check(ctx.lib.lv_kernel_attention(ctx.h, dout, dk, dv, dq, pos, backlog, heads, rot, batch))
        got = ctx.to_host(dout, (batch, dim), np.float32)
        want = orc.attention(kc, vc, q, pos, heads, rot)
        assert np.max(np.abs(got - want)) < 2e-5 * max(1.0, np.max(np.abs(want)))
    for p in (dk, dv, dq, dout):
        ctx.free(p)


def test_errors_are_reported_not_fatal(lva, ctx):
    lib = ctx.lib
    m = lva.C.c_void_p()
    blocks = np.zeros(18 * 4, dtype=np.uint8)
    assert lib.lv_matrix_upload(ctx.h, blocks.ctypes.data_as(lva.C.c_void_p), lva.LV_Q4_0, 3, 4, 33, lva.C.byref(m)) == -1
    assert b"shape" in lib.lv_last_error()
    assert lib.lv_matrix_upload(ctx.h, blocks.ctypes.data_as(lva.C.c_void_p), lva.LV_Q4_0, 2, 4, 32, lva.C.byref(m)) == -1    # versions 1 and 3 only
    assert b"version" in lib.lv_last_error()
    assert lib.lv_matrix_upload(ctx.h, blocks.ctypes.data_as(lva.C.c_void_p), 3, 3, 4, 32, lva.C.byref(m)) == -1
    assert lib.lv_kernel_normalize(ctx.h, None, None, None, 16, 1) == -1
    assert lib.lv_kernel_kv_append(ctx.h, lva.C.c_void_p(8), lva.C.c_void_p(8), 128, 16, 1, 128) == -5
