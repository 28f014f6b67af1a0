"""Batched prompt path: the matrix-core GEMM (lv_kernel_gemm) against the oracle's fp32 GEMV at the same bound the
one-token GEMV is held to, and whole prompts evaluated as one batch against the oracle and against token-by-token
evaluation (reference: the *_batch shader variants and llava_session.cpp:197-229 with several pending tokens)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _abs_dot_bound(orc, blocks, ftype, rows, cols, x):
    w = np.abs(orc.dequant(blocks, ftype, rows * cols).reshape(rows, cols).astype(np.float64))
    return (w @ np.abs(x.astype(np.float64)).T).T      # [batch][rows]


@pytest.mark.parametrize("ftype_name", ["q4_0", "q8_0"])
@pytest.mark.parametrize("rows,cols,batch,accumulate", [
    (64, 32, 5, False),          # one quant block per row: K padded to 64 with zeros, a handful of tokens
    (128, 64, 128, False),       # half a row tile, one token tile, two K steps (the shortest K the pipeline sees)
    (256, 4096, 130, False),     # a second, almost empty token tile
    (704, 256, 17, True),        # rows not a multiple of the tile, residual add
    (96, 1376, 200, False),      # K = 43 blocks, padded to 44 with zeros; fewer rows than a tile
    (4096, 4096, 512, True),     # the 7B attention shape at a 512-token prompt batch (K cut in four slices, then reduced)
    (5120, 3168, 512, True),     # 80 tiles for 256 CUs: K cut in three slices of 17, 17 and 15.5 steps of 64, then reduced
    (8264, 160, 400, True),      # 33 row tiles (five of the eight XCDs get one more), ragged in rows, K and tokens
])
def test_gemm_matches_oracle(lva, orc, ctx, ftype_name, rows, cols, batch, accumulate):
    ftype = lva.LV_Q4_0 if ftype_name == "q4_0" else lva.LV_Q8_0
    blocks = lva.synth_quant(ftype, rows, cols, seed=61)
    x = lva.synth_normal(batch, cols, seed=62)
    x[0, :4] = [0.0, 1.0, -1000.25, 1e-7]              # zero, one, a large and a tiny activation
    prev = lva.synth_normal(batch, rows, seed=63)
    m = ctx.matrix(blocks, ftype, rows, cols)
    dx, dout = ctx.to_device(x), ctx.to_device(prev)
    lva.check(ctx.lib.lv_kernel_gemm(ctx.h, dout, m, dx, batch, int(accumulate)))
    got = ctx.to_host(dout, (batch, rows), np.float32)
    want = orc.gemv(blocks, ftype, rows, cols, x, out=prev if accumulate else None, accumulate=accumulate)
    bound = 1e-5 * _abs_dot_bound(orc, blocks, ftype, rows, cols, x) + 1e-7
    ratio = float(np.max(np.abs(got.astype(np.float64) - want) / bound))
    assert ratio <= 1.0, ratio
    # the one-token kernel on the same rows: each is within the bound of the oracle, so within 1.5 bounds of each other
    # (the fp16 halves carry 22 bits of an activation, fp32 carries 24)
    dout2 = ctx.to_device(prev)
    nb = min(batch, 64)
    lva.check(ctx.lib.lv_kernel_gemv(ctx.h, dout2, m, dx, nb, int(accumulate)))
    one = ctx.to_host(dout2, (batch, rows), np.float32)[:nb]
    assert float(np.max(np.abs(one.astype(np.float64) - got[:nb]) / bound[:nb])) <= 1.5
    for p in (dx, dout, dout2):
        ctx.free(p)
    ctx.matrix_free(m)


@pytest.mark.parametrize("scale", [1e-6, 1e-3, 3e4])
def test_gemm_holds_its_bound_at_any_activation_scale(lva, orc, ctx, scale):
    """the activation halves are written scaled by a power of two per token row, so the low half of an element stays a normal
    fp16 number whether the row is of order 1e-6 or 3e4 (unscaled, everything below 0.125 would lose its low bits and
    anything above 65504 would overflow); rows of very different sizes in one batch"""
    rows, cols, batch = 512, 1024, 96
    blocks = lva.synth_quant(lva.LV_Q8_0, rows, cols, seed=71)
    x = lva.synth_normal(batch, cols, seed=72) * np.float32(scale)
    x[1] *= np.float32(1e3)                               # one row a thousand times larger than its neighbours
    x[2] = 0.0                                            # an all-zero row
    m = ctx.matrix(blocks, lva.LV_Q8_0, rows, cols)
    dx, dout = ctx.to_device(x), ctx.alloc(batch * rows * 4)
    lva.check(ctx.lib.lv_kernel_gemm(ctx.h, dout, m, dx, batch, 0))
    got = ctx.to_host(dout, (batch, rows), np.float32)
    want = orc.gemv(blocks, lva.LV_Q8_0, rows, cols, x)
    bound = 1e-5 * _abs_dot_bound(orc, blocks, lva.LV_Q8_0, rows, cols, x)
    assert np.all(got[2] == 0.0)
    live = bound > 0
    assert float(np.max(np.abs(got.astype(np.float64) - want)[live] / bound[live])) <= 1.0
    for p in (dx, dout):
        ctx.free(p)
    ctx.matrix_free(m)


def test_gemm_special_inputs(lva, orc, ctx):
    """all codes 8 -> exact zeros; one-hot activations -> exact dequantised columns"""
    rows, cols, batch = 128, 128, 128
    blocks = lva.synth_quant(lva.LV_Q4_0, rows, cols, seed=64)
    m = ctx.matrix(blocks, lva.LV_Q4_0, rows, cols)
    x = np.zeros((batch, cols), dtype=np.float32)
    x[np.arange(batch), np.arange(batch)] = 1.0
    dx, dout = ctx.to_device(x), ctx.alloc(batch * rows * 4)
    lva.check(ctx.lib.lv_kernel_gemm(ctx.h, dout, m, dx, batch, 0))
    got = ctx.to_host(dout, (batch, rows), np.float32)
    w = orc.dequant(blocks, lva.LV_Q4_0, rows * cols).reshape(rows, cols)
    assert np.array_equal(got, w.T)                      # hi + lo halves restore every weight exactly
    for p in (dx, dout):
        ctx.free(p)
    ctx.matrix_free(m)


def test_gemm_calls_in_a_row_keep_their_workspace(lva, orc, ctx):
    """lv_kernel_gemm keeps a matrix's prompt copy with the matrix and the activation workspace with the context: calls of
    different sizes and on different matrices queued without a wait between them must not disturb each other, and a matrix
    may be destroyed right after its call"""
    shapes = [(lva.LV_Q8_0, 512, 1024, 96), (lva.LV_Q4_0, 256, 4096, 130), (lva.LV_Q8_0, 512, 1024, 17), (lva.LV_Q4_0, 4096, 4096, 512)]
    mats, keep = {}, []
    for i, (ftype, rows, cols, batch) in enumerate(shapes):
        key = (ftype, rows, cols)
        if key not in mats:
            blocks = lva.synth_quant(ftype, rows, cols, seed=90 + i)
            mats[key] = (blocks, ctx.matrix(blocks, ftype, rows, cols))
        blocks, m = mats[key]
        x = lva.synth_normal(batch, cols, seed=95 + i)
        dx, dout = ctx.to_device(x), ctx.alloc(batch * rows * 4)
        lva.check(ctx.lib.lv_kernel_gemm(ctx.h, dout, m, dx, batch, 0))     # queued; nothing waits here
        keep.append((blocks, ftype, rows, cols, batch, x, dx, dout))
    for blocks, m in mats.values():
        ctx.matrix_free(m)
    for blocks, ftype, rows, cols, batch, x, dx, dout in keep:
        got = ctx.to_host(dout, (batch, rows), np.float32)
        want = orc.gemv(blocks, ftype, rows, cols, x)
        bound = 1e-5 * _abs_dot_bound(orc, blocks, ftype, rows, cols, x) + 1e-7
        assert float(np.max(np.abs(got.astype(np.float64) - want) / bound)) <= 1.0, (rows, cols, batch)
        ctx.free(dx)
        ctx.free(dout)


def test_gemm_refuses_a_matrix_of_another_context(lva, ctx):
    """the prompt copy lv_kernel_gemm makes is freed with the matrix after a wait for the matrix's context: a launch queued
    on another context's stream could outlive it, so that call is refused"""
    other = lva.Context(0)
    blocks = lva.synth_quant(lva.LV_Q8_0, 128, 128, seed=3)
    m = ctx.matrix(blocks, lva.LV_Q8_0, 128, 128)
    dx, dout = other.to_device(lva.synth_normal(16, 128, seed=4)), other.alloc(16 * 128 * 4)
    with pytest.raises(lva.LvError) as err:
        lva.check(other.lib.lv_kernel_gemm(other.h, dout, m, dx, 16, 0))
    assert err.value.code == -1 and "another context" in str(err.value)       # LV_ERR_ARG
    other.free(dx); other.free(dout)
    ctx.matrix_free(m)
    other.close()


@pytest.mark.parametrize("name,n_prompt", [("tiny_q4", 40), ("tiny_q8", 130), ("small_q4", 77), ("pair_q4", 150), ("pair_q8", 33)])
def test_prompt_as_one_batch_matches_oracle(lva, orc, ctx, tiny_models, name, n_prompt):
    path = tiny_models[name]
    om = orc.Model(path)
    vocab, layers = om.hp["vocab"], om.hp["layers"]
    osess = orc.Session(om, 256)
    model = lva.Model(ctx, path)
    a, b = lva.Session(model, 256), lva.Session(model, 256)
    prompt = lva.synth_tokens(n_prompt, 3, vocab, seed=9)
    want = osess.eval(prompt)
    a.begin(prompt, 0)                                   # one step: the matrix-core path
    for i, t in enumerate(prompt):                       # token by token: the one-token kernels
        b.begin([int(t)], i)
        b.wait()
    la, lb = a.logits(), b.logits()
    tol = 1e-2 + 1e-3 * np.abs(want)
    assert np.all(np.abs(la - want) <= tol) and np.all(np.abs(lb - want) <= tol)
    assert float(np.max(np.abs(la - lb))) <= 1e-4 * max(1.0, float(np.max(np.abs(lb))))
    for layer in range(layers):
        for which in (0, 1):
            ra = a.kv(layer, which, n_prompt).view(np.float16).astype(np.float32)
            rb = b.kv(layer, which, n_prompt).view(np.float16).astype(np.float32)
            # different summation orders flip the last fp16 bit of some entries, never more than that
            assert np.mean(ra != rb) < 0.5 and np.max(np.abs(ra - rb)) <= 2e-3 * float(np.max(np.abs(rb)))
    # greedy continuation from the batched cache
    pos, logits = n_prompt, want
    for step in range(16):
        tok = orc.greedy(logits)
        assert a.argmax() == tok, step
        logits = osess.eval(np.array([tok], dtype=np.uint32))
        a.begin([tok], pos)
        pos += 1
    a.close(); b.close(); model.close(); osess.close(); om.close()


def test_prompt_batch_of_a_model_wider_than_the_fused_norm_pass(lva, orc, ctx, tmp_path):
    """rows of 8256 floats: the pass that sums the K slices, normalises and splits in one kernel holds at most 8192 per
    row in registers, so this model takes the three separate kernels, with three K slices pending between the layers"""
    path = str(tmp_path / "wide.ggml")
    lva.write_model(path, wtype=lva.LV_Q4_0, seed=21, vocab=320, layers=2, dim=8256, heads=129, ff=96)
    om = orc.Model(path)
    osess = orc.Session(om, 64)
    model = lva.Model(ctx, path)
    s = lva.Session(model, 64)
    prompt = lva.synth_tokens(24, 3, 320, seed=22)
    want = osess.eval(prompt)
    s.begin(prompt, 0)
    got = s.logits()
    assert np.all(np.abs(got - want) <= 1e-2 + 1e-3 * np.abs(want)), float(np.max(np.abs(got - want)))
    assert s.argmax() == orc.greedy(want)
    s.close(); model.close(); osess.close(); om.close()


def test_second_batch_appends_behind_the_first(lva, orc, ctx, tiny_models):
    """two batched steps in a row (prompt, then a long addition): rows of the second see the cache of the first"""
    path = tiny_models["tiny_q4"]
    om = orc.Model(path)
    osess = orc.Session(om, 256)
    model = lva.Model(ctx, path)
    s = lva.Session(model, 256)
    toks = lva.synth_tokens(100, 3, om.hp["vocab"], seed=10)
    osess.eval(toks[:60])
    want = osess.eval(toks[60:])
    s.begin(toks[:60], 0)
    s.wait()
    s.begin(toks[60:], 60)
    got = s.logits()
    assert np.all(np.abs(got - want) <= 1e-2 + 1e-3 * np.abs(want))
    assert s.argmax() == orc.greedy(want)
    s.close(); model.close(); osess.close(); om.close()


def test_prompt_batch_of_a_width_that_64_does_not_divide(lva, orc, ctx, tmp_path):
    """dim 96 = 3 heads of 32: the GEMM pads K to 128, so the attention result goes through the split kernel (which writes
    the zero columns) instead of being written as halves by the attention kernel; ff 160 cannot be paired either"""
    path = str(tmp_path / "odd.ggml")
    lva.write_model(path, wtype=lva.LV_Q8_0, seed=23, vocab=320, layers=2, dim=96, heads=3, ff=160)
    om = orc.Model(path)
    osess = orc.Session(om, 64)
    model = lva.Model(ctx, path)
    s = lva.Session(model, 64)
    prompt = lva.synth_tokens(40, 3, 320, seed=24)
    want = osess.eval(prompt)
    s.begin(prompt, 0)
    got = s.logits()
    assert np.all(np.abs(got - want) <= 1e-2 + 1e-3 * np.abs(want)), float(np.max(np.abs(got - want)))
    assert s.argmax() == orc.greedy(want)
    s.close(); model.close(); osess.close(); om.close()


def test_prompt_batch_in_a_cache_whose_length_64_does_not_divide(lva, ctx, tiny_models):
    """a backlog of 100 rows: the attention planes are padded to 128 rows, the cache is not; the batch must agree with the
    same tokens evaluated one by one (the oracle's tree sums want a power-of-two backlog, so it cannot referee here)"""
    model = lva.Model(ctx, tiny_models["pair_q8"])
    a, b = lva.Session(model, 100), lva.Session(model, 100)
    prompt = lva.synth_tokens(90, 3, 512, seed=25)
    a.begin(prompt[:50], 0)
    a.wait()
    a.begin(prompt[50:], 50)
    for i, t in enumerate(prompt):
        b.begin([int(t)], i)
        b.wait()
    la, lb = a.logits(), b.logits()
    assert float(np.max(np.abs(la - lb))) <= 1e-4 * max(1.0, float(np.max(np.abs(lb))))
    for layer in range(2):
        for which in (0, 1):
            ra = a.kv(layer, which, 90).view(np.float16).astype(np.float32)
            rb = b.kv(layer, which, 90).view(np.float16).astype(np.float32)
            assert np.max(np.abs(ra - rb)) <= 2e-3 * float(np.max(np.abs(rb)))
    a.close(); b.close(); model.close()


def test_prompt_batch_whose_last_round_of_gate_up_tiles_is_cut_along_k(lva, orc, ctx, tmp_path):
    """ff 8448 = 66 row tiles of the paired gate/up copy at 4 token tiles: 64 fill a round, the last 2 are multiplied in two K
    halves by a second launch and pass through SwiGLU in a kernel of their own; dim 2048 gives the 32 K steps that needs"""
    path = str(tmp_path / "tail.ggml")
    lva.write_model(path, wtype=lva.LV_Q4_0, seed=31, vocab=320, layers=1, dim=2048, heads=16, ff=8448)
    om = orc.Model(path)
    osess = orc.Session(om, 512)
    model = lva.Model(ctx, path)
    a, b = lva.Session(model, 512), lva.Session(model, 512)
    prompt = lva.synth_tokens(390, 3, 320, seed=32)
    want = osess.eval(prompt)
    a.begin(prompt, 0)                       # 4 token tiles: the cut applies
    got = a.logits()
    assert np.all(np.abs(got - want) <= 1e-2 + 1e-3 * np.abs(want)), float(np.max(np.abs(got - want)))
    assert a.argmax() == orc.greedy(want)
    b.begin(prompt[:256], 0)                 # 2 token tiles each: one launch, no cut
    b.wait()
    b.begin(prompt[256:], 256)
    lb = b.logits()
    assert float(np.max(np.abs(got - lb))) <= 1e-4 * max(1.0, float(np.max(np.abs(lb))))
    a.close(); b.close(); model.close(); osess.close(); om.close()
