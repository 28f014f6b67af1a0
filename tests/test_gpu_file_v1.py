"""File version 1 (fp32 block scales, q4_0 nibbles interleaved as elements 2j / 2j+1; reference: ggml_file.cpp:95-122 for
the sizes, llava_buffer.cpp:66-71 and 193-224 for the split into a codes plane and a scale plane) through the kernels
and through whole models.  Version-1 data is made from version-3 data by tests/ggjt_builder.py, so every result also
has a version-3 twin with the same element values."""
import numpy as np
import pytest

import ggjt_builder as gb

pytestmark = pytest.mark.gpu


def _ftype(lva, name):
    return lva.LV_Q4_0 if name == "q4_0" else lva.LV_Q8_0


def _v1_blocks(lva, ftype, rows, cols, seed):
    """version-1 blocks whose scales use all 24 bits of an fp32 mantissa (a version-3 file cannot hold such scales)"""
    v3 = lva.synth_quant(ftype, rows, cols, seed=seed)
    v1 = gb.blocks_to_v1(v3, gb.Q4_0 if ftype == lva.LV_Q4_0 else gb.Q8_0).reshape(-1, 20 if ftype == lva.LV_Q4_0 else 36)
    rng = np.random.default_rng(seed)
    scale = v1[:, :4].copy().view(np.float32).reshape(-1)
    scale *= (1.0 + rng.uniform(-0.01, 0.01, scale.shape)).astype(np.float32)
    v1[:, :4] = scale.view(np.uint8).reshape(-1, 4)
    return v1.reshape(-1)


def _abs_dot_bound(orc, blocks, ftype, rows, cols, x):
    w = np.abs(orc.dequant(blocks, ftype, rows * cols, file_version=1).reshape(rows, cols).astype(np.float64))
    return (w @ np.abs(x.astype(np.float64)).T).T      # [batch][rows]


@pytest.mark.parametrize("ftype_name", ["q4_0", "q8_0"])
@pytest.mark.parametrize("rows,cols", [(8, 32), (64, 4096), (40, 11008), (100, 96), (33, 2048 + 64)])
def test_v1_dequant_bit_exact(lva, orc, ctx, ftype_name, rows, cols):
    ftype = _ftype(lva, ftype_name)
    blocks = _v1_blocks(lva, ftype, rows, cols, seed=71)
    b = blocks.reshape(-1, 20 if ftype == lva.LV_Q4_0 else 36)
    # scales no fp16 can hold: zero, an fp32 subnormal, the largest finite value, negatives, 1 + 2^-23
    special = np.array([0x00000000, 0x00000001, 0x7F7FFFFF, 0x80000001, 0xBF800001, 0x3F800001, 0x33800000], dtype=np.uint32)
    n_sp = min(len(special), b.shape[0])
    b[:n_sp, :4] = special[:n_sp].view(np.uint8).reshape(-1, 4)
    b[-1, 4:] = (np.arange(b.shape[1] - 4) * 17 % 256).astype(np.uint8)     # every nibble value, in both halves of a byte
    m = ctx.matrix(blocks, ftype, rows, cols, file_version=1)
    dst = ctx.alloc(rows * cols * 4)
    lva.check(ctx.lib.lv_kernel_dequant(ctx.h, m, 0, rows, dst))
    got = ctx.to_host(dst, (rows * cols,), np.float32)
    want = orc.dequant(blocks, ftype, rows * cols, file_version=1)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    ctx.free(dst)
    ctx.matrix_free(m)


@pytest.mark.parametrize("ftype_name", ["q4_0", "q8_0"])
@pytest.mark.parametrize("rows,cols,batch", [(64, 4096, 1), (37, 96, 3), (19, 2048 + 64, 1), (2049, 2048 + 64, 2), (4096, 4096, 1),
                                             (2500, 11008, 1)])
@pytest.mark.parametrize("accumulate", [False, True])
def test_v1_gemv_matches_oracle(lva, orc, ctx, ftype_name, rows, cols, batch, accumulate):
    ftype = _ftype(lva, ftype_name)
    blocks = _v1_blocks(lva, ftype, rows, cols, seed=72)
    x = lva.synth_normal(batch, cols, seed=73)
    prev = lva.synth_normal(batch, rows, seed=74)
    m = ctx.matrix(blocks, ftype, rows, cols, file_version=1)
    dx, dout = ctx.to_device(x), ctx.to_device(prev)
    lva.check(ctx.lib.lv_kernel_gemv(ctx.h, dout, m, dx, batch, int(accumulate)))
    got = ctx.to_host(dout, (batch, rows), np.float32)
    want = orc.gemv(blocks, ftype, rows, cols, x, out=prev if accumulate else None, accumulate=accumulate, file_version=1)
    bound = 1e-5 * _abs_dot_bound(orc, blocks, ftype, rows, cols, x) + 1e-7
    ratio = float(np.max(np.abs(got.astype(np.float64) - want) / bound))
    assert ratio <= 1.0, ratio
    for p in (dx, dout):
        ctx.free(p)
    ctx.matrix_free(m)


@pytest.mark.parametrize("ftype_name", ["q4_0", "q8_0"])
@pytest.mark.parametrize("rows,cols,batch", [(96, 4096, 1), (50, 256, 2), (11008, 4096, 1)])
def test_v1_gemv_silu_matches_oracle(lva, orc, ctx, ftype_name, rows, cols, batch):
    ftype = _ftype(lva, ftype_name)
    w3 = _v1_blocks(lva, ftype, rows, cols, seed=75)
    w1 = _v1_blocks(lva, ftype, rows, cols, seed=76)
    x = lva.synth_normal(batch, cols, seed=77)
    m3, m1 = ctx.matrix(w3, ftype, rows, cols, file_version=1), ctx.matrix(w1, ftype, rows, cols, file_version=1)
    dx, dout = ctx.to_device(x), ctx.alloc(batch * rows * 4)
    lva.check(ctx.lib.lv_kernel_gemv_silu(ctx.h, dout, m3, m1, dx, batch))
    got = ctx.to_host(dout, (batch, rows), np.float32)
    want = orc.gemv_silu(w3, w1, ftype, rows, cols, x, file_version=1)
    # error of a product of two dot products: |r2| d1 + 1.1 |r1| d2 (silu' <= 1.1), d = 1e-5 * sum |w x|
    r1 = orc.gemv(w3, ftype, rows, cols, x, file_version=1).astype(np.float64)
    r2 = orc.gemv(w1, ftype, rows, cols, x, file_version=1).astype(np.float64)
    d1 = 1e-5 * _abs_dot_bound(orc, w3, ftype, rows, cols, x)
    d2 = 1e-5 * _abs_dot_bound(orc, w1, ftype, rows, cols, x)
    bound = np.abs(r2) * d1 + 1.1 * np.abs(r1) * d2 + 1e-6
    assert float(np.max(np.abs(got.astype(np.float64) - want) / bound)) <= 1.0
    for p in (dx, dout):
        ctx.free(p)
    ctx.matrix_free(m3); ctx.matrix_free(m1)


@pytest.mark.parametrize("ftype_name", ["q4_0", "q8_0"])
@pytest.mark.parametrize("rows,cols,batch,accumulate", [(128, 64, 128, False), (704, 256, 17, True), (96, 1376, 200, False),
                                                        (4096, 4096, 256, True)])
def test_v1_gemm_matches_oracle(lva, orc, ctx, ftype_name, rows, cols, batch, accumulate):
    ftype = _ftype(lva, ftype_name)
    blocks = _v1_blocks(lva, ftype, rows, cols, seed=78)
    x = lva.synth_normal(batch, cols, seed=79)
    prev = lva.synth_normal(batch, rows, seed=80)
    m = ctx.matrix(blocks, ftype, rows, cols, file_version=1)
    dx, dout = ctx.to_device(x), ctx.to_device(prev)
    lva.check(ctx.lib.lv_kernel_gemm(ctx.h, dout, m, dx, batch, int(accumulate)))
    got = ctx.to_host(dout, (batch, rows), np.float32)
    want = orc.gemv(blocks, ftype, rows, cols, x, out=prev if accumulate else None, accumulate=accumulate, file_version=1)
    bound = 1e-5 * _abs_dot_bound(orc, blocks, ftype, rows, cols, x) + 1e-7
    assert float(np.max(np.abs(got.astype(np.float64) - want) / bound)) <= 1.0
    for p in (dx, dout):
        ctx.free(p)
    ctx.matrix_free(m)


def _check_logits(got, want):
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    assert np.all(err <= 1e-2 + 1e-3 * np.abs(want)), float(err.max())


@pytest.fixture(scope="module")
def v1_models(lva, tiny_models, tmp_path_factory):
    d = tmp_path_factory.mktemp("v1")
    out = {}
    for name in ("tiny_q4", "tiny_q8"):
        out[name] = str(d / f"{name}_v1.ggml")
        gb.convert_to_v1(tiny_models[name], out[name])
    # the widths of the 7B model, with a quantised embedding table as converted checkpoints have
    src = str(d / "wide_v3.ggml")
    lva.write_model(src, wtype=lva.LV_Q4_0, tok_type=lva.LV_Q4_0, seed=14, vocab=2048, layers=2, dim=4096, heads=32, ff=11008)
    out["wide_q4"] = str(d / "wide_v1.ggml")
    gb.convert_to_v1(src, out["wide_q4"])
    out["wide_q4_v3"] = src
    # the same with scales no fp16 holds: what the persistent kernel's fp32-scale tiles are for
    out["wide_q4_jit"] = str(d / "wide_v1_jit.ggml")
    gb.convert_to_v1(src, out["wide_q4_jit"], jitter_seed=5)
    return out


@pytest.mark.parametrize("name,mode", [("tiny_q4", "graph"), ("tiny_q4", "operator"), ("tiny_q8", "graph"), ("tiny_q8", "operator"),
                                       ("wide_q4", "graph"), ("wide_q4", "operator"), ("wide_q4", "persistent"),
                                       ("wide_q4_jit", "persistent"), ("wide_q4_jit", "graph")])
def test_v1_model_greedy_decode_matches_oracle(lva, orc, ctx, v1_models, name, mode):
    path = v1_models[name]
    om = orc.Model(path)
    assert om.hp["file_version"] == 1
    osess = orc.Session(om, 128)
    model = lva.Model(ctx, path)
    sess = lva.Session(model, 128)
    if name.startswith("wide"):
        # 7B layer widths, q4_0: the persistent kernel has a shape class whose tiles carry the fp32 scales of this version
        assert sess.path() == lva.PATH_PERSISTENT
        if mode != "persistent":
            sess.set_path(lva.PATH_GRAPH if mode == "graph" else lva.PATH_KERNELS)
    else:
        assert mode != "persistent" and sess.path() == lva.PATH_GRAPH
        assert ctx.lib.lv_session_set_path(sess.h, lva.PATH_PERSISTENT) == -1
    if mode != "persistent":
        sess.use_graph(mode == "graph")
    vocab = om.hp["vocab"]
    prompt = lva.synth_tokens(8, 3, vocab, seed=0)
    want = osess.eval(prompt)
    sess.begin(prompt, 0)
    got = sess.logits()
    _check_logits(got, want)
    pos = len(prompt)
    for step in range(12):
        tok_o = orc.greedy(want)
        assert sess.argmax() == tok_o == int(np.argmax(got)), f"step {step}"
        want = osess.eval([tok_o])
        sess.begin([tok_o], pos)
        got = sess.logits()
        _check_logits(got, want)
        pos += 1
    assert sess.path() == {"persistent": lva.PATH_PERSISTENT, "graph": lva.PATH_GRAPH, "operator": lva.PATH_KERNELS}[mode]
    sess.close(); model.close(); osess.close(); om.close()


@pytest.mark.parametrize("name", ["tiny_q4", "wide_q4"])
def test_v1_prompt_as_one_batch_matches_oracle(lva, orc, ctx, v1_models, name):
    """40 prompt tokens go through the matrix-core GEMM and the batched attention"""
    path = v1_models[name]
    om = orc.Model(path)
    osess = orc.Session(om, 128)
    model = lva.Model(ctx, path)
    sess = lva.Session(model, 128)
    prompt = lva.synth_tokens(40, 3, om.hp["vocab"], seed=3)
    want = osess.eval(prompt)
    sess.begin(prompt, 0)
    _check_logits(sess.logits(), want)
    assert sess.argmax() == orc.greedy(want)
    sess.close(); model.close(); osess.close(); om.close()


def test_v1_and_v3_twins_give_the_same_logits(lva, ctx, v1_models):
    """the same element values stored both ways: the operator chain computes the same numbers from either file"""
    outs = []
    for key in ("wide_q4_v3", "wide_q4"):
        model = lva.Model(ctx, v1_models[key])
        sess = lva.Session(model, 128)
        sess.set_path(lva.PATH_GRAPH)
        sess.begin(lva.synth_tokens(6, 3, 2048, seed=5), 0)
        outs.append(sess.logits().copy())
        sess.close(); model.close()
    assert np.array_equal(outs[0].view(np.uint32), outs[1].view(np.uint32))
