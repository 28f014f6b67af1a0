"""Whole-step parity on small seeded GGJT models: HIP path (through lv_step_begin) against the CPU checker.

Logit tolerance is the one the path is specified with: 1e-2 max-abs and 1e-3 relative to the largest logit;
greedy tokens must be identical.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

ABS_TOL, REL_TOL = 1e-2, 1e-3


def _check_logits(got, want):
    err = np.max(np.abs(got - want))
    assert err <= ABS_TOL, err
    assert err <= REL_TOL * np.max(np.abs(want)), (err, np.max(np.abs(want)))


@pytest.mark.parametrize("name", ["tiny_q4", "tiny_q8", "small_q4"])
@pytest.mark.parametrize("graph", [True, False])
def test_greedy_decode_matches_oracle(lva, orc, ctx, tiny_models, name, graph):
    path = tiny_models[name]
    om = orc.Model(path)
    osess = orc.Session(om, 128)
    model = lva.Model(ctx, path)
    sess = lva.Session(model, 128)
    sess.use_graph(graph)
    vocab = om.hp["vocab"]
    prompt = lva.synth_tokens(8, 3, vocab, seed=0)

    want = osess.eval(prompt)                 # the reference evaluates a prompt as one batch
    sess.begin(prompt, 0)
    got = sess.logits()
    _check_logits(got, want)
    pos = len(prompt)
    for step in range(32):
        tok_o = orc.greedy(want)
        tok_g = sess.argmax()
        assert tok_g == tok_o == int(np.argmax(got)), f"step {step}"
        want = osess.eval([tok_o])
        sess.begin([tok_g], pos)
        got = sess.logits()
        _check_logits(got, want)
        pos += 1
    # layer 0 sees identical inputs on both sides, so its cache rows agree except where the two fp32
    # summation orders fall on different sides of an fp16 rounding boundary: rare, and then by one ulp
    for which in (0, 1):
        g, o = sess.kv(0, which, pos), osess.kv(0, which, pos)
        assert np.mean(g != o) < 1e-2
        gf, of = g.view(np.float16).astype(np.float32), o.view(np.float16).astype(np.float32)
        assert np.max(np.abs(gf - of)) <= np.max(np.abs(of)) * 2.0 ** -10
    sess.close(); model.close(); osess.close(); om.close()


def test_prompt_as_batch_equals_token_by_token(lva, ctx, tiny_models):
    model = lva.Model(ctx, tiny_models["tiny_q4"])
    a, b = lva.Session(model, 128), lva.Session(model, 128)
    prompt = lva.synth_tokens(12, 3, 512, seed=3)
    a.begin(prompt, 0)
    la = a.logits()
    for i, t in enumerate(prompt):
        b.begin([t], i)
        lb = b.logits()
    assert np.array_equal(la, lb)
    for l in range(2):
        assert np.array_equal(a.kv(l, 0, 12), b.kv(l, 0, 12))
        assert np.array_equal(a.kv(l, 1, 12), b.kv(l, 1, 12))
    a.close(); b.close(); model.close()


def test_reserve_keeps_rows_and_zero_fills(lva, ctx, tiny_models):
    model = lva.Model(ctx, tiny_models["tiny_q4"])
    s = lva.Session(model, 128)
    prompt = lva.synth_tokens(20, 3, 512, seed=4)
    s.begin(prompt, 0)
    before = s.logits()
    k_before = s.kv(1, 0, 128)
    assert not np.any(k_before[20:])            # untouched rows are zero
    s.reserve(256)
    k_after = s.kv(1, 0, 256)
    assert np.array_equal(k_after[:128], k_before) and not np.any(k_after[128:])
    # decoding continues identically after the resize
    ref = lva.Session(model, 256)
    ref.begin(prompt, 0)
    assert np.array_equal(ref.logits(), before)
    nxt = int(np.argmax(before))
    s.begin([nxt], 20)
    ref.begin([nxt], 20)
    assert np.array_equal(s.logits(), ref.logits())
    s.close(); ref.close(); model.close()


def test_kv_write_restores_a_session(lva, ctx, tiny_models):
    model = lva.Model(ctx, tiny_models["tiny_q8"])
    a = lva.Session(model, 128)
    prompt = lva.synth_tokens(9, 3, 512, seed=5)
    a.begin(prompt, 0)
    la = a.logits()
    nxt = int(np.argmax(la))
    b = lva.Session(model, 128)
    for l in range(2):
        b.kv_write(l, 0, a.kv(l, 0, 9))
        b.kv_write(l, 1, a.kv(l, 1, 9))
    a.begin([nxt], 9)
    b.begin([nxt], 9)
    assert np.array_equal(a.logits(), b.logits())
    a.close(); b.close(); model.close()


def test_trace_buffers_match_oracle(lva, orc, ctx, tiny_models):
    path = tiny_models["tiny_q4"]
    om = orc.Model(path)
    osess = orc.Session(om, 128)
    model = lva.Model(ctx, path)
    s = lva.Session(model, 128)
    s.trace_enable(True)
    # nothing recorded yet: no rows; the last-row read gives the buffers' initial zeros
    assert s.trace_rows() == 0 and s.trace_all(0, lva.TRACE_OUT).shape == (0, om.hp["dim"])
    assert np.all(s.trace(0, lva.TRACE_OUT) == 0.0) and np.all(s.trace(1, lva.TRACE_ATTN) == 0.0)
    prompt = lva.synth_tokens(5, 3, 512, seed=6)
    osess.eval(prompt)
    s.begin(prompt, 0)
    s.wait()
    for layer in range(2):
        for which in range(5):
            got, want = s.trace(layer, which), osess.trace(layer, which)
            assert got.shape == want.shape
            assert np.max(np.abs(got - want)) <= 1e-4 * max(1.0, np.max(np.abs(want))), (layer, which)
        # attn_result: the softmax weights of the last row, [backlog][heads]; rows behind its position hold exact zeros
        got, want = s.trace(layer, lva.TRACE_ATTN).reshape(128, -1), osess.trace(layer, orc.TR_ATTN).reshape(128, -1)
        assert got.shape == want.shape == (128, om.hp["heads"])
        assert np.all(got[5:] == 0.0) and np.all(want[5:] == 0.0)
        assert np.max(np.abs(got - want)) <= 1e-5 and np.allclose(got.sum(axis=0), 1.0, atol=1e-5)
    # every row of the step is kept (llava_layer_session_data.cpp:80-85): row z is what a step of the first z + 1 tokens leaves
    assert s.trace_rows() == 5
    for z in range(5):
        oz = orc.Session(om, 128)
        oz.eval(prompt[:z + 1])
        for layer in range(2):
            for which in range(6):
                got, want = s.trace_all(layer, which, z, 1)[0], oz.trace(layer, which)
                assert got.shape == want.shape
                assert np.max(np.abs(got - want)) <= 1e-4 * max(1.0, np.max(np.abs(want))), (z, layer, which)
            a = s.trace_all(layer, lva.TRACE_ATTN, z, 1)[0].reshape(128, -1)
            assert np.all(a[z + 1:] == 0.0) and np.allclose(a.sum(axis=0), 1.0, atol=1e-5)
        oz.close()
    assert np.array_equal(s.trace_all(1, lva.TRACE_FF)[4], s.trace(1, lva.TRACE_FF))
    with pytest.raises(lva.LvError):
        s.trace_all(0, lva.TRACE_OUT, 3, 3)                   # rows 3..5 of a step of five
    # one more token: the weights now cover six rows; a larger backlog keeps the layout [backlog][heads]
    tok = orc.greedy(osess.eval([7]))
    s.begin([7], 5); s.wait()
    assert s.trace_rows() == 1
    s.reserve(256)
    assert np.all(s.trace(0, lva.TRACE_ATTN) == 0.0)          # a fresh buffer of the new size
    s.begin([tok], 6); s.wait()
    o2 = orc.Session(om, 256)
    o2.eval(list(prompt) + [7, tok])
    got, want = s.trace(1, lva.TRACE_ATTN).reshape(256, -1), o2.trace(1, orc.TR_ATTN).reshape(256, -1)
    assert np.all(got[7:] == 0.0) and np.max(np.abs(got - want)) <= 1e-5
    o2.close()
    s.close(); model.close(); osess.close(); om.close()


def test_step_api_state_errors(lva, ctx, tiny_models):
    model = lva.Model(ctx, tiny_models["tiny_q4"])
    s = lva.Session(model, 128)
    lib = ctx.lib
    toks = np.array([5], dtype=np.uint32)
    p = toks.ctypes.data_as(lva.C.c_void_p)
    out = np.empty(512, dtype=np.float32)
    assert lib.lv_logits_read(s.h, out.ctypes.data_as(lva.C.c_void_p)) == -4      # nothing computed yet
    assert lib.lv_step_begin(s.h, p, 1, 128) == -5                                 # past the backlog
    bad = np.array([512], dtype=np.uint32)
    assert lib.lv_step_begin(s.h, bad.ctypes.data_as(lva.C.c_void_p), 1, 0) == -5  # token id out of range
    assert lib.lv_step_begin(s.h, p, 1, 0) == 0
    assert lib.lv_step_begin(s.h, p, 1, 1) == -4                                   # previous step not waited for
    assert lib.lv_step_wait(s.h) == 0
    assert lib.lv_step_begin(s.h, p, 1, 1) == 0
    assert lib.lv_session_reserve(s.h, 256) == -4                                  # in flight
    assert lib.lv_step_wait(s.h) == 0
    s.close(); model.close()


WIDE_SHAPES = {   # the shape classes the persistent decode kernel is compiled for, cut down to 2 layers and a small vocabulary
    "7b_q4_0": dict(wtype="q4_0", dim=4096, heads=32, ff=11008),
    "7b_q8_0": dict(wtype="q8_0", dim=4096, heads=32, ff=11008),
    "13b_q4_0": dict(wtype="q4_0", dim=5120, heads=40, ff=13824),
    "13b_q8_0": dict(wtype="q8_0", dim=5120, heads=40, ff=13824),
}


@pytest.fixture(scope="module", params=list(WIDE_SHAPES))
def wide_model(request, lva, tmp_path_factory):
    """LLaMA-7B / 13B layer shapes with 2 layers and a small vocabulary"""
    cfg = dict(WIDE_SHAPES[request.param])
    wtype = lva.LV_Q4_0 if cfg.pop("wtype") == "q4_0" else lva.LV_Q8_0
    p = str(tmp_path_factory.mktemp("wide") / f"wide_{request.param}.ggml")
    lva.write_model(p, wtype=wtype, seed=9, vocab=2048, layers=2, **cfg)
    return p


def test_persistent_kernel_matches_oracle_and_operator_path(lva, orc, ctx, wide_model):
    om = orc.Model(wide_model)
    osess = orc.Session(om, 128)
    model = lva.Model(ctx, wide_model)
    pk, ops = lva.Session(model, 128), lva.Session(model, 128)
    assert pk.path() == lva.PATH_PERSISTENT          # chosen automatically for this shape
    ops.set_path(lva.PATH_KERNELS)
    prompt = lva.synth_tokens(8, 3, 2048, seed=1)
    want = osess.eval(prompt)
    pk.begin(prompt, 0)                               # a short prompt: one persistent launch per token
    ops.begin(prompt, 0)
    got_pk, got_ops = pk.logits(), ops.logits()
    _check_logits(got_pk, want)
    pos = len(prompt)
    for step in range(24):
        tok = orc.greedy(want)
        assert pk.argmax() == tok == ops.argmax(), f"step {step}"
        want = osess.eval([tok])
        pk.begin([tok], pos)
        ops.begin([tok], pos)
        got_pk, got_ops = pk.logits(), ops.logits()
        _check_logits(got_pk, want)
        _check_logits(got_ops, want)
        assert np.max(np.abs(got_pk - got_ops)) <= 3e-4 * np.max(np.abs(want))   # two fp32 summation orders
        pos += 1
    # both paths left the same cache behind (up to fp16 rounding of differently ordered fp32 sums)
    for layer in range(2):
        for which in (0, 1):
            a, b = pk.kv(layer, which, pos), ops.kv(layer, which, pos)
            af, bf = a.view(np.float16).astype(np.float32), b.view(np.float16).astype(np.float32)
            assert np.max(np.abs(af - bf)) <= np.max(np.abs(bf)) * 2.0 ** -9
    pk.close(); ops.close(); model.close(); osess.close(); om.close()


def test_persistent_kernel_is_deterministic_and_rearms(lva, ctx, wide_model):
    """Same tokens twice from scratch give bit-identical logits (fixed summation order, hand-over buffers re-armed
    between tokens), also when another session's steps are interleaved."""
    model = lva.Model(ctx, wide_model)
    a, b = lva.Session(model, 128), lva.Session(model, 128)
    toks = lva.synth_tokens(20, 3, 2048, seed=2)
    la, lb = [], []
    for i, t in enumerate(toks):
        a.begin([t], i)
        la.append(a.logits())
        b.begin([t], i)
        lb.append(b.logits())
    assert all(np.array_equal(x, y) for x, y in zip(la, lb))
    # rewind: decode the last 5 tokens again over the same cache rows
    for i in range(15, 20):
        a.begin([toks[i]], i)
        assert np.array_equal(a.logits(), la[i])
    a.close(); b.close(); model.close()


def test_persistent_kernel_hands_over_alike_inside_an_xcd_and_at_device_scope(lva, ctx, wide_model):
    """a head's q, k, v rows and partial sums travel through the XCD's L2 where the launch allows it, through memory otherwise:
    only the transport differs, so the logits are the same bits; with the switch off no launch may take the short way"""
    model = lva.Model(ctx, wide_model)
    a, b = lva.Session(model, 128), lva.Session(model, 128)
    assert not a.xcd_handover()                          # no persistent step yet
    b.set_xcd_handover(False)
    toks = lva.synth_tokens(12, 3, 2048, seed=4)
    inside = 0
    for i, t in enumerate(toks):
        a.begin([t], i)
        la = a.logits()
        inside += a.xcd_handover()
        b.begin([t], i)
        lb = b.logits()
        assert not b.xcd_handover()
        assert np.array_equal(la, lb), i
    print("steps that handed over inside an XCD:", inside, "of", len(toks))
    a.close(); b.close(); model.close()


def test_persistent_kernel_refused_for_other_shapes(lva, ctx, tiny_models):
    model = lva.Model(ctx, tiny_models["tiny_q4"])
    s = lva.Session(model, 128)
    assert s.path() == lva.PATH_GRAPH
    assert ctx.lib.lv_session_set_path(s.h, lva.PATH_PERSISTENT) == -1
    s.close(); model.close()


@pytest.mark.parametrize("wname,tname", [("q4_0", "q4_0"), ("q8_0", "q8_0"), ("q4_0", "q8_0")])
def test_quantised_embedding_table_all_paths(lva, orc, ctx, tmp_path, wname, tname):
    """files converted from real checkpoints quantise tok_embeddings like the matrices (llava_buffer.cpp:339-401 dequantises
    the token's row per step); the persistent kernel reads rows from an fp32 expansion made at upload, the operator
    chain dequantises the row on the device: both against the oracle, which dequantises the row on the host"""
    wt = {"q4_0": lva.LV_Q4_0, "q8_0": lva.LV_Q8_0}
    p = str(tmp_path / "qtok.ggml")
    lva.write_model(p, wtype=wt[wname], tok_type=wt[tname], seed=12, vocab=2048, layers=2, dim=4096, heads=32, ff=11008)
    om = orc.Model(p)
    osess = orc.Session(om, 128)
    model = lva.Model(ctx, p)
    pk, ops = lva.Session(model, 128), lva.Session(model, 128)
    assert pk.path() == lva.PATH_PERSISTENT
    ops.set_path(lva.PATH_GRAPH)
    prompt = lva.synth_tokens(5, 3, 2048, seed=2)
    want = osess.eval(prompt)
    pk.begin(prompt, 0); ops.begin(prompt, 0)
    pos = len(prompt)
    for step in range(6):
        _check_logits(pk.logits(), want)
        _check_logits(ops.logits(), want)
        tok = orc.greedy(want)
        assert pk.argmax() == tok == ops.argmax(), step
        want = osess.eval([tok])
        pk.begin([tok], pos); ops.begin([tok], pos)
        pos += 1
    pk.close(); ops.close(); model.close(); osess.close(); om.close()


def test_persistent_kernel_gives_up_a_wait_and_the_step_can_be_repeated(lva, orc, ctx, wide_model):
    """failure path: with the poll bound set to 1 the workgroups stop waiting for each other at once; the kernel still
    runs to its end (nothing hangs), the step is reported as failed, and the same step issued again with the default
    bound gives the oracle's result"""
    om = orc.Model(wide_model)
    osess = orc.Session(om, 128)
    model = lva.Model(ctx, wide_model)
    s = lva.Session(model, 128)
    assert s.path() == lva.PATH_PERSISTENT
    prompt = lva.synth_tokens(4, 3, 2048, seed=3)
    want = osess.eval(prompt)
    s.begin(prompt, 0)
    _check_logits(s.logits(), want)
    tok = orc.greedy(want)
    s.set_wait_limit(1)
    s.begin([tok], 4)
    with pytest.raises(lva.LvError):
        s.wait()
    s.set_wait_limit(0)
    want = osess.eval([tok])
    s.begin([tok], 4)                 # the same cache row again
    _check_logits(s.logits(), want)
    assert s.argmax() == orc.greedy(want)
    s.close(); model.close(); osess.close(); om.close()


def test_two_expired_waits_in_a_row_move_the_session_to_the_graph_path(lva, orc, ctx, wide_model):
    """with the poll bound at 1 every step of the persistent kernel fails; after the second failure in a row the session
    reports the graph path and the same step, issued a third time with the bound unchanged, gives the oracle's result
    there; choosing the persistent path again by hand brings the kernel back"""
    om = orc.Model(wide_model)
    osess = orc.Session(om, 128)
    model = lva.Model(ctx, wide_model)
    s = lva.Session(model, 128)
    prompt = lva.synth_tokens(4, 3, 2048, seed=4)
    want = osess.eval(prompt)
    s.begin(prompt, 0)
    _check_logits(s.logits(), want)
    tok = orc.greedy(want)
    want = osess.eval([tok])
    s.set_wait_limit(1)
    for attempt in range(2):
        assert s.path() == lva.PATH_PERSISTENT
        s.begin([tok], 4)
        with pytest.raises(lva.LvError):
            s.wait()
    assert s.path() == lva.PATH_GRAPH
    s.begin([tok], 4)                 # the bound is still 1: this step does not run the persistent kernel
    _check_logits(s.logits(), want)
    assert s.argmax() == orc.greedy(want)
    tok = orc.greedy(want)
    want = osess.eval([tok])
    s.begin([tok], 5)                 # graph replay
    _check_logits(s.logits(), want)
    s.set_wait_limit(0)
    s.set_path(lva.PATH_PERSISTENT)
    assert s.path() == lva.PATH_PERSISTENT
    tok = orc.greedy(want)
    want = osess.eval([tok])
    s.begin([tok], 6)
    _check_logits(s.logits(), want)
    assert s.argmax() == orc.greedy(want)
    # one failure, one success, one failure: not two in a row, the kernel stays
    s.set_path(lva.PATH_AUTO)
    for limit, fails in [(1, True), (0, False), (1, True)]:
        s.set_wait_limit(limit)
        s.begin([tok], 6)
        if fails:
            with pytest.raises(lva.LvError):
                s.wait()
        else:
            _check_logits(s.logits(), want)
    assert s.path() == lva.PATH_PERSISTENT
    s.close(); model.close(); osess.close(); om.close()


@pytest.mark.parametrize("vocab", [259, 2049])
def test_vocabulary_sizes_that_do_not_divide_over_the_workgroups(lva, orc, ctx, tmp_path, vocab):
    """the output matrix is split over 256 workgroups; 2049 rows leave the last ones short, 259 leave most of them
    without a row (their 'best logit' must not be mistaken for one): logits and greedy pick on both decode paths"""
    p = str(tmp_path / "odd.ggml")
    lva.write_model(p, wtype=lva.LV_Q4_0, seed=5, vocab=vocab, layers=2, dim=4096, heads=32, ff=11008)
    om = orc.Model(p)
    osess = orc.Session(om, 128)
    model = lva.Model(ctx, p)
    pk, ops = lva.Session(model, 128), lva.Session(model, 128)
    assert pk.path() == lva.PATH_PERSISTENT
    ops.set_path(lva.PATH_GRAPH)
    prompt = lva.synth_tokens(5, 3, vocab, seed=2)
    want = osess.eval(prompt)
    pk.begin(prompt, 0); ops.begin(prompt, 0)
    pos = len(prompt)
    for step in range(4):
        _check_logits(pk.logits(), want)
        _check_logits(ops.logits(), want)
        tok = orc.greedy(want)
        assert pk.argmax() == tok == ops.argmax(), step
        want = osess.eval([tok])
        pk.begin([tok], pos); ops.begin([tok], pos)
        pos += 1
    pk.close(); ops.close(); model.close(); osess.close(); om.close()


def test_persistent_kernel_up_to_the_last_cache_row(lva, orc, ctx, wide_model):
    """every position of a 128-row cache, the last one included (chunk boundaries of the attention phase move with the
    position); a step past the end is refused"""
    om = orc.Model(wide_model)
    osess = orc.Session(om, 128)
    model = lva.Model(ctx, wide_model)
    s = lva.Session(model, 128)
    assert s.path() == lva.PATH_PERSISTENT
    prompt = lva.synth_tokens(3, 3, 2048, seed=4)
    want = osess.eval(prompt)
    s.begin(prompt, 0)
    pos = len(prompt)
    while True:
        _check_logits(s.logits(), want)
        tok = orc.greedy(want)
        assert s.argmax() == tok, pos
        if pos == 128:
            break
        want = osess.eval([tok])
        s.begin([tok], pos)
        pos += 1
    with pytest.raises(lva.LvError):
        s.begin([tok], 128)
    s.close(); model.close(); osess.close(); om.close()


def _rows_match(got, want):
    tol = 1e-2 + 1e-3 * np.abs(want)
    assert got.shape == want.shape
    assert np.all(np.abs(got - want) <= tol), float(np.max(np.abs(got - want) / tol))


@pytest.mark.parametrize("name", ["tiny_q4", "tiny_q8", "pair_q8"])
def test_logits_of_every_row_of_a_step(lva, orc, ctx, tiny_models, name):
    """the reference's output_probs holds the logits of every row of a step (llava_session.cpp:49-79,
    llava_command_buffer.cpp:38-39); with lv_session_set_all_logits a step keeps them: a 5-token step (token by token on the
    operator chain), a 20-token step behind it (the batched path: final norm of all rows, output matrix on the matrix
    cores) and a one-token step (the captured graph), each row against the checker's row"""
    om = orc.Model(tiny_models[name])
    osess = orc.Session(om, 128)
    model = lva.Model(ctx, tiny_models[name])
    s = lva.Session(model, 128)
    with pytest.raises(lva.LvError):
        s.begin([5], 0)
        s.logits_rows(0, 1)                  # the switch is off: nothing was kept
    s.wait()
    s.keep_all_logits()
    toks = lva.synth_tokens(26, 3, om.hp["vocab"], seed=21)
    pos = 0
    for n in (5, 20, 1):
        want = osess.eval(toks[pos:pos + n], all_rows=True)
        s.begin(toks[pos:pos + n], pos)
        _rows_match(s.logits_rows(0, n), want)
        _rows_match(s.logits()[None, :], want[-1:])          # the last row is still where lv_logits_read finds it
        if n > 2:
            _rows_match(s.logits_rows(1, n - 2), want[1:n - 1])
            with pytest.raises(lva.LvError):
                s.logits_rows(1, n)          # past the end of the step
        pos += n
    s.keep_all_logits(False)
    s.begin(toks[:3], 0)
    with pytest.raises(lva.LvError):
        s.logits_rows(0, 1)
    s.close(); model.close(); osess.close(); om.close()


def test_logits_of_every_row_on_the_persistent_kernel(lva, orc, ctx, wide_model):
    """a short step on the persistent kernel is one launch per token, and every launch computes its logits: kept row by row"""
    om = orc.Model(wide_model)
    osess = orc.Session(om, 128)
    model = lva.Model(ctx, wide_model)
    s = lva.Session(model, 128)
    assert s.path() == lva.PATH_PERSISTENT
    s.keep_all_logits()
    toks = lva.synth_tokens(9, 3, 2048, seed=22)
    want = osess.eval(toks[:6], all_rows=True)
    s.begin(toks[:6], 0)
    _rows_match(s.logits_rows(0, 6), want)
    assert s.argmax() == orc.greedy(want[-1])
    want = osess.eval(toks[6:7], all_rows=True)
    s.begin(toks[6:7], 6)
    _rows_match(s.logits_rows(0, 1), want)
    _rows_match(s.logits()[None, :], want)
    s.close(); model.close(); osess.close(); om.close()
