"""The reference's own runnable case at full size: LLaMA-7B shape, q4_0, seed 0, eight prompt ids pushed as ids
(no BOS, no tokenizer), 32 greedy steps with the backlog left at 128 — GPU (persistent one-launch-per-token kernel)
against the oracle.  Tolerance: logits within 1e-2 absolute + 1e-3 relative of the oracle's, greedy tokens identical.

The model file (4.3 GB) is written once per box into /dev/shm (or /tmp) by the seeded generator and shared with
bench.py; the oracle needs about 0.2 s per token on 16 host threads."""
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

SHAPE = dict(vocab=32000, dim=4096, heads=32, layers=32, ff=11008)


@pytest.fixture(scope="module")
def model_7b(lva):
    base = "/dev/shm" if os.access("/dev/shm", os.W_OK) else "/tmp"
    path = os.path.join(base, "llava_bench_7b_q4_0_seed0.ggml")
    if not os.path.exists(path):
        lva.write_model(path + ".tmp", wtype=lva.LV_Q4_0, seed=0, **SHAPE)
        os.replace(path + ".tmp", path)
    return path


def test_7b_q4_0_prompt_8_then_32_greedy_steps(lva, orc, ctx, model_7b):
    om = orc.Model(model_7b)
    osess = orc.Session(om, 128)
    model = lva.Model(ctx, model_7b)
    s = lva.Session(model, 128)
    assert s.path() == lva.PATH_PERSISTENT, "a 7B q4_0 model on a 256-CU device must take the persistent kernel"
    prompt = lva.synth_tokens(8, 3, SHAPE["vocab"], seed=0)
    want = osess.eval(prompt)
    s.begin(prompt, 0)
    got = s.logits()
    pos, worst = 8, 0.0
    for step in range(32):
        tol = 1e-2 + 1e-3 * np.abs(want)
        assert np.all(np.abs(got - want) <= tol), (step, float(np.max(np.abs(got - want))))
        worst = max(worst, float(np.max(np.abs(got - want))))
        tok = orc.greedy(want)
        assert s.argmax() == tok, step
        want = osess.eval(np.array([tok], dtype=np.uint32))
        s.begin([tok], pos)
        got = s.logits()
        pos += 1
    print(f"max |dlogit| over 33 steps: {worst:.3g}")
    # Cache rows.  A 4096-term fp32 dot product carries a reassociation error of about sqrt(K)*2^-24 * sum|terms|, which
    # at this size is comparable to half an fp16 ulp of the result, so GPU and oracle rows legitimately differ in the
    # last fp16 bit in many places.  Both are therefore measured against an fp64 computation of layer 0's K and V rows:
    # the error allowed is half an fp16 ulp (the rounding) plus 1e-5 * sum|terms| (generous for fp32 accumulation).
    D = SHAPE["dim"]
    toks = np.asarray(prompt, dtype=np.int64)
    emb, _ = om.data("tok_embeddings.weight")
    x = emb.view(np.float32).reshape(SHAPE["vocab"], D)[toks].astype(np.float64)
    w, _ = om.data("layers.0.attention_norm.weight")
    w = w.view(np.float32).astype(np.float64)
    var = np.mean((x - x.mean(axis=1, keepdims=True)) ** 2, axis=1, keepdims=True)
    n = x * w / np.sqrt(var)
    for which, name in ((0, "wk"), (1, "wv")):
        blocks, t = om.data(f"layers.0.attention.{name}.weight")
        W = orc.dequant(blocks, t["ftype"], D * D).reshape(D, D).astype(np.float64)
        exact = n @ W.T
        slack = 1e-5 * (np.abs(n) @ np.abs(W).T)
        half_ulp = np.spacing(np.abs(exact).astype(np.float16)).astype(np.float64) / 2
        for label, rows in (("gpu", s.kv(0, which, 8)), ("oracle", osess.kv(0, which, 8))):
            err = np.abs(rows.view(np.float16).astype(np.float64) - exact)
            assert np.all(err <= half_ulp * 1.001 + slack), (label, name, float(np.max(err - half_ulp - slack)))
    # deeper layers: inputs already differ by fp32 rounding; rows agree within a few fp16 ulps
    for layer in (15, 31):
        for which in (0, 1):
            a = s.kv(layer, which, pos).view(np.float16).astype(np.float32)
            b = osess.kv(layer, which, pos).view(np.float16).astype(np.float32)
            assert np.max(np.abs(a - b)) <= 4e-3 * float(np.max(np.abs(b)))
    s.close(); model.close(); osess.close(); om.close()


def test_7b_operator_chain_agrees_with_persistent_kernel(lva, ctx, model_7b):
    """the two execution paths of the library on the same full-size model: same greedy tokens, logits within tolerance"""
    model = lva.Model(ctx, model_7b)
    a, b = lva.Session(model, 128), lva.Session(model, 128)
    b.set_path(lva.PATH_GRAPH)
    prompt = lva.synth_tokens(8, 3, SHAPE["vocab"], seed=0)
    a.begin(prompt, 0); b.begin(prompt, 0)
    pos = 8
    for step in range(8):
        la, lb = a.logits(), b.logits()
        assert np.all(np.abs(la - lb) <= 1e-2 + 1e-3 * np.abs(lb)), step
        ta, tb = a.argmax(), b.argmax()
        assert ta == tb, step
        a.begin([ta], pos); b.begin([tb], pos)
        pos += 1
    a.close(); b.close(); model.close()


SHAPE_13B = dict(vocab=32000, dim=5120, heads=40, layers=40, ff=13824)


@pytest.mark.parametrize("name,steps", [("7b", 300), ("13b", 150)])
def test_hand_overs_inside_an_xcd_and_at_device_scope_give_the_same_bits_at_full_depth(lva, ctx, model_7b, name, steps):
    """The hand-overs inside a head go through the XCD's L2 with plain stores and non-temporal loads where a launch places the
    head's workgroups on one XCD, at device scope otherwise.  Only the transport differs, so every logit of every step has
    to be the same bits, here over a few hundred steps of the full-depth 7B and 13B q4_0 models (a stale value read through
    the short way would change a logit; a value that never arrives ends the step with an error instead).  Stops at the first
    difference."""
    path = model_7b if name == "7b" else _model_file(lva, "13b_q4_0", lva.LV_Q4_0, 2, SHAPE_13B)
    shape = SHAPE if name == "7b" else SHAPE_13B
    model = lva.Model(ctx, path)
    a, b = lva.Session(model, 512), lva.Session(model, 512)
    b.set_xcd_handover(False)
    tok, inside = 17, 0
    for i in range(steps):
        a.begin([tok], i)
        la = a.logits()
        inside += a.xcd_handover()
        b.begin([tok], i)
        lb = b.logits()
        assert not b.xcd_handover()
        assert np.array_equal(la.view(np.uint32), lb.view(np.uint32)), (name, i)
        tok = a.argmax()
        assert tok == b.argmax() and tok < shape["vocab"]
    print(f"{name}: {inside} of {steps} steps handed over inside an XCD")
    a.close(); b.close(); model.close()


def _model_file(lva, name, wtype, seed, shape):
    base = "/dev/shm" if os.access("/dev/shm", os.W_OK) else "/tmp"
    path = os.path.join(base, f"llava_measure_{name}_seed{seed}.ggml")     # shared with llama-vulkan_amd/measure.py
    if not os.path.exists(path):
        lva.write_model(path + ".tmp", wtype=wtype, seed=seed, **shape)
        os.replace(path + ".tmp", path)
    return path


def test_13b_q4_0_prompt_8_then_8_greedy_steps(lva, orc, ctx):
    """the 13B layer shape at its full depth of 40 layers on the persistent kernel, against the oracle"""
    path = _model_file(lva, "13b_q4_0", lva.LV_Q4_0, 2, SHAPE_13B)
    om = orc.Model(path)
    osess = orc.Session(om, 128)
    model = lva.Model(ctx, path)
    s = lva.Session(model, 128)
    assert s.path() == lva.PATH_PERSISTENT
    prompt = lva.synth_tokens(8, 3, SHAPE_13B["vocab"], seed=2)
    want = osess.eval(prompt)
    s.begin(prompt, 0)
    pos = 8
    for step in range(8):
        got = s.logits()
        assert np.all(np.abs(got - want) <= 1e-2 + 1e-3 * np.abs(want)), (step, float(np.max(np.abs(got - want))))
        tok = orc.greedy(want)
        assert s.argmax() == tok, step
        want = osess.eval(np.array([tok], dtype=np.uint32))
        s.begin([tok], pos)
        pos += 1
    s.close(); model.close(); osess.close(); om.close()


def _prompt_then_steps_on_two_paths(lva, orc, ctx, path, shape, n_prompt, seed, steps):
    """the prompt as ONE step (batched path: matrix-core GEMMs and batched attention) against the oracle evaluating the same
    prompt itself, then greedy steps on the graph path and on the persistent kernel, each against the oracle"""
    om = orc.Model(path)
    osess = orc.Session(om, 256)
    model = lva.Model(ctx, path)
    graph, pers = lva.Session(model, 256), lva.Session(model, 256)
    graph.set_path(lva.PATH_GRAPH)
    assert pers.path() == lva.PATH_PERSISTENT and graph.path() == lva.PATH_GRAPH
    prompt = lva.synth_tokens(n_prompt, 3, shape["vocab"], seed=seed)
    want = osess.eval(prompt)
    worst = 0.0
    for s in (graph, pers):
        s.begin(prompt, 0)                # n_prompt >= 16: both sessions take the batched prompt path
        got = s.logits()
        assert np.all(np.abs(got - want) <= 1e-2 + 1e-3 * np.abs(want)), ("prompt", float(np.max(np.abs(got - want))))
        worst = max(worst, float(np.max(np.abs(got - want))))
        assert s.argmax() == orc.greedy(want)
    # cache rows the prompt left: fp16 roundings of fp32 sums taken in another order than the oracle's; an fp16 ulp where a
    # sum falls near a rounding boundary in layer 0, error carried from layer to layer below
    last = shape["layers"] - 1
    for layer, bound in ((0, 2.0 ** -10), (last // 2, 4e-3), (last, 4e-3)):
        for which in (0, 1):
            b = osess.kv(layer, which, n_prompt).view(np.float16).astype(np.float32)
            a = graph.kv(layer, which, n_prompt).view(np.float16).astype(np.float32)
            assert float(np.max(np.abs(a - b))) <= bound * float(np.max(np.abs(b))), (layer, which)
    pos = n_prompt
    for step in range(steps):
        tok = orc.greedy(want)
        want = osess.eval(np.array([tok], dtype=np.uint32))
        for label, s in (("graph", graph), ("persistent", pers)):
            s.begin([tok], pos)
            got = s.logits()
            assert np.all(np.abs(got - want) <= 1e-2 + 1e-3 * np.abs(want)), (label, step, float(np.max(np.abs(got - want))))
            worst = max(worst, float(np.max(np.abs(got - want))))
            assert s.argmax() == orc.greedy(want), (label, step)
        pos += 1
    print(f"max |dlogit| over the prompt and {steps} steps on two paths: {worst:.3g}")
    for h in (graph, pers, model, osess, om):
        h.close()


def test_13b_q4_0_prompt_of_32_as_one_step_then_steps_on_graph_and_persistent_paths(lva, orc, ctx):
    """LLaMA-13B shape, q4_0, seed 2, a 32-token prompt evaluated as one step (llava_session.cpp:197-229 with 32 pending
    tokens), 8 greedy steps"""
    path = _model_file(lva, "13b_q4_0", lva.LV_Q4_0, 2, SHAPE_13B)
    _prompt_then_steps_on_two_paths(lva, orc, ctx, path, SHAPE_13B, 32, seed=2, steps=8)


def _checker_from_cache(orc, om, sess, layers, pos, backlog):
    """a checker session that continues from a copy of the GPU session's first `pos` cache rows"""
    o = orc.Session(om, backlog)
    for layer in range(layers):
        for which in (0, 1):
            o.kv_load(layer, which, sess.kv(layer, which, pos))
    o.set_pos(pos)
    return o


def test_13b_q4_0_256_greedy_steps_on_graph_and_persistent_paths(lva, orc, ctx):
    """The whole length of the 13B q4_0 configuration: a 32-token prompt, then 256 greedy steps (positions 32..287) on the
    hipGraph of the operator chain and on the persistent kernel side by side.  Every step the two paths have to pick the
    same token; at steps 0..7, 128 and 255 the checker evaluates that step from a copy of the path's own cache rows and
    the logits have to agree within the tolerance (the checker needs 0.4 s a token: following all 256 would take minutes)."""
    path = _model_file(lva, "13b_q4_0", lva.LV_Q4_0, 2, SHAPE_13B)
    om = orc.Model(path)
    model = lva.Model(ctx, path)
    L = SHAPE_13B["layers"]
    graph, pers = lva.Session(model, 512), lva.Session(model, 512)
    graph.set_path(lva.PATH_GRAPH)
    prompt = lva.synth_tokens(32, 3, SHAPE_13B["vocab"], seed=2)
    for s in (graph, pers):
        s.begin(prompt, 0)
    tok = pers.argmax()
    assert graph.argmax() == tok
    pos, worst = 32, 0.0
    for step in range(256):
        check = step < 8 or step in (128, 255)
        if check:
            want = {}
            for label, s in (("graph", graph), ("persistent", pers)):
                o = _checker_from_cache(orc, om, s, L, pos, 512)
                want[label] = o.eval(np.array([tok], dtype=np.uint32))
                o.close()
        for s in (graph, pers):
            s.begin([tok], pos)
        if check:
            for label, s in (("graph", graph), ("persistent", pers)):
                got = s.logits()
                err = float(np.max(np.abs(got - want[label]) / (1e-2 + 1e-3 * np.abs(want[label]))))
                assert err <= 1.0, (label, step, err)
                worst = max(worst, err)
                assert s.argmax() == orc.greedy(want[label]), (label, step)
        tg, tp = graph.argmax(), pers.argmax()
        assert tg == tp, (step, tg, tp)
        tok = tp
        pos += 1
    assert pos == 288
    print(f"13B q4_0, 256 steps on two paths: same tokens throughout; worst checked error {worst:.2f} x tolerance")
    for h in (graph, pers, model, om):
        h.close()


def test_7b_q4_0_logits_of_all_128_prompt_rows(lva, orc, ctx, model_7b):
    """the reference's head runs over every row of a step (llava_command_buffer.cpp:38-39): with lv_session_set_all_logits the
    128-token prompt keeps 128 x 32000 logits (final norm of all rows, the 32000 x 4096 output matrix on the matrix
    cores), each row against the checker's"""
    om = orc.Model(model_7b)
    osess = orc.Session(om, 128)
    model = lva.Model(ctx, model_7b)
    s = lva.Session(model, 128)
    s.keep_all_logits()
    prompt = lva.synth_tokens(128, 3, SHAPE["vocab"], seed=5)
    want = osess.eval(prompt, all_rows=True)
    s.begin(prompt, 0)
    got = s.logits_rows(0, 128)
    worst = float(np.max(np.abs(got - want) / (1e-2 + 1e-3 * np.abs(want))))
    assert worst <= 1.0, worst
    assert np.array_equal(np.argmax(got, axis=1), np.argmax(want, axis=1))
    print(f"128 x 32000 logits: worst error {worst:.3f} x tolerance")
    s.close(); model.close(); osess.close(); om.close()


def test_7b_q4_0_prompt_of_128_as_one_step_then_steps(lva, orc, ctx, model_7b):
    """a 128-token prompt on the 7B q4_0 model: the q4_0 GEMM forms at K = 4096 and 11008 with full token tiles, checked
    against the oracle evaluating the 128 tokens itself"""
    _prompt_then_steps_on_two_paths(lva, orc, ctx, model_7b, SHAPE, 128, seed=5, steps=4)


def test_7b_q8_0_long_context_steps_match_oracle(lva, orc, ctx):
    """7B q8_0 with the cache filled to position 1920 by the batched prompt path, then the configuration's 128 greedy
    steps (positions 1920..2047, the last row of a 2048-row cache) on the persistent kernel.  The checker follows steps
    0..3 from a copy of the cache after the prompt (evaluating 1920 tokens on the CPU would take minutes), and evaluates
    steps 64 and 127 from a copy of the cache as it stands then; so this pins the decode steps at a long context, not
    the prompt evaluation (tests/test_gpu_gemm.py does that)."""
    path = _model_file(lva, "7b_q8_0", lva.LV_Q8_0, 1, SHAPE)
    model = lva.Model(ctx, path)
    s = lva.Session(model, 2048)
    assert s.path() == lva.PATH_PERSISTENT
    first = 1920
    prompt = lva.synth_tokens(first, 3, SHAPE["vocab"], seed=1)
    s.begin(prompt, 0)
    tok = s.argmax()
    om = orc.Model(path)
    osess = _checker_from_cache(orc, om, s, SHAPE["layers"], first, 2048)
    pos = first
    for step in range(128):
        if step in (64, 127):
            osess = _checker_from_cache(orc, om, s, SHAPE["layers"], pos, 2048)
        check = step < 4 or step in (64, 127)
        if check:
            want = osess.eval(np.array([tok], dtype=np.uint32))
        s.begin([tok], pos)
        if check:
            got = s.logits()
            assert np.all(np.abs(got - want) <= 1e-2 + 1e-3 * np.abs(want)), (step, float(np.max(np.abs(got - want))))
            assert s.argmax() == orc.greedy(want), step
            if step in (3, 64):
                osess.close()
        tok = s.argmax()
        pos += 1
    assert pos == 2048
    osess.close()
    s.close(); model.close(); om.close()


def _within(got, truth, factor=1.0):
    """every logit within factor x (1e-2 absolute + 1e-3 relative) of `truth`; returns the largest error as a multiple of the tolerance"""
    ratio = np.abs(np.asarray(got, dtype=np.float64) - truth) / (1e-2 + 1e-3 * np.abs(truth))
    worst = float(np.max(ratio))
    assert worst <= factor, worst
    return worst


def _rms(got, truth):
    return float(np.sqrt(np.mean((np.asarray(got, dtype=np.float64) - truth) ** 2)))


def test_13b_q8_0_prompt_of_512_as_one_batch(lva, orc, ctx):
    """The prompt case at full size: 512 tokens through the matrix-core GEMM and the batched attention of a 40-layer 13B
    q8_0 model.  This model is the least forgiving of the configurations: q8_0 codes up to 127 give every layer weights of
    order 1, attention scores so large that the softmax picks single rows, logits up to 9 — and it amplifies fp32 rounding
    ten-thousandfold: measured against the step in double precision (orc_forward_f64, pinned by an independent numpy
    forward pass) on the first 32 tokens, the CPU checker itself, which follows the shaders' own summation order, is 0.0023
    rms and 0.88 x the tolerance at the worst of its 32000 logits away; the persistent kernel 0.0026 rms / 1.00 x, the
    operator chain 0.0026 / 1.07 x, the batched path 0.0029 / 1.08 x.  The tolerance of 1e-2 + 1e-3 |l| is four standard
    deviations of that noise, so two fp32 evaluations that sum in different orders cannot be held to it against each other
    (expected worst of 32000: 0.014), and none can be held to it against the exact result more firmly than the checker is.
    What is asserted instead says that the GPU's error IS that noise and nothing else:
    (0) first 32 tokens, against double precision: the checker within the tolerance; the 32-token batch and the
        persistent kernel token by token no noisier than 1.3 x the checker's rms error and nowhere beyond 1.25 x the
        tolerance; GPU against checker within twice the tolerance (which follows), greedy token the same for all four;
        the first 32 cache rows inside the 512-token batch against the checker's;
    (1) all 512 tokens as one batch and token by token: each path's logits within the tolerance of the double-precision
        evaluation of the last token on top of that path's own 511 cache rows (evaluating all 512 rows in double would
        take minutes; a single step does not amplify), the cache rows of the two paths against each other;
    (2) from a copy of the batch path's cache the checker evaluates the next token, at the tolerance itself."""
    path = _model_file(lva, "13b_q8_0", lva.LV_Q8_0, 3, SHAPE_13B)
    model = lva.Model(ctx, path)
    om = orc.Model(path)
    L = SHAPE_13B["layers"]
    n = 512
    prompt = lva.synth_tokens(n, 3, SHAPE_13B["vocab"], seed=3)
    batch, single = lva.Session(model, 1024), lva.Session(model, 1024)
    assert single.path() == lva.PATH_PERSISTENT
    batch.begin(prompt, 0)
    got = batch.logits().copy()
    single_head = None
    for i in range(n):
        single.begin(prompt[i:i + 1], i)
        single.wait()
        if i == 31:
            single_head = single.logits().copy()
    want = single.logits().copy()
    assert batch.argmax() == single.argmax()

    # (0) the first 32 tokens against the double-precision step
    truth32 = om.forward_f64(prompt[:32])
    ohead = orc.Session(om, 128)
    head_want = ohead.eval(prompt[:32])
    head = lva.Session(model, 128)
    head.begin(prompt[:32], 0)
    head_got = head.logits()
    d_checker, r_checker = _within(head_want, truth32), _rms(head_want, truth32)
    report = [f"checker {d_checker:.2f} x tolerance at worst, rms {r_checker:.4f}"]
    for label, logits in (("32-token batch", head_got), ("persistent kernel", single_head)):
        d, r = _within(logits, truth32, 1.25), _rms(logits, truth32)
        assert r <= 1.3 * r_checker, (label, r, r_checker)
        between = _within(logits, head_want.astype(np.float64), 2.0)
        report.append(f"{label} {d:.2f} x, rms {r:.4f}, against the checker {between:.2f} x")
    print("32 tokens against double precision: " + "; ".join(report))
    assert head.argmax() == orc.greedy(head_want) == int(np.argmax(truth32))
    for layer, bound in ((0, 2.0 ** -10), (19, 4e-3), (39, 4e-3)):
        for which in (0, 1):
            b = ohead.kv(layer, which, 32).view(np.float16).astype(np.float32)
            for rows in (batch.kv(layer, which, 32), head.kv(layer, which, 32)):
                a = rows.view(np.float16).astype(np.float32)
                assert float(np.max(np.abs(a - b))) <= bound * float(np.max(np.abs(b))), (layer, which)
    head.close(); ohead.close()

    # (1) 512 tokens: each path against the double-precision evaluation of the last token on its own cache
    for label, sess, logits in (("batch", batch, got), ("token by token", single, want)):
        kv = [(sess.kv(layer, 0, n - 1), sess.kv(layer, 1, n - 1)) for layer in range(L)]
        truth = om.forward_f64(prompt[n - 1:], kv=kv)
        worst = _within(logits, truth)
        print(f"512 tokens, {label}: worst error / tolerance against double precision on its own cache {worst:.2f}")
        del kv
    _within(got, want.astype(np.float64), 2.0)
    # cache rows: fp16 values of fp32 sums taken in two different orders; they may differ by an fp16 ulp where a sum
    # falls near a rounding boundary, and by more only through error carried from layer to layer
    for layer, bound in ((0, 2.0 ** -10), (19, 1e-2), (39, 1e-2)):
        for which in (0, 1):
            a = batch.kv(layer, which, n).view(np.float16).astype(np.float32)
            b = single.kv(layer, which, n).view(np.float16).astype(np.float32)
            worst = float(np.max(np.abs(a - b))) / float(np.max(np.abs(b)))
            assert worst <= bound, (layer, which, worst)

    # (2) the checker continues from the batch path's cache
    osess = orc.Session(om, 1024)
    for layer in range(L):
        for which in (0, 1):
            osess.kv_load(layer, which, batch.kv(layer, which, n))
    osess.set_pos(n)
    tok = batch.argmax()
    ref = osess.eval(np.array([tok], dtype=np.uint32))
    batch.begin([tok], n)
    nxt = batch.logits()
    assert np.all(np.abs(nxt - ref) <= 1e-2 + 1e-3 * np.abs(ref)), float(np.max(np.abs(nxt - ref)))
    assert batch.argmax() == orc.greedy(ref)
    for h in (batch, single, model, osess, om):
        h.close()
