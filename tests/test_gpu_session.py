"""llava_session / llava_context (the C++ host classes in llama-vulkan_amd/host, mirroring the reference's
llava_session.cpp and llava_context.cpp) on the GPU, against the oracle: text in, greedy tokens out, cache reuse
between prompts, rewind, growth of the backlog, the snapshot and frame file formats and the seeded sampler."""
import importlib
import os
import struct
import subprocess
import sys

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

PROMPT = b"The quick brown fox"


@pytest.fixture(scope="module")
def hl():
    return importlib.import_module("llama-vulkan_amd.hostlib")


@pytest.fixture(scope="module")
def loaded(hl, tiny_models):
    c = hl.LlavaContext()
    assert c.load_model(tiny_models["tiny_q4"]), c.error()
    f = hl.GgmlFile(tiny_models["tiny_q4"])
    yield c, f, tiny_models["tiny_q4"]
    f.close()
    c.close()


def oracle_greedy(orc, path, tokens, steps, backlog=128):
    om = orc.Model(path)
    s = orc.Session(om, backlog)
    logits = s.eval(np.array(tokens, dtype=np.uint32))
    out, rows = [], [logits]
    for _ in range(steps):
        nxt = orc.greedy(logits)
        out.append(nxt)
        logits = s.eval(np.array([nxt], dtype=np.uint32))
        rows.append(logits)
    s.close(); om.close()
    return out, rows


def test_greedy_text_decode_matches_oracle(hl, orc, loaded):
    c, f, path = loaded
    s = hl.LlavaSession(c)
    assert s.good()
    assert s.set_text(PROMPT)
    toks = f.tokenize(PROMPT, True)
    assert s.tokens() == toks and toks[0] == 1
    want, rows = oracle_greedy(orc, path, toks, 24)
    got = []
    nxt = s.predict(True)
    for i in range(24):
        assert np.max(np.abs(s.logits() - rows[i])) <= 1e-2 + 1e-3 * np.max(np.abs(rows[i]))
        got.append(nxt)
        assert s.push_token(nxt)
        assert s.start()                       # asynchronous submit ...
        nxt = s.finish(True)                   # ... and the only wait
    assert got == want
    assert s.tokens_in_gpu() == len(toks) + 24
    s.close()


def test_set_text_reuses_the_common_prefix_and_rewind_drops_the_tail(hl, orc, loaded):
    c, f, path = loaded
    s = hl.LlavaSession(c)
    assert s.set_text(PROMPT + b" jumps")
    first = s.predict(True)
    n_full = s.token_count()
    assert s.tokens_in_gpu() == n_full
    # a new text that shares a prefix keeps those cache rows (the reference compares text lengths only:
    # llava_session.cpp:243-277; here the tokens themselves are compared)
    assert s.set_text(PROMPT + b" sleeps")
    shared = 0
    a, b = f.tokenize(PROMPT + b" jumps", True), f.tokenize(PROMPT + b" sleeps", True)
    while shared < min(len(a), len(b)) and a[shared] == b[shared]:
        shared += 1
    assert s.tokens_in_gpu() == shared and 0 < shared < len(b)
    got = s.predict(True)
    want, _ = oracle_greedy(orc, path, b, 1)
    assert got == want[0]
    # rewind to the first prompt's prefix and decode it again: same answer as the first time
    s.rewind(shared)
    assert s.token_count() == shared and s.tokens_in_gpu() == shared
    for t in a[shared:]:
        assert s.push_token(t)
    assert s.predict(True) == first
    s.rewind(10_000)                            # beyond the end: nothing happens (llava_session.cpp:390-395)
    assert s.token_count() == len(a)
    s.close()


def test_text_that_is_a_prefix_of_the_evaluated_context_is_evaluated_again(hl, orc, loaded):
    """set_text with the same prompt, and with a shorter prompt that is a prefix of it: all rows could be reused, but the
    logits on the device belong to the longer context, so the last token is evaluated again (the reference re-evaluates
    here: llava_session.cpp:257-277 finds no reusable prefix) and predict answers for the new text"""
    c, f, path = loaded
    s = hl.LlavaSession(c)
    long_text, short_text = PROMPT + b" jumps over", PROMPT
    a, b = f.tokenize(long_text, True), f.tokenize(short_text, True)
    assert a[:len(b)] == b and len(b) < len(a)
    assert s.set_text(long_text)
    first = s.predict(True)
    assert s.tokens_in_gpu() == len(a)
    assert s.set_text(long_text)                # the same text once more
    assert s.tokens_in_gpu() == len(a) - 1
    assert s.predict(True) == first
    assert s.set_text(short_text)               # a strict prefix of what the cache holds
    assert s.tokens_in_gpu() == len(b) - 1
    want, rows = oracle_greedy(orc, path, b, 1)
    assert s.predict(True) == want[0]
    assert np.max(np.abs(s.logits() - rows[0])) <= 1e-2 + 1e-3 * np.max(np.abs(rows[0]))
    assert s.set_text(short_text)               # and once more: still answers, for the same text
    assert s.predict(True) == want[0]
    s.close()


def test_a_failed_step_is_evaluated_again_by_the_next_start(hl, lva, orc, tmp_path):
    """failure path at the level of llava_session: the persistent kernel's poll bound set to 1 makes its workgroups stop
    waiting for each other at once (every kernel still runs to its end), finish reports the failure as ~0, and the rows of
    that step count as pending again: the next predict evaluates the same token into the same row and gives the oracle's
    token.  Without that the session would refuse ('GPU is already in sync') and go on over rows that hold nothing."""
    p = str(tmp_path / "wide.ggml")
    lva.write_model(p, wtype=lva.LV_Q4_0, seed=9, vocab=2048, layers=2, dim=4096, heads=32, ff=11008)
    c = hl.LlavaContext()
    assert c.load_model(p), c.error()
    s = hl.LlavaSession(c)
    import ctypes
    dev, path_now = s.device_session(), ctypes.c_int()
    assert lva.hip().lv_session_path(dev, ctypes.byref(path_now)) == 0 and path_now.value == lva.PATH_PERSISTENT
    prompt = [int(t) for t in lva.synth_tokens(4, 3, 2048, seed=3)]
    want, rows = oracle_greedy(orc, p, prompt, 2)
    for t in prompt:
        assert s.push_token(t)
    assert s.predict(True) == want[0]
    assert s.push_token(want[0])
    assert lva.hip().lv_session_set_wait_limit(dev, 1) == 0
    assert s.start()
    assert s.tokens_in_gpu() == 5
    assert s.finish(True) == 0xFFFFFFFF
    assert s.tokens_in_gpu() == 4               # the failed row is pending again
    assert lva.hip().lv_session_set_wait_limit(dev, 0) == 0
    assert s.predict(True) == want[1]
    assert np.max(np.abs(s.logits() - rows[1])) <= 1e-2 + 1e-3 * np.max(np.abs(rows[1]))
    # a failed step that is never finished (started, then another start) is settled and repeated the same way
    assert s.push_token(want[1])
    assert lva.hip().lv_session_set_wait_limit(dev, 1) == 0
    assert s.start()
    assert lva.hip().lv_session_set_wait_limit(dev, 0) == 0
    assert s.start() and s.tokens_in_gpu() == 6
    third = s.finish(True)
    more, _ = oracle_greedy(orc, p, prompt, 3)
    assert third == more[2]
    s.close()
    c.close()


def test_add_text_appends_through_the_detokenised_text(hl, loaded):
    c, f, _ = loaded
    s = hl.LlavaSession(c)
    assert s.set_text(b"abc")
    before = s.tokens()
    assert s.add_text(b"def")
    # llava_session.cpp:279-282: the whole token list is turned back into text (BOS prints as "<s>") and re-tokenised
    assert s.tokens() == f.tokenize(f.detokenize(before) + b"def", True)
    s.close()


def test_backlog_doubles_and_stops_at_2048(hl, orc, loaded):
    c, f, path = loaded
    s = hl.LlavaSession(c)
    assert s.backlog() == 128 and s.spevars()["backlog"] == 128 and s.spevars()["backlog_bits"] == 7
    rng = np.random.default_rng(0)
    toks = [1] + [int(t) for t in rng.integers(3, 512, 139)]
    for t in toks[:128]:
        assert s.push_token(t)
    assert s.backlog() == 128
    first = s.predict(True)                     # 128 rows are in the cache now
    for t in toks[128:]:
        assert s.push_token(t)                  # grows to 256 and keeps the cached rows
    assert s.backlog() == 256 and s.spevars()["backlog"] == 256 and s.tokens_in_gpu() == 128
    got = s.predict(True)
    om = orc.Model(path)
    o = orc.Session(om, 256)
    assert orc.greedy(o.eval(np.array(toks[:128], dtype=np.uint32))) == first
    want = o.eval(np.array(toks[128:], dtype=np.uint32))
    assert got == orc.greedy(want)
    assert np.max(np.abs(s.logits() - want)) <= 1e-2 + 1e-3 * np.max(np.abs(want))
    o.close(); om.close()
    assert not s.push_token(1 << 20)            # not a token of this vocabulary
    assert s.set_text(b"x" * 300)               # 301 tokens: 512 rows
    assert s.backlog() == 512
    assert not s.set_text(b"y" * 3000)          # would need more than 2048 rows (llava_session.cpp:253-262)
    assert s.backlog() == 512 and s.token_count() == 301
    s.close()


def test_snapshot_file_format_and_restore(hl, orc, loaded, tmp_path):
    c, f, path = loaded
    s = hl.LlavaSession(c)
    assert s.set_text(PROMPT)
    first = s.predict(True)
    toks = s.tokens()
    n = len(toks)
    snap = str(tmp_path / "snap.bin")
    assert s.snapshot(snap) == hl.RC_OK
    raw = open(snap, "rb").read()
    dim, layers = 256, 2
    # llava_session.cpp:447-520: u32 n, the tokens, then per layer the K rows followed by the V rows, fp16
    assert len(raw) == 4 + 4 * n + layers * 2 * n * dim * 2
    assert struct.unpack_from("<I", raw)[0] == n
    assert list(struct.unpack_from(f"<{n}I", raw, 4)) == toks
    om = orc.Model(path)
    o = orc.Session(om, 128)
    o.eval(np.array(toks, dtype=np.uint32))
    body = np.frombuffer(raw, dtype=np.uint16, offset=4 + 4 * n).reshape(layers, 2, n, dim)
    for layer in range(layers):
        for which in range(2):
            want = o.kv(layer, which, n)
            diff = np.abs(body[layer, which].view(np.float16).astype(np.float32) - want.view(np.float16).astype(np.float32))
            # summation order differs from the oracle's: the last fp16 bit of some entries may flip, nothing more
            assert np.mean(body[layer, which] != want) < 0.5 and np.max(diff) <= 2e-3 * np.max(np.abs(want.view(np.float16).astype(np.float32)))
    o.close(); om.close()

    # a fresh session restored from the file continues exactly like the one that wrote it
    t = hl.LlavaSession(c)
    assert t.restore(snap) == hl.RC_OK
    assert t.tokens() == toks and t.tokens_in_gpu() == n
    assert s.push_token(first) and t.push_token(first)
    a, b = s.predict(True), t.predict(True)
    assert a == b and np.array_equal(s.logits(), t.logits())

    # malformed snapshot files are refused and leave the session as it was (llava_session.cpp:522-603)
    before = t.tokens()
    open(str(tmp_path / "short.bin"), "wb").write(b"\x01\x00")
    assert t.restore(str(tmp_path / "short.bin")) == hl.RC_NOK
    open(str(tmp_path / "cut.bin"), "wb").write(raw[:-2])
    assert t.restore(str(tmp_path / "cut.bin")) == hl.RC_NOK
    open(str(tmp_path / "huge.bin"), "wb").write(struct.pack("<I", 1 << 30) + raw[4:])
    assert t.restore(str(tmp_path / "huge.bin")) == hl.RC_NOK
    assert t.restore(str(tmp_path / "absent.bin")) == hl.RC_NOK
    assert t.restore(str(tmp_path)) == hl.RC_NOK
    assert t.tokens() == before
    s.close(); t.close()


def test_save_frame_needs_tracing_and_writes_named_buffers(hl, orc, loaded, tmp_path):
    c, f, path = loaded
    s = hl.LlavaSession(c)
    frame = str(tmp_path / "frame.bin")
    assert not s.is_tracing()
    assert s.save_frame(frame) == hl.RC_NOT_TRACING
    assert s.set_options(1) == hl.RC_OK and s.is_tracing()
    assert s.set_text(PROMPT)
    s.predict(True)
    assert s.save_frame(frame) == hl.RC_OK
    raw = open(frame, "rb").read()
    om = orc.Model(path)
    toks = np.array(s.tokens(), dtype=np.uint32)
    n = len(toks)
    assert n > 1
    # the frame holds every row of the step, as the reference's batch-sized buffers do (llava_layer_session_data.cpp:80-85);
    # the oracle keeps the buffers of the last row it evaluated, so row z comes from a session fed the first z + 1 tokens
    per_row = []
    for z in range(n):
        o = orc.Session(om, 128)
        o.eval(toks[:z + 1])
        per_row.append({(layer, w): o.trace(layer, w).copy() for layer in range(2) for w in range(6)})
        o.close()
    which = {"normalized_input_logit": 0, "post_attn_logit": 1, "post_attn_norm_logit": 2, "ff_result": 3, "output_logit": 4, "attn_result": 5}
    cur, seen = 0, []
    while cur < len(raw):
        # llava_buffer.cpp:497-522: two shape words, the type, the name, zeros up to a multiple of 32, the values
        count, rows, ftype = struct.unpack_from("<3I", raw, cur)
        name = raw[cur + 12:raw.index(b"\0", cur + 12)].decode()
        head = (12 + len(name) + 1 + 31) // 32 * 32
        vals = np.frombuffer(raw, dtype=np.float32, count=count * rows, offset=cur + head)
        cur += head + 4 * count * rows
        _, layer, slot = name.split(".")
        # attn_result is (backlog, heads x rows) as in llava_layer_session_data.cpp:80; the vectors are (length, rows); in
        # memory both are one row of the step after the other (mhsa.comp:58, z_id * BACKLOG * HEAD_COUNT)
        assert ftype == 0 and (count, rows) == ((128, om.hp["heads"] * n) if slot == "attn_result" else (count, n))
        vals = vals.reshape(n, -1)
        for z in range(n):
            want = per_row[z][(int(layer), which[slot])]
            assert vals[z].shape == want.shape and np.max(np.abs(vals[z] - want)) <= 1e-4 * max(1.0, np.max(np.abs(want))), (name, z)
        seen.append(name)
    assert cur == len(raw) and len(seen) == 2 * 6 and seen[:2] == ["layer.0.attn_result", "layer.0.ff_result"]
    heads = om.hp["heads"]
    om.close()
    # the next step is one token long, and so is its frame
    assert s.push_token(5)
    s.predict(True)
    assert s.save_frame(frame) == hl.RC_OK
    raw = open(frame, "rb").read()
    count, rows, ftype = struct.unpack_from("<3I", raw, 0)
    assert (count, rows) == (128, heads)
    assert s.set_options(0) == hl.RC_OK and not s.is_tracing()
    s.close()


def test_seeded_sampler_is_reproducible_and_picks_plausible_tokens(hl, loaded):
    c, f, _ = loaded
    runs = []
    for seed in (7, 7, 8):
        s = hl.LlavaSession(c)
        s.seed(seed)
        assert s.set_text(PROMPT)
        out = []
        for _ in range(16):
            t = s.predict(False)
            assert t != 0xFFFFFFFF
            # the sampler keeps tokens that are at least 2^-mu likely at temperature 0.8 (llava_session.cpp:169-195);
            # whatever mu is, the pick can never be less likely than 2^-64
            p = np.exp(s.logits().astype(np.float64) / 0.8)
            assert p[t] / p.sum() > 2.0 ** -64
            out.append(t)
            assert s.push_token(t)
        runs.append(out)
        s.close()
    assert runs[0] == runs[1]
    assert len(set(runs[0])) > 1


def test_cli_prints_the_greedy_continuation(hl, orc, loaded):
    c, f, path = loaded
    exe = os.path.join(os.path.dirname(hl.__file__), "bin", "llava")
    assert os.path.exists(exe), "llama-vulkan_amd/bin/llava is not built"
    toks = f.tokenize(PROMPT, True)
    want, _ = oracle_greedy(orc, path, toks, 12)
    text = PROMPT
    for t in want:
        if t == 2:
            break
        text += f.token(t)[0]
    r = subprocess.run([exe, "-m", path, "--greedy", "-n", "12", PROMPT.decode()], capture_output=True, timeout=120)
    assert r.returncode == 0, r.stderr.decode(errors="replace")
    assert r.stdout.rstrip(b"\n") == text.rstrip(b"\n")
    r = subprocess.run([exe, "-m", path, "-s", "--port", "70000"], capture_output=True, timeout=60)
    assert r.returncode != 0 and b"port" in r.stderr
    r = subprocess.run([exe, "-m", path + ".absent", "hi"], capture_output=True, timeout=60)
    assert r.returncode != 0 and b"absent" in r.stderr


def test_two_threads_two_sessions_one_model(lva, orc, ctx, tmp_path):
    """the reference's threading contract (one session per thread, sessions share the context and the weights,
    llava_context.h:47-49): two threads decode at the same time on the persistent kernel, whose launches must take
    turns on the device; both must produce what a lone session produces"""
    import threading
    p = str(tmp_path / "two.ggml")
    lva.write_model(p, wtype=lva.LV_Q4_0, seed=13, vocab=2048, layers=2, dim=4096, heads=32, ff=11008)
    model = lva.Model(ctx, p)

    def run(seed, out):
        s = lva.Session(model, 128)
        assert s.path() == lva.PATH_PERSISTENT
        prompt = lva.synth_tokens(4, 3, 2048, seed=seed)
        s.begin(prompt, 0)
        toks, pos = [], 4
        for _ in range(60):
            t = s.argmax()
            toks.append(t)
            s.begin([t], pos)
            pos += 1
        toks.append(s.argmax())
        s.close()
        out.extend(toks)

    alone = [[], []]
    for i in range(2):
        run(20 + i, alone[i])
    together = [[], []]
    threads = [threading.Thread(target=run, args=(20 + i, together[i])) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert together == alone
    model.close()


def test_command_line_stops_at_a_signal(tiny_models):
    """an interrupt ends the token loop after the current token and the program exits normally (llava_context.cpp:352)"""
    import signal
    import time
    exe = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "llama-vulkan_amd", "bin", "llava")
    # the context holds 2048 tokens at most; without the signal the run would go on to that limit
    p = subprocess.Popen([exe, "-m", tiny_models["tiny_q4"], "--greedy", PROMPT.decode()], stdout=subprocess.PIPE, stderr=subprocess.PIPE)
    try:
        time.sleep(1.0)
        if p.poll() is None:
            p.send_signal(signal.SIGINT)
        assert p.wait(timeout=60) == 0
        assert p.stdout.read().startswith(PROMPT)
    finally:
        if p.poll() is None:
            p.kill()
            p.wait()
