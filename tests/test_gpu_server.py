"""The token server end to end on the GPU (llama-vulkan_amd/host/server; reference: server/session_wrapper.cpp): a client
feeds a prompt, ticks or starts generation, and the tokens that come back over TCP are the oracle's greedy tokens.  The
greedy option bit is an addition (the reference's server always samples stochastically)."""
import importlib
import os
import struct

import numpy as np
import pytest

import server_client as sc

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hl():
    return importlib.import_module("llama-vulkan_amd.hostlib")


@pytest.fixture(scope="module")
def served(hl, tiny_models):
    ctx = hl.LlavaContext()
    assert ctx.load_model(tiny_models["tiny_q4"]), ctx.error()
    server = hl.LlavaServer(ctx)
    yield server, tiny_models["tiny_q4"]
    server.stop()
    ctx.close()


def oracle_greedy(orc, path, tokens, steps):
    om = orc.Model(path)
    s = orc.Session(om, 128)
    logits = s.eval(np.array(tokens, dtype=np.uint32))
    out = []
    for _ in range(steps):
        out.append(orc.greedy(logits))
        logits = s.eval(np.array([out[-1]], dtype=np.uint32))
    s.close(); om.close()
    return out


def test_ticks_return_the_oracles_greedy_tokens(lva, orc, served):
    server, path = served
    c = sc.Client(server.port)
    sid = c.new_session()
    assert c.ack(sc.SET_OPTIONS, sid, sc.OPTION_GREEDY) == sc.RC_OK
    prompt = [int(t) for t in lva.synth_tokens(6, 3, 512, seed=21)]
    for t in prompt:
        assert c.ack(sc.ADD_TOKEN, sid, t) == sc.RC_OK
    assert c.ack(sc.ADD_TOKEN, sid, 512) == sc.RC_NOK          # not in the vocabulary
    assert c.tokens(sid) == prompt
    want = oracle_greedy(orc, path, prompt, 10)
    got = []
    for i in range(10):
        token, index = c.tick(sid)
        assert index == len(prompt) + i
        got.append(token)
    assert got == want
    assert c.tokens(sid) == prompt + want
    # rewind to the prompt: every remaining token is in the cache already, so there is nothing to evaluate and a step
    # is refused (llava_session.cpp:199-203 "GPU is already in sync"); take the last prompt token back too and go again
    assert c.ack(sc.REWIND, sid, len(prompt)) == sc.RC_OK
    assert c.tokens(sid) == prompt
    assert c.tick(sid) == sc.RC_NOK
    assert c.ack(sc.REWIND, sid, len(prompt) - 1) == sc.RC_OK
    assert c.ack(sc.ADD_TOKEN, sid, prompt[-1]) == sc.RC_OK
    assert [c.tick(sid)[0] for _ in range(4)] == want[:4]
    assert c.ack(sc.KILL, sid) == sc.RC_OK
    assert struct.unpack("<I", c.wait_unsolicited(sc.OUT_DROPPED))[0] == sid
    c.close()


def test_generation_streams_to_subscribers_until_stopped(lva, orc, served):
    server, path = served
    driver, listener, outsider = sc.Client(server.port), sc.Client(server.port), sc.Client(server.port)
    for c in (listener, outsider):
        c.sessions()                   # a round trip: the server has accepted the connection before the session is made
    sid = driver.new_session()
    assert driver.ack(sc.SET_OPTIONS, sid, sc.OPTION_GREEDY) == sc.RC_OK
    assert listener.ack(sc.SUBSCRIBE, sid) == sc.RC_OK
    prompt = [int(t) for t in lva.synth_tokens(5, 3, 512, seed=22)]
    for t in prompt:
        assert driver.ack(sc.ADD_TOKEN, sid, t) == sc.RC_OK
    assert driver.ack(sc.START, sid) == sc.RC_OK
    assert driver.tick(sid) == sc.RC_RUNNING                   # no single steps while it runs
    assert driver.ack(sc.RESTORE, sid, text=b"/tmp/none.bin") == sc.RC_RUNNING
    heard = [struct.unpack("<3I", listener.wait_unsolicited(sc.OUT_TOKEN)) for _ in range(12)]
    assert driver.ack(sc.STOP, sid) == sc.RC_OK
    assert [h[0] for h in heard] == [sid] * 12
    assert [h[2] for h in heard] == list(range(len(prompt), len(prompt) + 12))
    want = oracle_greedy(orc, path, prompt, 12)
    assert [h[1] for h in heard] == want
    # the buffer holds what was streamed (and whatever was produced before the stop arrived)
    buf = driver.tokens(sid)
    assert buf[:len(prompt) + 12] == prompt + want
    # somebody who did not subscribe heard nothing but the announcement of the session
    assert outsider.sessions() == [sid]
    assert [k for k, _ in outsider.unsolicited] == [sc.OUT_NEW_SESSION]
    # it runs until the context is full, then stops by itself: 128 rows, the reference's smallest backlog, grow to 2048
    assert listener.ack(sc.UNSUBSCRIBE, sid) == sc.RC_OK
    assert driver.ack(sc.KILL, sid) == sc.RC_OK
    for c in (driver, listener, outsider):
        c.close()


def test_two_sessions_snapshot_restore_and_frames(lva, orc, served, tmp_path):
    server, path = served
    c = sc.Client(server.port)
    s1, s2 = c.new_session(), c.new_session()
    prompt = [int(t) for t in lva.synth_tokens(7, 3, 512, seed=23)]
    want = oracle_greedy(orc, path, prompt, 6)
    for s in (s1, s2):
        assert c.ack(sc.SET_OPTIONS, s, sc.OPTION_GREEDY) == sc.RC_OK
    for t in prompt:
        assert c.ack(sc.ADD_TOKEN, s1, t) == sc.RC_OK
    assert [c.tick(s1)[0] for _ in range(3)] == want[:3]
    snap = str(tmp_path / "s1.snap").encode()
    assert c.ack(sc.SNAPSHOT, s1, text=snap) == sc.RC_OK
    # the other session picks the conversation up from the file and continues it
    assert c.ack(sc.RESTORE, s2, text=snap) == sc.RC_OK
    # (a snapshot holds the tokens whose rows are in the cache: the newest one was produced but not yet evaluated)
    assert c.tokens(s2) == prompt + want[:2]
    assert c.ack(sc.ADD_TOKEN, s2, want[2]) == sc.RC_OK
    assert [c.tick(s2)[0] for _ in range(3)] == want[3:6]
    assert c.ack(sc.RESTORE, s2, text=str(tmp_path / "absent").encode()) == sc.RC_NOK
    # frames need record mode
    frame = str(tmp_path / "frame.bin").encode()
    assert c.ack(sc.SAVE_FRAME, s1, text=frame) == sc.RC_NOT_TRACING
    assert c.ack(sc.SET_OPTIONS, s1, sc.OPTION_GREEDY | sc.OPTION_RECORD) == sc.RC_OK
    assert c.tick(s1)[0] == want[3]
    assert c.ack(sc.SAVE_FRAME, s1, text=frame) == sc.RC_OK
    assert os.path.getsize(frame) > 0
    # text goes through the model's tokenizer on the session thread
    assert c.ack(sc.ADD_TEXT, s2, text=b" hello") == sc.RC_OK
    assert len(c.tokens(s2)) > len(prompt) + 6
    for s in (s1, s2):
        assert c.ack(sc.KILL, s) == sc.RC_OK
    c.close()


def test_server_mode_of_the_command_line(tiny_models):
    """llava -s: load, listen, answer, leave on SIGTERM with exit code 0 (llava_context.cpp:333-336, server/server.cpp:171-179)"""
    import signal
    import socket
    import subprocess
    import time
    exe = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "llama-vulkan_amd", "bin", "llava")
    with socket.socket() as probe:
        probe.bind(("127.0.0.1", 0))
        port = probe.getsockname()[1]
    p = subprocess.Popen([exe, "-m", tiny_models["tiny_q4"], "-s", "--port", str(port), "--bind", "127.0.0.1"],
                         stdin=subprocess.DEVNULL, stdout=subprocess.PIPE, stderr=subprocess.PIPE)
    try:
        c = None
        for _ in range(300):                   # the model upload comes first
            try:
                c = sc.Client(port)
                break
            except OSError:
                assert p.poll() is None, p.stderr.read().decode(errors="replace")
                time.sleep(0.1)
        assert c is not None
        sid = c.new_session()
        assert c.ack(sc.SET_OPTIONS, sid, sc.OPTION_GREEDY) == sc.RC_OK
        assert c.ack(sc.ADD_TEXT, sid, text=b"The quick") == sc.RC_OK
        token, index = c.tick(sid)
        assert token < 512 and index == len(c.tokens(sid)) - 1
        p.send_signal(signal.SIGTERM)          # with a live session and a connected client
        assert p.wait(timeout=30) == 0
        assert b"Started server on 127.0.0.1:%d" % port in p.stdout.read()
        c.close()
    finally:
        if p.poll() is None:
            p.kill()
            p.wait()
