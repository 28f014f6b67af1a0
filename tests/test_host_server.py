"""The token server's wire protocol on the CPU (llama-vulkan_amd/host/server; reference: server/client.cpp for the
packet checks, server/server.cpp for session announcements).  The context holds a parsed model file and no device, so
sessions exist but refuse every step: what is tested is framing, dispatch, return codes, announcements and shutdown."""
import importlib
import socket
import struct
import time

import pytest

import ggjt_builder as gb
import server_client as sc


@pytest.fixture(scope="module")
def hl():
    return importlib.import_module("llama-vulkan_amd.hostlib")


@pytest.fixture()
def served(hl, tmp_path):
    path = str(tmp_path / "vocab.ggml")
    vocab = gb.tokenizer_vocab()
    gb.build(path, vocab, gb.minimal_tensors(vocab=len(vocab)))
    ctx = hl.LlavaContext()
    assert ctx.open_model_file(path), ctx.error()
    server = hl.LlavaServer(ctx)
    yield server, vocab
    server.stop()
    ctx.close()


def test_token_map_and_unknown_commands(served):
    server, vocab = served
    c = sc.Client(server.port)
    kind, payload = c.call(sc.GET_TOKEN_MAP)
    assert kind == sc.OUT_TOKEN_MAP
    pieces, cur = [], 0
    while cur < len(payload):
        n = struct.unpack_from("<I", payload, cur)[0]
        pieces.append(payload[cur + 4:cur + 4 + n])
        cur += 4 + n
    assert pieces == [p for p, _ in vocab]
    assert c.sessions() == []
    assert c.ack(5) == sc.RC_UNKNOWN                          # below 16: no such global command
    assert c.ack(24, 1) == sc.RC_NO_SUCH_SESSION              # the session is looked up before the command
    assert c.ack(40, 1, 2) == sc.RC_UNKNOWN
    assert c.ack(sc.SUBSCRIBE, 1, 2) == sc.RC_BAD_ARGS        # one word expected
    assert c.ack(sc.SUBSCRIBE) == sc.RC_BAD_ARGS
    assert c.ack(sc.REWIND, 1) == sc.RC_BAD_ARGS              # two words expected
    assert c.ack(sc.ADD_TEXT, 1) == sc.RC_BAD_ARGS            # text expected behind the session
    assert c.ack(sc.SUBSCRIBE, 99) == sc.RC_NO_SUCH_SESSION
    assert c.ack(sc.ADD_TOKEN, 99, 5) == sc.RC_NO_SUCH_SESSION
    assert c.ack(sc.SNAPSHOT, 99, text=b"/tmp/x") == sc.RC_NO_SUCH_SESSION
    c.close()


def test_sessions_are_announced_to_everyone_and_die_on_request(served):
    server, _ = served
    a, b = sc.Client(server.port), sc.Client(server.port)
    assert b.sessions() == []                                 # b is connected before a asks
    sid = a.new_session()                                     # a's request id comes back ...
    assert struct.unpack("<I", b.wait_unsolicited(sc.OUT_NEW_SESSION))[0] == sid   # ... b hears of it unasked
    sid2 = b.new_session()
    assert sid2 != sid and a.sessions() == sorted([sid, sid2])
    assert struct.unpack("<I", a.wait_unsolicited(sc.OUT_NEW_SESSION))[0] == sid2
    # no device behind this context: the session answers, and refuses the work
    assert a.tokens(sid) == []
    assert a.ack(sc.SUBSCRIBE, sid) == sc.RC_OK
    assert a.ack(sc.ADD_TOKEN, sid, 5) == sc.RC_NOK
    assert a.tick(sid) == sc.RC_NOK
    assert a.ack(sc.START, sid) == sc.RC_OK                   # generation is switched on, its first step fails and switches it off
    assert a.ack(sc.STATUS, sid) == sc.RC_OK
    assert a.ack(sc.SAVE_FRAME, sid, text=b"/tmp/never_written.bin") == sc.RC_NOT_TRACING
    assert a.ack(sc.SNAPSHOT, sid, text=b"/tmp/a\0b") == sc.RC_BAD_ARGS     # NUL inside a path
    assert a.ack(sc.KILL, sid) == sc.RC_OK
    for c in (a, b):
        assert struct.unpack("<I", c.wait_unsolicited(sc.OUT_DROPPED))[0] == sid
    assert a.sessions() == [sid2]
    assert a.ack(sc.UNSUBSCRIBE, sid) == sc.RC_NO_SUCH_SESSION
    a.close(); b.close()


def test_framing_split_and_merged_packets(served):
    server, _ = served
    c = sc.Client(server.port)
    # two requests in one write
    c.send_raw(struct.pack("<3I", sc.LIST_SESSIONS, 71, 0) + struct.pack("<3I", 9, 72, 0))
    assert c.read_packet() == (sc.OUT_SESSION_LIST, 71, b"")
    assert c.read_packet() == (sc.OUT_ACK, 72, struct.pack("<I", sc.RC_UNKNOWN))
    # one request byte by byte
    for byte in struct.pack("<4I", sc.SUBSCRIBE, 73, 4, 12345):
        c.send_raw(bytes([byte]))
        time.sleep(0.002)
    assert c.read_packet() == (sc.OUT_ACK, 73, struct.pack("<I", sc.RC_NO_SUCH_SESSION))
    c.close()


def test_oversized_packet_ends_that_connection_only(served):
    """a length field above 0x10000 is a protocol violation (server/client.cpp:129-133 stops parsing that client); here the
    connection is closed, so that its unread input cannot keep the poll loop busy, and other clients are served as before"""
    server, _ = served
    bad, good = sc.Client(server.port, timeout=5.0), sc.Client(server.port)
    bad.send_raw(struct.pack("<3I", sc.ADD_TEXT, 1, 0x10001))
    with pytest.raises((ConnectionError, OSError)):
        bad.send_raw(struct.pack("<3I", sc.LIST_SESSIONS, 2, 0) + b"x" * 0x30000)   # more than the input buffer holds
        bad.read_packet()
    assert good.sessions() == []
    bad.close(); good.close()


def test_client_that_never_reads_is_dropped_when_its_replies_pile_up(served):
    """each token map request queues a reply; a client that keeps asking and never reads is dropped once 16 MiB wait for it,
    and the server keeps answering others"""
    server, vocab = served
    greedy, good = sc.Client(server.port, timeout=5.0), sc.Client(server.port)
    kind, payload = good.call(sc.GET_TOKEN_MAP)
    per_reply = 12 + len(payload)
    wanted = (16 << 20) // per_reply + 64
    request = struct.pack("<3I", sc.GET_TOKEN_MAP, 7, 0)
    greedy.sock.settimeout(20.0)
    dropped = False
    try:
        for start in range(0, wanted * 4, 256):               # far more requests than the cap allows replies for
            greedy.send_raw(request * 256)
    except (ConnectionError, OSError):
        dropped = True
    if not dropped:                                           # everything was accepted into socket buffers: the close shows on read
        time.sleep(1.5)                                       # the replies pile up while nobody reads
        total = 0
        try:
            while True:
                chunk = greedy.sock.recv(1 << 20)
                if not chunk:
                    break
                total += len(chunk)
        except (ConnectionError, OSError):
            pass
        assert total < wanted * 4 * per_reply                 # not every request was answered: the connection ended first
    assert good.sessions() == []
    greedy.close(); good.close()


def test_stop_with_live_sessions_and_clients(hl, tmp_path):
    path = str(tmp_path / "vocab.ggml")
    vocab = gb.tokenizer_vocab()
    gb.build(path, vocab, gb.minimal_tensors(vocab=len(vocab)))
    ctx = hl.LlavaContext()
    assert ctx.open_model_file(path)
    server = hl.LlavaServer(ctx)
    c = sc.Client(server.port)
    sids = [c.new_session() for _ in range(3)]
    assert c.sessions() == sids
    t0 = time.time()
    server.stop()                      # kills the three sessions, joins their threads, closes the connection
    assert time.time() - t0 < 5.0
    with pytest.raises((ConnectionError, OSError)):
        for _ in range(16):
            c.read_packet()
    c.close(); ctx.close()


def test_random_bytes_do_not_hurt_the_server(served):
    """whatever one client sends, the others are served: random packets with plausible headers, then pure noise"""
    import random
    server, _ = served
    rng = random.Random(5)
    good = sc.Client(server.port)
    sid = good.new_session()
    for round_ in range(20):
        bad = sc.Client(server.port, timeout=0.2)
        blob = b""
        for _ in range(50):
            command = rng.choice([0, 1, 2, 3, 15, 16, 17, 19, 20, 22, 23, 31, 32, 33, 34, 35, 36, 37, 38, 39, 1 << 31])
            length = rng.choice([0, 1, 3, 4, 5, 8, 9, 64])
            body = bytes(rng.getrandbits(8) for _ in range(length))
            if length >= 4 and rng.random() < 0.5:
                body = struct.pack("<I", rng.choice([sid, sid + 1, 0])) + body[4:]
            if command in (36, 37, 38) and len(body) > 4:
                body = body[:4] + b"/nonexistent-dir/" + bytes(b % 26 + 97 for b in body[4:])     # never a real path
            blob += struct.pack("<3I", command, rng.getrandbits(32), len(body)) + body
        if round_ % 2:
            blob += bytes(rng.getrandbits(8) for _ in range(rng.randrange(1, 4000)))
        try:
            bad.send_raw(blob)
        except OSError:
            pass
        bad.close()
        listed = good.sessions()
        assert listed == sorted(listed) and all(s >= sid for s in listed)     # random cmdNewSession packets may have added some
        if sid not in listed:                                                  # ... and a random cmdKillSession may have hit ours
            sid = good.new_session()
    assert good.ack(sc.SUBSCRIBE, sid) == sc.RC_OK
    good.close()
