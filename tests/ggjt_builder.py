"""Builds small GGJT (v1/v3) files byte by byte from Python, independently of the C model writer, so that parser
and tokenizer tests control every field (vocabulary pieces, scores, duplicate pieces, record order, padding)."""
import struct

import numpy as np

F32, F16, Q4_0, Q8_0 = 0, 1, 2, 8
MAGIC = 0x67676A74


def payload_bytes(ftype, n, version=3):
    return {F32: n * 4, F16: n * 2, Q4_0: n // 32 * (20 if version == 1 else 18), Q8_0: n // 32 * (36 if version == 1 else 34)}[ftype]


def build(path, vocab, tensors, dim=64, heads=2, layers=1, multiple_of=256, version=3, ftype=2, tail=b""):
    """vocab: list of (bytes, score); tensors: list of (name, ftype, shape tuple (rows, cols) or (n,), payload bytes or None
    for a seeded fill).  Returns {name: (offset, size)}."""
    out = bytearray()
    out += struct.pack("<9I", MAGIC, version, len(vocab), dim, multiple_of, heads, layers, dim // heads, ftype)
    for piece, score in vocab:
        out += struct.pack("<i", len(piece)) + piece + struct.pack("<f", score)
    where = {}
    rng = np.random.default_rng(1234)
    for name, ft, shape, data in tensors:
        nm = name.encode()
        if len(shape) == 2:
            rows, cols = shape
            out += struct.pack("<5I", 2, len(nm), ft, cols, rows)   # ne0 = columns is written first
            n = rows * cols
        else:
            out += struct.pack("<4I", 1, len(nm), ft, shape[0])
            n = shape[0]
        out += nm
        out += b"\0" * ((-len(out)) % 32)
        size = payload_bytes(ft, n, version)
        if data is None:
            data = rng.integers(0, 256, size, dtype=np.uint8).tobytes() if ft != F32 else rng.standard_normal(n).astype(np.float32).tobytes()
        assert len(data) == size, (name, len(data), size)
        where[name] = (len(out), size)
        out += data
    out += tail
    with open(path, "wb") as f:
        f.write(out)
    return where


def minimal_tensors(dim=64, ff=96, vocab=None, wtype=Q4_0):
    """the smallest tensor set every parser here accepts (it needs layers.0.feed_forward.w1 to learn the ff size)"""
    t = [("tok_embeddings.weight", F32, (vocab or 8, dim), None), ("norm.weight", F32, (dim,), None), ("output.weight", wtype, (vocab or 8, dim), None)]
    p = "layers.0."
    for nm, shape in [("attention.wq", (dim, dim)), ("attention.wk", (dim, dim)), ("attention.wv", (dim, dim)), ("attention.wo", (dim, dim)),
                      ("feed_forward.w1", (ff, dim)), ("feed_forward.w2", (dim, ff)), ("feed_forward.w3", (ff, dim))]:
        t.append((p + nm + ".weight", wtype, shape, None))
    t.append((p + "attention_norm.weight", F32, (dim,), None))
    t.append((p + "ffn_norm.weight", F32, (dim,), None))
    return t


def tokenizer_vocab():
    """A vocabulary that exercises the merge rules: byte tokens at ids 3..258, multi-byte pieces with distinct and with
    equal scores, a piece that occurs twice (the lower id must win), UTF-8 pieces and a piece only reachable through
    an intermediate merge."""
    v = [(b"<unk>", 0.0), (b"<s>", 0.0), (b"</s>", 0.0)]
    v += [(bytes([b]), -100.0 - b) for b in range(256)]            # ids 3..258
    extra = [
        (b"he", -1.0), (b"ll", -2.0), (b"lo", -2.0),                # 259, 260, 261: "ll" and "lo" tie on score
        (b"hell", -3.0), (b"hello", -4.0), (b"llo", -2.5),          # 262, 263, 264
        (b" w", -1.5), (b"or", -1.2), (b"ld", -1.1), (b"wor", -5.0), (b"world", -6.0), (b" world", -0.5),   # 265..270
        (b"ab", -7.0), (b"ab", -0.1),                               # 271, 272: same piece twice, the first id wins and ITS score counts
        (b"abab", -8.0),                                            # 273
        ("é".encode(), -9.0), ("日本".encode(), -9.5), ("日".encode(), -9.6), ("本".encode(), -9.7),  # 274..277
        (b"aa", -3.0), (b"aaa", -2.0), (b"aaaa", -1.0),             # 278..280
        (b"xyz", -0.2),                                             # 281: no "xy" or "yz" piece, so it can never be formed
    ]
    return v + extra


TOKENIZER_TEXTS = [
    "", "h", "hello", "hello world", "hellohello", " world", "world", "ab", "abab", "ababab", "aaaaaaa", "aaaa", "xyz", "xy",
    "é", "日本", "日本語", "héllo wörld", "\x00\x01\xff", "a" * 33, "llo", "lllo", "hell", "hel", "\xe6\x97",
]


def blocks_to_v1(blocks, ftype):
    """Re-encodes version-3 quantised blocks (fp16 scale; q4_0 byte j = elements j and j+16) as version-1 blocks
    (fp32 scale of the same value; q4_0 byte j = elements 2j and 2j+1).  The element values are unchanged, so a
    version-1 file made this way must give the same results as its version-3 source."""
    stride = 18 if ftype == Q4_0 else 34
    b = np.ascontiguousarray(blocks, dtype=np.uint8).reshape(-1, stride)
    scale = b[:, :2].copy().view(np.float16).astype(np.float32)             # exact widening
    codes = b[:, 2:]
    if ftype == Q4_0:
        elem = np.concatenate([codes & 15, codes >> 4], axis=1)             # elements 0..31 in order
        codes = (elem[:, 0::2] | (elem[:, 1::2] << 4)).astype(np.uint8)
    out = np.empty((b.shape[0], 4 + codes.shape[1]), dtype=np.uint8)
    out[:, :4] = scale.view(np.uint8).reshape(-1, 4)
    out[:, 4:] = codes
    return out.reshape(-1)


def convert_to_v1(src, dst, jitter_seed=None):
    """Rewrites a version-3 GGJT file as version 1, tensor by tensor, keeping names, shapes and vocabulary.  With
    jitter_seed every block scale is moved by up to 1 %, so that it needs the 24 bits of the fp32 a version-1 block holds
    (a converted scale alone is an fp16 value)."""
    rng = np.random.default_rng(jitter_seed) if jitter_seed is not None else None
    data = np.fromfile(src, dtype=np.uint8)
    hdr = np.frombuffer(data[:36].tobytes(), dtype=np.uint32).copy()
    assert hdr[0] == MAGIC and hdr[1] == 3
    cur = 36
    for _ in range(int(hdr[2])):
        ln = struct.unpack_from("<i", data, cur)[0]
        cur += 8 + ln
    hdr[1] = 1
    out = bytearray(hdr.tobytes()) + bytearray(data[36:cur].tobytes())
    while cur != data.shape[0]:
        n_dims, name_len, ft = struct.unpack_from("<3I", data, cur)
        head_len = 12 + 4 * n_dims + name_len
        ne = struct.unpack_from(f"<{n_dims}I", data, cur + 12)
        n = int(np.prod(ne))
        out += data[cur:cur + head_len].tobytes()
        out += b"\0" * ((-len(out)) % 32)
        cur = (cur + head_len + 31) & ~31
        size = payload_bytes(ft, n, 3)
        payload = data[cur:cur + size]
        if ft in (Q4_0, Q8_0):
            v1 = blocks_to_v1(payload, ft)
            if rng is not None:
                b = v1.reshape(-1, 20 if ft == Q4_0 else 36)
                scale = b[:, :4].copy().view(np.float32).reshape(-1)
                scale *= (1.0 + rng.uniform(-0.01, 0.01, scale.shape)).astype(np.float32)
                b[:, :4] = scale.view(np.uint8).reshape(-1, 4)
                v1 = b.reshape(-1)
            out += v1.tobytes()
        else:
            out += payload.tobytes()
        cur += size
    with open(dst, "wb") as f:
        f.write(out)
