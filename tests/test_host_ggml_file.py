"""Host-side ggml_file (model file parser + tokenizer) against
  * the committed golden vectors, which the REFERENCE's own ggml_file class produced (tests/golden/make_fixtures.py),
  * the reference-built parser itself where oracle/_ref/libref_ggml.so exists (build container only),
  * the oracle's independent GGJT reader,
and its behaviour on malformed files (reference: ggml_file.cpp:30-140 aborts through assert; this parser must
leave the object closed with a message instead).  No GPU is touched: libllava_hip.so is only loaded."""
import importlib
import json
import os
import struct

import numpy as np
import pytest

import ggjt_builder as gb

HERE = os.path.dirname(os.path.abspath(__file__))
GOLDEN = os.path.join(HERE, "golden")


@pytest.fixture(scope="module")
def hl():
    return importlib.import_module("llama-vulkan_amd.hostlib")


@pytest.fixture(scope="module")
def tok_file(hl, tmp_path_factory):
    gold = json.load(open(os.path.join(GOLDEN, "ggjt_tokenizer.json")))
    vocab = [(bytes.fromhex(p), s) for p, s in gold["vocab"]]
    assert vocab == gb.tokenizer_vocab(), "the fixture was generated from another vocabulary: re-run tests/golden/make_fixtures.py"
    path = str(tmp_path_factory.mktemp("tok") / "tok.ggml")
    gb.build(path, vocab, gb.minimal_tensors(vocab=len(vocab)))
    f = hl.GgmlFile(path)
    assert f.is_open(), f.error()
    yield f, gold, path
    f.close()


def test_tokenizer_matches_reference_vectors(tok_file):
    f, gold, _ = tok_file
    assert len(gold["cases"]) >= 50
    for case in gold["cases"]:
        raw = bytes.fromhex(case["text_hex"])
        ids = f.tokenize(raw, case["bos"])
        assert ids == case["ids"], (raw, case["bos"])
        assert f.detokenize(ids) == bytes.fromhex(case["detok_hex"]), raw


def test_tokenizer_invariants(tok_file):
    """facts that hold for any correct greedy-merge tokenizer over this vocabulary, independent of the fixture"""
    f, gold, _ = tok_file
    vocab = [bytes.fromhex(p) for p, _ in gold["vocab"]]
    rng = np.random.default_rng(3)
    alphabet = b"helo wrdabxyz\xc3\xa9"
    for n in (1, 2, 5, 17, 64, 300):
        raw = bytes(rng.choice(list(alphabet), n).tolist())
        for bos in (False, True):
            ids = f.tokenize(raw, bos)
            assert (ids[0] == 1) == bos
            body = ids[1:] if bos else ids
            assert b"".join(vocab[i] for i in body) == raw          # pieces concatenate back to the text
            assert 281 not in body                                  # "xyz" has no intermediate piece to grow from
            assert all(i != 272 for i in body)                      # the duplicate piece resolves to its first id
    assert f.tokenize(b"", False) == []
    assert f.tokenize(b"xyz", False) == [3 + ord("x"), 3 + ord("y"), 3 + ord("z")]   # unreachable without an intermediate piece


def test_tokenizer_against_reference_build(tok_file, orc):
    if not orc.ref_available():
        pytest.skip("reference-built parser only exists where /root/reference does")
    f, _, path = tok_file
    ref = orc.RefGgml(path)
    rng = np.random.default_rng(11)
    alphabet = list(b"helo wrdabxyz") + [0xC3, 0xA9, 0xE6, 0x97, 0xA5, 0xE6, 0x9C, 0xAC, 0, 255]
    for trial in range(200):
        raw = bytes(rng.choice(alphabet, int(rng.integers(0, 40))).tolist())
        for bos in (False, True):
            ids = ref.tokenize(raw, bos)
            assert f.tokenize(raw, bos) == ids, raw
            assert f.detokenize(ids) == ref.detokenize(ids)
    ref.close()


def _table_files(lva, tmp):
    gold = json.load(open(os.path.join(GOLDEN, "ggjt_table.json")))
    out = []
    for label, g in gold.items():
        p = os.path.join(tmp, label + ".ggml")
        if g["params"] is not None:
            lva.write_model(p, **g["params"])
        else:
            vocab = gb.tokenizer_vocab()
            gb.build(p, vocab[:40], gb.minimal_tensors(dim=64, ff=96, vocab=40, wtype=gb.Q8_0), dim=64, heads=2)
        out.append((label, p, g))
    return out


def test_parser_matches_reference_tables(hl, lva, orc, tmp_path):
    for label, p, g in _table_files(lva, str(tmp_path)):
        assert os.path.getsize(p) == g["file_size"], label      # the seeded writer is byte-stable
        f = hl.GgmlFile(p)
        assert f.is_open(), f.error()
        h = f.header()
        for k, v in g["header"].items():
            assert h[k] == v, (label, k)
        mine = {t["name"]: t for t in f.tensors()}
        assert len(mine) == len(g["tensors"]) == h["n_tensors"]
        for t in g["tensors"]:
            m = mine[t["name"]]
            assert {k: m[k] for k in ("ftype", "offset", "rows", "cols", "size")} == {k: t[k] for k in ("ftype", "offset", "rows", "cols", "size")}, (label, t["name"])
            short = t["name"][:-7] if t["name"].endswith(".weight") else t["name"]
            assert f.tensor(short)["offset"] == t["offset"]             # lookup without the ".weight" suffix
        with pytest.raises(KeyError):
            f.tensor("layers.99.attention.wq")
        assert h["vocab"] == g["vocab_size"]
        for i, (piece, score) in enumerate(g["vocab_head"]):
            assert f.token(i) == (bytes.fromhex(piece), score)
        for k, (piece, score) in enumerate(g["vocab_tail"]):
            assert f.token(h["vocab"] - len(g["vocab_tail"]) + k) == (bytes.fromhex(piece), score)
        # the oracle's reader and the package's numpy reader agree on every payload location too
        om = orc.Model(p)
        _, _, table = lva.read_ggjt_table(p)
        for name, ftype, offset, rows, cols, size in table:
            assert (mine[name]["ftype"], mine[name]["offset"], mine[name]["size"]) == (ftype, offset, size)
            assert om.tensor(name)["offset"] == offset
        om.close()
        f.close()


def test_parser_v1_blocks(hl, tmp_path):
    """file version 1 stores fp32 block scales (20/36-byte blocks); sizes follow (reference: ggml_file.cpp:95-122)"""
    p = str(tmp_path / "v1.ggml")
    where = gb.build(p, gb.tokenizer_vocab()[:16], gb.minimal_tensors(vocab=16), version=1)
    f = hl.GgmlFile(p)
    assert f.is_open(), f.error()
    assert f.header()["file_version"] == 1
    for t in f.tensors():
        assert (t["offset"], t["size"]) == where[t["name"]]
    f.close()


def _good_bytes(tmp_path):
    p = str(tmp_path / "good.ggml")
    gb.build(p, gb.tokenizer_vocab()[:16], gb.minimal_tensors(vocab=16))
    return open(p, "rb").read()


@pytest.mark.parametrize("case", ["missing", "empty", "short_header", "bad_magic", "zero_heads", "truncated_vocab", "huge_piece", "truncated_record",
                                  "three_dims", "unknown_type", "payload_past_end", "duplicate", "no_w1", "nul_in_name"])
def test_parser_rejects_malformed(hl, tmp_path, case):
    good = _good_bytes(tmp_path)
    vocab16 = gb.tokenizer_vocab()[:16]
    p = str(tmp_path / "bad.ggml")
    if case == "missing":
        p = str(tmp_path / "nothing_here.ggml")
    elif case == "empty":
        open(p, "wb").close()
    elif case == "short_header":
        open(p, "wb").write(good[:20])
    elif case == "bad_magic":
        open(p, "wb").write(b"GGUF" + good[4:])
    elif case == "zero_heads":
        open(p, "wb").write(good[:20] + struct.pack("<I", 0) + good[24:])
    elif case == "truncated_vocab":
        open(p, "wb").write(good[:60])
    elif case == "huge_piece":
        open(p, "wb").write(good[:36] + struct.pack("<I", 0x7FFFFFF0) + good[40:])
    elif case == "truncated_record":
        where = gb.build(p, vocab16, gb.minimal_tensors(vocab=16))
        first = min(o for o, _ in where.values())
        open(p, "wb").write(open(p, "rb").read()[:first - 40])
    elif case == "three_dims":
        gb.build(p, vocab16, [], tail=struct.pack("<6I", 3, 1, 0, 2, 2, 2) + b"x")
    elif case == "unknown_type":
        gb.build(p, vocab16, [], tail=struct.pack("<4I", 1, 1, 77, 32) + b"x" + b"\0" * 256)
    elif case == "payload_past_end":
        open(p, "wb").write(good[:-100])
    elif case == "duplicate":
        t = gb.minimal_tensors(vocab=16)
        gb.build(p, vocab16, t + [t[1]])
    elif case == "no_w1":
        gb.build(p, vocab16, [t for t in gb.minimal_tensors(vocab=16) if "w1" not in t[0]])
    elif case == "nul_in_name":
        gb.build(p, vocab16, gb.minimal_tensors(vocab=16) + [("a\0b", gb.F32, (8,), None)])
    f = hl.GgmlFile(p)
    assert not f.is_open()
    assert len(f.error()) > 8, case
    f.close()


def test_context_refuses_bad_model_without_touching_the_gpu(hl, tmp_path):
    c = hl.LlavaContext()
    assert not c.load_model(str(tmp_path / "absent.ggml"))
    assert "absent.ggml" in c.error()
    c.close()


def test_c_abi_exports_every_declared_symbol(lva):
    import ctypes
    lib = ctypes.CDLL(os.path.join(os.path.dirname(lva.__file__), "libllava_hip.so"))
    names = lva.exported_symbols()
    assert len(names) >= 40
    for n in names:
        assert hasattr(lib, n), f"include/llava_hip.h declares {n} but libllava_hip.so does not export it"


def test_every_python_file_of_the_package_compiles():
    """measure.py, build.py and bench.py only run on a GPU box: a syntax error in them must not wait for one"""
    import glob
    import py_compile
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    files = glob.glob(os.path.join(root, "*.py")) + glob.glob(os.path.join(root, "llama-vulkan_amd", "*.py")) + \
        glob.glob(os.path.join(root, "oracle", "*.py")) + glob.glob(os.path.join(root, "tests", "**", "*.py"), recursive=True)
    assert len(files) > 10
    for f in files:
        py_compile.compile(f, doraise=True)


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU; any other --gpus ends before anything touches a device, with a message that says so"""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "ONE GPU" in r.stderr and "--gpus 1" in r.stderr
    assert r.stdout.strip() == ""
