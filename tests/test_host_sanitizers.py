"""AddressSanitizer + UndefinedBehaviorSanitizer over the host parser and tokenizer (llama-vulkan_amd/host/ggml_file.cpp,
the part of the host that reads untrusted bytes): a valid file, the same file cut at every interesting length, and the
same file with bytes flipped in the header, the vocabulary and the tensor records.  The parser must refuse or accept each
of them without reading outside the mapping (the reference asserts or exits on malformed files, ggml_file.cpp:104-115)."""
import os
import shutil
import subprocess

import numpy as np
import pytest

import ggjt_builder as gb

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HOST = os.path.join(ROOT, "llama-vulkan_amd", "host")


@pytest.fixture(scope="module")
def driver(tmp_path_factory):
    if not shutil.which("g++"):
        pytest.skip("no g++")
    exe = str(tmp_path_factory.mktemp("san") / "host_sanitize")
    cmd = ["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=all", "-static-libasan",
           "-static-libubsan", "-I", HOST, os.path.join(ROOT, "tests", "host_sanitize_main.cpp"), os.path.join(HOST, "ggml_file.cpp"),
           os.path.join(HOST, "utils.cpp"), "-o", exe]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        pytest.skip("sanitizer build unavailable here: " + r.stderr[-400:])
    return exe


def run(exe, paths):
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="halt_on_error=1:print_stacktrace=1")
    return subprocess.run([exe, *paths], capture_output=True, text=True, env=env, timeout=300)


def test_parser_and_tokenizer_under_sanitizers(driver, tmp_path):
    good = str(tmp_path / "good.ggml")
    vocab = gb.tokenizer_vocab()
    where = gb.build(good, vocab, gb.minimal_tensors(vocab=len(vocab)))
    data = np.fromfile(good, dtype=np.uint8)
    first_tensor = min(off for off, _ in where.values())
    first_record = 36 + sum(8 + len(piece) for piece, _ in vocab)   # the first tensor record follows the vocabulary
    paths = [good]
    # truncations: inside the header, inside the vocabulary, inside a tensor record, inside a payload, one byte short
    cuts = [0, 1, 35, 36, 40, 200, first_tensor - 40, first_tensor - 1, first_tensor, first_tensor + 100, len(data) // 2, len(data) - 1]
    for n in cuts:
        p = str(tmp_path / f"cut_{n}.ggml")
        data[:n].tofile(p)
        paths.append(p)
    # byte flips and hostile field values, each in a copy of its own
    rng = np.random.default_rng(7)
    record_zone = np.arange(36, min(first_tensor + 4096, len(data)))
    for k in range(160):
        mutated = data.copy()
        if k < 40:
            at = int(rng.integers(0, 36))                      # header words: version, vocab size, dims, counts
            mutated[at] = rng.integers(0, 256)
        elif k < 80:
            at = int(rng.choice(record_zone))
            mutated[at] ^= 1 << int(rng.integers(0, 8))
        else:
            at = int(rng.choice(record_zone)) & ~3
            mutated[at:at + 4] = np.frombuffer(np.uint32(rng.choice([0xFFFFFFFF, 0x80000000, 0x7FFFFFFF, 0, 1 << 20])).tobytes(), dtype=np.uint8)
        p = str(tmp_path / f"mut_{k}.ggml")
        mutated.tofile(p)
        paths.append(p)
    # size fields far beyond the file: a 100-byte file whose header claims 2^31-1 or 2^32-1 tokens, the full file with the
    # same claim, a first token and a first tensor name of such a length.  None may be sized by the claim before it is checked.
    for k, value in enumerate([0x7FFFFFFF, 0xFFFFFFFF, 0x10000000]):
        word = np.frombuffer(np.uint32(value).tobytes(), dtype=np.uint8)
        for label, base, at in [("vocab_short", data[:100], 8), ("vocab_full", data, 8), ("toklen", data, 36), ("namelen", data, first_record + 4)]:
            mutated = base.copy()
            mutated[at:at + 4] = word
            p = str(tmp_path / f"huge_{label}_{k}.ggml")
            mutated.tofile(p)
            paths.append(p)
    r = run(driver, paths)
    assert r.returncode == 0, (r.stdout[-500:], r.stderr[-3000:])
    assert "opened" in r.stdout
    opened = int(r.stdout.split()[1])
    assert 1 <= opened < len(paths)        # the valid file parses; the truncated ones cannot all parse
