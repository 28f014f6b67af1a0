#!/usr/bin/env python3
"""Writes the golden fixtures under tests/golden/ with the REFERENCE's own ggml_file class (compiled from the
reference sources by oracle/Makefile into oracle/_ref/libref_ggml.so).  Run in the build container, where
/root/reference exists; the GPU box only reads the committed JSON.

    python tests/golden/make_fixtures.py

Fixtures:
  ggjt_tokenizer.json   ids the reference tokenizer produces for a fixed vocabulary and a list of texts (with and
                        without BOS), and the text it re-assembles from them
  ggjt_table.json       header fields and the full tensor table the reference parser reads from a seeded tiny model
                        written by llama-vulkan_amd/mkggml.c and from a hand-built file
"""
import importlib
import json
import os
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

import ggjt_builder as gb  # noqa: E402
import oracle              # noqa: E402


def main():
    if not oracle.ref_available():
        sys.exit("oracle/_ref/libref_ggml.so is missing: run `make -C oracle ref` where /root/reference exists")
    lva = importlib.import_module("llama-vulkan_amd")
    with tempfile.TemporaryDirectory() as tmp:
        # ---- tokenizer ----
        vocab = gb.tokenizer_vocab()
        path = os.path.join(tmp, "tok.ggml")
        gb.build(path, vocab, gb.minimal_tensors(vocab=len(vocab)))
        ref = oracle.RefGgml(path)
        cases = []
        for text in gb.TOKENIZER_TEXTS:
            raw = text.encode("utf-8")
            for bos in (False, True):
                ids = ref.tokenize(raw, bos)
                cases.append({"text_hex": raw.hex(), "bos": bos, "ids": ids, "detok_hex": ref.detokenize(ids).hex()})
        # raw byte strings that are not valid UTF-8
        for raw in (b"\x00\x01\xff", b"\xe6\x97", b"\xf0\x9f", b"ab\xc3"):
            for bos in (False, True):
                ids = ref.tokenize(raw, bos)
                cases.append({"text_hex": raw.hex(), "bos": bos, "ids": ids, "detok_hex": ref.detokenize(ids).hex()})
        ref.close()
        json.dump({"vocab": [[p.hex(), s] for p, s in vocab], "cases": cases}, open(os.path.join(HERE, "ggjt_tokenizer.json"), "w"), indent=0)

        # ---- tensor tables ----
        tables = {}
        tiny = os.path.join(tmp, "tiny.ggml")
        lva.write_model(tiny, wtype=lva.LV_Q4_0, seed=5, vocab=512, dim=256, heads=4, layers=2, ff=704)
        tiny8 = os.path.join(tmp, "tiny8.ggml")
        lva.write_model(tiny8, wtype=lva.LV_Q8_0, seed=6, vocab=300, dim=128, heads=1, layers=1, ff=160)
        hand = os.path.join(tmp, "hand.ggml")
        gb.build(hand, vocab[:40], gb.minimal_tensors(dim=64, ff=96, vocab=40, wtype=gb.Q8_0), dim=64, heads=2)
        for label, p, params in [("mkggml_tiny_q4_seed5", tiny, dict(wtype=2, seed=5, vocab=512, dim=256, heads=4, layers=2, ff=704)),
                                 ("mkggml_tiny_q8_seed6", tiny8, dict(wtype=8, seed=6, vocab=300, dim=128, heads=1, layers=1, ff=160)),
                                 ("hand_built_q8", hand, None)]:
            ref = oracle.RefGgml(p)
            _, _, table = lva.read_ggjt_table(p)   # only for the list of names to ask the reference about
            entries = []
            for name, *_ in table:
                d = ref.tensor(name)
                short = name[:-7] if name.endswith(".weight") else name
                assert ref.tensor(short) == d      # the ".weight" fallback
                entries.append({"name": name, **d})
            voc = ref.vocab()
            tables[label] = {"params": params, "header": ref.header(), "tensors": entries, "file_size": os.path.getsize(p),
                             "vocab_size": len(voc), "vocab_head": [[t.hex(), s] for t, s in voc[:8]], "vocab_tail": [[t.hex(), s] for t, s in voc[-3:]]}
            ref.close()
        json.dump(tables, open(os.path.join(HERE, "ggjt_table.json"), "w"), indent=0)
    print("wrote ggjt_tokenizer.json, ggjt_table.json")


if __name__ == "__main__":
    main()
