#!/usr/bin/env python3
"""Decode benchmark: LLaMA-7B-shaped q4_0, batch 1, greedy, ending at a 512-token context, on one MI355X.

A "step" is one decode token through the C-ABI (lv_step_begin -> lv_argmax), inputs already resident in HBM.
Prints ONE JSON line:

  value      tokens/s over the K timed steps (wall clock, host sampling included)
  roofline   the persistent decode kernel (one launch = one token): algorithmic bytes per launch / average launch
             duration measured with HIP events on the session's stream, against the 8 TB/s HBM peak
  cpu_baseline  the CPU checker (oracle/) timed on the same decode steps (same model, same tokens and positions; 64 steps are 10-15 s), on
             this box's host cores; reported beside the GPU number, never the target

Weights and prompt are synthetic (seeded writer, llama-vulkan_amd/mkggml.c).
"""
import argparse
import importlib
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

CONTEXT = 512
HBM_PEAK_GBS = 8000.0
SHAPE = dict(vocab=32000, dim=4096, heads=32, layers=32, ff=11008)


def recorded_traffic():
    """HBM bytes per launch of the decode kernel as counted by the hardware (FETCH_SIZE + WRITE_SIZE, calibrated on a
    plain copy): a figure from a separate rocprofv3 --pmc run, kept with its commands under profiles/; None if absent."""
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", "mega_decode_kernel_7b_q4_0_ctx512_pmc.md")
    try:
        m = re.search(r"^traffic_bytes_per_launch = (\d+)", open(path).read(), re.M)
        return int(m.group(1)) if m else None
    except OSError:
        return None


def algorithmic_bytes(pos):
    """HBM bytes one decode step at cache position `pos` has to move: GGML storage cost of every weight
    (18 B / 32 weights), fp32 norm vectors, the fp16 K/V rows 0..pos of all layers, the new K/V row, the embedding
    row in and the logits out."""
    D, F, V, L = SHAPE["dim"], SHAPE["ff"], SHAPE["vocab"], SHAPE["layers"]
    per_layer = (4 * D * D + 3 * D * F) // 32 * 18
    weights = L * per_layer + V * D // 32 * 18
    norms = (2 * L + 1) * D * 4
    kv_read = L * 2 * D * 2 * (pos + 1)
    kv_write = L * 2 * D * 2
    return weights + norms + kv_read + kv_write + V * 4 + D * 4


def model_path():
    base = "/dev/shm" if os.access("/dev/shm", os.W_OK) else "/tmp"
    return os.path.join(base, "llava_bench_7b_q4_0_seed0.ggml")


def prefill_report(n, ms):
    """the prompt of n tokens as one batched step (MFMA GEMM on integer codes, batched attention): useful flops are
    2 * n * layer weights + 2 * output matrix (the head sees the last row only) and frac_of_mfma_peak counts those; the GEMM
    executes every product twice (activations split in two fp16 halves), so the matrix cores run at twice that rate
    (executed_frac)"""
    D, F, V, L = SHAPE["dim"], SHAPE["ff"], SHAPE["vocab"], SHAPE["layers"]
    flops = 2.0 * n * L * (4 * D * D + 3 * D * F) + 2.0 * V * D
    tf = flops / (ms * 1e-3) / 1e12
    return {"tokens": n, "ms": round(ms, 3), "tok_s": round(n / ms * 1e3, 1), "useful_tflops": round(tf, 1),
            "executed_tflops": round(2 * tf, 1), "mfma_peak_tflops": 2500.0, "frac_of_mfma_peak": round(tf / 2500.0, 4),
            "executed_frac": round(2 * tf / 2500.0, 4)}


def lavapipe_status():
    """The baseline this metric would ideally sit beside is the reference's own Vulkan build run on the host cores by Mesa
    lavapipe.  That needs a Vulkan loader, the lavapipe ICD, a GLSL compiler for the 30 shaders and the reference's
    sources, and a patched device selection (the reference accepts discrete and integrated GPUs only,
    llava_context.cpp:36-60).  Reports what is missing on this machine."""
    import ctypes.util
    import glob
    import shutil
    missing = []
    if not ctypes.util.find_library("vulkan"):
        missing.append("no libvulkan")
    if not glob.glob("/usr/share/vulkan/icd.d/*lvp*") and not glob.glob("/etc/vulkan/icd.d/*lvp*"):
        missing.append("no lavapipe ICD")
    if not (shutil.which("glslc") or shutil.which("glslangValidator")):
        missing.append("no GLSL compiler")
    missing.append("the reference's sources and build are not on this machine")
    return "unavailable: " + ", ".join(missing)


def other_cases(lva, ctx, headline_picks=None, headline_first=0):
    """The other configurations under the same clock, after the headline's timed region: isolated GEMVs at the 7B decode
    shapes in both weight types, the 512-token GEMM at the 13B layer shapes, 7B q8_0 at positions 1920..2047, 13B q4_0 with a 32-token prompt and 256 steps (on the
    persistent kernel and on the hipGraph of the operator chain, which have to pick the same tokens), the 7B q4_0 headline
    workload on the hipGraph path (same tokens as the headline run), and the 13B q8_0 512-token prompt.  Each entry carries
    tok_s or ms or us, and frac of the roofline that bounds it (HBM for decode and GEMV; matrix cores for the prompt, where
    frac counts the flops the work needs and executed_frac the flops the kernel issues).  A case that fails leaves an
    entry with its error and the others still run."""
    measure = importlib.import_module("llama-vulkan_amd.measure")
    q = measure.quiet
    cases = []

    def attempt(name, fn):
        try:
            fn()
        except Exception as e:       # a side case must not take the measured headline with it
            cases.append({"name": name, "error": f"{type(e).__name__}: {e}"})

    def gemvs():
        for g in measure.gemv_cases(ctx, report=q):
            cases.append({"name": f"gemv {g['wtype']} {g['rows']}x{g['cols']} {g['mode']}", "us": g["us"], "GBps": g["GBps"], "frac": g["frac_of_peak"],
                          "bound": "hbm"})
    attempt("gemv", gemvs)
    picks = {}
    for name, key, other, args, kw in (
            ("7B q8_0 decode, positions 1920..2047", "q8", None, ("decode-q8", "7b", lva.LV_Q8_0, 1, 2048, 1916, 128), {}),
            ("13B q4_0 decode, 32-token prompt + 256 steps, persistent kernel", "13b", None, ("decode-13b", "13b", lva.LV_Q4_0, 2, 512, 32, 256), {}),
            ("13B q4_0 decode, 32-token prompt + 256 steps, hipGraph", "13b-graph", "13b", ("decode-13b-graph", "13b", lva.LV_Q4_0, 2, 512, 32, 256),
             {"force_path": lva.PATH_GRAPH}),
            ("7B q4_0 decode, positions 444..511, hipGraph", "7b-graph", "headline", ("decode-7b-graph", "7b", lva.LV_Q4_0, 0, 512, 440, 68),
             {"force_path": lva.PATH_GRAPH})):
        def decode(name=name, key=key, other=other, args=args, kw=kw):
            expect = picks.get(other)
            if other == "headline" and headline_picks is not None and headline_first >= args[5]:
                # the headline's run fed headline_picks[i] at position headline_first + i; this case starts feeding at args[5]
                expect = [None] * (headline_first - args[5]) + list(headline_picks)
            d = measure.decode_case(ctx, *args, report=q, expect_picks=_known(expect), **kw)
            picks[key] = d["picks"]
            cases.append({"name": name, "path": d["path"], "tok_s": d["tok_s"], "ms": d["ms_per_token"], "GBps": d["GBps"], "frac": d["frac_of_peak"],
                          "bound": "hbm", "same_tokens_as": None if expect is None else other})
        attempt(name, decode)

    def gemms():
        for g in measure.gemm_cases(ctx, report=q):
            cases.append({"name": f"gemm {g['wtype']} {g['rows']}x{g['cols']}, {g['tokens']} tokens (one lv_kernel_gemm call)", "us": g["us"],
                          "useful_TFLOPs": g["useful_TFLOPs"], "executed_TFLOPs": g["executed_TFLOPs"], "frac": g["frac_of_mfma_peak"],
                          "executed_frac": g["executed_frac"], "bound": "mfma"})
    attempt("gemm", gemms)

    def prompt():
        p = measure.prefill_case(ctx, "prefill-13b", "13b", lva.LV_Q8_0, report=q)
        cases.append({"name": "13B q8_0 prompt of 512 tokens as one step", "tok_s": p["tok_s"], "ms": p["ms"], "useful_TFLOPs": p["TFLOPs"],
                      "executed_TFLOPs": p["executed_TFLOPs"], "frac": p["frac_of_mfma_peak"], "executed_frac": p["executed_frac"], "bound": "mfma"})
    attempt("13B q8_0 prompt of 512 tokens as one step", prompt)
    return cases


class _Any:
    """compares equal to every token: positions of another run's pick list that this run does not cover"""
    def __eq__(self, other):
        return True

    def __ne__(self, other):
        return False


def _known(expect):
    return None if expect is None else [_Any() if t is None else t for t in expect]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--cpu-steps", type=int, default=64, help="decode steps the CPU checker is timed on, the last ones of the timed region (0 = skip)")
    ap.add_argument("--no-cases", action="store_true", help="skip the other configurations (the \"cases\" key)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs the decode path on ONE GPU (batch-1 decode has nothing to shard in this "
                 "round); run it with --gpus 1")
    if args.steps < 1 or args.warmup < 0 or args.steps + args.warmup >= CONTEXT:
        sys.exit(f"bench.py: need 1 <= steps and steps + warmup < {CONTEXT}")

    lva = importlib.import_module("llama-vulkan_amd")
    ctx = lva.Context(0)
    device, cus, _ = ctx.info()

    path = model_path()
    if not os.path.exists(path):
        lva.write_model(path + ".tmp", wtype=lva.LV_Q4_0, seed=0, **SHAPE)
        os.replace(path + ".tmp", path)
    model = lva.Model(ctx, path)
    sess = lva.Session(model, CONTEXT)
    path_kind = {lva.PATH_KERNELS: "kernels", lva.PATH_GRAPH: "graph", lva.PATH_PERSISTENT: "persistent"}[sess.path()]

    # fill the cache up to the first warm-up position with a seeded prompt, then decode greedily
    first = CONTEXT - args.steps - args.warmup
    prompt = lva.synth_tokens(first, 3, SHAPE["vocab"], seed=0)
    sess.begin(prompt, 0)            # untimed: allocates the prompt workspace
    sess.wait()
    sess.timer_start()
    sess.begin(prompt, 0)            # the same rows again, timed with HIP events on the session's stream
    prefill_ms = sess.timer_stop()
    tok = sess.argmax()
    pos = first
    for _ in range(args.warmup):
        sess.begin([tok], pos)
        tok = sess.argmax()
        pos += 1

    # ---- timed region: K steps, synchronised on both sides -------------------------------------------------
    timed_first = pos
    tokens = [tok]
    sess.wait()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        sess.begin([tok], pos)
        tok = sess.argmax()          # the kernel leaves its greedy pick in pinned memory: the sampler is inside the step
        tokens.append(tok)
        pos += 1
    sess.wait()
    dt = time.perf_counter() - t0
    tok_s = args.steps / dt

    # ---- the dominant kernel by itself: same steps again (same cache rows, same tokens), one event pair each ----
    kern_ms = []
    for i in range(args.steps):
        sess.timer_start()
        sess.begin([tokens[i]], timed_first + i)
        kern_ms.append(sess.timer_stop())
    avg_ms = sum(kern_ms) / len(kern_ms)
    avg_bytes = sum(algorithmic_bytes(timed_first + i) for i in range(args.steps)) / args.steps
    achieved = avg_bytes / (avg_ms * 1e-3) / 1e9

    # ---- CPU baseline: the checker on the same model, cache restored from the GPU session, last positions ------
    cpu = None
    if args.cpu_steps > 0:
        import numpy as np
        import oracle
        n_cpu = min(args.cpu_steps, args.steps)
        start = pos - n_cpu
        om = oracle.Model(path)
        osess = oracle.Session(om, CONTEXT)
        for layer in range(SHAPE["layers"]):
            for which in (0, 1):
                osess.kv_load(layer, which, sess.kv(layer, which, start))
        osess.set_pos(start)
        differing = []
        t1 = time.perf_counter()
        for i in range(n_cpu):
            want = osess.eval([tokens[start - timed_first + i]])
            tok_cpu = oracle.greedy(want)
            tok_gpu = tokens[start - timed_first + i + 1]
            if tok_cpu != tok_gpu:
                differing.append((start + i, tok_gpu, tok_cpu, want.copy()))
        cpu_dt = time.perf_counter() - t1
        # logits of the last step, GPU against checker
        bar = lambda w: min(1e-2, 1e-3 * float(np.max(np.abs(w))))
        sess.begin([tokens[pos - 1 - timed_first]], pos - 1)
        worst = float(np.max(np.abs(sess.logits() - want)))
        if not worst <= bar(want):
            raise SystemExit(f"bench.py: logits differ from the CPU checker by {worst}")
        # A different pick is an error unless it is a tie inside the arithmetic's own noise: the step is run again on the GPU
        # (same cache rows, same token), its logits have to agree with the checker's within the bar, and the checker's two
        # candidates may be no further apart than twice the difference measured between the two sets of logits.
        for p_, tok_gpu, tok_cpu, w in differing:
            sess.begin([tokens[p_ - timed_first]], p_)
            d = float(np.max(np.abs(sess.logits() - w)))
            if not (d <= bar(w) and float(w[tok_cpu] - w[tok_gpu]) <= 2 * d):
                raise SystemExit(f"bench.py: greedy token at position {p_} differs from the CPU checker ({tok_gpu} vs {tok_cpu}; "
                                 f"logits differ by {d}, the checker's candidates by {float(w[tok_cpu] - w[tok_gpu])})")
        ties = len(differing)
        cpu = {"value": round(n_cpu / cpu_dt, 3), "unit": "tok/s", "cores": oracle.num_threads(), "kind": "port",
               "sample": f"{n_cpu} greedy decode steps of the same model at positions {start}..{pos - 1} "
                         f"(cache restored from the GPU run; "
                         + ("tokens identical" if ties == 0 else f"picks differ at positions {[d[0] for d in differing]}, each a tie within twice the measured logit difference")
                         + f", max |dlogit| of the last step {worst:.1e})",
               "lavapipe": lavapipe_status()}
        osess.close()
        om.close()

    out = {
        "metric": "decode tok/s LLaMA-7B q4_0 bs1 on 1 MI355X; achieved HBM GB/s vs peak",
        "value": round(tok_s, 2),
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(dt / args.steps * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": f"LLaMA-7B-shaped q4_0 GGJT (dim 4096, 32 layers, 32 heads, ff 11008, vocab 32000, seed 0), "
                               f"batch 1 greedy decode, cache positions {timed_first}..{pos - 1} of a {CONTEXT}-token context",
                   "decode_path": path_kind, "device": device, "compute_units": cus},
        "roofline": {"bound": "hbm", "kernel": "mega_decode_kernel (one launch per token)" if path_kind == "persistent" else "decode step (all launches)",
                     "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "algorithmic_bytes_per_launch": int(avg_bytes), "avg_launch_ms": round(avg_ms, 4), "traffic": recorded_traffic()},
        "cpu_baseline": cpu,
        "prefill": prefill_report(first, prefill_ms),
    }
    sess.close()
    model.close()
    # the second denominator: what a kernel that only reads memory reaches on this very device, measured now
    measure = importlib.import_module("llama-vulkan_amd.measure")
    try:
        stream = measure.read_stream_case(ctx, report=measure.quiet)["GBps"]
        out["roofline"]["achievable"] = stream
        out["roofline"]["achievable_by"] = "lv_dev_read: 4 GiB read 8 times by a kernel that only reads (16-byte non-temporal loads)"
        out["roofline"]["frac_of_achievable"] = round(achieved / stream, 4)
    except Exception as e:
        out["roofline"]["achievable"] = None
        out["roofline"]["achievable_error"] = f"{type(e).__name__}: {e}"
    if not args.no_cases:
        out["cases"] = other_cases(lva, ctx, headline_picks=tokens, headline_first=timed_first)
    print(json.dumps(out), flush=True)
    ctx.close()


if __name__ == "__main__":
    main()
