#!/usr/bin/env python3
"""Measurements of the decode path beyond the headline bench: one JSON line per case.

    python llama-vulkan_amd/measure.py gemv          isolated dequant-fused GEMVs at the 7B shapes, q4_0 and q8_0
    python llama-vulkan_amd/measure.py attention     the one-token attention kernel by itself (7B heads) over 512 and 2048 cache rows
    python llama-vulkan_amd/measure.py decode-q8     7B q8_0, cache positions 1920..2047 (128 greedy steps)
    python llama-vulkan_amd/measure.py decode-q8-graph    the same on the hipGraph of the operator chain (attention_kernel over 2048 rows)
    python llama-vulkan_amd/measure.py gemv-13b      the same GEMVs at the 13B layer shapes
    python llama-vulkan_amd/measure.py decode-13b    13B q4_0, 32-token prompt + 256 greedy steps (persistent kernel)
    python llama-vulkan_amd/measure.py decode-13b-graph   the same on the hipGraph of the operator chain
    python llama-vulkan_amd/measure.py decode-7b-graph    7B q4_0, positions 444..511 on the hipGraph of the operator chain
    python llama-vulkan_amd/measure.py prefill-13b   13B q8_0, 512-token prompt evaluated in one lv_step_begin
    python llama-vulkan_amd/measure.py prefill-7b    7B q4_0, the same
    python llama-vulkan_amd/measure.py prefill-13b-q4  13B q4_0, the same
    python llama-vulkan_amd/measure.py gemm          isolated 512-token GEMMs at the 13B shapes, q8_0 (for kernel traces and counters)
    python llama-vulkan_amd/measure.py copy          1 GiB device-to-device copy: achievable bandwidth, counter calibration
    python llama-vulkan_amd/measure.py read-stream   4 GiB read by a kernel that only reads: the bandwidth a weight stream can reach
    python llama-vulkan_amd/measure.py all

Every figure is algorithmic bytes (weights as stored in the GGML file, 18 B / 34 B per 32 weights, plus vectors and the
fp16 cache rows a step reads) divided by the time measured with HIP events on the stream that runs the kernels.
Models are seeded synthetic GGJT files written to /dev/shm (or /tmp) on first use.  Every case function returns its
figures as a dict (bench.py collects them under "cases"); run as a script, each is printed as one JSON line."""
import importlib
import json
import os
import sys
import time

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
lva = importlib.import_module("llama-vulkan_amd")
HBM_PEAK_GBS = 8000.0
SHAPES = {"7b": dict(vocab=32000, dim=4096, heads=32, layers=32, ff=11008), "13b": dict(vocab=32000, dim=5120, heads=40, layers=40, ff=13824)}


def emit(**kw):
    print(json.dumps({k: v for k, v in kw.items() if k != "picks"}), flush=True)
    return kw


def block_bytes(ftype):
    return 18 if ftype == lva.LV_Q4_0 else 34


GEMV_SHAPES_7B = ((4096, 4096, "store"), (11008, 4096, "silu"), (4096, 11008, "add"), (32000, 4096, "store"))
GEMV_SHAPES_13B = ((5120, 5120, "store"), (13824, 5120, "silu"), (5120, 13824, "add"), (32000, 5120, "store"))


def gemv_cases(ctx, report=emit, shapes=GEMV_SHAPES_7B):
    """reference: matmul.glsl / matmul_q8.glsl / matmul_silu_ff.comp at the three layer shapes and the output matrix"""
    out_cases = []
    for ftype, tname in ((lva.LV_Q4_0, "q4_0"), (lva.LV_Q8_0, "q8_0")):
        for rows, cols, mode in shapes:
            nbytes = rows * cols // 32 * block_bytes(ftype) * (2 if mode == "silu" else 1) + 4 * cols + 4 * rows * (2 if mode == "add" else 1)
            # enough distinct matrices that the working set exceeds the 256 MB last-level cache
            nmat = max(2, min(12, int(1.5e9 // nbytes)))
            mats = []
            for i in range(nmat * (2 if mode == "silu" else 1)):
                mats.append(ctx.matrix(lva.synth_quant(ftype, rows, cols, seed=100 + i), ftype, rows, cols))
            x = ctx.to_device(lva.synth_normal(1, cols, seed=1))
            out = ctx.zeros(rows * 4)

            def run(i):
                if mode == "silu":
                    lva.check(ctx.lib.lv_kernel_gemv_silu(ctx.h, out, mats[2 * i], mats[2 * i + 1], x, 1))
                else:
                    lva.check(ctx.lib.lv_kernel_gemv(ctx.h, out, mats[i], x, 1, 1 if mode == "add" else 0))
            for i in range(nmat):
                run(i)
            ctx.sync()
            iters = 20
            ctx.timer_start()
            for _ in range(iters):
                for i in range(nmat):
                    run(i)
            us = ctx.timer_stop() * 1e3 / (iters * nmat)
            out_cases.append(report(case="gemv", wtype=tname, rows=rows, cols=cols, mode=mode, us=round(us, 2), algorithmic_bytes=nbytes,
                                    GBps=round(nbytes / us / 1e3, 1), frac_of_peak=round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4)))
            for m in mats:
                ctx.matrix_free(m)
            ctx.free(x)
            ctx.free(out)
    return out_cases


def quiet(**kw):
    return kw


def attention_cases(ctx, report=emit):
    """reference: mhsa.comp + softmax.comp + kqv_matching.comp for one query.  32 heads of 128 at the last row of a 512- and
    of a 2048-row cache; algorithmic bytes = the fp16 K and V rows 0..pos (4 * (pos + 1) * dim bytes) plus q in and out.
    Sixteen caches in turn (0.5 / 2 GB), so that the rows come from HBM."""
    import numpy as np
    out_cases = []
    heads, rot = 32, 128
    dim = heads * rot
    for backlog in (512, 2048):
        pos = backlog - 1
        ncache = 16
        rng = np.random.default_rng(backlog)
        host = (rng.standard_normal((backlog, dim)) * 0.5).astype(np.float16)
        ks = [ctx.to_device(host) for _ in range(ncache)]
        vs = [ctx.to_device(host) for _ in range(ncache)]
        q = ctx.to_device(lva.synth_normal(1, dim, seed=3))
        out = ctx.zeros(dim * 4)
        for i in range(ncache):
            lva.check(ctx.lib.lv_kernel_attention(ctx.h, out, ks[i], vs[i], q, pos, backlog, heads, rot, 1))
        ctx.sync()
        iters = 20
        ctx.timer_start()
        for _ in range(iters):
            for i in range(ncache):
                lva.check(ctx.lib.lv_kernel_attention(ctx.h, out, ks[i], vs[i], q, pos, backlog, heads, rot, 1))
        us = ctx.timer_stop() * 1e3 / (iters * ncache)
        nbytes = 4 * (pos + 1) * dim + 8 * dim
        out_cases.append(report(case="attention", heads=heads, head_size=rot, rows=pos + 1, us=round(us, 2), algorithmic_bytes=nbytes,
                                GBps=round(nbytes / us / 1e3, 1), frac_of_peak=round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4)))
        for b in ks + vs + [q, out]:
            ctx.free(b)
    return out_cases


def attention_batch_cases(ctx, report=emit):
    """The prompt form of the same chain (lv_kernel_attention with 16 rows or more: attention_prepare_kernel, then
    attention_batch_kernel): n query rows at cache positions pos .. pos+n-1, 13B and 7B head counts.  Useful flops =
    4 * head_size * sum over the rows of the positions each sees (scores and sums, a multiply-add = 2); the kernels execute 4 x
    that (3 + 5 products of 16-bit operand pieces)."""
    import numpy as np
    out_cases = []
    rot = 128
    for heads, pos, n in ((40, 0, 512), (32, 0, 512), (40, 1536, 512), (40, 0, 128)):
        dim, backlog = heads * rot, 2048
        rng = np.random.default_rng(heads + pos)
        host = (rng.standard_normal((backlog, dim)) * 0.5).astype(np.float16)
        k, v = ctx.to_device(host), ctx.to_device(host)
        q = ctx.to_device(lva.synth_normal(n, dim, seed=3))
        out = ctx.zeros(n * dim * 4)
        for _ in range(3):
            lva.check(ctx.lib.lv_kernel_attention(ctx.h, out, k, v, q, pos, backlog, heads, rot, n))
        ctx.sync()
        iters = 50
        ctx.timer_start()
        for _ in range(iters):
            lva.check(ctx.lib.lv_kernel_attention(ctx.h, out, k, v, q, pos, backlog, heads, rot, n))
        us = ctx.timer_stop() * 1e3 / iters
        pairs = sum(pos + z + 1 for z in range(n))
        flops = 4.0 * rot * pairs * heads
        out_cases.append(report(case="attention-batch", heads=heads, head_size=rot, first_position=pos, rows=n, us_both_kernels=round(us, 2),
                                useful_TFLOPs=round(flops / us / 1e6, 1), executed_TFLOPs=round(4 * flops / us / 1e6, 1)))
        for b in (k, v, q, out):
            ctx.free(b)
    return out_cases


def copy_case(ctx):
    n = 1 << 30
    src, dst = ctx.zeros(n), ctx.zeros(n)
    lva.check(ctx.lib.lv_dev_copy(ctx.h, dst, src, n))
    ctx.sync()
    ctx.timer_start()
    for _ in range(4):
        lva.check(ctx.lib.lv_dev_copy(ctx.h, dst, src, n))
    ms = ctx.timer_stop() / 4
    emit(case="copy", bytes_read=n, bytes_written=n, ms=round(ms, 4), GBps_read_plus_write=round(2 * n / ms / 1e6, 1))
    ctx.free(src)
    ctx.free(dst)


def read_stream_case(ctx, report=emit, gib=4):
    """What a kernel that only reads memory reaches on this device (lv_dev_read: contiguous share per workgroup, 16-byte
    non-temporal loads, eight in flight): a buffer far larger than the 256 MB last-level cache, read 8 times.  The decode
    kernel's bytes per second are reported against this figure as well as against the 8 TB/s of the datasheet."""
    n = gib << 30
    src = ctx.zeros(n)
    lva.check(ctx.lib.lv_dev_read(ctx.h, src, n))
    ctx.sync()
    reps = 8
    ctx.timer_start()
    for _ in range(reps):
        lva.check(ctx.lib.lv_dev_read(ctx.h, src, n))
    ms = ctx.timer_stop() / reps
    ctx.free(src)
    return report(case="read-stream", bytes_read=n, ms=round(ms, 4), GBps=round(n / ms / 1e6, 1), frac_of_peak=round(n / ms / 1e6 / HBM_PEAK_GBS, 4))


def model_file(preset, wtype, seed):
    base = "/dev/shm" if os.access("/dev/shm", os.W_OK) else "/tmp"
    path = os.path.join(base, f"llava_measure_{preset}_{'q4_0' if wtype == lva.LV_Q4_0 else 'q8_0'}_seed{seed}.ggml")
    if (preset, wtype, seed) == ("7b", lva.LV_Q4_0, 0):
        path = os.path.join(base, "llava_bench_7b_q4_0_seed0.ggml")      # the file bench.py and the full-size tests use
    if not os.path.exists(path):
        lva.write_model(path + ".tmp", wtype=wtype, seed=seed, **SHAPES[preset])
        os.replace(path + ".tmp", path)
    return path


def step_bytes(shape, wtype, pos):
    D, F, V, L = shape["dim"], shape["ff"], shape["vocab"], shape["layers"]
    per_layer = (4 * D * D + 3 * D * F) // 32 * block_bytes(wtype)
    return L * per_layer + V * D // 32 * block_bytes(wtype) + (2 * L + 1) * D * 4 + L * 2 * D * 2 * (pos + 2) + V * 4 + D * 4


def decode_case(ctx, name, preset, wtype, seed, backlog, first, steps, force_path=None, report=emit, expect_picks=None):
    shape = SHAPES[preset]
    path = model_file(preset, wtype, seed)
    model = lva.Model(ctx, path)
    s = lva.Session(model, backlog)
    if force_path is not None:
        s.set_path(force_path)
    kind = {lva.PATH_KERNELS: "kernels", lva.PATH_GRAPH: "graph", lva.PATH_PERSISTENT: "persistent"}[s.path()]
    prompt = lva.synth_tokens(first, 3, shape["vocab"], seed=seed)
    t0 = time.perf_counter()
    s.begin(prompt, 0)
    tok = s.argmax()
    prefill_s = time.perf_counter() - t0
    pos = first
    picks = [tok]                      # picks[k] is the token fed at position first + k
    for _ in range(4):
        s.begin([tok], pos)
        tok = s.argmax()
        picks.append(tok)
        pos += 1
    t0 = time.perf_counter()
    total = 0
    for _ in range(steps):
        s.begin([tok], pos)
        tok = s.argmax()
        picks.append(tok)
        total += step_bytes(shape, wtype, pos)
        pos += 1
    dt = time.perf_counter() - t0
    if expect_picks is not None:       # another path's run of the same case: the greedy continuation has to be the same
        n = min(len(expect_picks), len(picks))
        diff = [k for k in range(n) if picks[k] != expect_picks[k]]
        if diff:
            raise RuntimeError(f"{name}: greedy token at position {first + diff[0]} differs from the other path's ({picks[diff[0]]} vs {expect_picks[diff[0]]})")
    r = report(case=name, model=preset, wtype="q4_0" if wtype == lva.LV_Q4_0 else "q8_0", path=kind, positions=[first + 4, pos - 1], steps=steps,
               tok_s=round(steps / dt, 1), ms_per_token=round(dt / steps * 1e3, 4), GBps=round(total / dt / 1e9, 1),
               frac_of_peak=round(total / dt / 1e9 / HBM_PEAK_GBS, 4), prompt_tokens=first, prompt_s=round(prefill_s, 3),
               same_picks_as_other_path=None if expect_picks is None else True)
    s.close()
    model.close()
    r = dict(r)
    r["picks"] = picks
    return r


MFMA_PEAK_TFLOPS = 2500.0


def prefill_case(ctx, case, name, wtype, report=emit):
    shape = SHAPES[name]
    path = model_file(name, wtype, 3)
    model = lva.Model(ctx, path)
    s = lva.Session(model, 512)
    prompt = lva.synth_tokens(512, 3, shape["vocab"], seed=3)
    s.begin(prompt, 0)          # untimed: allocates the prompt workspace and makes the model's prompt copy
    s.wait()
    s.timer_start()
    s.begin(prompt, 0)          # the same rows again
    ms = s.timer_stop()
    D, F, V, L = shape["dim"], shape["ff"], shape["vocab"], shape["layers"]
    flops = 2.0 * 512 * L * (4 * D * D + 3 * D * F) + 2.0 * V * D      # the output matrix sees the last row only
    # frac_of_mfma_peak counts the flops the prompt needs (2 per weight and token); the GEMM executes every product twice
    # (activations are a pair of fp16 halves), so the matrix cores run at twice that rate: executed_frac
    r = report(case=case, model=name, wtype="q4_0" if wtype == lva.LV_Q4_0 else "q8_0", tokens=512, ms=round(ms, 2),
               tok_s=round(512 / ms * 1e3, 1), TFLOPs=round(flops / ms / 1e9, 2), executed_TFLOPs=round(2 * flops / ms / 1e9, 2),
               frac_of_mfma_peak=round(flops / ms / 1e9 / MFMA_PEAK_TFLOPS, 4), executed_frac=round(2 * flops / ms / 1e9 / MFMA_PEAK_TFLOPS, 4))
    s.close()
    model.close()
    return r


def gemm_cases(ctx, report=emit):
    """reference: the *_batch shaders on 512 pending tokens (llava_session.cpp:243-255).  One lv_kernel_gemm call = the split of
    the activations into fp16 halves + gemm_kernel (+ the sum of the K slices where the grid would not fill the device), at
    the 13B layer shapes; the matrix's prompt copy and the workspace exist after the first call.  flops = 2 * tokens *
    rows * cols; every product is executed twice (two activation halves)."""
    n, wtype = 512, lva.LV_Q8_0
    out_cases = []
    for rows, cols in ((5120, 5120), (13824, 5120), (5120, 13824)):
        m = ctx.matrix(lva.synth_quant(wtype, rows, cols, seed=1), wtype, rows, cols)
        x = ctx.to_device(lva.synth_normal(n, cols, seed=2))
        out = ctx.zeros(n * rows * 4)
        for _ in range(3):
            lva.check(ctx.lib.lv_kernel_gemm(ctx.h, out, m, x, n, 0))
        ctx.sync()
        reps = 20
        ctx.timer_start()
        for _ in range(reps):
            lva.check(ctx.lib.lv_kernel_gemm(ctx.h, out, m, x, n, 0))
        us = ctx.timer_stop() * 1e3 / reps
        useful = 2.0 * n * rows * cols / us / 1e6
        out_cases.append(report(case="gemm", wtype="q8_0", rows=rows, cols=cols, tokens=n, launches=reps, us=round(us, 1),
                                useful_TFLOPs=round(useful, 1), executed_TFLOPs=round(2 * useful, 1),
                                frac_of_mfma_peak=round(useful / MFMA_PEAK_TFLOPS, 4), executed_frac=round(2 * useful / MFMA_PEAK_TFLOPS, 4)))
        ctx.matrix_free(m)
        ctx.free(x)
        ctx.free(out)
    return out_cases


def main():
    which = sys.argv[1] if len(sys.argv) > 1 else "all"
    ctx = lva.Context(0)
    name, cus, hbm = ctx.info()
    emit(case="device", name=name, compute_units=cus, hbm_GiB=hbm >> 30)
    if which in ("copy", "all"):
        copy_case(ctx)
    if which in ("read-stream", "all"):
        read_stream_case(ctx)
    if which in ("gemv", "all"):
        gemv_cases(ctx)
    if which == "gemv-13b":
        gemv_cases(ctx, shapes=GEMV_SHAPES_13B)
    if which in ("attention", "all"):
        attention_cases(ctx)
    if which == "attention-batch":
        attention_batch_cases(ctx)
    if which == "gemm":
        gemm_cases(ctx)
    if which in ("decode-q8", "all"):
        decode_case(ctx, "decode-q8", "7b", lva.LV_Q8_0, 1, 2048, 1916, 128)
    if which in ("decode-q8-graph", "all"):
        decode_case(ctx, "decode-q8-graph", "7b", lva.LV_Q8_0, 1, 2048, 1916, 128, force_path=lva.PATH_GRAPH)
    if which in ("decode-13b", "all"):
        decode_case(ctx, "decode-13b", "13b", lva.LV_Q4_0, 2, 512, 32, 256)
    if which in ("decode-13b-graph", "all"):
        decode_case(ctx, "decode-13b-graph", "13b", lva.LV_Q4_0, 2, 512, 32, 256, force_path=lva.PATH_GRAPH)
    if which in ("decode-7b-graph", "all"):
        decode_case(ctx, "decode-7b-graph", "7b", lva.LV_Q4_0, 0, 512, 440, 68, force_path=lva.PATH_GRAPH)
    if which in ("prefill-13b", "all"):
        prefill_case(ctx, "prefill-13b", "13b", lva.LV_Q8_0)
    if which in ("prefill-13b-q4", "all"):
        prefill_case(ctx, "prefill-13b-q4", "13b", lva.LV_Q4_0)
    if which in ("prefill-7b", "all"):
        prefill_case(ctx, "prefill-7b", "7b", lva.LV_Q4_0)
    ctx.close()       # nothing of the library is left to the interpreter's exit


if __name__ == "__main__":
    main()
