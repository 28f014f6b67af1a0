"""Pins the CPU checker (oracle/) before anything trusts it.

The reference ships no tests, fixtures or golden vectors for this path, so every checker function is checked here
against something that does not share its code: numpy's float16, exhaustive closed-form products, fp64 brute force
with numpy, scipy's softmax, textbook RoPE applied to both operands, numpy's population standard deviation, and an
independent fp64 forward pass of a tiny model written with the textbook formulation.  Each test is chosen so that a
plausible slip (dropped term, wrong nibble order, swapped gate/up matrix, transposed operand, RMS instead of the
centred variance, rotation by the wrong sign) fails it.
"""
import numpy as np
import pytest
import scipy.special

Q4, Q8 = 2, 8


# ---------------------------------------------------------------------------------------------------------------
# helpers that build GGML blocks by hand (independent of the model writer)
# ---------------------------------------------------------------------------------------------------------------
def q4_blocks(scales_f16_bits, codes):
    """scales: uint16 [n]; codes: uint8 [n][32] values 0..15 in ELEMENT order -> GGML v3 blocks (18 B)"""
    n = len(scales_f16_bits)
    out = np.zeros((n, 18), dtype=np.uint8)
    out[:, 0:2] = np.asarray(scales_f16_bits, dtype=np.uint16).view(np.uint8).reshape(n, 2)
    codes = np.asarray(codes, dtype=np.uint8)
    out[:, 2:] = codes[:, :16] | (codes[:, 16:] << 4)   # byte j: element j low nibble, element j+16 high nibble
    return out.reshape(-1)


def q8_blocks(scales_f16_bits, codes):
    n = len(scales_f16_bits)
    out = np.zeros((n, 34), dtype=np.uint8)
    out[:, 0:2] = np.asarray(scales_f16_bits, dtype=np.uint16).view(np.uint8).reshape(n, 2)
    out[:, 2:] = np.asarray(codes, dtype=np.int8).view(np.uint8)
    return out.reshape(-1)


def dequant_np(blocks, ftype, rows, cols):
    """fp64 weights from raw blocks with numpy only"""
    stride = 18 if ftype == Q4 else 34
    b = np.asarray(blocks, dtype=np.uint8).reshape(-1, stride)
    d = b[:, 0:2].copy().view(np.float16).astype(np.float64)
    if ftype == Q4:
        q = np.concatenate([(b[:, 2:] & 0xF).astype(np.int32), (b[:, 2:] >> 4).astype(np.int32)], axis=1) - 8
    else:
        q = b[:, 2:].copy().view(np.int8).astype(np.int32)
    return (q * d).reshape(rows, cols)


# ---------------------------------------------------------------------------------------------------------------
# fp16
# ---------------------------------------------------------------------------------------------------------------
def test_half_to_float_all_patterns(orc):
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = orc.half_to_float(bits)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_float_to_half_round_to_nearest_even(orc):
    rng = np.random.default_rng(1)
    halves = np.arange(65536, dtype=np.uint16).view(np.float16)
    finite = halves[np.isfinite(halves)].astype(np.float32)
    # every representable half, every midpoint between neighbours (ties), values a hair off the midpoints,
    # random floats over the whole exponent range, and the overflow / underflow edges
    s = np.sort(finite.astype(np.float64))
    mids = ((s[:-1] + s[1:]) / 2).astype(np.float32)
    near = np.concatenate([np.nextafter(mids, np.float32(np.inf)), np.nextafter(mids, np.float32(-np.inf))])
    rnd = (rng.standard_normal(60000) * np.exp(rng.uniform(-20, 12, 60000))).astype(np.float32)
    edges = np.array([0.0, -0.0, 65504, 65519.99, 65520, 65536, 1e10, -1e10, np.inf, -np.inf, 2.0**-24, 2.0**-25,
                      np.nextafter(np.float32(2.0**-25), np.float32(1)), 2.0**-26, 6.1e-5, 6.0e-5], dtype=np.float32)
    vals = np.concatenate([finite, mids, near, rnd, edges])
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    got = orc.float_to_half(vals)
    assert np.array_equal(got, want)
    assert np.isnan(np.array([orc.float_to_half([np.nan])[0]], dtype=np.uint16).view(np.float16)[0])


# ---------------------------------------------------------------------------------------------------------------
# dequantisation: exhaustive over (scale, code)
# ---------------------------------------------------------------------------------------------------------------
def test_q4_dequant_every_scale_every_code(orc):
    scales = np.arange(65536, dtype=np.uint16)
    codes = np.tile(np.concatenate([np.arange(16), np.arange(15, -1, -1)]).astype(np.uint8), (65536, 1))
    got = orc.dequant(q4_blocks(scales, codes), Q4, 65536 * 32).reshape(65536, 32)
    d = scales.view(np.float16).astype(np.float64)[:, None]
    with np.errstate(invalid="ignore"):
        want = ((codes.astype(np.float64) - 8.0) * d).astype(np.float32)   # exact product: 5-bit int x 11-bit significand
    ok = np.isfinite(want)
    assert np.array_equal(got[ok].view(np.uint32), want[ok].view(np.uint32))
    assert np.array_equal(np.isnan(got), np.isnan(want))


def test_q8_dequant_every_scale_every_code(orc):
    all_codes = np.arange(-128, 128, dtype=np.int8).reshape(8, 32)
    for lo in range(0, 65536, 8192):
        scales = np.repeat(np.arange(lo, lo + 8192, dtype=np.uint16), 8)
        codes = np.tile(all_codes, (8192, 1))
        got = orc.dequant(q8_blocks(scales, codes), Q8, len(scales) * 32).reshape(-1, 32)
        with np.errstate(invalid="ignore"):
            want = (codes.astype(np.float64) * scales.view(np.float16).astype(np.float64)[:, None]).astype(np.float32)
        ok = np.isfinite(want)
        assert np.array_equal(got[ok].view(np.uint32), want[ok].view(np.uint32))


def test_q4_element_order_and_v1_layout(orc):
    # v3: byte j carries element j (low nibble) and element j+16 (high nibble)
    blk = np.zeros(18, dtype=np.uint8)
    blk[0:2] = np.array([1.0], dtype=np.float16).view(np.uint8)
    blk[2] = 0x0F | (0x01 << 4)       # element 0 = 15-8 = 7, element 16 = 1-8 = -7
    blk[2 + 5] = 0x03                 # element 5 = -5, element 21 = -8
    got = orc.dequant(blk, Q4, 32)
    want = np.full(32, -8.0, dtype=np.float32)
    want[0], want[16], want[5] = 7.0, -7.0, -5.0
    assert np.array_equal(got, want)
    # v1: f32 scale, byte j carries elements 2j (low) and 2j+1 (high); 20-byte blocks
    blk1 = np.zeros(20, dtype=np.uint8)
    blk1[0:4] = np.array([0.5], dtype=np.float32).view(np.uint8)
    blk1[4] = 0x0F | (0x01 << 4)      # element 0 = 7*0.5, element 1 = -7*0.5
    got1 = orc.dequant(blk1, Q4, 32, file_version=1)
    want1 = np.full(32, -4.0, dtype=np.float32)
    want1[0], want1[1] = 3.5, -3.5
    assert np.array_equal(got1, want1)
    assert orc.lib().orc_tensor_bytes(Q4, 3, 64) == 36 and orc.lib().orc_tensor_bytes(Q4, 1, 64) == 40
    assert orc.lib().orc_tensor_bytes(Q8, 3, 64) == 68 and orc.lib().orc_tensor_bytes(Q8, 1, 64) == 72


# ---------------------------------------------------------------------------------------------------------------
# GEMV family
# ---------------------------------------------------------------------------------------------------------------
def _rand_matrix(rng, ftype, rows, cols):
    n = rows * cols // 32
    scales = np.abs(rng.standard_normal(n) * 0.02).astype(np.float16).view(np.uint16)
    if ftype == Q4:
        return q4_blocks(scales, rng.integers(0, 16, (n, 32)))
    return q8_blocks(scales, rng.integers(-127, 128, (n, 32)))


@pytest.mark.parametrize("ftype", [Q4, Q8])
@pytest.mark.parametrize("rows,cols,batch", [(7, 32, 1), (33, 4096, 1), (5, 11008, 2), (9, 5120, 1), (12, 96, 3)])
def test_gemv_against_fp64(orc, ftype, rows, cols, batch):
    rng = np.random.default_rng(rows * cols)
    blocks = _rand_matrix(rng, ftype, rows, cols)
    W = dequant_np(blocks, ftype, rows, cols)
    x = rng.standard_normal((batch, cols)).astype(np.float32)
    want = x.astype(np.float64) @ W.T
    got = orc.gemv(blocks, ftype, rows, cols, x)
    bound = 4e-7 * np.sqrt(cols) * (np.abs(x).astype(np.float64) @ np.abs(W).T) / np.sqrt(cols) + 1e-9
    assert np.all(np.abs(got - want) <= 8 * bound)
    # accumulate form adds to what is there
    prev = rng.standard_normal((batch, rows)).astype(np.float32)
    acc = orc.gemv(blocks, ftype, rows, cols, x, out=prev, accumulate=True)
    assert np.allclose(acc, prev + got, rtol=0, atol=1e-6 * np.max(np.abs(prev) + np.abs(got)))
    # the number of partial sums per row changes the order, not the value
    for workers in (1, 4, 32):
        alt = orc.gemv(blocks, ftype, rows, cols, x, workers=workers)
        assert np.all(np.abs(alt - want) <= 8 * bound)


@pytest.mark.parametrize("ftype", [Q4, Q8])
def test_gemv_special_cases(orc, ftype):
    rng = np.random.default_rng(5)
    rows, cols = 16, 256
    blocks = _rand_matrix(rng, ftype, rows, cols)
    W32 = orc.dequant(blocks, ftype, rows * cols).reshape(rows, cols)
    # one-hot x picks a column of the dequantised matrix exactly (a single product, a single rounding)
    for k in (0, 17, 31, 32, 255):
        x = np.zeros(cols, dtype=np.float32)
        x[k] = 1.0
        assert np.array_equal(orc.gemv(blocks, ftype, rows, cols, x)[0], W32[:, k])
    # x = 1 gives row sums
    ones = np.ones(cols, dtype=np.float32)
    assert np.allclose(orc.gemv(blocks, ftype, rows, cols, ones)[0], W32.astype(np.float64).sum(axis=1), rtol=0, atol=1e-5)
    # the zero matrix (q4_0: every code 8) contributes exactly nothing, also in the accumulate form
    n = rows * cols // 32
    zero = q4_blocks(np.full(n, 0x3C00, np.uint16), np.full((n, 32), 8)) if ftype == Q4 else q8_blocks(np.full(n, 0x3C00, np.uint16), np.zeros((n, 32)))
    x = rng.standard_normal(cols).astype(np.float32)
    assert not np.any(orc.gemv(zero, ftype, rows, cols, x))
    prev = rng.standard_normal((1, rows)).astype(np.float32)
    assert np.array_equal(orc.gemv(zero, ftype, rows, cols, x, out=prev, accumulate=True), prev)
    # refused shapes
    with pytest.raises(ValueError):
        orc.gemv(blocks, ftype, rows, 48, x[:48])
    with pytest.raises(ValueError):
        orc.gemv(blocks, 0, rows, cols, x)


@pytest.mark.parametrize("ftype", [Q4, Q8])
def test_gemv_silu_gate_and_up_roles(orc, ftype):
    rng = np.random.default_rng(6)
    rows, cols = 24, 512
    w3, w1 = _rand_matrix(rng, ftype, rows, cols), _rand_matrix(rng, ftype, rows, cols)
    x = rng.standard_normal((2, cols)).astype(np.float32)
    up = x.astype(np.float64) @ dequant_np(w3, ftype, rows, cols).T     # first matrix: multiplied in plainly
    gate = x.astype(np.float64) @ dequant_np(w1, ftype, rows, cols).T   # second matrix: goes through SiLU
    want = up * gate / (1.0 + np.exp(-gate))
    got = orc.gemv_silu(w3, w1, ftype, rows, cols, x)
    assert np.allclose(got, want, rtol=2e-4, atol=1e-6 * np.max(np.abs(want)))
    swapped = gate * up / (1.0 + np.exp(-up))
    assert not np.allclose(got, swapped, rtol=1e-3, atol=1e-4)            # the roles are not interchangeable


# ---------------------------------------------------------------------------------------------------------------
# normalisation: centred variance, no epsilon
# ---------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dim", [64, 4096, 5120])
def test_normalize_is_population_std_not_rms(orc, dim):
    rng = np.random.default_rng(dim)
    x = (rng.standard_normal((3, dim)) * 0.3 + 1.5).astype(np.float32)      # mean far from zero
    w = (rng.standard_normal(dim) * 0.02).astype(np.float32)
    got = orc.normalize(x, w)
    x64 = x.astype(np.float64)
    want = x64 * w / np.std(x64, axis=1, keepdims=True)                      # numpy's std is mean-centred (ddof=0)
    assert np.allclose(got, want, rtol=3e-6, atol=1e-9)
    rms = x64 * w / np.sqrt(np.mean(x64 * x64, axis=1, keepdims=True))
    assert np.max(np.abs(got - rms)) > 10 * np.max(np.abs(got - want)) + 1e-3   # textbook RMSNorm is a different function
    # the work-group size only reorders the sums
    assert np.allclose(orc.normalize(x, w, wgs=64), want, rtol=3e-6, atol=1e-9)


def test_normalize_constant_input_has_no_epsilon(orc):
    x = np.full((1, 256), 0.25, dtype=np.float32)
    w = np.ones(256, dtype=np.float32)
    with np.errstate(all="ignore"):
        out = orc.normalize(x, w)
    assert not np.any(np.isfinite(out))      # variance 0, rsqrt(0) = inf: the shader has no epsilon either


# ---------------------------------------------------------------------------------------------------------------
# cache append, attention pieces
# ---------------------------------------------------------------------------------------------------------------
def test_kv_append_rounding_and_indexing(orc):
    rng = np.random.default_rng(7)
    dim, backlog = 96, 16
    rows = (rng.standard_normal((3, dim)) * np.exp(rng.uniform(-12, 8, (3, dim)))).astype(np.float32)
    rows[0, :4] = np.array([0x3F801000, 0x3F803000, 0x3F801001, 0x33000000], dtype=np.uint32).view(np.float32)
    cache = np.full((backlog, dim), 0xBEEF, dtype=np.uint16)
    orc.kv_append(cache, rows, 5)
    with np.errstate(over="ignore"):
        assert np.array_equal(cache[5:8], rows.astype(np.float16).view(np.uint16))
    untouched = np.ones(backlog, bool)
    untouched[5:8] = False
    assert np.all(cache[untouched] == 0xBEEF)


def _rope(v, pos, rot):
    """textbook RoPE on the last axis: adjacent pairs (2i, 2i+1), theta_i = 10000^(-2i/rot)"""
    half = rot // 2
    theta = pos * 10000.0 ** (-np.arange(half) / half)
    c, s = np.cos(theta), np.sin(theta)
    out = np.empty_like(v, dtype=np.float64)
    out[..., 0::2] = v[..., 0::2] * c - v[..., 1::2] * s
    out[..., 1::2] = v[..., 0::2] * s + v[..., 1::2] * c
    return out


@pytest.mark.parametrize("heads,rot,backlog,pos,batch", [(4, 64, 32, 0, 1), (2, 128, 64, 40, 1), (8, 32, 32, 9, 3), (3, 128, 128, 127, 1)])
def test_mhsa_is_textbook_rope_with_unrotated_fp16_cache(orc, heads, rot, backlog, pos, batch):
    rng = np.random.default_rng(pos + rot)
    dim = heads * rot
    kc = np.zeros((backlog, dim), dtype=np.uint16)
    kc[:pos + batch] = rng.standard_normal((pos + batch, dim)).astype(np.float16).view(np.uint16)
    q = rng.standard_normal((batch, dim)).astype(np.float32)
    got = orc.mhsa(kc, q, pos, heads, rot)                      # [batch][backlog][heads]
    k64 = kc.view(np.float16).astype(np.float64).reshape(backlog, heads, rot)
    for z in range(batch):
        cur = pos + z
        qr = _rope(q[z].astype(np.float64).reshape(heads, rot), cur, rot)
        for p in range(cur + 1):
            want = np.sum(qr * _rope(k64[p], p, rot), axis=1)  # rotate BOTH by their absolute positions, then dot
            tol = 2e-3 if cur - p > 64 else 3e-4                # fp32 angle (cur-p)*theta loses bits at long range
            assert np.allclose(got[z, p], want, rtol=0, atol=tol * np.sqrt(rot)), (z, p)
        assert not np.any(got[z, cur + 1:])
    # same position: rotation is the identity, plain dot product of q with the fp16-rounded key
    z, cur = batch - 1, pos + batch - 1
    plain = np.sum(q[z].astype(np.float64).reshape(heads, rot) * k64[cur], axis=1)
    assert np.allclose(got[z, cur], plain, rtol=0, atol=1e-5 * rot)


def test_mhsa_rotation_sign(orc):
    # a key at an earlier position must be rotated forward relative to the query, not backward
    heads, rot, backlog = 1, 32, 8
    k = np.zeros((backlog, rot), dtype=np.float16)
    k[0, 0] = 1.0                                   # K = e_x of the first (fastest) pair, cached at position 0
    q = np.zeros((1, rot), dtype=np.float32)
    q[0, 1] = 1.0                                   # Q = e_y of the same pair, at position 1
    got = orc.mhsa(k.view(np.uint16), q, 1, heads, rot)[0, 0, 0]
    # R(1)q . R(0)k = (-sin 1, cos 1) . (1, 0) = -sin(1)
    assert abs(got - (-np.sin(1.0))) < 1e-6


@pytest.mark.parametrize("heads,rot,backlog,pos,batch", [(4, 64, 32, 5, 1), (2, 128, 128, 100, 2)])
def test_softmax_and_weighted_values(orc, heads, rot, backlog, pos, batch):
    rng = np.random.default_rng(3)
    scores = (rng.standard_normal((batch, backlog, heads)) * 4).astype(np.float32)
    got = orc.softmax(scores, pos, rot)
    for z in range(batch):
        n = pos + z + 1
        want = scipy.special.softmax(scores[z, :n].astype(np.float64) / np.sqrt(rot), axis=0)
        assert np.allclose(got[z, :n], want, rtol=2e-6, atol=1e-9)
        assert np.allclose(got[z].sum(axis=0), 1.0, atol=1e-6)
        assert not np.any(got[z, n:])                # masked slots are exactly zero
    dim = heads * rot
    vc = rng.standard_normal((backlog, dim)).astype(np.float16)
    out = orc.kqv(vc.view(np.uint16), got, heads, rot)
    want = np.einsum("zph,phr->zhr", got.astype(np.float64), vc.astype(np.float64).reshape(backlog, heads, rot)).reshape(batch, dim)
    assert np.allclose(out, want, rtol=0, atol=2e-6 * np.max(np.abs(want)) + 1e-7)
    # one-hot attention returns the fp16 row exactly
    onehot = np.zeros((1, backlog, heads), dtype=np.float32)
    onehot[0, 3, :] = 1.0
    assert np.array_equal(orc.kqv(vc.view(np.uint16), onehot, heads, rot)[0], vc[3].astype(np.float32))


def test_greedy_is_first_strict_maximum(orc):
    assert orc.greedy(np.array([1, 5, 5, 2], dtype=np.float32)) == 1
    assert orc.greedy(np.array([-3, -3, -3], dtype=np.float32)) == 0
    assert orc.greedy(np.array([0, -1, 7, 7.0000005], dtype=np.float32)) == 3


# ---------------------------------------------------------------------------------------------------------------
# whole step: an independent fp64 forward pass (textbook RoPE on q and k, standard softmax, SwiGLU, the
# reference's centred-variance normalisation) on a tiny seeded model
# ---------------------------------------------------------------------------------------------------------------
def _forward_np(orc_model, tokens, half_from_double=False):
    hp = orc_model.hp
    D, H, R, L, V = hp["dim"], hp["heads"], hp["rot"], hp["layers"], hp["vocab"]

    def mat(name):
        raw, t = orc_model.data(name)
        return dequant_np(raw, t["ftype"], t["rows"], t["cols"])

    def vec(name):
        raw, t = orc_model.data(name)
        return raw.view(np.float32).astype(np.float64)

    def norm(x, w):
        return x * w / np.std(x, axis=-1, keepdims=True)

    emb, _ = orc_model.data("tok_embeddings")
    x = emb.view(np.float32).reshape(V, D)[np.asarray(tokens)].astype(np.float64)
    n = len(tokens)
    kcache, vcache = [], []
    for l in range(L):
        p = f"layers.{l}."
        h = norm(x, vec(p + "attention_norm"))
        q, k, v = h @ mat(p + "attention.wq").T, h @ mat(p + "attention.wk").T, h @ mat(p + "attention.wv").T
        if half_from_double:     # one rounding, from the double value (what orc_forward_f64 does)
            k16, v16 = k.astype(np.float16).astype(np.float64), v.astype(np.float16).astype(np.float64)
        else:                    # the cache keeps fp16, rounded from an fp32 value as in the shader
            k16 = k.astype(np.float32).astype(np.float16).astype(np.float64)
            v16 = v.astype(np.float32).astype(np.float16).astype(np.float64)
        kcache.append(k16.astype(np.float16)); vcache.append(v16.astype(np.float16))
        o = np.zeros_like(x)
        for z in range(n):
            qz = _rope(q[z].reshape(H, R), z, R)
            kz = np.stack([_rope(k16[p_].reshape(H, R), p_, R) for p_ in range(z + 1)])   # [p][H][R]
            att = scipy.special.softmax(np.einsum("hr,phr->ph", qz, kz) / np.sqrt(R), axis=0)
            o[z] = np.einsum("ph,phr->hr", att, v16[:z + 1].reshape(z + 1, H, R)).reshape(D)
        x = x + o @ mat(p + "attention.wo").T
        m = norm(x, vec(p + "ffn_norm"))
        gate, up = m @ mat(p + "feed_forward.w1").T, m @ mat(p + "feed_forward.w3").T
        x = x + (up * gate / (1 + np.exp(-gate))) @ mat(p + "feed_forward.w2").T
    return norm(x, vec("norm")) @ mat("output").T, kcache, vcache


@pytest.mark.parametrize("name", ["tiny_q4", "tiny_q8"])
def test_whole_step_against_independent_forward_pass(lva, orc, tiny_models, name):
    om = orc.Model(tiny_models[name])
    toks = lva.synth_tokens(9, 3, om.hp["vocab"], seed=11)
    want, kc, vc = _forward_np(om, toks)
    s = orc.Session(om, 128)
    got = s.eval(toks, all_rows=True)
    scale = np.max(np.abs(want))
    assert np.max(np.abs(got - want)) <= 2e-4 * scale
    assert np.array_equal(np.argmax(got, axis=1), np.argmax(want, axis=1))
    # cache rows: un-rotated fp16 keys and values, position p in row p
    for layer in range(om.hp["layers"]):
        gk = s.kv(layer, 0, 9).view(np.float16).astype(np.float32)
        gv = s.kv(layer, 1, 9).view(np.float16).astype(np.float32)
        assert np.max(np.abs(gk - kc[layer].astype(np.float32))) <= np.max(np.abs(gk)) * 2.0 ** -9
        assert np.max(np.abs(gv - vc[layer].astype(np.float32))) <= np.max(np.abs(gv)) * 2.0 ** -9
    s.close()
    om.close()


@pytest.mark.parametrize("name", ["tiny_q4", "tiny_q8", "small_q4"])
def test_double_precision_yardstick_against_independent_forward_pass(lva, orc, tiny_models, name):
    """orc_forward_f64 is what the full-size tests measure both the GPU and the fp32 checker against: it has to be the
    formulas' own result.  Pinned by the numpy forward pass above (textbook RoPE on q and k separately, scipy softmax with
    max subtraction, numpy std), which shares no code with it; both are double and round cache rows to fp16 once, from the
    double value, so they agree to the rounding of double sums (a cache value within 1e-16 of an fp16 rounding boundary
    could flip an ulp: not seen with these seeds)."""
    om = orc.Model(tiny_models[name])
    toks = lva.synth_tokens(9, 3, om.hp["vocab"], seed=11)
    want, _, _ = _forward_np(om, toks, half_from_double=True)
    got = om.forward_f64(toks)
    scale = np.max(np.abs(want[-1]))
    assert np.max(np.abs(got - want[-1])) <= 1e-12 * scale
    # and the fp32 checker sits within fp32 rounding of it
    s = orc.Session(om, 128)
    f32 = s.eval(toks)
    assert np.max(np.abs(f32 - got)) <= 2e-4 * scale
    # continued from a cache: the last three tokens on top of the first six rows of the checker's cache give what the
    # checker's own continuation gives (to fp32 rounding), and exactly the whole-prompt result when the rows are its own
    kv = [(s.kv(l, 0, 6), s.kv(l, 1, 6)) for l in range(om.hp["layers"])]
    cont = om.forward_f64(toks[6:], kv=kv)
    assert np.max(np.abs(cont - f32)) <= 2e-4 * scale
    s.close()
    om.close()


def test_prompt_as_one_batch_equals_token_by_token(lva, orc, tiny_models):
    om = orc.Model(tiny_models["small_q4"])
    toks = lva.synth_tokens(7, 3, om.hp["vocab"], seed=12)
    a, b = orc.Session(om, 128), orc.Session(om, 128)
    batched = a.eval(toks, all_rows=True)
    for i, t in enumerate(toks):
        single = b.eval([t])
        assert np.array_equal(single, batched[i])      # same arithmetic row by row, bit for bit
    assert a.pos == b.pos == 7
    for layer in range(om.hp["layers"]):
        assert np.array_equal(a.kv(layer, 0, 7), b.kv(layer, 0, 7))
    # overflow and bad token ids are refused (llava_session.cpp:214-217)
    with pytest.raises(ValueError):
        a.eval(np.zeros(122, dtype=np.uint32))
    with pytest.raises(ValueError):
        a.eval([om.hp["vocab"]])
    # rewind forgets positions but keeps the rows; re-evaluating gives the same logits
    b.rewind(4)
    assert b.pos == 4
    again = b.eval(toks[4:], all_rows=True)
    assert np.array_equal(again, batched[4:])
    a.close(); b.close(); om.close()


@pytest.mark.parametrize("name", ["tiny_q4", "tiny_q8"])
def test_version_1_file_gives_the_logits_of_its_version_3_twin(lva, orc, tiny_models, tmp_path, name):
    """the same element values stored as version-1 blocks (fp32 scale, interleaved nibbles; ggml_file.cpp:95-122):
    the file is a different byte stream, the arithmetic on the decoded values is the same, bit for bit"""
    import ggjt_builder as gb
    p1 = str(tmp_path / "v1.ggml")
    gb.convert_to_v1(tiny_models[name], p1)
    toks = lva.synth_tokens(6, 3, 512, seed=4)
    outs = []
    for path, ver in ((tiny_models[name], 3), (p1, 1)):
        om = orc.Model(path)
        assert om.hp["file_version"] == ver
        s = orc.Session(om, 128)
        outs.append(s.eval(toks, all_rows=True).copy())
        s.close(); om.close()
    assert np.array_equal(outs[0].view(np.uint32), outs[1].view(np.uint32))
