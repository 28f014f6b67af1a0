"""The arithmetic of the stochastic pick (llama-vulkan_amd/host/llava_session.cpp sample_token; reference
llava_session.cpp:154-194) on small hand-made cases.  Logits are chosen as 0.8 * ln(k), so that exp(l / 0.8) is the integer
k and every probability below is a fraction written out by hand.  What the random generator draws among several kept
tokens is not checked (the reference seeds it with the time of day: parity unpinned); everything before and after it is.
Runs on the CPU: the function takes its logits as an argument."""
import importlib
import math

import pytest


@pytest.fixture(scope="module")
def hl():
    return importlib.import_module("llama-vulkan_amd.hostlib")


def lg(k):
    return 0.8 * math.log(k)


def test_softmax_at_temperature_and_the_cut(hl):
    # weights 8, 4, 2, 1, 1 -> total 16 -> p = 1/2, 1/4, 1/8, 1/16, 1/16
    logits = [lg(8), lg(4), lg(2), lg(1), lg(1)]
    # mu = 3: cut = 1/8, kept = {0, 1, 2} with mass 7/8
    tok, mu, ids, ps, total, pick = hl.sample_token(logits, [], 3.0, seed=1)
    assert ids == [0, 1, 2]
    assert ps == pytest.approx([0.5, 0.25, 0.125], rel=1e-6)
    assert total == pytest.approx(0.875, rel=1e-6)
    assert tok == ids[pick]
    # mu' = mu + 0.1 * (5 + log2(p_pick / 0.875))
    assert mu == pytest.approx(3.0 + 0.1 * (5 + math.log2(ps[pick] / 0.875)), abs=1e-6)
    # mu = 4: cut = 1/16 and the comparison is >=, so all five stay
    _, _, ids, ps, total, _ = hl.sample_token(logits, [], 4.0, seed=1)
    assert ids == [0, 1, 2, 3, 4] and total == pytest.approx(1.0, rel=1e-6)
    # mu = 1: cut = 1/2, only token 0; a single kept token is drawn whatever the generator does, and
    # mu' = 1 + 0.1 * (5 + log2(1)) = 1.5
    for seed in (1, 2, 3):
        tok, mu, ids, ps, total, pick = hl.sample_token(logits, [], 1.0, seed=seed)
        assert (tok, ids, pick) == (0, [0], 0)
        assert total == pytest.approx(0.5, rel=1e-6) and mu == pytest.approx(1.5, abs=1e-6)


def test_nothing_passes_the_cut(hl):
    # four equal tokens: p = 1/4 each; mu = 1 -> cut 1/2 -> nothing kept.  The reference indexes an empty vector there;
    # this build returns the likeliest token (the first of equals) and leaves mu alone
    tok, mu, ids, _, total, pick = hl.sample_token([0.0] * 4, [], 1.0, seed=5)
    assert (tok, ids, pick, total) == (0, [], -1, 0.0) and mu == 1.0


def test_penalty_touches_token_13_only(hl):
    # vocabulary of 14; tokens 0 and 13 matter, the rest weigh 1 each (12 of them)
    # token 13 seen twice in the history: l' = l / 1.1 - (0.1 * 2 + 0) for l > 0.  l = 1.1 * (lg(4) + 0.2) -> l' = lg(4)
    logits = [lg(4)] + [0.0] * 12 + [1.1 * (lg(4) + 0.2)]
    history = [13, 5, 13, 0, 0, 0]          # token 0 three times, token 5 once: neither is penalised
    _, _, ids, ps, total, _ = hl.sample_token(logits, history, 10.0, seed=1)
    # weights 4, 1 x 12, 4 -> total 20
    assert ids == list(range(14))
    assert ps[0] == pytest.approx(0.2, rel=1e-5) and ps[13] == pytest.approx(0.2, rel=1e-5) and ps[5] == pytest.approx(0.05, rel=1e-5)
    # a logit <= 0 is multiplied: l' = 1.1 * l - 0.1 * count.  l = (lg(0.5) + 0.1) / 1.1 with count 1 -> l' = lg(0.5)
    logits[13] = (lg(0.5) + 0.1) / 1.1
    _, _, ids, ps, total, _ = hl.sample_token(logits, [13], 10.0, seed=1)
    # weights 4, 1 x 12, 0.5 -> total 16.5
    assert ps[13] == pytest.approx(0.5 / 16.5, rel=1e-5) and ps[0] == pytest.approx(4 / 16.5, rel=1e-5)
    # without 13 in the history nothing changes: weight exp(l / 0.8) as it stands
    _, _, ids, ps, total, _ = hl.sample_token(logits, [1, 2, 3], 10.0, seed=1)
    w13 = math.exp(logits[13] / 0.8)
    assert ps[13] == pytest.approx(w13 / (16 + w13), rel=1e-5)
    # only the last 64 tokens of the history count: a 13 that is 65 tokens back is forgotten, one 64 back is not
    _, _, _, ps, _, _ = hl.sample_token(logits, [13] + [1] * 64, 10.0, seed=1)
    assert ps[13] == pytest.approx(w13 / (16 + w13), rel=1e-5)
    _, _, _, ps, _, _ = hl.sample_token(logits, [13] + [1] * 63, 10.0, seed=1)
    assert ps[13] == pytest.approx(0.5 / 16.5, rel=1e-5)


def test_mu_runs_over_several_picks(hl):
    # two tokens, p = 3/4 and 1/4, mu large enough to keep both: the mass kept is 1, so whichever is drawn,
    # mu' = mu + 0.1 * (5 + log2(p)): +0.5 - 0.0415 for token 0, +0.5 - 0.2 = +0.3 for token 1
    logits = [lg(3), lg(1)]
    mu = 10.0
    for seed in range(8):
        tok, mu2, ids, ps, total, pick = hl.sample_token(logits, [], mu, seed=seed)
        assert ids == [0, 1] and total == pytest.approx(1.0, rel=1e-6)
        step = 0.5 + 0.1 * math.log2(0.75) if tok == 0 else 0.3
        assert mu2 == pytest.approx(mu + step, abs=2e-6)
        mu = mu2
