"""The plain restatement of the Kukulorn decoder (oracle/kukulorn_ref.py) against independent forms of its mechanisms, on the
CPU: the convolution against torch's, the rotation's invariants, the three regimes of the frequency scaling, the distance
buckets, the window with kept first tokens by explicit loops, the state-space recurrence against its quadratic (attention-like)
form, the order of the layer runs, causality of the whole model."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as Fn

import kukulorn_common as C
from oracle import kukulorn_ref as R

F = torch.float64


def test_time_convolution_matches_torch_conv1d():
    g = torch.Generator().manual_seed(0)
    for K in (1, 2, 5):
        u, c, b = torch.randn(13, 7, generator=g, dtype=F), torch.randn(7, K, generator=g, dtype=F), torch.randn(7, generator=g, dtype=F)
        ref = Fn.conv1d(Fn.pad(u.T[None], (K - 1, 0)), c[:, None, :], bias=b, groups=7)[0].T
        assert torch.allclose(R.tconv(u, c, b), ref, atol=1e-12)
        assert torch.allclose(R.tconv(u, c)[0], c[:, -1] * u[0], atol=1e-12)       # the first token sees zeros before it


def test_rotation_keeps_lengths_and_depends_on_distance_only():
    rot = {"dims": 6, "base": 40.0}
    g = torch.Generator().manual_seed(1)
    q, k = torch.randn(1, 1, 10, generator=g, dtype=F), torch.randn(1, 1, 10, generator=g, dtype=F)
    qs, ks = R.rotate_halves(q.repeat(30, 1, 1), rot), R.rotate_halves(k.repeat(30, 1, 1), rot)
    assert torch.allclose(qs[0], q[0]) and torch.allclose(qs[:, :, 6:], q.repeat(30, 1, 1)[:, :, 6:])
    assert torch.allclose((qs * qs).sum(-1), (q * q).sum(-1).expand(30, 1))
    d5 = [(qs[p + 5, 0] * ks[p, 0]).sum() for p in range(25)]
    assert max(abs(float(v - d5[0])) for v in d5) < 1e-12
    # the pair is (i, i + dims / 2), not neighbours: turning value 0 by a quarter turn lands on value 3
    e = torch.zeros(2, 1, 10, dtype=F)
    e[:, 0, 0] = 1.0
    out = R.rotate_halves(e, {"dims": 6, "base": 1.0})          # base 1: every frequency is 1
    assert abs(float(out[1, 0, 0]) - math.cos(1.0)) < 1e-12 and abs(float(out[1, 0, 3]) - math.sin(1.0)) < 1e-12


def test_frequency_scaling_has_three_regimes_and_no_jumps():
    rot = {"dims": 12, "base": 1000.0, "scaling": {"factor": 3.0, "low": 1.0, "high": 4.0, "original": 64}}
    plain = R.rotation_frequencies({"dims": 12, "base": 1000.0})
    f = R.rotation_frequencies(rot)
    assert [round(2 * math.pi / v) for v in plain] == [6, 20, 63, 199, 628, 1987]
    assert f[0] == plain[0]                                                  # wave 6 < 64 / 4
    assert all(abs(f[i] - plain[i] / 3.0) < 1e-15 for i in (3, 4, 5))        # waves beyond 64 / 1
    assert plain[1] / 3.0 < f[1] < plain[1] and plain[2] / 3.0 < f[2] < plain[2]
    # at the band's edges the blend meets its neighbours
    for wave, want in ((16.0, 1.0), (64.0, 1.0 / 3.0)):
        s = (64 / wave - 1.0) / (4.0 - 1.0)
        assert abs(((1 - s) / 3.0 + s) - want) < 1e-12


def test_distance_buckets():
    rows, far = 10, 50
    b = [R.distance_bucket(d, rows, far) for d in range(200)]
    assert b[:5] == [0, 1, 2, 3, 4] and b[5] == 5
    assert all(x <= y for x, y in zip(b, b[1:])) and b[far] == rows - 1 and b[-1] == rows - 1
    assert b[far - 1] <= rows - 1 and len(set(b)) == rows
    # the logarithmic part: bucket 5 + j starts where (d / 5) reaches (50 / 5)^(j / 5)
    for j in range(1, 5):
        edge = 5 * 10 ** (j / 5)
        assert R.distance_bucket(math.ceil(edge), rows, far) >= 5 + j and R.distance_bucket(math.floor(edge - 1e-9), rows, far) <= 5 + j - (edge != int(edge))


def test_window_with_kept_first_tokens_by_loops():
    n, size, keep = 30, 7, 3
    vis = R.window_with_kept_first(n, size, keep)
    for i in range(n):
        for j in range(n):
            assert bool(vis[i, j]) == (j <= i and (i - j < size or j < keep))
    assert bool(vis[20, 14]) and not bool(vis[20, 13]) and bool(vis[20, 2]) and not bool(vis[20, 3])


def test_state_space_recurrence_equals_its_quadratic_form():
    cfg = C.config_a()
    w = {k: v.to(F) for k, v in C.random_weights(cfg, 3).items()}
    m, p = cfg["layers"][0]["mixer"]["right"], "l0.mix.right"
    n = 19
    h = torch.randn(n, cfg["width"], generator=torch.Generator().manual_seed(2), dtype=F)
    ref = R.state_space(h, w, p, m, 1e-6)
    Hh, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = Hh * P
    a = h @ w[p + ".in"].T
    z, xbc, dt = a[:, :inner], a[:, inner:2 * inner + 2 * G * N], a[:, 2 * inner + 2 * G * N:]
    xbc = Fn.silu(Fn.conv1d(Fn.pad(xbc.T[None], (m["conv"] - 1, 0)), w[p + ".conv"][:, None, :], bias=w[p + ".conv.b"], groups=xbc.shape[1])[0].T)
    x, B, Cm = xbc[:, :inner].view(n, Hh, P), xbc[:, inner:inner + G * N].view(n, G, N), xbc[:, inner + G * N:].view(n, G, N)
    dt = Fn.softplus(dt + w[p + ".dt_bias"])
    la = -torch.exp(w[p + ".A_log"]) * dt                     # log decay per (token, head)
    cum = torch.cumsum(la, 0)
    y = torch.zeros(n, Hh, P, dtype=F)
    for hd in range(Hh):
        g = hd // (Hh // G)
        L = torch.tril(torch.exp(cum[:, None, hd] - cum[None, :, hd]))        # decay from s + 1 .. t
        att = (Cm[:, g] @ B[:, g].T) * L * dt[None, :, hd]
        y[:, hd] = att @ x[:, hd] + w[p + ".D"][hd] * x[:, hd]
    y = y.reshape(n, inner) * Fn.silu(z)
    ng = m["norm_groups"]
    y = R.rms(y.view(n, ng, inner // ng), 1e-6).reshape(n, inner) * w[p + ".norm"]
    assert torch.allclose(ref, y @ w[p + ".o"].T, atol=1e-9)


def test_layer_runs_and_pass_openings():
    cfg = C.config_a(3)
    runs = R.layer_runs(cfg)
    assert [i for i, _ in runs] == [0, 1, 2, 3, 1, 2, 3, 1, 2, 3, 4]
    assert [o for _, o in runs] == [False, True, False, False, True, False, False, True, False, False, False]
    assert R.layer_runs(C.config_odd()) == [(0, False), (1, False), (2, False)]
    assert R.layer_runs(C.config_b()) == [(0, True), (1, False), (2, False)]


@pytest.mark.parametrize("name", ["a", "odd", "b"])
def test_whole_model_is_causal_and_capped(name):
    cfg = C.CONFIGS[name]()
    w = C.random_weights(cfg, 5)
    toks = C.tokens_for(cfg, 40, 1)
    whole, hid = C.oracle_logits(cfg, w, toks, hidden=True)
    part = C.oracle_logits(cfg, w, toks[:23])
    assert np.abs(whole[:23] - part).max() < 1e-9
    assert hid.shape == (len(R.layer_runs(cfg)), 40, cfg["width"])
    if cfg.get("logit_softcap"):
        assert np.abs(whole).max() < cfg["logit_softcap"]
    other = list(toks)
    other[30] = (other[30] + 1) % cfg["vocab"]
    assert np.abs(C.oracle_logits(cfg, w, other)[:30] - whole[:30]).max() < 1e-9


def test_a_kept_first_token_and_the_window_edge_show_in_the_output():
    """one value row stands out: the output of a later token moves exactly when that token is inside the window or among the
    kept first ones"""
    cfg = C.config_a()
    w = {k: v.to(F) for k, v in C.random_weights(cfg, 6).items()}
    m, p = cfg["layers"][0]["mixer"]["left"], "l0.mix.left"          # window 21, 5 kept
    n = 60
    h = torch.randn(n, cfg["width"], generator=torch.Generator().manual_seed(3), dtype=F)
    base_out = R.windowed_attention(h, w, p, m, 1e-6)
    for marked, seen_by, unseen_by in ((4, 59, None), (5, 25, 26), (30, 50, 51)):
        h2 = h.clone()
        h2[marked] = h2[marked] * 3.0 + 1.0
        out = R.windowed_attention(h2, w, p, m, 1e-6)
        assert (out[seen_by] - base_out[seen_by]).abs().max() > 1e-6
        if unseen_by is not None:
            assert (out[unseen_by] - base_out[unseen_by]).abs().max() < 1e-12
