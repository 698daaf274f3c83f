"""CPU checks of the plain Ramalix restatement (oracle/ramalix_ref.py) against independent forms of the same equations, so that
the thing the GPU tests compare with is itself pinned: the two-map attention against explicit per-row sums, the block mask
against the visible sets written out, the sink against a softmax with one more column, the channel-decay delta rule against an
element-by-element loop, the router on a hand-made case, the expansion of the repeated span, causality and reach."""
import math

import numpy as np
import torch

import ramalix_common as C
from oracle import ramalix_ref as R

F = torch.float64


def test_time_convolution_matches_conv1d_and_last_column_is_the_current_token():
    g = torch.Generator().manual_seed(1)
    h, c = torch.randn(9, 5, generator=g, dtype=F), torch.randn(5, 4, generator=g, dtype=F)
    ref = torch.nn.functional.conv1d(torch.nn.functional.pad(h.T[None], (3, 0)), c[:, None, :], groups=5)[0].T
    assert torch.allclose(R.tconv(h, c), ref, atol=1e-12)
    only_now = torch.zeros(5, 4, dtype=F)
    only_now[:, -1] = 2.0
    assert torch.allclose(R.tconv(h, only_now), 2.0 * h)


def test_one_number_norm():
    x = torch.tensor([[3.0, -4.0, 0.0, 0.0]], dtype=F)
    assert torch.allclose(R.snorm(x, torch.tensor(2.0, dtype=F), 0.0), x / 2.5 * 2.0)
    assert float(R.snorm(torch.zeros(1, 4, dtype=F), torch.tensor(2.0, dtype=F), 1e-6).abs().max()) == 0.0


def test_layer_runs_expand_the_repeated_span():
    cfg = {"layers": [0] * 5, "loop": {"start": 1, "stop": 3, "times": 3}}
    assert R.layer_runs(cfg) == [(0, None), (1, 0), (2, None), (1, 1), (2, None), (1, 2), (2, None), (3, None), (4, None)]
    assert R.layer_runs({"layers": [0] * 2}) == [(0, None), (1, None)]
    assert R.layer_runs({"layers": [0] * 2, "loop": {"start": 0, "stop": 2, "times": 1}}) == [(0, 0), (1, None)]


def test_query_temperature_steps_with_the_block_number():
    t = R.query_temperature(20, 0.5, 7)
    assert float(t[5]) == 1.0                                     # positions 0 .. 5: floor((p + 1) / 7) = 0
    assert abs(float(t[6]) - (1 + 0.5 * math.log(2))) < 1e-12     # position 6 is the first of block number 1
    assert abs(float(t[19]) - (1 + 0.5 * math.log(3))) < 1e-12    # (19 + 1) // 7 = 2


def test_two_map_attention_against_explicit_sums():
    cfg = C.config_a()
    m = cfg["layers"][2]["mixer"]
    w = C.random_weights(cfg, 3)
    p = "l2.mix"
    n = 17
    h = torch.randn(n, cfg["width"], generator=torch.Generator().manual_seed(4), dtype=F)
    got = R.differential_attention(h, w, p, m, 1e-5)
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = h @ w[p + ".q"].to(F).T + w[p + ".q.b"].to(F)
    k = h @ w[p + ".k"].to(F).T + w[p + ".k.b"].to(F)
    v = h @ w[p + ".v"].to(F).T + w[p + ".v.b"].to(F)
    lam = math.exp(float(w[p + ".lq1"].to(F) @ w[p + ".lk1"].to(F))) - math.exp(float(w[p + ".lq2"].to(F) @ w[p + ".lk2"].to(F))) + m["diff"]
    assert abs(lam - R.diff_lambda(w, p, m["diff"])) < 1e-12
    rows = torch.zeros(n, H * dv, dtype=F)
    for i in range(n):
        temp = 1 + m["q_temp"]["coef"] * math.log((i + 1) // m["q_temp"]["every"] + 1)
        for hh in range(H):
            g = hh // (H // G)
            outs = []
            for c in range(2):       # row layout: head by head, [map 1 | map 2]
                qv = q[i, (2 * hh + c) * d:(2 * hh + c + 1) * d] * temp
                sc = torch.stack([qv @ k[j, (2 * g + c) * d:(2 * g + c + 1) * d] for j in range(i + 1)]) * m["scale"]
                pr = torch.exp(sc - sc.max())
                pr = pr / pr.sum()
                outs.append(sum(pr[j] * v[j, g * dv:(g + 1) * dv] for j in range(i + 1)))
            o = outs[0] - lam * outs[1]
            rows[i, hh * dv:(hh + 1) * dv] = o / torch.sqrt((o * o).mean() + 1e-5) * (1 - m["diff"])
    assert torch.allclose(got, rows @ w[p + ".o"].to(F).T + w[p + ".o.b"].to(F), atol=1e-9)


def test_block_mask_is_the_own_block_up_to_the_query():
    mk = R.block_mask(11, 4)
    for i in range(11):
        assert [j for j in range(11) if mk[i, j]] == list(range((i // 4) * 4, i + 1))


def test_sink_is_one_more_column_of_the_softmax_without_a_value():
    cfg = C.config_a()
    m = dict(cfg["layers"][0]["mixer"])
    w = C.random_weights(cfg, 5)
    p = "l0.mix"
    n = 30
    h = torch.randn(n, cfg["width"], generator=torch.Generator().manual_seed(6), dtype=F)
    got = R.sink_block_attention(h, w, p, m, 1e-5)
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(n)
    q = R.rope_pairs((h @ w[p + ".q"].to(F).T).reshape(n, H, d), pos, m["rot"]["base"], m["rot"]["dims"])
    k = R.rope_pairs((h @ w[p + ".k"].to(F).T).reshape(n, G, d), pos, m["rot"]["base"], m["rot"]["dims"])
    v = (h @ w[p + ".v"].to(F).T).reshape(n, G, dv)
    rows = torch.zeros(n, H, dv, dtype=F)
    for i in range(n):
        lo = (i // m["mask"]["size"]) * m["mask"]["size"]
        for hh in range(H):
            g = hh // (H // G)
            sc = torch.stack([q[i, hh] @ k[j, g] for j in range(lo, i + 1)]) * m["scale"]
            pr = torch.softmax(torch.cat([sc, w[p + ".sink"].to(F)[hh:hh + 1]]), 0)      # the sink: unscaled, last column
            rows[i, hh] = sum(pr[j - lo] * v[j, g] for j in range(lo, i + 1))
            assert float(pr[:-1].sum()) < 1.0
    assert torch.allclose(got, rows.reshape(n, H * dv) @ w[p + ".o"].to(F).T, atol=1e-9)


def test_pair_rotation_is_a_complex_multiplication_on_the_first_dims_only():
    g = torch.Generator().manual_seed(3)
    x = torch.randn(6, 2, 10, generator=g, dtype=F)
    pos = torch.arange(6)
    out = R.rope_pairs(x, pos, 100.0, 6)
    assert torch.equal(out[..., 6:], x[..., 6:])
    for i in range(3):
        z = torch.complex(x[..., 2 * i], x[..., 2 * i + 1]) * torch.exp(1j * pos.to(F) * 100.0 ** (-2.0 * i / 6))[:, None]
        assert torch.allclose(out[..., 2 * i], z.real) and torch.allclose(out[..., 2 * i + 1], z.imag)


def test_channel_delta_against_an_element_by_element_loop():
    cfg = C.config_a()
    m = cfg["layers"][1]["mixer"]
    w = C.random_weights(cfg, 7)
    p = "l1.mix"
    n = 9
    h = torch.randn(n, cfg["width"], generator=torch.Generator().manual_seed(8), dtype=F)
    got = R.channel_delta(h, w, p, m, 1e-5)
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    silu = torch.nn.functional.silu
    q = silu(R.tconv(h @ w[p + ".q"].to(F).T, w[p + ".q.conv"].to(F))).reshape(n, G, d)
    k = silu(R.tconv(h @ w[p + ".k"].to(F).T, w[p + ".k.conv"].to(F))).reshape(n, G, d)
    v = silu(R.tconv(h @ w[p + ".v"].to(F).T, w[p + ".v.conv"].to(F))).reshape(n, H, dv)
    a = ((h @ w[p + ".a1"].to(F).T) @ w[p + ".a2"].to(F).T + w[p + ".dt_bias"].to(F)).reshape(n, H, d)
    beta = 1 / (1 + torch.exp(-(h @ w[p + ".b"].to(F).T)))
    gate = 1 / (1 + torch.exp(-((h @ w[p + ".g1"].to(F).T) @ w[p + ".g2"].to(F).T))).reshape(n, H, dv)
    out = torch.zeros(n, H, dv, dtype=F)
    for hh in range(H):
        g = hh // (H // G)
        S = [[0.0] * dv for _ in range(d)]
        rate = math.exp(float(w[p + ".A_log"][hh]))
        for t in range(n):
            qn = q[t, g] / math.sqrt(float((q[t, g] ** 2).sum()) + 1e-6) / math.sqrt(d)
            kn = k[t, g] / math.sqrt(float((k[t, g] ** 2).sum()) + 1e-6)
            for i in range(d):       # the decay of key channel i scales ROW i of the state
                dec = math.exp(-rate * math.log1p(math.exp(float(a[t, hh, i]))))
                for j in range(dv):
                    S[i][j] *= dec
            for j in range(dv):      # one column at a time: read, correct, write, read out
                u = float(beta[t, hh]) * (float(v[t, hh, j]) - sum(S[i][j] * float(kn[i]) for i in range(d)))
                for i in range(d):
                    S[i][j] += float(kn[i]) * u
                out[t, hh, j] = sum(S[i][j] * float(qn[i]) for i in range(d))
    o = out / torch.sqrt((out * out).mean(-1, keepdim=True) + 1e-5) * w[p + ".norm"].to(F) * gate
    assert torch.allclose(got, o.reshape(n, H * dv) @ w[p + ".o"].to(F).T, atol=1e-9)


def test_router_keeps_the_best_groups_by_their_best_expert_and_renormalises():
    # six experts in three groups of two; logits chosen so that group 1 holds the second-best expert overall but is outranked
    # by groups 0 and 2 when a group counts by its best member only ... and wins when keep = 1 on its best member
    z = torch.tensor([[2.0, -3.0, 1.9, 1.8, 3.0, -5.0]], dtype=F)
    w = {"r.router": torch.eye(6)}
    idx, val = R.router(z, w, "r", {"experts": 6, "top": 2, "groups": {"count": 3, "keep": 2}})
    assert sorted(idx[0].tolist()) == [0, 4]                       # groups 2 and 0 stay; expert 2 (group 1) is out
    s = torch.softmax(z[0], 0)
    assert torch.allclose(val[0].sum(), torch.tensor(1.0, dtype=F)) and torch.allclose(val[0], s[idx[0]] / s[idx[0]].sum())
    idx, _ = R.router(z, w, "r", {"experts": 6, "top": 2, "groups": {"count": 3, "keep": 1}})
    assert sorted(idx[0].tolist()) == [4, 5]                       # only group 2: its weak second member is taken before any outsider
    idx, _ = R.router(z, w, "r", {"experts": 6, "top": 3})
    assert sorted(idx[0].tolist()) == [0, 2, 4]                    # no groups: plain top 3


def test_shared_expert_is_scaled_by_a_sigmoid_gate_per_token():
    cfg = C.config_tiny()
    w = C.random_weights(cfg, 9)
    x = torch.randn(3, cfg["width"], generator=torch.Generator().manual_seed(1), dtype=F)
    mlp = cfg["layers"][0]["mlp"]
    full = R.routed_ff(x, w, "l0.mlp", mlp)
    w2 = dict(w)
    w2["l0.mlp.shared.sg"] = torch.zeros_like(w["l0.mlp.shared.sg"])      # gate 1/2 for every token
    half = R.routed_ff(x, w2, "l0.mlp", mlp)
    no_shared = R.routed_ff(x, w, "l0.mlp", {k: v for k, v in mlp.items() if k != "shared"})
    sg = torch.sigmoid(x @ w["l0.mlp.shared.sg"].to(F).T)
    assert torch.allclose(full - no_shared, 2 * sg * (half - no_shared), atol=1e-12)


def test_the_model_is_causal_and_every_layer_kind_sees_the_past():
    cfg = C.config_a()
    w = C.random_weights(cfg, 6)
    toks = C.tokens_for(cfg, 14, 1)
    base = C.oracle_logits(cfg, w, toks)
    other = list(toks)
    other[9] = (other[9] + 1) % cfg["vocab"]
    moved = C.oracle_logits(cfg, w, other)
    assert np.abs(moved[:9] - base[:9]).max() == 0.0
    assert all(np.abs(moved[t] - base[t]).max() > 1e-6 for t in range(9, 14))


def test_block_attention_alone_does_not_look_past_its_block():
    """a model of block-masked attention only, one tap (no convolution history): a token changed in block 0 moves nothing from
    block 1 on, a token changed in block 1 moves the rest of block 1 only"""
    cfg = C.base(32, 40, 1, [C.block_attn(2, 1, 8, 8, 0.35, size=5, rot=(4, 10.0))], mult=0.9)
    w = C.random_weights(cfg, 2)
    toks = C.tokens_for(cfg, 15, 3)
    base = C.oracle_logits(cfg, w, toks)
    other = list(toks)
    other[6] = (other[6] + 1) % cfg["vocab"]
    moved = C.oracle_logits(cfg, w, other)
    changed = [t for t in range(15) if np.abs(moved[t] - base[t]).max() > 0]
    assert changed == [6, 7, 8, 9]
