"""Small Ramalix configurations with random weights for the tests.  Sizes are chosen so that values a real model tends to make
equal differ here (query / value sizes, taps of the input convolutions and of the mixer's convolutions, the ranks of the two
low-rank projection pairs, block sizes that are no multiple of a page or a key tile), and so that the special cases are met:
a repeated span that starts after the first layer and ends before the last, a span walked once, no span at all, a layer without
feed-forward, a router without groups, without shared expert, with top 1, one tap (no history), attention without rotation,
without block mask, without query temperature, one key/value head and several, more query heads per key/value head than one
attention workgroup holds, residual factor and logit factor 1."""
import numpy as np
import torch

from oracle import ramalix_ref as R


def diff_attn(heads, kv, dim, vdim, diff, scale, qt=None, mlp=None):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "diff": diff, "scale": scale}
    if qt:
        m["q_temp"] = {"coef": qt[0], "every": qt[1]}
    return {"type": "attention", "mixer": m, "mlp": mlp}


def block_attn(heads, kv, dim, vdim, scale, size=None, rot=None, mlp=None):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale}
    if size:
        m["mask"] = {"size": size}
    if rot:
        m["rot"] = {"dims": rot[0], "base": rot[1]}
    return {"type": "attention_2", "mixer": m, "mlp": mlp}


def channel_delta(heads, kv, dim, vdim, conv, ranks=(5, 7), mlp=None):
    """ranks: sizes of the low-rank projection pairs; they are NOT part of the configuration a model ships (tensor shapes give
    them) and are popped before the configuration reaches an engine"""
    return {"type": "channel_delta", "mixer": {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "conv": conv},
            "mlp": mlp, "_ranks": ranks}


def moe(ff, experts, top, groups=None, shared=None):
    d = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if groups:
        d["router"]["groups"] = {"count": groups[0], "keep": groups[1]}
    if shared:
        d["shared"] = {"ff": shared}
    return d


def base(width, vocab, taps, layers, loop=None, mult=1.0, logit_scale=1.0, eps=1e-5):
    c = {"architecture": "Ramalix", "width": width, "vocab": vocab, "norm": {"eps": eps}, "canon": {"taps": taps},
         "residual_mult": mult, "logit_scale": logit_scale, "layers": layers}
    if loop:
        c["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return c


def config_a(times=3):
    """every mixer kind; the span 1 .. 3 walked three times; blocks of 24 positions (no multiple of a page of 16 or a key tile
    of 64); the query temperature changes every 7 positions"""
    return base(96, 131, 4, [
        block_attn(6, 2, 16, 24, 0.3, size=24, rot=(8, 1000.0), mlp=moe(24, 12, 2, groups=(3, 2), shared=40)),
        channel_delta(4, 2, 24, 20, 2, ranks=(6, 9), mlp=moe(16, 6, 3, groups=(2, 1), shared=24)),
        diff_attn(3, 1, 12, 28, 0.35, 0.4, qt=(0.7, 7), mlp=moe(32, 5, 2)),
        block_attn(2, 2, 40, 8, 0.11, size=80, rot=(40, 50.0)),
        channel_delta(3, 3, 8, 12, 5, ranks=(3, 4), mlp=moe(24, 8, 1, groups=(4, 4), shared=16)),
    ], loop=(1, 4, times), mult=0.6, logit_scale=0.3)


def config_b():
    """one tap everywhere (no history), top 1, one group, no shared expert, single heads, no rotation, no block mask, no query
    temperature, a span walked once, factors of 1"""
    return base(64, 77, 1, [
        block_attn(1, 1, 32, 16, 0.2, mlp=moe(16, 5, 1)),
        diff_attn(2, 2, 8, 8, 0.5, 0.3, mlp=moe(40, 4, 3, groups=(1, 1), shared=8)),
        channel_delta(1, 1, 12, 4, 1, ranks=(2, 2)),
    ], loop=(0, 2, 1), eps=1e-6)


def config_odd():
    """nothing is a multiple of 8; no repeated span at all"""
    return base(50, 61, 2, [
        diff_attn(3, 3, 10, 6, 0.25, 0.33, qt=(0.3, 5), mlp=moe(10, 6, 2, groups=(3, 1), shared=14)),
        channel_delta(5, 1, 6, 11, 3, ranks=(7, 3), mlp=moe(14, 9, 2, groups=(3, 3))),
        block_attn(3, 3, 10, 6, 0.3, size=9, rot=(4, 30.0)),
    ], mult=0.8, logit_scale=1.7)


def config_wide_heads():
    """more query heads per key/value head than an attention workgroup's 16 rows; memories wider than one column block
    (vdim > 64) and deeper than the smallest register layouts (dim > 64); attention values over more than 64 columns; two maps
    of 100 values; the whole model is the repeated span"""
    return base(128, 90, 3, [
        block_attn(20, 1, 8, 72, 0.3, size=50, rot=(6, 200.0), mlp=moe(32, 4, 2, shared=24)),
        channel_delta(2, 1, 80, 72, 4, ranks=(16, 8)),
        diff_attn(4, 2, 100, 136, 0.7, 0.08, qt=(0.5, 16), mlp=moe(16, 16, 4, groups=(4, 2))),
    ], loop=(0, 3, 2), mult=0.5, logit_scale=0.5)


def config_only_delta():
    """no attention anywhere: no cache part at all"""
    return base(40, 33, 3, [channel_delta(2, 1, 8, 12, 2 + i % 3, ranks=(4, 4), mlp=moe(16, 4, 2, shared=8) if i % 2 else None)
                            for i in range(3)], loop=(1, 3, 2), mult=0.7)


def config_tiny():
    return base(48, 50, 2, [channel_delta(2, 2, 8, 8, 2, ranks=(4, 4), mlp=moe(16, 4, 2, groups=(2, 1), shared=16)),
                            block_attn(2, 1, 8, 8, 0.35, size=70, rot=(8, 100.0), mlp=moe(16, 4, 2, shared=16)),
                            diff_attn(2, 1, 8, 8, 0.3, 0.35, qt=(0.5, 32))], loop=(0, 2, 2), mult=0.7, logit_scale=0.5)


def shipped(cfg):
    """the configuration as a model folder holds it: without the test-side rank entries"""
    out = dict(cfg)
    out["layers"] = [{k: v for k, v in l.items() if k != "_ranks"} for l in cfg["layers"]]
    return out


def bf16_round(a):
    return torch.as_tensor(np.asarray(a, dtype=np.float32)).bfloat16().float()


def random_weights(cfg, seed=0, soft=False):
    """{name: float32 tensor holding bf16 values}.  soft: the routed experts of a layer nearly alike and half the size, queries
    and keys half the size - see weights_for()"""
    g = torch.Generator().manual_seed(seed)
    D, V, K = cfg["width"], cfg["vocab"], cfg["canon"]["taps"]
    w = {}

    def lin(name, o, i, gain=1.0):
        w[name] = bf16_round(torch.randn(o, i, generator=g) * gain / i ** 0.5)

    def vec(name, n, mean=0.0, std=1.0):
        w[name] = bf16_round(mean + std * torch.randn(n, generator=g))

    def one(name, mean=1.0, std=0.2):
        w[name] = bf16_round(mean + std * torch.randn((), generator=g))

    def glu(p, ff, out_gain=2.0):
        lin(p + ".gate", ff, D, 2.0)
        lin(p + ".up", ff, D, 2.0)
        lin(p + ".down", D, ff, out_gain)

    qk_gain = 1.0 if soft else 2.0

    w["embed"] = bf16_round(torch.randn(V, D, generator=g))
    lp = cfg.get("loop")
    if lp and lp["stop"] > lp["start"]:
        w["loop.step"] = bf16_round(0.5 * torch.randn(lp["times"], D, generator=g))
    for i, l in enumerate(cfg["layers"]):
        p, m, q = "l%d" % i, l["mixer"], "l%d.mix" % i
        one(p + ".norm1")
        w[p + ".canon1"] = bf16_round(0.4 * torch.randn(D, K, generator=g))
        if l["type"] == "channel_delta":
            ra, rg = l["_ranks"]
            for n, rows in (("q", m["kv_heads"] * m["dim"]), ("k", m["kv_heads"] * m["dim"]), ("v", m["heads"] * m["vdim"])):
                lin("%s.%s" % (q, n), rows, D, 2.0)
                w["%s.%s.conv" % (q, n)] = bf16_round(0.5 * torch.randn(rows, m["conv"], generator=g))
            lin(q + ".b", m["heads"], D, 2.0)
            lin(q + ".a1", ra, D, 1.5)
            lin(q + ".a2", m["heads"] * m["dim"], ra, 1.5)
            vec(q + ".A_log", m["heads"], -0.5, 0.7)
            vec(q + ".dt_bias", m["heads"] * m["dim"], 0.0, 0.5)
            vec(q + ".norm", m["vdim"], 1.0, 0.2)
            lin(q + ".g1", rg, D, 2.0)
            lin(q + ".g2", m["heads"] * m["vdim"], rg, 2.0)
            lin(q + ".o", D, m["heads"] * m["vdim"], 2.0)
        else:
            maps = 2 if l["type"] == "attention" else 1
            lin(q + ".q", m["heads"] * maps * m["dim"], D, qk_gain)
            lin(q + ".k", m["kv_heads"] * maps * m["dim"], D, qk_gain)
            lin(q + ".v", m["kv_heads"] * m["vdim"], D, 2.0)
            lin(q + ".o", D, m["heads"] * m["vdim"], 2.0)
            if maps == 2:
                vec(q + ".q.b", m["heads"] * 2 * m["dim"], 0.0, 0.3)
                vec(q + ".k.b", m["kv_heads"] * 2 * m["dim"], 0.0, 0.3)
                vec(q + ".v.b", m["kv_heads"] * m["vdim"], 0.0, 0.3)
                vec(q + ".o.b", D, 0.0, 0.3)
                for n in ("lq1", "lk1", "lq2", "lk2"):
                    vec("%s.%s" % (q, n), m["dim"], 0.0, 0.4 / m["dim"] ** 0.25)
            else:
                vec(q + ".sink", m["heads"], 0.5, 1.0)
        f = l["mlp"]
        if not f:
            continue
        one(p + ".norm2")
        w[p + ".canon2"] = bf16_round(0.4 * torch.randn(D, K, generator=g))
        for e in range(f["router"]["experts"]):
            glu("%s.mlp.e%d" % (p, e), f["expert"]["ff"], 1.0 if soft else 2.0)
        if soft:      # every expert = the layer's first one + a sixth of its own draw: a flipped choice changes little
            for e in range(1, f["router"]["experts"]):
                for n in (".gate", ".up", ".down"):
                    own, first = "%s.mlp.e%d%s" % (p, e, n), "%s.mlp.e0%s" % (p, n)
                    w[own] = bf16_round(w[first] + w[own] / 6.0)
        lin(p + ".mlp.router", f["router"]["experts"], D, 4.0)
        if f.get("shared"):
            glu(p + ".mlp.shared", f["shared"]["ff"])
            lin(p + ".mlp.shared.sg", 1, D, 2.0)
    one("final.norm")
    w["head"] = bf16_round(torch.randn(V, D, generator=g) / D ** 0.5)
    return w


def config_for(name, dtype):
    """the named configuration; in bf16 the repeated span of config_a is walked twice instead of three times (see weights_for)"""
    if name == "a":
        return config_a(3 if dtype == "float32" else 2)
    return {"b": config_b, "odd": config_odd, "wide": config_wide_heads, "only_delta": config_only_delta, "tiny": config_tiny}[name]()


def weights_for(cfg, seed, dtype):
    """Small random models of this design are sensitive: every layer routes, a rounding that flips one near-tied expert choice
    moves that row, and through caches, states and the repeated span every later row.  Measured on the CPU: with nothing but
    the sublayers' inputs rounded to bf16 the plain restatement moves away from itself by 0.09 (median over the rows of
    config_a, 0.47 at the 90 % quantile), and one flip in a prompt's first tokens stays in the delta rule's state for good.
    With the routed experts of a layer nearly alike (so that a flipped choice changes little) and half the size, queries and
    keys half the size and two passes instead of three it moves by about 0.01 - something a bf16 engine can be held to.
    fp32 runs take the full sizes and unrelated experts."""
    return random_weights(cfg, seed, soft=dtype != "float32")


def engine_for(cfg, w, dtype, max_tokens=512, max_requests=4):
    from pegainfer_amd.ramalix import RamalixEngine
    eng = RamalixEngine(shipped(cfg), max_tokens=max_tokens, max_requests=max_requests, dtype=dtype)
    return eng.load_tensors({k: v.numpy() for k, v in w.items()})


def oracle_logits(cfg, w, tokens, hidden=False):
    out = R.forward(cfg, w, tokens, return_hidden=hidden)
    return (out[0].numpy(), out[1].numpy()) if hidden else out.numpy()


def row_err(got, ref):
    """per row: rms of the difference with its mean taken off, relative to the rms of the reference rows"""
    d = np.asarray(got, dtype=np.float64) - ref
    d = d - d.mean(-1, keepdims=True)
    return np.sqrt((d ** 2).mean(-1)) / np.sqrt(((ref - ref.mean(-1, keepdims=True)) ** 2).mean())


TOL = {"float32": 3e-5, "bfloat16": 8e-2}


def tokens_for(cfg, n, seed):
    return np.random.default_rng(seed).integers(0, cfg["vocab"], n).tolist()
