"""Small Kukulorn configurations with random weights for the tests.  Sizes are chosen so that values a real model tends to make
equal differ here (query / value sizes, taps of the attention's and the state-space layer's convolutions, state size and head
size, window sizes that are no multiple of a page or a key tile, bucket counts), and so that the special cases are met: a
repeated span that starts after the first layer and ends before the last, a span walked once, no span at all, layers without
feed-forward, one tap (no history), attention without rotation scaling, with every value rotated, without soft cap, a window
without kept tokens and one wider than any sequence, one key/value head and several, more query heads per key/value head than
one attention workgroup holds, one group and one norm group, no logit cap."""
import numpy as np
import torch

from oracle import kukulorn_ref as R


def attn(heads, kv, dim, vdim, scale, conv=3, rot=None, softcap=None, mlp=None):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale}
    if conv:
        m["conv"] = conv
    if rot:
        m["rot"] = {"dims": rot[0], "base": rot[1]}
        if len(rot) > 2:
            m["rot"]["scaling"] = dict(zip(("factor", "low", "high", "original"), rot[2]))
    if softcap:
        m["softcap"] = softcap
    return {"type": "attention", "mixer": m, "mlp": {"kind": "dense", "ff": mlp} if mlp else None}


def parallel(left, right, mlp=None, rel_rows=None):
    """left: (heads, kv, dim, vdim, scale, window or None, keep_first, bias_max or None); right: (heads, vdim, state, groups,
    norm_groups, conv).  rel_rows: rows of the bias table - NOT part of the configuration a model ships (the tensor's shape gives
    it); popped before the configuration reaches an engine"""
    lm = {"heads": left[0], "kv_heads": left[1], "dim": left[2], "vdim": left[3], "scale": left[4]}
    if left[5]:
        lm["mask"] = {"size": left[5], "keep_first": left[6]}
    if left[7]:
        lm["bias_max"] = left[7]
    rm = dict(zip(("heads", "vdim", "state", "groups", "norm_groups", "conv"), right))
    return {"type": "parallel", "mixer": {"left": lm, "right": rm}, "mlp": {"kind": "dense", "ff": mlp} if mlp else None,
            "_rel_rows": rel_rows}


def base(width, vocab, layers, loop=None, cap=None, eps=1e-6):
    c = {"architecture": "Kukulorn", "width": width, "vocab": vocab, "norm": {"eps": eps}, "layers": layers}
    if cap:
        c["logit_softcap"] = cap
    if loop:
        c["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return c


def config_a(times=3):
    """both mixer kinds; the span 1 .. 3 walked three times; a window of 21 positions with 5 kept tokens (no multiple of a page
    of 16 or a key tile of 64); frequency scaling that meets all three regimes (waves of 6, 20, 63, 199, 628, 1987 positions
    against 64 / 4 and 64 / 1); ten distance buckets up to distance 50"""
    return base(88, 131, [
        parallel((6, 2, 20, 12, 0.3, 21, 5, 50), (4, 12, 24, 2, 3, 3), mlp=40, rel_rows=10),
        attn(4, 2, 24, 16, 0.21, conv=4, rot=(12, 1000.0, (3.0, 1.0, 4.0, 64)), softcap=6.0, mlp=56),
        attn(3, 1, 16, 20, 0.3, conv=2, rot=(16, 50.0), softcap=30.0),
        parallel((2, 2, 28, 8, 0.17, 40, 0, 33), (6, 4, 10, 3, 2, 5), mlp=24, rel_rows=7),
        attn(2, 1, 12, 28, 0.4, conv=3, rot=(4, 300.0, (8.0, 0.5, 2.0, 40)), mlp=32),
    ], loop=(1, 4, times), cap=20.0)


def config_b():
    """one tap (no history), single heads, one group, one norm group, no kept tokens beside a window wider than any test
    sequence, no distance bias, every value rotated without scaling, no soft cap anywhere, a span walked once"""
    return base(64, 77, [
        attn(1, 1, 32, 16, 0.2, conv=1, rot=(32, 10000.0), mlp=48),
        parallel((1, 1, 24, 40, 0.2, 4096, 0, None), (1, 16, 12, 1, 1, 1)),
        attn(2, 2, 8, 8, 0.5, conv=0, mlp=16),
    ], loop=(0, 2, 1), eps=1e-5)


def config_odd():
    """nothing is a multiple of 8; no repeated span at all; a window of three positions"""
    return base(50, 61, [
        attn(3, 3, 10, 6, 0.25, conv=5, rot=(6, 30.0), softcap=3.0, mlp=14),
        parallel((3, 1, 6, 11, 0.33, 3, 2, 19), (5, 3, 7, 5, 5, 2), mlp=10, rel_rows=5),
        parallel((2, 2, 10, 6, 0.3, 9, 9, 11), (3, 9, 5, 1, 3, 4), rel_rows=9),
    ], cap=7.0)


def config_wide_heads():
    """more query heads per key/value head than an attention workgroup's 16 rows; state-space heads wider than one column block
    (vdim > 64) with more states than the smallest register layouts (state > 64); attention values over more than 64 columns;
    a window of 70 positions that keeps 17; the whole model is the repeated span"""
    return base(128, 90, [
        attn(20, 1, 8, 72, 0.3, conv=3, rot=(6, 200.0), softcap=10.0, mlp=32),
        parallel((4, 2, 100, 136, 0.08, 70, 17, 200), (2, 72, 80, 1, 2, 4), mlp=24, rel_rows=32),
    ], loop=(0, 2, 2), cap=30.0)


def config_only_attention():
    return base(40, 33, [attn(2, 1, 8, 12, 0.35, conv=2 + i % 3, rot=(8, 100.0), softcap=5.0, mlp=16 if i % 2 else None)
                         for i in range(3)], loop=(1, 3, 2))


def config_only_parallel():
    return base(48, 35, [parallel((2, 1, 8, 12, 0.35, 10 + 7 * i, i, 64), (2, 8, 16, 2, 1, 2 + i), mlp=16 if i != 1 else None, rel_rows=8)
                         for i in range(3)], loop=(0, 1, 2), cap=15.0)


def config_tiny():
    return base(48, 50, [attn(2, 1, 8, 8, 0.35, conv=2, rot=(8, 100.0), softcap=9.0, mlp=16),
                         parallel((2, 1, 8, 8, 0.3, 70, 3, 100), (2, 8, 16, 1, 2, 3), mlp=16, rel_rows=12)], loop=(0, 2, 2), cap=12.0)


def shipped(cfg):
    """the configuration as a model folder holds it: without the test-side entries"""
    out = dict(cfg)
    out["layers"] = [{k: v for k, v in l.items() if not k.startswith("_")} for l in cfg["layers"]]
    return out


def bf16_round(a):
    return torch.as_tensor(np.asarray(a, dtype=np.float32)).bfloat16().float()


def random_weights(cfg, seed=0):
    """{name: float32 tensor holding bf16 values}"""
    g = torch.Generator().manual_seed(seed)
    D, V = cfg["width"], cfg["vocab"]
    w = {}

    def lin(name, o, i, gain=1.0):
        w[name] = bf16_round(torch.randn(o, i, generator=g) * gain / i ** 0.5)

    def vec(name, n, mean=0.0, std=1.0):
        w[name] = bf16_round(mean + std * torch.randn(n, generator=g))

    def qkv(q, m, bias_std=0.3):
        lin(q + ".q", m["heads"] * m["dim"], D, 2.0)
        lin(q + ".k", m["kv_heads"] * m["dim"], D, 2.0)
        lin(q + ".v", m["kv_heads"] * m["vdim"], D, 2.0)
        vec(q + ".q.b", m["heads"] * m["dim"], 0.0, bias_std)
        vec(q + ".k.b", m["kv_heads"] * m["dim"], 0.0, bias_std)
        vec(q + ".v.b", m["kv_heads"] * m["vdim"], 0.0, bias_std)
        lin(q + ".o", D, m["heads"] * m["vdim"], 2.0)

    w["embed"] = bf16_round(torch.randn(V, D, generator=g))
    lp = cfg.get("loop")
    if lp and lp["stop"] > lp["start"]:
        w["loop.in"] = bf16_round(torch.cat([torch.eye(D) * 0.8, torch.eye(D) * 0.5], 1) + 0.6 * torch.randn(D, 2 * D, generator=g) / D ** 0.5)
    for i, l in enumerate(cfg["layers"]):
        p, q = "l%d" % i, "l%d.mix" % i
        vec(p + ".norm1", D, 1.0, 0.2)
        if l["type"] == "attention":
            m = l["mixer"]
            qkv(q, m)
            if m.get("conv"):
                for n, rows in (("q", m["heads"] * m["dim"]), ("k", m["kv_heads"] * m["dim"]), ("v", m["kv_heads"] * m["vdim"])):
                    w["%s.%s.conv" % (q, n)] = bf16_round(0.5 * torch.randn(rows, m["conv"], generator=g))
            lin(q + ".g", m["heads"] * m["vdim"], D, 2.0)
        else:
            lm, rm = l["mixer"]["left"], l["mixer"]["right"]
            qkv(q + ".left", lm)
            vec(q + ".left.o.b", D, 0.0, 0.3)
            vec(q + ".left.q.norm", lm["heads"] * lm["dim"], 1.0, 0.3)
            vec(q + ".left.k.norm", lm["kv_heads"] * lm["dim"], 1.0, 0.3)
            if lm.get("bias_max"):
                w[q + ".left.rel"] = bf16_round(1.5 * torch.randn(l["_rel_rows"], lm["heads"], generator=g))
            lin(q + ".left.g", lm["heads"], D, 2.0)
            inner, gn = rm["heads"] * rm["vdim"], rm["groups"] * rm["state"]
            lin(q + ".right.in", 2 * inner + 2 * gn + rm["heads"], D, 2.0)
            w[q + ".right.conv"] = bf16_round(0.5 * torch.randn(inner + 2 * gn, rm["conv"], generator=g))
            vec(q + ".right.conv.b", inner + 2 * gn, 0.0, 0.3)
            vec(q + ".right.dt_bias", rm["heads"], -0.5, 0.7)
            vec(q + ".right.A_log", rm["heads"], -0.5, 0.7)
            vec(q + ".right.D", rm["heads"], 1.0, 0.3)
            vec(q + ".right.norm", inner, 1.0, 0.2)
            lin(q + ".right.o", D, inner, 2.0)
            vec(q + ".left.out", D, 1.0, 0.3)
            vec(q + ".right.out", D, 1.0, 0.3)
        if l.get("mlp"):
            ff = l["mlp"]["ff"]
            lin(p + ".mlp.gate", ff, D, 2.0)
            lin(p + ".mlp.up", ff, D, 2.0)
            lin(p + ".mlp.down", D, ff, 2.0)
    vec("final.norm", D, 1.0, 0.2)
    return w


CONFIGS = {"a": config_a, "b": config_b, "odd": config_odd, "wide": config_wide_heads, "only_attention": config_only_attention,
           "only_parallel": config_only_parallel, "tiny": config_tiny}


def engine_for(cfg, w, dtype, max_tokens=512, max_requests=4):
    from pegainfer_amd.kukulorn import KukulornEngine
    eng = KukulornEngine(shipped(cfg), max_tokens=max_tokens, max_requests=max_requests, dtype=dtype)
    return eng.load_tensors({k: v.numpy() for k, v in w.items()})


def oracle_logits(cfg, w, tokens, hidden=False):
    out = R.forward(cfg, w, tokens, return_hidden=hidden)
    return (out[0].numpy(), out[1].numpy()) if hidden else out.numpy()


def row_err(got, ref):
    """per row: rms of the difference with its mean taken off, relative to the rms of the reference rows"""
    d = np.asarray(got, dtype=np.float64) - ref
    d = d - d.mean(-1, keepdims=True)
    return np.sqrt((d ** 2).mean(-1)) / np.sqrt(((ref - ref.mean(-1, keepdims=True)) ** 2).mean())


TOL = {"float32": 3e-5, "bfloat16": 6e-2}


def tokens_for(cfg, n, seed):
    return np.random.default_rng(seed).integers(0, cfg["vocab"], n).tolist()
