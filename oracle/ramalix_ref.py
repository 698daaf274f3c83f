"""Plain, slow restatement of the Ramalix decoder (TEST INFRASTRUCTURE ONLY; nothing in pegainfer_amd/ imports it).

One function per mechanism, one whole sequence at a time, float64 on the CPU, no cache, no state carried between calls:
every recurrence is a Python loop over the tokens from position 0.

Notation (n tokens, residual width D, m = residual_mult):
  snorm(x; g)     : x / sqrt(mean(x^2) + eps) * g, g ONE number for the whole row
  tconv(h; c)     : causal per-channel convolution over time, taps K: out_t = sum_j c[:, j] h_(t-K+1+j), zeros before 0
  sublayer        : r = snorm(x; g);  r <- r + tconv(r; canon);  x <- x + m * f(r)      f = mixer, then the feed-forward
  layer runs      : layers[start .. stop) are walked `times` times on the same weights (each pass with a cache / state of
                    its own); pass t first adds the embedding rows (t > 0) and the row loop.step[t] to x
  attention       : two softmax maps per head over the same values (query / key rows hold [map 1 | map 2] per head), biases
                    on q / k / v / o, no rotation, q times 1 + coef ln(floor((p + 1) / every) + 1);
                    o = a1 - lambda a2, lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff;  o / rms(o) * (1 - diff)
  attention_2     : one map, interleaved partial rotation, keys visible inside the query's own block of mask.size positions
                    only, a per-head sink logit in the softmax denominator
  channel_delta   : gated delta rule with one decay per (head, key channel), decay and output gate through two-step
                    (low-rank) projections
  feed-forward    : softmax router, experts restricted to the best groups (a group's score = its best expert), `top`
                    experts, weights renormalised; a shared expert scaled by a per-token sigmoid gate
"""
import json
import math
import os

import torch
import torch.nn.functional as Fn

F = torch.float64


def read_config(path):
    with open(path if path.endswith(".json") else os.path.join(path, "config.json")) as f:
        return json.load(f)


def snorm(x, g, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * g


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def tconv(h, c):
    """h [n, C], c [C, K]; the last column of c multiplies the current token"""
    n, C = h.shape
    K = c.shape[1]
    pad = torch.cat([torch.zeros(K - 1, C, dtype=F), h], 0)
    out = torch.zeros(n, C, dtype=F)
    for j in range(K):
        out += pad[j:j + n] * c[:, j][None, :]
    return out


def rope_pairs(x, pos, base, dims):
    """x [n, heads, d]: neighbours (2i, 2i+1) of the first `dims` values are rotated by pos * base^(-2i/dims)"""
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F)
    ang = pos.to(F)[:, None] * f[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    rot = torch.stack([u * c - v * s, v * c + u * s], -1).reshape(x.shape[0], x.shape[1], dims)
    return torch.cat([rot, x[..., dims:]], -1)


def query_temperature(n, coef, every):
    p = torch.arange(n)
    return 1.0 + coef * torch.log(torch.div(p + 1, every, rounding_mode="floor").to(F) + 1.0)


def diff_lambda(w, p, diff):
    a = torch.exp((w[p + ".lq1"].to(F) * w[p + ".lk1"].to(F)).sum())
    b = torch.exp((w[p + ".lq2"].to(F) * w[p + ".lk2"].to(F)).sum())
    return float(a - b + diff)


def differential_attention(h, w, p, m, eps):
    n = h.shape[0]
    H, G, d, dv, diff = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["diff"]
    q = (h @ w[p + ".q"].to(F).T + w[p + ".q.b"].to(F)).reshape(n, H, 2, d)
    k = (h @ w[p + ".k"].to(F).T + w[p + ".k.b"].to(F)).reshape(n, G, 2, d)
    v = (h @ w[p + ".v"].to(F).T + w[p + ".v.b"].to(F)).reshape(n, G, dv)
    qt = m.get("q_temp")
    if qt:
        q = q * query_temperature(n, qt["coef"], qt["every"])[:, None, None, None]
    lam = diff_lambda(w, p, diff)
    mask = torch.tril(torch.ones(n, n, dtype=torch.bool))
    out = torch.zeros(n, H, dv, dtype=F)
    for hh in range(H):
        g = hh // (H // G)
        maps = []
        for c in range(2):
            sc = (q[:, hh, c] @ k[:, g, c].T) * m["scale"]
            maps.append(torch.softmax(sc.masked_fill(~mask, -math.inf), -1) @ v[:, g])
        out[:, hh] = rms(maps[0] - lam * maps[1], eps) * (1.0 - diff)
    return out.reshape(n, H * dv) @ w[p + ".o"].to(F).T + w[p + ".o.b"].to(F)


def block_mask(n, size):
    i = torch.arange(n)
    same = torch.div(i, size, rounding_mode="floor")[:, None] == torch.div(i, size, rounding_mode="floor")[None, :]
    return same & (i[None, :] <= i[:, None])


def sink_block_attention(h, w, p, m, eps):
    n = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[p + ".q"].to(F).T).reshape(n, H, d)
    k = (h @ w[p + ".k"].to(F).T).reshape(n, G, d)
    v = (h @ w[p + ".v"].to(F).T).reshape(n, G, dv)
    pos = torch.arange(n)
    rot = m.get("rot")
    if rot:
        q = rope_pairs(q, pos, rot["base"], rot["dims"])
        k = rope_pairs(k, pos, rot["base"], rot["dims"])
    mask = block_mask(n, m["mask"]["size"]) if m.get("mask") else torch.tril(torch.ones(n, n, dtype=torch.bool))
    sink = w[p + ".sink"].to(F)
    out = torch.zeros(n, H, dv, dtype=F)
    for hh in range(H):
        g = hh // (H // G)
        sc = ((q[:, hh] @ k[:, g].T) * m["scale"]).masked_fill(~mask, -math.inf)
        top = torch.maximum(sc.max(-1).values, sink[hh])
        e = torch.exp(sc - top[:, None])
        den = e.sum(-1) + torch.exp(sink[hh] - top)
        out[:, hh] = (e / den[:, None]) @ v[:, g]
    return out.reshape(n, H * dv) @ w[p + ".o"].to(F).T


def channel_delta(h, w, p, m, eps):
    n = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = Fn.silu(tconv(h @ w[p + ".q"].to(F).T, w[p + ".q.conv"].to(F))).reshape(n, G, d)
    k = Fn.silu(tconv(h @ w[p + ".k"].to(F).T, w[p + ".k.conv"].to(F))).reshape(n, G, d)
    v = Fn.silu(tconv(h @ w[p + ".v"].to(F).T, w[p + ".v.conv"].to(F))).reshape(n, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ w[p + ".b"].to(F).T)
    a = (h @ w[p + ".a1"].to(F).T) @ w[p + ".a2"].to(F).T + w[p + ".dt_bias"].to(F)
    rate = torch.exp(w[p + ".A_log"].to(F))                                   # one per head
    decay = torch.exp(-rate[None, :, None] * Fn.softplus(a).reshape(n, H, d))   # one per (head, key channel)
    out = torch.zeros(n, H, dv, dtype=F)
    for hh in range(H):
        g = hh // (H // G)
        S = torch.zeros(d, dv, dtype=F)
        for t in range(n):
            S = decay[t, hh][:, None] * S
            u = beta[t, hh] * (v[t, hh] - S.T @ k[t, g])
            S = S + torch.outer(k[t, g], u)
            out[t, hh] = S.T @ q[t, g]
    o = rms(out, eps) * w[p + ".norm"].to(F)
    gate = torch.sigmoid((h @ w[p + ".g1"].to(F).T) @ w[p + ".g2"].to(F).T)
    return (o.reshape(n, H * dv) * gate) @ w[p + ".o"].to(F).T


def swiglu(x, w, p):
    return (Fn.silu(x @ w[p + ".gate"].to(F).T) * (x @ w[p + ".up"].to(F).T)) @ w[p + ".down"].to(F).T


def router(x, w, p, r):
    """(experts [n, top], weights [n, top]): softmax over all experts; only experts of the `keep` groups with the largest
    best score are eligible; the `top` largest eligible scores, divided by their sum"""
    s = torch.softmax(x @ w[p + ".router"].to(F).T, -1)
    n, E = s.shape
    grp = r.get("groups") or {"count": 1, "keep": 1}
    per = E // grp["count"]
    best = s.reshape(n, grp["count"], per).max(-1).values
    kept = torch.topk(best, grp["keep"], dim=-1).indices
    ok = torch.zeros(n, grp["count"], dtype=torch.bool)
    ok.scatter_(1, kept, True)
    ok = ok[:, :, None].expand(n, grp["count"], per).reshape(n, E)
    val, idx = torch.topk(s.masked_fill(~ok, -1.0), r["top"], dim=-1)
    return idx, val / (val.sum(-1, keepdim=True) + 1e-20)


def routed_ff(x, w, p, mlp):
    idx, val = router(x, w, p, mlp["router"])
    out = torch.zeros_like(x)
    for t in range(x.shape[0]):
        for c in range(idx.shape[1]):
            out[t] += val[t, c] * swiglu(x[t:t + 1], w, "%s.e%d" % (p, int(idx[t, c])))[0]
    if mlp.get("shared"):
        out = out + swiglu(x, w, p + ".shared") * torch.sigmoid(x @ w[p + ".shared.sg"].to(F).T)
    return out


MIXERS = {"attention": differential_attention, "attention_2": sink_block_attention, "channel_delta": channel_delta}


def layer_runs(cfg):
    """[(layer index, pass number or None)]: pass t is given at the first layer of the t-th walk over the repeated span"""
    n = len(cfg["layers"])
    lp = cfg.get("loop") or {"start": 0, "stop": 0, "times": 1}
    runs = [(i, None) for i in range(lp["start"])]
    for t in range(lp["times"] if lp["stop"] > lp["start"] else 0):
        runs += [(i, t if i == lp["start"] else None) for i in range(lp["start"], lp["stop"])]
    return runs + [(i, None) for i in range(max(lp["stop"], lp["start"]), n)]


def forward(cfg, w, tokens, return_hidden=False):
    """logits [n, vocab] (and the stream after every layer run, [runs, n, D]) of one sequence"""
    eps, mult = cfg["norm"]["eps"], cfg["residual_mult"]
    x0 = w["embed"].to(F)[torch.as_tensor(tokens, dtype=torch.long)]
    x, hidden = x0, []
    for i, t in layer_runs(cfg):
        layer, p = cfg["layers"][i], "l%d" % i
        if t is not None:
            if t > 0:
                x = x + x0
            x = x + w["loop.step"].to(F)[t]
        r = snorm(x, w[p + ".norm1"].to(F), eps)
        r = r + tconv(r, w[p + ".canon1"].to(F))
        x = x + mult * MIXERS[layer["type"]](r, w, p + ".mix", layer["mixer"], eps)
        if layer.get("mlp"):
            r = snorm(x, w[p + ".norm2"].to(F), eps)
            r = r + tconv(r, w[p + ".canon2"].to(F))
            x = x + mult * routed_ff(r, w, p + ".mlp", layer["mlp"])
        hidden.append(x)
    logits = snorm(x, w["final.norm"].to(F), eps) @ w["head"].to(F).T * cfg["logit_scale"]
    return (logits, torch.stack(hidden)) if return_hidden else logits
