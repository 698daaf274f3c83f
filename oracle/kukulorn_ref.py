"""Plain, slow restatement of the Kukulorn decoder (TEST INFRASTRUCTURE ONLY; nothing in pegainfer_amd/ imports it).

One function per mechanism, one whole sequence at a time, float64 on the CPU, no cache, no state carried between calls:
every recurrence is a Python loop over the tokens from position 0.

Notation (n tokens, residual width D, X0 = the embedding rows, p = a token's position counted from 0):
  rms(x)          : x / sqrt(mean(x^2) + eps), over the last axis
  layer           : h = rms(x) * norm1;  x <- x + mixer(h) + ff(h)          ONE norm, both sublayers read h; ff may be absent
  layer runs      : layers[start .. stop) are walked `times` times on the same weights, each pass with its own cache and
                    state; right before the first layer of every pass  x <- W_in [x ; X0]
  tconv(u; c)     : causal per-channel convolution over time, taps K: out_t = sum_j c[:, j] u_(t-K+1+j), zeros before 0
  attention       : q, k, v = W h + b, then tconv on each; the halves (i, i + dims/2) of the first rot.dims values of every q / k
                    head turned by p * f_i, f_i = base^(-2i/dims) rescaled by wavelength for long contexts; q and k heads
                    brought to unit root mean square; s = cap tanh((q . k) scale / cap); causal softmax; heads times
                    sigmoid(W_g h) value by value; W_o
  parallel, left  : q, k, v = W h + b; q and k normed as WHOLE rows (all heads at once) with a weight; s = (q . k) scale +
                    rel[bucket(i - j), head]; key j visible to i if j <= i and (i - j < size or j < keep_first); softmax; head
                    times sigmoid(W_g h)_head; W_o + b_o
  parallel, right : [z | x | B | C | dt] = W_in h; x | B | C through tconv with bias, then silu; dt = softplus(dt + dt_bias);
                    per head S <- exp(-exp(A_log) dt) S + dt B x^T, y = S^T C + D x; (y silu(z)) normed in norm_groups parts,
                    times a weight; W_o
  parallel        : (rms(left) * w_l + rms(right) * w_r) / 2
  feed-forward    : W_down (relu(W_gate h) * (W_up h))
  logits          : c tanh(E (rms(x) * final.norm) / c), E the embedding table
"""
import json
import math
import os

import torch

F = torch.float64


def read_config(path):
    with open(path if path.endswith(".json") else os.path.join(path, "config.json")) as f:
        return json.load(f)


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def tconv(u, c, bias=None):
    """u [n, C], c [C, K]; the last column of c multiplies the current token; bias [C] is added to the sum"""
    n, C = u.shape
    K = c.shape[1]
    out = torch.zeros(n, C, dtype=F)
    for t in range(n):
        for j in range(K):
            src = t - K + 1 + j
            if src >= 0:
                out[t] += c[:, j] * u[src]
    return out if bias is None else out + bias


def rotation_frequencies(rot):
    """f_i = base^(-2i/dims); with `scaling`: waves shorter than original/high stay, waves longer than original/low are slowed
    by `factor`, those between are blended linearly in original/wavelength"""
    dims, out = rot["dims"], []
    sc = rot.get("scaling")
    for i in range(dims // 2):
        f = rot["base"] ** (-2.0 * i / dims)
        if sc:
            wave = 2.0 * math.pi / f
            if wave > sc["original"] / sc["low"]:
                f = f / sc["factor"]
            elif wave >= sc["original"] / sc["high"]:
                s = (sc["original"] / wave - sc["low"]) / (sc["high"] - sc["low"])
                f = (1.0 - s) * f / sc["factor"] + s * f
        out.append(f)
    return out


def rotate_halves(x, rot):
    """x [n, heads, d]: value i and value i + dims/2 of every head form a pair that turns by p * f_i; values from dims on stay"""
    n = x.shape[0]
    dims = rot["dims"]
    half = dims // 2
    f = rotation_frequencies(rot)
    out = x.clone()
    for p in range(n):
        for i in range(half):
            a = p * f[i]
            c, s = math.cos(a), math.sin(a)
            u, v = x[p, :, i], x[p, :, i + half]
            out[p, :, i] = u * c - v * s
            out[p, :, i + half] = v * c + u * s
    return out


def softmax_over_visible(s, visible):
    """s [n, n] scores of one head, visible [n, n] bool; rows are queries"""
    s = s.masked_fill(~visible, float("-inf"))
    s = s - s.max(-1, keepdim=True).values
    e = torch.exp(s)
    return e / e.sum(-1, keepdim=True)


def causal(n):
    i = torch.arange(n)
    return i[None, :] <= i[:, None]


def window_with_kept_first(n, size, keep_first):
    i = torch.arange(n)
    d = i[:, None] - i[None, :]
    return (d >= 0) & ((d < size) | (i[None, :] < keep_first))


def distance_bucket(d, rows, far):
    """one bucket per distance below rows // 2, then logarithmic steps that reach the last bucket at distance `far`"""
    hb = rows // 2
    if d < hb:
        return d
    return min(rows - 1, hb + int(math.floor(math.log(d / hb) / math.log(far / hb) * (rows - hb))))


def conv_attention(h, w, p, m, eps):
    """the "attention" mixer; h [n, D] -> [n, D]"""
    n = h.shape[0]
    H, G, dim, vd = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = h @ w[p + ".q"].T + w[p + ".q.b"]
    k = h @ w[p + ".k"].T + w[p + ".k.b"]
    v = h @ w[p + ".v"].T + w[p + ".v.b"]
    if m.get("conv"):
        q, k, v = tconv(q, w[p + ".q.conv"]), tconv(k, w[p + ".k.conv"]), tconv(v, w[p + ".v.conv"])
    q, k, v = q.view(n, H, dim), k.view(n, G, dim), v.view(n, G, vd)
    if m.get("rot"):
        q, k = rotate_halves(q, m["rot"]), rotate_halves(k, m["rot"])
    q, k = rms(q, eps), rms(k, eps)
    gate = torch.sigmoid(h @ w[p + ".g"].T).view(n, H, vd)
    vis = causal(n)
    heads = []
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * m["scale"]
        if m.get("softcap"):
            s = m["softcap"] * torch.tanh(s / m["softcap"])
        heads.append(softmax_over_visible(s, vis) @ v[:, g] * gate[:, hd])
    return torch.cat(heads, -1) @ w[p + ".o"].T


def windowed_attention(h, w, p, m, eps):
    """the left half of "parallel"; h [n, D] -> [n, D]"""
    n = h.shape[0]
    H, G, dim, vd = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rms(h @ w[p + ".q"].T + w[p + ".q.b"], eps) * w[p + ".q.norm"]
    k = rms(h @ w[p + ".k"].T + w[p + ".k.b"], eps) * w[p + ".k.norm"]
    v = h @ w[p + ".v"].T + w[p + ".v.b"]
    q, k, v = q.view(n, H, dim), k.view(n, G, dim), v.view(n, G, vd)
    mk = m.get("mask")
    vis = window_with_kept_first(n, mk["size"], mk.get("keep_first", 0)) if mk else causal(n)
    gate = torch.sigmoid(h @ w[p + ".g"].T)
    bias = None
    if m.get("bias_max"):
        rel = w[p + ".rel"]
        bk = torch.tensor([[distance_bucket(i - j, rel.shape[0], m["bias_max"]) if j <= i else 0 for j in range(n)] for i in range(n)])
        bias = rel[bk]          # [n, n, H]
    heads = []
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * m["scale"]
        if bias is not None:
            s = s + bias[:, :, hd]
        heads.append(softmax_over_visible(s, vis) @ v[:, g] * gate[:, hd:hd + 1])
    return torch.cat(heads, -1) @ w[p + ".o"].T + w[p + ".o.b"]


def softplus(x):
    return torch.where(x > 30.0, x, torch.log1p(torch.exp(torch.clamp(x, max=30.0))))


def silu(x):
    return x * torch.sigmoid(x)


def state_space(h, w, p, m, eps):
    """the right half of "parallel"; h [n, D] -> [n, D]"""
    n = h.shape[0]
    Hh, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = Hh * P
    a = h @ w[p + ".in"].T
    z, xbc, dt = a[:, :inner], a[:, inner:2 * inner + 2 * G * N], a[:, 2 * inner + 2 * G * N:]
    xbc = silu(tconv(xbc, w[p + ".conv"], w[p + ".conv.b"]))
    x = xbc[:, :inner].view(n, Hh, P)
    B = xbc[:, inner:inner + G * N].view(n, G, N)
    C = xbc[:, inner + G * N:].view(n, G, N)
    dt = softplus(dt + w[p + ".dt_bias"])
    rate = torch.exp(w[p + ".A_log"])
    y = torch.zeros(n, Hh, P, dtype=F)
    for hd in range(Hh):
        g = hd // (Hh // G)
        S = torch.zeros(N, P, dtype=F)
        for t in range(n):
            S = math.exp(-float(rate[hd]) * float(dt[t, hd])) * S + dt[t, hd] * torch.outer(B[t, g], x[t, hd])
            y[t, hd] = S.T @ C[t, g] + w[p + ".D"][hd] * x[t, hd]
    y = y.reshape(n, inner) * silu(z)
    ng = m.get("norm_groups", 1)
    y = rms(y.view(n, ng, inner // ng), eps).reshape(n, inner) * w[p + ".norm"]
    return y @ w[p + ".o"].T


def parallel_mixer(h, w, p, m, eps):
    a = windowed_attention(h, w, p + ".left", m["left"], eps)
    b = state_space(h, w, p + ".right", m["right"], eps)
    return 0.5 * (rms(a, eps) * w[p + ".left.out"] + rms(b, eps) * w[p + ".right.out"])


def relu_glu(h, w, p):
    return (torch.relu(h @ w[p + ".gate"].T) * (h @ w[p + ".up"].T)) @ w[p + ".down"].T


def layer_runs(cfg):
    """[(layer index, opens a pass)] in the order the layers run"""
    L = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp or lp["stop"] <= lp["start"]:
        return [(i, False) for i in range(L)]
    out = [(i, False) for i in range(lp["start"])]
    for _ in range(lp["times"]):
        out += [(i, i == lp["start"]) for i in range(lp["start"], lp["stop"])]
    return out + [(i, False) for i in range(lp["stop"], L)]


def forward(cfg, w, tokens, return_hidden=False):
    """w: {name: tensor}; -> logits [n, vocab] (and the stream after every layer run [runs, n, D])"""
    w = {k: v.to(F) for k, v in w.items()}
    eps = cfg["norm"]["eps"]
    x0 = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    x = x0
    hidden = []
    for i, opens in layer_runs(cfg):
        l, p = cfg["layers"][i], "l%d" % i
        if opens:
            x = torch.cat([x, x0], -1) @ w["loop.in"].T
        h = rms(x, eps) * w[p + ".norm1"]
        if l["type"] == "attention":
            out = conv_attention(h, w, p + ".mix", l["mixer"], eps)
        elif l["type"] == "parallel":
            out = parallel_mixer(h, w, p + ".mix", l["mixer"], eps)
        else:
            raise ValueError(l["type"])
        if l.get("mlp"):
            out = out + relu_glu(h, w, p + ".mlp")
        x = x + out
        hidden.append(x)
    lg = (rms(x, eps) * w["final.norm"]) @ w["embed"].T
    cap = cfg.get("logit_softcap")
    if cap:
        lg = cap * torch.tanh(lg / cap)
    return (lg, torch.stack(hidden)) if return_hidden else lg
