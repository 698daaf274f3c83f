"""Every Ramalix mechanism alone on the GPU (torch wrappers of pegainfer_amd/ops_blocks.py over the HIP blocks) against its
function in the plain restatement (oracle/ramalix_ref.py), in both storage types; and crafted inputs where random weights
would hide a fault: one far key whose score stands out, marked keys just inside and just outside a block's edge in prompts
and in decoding, a sink that takes nearly all of the weight, a far write that one key channel keeps and another forgets,
state regions used by another request before."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as Fn

import ramalix_common as C
from oracle import ramalix_ref as R

pytestmark = pytest.mark.gpu

DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
F = torch.float64


def dev(t, dtype):
    return t.to(DT[dtype]).cuda().contiguous()


def close(got, ref, dtype, tol32=2e-5, tol16=3e-2):
    got, ref = got.detach().double().cpu(), ref.double()
    err = float((got - ref).abs().max() / ref.abs().max().clamp_min(1e-9))
    assert err < (tol32 if dtype == "float32" else tol16), err


def B():
    from pegainfer_amd import ops_blocks
    return ops_blocks


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("d", [50, 1024, 1300, 5000, 9001])        # one to thirty-two values per thread, then the two-pass form
def test_residual_sum_and_one_number_norm(dtype, d):
    g = torch.Generator().manual_seed(d)
    rows = 5
    x, extra = torch.randn(rows, d, generator=g) * 3, torch.randn(rows, d, generator=g)
    y, bias, vec = (C.bf16_round(torch.randn(*s, generator=g)) for s in ((rows, d), (d,), (d,)))
    gain = C.bf16_round(torch.tensor(1.3))
    r, n = B().scalar_rms_add(x.cuda(), dev(gain, dtype), 1e-5, y=dev(y, dtype), bias=dev(bias, dtype), mult=0.7, add_rows=extra.cuda(),
                              add_vec=dev(vec, dtype))
    ref = x.double() + 0.7 * (y.double() + bias.double()) + extra.double() + vec.double()
    close(r, ref, "float32", tol32=2e-6)
    close(n, R.snorm(ref, gain.double(), 1e-5), "float32", tol32=2e-6)
    xd = x.cuda()
    _, n = B().scalar_rms_add(xd, dev(gain, dtype), 1e-5)                                 # the norm alone: the first layer's form
    close(n, R.snorm(x.double(), gain.double(), 1e-5), "float32", tol32=2e-6)
    r, none = B().scalar_rms_add(xd, dev(gain, dtype), 1e-5, y=dev(y, dtype), mult=2.0, norm=False)   # the sum alone: the last layer's
    close(r, x.double() + 2.0 * y.double(), "float32", tol32=2e-6)
    assert none is None


class Paged:
    """one request's cache part over scattered pages, as a runtime lays it out: [k: slot, kv head, qd | v: slot, kv head, vdim]
    at offsets that do not start the page"""

    def __init__(self, page_ids, G, qd, dv, dtype, page_size=16):
        self.page_size = page_size
        self.k_off, self.v_off = 5 * 16, 5 * 16 + page_size * G * qd
        self.page_stride = self.v_off + page_size * G * dv + 3
        self.cache = torch.full(((max(page_ids) + 2) * self.page_stride,), float("nan"), dtype=DT[dtype], device="cuda")
        self.indptr = torch.tensor([0, len(page_ids)], dtype=torch.int32, device="cuda")
        self.pids = torch.tensor(page_ids, dtype=torch.int32, device="cuda")


def run_two_map(m, w, p, h, dtype, plan, page_ids, eps=1e-5):
    """the two-map attention as the runtime strings it together; plan: rows per step of ONE request whose pages are page_ids"""
    Bk = B()
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    Wp = torch.cat([w[p + ".q"], w[p + ".k"], w[p + ".v"]])
    offs = [0, H * 2 * d, (H + G) * 2 * d]
    pc = Paged(page_ids, G, 2 * d, dv, dtype)
    qt = m.get("q_temp") or {"coef": 0.0, "every": 0}
    lam = R.diff_lambda(w, p, m["diff"])
    outs, at = [], 0
    for n in plan:
        rg = Bk.Ragged([n], starts=[at])
        proj = Bk.linear(dev(h[at:at + n], dtype), dev(Wp, dtype), plain=True)
        q = Bk.qk_prep_paged(proj, offs, H, G, 2 * d, dv, rg, pc.indptr, pc.pids, pc.cache, pc.page_stride, pc.k_off, pc.v_off, 16,
                             q_bias=dev(w[p + ".q.b"], dtype), k_bias=dev(w[p + ".k.b"], dtype), v_bias=dev(w[p + ".v.b"], dtype),
                             qt_coef=qt["coef"], qt_every=qt["every"])
        mix = Bk.paged_attention_ex(q, pc.cache, pc.page_stride, pc.k_off, pc.v_off, 16, rg, pc.indptr, pc.pids, G, dv, m["scale"],
                                    factor=1.0 - m["diff"], maps=2, lam=lam, head_norm=True, norm_eps=eps)
        outs.append(Bk.linear(mix, dev(w[p + ".o"], dtype), plain=True).float() + w[p + ".o.b"].cuda())
        at += n
    return torch.cat(outs)


def run_block(m, w, p, h, dtype, plan, page_ids):
    Bk = B()
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    Wp = torch.cat([w[p + ".q"], w[p + ".k"], w[p + ".v"]])
    offs = [0, H * d, (H + G) * d]
    pc = Paged(page_ids, G, d, dv, dtype)
    rot = m.get("rot") or {"dims": 0, "base": 1.0}
    inv_freq = torch.tensor([rot["base"] ** (-2.0 * i / rot["dims"]) for i in range(rot["dims"] // 2)] or [0.0], dtype=torch.float32).cuda()
    outs, at = [], 0
    for n in plan:
        rg = Bk.Ragged([n], starts=[at])
        proj = Bk.linear(dev(h[at:at + n], dtype), dev(Wp, dtype), plain=True)
        q = Bk.qk_prep_paged(proj, offs, H, G, d, dv, rg, pc.indptr, pc.pids, pc.cache, pc.page_stride, pc.k_off, pc.v_off, 16,
                             inv_freq=inv_freq, rot_dims=rot["dims"])
        mix = Bk.paged_attention_ex(q, pc.cache, pc.page_stride, pc.k_off, pc.v_off, 16, rg, pc.indptr, pc.pids, G, dv, m["scale"],
                                    block=(m.get("mask") or {"size": 0})["size"], sink=dev(w[p + ".sink"], dtype))
        outs.append(Bk.linear(mix, dev(w[p + ".o"], dtype), plain=True))
        at += n
    return torch.cat(outs)


PAGES = [7, 2, 11, 0, 5, 9, 3, 12, 1, 10]        # ten pages of 16 tokens, in no order
# portions that end just before, at and just after page (16), block (24 / 50 / 80) and key tile (64) borders, then token by token
PORTIONS = [15, 1, 1, 6, 2, 23, 1, 1, 14, 2, 14] + [1] * 70


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("layer", [("a", 2), ("wide", 2), ("odd", 0), ("b", 1)])
def test_two_map_attention_whole_and_in_portions_over_scattered_pages(dtype, layer):
    cfg = {"a": C.config_a, "wide": C.config_wide_heads, "odd": C.config_odd, "b": C.config_b}[layer[0]]()
    w = C.random_weights(cfg, 4)
    p, m = "l%d.mix" % layer[1], cfg["layers"][layer[1]]["mixer"]
    n = 150
    h = C.bf16_round(torch.randn(n, cfg["width"], generator=torch.Generator().manual_seed(8)))
    ref = R.differential_attention(h.double(), w, p, m, 1e-5)
    close(run_two_map(m, w, p, h, dtype, [n], PAGES), ref, dtype, tol32=1e-4, tol16=6e-2)
    close(run_two_map(m, w, p, h, dtype, PORTIONS, PAGES), ref, dtype, tol32=1e-4, tol16=6e-2)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("layer", [("a", 0), ("a", 3), ("wide", 0), ("odd", 2), ("b", 0)])
def test_block_attention_whole_and_in_portions_over_scattered_pages(dtype, layer):
    cfg = {"a": C.config_a, "wide": C.config_wide_heads, "odd": C.config_odd, "b": C.config_b}[layer[0]]()
    w = C.random_weights(cfg, 5)
    p, m = "l%d.mix" % layer[1], cfg["layers"][layer[1]]["mixer"]
    n = 150
    h = C.bf16_round(torch.randn(n, cfg["width"], generator=torch.Generator().manual_seed(9)))
    ref = R.sink_block_attention(h.double(), w, p, m, 1e-5)
    close(run_block(m, w, p, h, dtype, [n], PAGES), ref, dtype, tol32=1e-4, tol16=6e-2)
    close(run_block(m, w, p, h, dtype, PORTIONS, PAGES), ref, dtype, tol32=1e-4, tol16=6e-2)


def marked_keys(n, d, dv, marks, askers, seed=2):
    """projection rows [q | k | v] in which every query and key looks along `base`, except the keys at `marks` and the queries
    at `askers`, which look along a direction orthogonal to it: an asker's weight goes to the marked keys it can see"""
    g = torch.Generator().manual_seed(seed)
    proj = torch.zeros(n, 2 * d + dv)
    base = torch.randn(d, generator=g)
    mark = torch.randn(d, generator=g)
    mark -= base * (mark @ base) / (base @ base)
    proj[:, :d] = base
    proj[:, d:2 * d] = base
    proj[:, 2 * d:] = torch.randn(n, dv, generator=g)
    for j in marks:
        proj[j, d:2 * d] = mark * 3
    for i in askers:
        proj[i, :d] = mark * 3
    return proj


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("n_split", [2, 5, 16])
def test_key_splits_agree_with_the_unsplit_launch(dtype, n_split):
    """decoding over a long context deals a row's key tiles to several workgroups and folds their softmax states: both attention
    forms, splits that get no tile at all (16 splits over 3 key tiles), a block that begins in the middle of a key tile"""
    Bk = B()
    cfg = C.config_wide_heads()
    w = C.random_weights(cfg, 7)
    n = 150
    h = C.bf16_round(torch.randn(n, cfg["width"], generator=torch.Generator().manual_seed(11)))
    for li, maps in ((2, 2), (0, 1)):
        p, m = "l%d.mix" % li, cfg["layers"][li]["mixer"]
        H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        qd = maps * d
        pc = Paged(PAGES, G, qd, dv, dtype)
        proj = Bk.linear(dev(h, dtype), dev(torch.cat([w[p + ".q"], w[p + ".k"], w[p + ".v"]]), dtype), plain=True)
        offs = [0, H * qd, (H + G) * qd]
        rg = Bk.Ragged([n])
        Bk.qk_prep_paged(proj, offs, H, G, qd, dv, rg, pc.indptr, pc.pids, pc.cache, pc.page_stride, pc.k_off, pc.v_off, 16)
        form = dict(maps=2, lam=0.37, head_norm=True, norm_eps=1e-5, factor=0.3) if maps == 2 else \
            dict(block=50, sink=dev(w[p + ".sink"], dtype))
        for at in (n - 1, 127, 128, 3):          # single rows at several positions, as decoding brings them
            one = Bk.Ragged([1], starts=[at])
            q = Bk.qk_prep_paged(proj[at:at + 1], offs, H, G, qd, dv, one, pc.indptr, pc.pids, pc.cache, pc.page_stride, pc.k_off,
                                 pc.v_off, 16)
            args = (q, pc.cache, pc.page_stride, pc.k_off, pc.v_off, 16, one, pc.indptr, pc.pids, G, dv, m["scale"])
            whole = Bk.paged_attention_ex(*args, **form)
            cut = Bk.paged_attention_ex(*args, n_split=n_split, **form)
            close(cut, whole.double().cpu(), "float32", tol32=2e-6 if dtype == "float32" else 1e-2)
            if dtype == "bfloat16":      # the matrix-core kernel (the default for a bf16 cache) against the fp32-FMA kernel
                close(Bk.paged_attention_ex(*args, plain=True, **form), whole.double().cpu(), "float32", tol32=2e-2)
                close(Bk.paged_attention_ex(*args, plain=True, n_split=n_split, **form), whole.double().cpu(), "float32", tol32=2e-2)


def attend(proj, d, dv, plan, scale=4.0, **form):
    Bk = B()
    n = proj.shape[0]
    pages = list(range((n + 15) // 16))[::-1]
    pc = Paged(pages, 1, d, dv, "float32")
    pc.cache.zero_()
    rows, at = [], 0
    for k in plan:
        rg = Bk.Ragged([k], starts=[at])
        q = Bk.qk_prep_paged(proj[at:at + k].cuda().contiguous(), [0, d, 2 * d], 1, 1, d, dv, rg, pc.indptr, pc.pids, pc.cache,
                             pc.page_stride, pc.k_off, pc.v_off, 16)
        rows.append(Bk.paged_attention_ex(q, pc.cache, pc.page_stride, pc.k_off, pc.v_off, 16, rg, pc.indptr, pc.pids, 1, dv, scale, **form))
        at += k
    return torch.cat(rows).cpu()


def test_attention_finds_one_far_key_among_hundreds_and_stops_at_the_causal_edge():
    n, d, dv = 700, 16, 24
    proj = marked_keys(n, d, dv, marks=[5, n - 1], askers=[n - 2, n - 1])
    v = proj[:, 2 * d:]
    for plan in ([n], [5, 1, 58, 1, 634, 1]):
        out = attend(proj, d, dv, plan)
        assert float((out[n - 2] - v[5]).abs().max()) < 1e-3          # the far key alone; key n - 1 is in this row's future
        assert float((out[n - 1] - 0.5 * (v[5] + v[n - 1])).abs().max()) < 1e-3
        assert float((out[3] - v[:4].mean(0)).abs().max()) < 1e-4     # the first tokens: equal scores, the mean of what is visible


@pytest.mark.parametrize("size", [24, 64, 100])
def test_block_edges_in_prompts_and_in_decoding(size):
    """marked keys at the last position of block 1 and the first of block 2; askers on both sides of that edge and at the far
    end of block 2: the asker in block 1 sees the first mark only, the askers in block 2 see the second only, never the first,
    however the prompt is cut (whole, a portion that ends ON the edge, single tokens across it)"""
    d, dv = 16, 24
    e = 2 * size                                       # first position of block 2
    n = 3 * size
    proj = marked_keys(n, d, dv, marks=[e - 1, e], askers=[e - 1, e, e + 1, n - 1])
    v = proj[:, 2 * d:]
    for plan in ([n], [e, n - e], [e - 1] + [1] * 3 + [n - e - 2], [e + 1] + [1] * (n - e - 1)):
        out = attend(proj, d, dv, plan, block=size)
        assert float((out[e - 1] - v[e - 1]).abs().max()) < 1e-3
        for i in (e, e + 1, n - 1):
            assert float((out[i] - v[e]).abs().max()) < 1e-3, (plan, i)
        i = e + 3                                      # an ordinary row of block 2: the mean over its block so far - but key e
        sc = torch.full((4,), 4.0 * float(proj[i, :d] @ proj[i, d:2 * d]))      # looks elsewhere and scores 0 against `base`
        sc[0] = 0.0
        pr = torch.softmax(sc, 0)
        assert float((out[i] - (pr[:, None] * v[e:e + 4]).sum(0)).abs().max()) < 1e-4


def test_sink_takes_its_share_of_the_weight():
    """all scores equal to zero (zero queries): with a sink logit s over j visible keys every key weighs 1 / (j + e^s)"""
    n, d, dv = 70, 8, 12
    proj = torch.zeros(n, 2 * d + dv)
    proj[:, 2 * d:] = torch.randn(n, dv, generator=torch.Generator().manual_seed(1))
    v = proj[:, 2 * d:]
    for s in (-30.0, 0.0, 2.0, 30.0):
        out = attend(proj, d, dv, [n], sink=torch.tensor([s], device="cuda"))
        for i in (0, 1, 63, 64, 69):
            ref = v[:i + 1].sum(0) / (i + 1 + math.exp(s))
            assert float((out[i] - ref).abs().max()) < 1e-5, (s, i)


def run_channel_delta(m, w, p, h, dtype, plan, ranks, eps=1e-5, slot=1):
    Bk = B()
    H, G, d, dv, taps = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]
    cc = 2 * G * d + H * dv
    pad8 = lambda v: (v + 7) // 8 * 8  # noqa: E731
    o_b, o_a1 = pad8(cc), pad8(pad8(cc) + H)
    o_g1 = pad8(o_a1 + ranks[0])
    rows = pad8(o_g1 + ranks[1])
    Wp = torch.zeros(rows, h.shape[1])
    at_ = 0
    for name in (".q", ".k", ".v"):
        Wp[at_:at_ + w[p + name].shape[0]] = w[p + name]
        at_ += w[p + name].shape[0]
    Wp[o_b:o_b + H] = w[p + ".b"]
    Wp[o_a1:o_a1 + ranks[0]] = w[p + ".a1"]
    Wp[o_g1:o_g1 + ranks[1]] = w[p + ".g1"]
    Wc = torch.cat([w[p + ".q.conv"], w[p + ".k.conv"], w[p + ".v.conv"]])
    conv_state = torch.full((3, max(taps - 1, 1), cc), 7.0, device="cuda")
    mem = torch.full((3, H * d * dv), 7.0, device="cuda")        # dirty neighbours; the request's own slot starts from zero
    conv_state[slot].zero_()
    mem[slot].zero_()
    outs, at = [], 0
    for n in plan:
        rg = Bk.Ragged([n], slots=[slot])
        proj = Bk.linear(dev(h[at:at + n], dtype), dev(Wp, dtype), plain=True)
        qkv = Bk.time_conv(proj, dev(Wc, dtype), conv_state if taps > 1 else conv_state[:, :0], rg, silu=True, out_dtype=torch.float32,
                           channels=cc)
        a = Bk.linear(proj[:, o_a1:o_a1 + ranks[0]], dev(w[p + ".a2"], dtype), out_dtype=torch.float32, plain=True)
        gate = Bk.linear(proj[:, o_g1:o_g1 + ranks[1]], dev(w[p + ".g2"], dtype), plain=True)
        o = Bk.delta_rule_channel(qkv, proj, o_b, a, dev(w[p + ".A_log"], dtype), dev(w[p + ".dt_bias"], dtype), mem, H, G, d, dv, rg)
        mix = Bk.head_rms_gate(o, dev(w[p + ".norm"], dtype), gate, "sigmoid", 1.0, eps, H, dv)
        outs.append(Bk.linear(mix, dev(w[p + ".o"], dtype), plain=True))
        at += n
    assert float(mem[0].min()) == 7.0 and float(mem[2].max()) == 7.0
    return torch.cat(outs)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("layer", [("a", 1), ("a", 4), ("wide", 1), ("odd", 1), ("b", 2)])
def test_channel_delta_whole_and_in_portions(dtype, layer):
    cfg = {"a": C.config_a, "wide": C.config_wide_heads, "odd": C.config_odd, "b": C.config_b}[layer[0]]()
    w = C.random_weights(cfg, 6)
    L = cfg["layers"][layer[1]]
    p, m = "l%d.mix" % layer[1], L["mixer"]
    n = 75
    h = C.bf16_round(torch.randn(n, cfg["width"], generator=torch.Generator().manual_seed(10)))
    ref = R.channel_delta(h.double(), w, p, m, 1e-5)
    close(run_channel_delta(m, w, p, h, dtype, [n], L["_ranks"]), ref, dtype, tol32=1e-4, tol16=8e-2)
    # portions shorter than the convolution's reach, rounds of 16 tokens that end inside a portion, single tokens
    close(run_channel_delta(m, w, p, h, dtype, [2, 1, 1, 13, 16, 17, 2] + [1] * 23, L["_ranks"]), ref, dtype, tol32=1e-4, tol16=8e-2)


def test_a_far_write_is_kept_by_one_key_channel_and_forgotten_by_another():
    """two writes at token 1 and 2, along key channels 0 and 1; channel 0 never decays (decay input -40: softplus = 0), channel
    1 loses a tenth per token; 400 tokens of nothing later (beta = 0) a query along channel 0 reads its value back whole, a
    query along channel 1 reads 0.9^398 of its value - per CHANNEL, not per head"""
    Bk = B()
    n, d, dv = 402, 8, 20
    g = torch.Generator().manual_seed(3)
    vals = torch.randn(2, dv, generator=g)
    qkv = torch.zeros(n, 2 * d + dv)
    qkv[1, d + 0] = 1.0                      # key of token 1: channel 0
    qkv[2, d + 1] = 1.0                      # key of token 2: channel 1
    qkv[1, 2 * d:] = vals[0]
    qkv[2, 2 * d:] = vals[1]
    qkv[n - 2, 0] = 1.0                      # query of token n - 2 along channel 0, of token n - 1 along channel 1
    qkv[n - 1, 1] = 1.0
    proj = torch.full((n, 1), -40.0)         # beta = sigmoid(-40): nothing is written ...
    proj[1] = proj[2] = 40.0                 # ... except at tokens 1 and 2
    a = torch.full((n, d), -40.0)
    a[:, 1] = math.log(math.expm1(-math.log(0.9)))       # softplus^-1(-ln 0.9): channel 1 decays by 0.9 per token
    zero = torch.zeros(d, device="cuda")
    for plan in ([n], [1, 1, 1, 199, 1, 198, 1]):
        mem = torch.zeros(1, d * dv, device="cuda")
        outs, at = [], 0
        for k in plan:
            outs.append(Bk.delta_rule_channel(qkv[at:at + k].cuda().contiguous(), proj[at:at + k].cuda().contiguous(), 0,
                                              a[at:at + k].cuda().contiguous(), torch.zeros(1, device="cuda"), zero, mem, 1, 1, d, dv,
                                              Bk.Ragged([k])))
            at += k
        out = torch.cat(outs).cpu() * d ** 0.5           # the rule scales its queries by dim^-1/2
        assert float((out[n - 2] - vals[0]).abs().max()) < 1e-4
        assert float((out[n - 1] - vals[1] * 0.9 ** (n - 1 - 2)).abs().max()) < 1e-4 * 0.9 ** (n - 3) + 1e-12
        assert float(out[n - 1].abs().max()) > 0


@pytest.mark.parametrize("groups", [(1, 1), (2, 1), (4, 2), (3, 3), (12, 5)])
@pytest.mark.parametrize("top", [1, 2])
def test_group_limited_router_from_logits_beside_other_columns(groups, top):
    g = torch.Generator().manual_seed(groups[0] * 10 + top)
    E, rows = 12, 37
    z = torch.randn(rows, E + 3, generator=g) * 2           # three more columns after the experts: they are not read
    e, wgt = B().route_from_logits_ex(z.cuda(), E, top, n_groups=groups[0], keep_groups=groups[1])
    idx, val = R.router(z[:, :E].double(), {"r.router": torch.eye(E)}, "r", {"experts": E, "top": top,
                                                                            "groups": {"count": groups[0], "keep": groups[1]}})
    assert torch.equal(e.cpu().long(), idx)
    assert torch.allclose(wgt.cpu().double(), val, atol=1e-6)
    assert torch.allclose(wgt.sum(-1).cpu(), torch.ones(rows), atol=1e-6)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_weighted_sum_with_a_gated_shared_row(dtype):
    g = torch.Generator().manual_seed(5)
    rows, top, d = 6, 3, 70
    y, wgt = torch.randn(rows * top, d, generator=g), torch.rand(rows, top, generator=g)
    add = C.bf16_round(torch.randn(rows, d, generator=g))
    logits = torch.randn(rows, 9, generator=g)
    out = B().route_combine_gated(y.cuda(), wgt.cuda(), dev(add, dtype), logits.cuda()[:, 8], DT[dtype])
    ref = (wgt[:, :, None].double() * y.reshape(rows, top, d).double()).sum(1) + torch.sigmoid(logits[:, 8:9].double()) * add.double()
    close(out, ref, dtype, tol32=2e-6, tol16=1e-2)
    out = B().route_combine_gated(y.cuda(), wgt.cuda(), None, None, DT[dtype])
    close(out, (wgt[:, :, None].double() * y.reshape(rows, top, d).double()).sum(1), dtype, tol32=2e-6, tol16=1e-2)
