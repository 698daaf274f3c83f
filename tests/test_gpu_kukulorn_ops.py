"""Every Kukulorn mechanism alone on the GPU (torch wrappers of pegainfer_amd/ops_blocks.py over the HIP blocks) against its
function in the plain restatement (oracle/kukulorn_ref.py), in both storage types; and crafted inputs where random weights would
hide a fault: one far key whose score stands out among hundreds, marked keys just inside and just outside the window and the kept
first tokens in prompts and in decoding, a soft cap that binds, a distance bias that decides the softmax, a state that one old
token wrote and a fast decay forgets, state regions and pages used by another request before."""
import math

import numpy as np
import pytest
import torch

import kukulorn_common as C
from oracle import kukulorn_ref as R

pytestmark = pytest.mark.gpu

DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
F = torch.float64


def dev(t, dtype):
    return t.to(DT[dtype]).cuda().contiguous()


def close(got, ref, dtype, tol32=2e-5, tol16=3e-2):
    got, ref = got.detach().double().cpu(), ref.double()
    err = float((got - ref).abs().max() / ref.abs().max().clamp_min(1e-9))
    assert err < (tol32 if dtype == "float32" else tol16), err


def close_rows(got, ref, dtype, tol32=1e-4, tol16=6e-2):
    """fp32: every value.  bf16: per row; one row in fifty (or one) may be off by more.  A single-headed state-space layer reads
    y = (dt B.C + D) x through a norm that forgets its scale: where that factor happens to cancel, rounding the projection to bf16
    moves the restatement itself by 8 % (measured on the CPU); a fault that hits single rows is the fp32 run's to find."""
    if dtype == "float32":
        return close(got, ref, dtype, tol32=tol32)
    got, ref = got.detach().double().cpu(), ref.double()
    err = (got - ref).abs().max(-1).values / ref.abs().max().clamp_min(1e-9)
    assert float(err.median()) < tol16 / 2 and int((err > tol16).sum()) <= max(1, err.numel() // 50), (float(err.median()), float(err.max()))


def B():
    from pegainfer_amd import ops_blocks
    return ops_blocks


def w64(w):
    return {k: v.double() for k, v in w.items()}


# ------------------------------------------------------------------ norms, sums, activations
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("d", [50, 1024, 1300, 5000, 9001])        # one to thirty-two values per thread, then the two-pass form
def test_sum_of_normed_and_plain_terms_then_norm(dtype, d):
    g = torch.Generator().manual_seed(d)
    rows, eps = 5, 1e-6
    x = torch.randn(rows, d, generator=g) * 3
    y1, y2, y3, b1, w1, w2, gain = (C.bf16_round(torch.randn(*s, generator=g)) for s in
                                    ((rows, d), (rows, d), (rows, d), (d,), (d,), (d,), (d,)))
    terms = [(dev(y1, dtype), dev(b1, dtype), dev(w1, dtype), 0.5), (dev(y2, dtype), None, dev(w2, dtype), 0.5), (dev(y3, dtype), None, None, 1.0)]
    r, n = B().terms_rms_add(x.cuda(), terms, gain=dev(gain, dtype), eps=eps, out_dtype=torch.float32)
    ref = x.double() + 0.5 * R.rms(y1.double() + b1.double(), eps) * w1.double() + 0.5 * R.rms(y2.double(), eps) * w2.double() + y3.double()
    close(r, ref, "float32", tol32=3e-6)
    close(n, R.rms(ref, eps) * gain.double(), "float32", tol32=3e-6)
    r, n = B().terms_rms_add(x.cuda(), [], gain=dev(gain, dtype), eps=eps)                   # the norm alone, stored type out
    close(n, R.rms(x.double(), eps) * gain.double(), dtype, tol32=3e-6, tol16=1e-2)
    r, n = B().terms_rms_add(x.cuda(), terms[2:], gain=None)                                 # the sum alone
    close(r, x.double() + y3.double(), "float32", tol32=3e-6)
    assert n is None
    wide = dev(torch.cat([y1, y3], 1), dtype)                                                # a term that is a column range
    r, _ = B().terms_rms_add(x.cuda(), [(wide[:, d:], None, None, 2.0)], gain=None)
    close(r, x.double() + 2.0 * y3.double(), "float32", tol32=3e-6)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_glu_activations_and_soft_cap(dtype):
    g = torch.Generator().manual_seed(1)
    gu = C.bf16_round(torch.randn(7, 2 * 37 + 5, generator=g) * 2)
    d = dev(gu, dtype)
    gate, up = gu[:, :37].double(), gu[:, 40:77].double()
    for act, fn in (("relu", torch.relu), ("silu", lambda t: t * torch.sigmoid(t)),
                    ("gelu_tanh", lambda t: 0.5 * t * (1 + torch.tanh(math.sqrt(2 / math.pi) * (t + 0.044715 * t ** 3))))):
        close(B().glu_rows(d[:, :37], d[:, 40:77], act), fn(gate) * up, dtype, tol16=1e-2)
    x = torch.randn(3, 1000, generator=g) * 40
    close(B().softcap_rows(x.cuda(), 30.0), 30.0 * torch.tanh(x.double() / 30.0), "float32", tol32=1e-6)
    assert float(B().softcap_rows(x.cuda(), 30.0).abs().max()) <= 30.0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", [(3, 16), (1, 100), (5, 7), (2, 200)])
def test_gate_before_the_norm_in_groups(dtype, shape):
    heads, vd = shape
    g = torch.Generator().manual_seed(heads)
    o = torch.randn(9, heads * vd, generator=g)
    z, w = C.bf16_round(torch.randn(9, heads * vd + 3, generator=g)), C.bf16_round(1 + 0.2 * torch.randn(heads * vd, generator=g))
    zd = dev(z, dtype)
    got = B().head_gate_rms(o.cuda(), dev(w, dtype), zd[:, 3:], "silu", 1e-6, heads, vd, gate_first=True)
    gated = o.double() * R.silu(z[:, 3:].double())
    close(got, R.rms(gated.view(9, heads, vd), 1e-6).reshape(9, -1) * w.double(), dtype, tol16=2e-2)
    got = B().head_gate_rms(o.cuda(), dev(w, dtype), zd[:, 3:], "silu", 1e-6, heads, vd, gate_first=False)       # the other order differs
    close(got, R.rms(o.double().view(9, heads, vd), 1e-6).reshape(9, -1) * w.double() * R.silu(z[:, 3:].double()), dtype, tol16=2e-2)


# ------------------------------------------------------------------ time convolution with biases
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("taps", [1, 2, 4, 7])
def test_time_convolution_with_input_and_output_bias_in_portions(dtype, taps):
    g = torch.Generator().manual_seed(taps)
    C_, lens = 70, [150, 9]
    u = [C.bf16_round(torch.randn(n, C_ + 4, generator=g)) for n in lens]
    w, ib, ob = (C.bf16_round(torch.randn(*s, generator=g) * 0.5) for s in ((C_, taps), (C_,), (C_,)))
    ref = [R.silu(R.tconv(x[:, 2:2 + C_].double() + ib.double(), w.double(), ob.double())) for x in u]
    for plan in ([[150, 9]], [[149, 1], [1, 8]], [[3, 2], [2, 1], [1, 1], [1, 1], [143, 4]]):
        state = torch.full((3, max(taps - 1, 1), C_), 7.0, device="cuda")       # slots 2 and 0 hold another request's tail
        state[[2, 0]] = 0.0
        outs, at = [[], []], [0, 0]
        for step in plan:
            rg = B().Ragged(step, slots=[2, 0])
            x = dev(torch.cat([u[i][at[i]:at[i] + n] for i, n in enumerate(step)]), dtype)
            o = B().time_conv(x[:, 2:], dev(w, dtype), state, rg, silu=True, out_dtype=torch.float32, channels=C_, in_bias=dev(ib, dtype),
                              out_bias=dev(ob, dtype))
            row = 0
            for i, n in enumerate(step):
                outs[i].append(o[row:row + n])
                at[i] += n
                row += n
        for i in range(2):
            close(torch.cat(outs[i]), ref[i], dtype, tol16=1e-2)
        assert float(state[1].min()) == 7.0                                      # a slot that is not in the step stays as it was


# ------------------------------------------------------------------ attention
class Paged:
    """one request's cache part over scattered pages, as a runtime lays it out: [k: slot, kv head, dim | v: slot, kv head, vdim]
    at offsets that do not start the page"""

    def __init__(self, page_ids, G, dim, dv, dtype, page_size=16):
        self.page_size = page_size
        self.k_off, self.v_off = 5 * 16, 5 * 16 + page_size * G * dim
        self.page_stride = self.v_off + page_size * G * dv + 3
        self.cache = torch.full(((max(page_ids) + 2) * self.page_stride,), float("nan"), dtype=DT[dtype], device="cuda")
        self.indptr = torch.tensor([0, len(page_ids)], dtype=torch.int32, device="cuda")
        self.pids = torch.tensor(page_ids, dtype=torch.int32, device="cuda")


PAGES = [7, 2, 11, 0, 5, 9, 3, 12, 1, 10, 4, 6, 8, 13, 14, 15, 16, 17, 18, 19]        # twenty pages of 16 tokens, in no order
# portions that end just before, at and just after page (16), window (21 / 40 / 70) and key tile (64) borders, then token by token
PORTIONS = [15, 1, 1, 6, 2, 23, 1, 1, 14, 2, 14] + [1] * 70


def dist_table(rel, bias_max):
    """the bias table expanded to one row per distance, as a runtime hands it to the attention"""
    rows = rel.shape[0]
    nd = 1
    while R.distance_bucket(nd - 1, rows, bias_max) < rows - 1:
        nd += 1
    return torch.stack([rel[R.distance_bucket(d, rows, bias_max)] for d in range(nd)]).float().cuda()


def run_conv_attention(m, w, p, h, dtype, plan, eps=1e-6):
    """the "attention" mixer as the runtime strings it together; plan: rows per step of ONE request"""
    Bk = B()
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    Wp = torch.cat([w[p + ".q"], w[p + ".k"], w[p + ".v"], w[p + ".g"]])
    ch = (H + G) * d + G * dv
    offs = [0, H * d, (H + G) * d]
    bias = torch.cat([w[p + ".q.b"], w[p + ".k.b"], w[p + ".v.b"]])
    pc = Paged(PAGES, G, d, dv, dtype)
    taps = m.get("conv", 0)
    state = torch.zeros((1, max(taps - 1, 1), ch), device="cuda")
    rot = m.get("rot")
    inv_freq = torch.tensor(R.rotation_frequencies(rot) if rot else [0.0], dtype=torch.float32).cuda()
    outs, at = [], 0
    for n in plan:
        rg = Bk.Ragged([n], starts=[at])
        proj = Bk.linear(dev(h[at:at + n], dtype), dev(Wp, dtype), plain=True)
        if taps:
            cw = torch.cat([w[p + ".q.conv"], w[p + ".k.conv"], w[p + ".v.conv"]])
            qkv = Bk.time_conv(proj, dev(cw, dtype), state, rg, out_dtype=torch.float32, channels=ch, in_bias=dev(bias, dtype))
            kw = {}
        else:
            qkv = proj
            kw = dict(q_bias=dev(w[p + ".q.b"], dtype), k_bias=dev(w[p + ".k.b"], dtype), v_bias=dev(w[p + ".v.b"], dtype))
        q = Bk.qk_prep_paged_form(qkv, offs, H, G, d, dv, rg, pc.indptr, pc.pids, pc.cache, pc.page_stride, pc.k_off, pc.v_off, 16,
                                  norm_kind="head_unit_after", eps=eps, inv_freq=inv_freq, rot_dims=rot["dims"] if rot else 0, halves=True, **kw)
        mix = Bk.paged_attention_masked(q, pc.cache, pc.page_stride, pc.k_off, pc.v_off, 16, rg, pc.indptr, pc.pids, G, dv, m["scale"],
                                        softcap=m.get("softcap", 0.0), gate=proj[:, ch:])
        outs.append(Bk.linear(mix, dev(w[p + ".o"], dtype), plain=True))
        at += n
    return torch.cat(outs)


def run_windowed_attention(m, w, p, h, dtype, plan, eps=1e-6, n_split=1):
    Bk = B()
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    Wp = torch.cat([w[p + ".q"], w[p + ".k"], w[p + ".v"], w[p + ".g"]])
    ch = (H + G) * d + G * dv
    offs = [0, H * d, (H + G) * d]
    pc = Paged(PAGES, G, d, dv, dtype)
    mk = m.get("mask") or {"size": 0, "keep_first": 0}
    tab = dist_table(w[p + ".rel"], m["bias_max"]) if m.get("bias_max") else None
    outs, at = [], 0
    for n in plan:
        rg = Bk.Ragged([n], starts=[at])
        proj = Bk.linear(dev(h[at:at + n], dtype), dev(Wp, dtype), plain=True)
        q = Bk.qk_prep_paged_form(proj, offs, H, G, d, dv, rg, pc.indptr, pc.pids, pc.cache, pc.page_stride, pc.k_off, pc.v_off, 16,
                                  q_norm=dev(w[p + ".q.norm"], dtype), k_norm=dev(w[p + ".k.norm"], dtype), norm_kind="all_weight", eps=eps,
                                  q_bias=dev(w[p + ".q.b"], dtype), k_bias=dev(w[p + ".k.b"], dtype), v_bias=dev(w[p + ".v.b"], dtype))
        mix = Bk.paged_attention_masked(q, pc.cache, pc.page_stride, pc.k_off, pc.v_off, 16, rg, pc.indptr, pc.pids, G, dv, m["scale"],
                                        window=mk["size"], keep_first=mk.get("keep_first", 0), dist_bias=tab, gate=proj[:, ch:],
                                        gate_per_head=True, n_split=n_split)
        outs.append(Bk.linear(mix, dev(w[p + ".o"], dtype), plain=True).float() + w[p + ".o.b"].cuda())
        at += n
    return torch.cat(outs)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("layer", [("a", 1), ("a", 2), ("a", 4), ("wide", 0), ("odd", 0), ("b", 0), ("b", 2)])
def test_convolved_rotated_capped_attention_whole_and_in_portions(dtype, layer):
    cfg = C.CONFIGS[layer[0]]()
    w = C.random_weights(cfg, 4)
    p, m = "l%d.mix" % layer[1], cfg["layers"][layer[1]]["mixer"]
    n = 150
    h = C.bf16_round(torch.randn(n, cfg["width"], generator=torch.Generator().manual_seed(8)))
    ref = R.conv_attention(h.double(), w64(w), p, m, 1e-6)
    close(run_conv_attention(m, w, p, h, dtype, [n]), ref, dtype, tol32=1e-4, tol16=6e-2)
    close(run_conv_attention(m, w, p, h, dtype, PORTIONS), ref, dtype, tol32=1e-4, tol16=6e-2)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("layer", [("a", 0), ("a", 3), ("wide", 1), ("odd", 1), ("odd", 2), ("b", 1)])
def test_windowed_biased_attention_whole_and_in_portions(dtype, layer):
    cfg = C.CONFIGS[layer[0]]()
    w = C.random_weights(cfg, 5)
    p, m = "l%d.mix.left" % layer[1], cfg["layers"][layer[1]]["mixer"]["left"]
    n = 150
    h = C.bf16_round(torch.randn(n, cfg["width"], generator=torch.Generator().manual_seed(9)))
    ref = R.windowed_attention(h.double(), w64(w), p, m, 1e-6)
    close(run_windowed_attention(m, w, p, h, dtype, [n]), ref, dtype, tol32=1e-4, tol16=6e-2)
    close(run_windowed_attention(m, w, p, h, dtype, PORTIONS), ref, dtype, tol32=1e-4, tol16=6e-2)
    close(run_windowed_attention(m, w, p, h, dtype, [100] + [1] * 50, n_split=5), ref, dtype, tol32=1e-4, tol16=6e-2)


def crafted_attention(dtype, n, plan, window=0, keep_first=0, softcap=0.0, tab=None, scale=1.0, hot=None, q_gain=1.0, n_split=1):
    """One head of 8 values whose queries and keys point along one axis: the key at `hot` is q_gain times longer, every value row
    carries its own position in its first column.  Returns what each row read from that column = the weighted mean position."""
    Bk = B()
    d = dv = 8
    q = torch.zeros(n, d)
    q[:, 0] = 1.0
    k = torch.zeros(n, d)
    k[:, 0] = 1.0
    if hot is not None:
        k[hot, 0] = q_gain
    v = torch.zeros(n, dv)
    v[:, 0] = torch.arange(n).float() / 64.0          # exact in bf16 up to 255 / 64... positions are told apart below by halves
    v[:, 1] = 1.0
    proj = dev(torch.cat([q, k, v], 1), dtype)
    pc = Paged(PAGES, 1, d, dv, dtype)
    outs, at = [], 0
    for m_ in plan:
        rg = Bk.Ragged([m_], starts=[at])
        qq = Bk.qk_prep_paged_form(proj[at:at + m_], [0, d, 2 * d], 1, 1, d, dv, rg, pc.indptr, pc.pids, pc.cache, pc.page_stride, pc.k_off,
                                   pc.v_off, 16)
        outs.append(Bk.paged_attention_masked(qq, pc.cache, pc.page_stride, pc.k_off, pc.v_off, 16, rg, pc.indptr, pc.pids, 1, dv, scale,
                                              softcap=softcap, window=window, keep_first=keep_first, dist_bias=tab, n_split=n_split))
        at += m_
    return torch.cat(outs).double().cpu()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("plan", [[300], [290] + [1] * 10, [64, 64, 2, 62, 2, 96, 10]])
def test_one_far_key_among_hundreds_takes_the_weight(dtype, plan):
    """key 3 scores 30 against 1 for every other key: every later row reads (nearly) position 3, in a prompt's portion and in
    decoding, with the keys cut over workgroups or not"""
    for n_split in (1, 7):
        out = crafted_attention(dtype, 300, plan, hot=3, q_gain=30.0, n_split=n_split)
        assert float((out[10:, 0] * 64.0 - 3.0).abs().max()) < 1e-3 and float((out[:3, 0] * 64.0 - 3.0).abs().min()) > 0.5
    # the same key under a soft cap of 2: its score is held at 2 tanh(15), the others at 2 tanh(0.5): it no longer wins alone
    out = crafted_attention(dtype, 300, plan, hot=3, q_gain=30.0, softcap=2.0)
    e_hot, e_rest = math.exp(2.0 * math.tanh(15.0)), math.exp(2.0 * math.tanh(0.5))
    for i in (50, 299):
        want = (3 * e_hot + (i * (i + 1) / 2 - 3) * e_rest) / (e_hot + i * e_rest) / 64.0
        assert abs(float(out[i, 0]) - want) < (1e-5 if dtype == "float32" else 2e-2) * want


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("plan", [[200], [120] + [1] * 80, [60, 2, 2, 1, 1, 70, 64]])
@pytest.mark.parametrize("shape", [(21, 5), (64, 0), (70, 17), (3, 2), (16, 16)])
def test_marked_keys_at_the_window_edge_and_among_the_kept_first(dtype, plan, shape):
    """a key 30 times longer than the rest is seen exactly by the rows whose window holds it - or by all later rows when it is
    one of the kept first tokens"""
    size, keep = shape
    for hot in (max(keep - 1, 0), keep, keep + 40, 100):
        out = crafted_attention(dtype, 200, plan, window=size, keep_first=keep, hot=hot, q_gain=30.0)[:, 0] * 64.0
        for i in (hot, hot + 1, hot + size - 1, hot + size, hot + size + 1, 199):
            if i >= 200:
                continue
            seen = hot < keep or i - hot < size
            if seen:
                assert abs(float(out[i]) - hot) < 1e-2, (hot, i, float(out[i]))
            else:        # the row reads the mean position of what it does see (a bf16 output holds positions near 170 to +- 0.5)
                vis = [j for j in range(i + 1) if i - j < size or j < keep]
                assert abs(float(out[i]) - sum(vis) / len(vis)) < (1e-3 if dtype == "float32" else 1.01), (hot, i, float(out[i]))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_distance_bias_decides_the_softmax(dtype):
    """all keys alike; the bias table favours distance 9 by 25: every row reads the position 9 back (rows before 9: the mean of
    what they see); distances beyond the table's last row take that row"""
    tab = torch.zeros(12, 1)
    tab[9, 0] = 25.0
    for plan in ([100], [50] + [1] * 50):
        out = crafted_attention(dtype, 100, plan, tab=tab.cuda())[:, 0] * 64.0
        assert float((out[9:] - (torch.arange(9, 100).double() - 9)).abs().max()) < 1e-3
        assert abs(float(out[5]) - 2.5) < 1e-3
    tab = torch.zeros(12, 1)
    tab[11, 0] = 25.0               # every distance >= 11: the mean of positions 0 .. i - 11
    out = crafted_attention(dtype, 100, [100], tab=tab.cuda())[:, 0] * 64.0
    assert abs(float(out[99]) - 44.0) < (1e-3 if dtype == "float32" else 0.3) and abs(float(out[11]) - 0.0) < 1e-3


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_rotation_of_halves_with_given_frequencies_and_norm_after(dtype):
    g = torch.Generator().manual_seed(3)
    n, H, G, d, dv = 40, 3, 1, 14, 6
    rot = {"dims": 10, "base": 77.0, "scaling": {"factor": 5.0, "low": 1.0, "high": 3.0, "original": 30}}
    x = torch.randn(n, (H + G) * d + G * dv, generator=g)
    pc = Paged(PAGES, G, d, dv, dtype)
    rg = B().Ragged([n], starts=[100])           # a portion that starts at position 100
    inv_freq = torch.tensor(R.rotation_frequencies(rot), dtype=torch.float32).cuda()
    q = B().qk_prep_paged_form(x.cuda(), [0, H * d, (H + G) * d], H, G, d, dv, rg, pc.indptr, pc.pids, pc.cache, pc.page_stride, pc.k_off,
                               pc.v_off, 16, norm_kind="head_unit_after", eps=1e-6, inv_freq=inv_freq, rot_dims=10, halves=True)
    full = torch.zeros(140, H, d, dtype=F)
    full[100:] = x[:, :H * d].double().view(n, H, d)
    ref = R.rms(R.rotate_halves(full, rot), 1e-6)[100:]
    close(q, ref, "float32", tol32=3e-5)
    page, slot = PAGES[105 // 16], 105 % 16       # the key of position 105 sits in its page's slot
    kref = R.rms(R.rotate_halves(torch.cat([torch.zeros(100, G, d, dtype=F), x[:, H * d:(H + G) * d].double().view(n, G, d)]), rot), 1e-6)[105]
    got = pc.cache[page * pc.page_stride + pc.k_off + slot * G * d:][:G * d]
    close(got, kref.reshape(-1), dtype, tol32=3e-5, tol16=1e-2)


# ------------------------------------------------------------------ state-space scan
def run_state_space(m, w, p, h, dtype, plan, slots, state, conv_state, eps=1e-6):
    """the right half of "parallel" as the runtime strings it together; plan: steps of rows per entry; slots: entry -> state slot"""
    Bk = B()
    Hh, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner, ch = Hh * P, Hh * P + 2 * G * N
    outs, at = [[] for _ in h], [0] * len(h)
    for step in plan:
        live = [i for i, n in enumerate(step) if n]
        rg = Bk.Ragged([step[i] for i in live], slots=[slots[i] for i in live])
        x = dev(torch.cat([h[i][at[i]:at[i] + step[i]] for i in live]), dtype)
        proj = Bk.linear(x, dev(w[p + ".in"], dtype), plain=True)
        xbc = Bk.time_conv(proj[:, inner:], dev(w[p + ".conv"], dtype), conv_state, rg, silu=True, out_dtype=torch.float32, channels=ch,
                           out_bias=dev(w[p + ".conv.b"], dtype))
        y = Bk.ssd_scan(xbc, proj, inner + ch, dev(w[p + ".A_log"], dtype), dev(w[p + ".dt_bias"], dtype), dev(w[p + ".D"], dtype), state,
                        Hh, G, N, P, rg)
        ng = m.get("norm_groups", 1)
        mix = Bk.head_gate_rms(y, dev(w[p + ".norm"], dtype), proj, "silu", eps, ng, inner // ng, gate_first=True)
        o = Bk.linear(mix, dev(w[p + ".o"], dtype), plain=True)
        row = 0
        for i in live:
            outs[i].append(o[row:row + step[i]])
            at[i] += step[i]
            row += step[i]
    return [torch.cat(o) for o in outs]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("layer", [("a", 0), ("a", 3), ("wide", 1), ("odd", 1), ("odd", 2), ("b", 1)])
def test_state_space_layer_whole_in_portions_and_in_dirty_slots(dtype, layer):
    cfg = C.CONFIGS[layer[0]]()
    w = C.random_weights(cfg, 6)
    p, m = "l%d.mix.right" % layer[1], cfg["layers"][layer[1]]["mixer"]["right"]
    g = torch.Generator().manual_seed(10)
    h = [C.bf16_round(torch.randn(n, cfg["width"], generator=g)) for n in (90, 37)]
    ref = [R.state_space(x.double(), w64(w), p, m, 1e-6) for x in h]
    floats = m["heads"] * m["state"] * m["vdim"]
    ch = m["heads"] * m["vdim"] + 2 * m["groups"] * m["state"]
    for plan in ([[90, 37]], [[17, 1], [1, 1], [2, 2], [33, 0], [1, 33], [36, 0]], [[40, 30]] + [[1, 1]] * 7 + [[1, 0]] * 43):
        state = torch.full((4, floats), 3.0, device="cuda")              # slots 3 and 1 start from zero, the others hold strangers' state
        conv_state = torch.full((4, max(m["conv"] - 1, 1), ch), -2.0, device="cuda")
        state[[3, 1]] = 0.0
        conv_state[[3, 1]] = 0.0
        got = run_state_space(m, w, p, h, dtype, plan, [3, 1], state, conv_state)
        for i in range(2):
            close_rows(got[i], ref[i], dtype)
        assert float(state[0].min()) == 3.0 and float(state[2].max()) == 3.0


def test_an_old_write_is_kept_by_a_slow_head_and_forgotten_by_a_fast_one():
    """two heads read the same inputs; head 0 decays by exp(-0.001 dt), head 1 by exp(-20 dt).  Token 2 alone writes a large
    value: two hundred tokens later head 0 still reads it, head 1 reads nothing of it - in one step or token by token"""
    Bk = B()
    n, N, P = 260, 16, 8
    xbc = torch.zeros(n, 2 * P + 2 * N)
    xbc[:, 2 * P] = 1.0                      # B along the first state
    xbc[:, 2 * P + N] = 1.0                  # C along the first state
    xbc[2, :2 * P] = 50.0                    # the write
    proj = torch.zeros(n, 2)                 # raw step sizes 0: dt = softplus(0 + bias)
    A_log = torch.tensor([math.log(0.001), math.log(20.0)])
    dt_bias = torch.tensor([math.log(math.e - 1.0)] * 2)       # softplus -> 1
    D = torch.zeros(2)
    for plan in ([n], [10] + [1] * 250, [3, 1, 64, 64, 64, 64]):
        state = torch.zeros(1, 2 * N * P, device="cuda")
        ys, at = [], 0
        for m_ in plan:
            rg = Bk.Ragged([m_])
            ys.append(Bk.ssd_scan(xbc[at:at + m_].cuda(), proj[at:at + m_].cuda(), 0, A_log.cuda(), dt_bias.cuda(), D.cuda(), state, 2, 1, N, P, rg))
            at += m_
        y = torch.cat(ys).cpu()
        assert abs(float(y[202, 0]) - 50.0 * math.exp(-0.001 * 200)) < 1e-3 and abs(float(y[202, P])) < 1e-30
        assert abs(float(y[2, P]) - 50.0) < 1e-4 and float(y[1].abs().max()) == 0.0
