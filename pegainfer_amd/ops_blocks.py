"""Torch-tensor wrappers over include/pegainfer_kernels_blocks.h: the model-independent blocks that exist in a bf16 and a
true-fp32 instance (Dynamic-Tanh norms over an fp32 stream, activations, the strided / batched / grouped GEMM, attention
over a paged latent cache, routing; time convolutions with carried tails, grouped output norms with a depth-weighted
sum, clamp-GLU, recurrent matrix memories over per-request state, attention over a paged key/value cache).  Tensors are torch CUDA tensors used as device memory; the
storage type of a call (bf16 / fp32) is taken from the activation tensor.  Work is enqueued on torch's current stream.
No CPU fallback: without the HIP library every call raises ImportError.
"""
import ctypes

import torch

from . import ffi
from .ops import _chk, _p, _stream

EPI_NONE, EPI_RELU_SQ, EPI_SIGMOID_GATE = 0, 1, 2


def _dt(t):
    if t.dtype == torch.bfloat16:
        return 0
    if t.dtype == torch.float32:
        return 1
    raise TypeError("bf16 or fp32 tensors only")


class GemmDesc(ctypes.Structure):
    _fields_ = [("x", ctypes.c_void_p), ("w", ctypes.c_void_p), ("y", ctypes.c_void_p),
                ("x_dtype", ctypes.c_int32), ("w_dtype", ctypes.c_int32), ("y_dtype", ctypes.c_int32),
                ("m", ctypes.c_int32), ("k", ctypes.c_int32), ("rows", ctypes.c_int32), ("groups", ctypes.c_int32),
                ("x_row_stride", ctypes.c_int64), ("x_group_stride", ctypes.c_int64),
                ("w_m_stride", ctypes.c_int64), ("w_k_stride", ctypes.c_int64), ("w_group_stride", ctypes.c_int64),
                ("y_row_stride", ctypes.c_int64), ("y_group_stride", ctypes.c_int64),
                ("tile_group", ctypes.c_void_p), ("tile_row0", ctypes.c_void_p), ("tile_rows", ctypes.c_void_p),
                ("n_tiles", ctypes.c_void_p), ("max_tiles", ctypes.c_int32),
                ("x_row_index", ctypes.c_void_p), ("y_row_index", ctypes.c_void_p),
                ("epilogue", ctypes.c_int32), ("gate", ctypes.c_void_p), ("gate_dtype", ctypes.c_int32),
                ("gate_row_stride", ctypes.c_int64), ("max_tile_rows", ctypes.c_int32), ("tile_rows_cap", ctypes.c_int32),
                ("plain", ctypes.c_int32)]


def embed_f32(embed, token_ids_u32):
    out = torch.empty((token_ids_u32.numel(), embed.shape[1]), dtype=torch.float32, device=embed.device)
    _chk(ffi.lib().pegainfer_embed_f32(_p(embed), _p(token_ids_u32), _p(out), embed.shape[1], token_ids_u32.numel(),
                                       _dt(embed), _stream()), "embed_f32")
    return out


def dyt_norm(x_f32, alpha, w, b):
    """out = tanh(alpha x) w + b; x fp32 [rows, d]; alpha / w / b (and the result) in the storage type of w"""
    assert x_f32.dtype == torch.float32 and x_f32.is_contiguous()
    out = torch.empty(x_f32.shape, dtype=w.dtype, device=x_f32.device)
    _chk(ffi.lib().pegainfer_dyt_norm(_p(x_f32), _p(alpha), _p(w), _p(b), _p(out), x_f32.shape[-1],
                                      x_f32.numel() // x_f32.shape[-1], _dt(w), _stream()), "dyt_norm")
    return out


def dyt_add_norm(x_f32, y, post, nxt=None):
    """x += dyt(y; post) in place; returns dyt(x; nxt) when nxt = (alpha, w, b) is given"""
    assert x_f32.dtype == torch.float32 and x_f32.is_contiguous() and y.is_contiguous()
    out = torch.empty(y.shape, dtype=y.dtype, device=y.device) if nxt else None
    n = nxt or (None, None, None)
    _chk(ffi.lib().pegainfer_dyt_add_norm(_p(x_f32), _p(y), _p(post[0]), _p(post[1]), _p(post[2]), _p(n[0]), _p(n[1]), _p(n[2]),
                                          _p(out), y.shape[-1], y.numel() // y.shape[-1], _dt(y), _stream()), "dyt_add_norm")
    return out


def relu_sq(x):
    out = torch.empty_like(x)
    _chk(ffi.lib().pegainfer_relu_sq(_p(x), _p(out), x.numel(), _dt(x), _stream()), "relu_sq")
    return out


def silu_mul_rows(gate_up):
    rows, two_i = gate_up.shape
    out = torch.empty((rows, two_i // 2), dtype=gate_up.dtype, device=gate_up.device)
    _chk(ffi.lib().pegainfer_silu_mul_rows(_p(gate_up), _p(out), two_i // 2, rows, _dt(gate_up), _stream()), "silu_mul_rows")
    return out


def gemm_strided(desc):
    _chk(ffi.lib().pegainfer_gemm_strided(ctypes.addressof(desc), _stream()), "gemm_strided")


def linear(x, w, out_dtype=None, epilogue=EPI_NONE, plain=False):
    """y[T, M] = x[T, K] w[M, K]^T through pegainfer_gemm_strided (any sizes, bf16 or fp32 operands, fp32 accumulation; x may be
    a column range of a wider matrix); plain = the fp32-FMA tile kernel whatever the shape"""
    T, K = x.shape
    M = w.shape[0]
    y = torch.empty((T, M), dtype=out_dtype or x.dtype, device=x.device)
    d = GemmDesc(x=_p(x), w=_p(w), y=_p(y), x_dtype=_dt(x), w_dtype=_dt(w), y_dtype=_dt(y), m=M, k=K, rows=T, groups=1,
                 x_row_stride=x.stride(0), w_m_stride=K, w_k_stride=1, y_row_stride=M, epilogue=epilogue, plain=int(plain))
    gemm_strided(d)
    return y


def latent_prep(proj, dkv_offset, c_norm_w, eps, inv_freq, rot_dims, positions, token_req, page_indptr, page_ids, cache,
                page_stride, layer_off, page_size, qc, heads, nope, rot, rank):
    _chk(ffi.lib().pegainfer_latent_prep(_p(proj), proj.shape[1], dkv_offset, _p(c_norm_w), float(eps), _p(inv_freq), rot_dims,
                                         _p(positions), _p(token_req), _p(page_indptr), _p(page_ids), _p(cache), page_stride,
                                         layer_off, page_size, _p(qc), heads, nope, rot, rank, proj.shape[0], _dt(proj),
                                         _stream()), "latent_prep")


def row_tiles(lens, heads, device="cuda"):
    """the flattened (token, head) rows of a step with entries of `lens` tokens, cut into runs of <= 64 rows inside one entry"""
    row0, rows, at = [], [], 0
    for n in lens:
        for r in range(0, n * heads, 64):
            row0.append(at * heads + r)
            rows.append(min(64, n * heads - r))
        at += n
    return (torch.tensor(row0, dtype=torch.int32, device=device), torch.tensor(rows, dtype=torch.int32, device=device))


def latent_attention(qc, cache, page_stride, layer_off, page_size, positions, token_req, page_indptr, page_ids, rank, rot,
                     scale, max_kv_len, split_keys=0, tiles=None):
    """qc fp32 [T, heads, rank + rot] -> o_lat fp32 [T, heads, rank]; tiles = row_tiles(...) selects the matrix-core form"""
    T, H, E = qc.shape
    assert E == rank + rot and qc.dtype == torch.float32
    o = torch.empty((T, H, rank), dtype=torch.float32, device=qc.device)
    n = ffi.lib().pegainfer_latent_attention_workspace(T, H, rank, max_kv_len, split_keys)
    ws = torch.empty(max(int(n), 1), dtype=torch.float32, device=qc.device)
    t0, tr = tiles if tiles is not None else (None, None)
    _chk(ffi.lib().pegainfer_latent_attention(_p(qc), _p(o), _p(cache), page_stride, layer_off, page_size, _p(positions),
                                              _p(token_req), _p(page_indptr), _p(page_ids), H, rank, rot, float(scale), T,
                                              max_kv_len, split_keys, _p(ws), _p(t0), _p(tr), 0 if t0 is None else t0.numel(),
                                              _dt(cache), _stream()), "latent_attention")
    return o


def route(h, w_router, correction, n_groups, keep_groups, top):
    rows, d = h.shape
    e = torch.empty((rows, top), dtype=torch.int32, device=h.device)
    w = torch.empty((rows, top), dtype=torch.float32, device=h.device)
    _chk(ffi.lib().pegainfer_route_sigmoid_grouped(_p(h), _p(w_router), _p(correction), _p(e), _p(w), d, w_router.shape[0],
                                                   n_groups, keep_groups, top, rows, _dt(h), _stream()), "route")
    return e, w


def route_sort(expert, experts, rows_per_tile=64):
    """-> pos_pair, pos_row, tile_group, tile_row0, tile_rows, n_tiles (int32 device tensors), max_tiles"""
    rows, top = expert.shape
    P = rows * top
    max_tiles = (P + rows_per_tile - 1) // rows_per_tile + experts
    dev = expert.device
    pos_pair, pos_row = torch.empty(P, dtype=torch.int32, device=dev), torch.empty(P, dtype=torch.int32, device=dev)
    tg, t0, tr = (torch.zeros(max_tiles, dtype=torch.int32, device=dev) for _ in range(3))
    nt = torch.zeros(1, dtype=torch.int32, device=dev)
    _chk(ffi.lib().pegainfer_route_sort(_p(expert), P, top, experts, _p(pos_pair), _p(pos_row), _p(tg), _p(t0), _p(tr), _p(nt),
                                        max_tiles, rows_per_tile, _stream()), "route_sort")
    return pos_pair, pos_row, tg, t0, tr, nt, max_tiles


def route_combine(y_pairs, weight, out_dtype):
    rows, top = weight.shape
    d = y_pairs.shape[1]
    out = torch.empty((rows, d), dtype=out_dtype, device=y_pairs.device)
    _chk(ffi.lib().pegainfer_route_combine(_p(y_pairs), _p(weight), _p(out), d, top, rows, _dt(out), _stream()), "route_combine")
    return out


# ---- sequences with state: ragged batches (entry e = rows entry_row0[e] .. entry_row0[e + 1] - 1, state slot entry_slot[e]) ----
class Ragged:
    """device index arrays of a step whose entries have `lens` rows and use the state slots `slots`; positions start at
    `starts` (default 0)"""

    def __init__(self, lens, slots=None, starts=None, device="cuda"):
        slots = list(range(len(lens))) if slots is None else slots
        starts = [0] * len(lens) if starts is None else starts
        row0, ent, pos = [0], [], []
        for i, n in enumerate(lens):
            row0.append(row0[-1] + n)
            ent += [i] * n
            pos += list(range(starts[i], starts[i] + n))
        i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=device)  # noqa: E731
        self.lens, self.n, self.rows = list(lens), len(lens), row0[-1]
        self.entry_row0, self.entry_slot, self.row_entry, self.positions = i32(row0), i32(slots), i32(ent), i32(pos)


def time_conv(x, w, state, rg, residual=False, silu=False, out_dtype=None, channels=None, in_bias=None, out_bias=None):
    """causal per-channel convolution over time; state fp32 [slots, taps - 1, C] is read, then moved on by the step's rows.
    in_bias [C] joins every real input (and so the carried ones), out_bias [C] the sum before the activation; both in w's type"""
    C = channels or w.shape[0]
    taps = w.shape[1]
    out = torch.empty((x.shape[0], C), dtype=out_dtype or x.dtype, device=x.device)
    slot_stride = state.shape[1] * state.shape[2] if state.dim() == 3 else 0
    L = ffi.lib()
    if all(n == 1 for n in rg.lens):      # decoding: output and the moved-on tail in one launch
        _chk(L.pegainfer_time_conv_step_biased(_p(x), _dt(x), x.stride(0), _p(w), _dt(w), _p(in_bias), _p(out_bias), _p(state),
                                               slot_stride, _p(out), _dt(out), C, C, taps, (1 if residual else 0) | (2 if silu else 0),
                                               _p(rg.entry_slot), rg.n, _stream()), "time_conv_step")
        return out
    _chk(L.pegainfer_time_conv_biased(_p(x), _dt(x), x.stride(0), _p(w), _dt(w), _p(in_bias), _p(out_bias), _p(state), slot_stride,
                                      _p(out), _dt(out), C, C, taps, (1 if residual else 0) | (2 if silu else 0), _p(rg.row_entry),
                                      _p(rg.entry_row0), _p(rg.entry_slot), x.shape[0], _stream()), "time_conv")
    _chk(L.pegainfer_time_conv_commit_biased(_p(x), _dt(x), x.stride(0), _p(in_bias), _dt(w), _p(state), slot_stride, C, taps,
                                             _p(rg.entry_row0), _p(rg.entry_slot), rg.n, _stream()), "time_conv_commit")
    return out


def group_rms_add(y, w, groups, eps, x=None, stack=None, coef=None):
    """r = (x or 0) + grouped_rms(y) * w  -> (r fp32, r in w's dtype, mix fp32 or None) with
    mix = sum_j coef[j] stack[j] + coef[-1] r over the len(coef) - 1 streams of `stack` (fp32 [n, rows, d])"""
    rows, d = y.shape
    r32 = torch.empty((rows, d), dtype=torch.float32, device=y.device)
    rb = torch.empty((rows, d), dtype=w.dtype, device=y.device)
    n_mix = 0 if coef is None else coef.numel()
    mix = torch.empty((rows, d), dtype=torch.float32, device=y.device) if n_mix else None
    _chk(ffi.lib().pegainfer_group_rms_add(_p(x), _p(y), _dt(y), _p(w), groups, float(eps), _p(r32), _p(rb), d, rows, _dt(w),
                                           _p(stack), 0 if stack is None else stack.stride(0), _p(coef), n_mix, _p(mix), None,
                                           _stream()), "group_rms_add")
    return r32, rb, mix


def clamp_glu_rows(gate_up, limit, alpha=1.702):
    rows, two_i = gate_up.shape
    out = torch.empty((rows, two_i // 2), dtype=gate_up.dtype, device=gate_up.device)
    _chk(ffi.lib().pegainfer_clamp_glu_rows(_p(gate_up), _p(out), two_i // 2, rows, float(limit), float(alpha), _dt(gate_up),
                                            _stream()), "clamp_glu_rows")
    return out


def route_topk(h, w_router, top, score="softmax", correction=None, n_groups=1, keep_groups=1):
    rows, d = h.shape
    e = torch.empty((rows, top), dtype=torch.int32, device=h.device)
    w = torch.empty((rows, top), dtype=torch.float32, device=h.device)
    _chk(ffi.lib().pegainfer_route_topk(_p(h), _p(w_router), _p(correction), _p(e), _p(w), d, w_router.shape[0], n_groups,
                                        keep_groups, top, rows, 1 if score == "softmax" else 0, _dt(h), _stream()), "route_topk")
    return e, w


def route_from_logits(logits_f32, top, score="softmax", correction=None, n_groups=1, keep_groups=1, dtype=torch.bfloat16):
    rows, E = logits_f32.shape
    e = torch.empty((rows, top), dtype=torch.int32, device=logits_f32.device)
    w = torch.empty((rows, top), dtype=torch.float32, device=logits_f32.device)
    _chk(ffi.lib().pegainfer_route_from_logits(_p(logits_f32), _p(correction), _p(e), _p(w), E, n_groups, keep_groups, top, rows,
                                               1 if score == "softmax" else 0, 0 if dtype == torch.bfloat16 else 1, _stream()),
         "route_from_logits")
    return e, w


def route_combine_add(y_pairs, weight, add, out_dtype):
    rows, top = weight.shape
    d = y_pairs.shape[1]
    out = torch.empty((rows, d), dtype=out_dtype, device=y_pairs.device)
    _chk(ffi.lib().pegainfer_route_combine_add(_p(y_pairs), _p(weight), _p(add), _p(out), d, top, rows, _dt(out), _stream()),
         "route_combine_add")
    return out


def delta_rule(qkv_f32, proj, b_off, a_off, A_log, dt_bias, state, heads, kv_heads, dim, vdim, rg):
    """qkv fp32 [rows, 2 kv dim + heads vdim] (after convolution and silu), proj [rows, *] with the beta / decay inputs;
    state fp32 [slots, heads, dim, vdim] is updated in place, and so are the q / k parts of qkv (made unit vectors);
    returns o fp32 [rows, heads * vdim]"""
    o = torch.empty((qkv_f32.shape[0], heads * vdim), dtype=torch.float32, device=proj.device)
    gates = torch.empty((qkv_f32.shape[0], 2 * heads), dtype=torch.float32, device=proj.device)
    _chk(ffi.lib().pegainfer_delta_rule(_p(qkv_f32), qkv_f32.stride(0), _p(proj), proj.stride(0), b_off, a_off, _p(A_log),
                                        _p(dt_bias), _p(gates), _p(state), state.stride(0), _p(o), heads, kv_heads, dim, vdim,
                                        qkv_f32.shape[0], _p(rg.entry_row0), _p(rg.entry_slot), rg.n, _dt(proj), _stream()),
         "delta_rule")
    return o


def gated_matrix_memory(proj, offs, i_bias, f_bias, cap, state, heads, dim, vdim, rg):
    """proj [rows, *] with q / k / v / i / f at the column offsets `offs`; state fp32 [slots, heads (dim vdim + dim + 1)] laid
    out [S of all heads | n of all heads | m of all heads]; returns o fp32 [rows, heads * vdim]"""
    o = torch.empty((proj.shape[0], heads * vdim), dtype=torch.float32, device=proj.device)
    _chk(ffi.lib().pegainfer_gated_matrix_memory(_p(proj), proj.stride(0), offs[0], offs[1], offs[2], offs[3], offs[4], _p(i_bias),
                                                 _p(f_bias), float(cap), _p(state), state.stride(0), _p(o), heads, dim, vdim,
                                                 _p(rg.entry_row0), _p(rg.entry_slot), rg.n, _dt(proj), _stream()),
         "gated_matrix_memory")
    return o


def head_rms_gate(o_f32, w, gate, gate_kind, factor, eps, heads, vdim, out=None):
    """gate: a [rows, heads * vdim] view (row stride free) in w's dtype; gate_kind "silu" | "sigmoid" """
    rows = o_f32.shape[0]
    out = torch.empty((rows, heads * vdim), dtype=w.dtype, device=w.device) if out is None else out
    _chk(ffi.lib().pegainfer_head_rms_gate(_p(o_f32), _p(w), int(w.numel() != vdim),
                                           _p(gate), gate.stride(0), 0 if gate_kind == "silu" else 1, float(factor), float(eps),
                                           _p(out), out.stride(0), heads, vdim, rows, _dt(w), _stream()), "head_rms_gate")
    return out


def attention_tiles(lens, per_group, device="cuda"):
    """row tiles of pegainfer_paged_attention for entries of `lens` rows: runs of token rows times runs of the per_group query
    heads of a key/value head, at most 16 rows each"""
    row0, ntok, qh0, nqh, at = [], [], [], [], 0
    for n in lens:
        if per_group <= 16:
            tpt = 16 // per_group
            for t0 in range(0, n, tpt):
                row0.append(at + t0); ntok.append(min(tpt, n - t0)); qh0.append(0); nqh.append(per_group)  # noqa: E702
        else:
            for t0 in range(n):
                for q0 in range(0, per_group, 16):
                    row0.append(at + t0); ntok.append(1); qh0.append(q0); nqh.append(min(16, per_group - q0))  # noqa: E702
        at += n
    return tuple(torch.tensor(v, dtype=torch.int32, device=device) for v in (row0, ntok, qh0, nqh))


def qk_norm_rope_paged(proj, offs, heads, kv_heads, dim, vdim, q_norm, k_norm, eps, inv_freq, rot_dims, rg, page_indptr,
                       page_ids, cache, page_stride, k_off, v_off, page_size):
    q = torch.empty((proj.shape[0], heads, dim), dtype=torch.float32, device=proj.device)
    _chk(ffi.lib().pegainfer_qk_norm_rope_paged(_p(proj), proj.stride(0), offs[0], offs[1], offs[2], heads, kv_heads, dim, vdim,
                                                _p(q_norm), _p(k_norm), float(eps), _p(inv_freq), rot_dims, _p(rg.positions),
                                                _p(rg.row_entry), _p(page_indptr), _p(page_ids), _p(cache), page_stride, k_off,
                                                v_off, page_size, _p(q), None, proj.shape[0], _dt(proj), _stream()), "qk_norm_rope_paged")
    return q


def paged_attention(q, cache, page_stride, k_off, v_off, page_size, rg, page_indptr, page_ids, kv_heads, vdim, scale, factor=1.0):
    T, H, dim = q.shape
    out = torch.empty((T, H * vdim), dtype=cache.dtype, device=q.device)
    t = attention_tiles(rg.lens, H // kv_heads, q.device)
    _chk(ffi.lib().pegainfer_paged_attention(_p(q), _p(cache), page_stride, k_off, v_off, page_size, _p(rg.positions),
                                             _p(rg.row_entry), _p(page_indptr), _p(page_ids), H, kv_heads, dim, vdim,
                                             float(scale), float(factor), _p(t[0]), _p(t[1]), _p(t[2]), _p(t[3]), t[0].numel(),
                                             _p(out), out.stride(0), _dt(cache), _stream()), "paged_attention")
    return out


# ---- one-number RMS gains, attention with options, channel decays, group-limited routing ----
def scalar_rms_add(x, gain, eps, y=None, bias=None, mult=1.0, add_rows=None, add_vec=None, norm=True):
    """r = x + mult (y + bias) + add_rows + add_vec (fp32), n = r / rms(r) * gain[0] (fp32) -> (r, n or None);
    x fp32 [rows, d]; y / bias / add_vec / gain in the storage type of gain"""
    rows, d = x.shape
    r = torch.empty_like(x)
    n = torch.empty_like(x) if norm else None
    _chk(ffi.lib().pegainfer_scalar_rms_add(_p(x), _p(y), _dt(y) if y is not None else _dt(gain), _p(bias), float(mult), _p(add_rows),
                                            _p(add_vec), _p(r), _p(gain) if norm else None, float(eps), _p(n), d, rows, _dt(gain),
                                            _stream()), "scalar_rms_add")
    return r, n


def qk_prep_paged(proj, offs, heads, kv_heads, dim, vdim, rg, page_indptr, page_ids, cache, page_stride, k_off, v_off, page_size,
                  q_norm=None, k_norm=None, eps=0.0, q_bias=None, k_bias=None, v_bias=None, qt_coef=0.0, qt_every=0, inv_freq=None,
                  rot_dims=0):
    """queries -> fp32 [rows, heads, dim]; keys and values -> the cache entry of (request, position).  dim counts ALL values of
    a query / key head (both maps of a two-map attention)"""
    q = torch.empty((proj.shape[0], heads, dim), dtype=torch.float32, device=proj.device)
    _chk(ffi.lib().pegainfer_qk_prep_paged(_p(proj), proj.stride(0), offs[0], offs[1], offs[2], heads, kv_heads, dim, vdim, _p(q_norm),
                                           _p(k_norm), float(eps), _p(q_bias), _p(k_bias), _p(v_bias), float(qt_coef), int(qt_every),
                                           _p(inv_freq), rot_dims, _p(rg.positions), _p(rg.row_entry), _p(page_indptr), _p(page_ids),
                                           _p(cache), page_stride, k_off, v_off, page_size, _p(q), None, proj.shape[0], _dt(proj),
                                           _stream()), "qk_prep_paged")
    return q


def paged_attention_ex(q, cache, page_stride, k_off, v_off, page_size, rg, page_indptr, page_ids, kv_heads, vdim, scale, factor=1.0,
                       maps=1, lam=0.0, block=0, sink=None, head_norm=False, norm_eps=0.0, n_split=1, plain=False):
    """q fp32 [rows, heads, maps * dim]; n_split > 1: the keys of every tile dealt to that many workgroups, then merged; a bf16 cache runs on
    the matrix cores unless plain"""
    T, H, qd = q.shape
    out = torch.empty((T, H * vdim), dtype=cache.dtype, device=q.device)
    t = attention_tiles(rg.lens, H // kv_heads, q.device)
    ws = None
    if n_split > 1:
        ws = torch.empty(ffi.lib().pegainfer_paged_attention_workspace(t[0].numel(), kv_heads, vdim, maps, n_split),
                         dtype=torch.float32, device=q.device)
    _chk(ffi.lib().pegainfer_paged_attention_ex(_p(q), _p(cache), page_stride, k_off, v_off, page_size, _p(rg.positions),
                                                _p(rg.row_entry), _p(page_indptr), _p(page_ids), H, kv_heads, qd // maps, vdim,
                                                float(scale), float(factor), _p(t[0]), _p(t[1]), _p(t[2]), _p(t[3]), t[0].numel(),
                                                _p(out), out.stride(0), maps, float(lam), int(block), _p(sink), int(bool(head_norm)),
                                                float(norm_eps), int(n_split), _p(ws), int(bool(plain)), _dt(cache), _stream()), "paged_attention_ex")
    return out


def delta_rule_channel(qkv_f32, proj, b_off, a_f32, A_log, dt_bias, state, heads, kv_heads, dim, vdim, rg):
    """the gated delta rule with a decay per (head, key channel); a_f32 [rows, heads * dim] the decay inputs; otherwise as
    delta_rule"""
    o = torch.empty((qkv_f32.shape[0], heads * vdim), dtype=torch.float32, device=proj.device)
    gates = torch.empty((qkv_f32.shape[0], heads * dim + heads), dtype=torch.float32, device=proj.device)
    _chk(ffi.lib().pegainfer_delta_rule_channel(_p(qkv_f32), qkv_f32.stride(0), _p(proj), proj.stride(0), b_off, _p(a_f32),
                                                a_f32.stride(0), _p(A_log), _p(dt_bias), _p(gates), _p(state), state.stride(0), _p(o),
                                                heads, kv_heads, dim, vdim, qkv_f32.shape[0], _p(rg.entry_row0), _p(rg.entry_slot),
                                                rg.n, _dt(proj), _stream()), "delta_rule_channel")
    return o


def route_from_logits_ex(logits_f32, experts, top, n_groups=1, keep_groups=1, score="softmax", group="max", renorm=True,
                         dtype=torch.bfloat16):
    """logits fp32 [rows, >= experts] (columns beyond `experts` are not read)"""
    rows = logits_f32.shape[0]
    e = torch.empty((rows, top), dtype=torch.int32, device=logits_f32.device)
    w = torch.empty((rows, top), dtype=torch.float32, device=logits_f32.device)
    _chk(ffi.lib().pegainfer_route_from_logits_ex(_p(logits_f32), logits_f32.stride(0), None, _p(e), _p(w), experts, n_groups,
                                                  keep_groups, top, rows, 1 if score == "softmax" else 0, 1 if group == "max" else 0,
                                                  int(bool(renorm)), 0 if dtype == torch.bfloat16 else 1, _stream()),
         "route_from_logits_ex")
    return e, w


def route_combine_gated(y_pairs, weight, add, add_gate_f32, out_dtype):
    """sum_c weight[row, c] y_pairs[row * top + c] + sigmoid(add_gate[row]) * add[row]; add_gate: an fp32 [rows] view (stride free)"""
    rows, top = weight.shape
    d = y_pairs.shape[1]
    out = torch.empty((rows, d), dtype=out_dtype, device=y_pairs.device)
    _chk(ffi.lib().pegainfer_route_combine_gated(_p(y_pairs), _p(weight), _p(add), _p(add_gate_f32),
                                                 0 if add_gate_f32 is None else add_gate_f32.stride(0), _p(out), d, top, rows,
                                                 _dt(out), _stream()), "route_combine_gated")
    return out


# ---- several sublayers behind one norm, attention with shaped scores and gates, state-space scan ----
class SumTerm(ctypes.Structure):
    _fields_ = [("y", ctypes.c_void_p), ("y_row_stride", ctypes.c_int64), ("bias", ctypes.c_void_p), ("norm_w", ctypes.c_void_p),
                ("factor", ctypes.c_float)]


def terms_rms_add(x, terms, gain=None, eps=1e-6, out_dtype=None):
    """r = x + sum_t factor_t * (norm_w_t ? rms_norm(y_t + bias_t) * norm_w_t : y_t + bias_t);  n = rms_norm(r) * gain.
    x fp32 [rows, d] or None; terms: up to three (y, bias or None, norm_w or None, factor); -> (r fp32, n in out_dtype or None)"""
    ref = terms[0][0] if terms else gain
    rows, d = (x.shape if x is not None else terms[0][0].shape)
    arr = (SumTerm * max(1, len(terms)))()
    for i, (y, bias, nw, f) in enumerate(terms):
        arr[i] = SumTerm(_p(y), y.stride(0), _p(bias), _p(nw), float(f))
    r = torch.empty((rows, d), dtype=torch.float32, device=ref.device)
    n = torch.empty((rows, d), dtype=out_dtype or ref.dtype, device=ref.device) if gain is not None else None
    _chk(ffi.lib().pegainfer_terms_rms_add(_p(x), ctypes.addressof(arr) if terms else None, len(terms), _p(r), _p(gain), float(eps), _p(n),
                                           _dt(n) if n is not None else 0, d, rows, _dt(ref), _stream()), "terms_rms_add")
    return r, n


def glu_rows(gate, up, act="relu"):
    """act(gate) * up; gate and up are [rows, I] views of rows with one stride (column ranges of a wider matrix)"""
    rows, I = gate.shape
    assert gate.stride(0) == up.stride(0)
    out = torch.empty((rows, I), dtype=gate.dtype, device=gate.device)
    _chk(ffi.lib().pegainfer_glu_rows(_p(gate), _p(up), gate.stride(0), _p(out), I, I, rows, {"silu": 0, "relu": 1, "gelu_tanh": 2}[act],
                                      _dt(gate), _stream()), "glu_rows")
    return out


def softcap_rows(x_f32, cap):
    out = torch.empty_like(x_f32)
    _chk(ffi.lib().pegainfer_softcap_rows(_p(x_f32), _p(out), x_f32.numel(), float(cap), _stream()), "softcap_rows")
    return out


def head_gate_rms(o_f32, w, gate, gate_kind, eps, heads, vdim, gate_first=True, factor=1.0):
    """head_rms_gate with the order chosen: gate_first norms the gated values"""
    rows = o_f32.shape[0]
    out = torch.empty((rows, heads * vdim), dtype=w.dtype, device=w.device)
    _chk(ffi.lib().pegainfer_head_gate_rms(_p(o_f32), _p(w), int(w.numel() != vdim), _p(gate), gate.stride(0),
                                           0 if gate_kind == "silu" else 1, int(bool(gate_first)), float(factor), float(eps), _p(out),
                                           out.stride(0), heads, vdim, rows, _dt(w), _stream()), "head_gate_rms")
    return out


QKNORM = {"head_weight": 0, "head_unit_after": 1, "all_weight": 2}


def qk_prep_paged_form(proj, offs, heads, kv_heads, dim, vdim, rg, page_indptr, page_ids, cache, page_stride, k_off, v_off, page_size,
                       q_norm=None, k_norm=None, norm_kind="head_weight", eps=0.0, q_bias=None, k_bias=None, v_bias=None, inv_freq=None,
                       rot_dims=0, halves=False):
    """proj: rows of the cache's type or fp32 (what a convolution left); queries -> fp32 [rows, heads, dim]; keys and values -> the
    cache entry of (request, position)"""
    q = torch.empty((proj.shape[0], heads, dim), dtype=torch.float32, device=proj.device)
    _chk(ffi.lib().pegainfer_qk_prep_paged_form(_p(proj), _dt(proj), proj.stride(0), offs[0], offs[1], offs[2], heads, kv_heads, dim, vdim,
                                                _p(q_norm), _p(k_norm), QKNORM[norm_kind], float(eps), _p(q_bias), _p(k_bias), _p(v_bias),
                                                0.0, 0, _p(inv_freq), rot_dims, int(bool(halves)), _p(rg.positions), _p(rg.row_entry),
                                                _p(page_indptr), _p(page_ids), _p(cache), page_stride, k_off, v_off, page_size, _p(q), None,
                                                proj.shape[0], _dt(cache), _stream()), "qk_prep_paged_form")
    return q


def paged_attention_masked(q, cache, page_stride, k_off, v_off, page_size, rg, page_indptr, page_ids, kv_heads, vdim, scale, softcap=0.0,
                           window=0, keep_first=0, dist_bias=None, gate=None, gate_per_head=False, block=0, sink=None, n_split=1,
                           plain=False):
    """q fp32 [rows, heads, dim]; dist_bias fp32 [n_dist, heads]; gate: a view of rows in the cache's type ([rows, heads * vdim] or
    [rows, heads])"""
    T, H, dim = q.shape
    out = torch.empty((T, H * vdim), dtype=cache.dtype, device=q.device)
    t = attention_tiles(rg.lens, H // kv_heads, q.device)
    ws = None
    if n_split > 1:
        ws = torch.empty(ffi.lib().pegainfer_paged_attention_workspace(t[0].numel(), kv_heads, vdim, 1, n_split), dtype=torch.float32,
                         device=q.device)
    _chk(ffi.lib().pegainfer_paged_attention_masked(_p(q), _p(cache), page_stride, k_off, v_off, page_size, _p(rg.positions),
                                                    _p(rg.row_entry), _p(page_indptr), _p(page_ids), H, kv_heads, dim, vdim, float(scale),
                                                    1.0, _p(t[0]), _p(t[1]), _p(t[2]), _p(t[3]), t[0].numel(), _p(out), out.stride(0), 1,
                                                    0.0, int(block), _p(sink), 0, 0.0, float(softcap), int(window), int(keep_first),
                                                    _p(dist_bias), 0 if dist_bias is None else dist_bias.shape[0], _p(gate),
                                                    0 if gate is None else gate.stride(0),
                                                    0 if gate is None else (2 if gate_per_head else 1), int(n_split), _p(ws),
                                                    int(bool(plain)), _dt(cache), _stream()), "paged_attention_masked")
    return out


def ssd_scan(xbc_f32, proj, dt_off, A_log, dt_bias, D, state, heads, groups, n_state, vdim, rg):
    """selective state-space scan; xbc fp32 [rows, heads * vdim + 2 * groups * n_state]; proj rows (storage type) hold the raw step
    sizes at dt_off; state fp32 [slots, heads * n_state * vdim] is read and moved on; -> y fp32 [rows, heads * vdim]"""
    y = torch.empty((xbc_f32.shape[0], heads * vdim), dtype=torch.float32, device=proj.device)
    _chk(ffi.lib().pegainfer_ssd_scan(_p(xbc_f32), xbc_f32.stride(0), _p(proj), proj.stride(0), dt_off, _p(A_log), _p(dt_bias), _p(D),
                                      _p(state), state.stride(0), _p(y), heads, groups, n_state, vdim, _p(rg.entry_row0), _p(rg.entry_slot),
                                      rg.n, _dt(proj), _stream()), "ssd_scan")
    return y
