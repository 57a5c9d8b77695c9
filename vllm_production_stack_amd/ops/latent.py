"""Ops of decoders with a 32-bit residual stream, latent attention and group-limited sigmoid
routing (``csrc/kernels/latent.hip``).  Device tensors run the HIP kernels in bf16 or fp32
activations; CPU tensors run the PyTorch definitions of ``reference.py``.

The latent KV pool is ``[pages, page_elems]``: a page holds, for every caching layer, PAGE entries
of ``rank + rot`` values (RMS-normed latent | rotated shared key part) starting ``offset`` elements
into the page, so a page's whole depth stays one contiguous run.
"""

from __future__ import annotations

from ctypes import c_float, c_int, c_long, c_void_p

import torch

from . import reference
from .reference import PAGE

_DT = {torch.bfloat16: 0, torch.float32: 1}


def _ops():
    from .. import ops

    return ops


def _dt(*ts) -> int:
    d = None
    for t in ts:
        if t is None:
            continue
        if not t.is_cuda or t.dtype not in _DT:
            raise TypeError("latent kernels take bf16 or fp32 device tensors")
        if d is not None and _DT[t.dtype] != d:
            raise TypeError("latent kernels: mixed activation dtypes")
        d = _DT[t.dtype]
    return d


def _f32(*ts):
    for t in ts:
        if t is not None and (t.dtype != torch.float32 or not t.is_contiguous()):
            raise TypeError("expected a contiguous fp32 tensor")


def _rows(t) -> bool:  # a 2-D view whose rows are contiguous runs
    return t.dim() == 2 and t.stride(1) == 1


def embed_scale(ids, embed, scale: float):
    """fp32 [T, width] = embed[ids] * scale."""
    if not embed.is_cuda:
        return reference.embed_scale(ids, embed, scale)
    o = _ops()
    assert ids.dtype == torch.int64 and embed.is_contiguous()
    out = torch.empty((ids.shape[0], embed.shape[1]), dtype=torch.float32, device=embed.device)
    o._check(o._kernels().vpsa_embed_scale(o._p(ids), o._p(embed), o._p(out), c_int(ids.shape[0]),
                                           c_int(embed.shape[1]), c_float(scale), c_int(_dt(embed)), o._stream()),
             "embed_scale")
    return out


def add_rms_norm(residual, delta, weight, eps: float, out_dtype, want_out: bool = True):
    """residual (fp32, in place) += delta; returns rmsnorm(residual) * weight in ``out_dtype``."""
    if not residual.is_cuda:
        return reference.add_rms_norm(residual, delta, weight, eps, out_dtype, want_out)
    o = _ops()
    _f32(residual, weight)
    t, n = residual.shape
    assert delta is None or (_rows(delta) and delta.shape == residual.shape and delta.dtype == out_dtype)
    y = torch.empty((t, n), dtype=out_dtype, device=residual.device) if want_out else None
    if y is None and delta is None:
        return None
    o._check(o._kernels().vpsa_add_rmsnorm(o._p(residual), o._p(delta), c_long(delta.stride(0) if delta is not None else 0),
                                           o._p(weight), o._p(y), c_long(n), c_int(t), c_int(n), c_float(eps),
                                           c_int(_DT[out_dtype]), o._stream()), "add_rms_norm")
    return y


def gated_add_rms_norm(residual, deltas, gate, gate_bias, weight, eps: float, out_dtype, *, extra=None, extra_vec=None,
                       want_out: bool = True):
    """A gated residual in front of a pre-norm.  residual (fp32, in place) +=
    sigmoid(gate + gate_bias) * sum_i c_i n_i(d_i) + extra + extra_vec over ``deltas``, up to two (tensor, norm weight
    or None, factor) triples: n(d) = rmsnorm(d) * norm weight where one is given, d itself otherwise.  The first
    delta is in the activation dtype or fp32 (a mixture's sum), the second in the activation dtype; ``gate`` is a
    [T, n] view (of a wider projection, say) in the activation dtype or None (no gate), ``gate_bias`` fp32 [n] or
    None; ``extra`` fp32 [T, n] (a stream that re-enters) and ``extra_vec`` fp32 [n] are added ungated.
    Returns rmsnorm(residual) * weight in ``out_dtype`` (None without ``want_out``)."""
    deltas = list(deltas)
    assert len(deltas) <= 2
    if not residual.is_cuda:
        return reference.gated_add_rms_norm(residual, deltas, gate, gate_bias, extra, extra_vec, weight, eps, out_dtype,
                                            want_out)
    o = _ops()
    _f32(residual, weight, gate_bias, extra, extra_vec)
    t, n = residual.shape
    if t == 0:
        return torch.empty((0, n), dtype=out_dtype, device=residual.device) if want_out else None
    ds = deltas + [(None, None, 0.0)] * (2 - len(deltas))
    (d1, w1, c1), (d2, w2, c2) = ds
    _f32(w1, w2)
    assert d1 is None or (_rows(d1) and d1.shape == (t, n) and d1.dtype in (out_dtype, torch.float32))
    assert d2 is None or (_rows(d2) and d2.shape == (t, n) and d2.dtype == out_dtype)
    assert gate is None or (_rows(gate) and gate.shape == (t, n) and gate.dtype == out_dtype)
    assert extra is None or (extra.is_contiguous() and extra.shape == (t, n))
    y = torch.empty((t, n), dtype=out_dtype, device=residual.device) if want_out else None
    o._check(o._kernels().vpsa_gated_add_rmsnorm(
        o._p(residual), o._p(d1), c_long(d1.stride(0) if d1 is not None else 0),
        c_int(1 if (d1 is not None and d1.dtype == torch.float32) else 0), o._p(w1), c_float(c1), o._p(d2),
        c_long(d2.stride(0) if d2 is not None else 0), o._p(w2), c_float(c2), o._p(gate),
        c_long(gate.stride(0) if gate is not None else 0), o._p(gate_bias), o._p(extra), o._p(extra_vec), o._p(weight),
        o._p(y), c_int(t), c_int(n), c_float(eps), c_int(_DT[out_dtype]), o._stream()), "gated_add_rms_norm")
    return y


def rms_norm_add(residual, delta, weight, eps: float, out_dtype, want_out: bool = True):
    """A norm on a sublayer's output: residual (fp32, in place) += rmsnorm(delta) * weight.  ``delta`` is in
    ``out_dtype`` or fp32 (a mixture's sum).  Returns the new residual rounded to ``out_dtype``: the next
    sublayer's input, for designs whose sublayers read the stream itself."""
    if not residual.is_cuda:
        return reference.rms_norm_add(residual, delta, weight, eps, out_dtype, want_out)
    o = _ops()
    _f32(residual, weight)
    t, n = residual.shape
    assert _rows(delta) and delta.shape == residual.shape and delta.dtype in (out_dtype, torch.float32)
    y = torch.empty((t, n), dtype=out_dtype, device=residual.device) if want_out else None
    o._check(o._kernels().vpsa_rmsnorm_add(o._p(residual), o._p(delta), c_long(delta.stride(0)),
                                           c_int(1 if delta.dtype == torch.float32 else 0), o._p(weight), o._p(y), c_int(t),
                                           c_int(n), c_float(eps), c_int(_DT[out_dtype]), o._stream()), "rms_norm_add")
    return y


def rms_norm_rows(x, weight, eps: float):
    """rmsnorm over the columns of a 2-D view (a column range of a wider projection output)."""
    if not x.is_cuda:
        return reference.rms_norm_rows(x, weight, eps)
    o = _ops()
    _f32(weight)
    assert _rows(x) and weight.numel() == x.shape[1]
    y = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    o._check(o._kernels().vpsa_rmsnorm_rows(o._p(x), c_long(x.stride(0)), o._p(weight), o._p(y), c_long(x.shape[1]),
                                            c_int(x.shape[0]), c_int(x.shape[1]), c_float(eps), c_int(_dt(x)),
                                            o._stream()), "rms_norm_rows")
    return y


def _layer_base(pool, offset: int, entry: int):
    assert pool.dim() == 2 and pool.stride(1) == 1 and offset + PAGE * entry <= pool.shape[1]
    return c_void_p(pool.data_ptr() + offset * pool.element_size())


def latent_kv_write(x, weight, positions, slots, cos_sin, pool, offset: int, rank: int, rot: int, rot_dims: int,
                    eps: float):
    """Rows of x [T, rank + rot] (a view) -> cache entries: RMS-normed latent | rotated key part."""
    if not x.is_cuda:
        return reference.latent_kv_write(x, weight, positions, slots, cos_sin, pool, offset, rank, rot, rot_dims, eps)
    o = _ops()
    _f32(weight, cos_sin)
    assert _rows(x) and x.shape[1] == rank + rot and positions.dtype == torch.int32 and slots.dtype == torch.int64
    assert cos_sin.shape[1] == rot_dims and weight.numel() == rank
    o._check(o._kernels().vpsa_latent_kv_write(o._p(x), c_long(x.stride(0)), o._p(weight), o._p(positions), o._p(slots),
                                               o._p(cos_sin), _layer_base(pool, offset, rank + rot),
                                               c_long(pool.stride(0)), c_int(x.shape[0]), c_int(rank), c_int(rot),
                                               c_int(rot_dims), c_float(eps), c_int(_dt(x, pool)), o._stream()),
             "latent_kv_write")


def rope_pairs(q, positions, cos_sin, col0: int, rot_dims: int):
    """Interleaved-pair rotary embedding of columns [col0, col0 + rot_dims) of every head of
    q [T, heads, d], in place.  cos_sin [max_pos, rot_dims] = cos | sin of the rot_dims / 2 angles."""
    if not q.is_cuda:
        return reference.rope_pairs(q, positions, cos_sin, col0, rot_dims)
    o = _ops()
    _f32(cos_sin)
    assert q.dim() == 3 and q.stride(2) == 1 and positions.dtype == torch.int32 and cos_sin.shape[1] == rot_dims
    assert col0 + rot_dims <= q.shape[2]
    o._check(o._kernels().vpsa_rope_pairs(o._p(q), c_long(q.stride(0)), c_long(q.stride(1)), o._p(positions),
                                          o._p(cos_sin), c_int(q.shape[0]), c_int(q.shape[1]), c_int(col0),
                                          c_int(rot_dims), c_int(_dt(q)), o._stream()), "rope_pairs")


LATENT_TILE_SLOTS = 64  # (token, head) pairs of one tile of the matrix-core kernel
LATENT_MFMA = True      # False: every call takes the plain kernel (A/B runs, tests of the plain kernel)


def latent_mfma_supported(rank: int, rot: int) -> bool:
    return bool(_ops()._kernels().vpsa_latent_mfma_supported(c_int(rank), c_int(rot)))


def build_latent_tiles(q_lens, ctx_lens, heads: int):
    """Work list of the matrix-core kernel for the prefill part of a batch: int32 rows (sequence, first
    query row, tokens, position of the first token, first head, heads per token), a tile holding up to
    64 (token, head) pairs of consecutive tokens of one sequence.  Longest contexts first."""
    import numpy as np

    per_tok = max(1, LATENT_TILE_SLOTS // heads)
    runs = [(h0, min(LATENT_TILE_SLOTS, heads - h0)) for h0 in range(0, heads, LATENT_TILE_SLOTS)]
    parts = []
    row = 0
    for i, (n, ctx) in enumerate(zip(q_lens, ctx_lens)):
        k = np.arange(0, n, per_tok, dtype=np.int64)
        for h0, hc in runs:
            parts.append(np.stack([np.full_like(k, i), row + k, np.minimum(per_tok, n - k), ctx - n + k,
                                   np.full_like(k, h0), np.full_like(k, hc)], axis=1))
        row += n
    if not parts:
        return np.zeros((0, 6), dtype=np.int32)
    tiles = np.concatenate(parts)
    order = np.argsort(-(tiles[:, 3] + tiles[:, 2]), kind="stable")
    return tiles[order].astype(np.int32)


def _mfma_ok(q_lat, q_rot, pool, out) -> bool:
    if not (LATENT_MFMA and q_lat.dtype == torch.bfloat16 and pool.dtype == torch.bfloat16):
        return False
    rank, rot = q_lat.shape[2], q_rot.shape[2]
    if not latent_mfma_supported(rank, rot):
        return False
    return (q_lat.data_ptr() % 16 == 0 and q_rot.data_ptr() % 16 == 0 and out.data_ptr() % 8 == 0
            and all(s % 8 == 0 for s in (q_lat.stride(0), q_lat.stride(1), q_rot.stride(0), q_rot.stride(1)))
            and out.stride(0) % 4 == 0 and out.stride(1) % 4 == 0 and pool.stride(0) % 8 == 0)


def latent_tile_kernel_takes(q_lat, q_rot, pool, out) -> bool:
    """Would ``latent_attention`` run these operands on the matrix-core tile kernel?"""
    return bool(q_lat.is_cuda and _mfma_ok(q_lat, q_rot, pool, out))


def latent_attention(q_lat, q_rot, pool, offset: int, block_tables, row_seq, positions, sink, scale: float, out=None,
                     tiles=None, splits: int = 1):
    """Causal attention of query rows over their sequences' cache entries, in latent space.

    q_lat [T, heads, rank] and q_rot [T, heads, rot] (views with contiguous last dim); row ``i``
    belongs to sequence ``row_seq[i]`` (``None``: row i is sequence i, a decode batch) whose pages are
    ``block_tables[seq]`` and sees entries 0 .. positions[i].  ``sink`` [heads] fp32 or None: a logit
    that joins the softmax denominator only.  Returns [T, heads, rank].

    bf16 entries of a shape the matrix-core kernel tiles take it: decode batches as they are (with
    ``splits`` key ranges per row, merged by a second launch), prefill rows when ``tiles`` (the device
    copy of ``build_latent_tiles``) describes them.  Everything else takes the plain kernel."""
    t, heads, rank = q_lat.shape
    if out is None:
        out = torch.empty((t, heads, rank), dtype=q_lat.dtype, device=q_lat.device)
    if t == 0:
        return out
    if not q_lat.is_cuda:
        return reference.latent_attention(q_lat, q_rot, pool, offset, block_tables, row_seq, positions, sink, scale, out)
    o = _ops()
    rot = q_rot.shape[2]
    _f32(sink)
    assert q_lat.stride(2) == 1 and q_rot.stride(2) == 1 and out.stride(2) == 1 and q_rot.shape[:2] == (t, heads)
    assert block_tables.dtype == torch.int32 and block_tables.stride(1) == 1 and positions.dtype == torch.int32
    assert row_seq is None or (row_seq.dtype == torch.int32 and row_seq.numel() == t)
    dt = _dt(q_lat, q_rot, pool, out)
    if (tiles is not None or row_seq is None) and _mfma_ok(q_lat, q_rot, pool, out):
        if tiles is not None:
            assert tiles.dtype == torch.int32 and tiles.is_contiguous() and tiles.shape[1] == 6
            n_tiles, splits = tiles.shape[0], 1
        else:
            n_tiles = t * ((heads + LATENT_TILE_SLOTS - 1) // LATENT_TILE_SLOTS)
        ws_o = ws_ml = None
        if splits > 1:
            ws_o = torch.empty((n_tiles * splits * LATENT_TILE_SLOTS * rank,), dtype=torch.float32, device=out.device)
            ws_ml = torch.empty((n_tiles * splits * LATENT_TILE_SLOTS * 2,), dtype=torch.float32, device=out.device)
        o._check(o._kernels().vpsa_latent_attention_mfma(
            o._p(q_lat), c_long(q_lat.stride(0)), c_long(q_lat.stride(1)), o._p(q_rot), c_long(q_rot.stride(0)),
            c_long(q_rot.stride(1)), _layer_base(pool, offset, rank + rot), c_long(pool.stride(0)), o._p(block_tables),
            c_int(block_tables.stride(0)), o._p(tiles), o._p(positions), c_int(n_tiles), c_int(heads), o._p(sink),
            o._p(out), c_long(out.stride(0)), c_long(out.stride(1)), c_int(rank), c_int(rot), c_float(scale),
            c_int(splits), o._p(ws_o), o._p(ws_ml), o._stream()), "latent_attention_mfma")
        return out
    o._check(o._kernels().vpsa_latent_attention(
        o._p(q_lat), c_long(q_lat.stride(0)), c_long(q_lat.stride(1)), o._p(q_rot), c_long(q_rot.stride(0)),
        c_long(q_rot.stride(1)), _layer_base(pool, offset, rank + rot), c_long(pool.stride(0)), o._p(block_tables),
        c_int(block_tables.stride(0)), o._p(row_seq), o._p(positions), o._p(sink), o._p(out), c_long(out.stride(0)),
        c_long(out.stride(1)), c_int(t), c_int(heads), c_int(rank), c_int(rot), c_float(scale),
        c_int(dt), o._stream()), "latent_attention")
    return out


def sigmoid_gate(y, g):
    """y [T, heads, v] (contiguous, in place) *= sigmoid(g [T, heads]) (a view of a wider projection)."""
    if not y.is_cuda:
        return reference.sigmoid_gate(y, g)
    o = _ops()
    assert y.is_contiguous() and g.stride(1) == 1 and g.shape == y.shape[:2]
    o._check(o._kernels().vpsa_sigmoid_gate(o._p(y), o._p(g), c_long(g.stride(0)), c_int(y.shape[0]), c_int(y.shape[1]),
                                            c_int(y.shape[2]), c_int(_dt(y, g)), o._stream()), "sigmoid_gate")
    return y


def relu_sq(x):
    if not x.is_cuda:
        return reference.relu_sq(x)
    o = _ops()
    assert x.is_contiguous()
    y = torch.empty_like(x)
    o._check(o._kernels().vpsa_relu_sq(o._p(x), o._p(y), c_long(x.numel()), c_int(_dt(x)), o._stream()), "relu_sq")
    return y


def glu_clamp(x, limit: float, alpha: float = 1.702, up_bias: float = 1.0):
    """x [rows, 2 I] = gate | up  ->  min(g, limit) * sigmoid(alpha min(g, limit)) * (clamp(u, +-limit) + up_bias)."""
    if not x.is_cuda:
        return reference.glu_clamp(x, limit, alpha, up_bias)
    o = _ops()
    assert _rows(x) and x.shape[1] % 2 == 0
    inter = x.shape[1] // 2
    y = torch.empty((x.shape[0], inter), dtype=x.dtype, device=x.device)
    o._check(o._kernels().vpsa_glu_clamp(o._p(x), c_long(x.stride(0)), o._p(y), c_int(x.shape[0]), c_int(inter),
                                         c_float(limit), c_float(alpha), c_float(up_bias), c_int(_dt(x)), o._stream()),
             "glu_clamp")
    return y


GLU_ACTS = {"silu": 0, "gelu_tanh": 1}


def glu_act(x, act: str):
    """x [rows, 2 I] = gate | up  ->  act(gate) * up, act = silu or the tanh form of gelu."""
    if not x.is_cuda:
        return reference.glu_act(x, act)
    o = _ops()
    assert _rows(x) and x.shape[1] % 2 == 0
    inter = x.shape[1] // 2
    y = torch.empty((x.shape[0], inter), dtype=x.dtype, device=x.device)
    o._check(o._kernels().vpsa_glu_act(o._p(x), c_long(x.stride(0)), o._p(y), c_int(x.shape[0]), c_int(inter),
                                       c_int(GLU_ACTS[act]), c_int(_dt(x)), o._stream()), "glu_act")
    return y


def gate_up_act(x, w_gate_up, act: str, packed=None):
    """act(x @ Wg.T) * (x @ Wu.T) for ``w_gate_up = [Wg; Wu]``.  silu in bf16 is the fused path of the other
    decoders (``gate_up_silu``); the tanh form of gelu runs in the prefill GEMM's epilogue when that kernel
    takes the shape; everything else is the projection and the activation kernel."""
    o = _ops()
    if act == "silu" and x.is_cuda and x.dtype == torch.bfloat16:
        return o.gate_up_silu(x, w_gate_up, packed)
    rows = o.tile_rows(x, w_gate_up, True) if (x.is_cuda and act == "gelu_tanh" and o.TILE_GELU_GLU) else 0
    if rows:
        out = torch.empty((x.shape[0], w_gate_up.shape[0] // 2), dtype=x.dtype, device=x.device)
        o.tile_gemm(x[:rows], w_gate_up, gelu_mul=True, out=out[:rows])
        if rows < x.shape[0]:
            out[rows:] = glu_act(o.linear(x[rows:], w_gate_up), act)
        return out
    return glu_act(o.linear(x, w_gate_up), act)


def route_softmax(logits, n: int, experts: int, groups: int, keep: int, topk: int, bias=None, route_scale: float = 1.0,
                  park_in_bucket: bool = True):
    """Router logits fp32 [T, >= n] -> (weights fp32 [T, topk], ids int32 [T, topk], gate fp32 [T] or None).
    Scores are the softmax over all ``n`` outputs; an output is chosen by score + ``bias`` (fp32 [n]) and
    weighted by the score alone (times ``route_scale``, not renormalised).  Outputs form ``groups`` equal
    runs of neighbours, a group scores its largest biased score, and only outputs of the ``keep`` best
    groups can be chosen.  Outputs ``experts .. n`` are identity experts (their output is the token itself):
    a chosen one leaves the pair list (weight 0, id ``experts`` with ``park_in_bucket``, a bucket that sorting
    kernels put behind the last expert and no product visits, else id 0) and its score is added to ``gate``."""
    if not logits.is_cuda:
        return reference.route_softmax(logits, n, experts, groups, keep, topk, bias, route_scale, park_in_bucket)
    o = _ops()
    _f32(logits, bias)
    t = logits.shape[0]
    w = torch.empty((t, topk), dtype=torch.float32, device=logits.device)
    ids = torch.empty((t, topk), dtype=torch.int32, device=logits.device)
    gate = torch.empty((t,), dtype=torch.float32, device=logits.device) if experts < n else None
    o._check(o._kernels().vpsa_route_softmax(o._p(logits), c_int(logits.shape[1]), o._p(bias), o._p(w), o._p(ids),
                                             o._p(gate), c_int(t), c_int(n), c_int(experts), c_int(groups), c_int(keep),
                                             c_int(topk), c_float(route_scale), c_int(experts if park_in_bucket else 0),
                                             o._stream()), "route_softmax")
    return w, ids, gate


def group_topk(logits, experts: int, groups: int, keep: int, topk: int, route_scale: float, extra: bool = False,
               normalize: bool = False):
    """Router logits fp32 [T, >= experts (+1)] -> (weights fp32 [T, topk], ids int32 [T, topk], extra).

    Scores are sigmoids; experts form ``groups`` equal runs of neighbours, a group scores the sum of
    its two largest scores, and only experts of the ``keep`` best groups can be chosen; weights are
    the chosen scores (``normalize``: divided by their sum + 1e-20) times ``route_scale``.  ``extra``: column ``experts`` is one more logit per
    token, returned as its sigmoid (a shared unit's gate)."""
    if not logits.is_cuda:
        return reference.group_topk(logits, experts, groups, keep, topk, route_scale, extra, normalize)
    o = _ops()
    _f32(logits)
    t = logits.shape[0]
    w = torch.empty((t, topk), dtype=torch.float32, device=logits.device)
    ids = torch.empty((t, topk), dtype=torch.int32, device=logits.device)
    ex = torch.empty((t,), dtype=torch.float32, device=logits.device) if extra else None
    o._check(o._kernels().vpsa_group_topk(o._p(logits), c_int(logits.shape[1]), o._p(w), o._p(ids), o._p(ex), c_int(t),
                                          c_int(experts), c_int(groups), c_int(keep), c_int(topk),
                                          c_float(route_scale), c_int(1 if normalize else 0), o._stream()), "group_topk")
    return w, ids, ex


def gather_rows(x, idx):
    if not x.is_cuda:
        return x[idx.long()]
    o = _ops()
    assert x.is_contiguous() and idx.dtype == torch.int32
    xs = torch.empty((idx.numel(), x.shape[1]), dtype=x.dtype, device=x.device)
    o._check(o._kernels().vpsa_gather_rows(o._p(x), o._p(idx), o._p(xs), c_int(idx.numel()), c_int(x.shape[1]),
                                           c_int(_dt(x)), o._stream()), "gather_rows")
    return xs


def moe_finish(residual, y, weights, pos, shared=None, gate=None, overwrite: bool = False):
    """residual fp32 [T, n] += sum_k weights[t, k] * y[pos[t * K + k]] (+ gate[t] * shared[t]).  ``overwrite``: the sum
    replaces what ``residual`` held (a buffer that need not be cleared first)."""
    if not residual.is_cuda:
        if overwrite:
            residual.zero_()
        return reference.moe_finish(residual, y, weights, pos, shared, gate)
    o = _ops()
    _f32(residual, weights, gate)
    t, n = residual.shape
    assert y.is_contiguous() and y.shape[1] == n and pos.dtype == torch.int32
    assert shared is None or (shared.is_contiguous() and shared.shape == (t, n))
    o._check(o._kernels().vpsa_moe_finish(o._p(residual), o._p(y), o._p(weights), o._p(pos), c_int(weights.shape[1]),
                                          o._p(shared), o._p(gate), c_int(t), c_int(n), c_int(1 if overwrite else 0),
                                          c_int(_dt(y, shared)), o._stream()), "moe_finish")
    return residual


def gate_up_glu_clamp(x, w_gate_up, limit: float, alpha: float = 1.702, up_bias: float = 1.0):
    """The clamped gated unit's activation of ``x @ [Wg; Wu].T``: in the epilogue of the prefill GEMM when
    that kernel takes the shape, else the projection (``ops.linear``) and the activation kernel."""
    o = _ops()
    rows = o.tile_rows(x, w_gate_up, True) if x.is_cuda else 0
    if rows:
        return o.tile_gemm(x, w_gate_up, glu_clamp=(limit, alpha, up_bias))
    return glu_clamp(o.linear(x, w_gate_up), limit, alpha, up_bias)


def up_relu_sq(x, w_up):
    """relu(x @ W.T)^2, fused into the prefill GEMM's epilogue when that kernel takes the shape."""
    o = _ops()
    rows = o.tile_rows(x, w_up) if x.is_cuda else 0
    if rows:
        return o.tile_gemm(x, w_up, relu_sq=True)
    return relu_sq(o.linear(x, w_up))


def moe_glu_grouped_supported(x, w13, w2) -> bool:
    o = _ops()
    return (x.is_cuda and x.dtype == torch.bfloat16 and x.is_contiguous() and w13.is_contiguous() and w2.is_contiguous()
            and o.tile_gemm_supported(w13.shape[1], w13.shape[2], True) and o.tile_gemm_supported(w2.shape[1], w2.shape[2]))


def moe_glu_grouped(x, w13, w2, ids, limit: float, alpha: float = 1.702, up_bias: float = 1.0):
    """Clamped gated units of a mixture over the device-sorted (token, unit) pairs: two grouped
    matrix-core GEMMs (the first gathers its token rows and applies the activation in its epilogue).
    The host never reads the per-unit counts: no synchronisation, HIP-graph capturable.
    Returns (y [T * K, hidden] in sorted order, pos [T * K]: the sorted row of pair t * K + k)."""
    o = _ops()
    t, k = ids.shape
    offsets, pos, sorted_tok = o.moe_align(ids, w13.shape[0])
    hidden, inter = x.shape[1], w2.shape[2]
    if t <= o.MOE_MFMA_MAX_TOKENS and o.moe_mfma_supported(hidden, inter) and limit > 0:
        # decode-sized batches: each routed unit's weights streamed once against its few tokens
        # (the kernels of the top-k softmax mixtures, with this unit's activation)
        act = torch.empty((t * k, inter), dtype=x.dtype, device=x.device)
        y = torch.empty((t * k, hidden), dtype=x.dtype, device=x.device)
        o._check(o._kernels().vpsa_moe_mfma_act(o._p(x), o._p(w13), o._p(w2), o._p(offsets), o._p(sorted_tok), o._p(act),
                                                o._p(y), c_int(t), c_int(k), c_int(w13.shape[0]), c_int(hidden),
                                                c_int(inter), c_float(limit), c_float(alpha), c_float(up_bias),
                                                o._stream()), "moe_mfma_act")
        return y, pos
    act = o.tile_gemm(x, w13, offsets, rows=t * k, arow_idx=sorted_tok, glu_clamp=(limit, alpha, up_bias))
    return o.tile_gemm(act, w2, offsets, rows=t * k), pos
