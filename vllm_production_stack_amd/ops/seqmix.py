"""Ops of sequence mixers that carry state from token to token (``csrc/kernels/seqmix.hip``):
linear-attention recurrences, a short convolution in front of a windowed softmax attention with
kept first tokens, a sink and post-softmax head mixing, the Dynamic Tanh norm on the fp32 residual
stream and the xIELU activation.  Device tensors run the HIP kernels in bf16 or fp32 activations;
CPU tensors run the PyTorch definitions of ``reference.py``.

Two stores, both owned by the engine's runner:

- the paged pool ``[pages, page_elems]`` (activation dtype): a layer with windowed attention keeps, per
  page and ``cache_off`` elements into it, ``K [PAGE, kv_heads * dim]`` then V transposed,
  ``[kv_heads * vdim, PAGE]`` (a channel's 64 keys are contiguous); a layer that also sees pooled blocks of
  tokens keeps a second region of the same shape behind it for the blocks' mean keys and values;
- the state pool ``[slots, state_elems]`` (fp32): a sequence's slot holds, per layer and ``state_off``
  elements into it, a recurrence's ``[heads, dim, vdim]`` matrix or the ``conv - 1`` projected rows
  a convolution still needs.  A chunk that starts at position 0 starts from zeros, whatever the slot
  held before.

A batch is described by ``seq_cu`` (int32 [S + 1]: first row of every sequence, decode rows are
sequences of one row), ``seq_state`` (int32 [S]: the sequence's slot, -1 = rows of no sequence) and,
for row-wise kernels, ``row_seq`` (int32 [T], None = row i is sequence i).
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
            raise TypeError("sequence-mixer kernels take bf16 or fp32 device tensors")
        if d is not None and _DT[t.dtype] != d:
            raise TypeError("sequence-mixer kernels: mixed activation dtypes")
        d = _DT[t.dtype]
    return d


def _f32(*ts):
    for t in ts:
        if t is not None and (t.dtype != torch.float32 or not t.is_contiguous()):
            raise TypeError("expected a contiguous fp32 tensor")


def _i32(*ts):
    for t in ts:
        if t is not None and (t.dtype != torch.int32 or not t.is_contiguous()):
            raise TypeError("expected a contiguous int32 tensor")


def _rows(t) -> bool:
    return t.dim() == 2 and t.stride(1) == 1


def _at(t, offset: int):
    return c_void_p(t.data_ptr() + offset * t.element_size())


def add_dyt_norm(residual, deltas, weight, bias, alpha, out_dtype, want_out: bool = True):
    """residual (fp32, in place) += sum of scale * delta over ``deltas`` (up to two (tensor, scale)
    pairs); returns tanh(alpha * residual) * weight + bias in ``out_dtype`` (Dynamic Tanh: no mean, no
    variance).  ``alpha`` is a one-element fp32 tensor."""
    if not residual.is_cuda:
        return reference.add_dyt_norm(residual, deltas, weight, bias, alpha, out_dtype, want_out)
    o = _ops()
    _f32(residual, weight, bias, alpha)
    t, n = residual.shape
    assert len(deltas) <= 2
    if not deltas and not want_out:
        return None
    ds = list(deltas) + [(None, 0.0)] * (2 - len(deltas))
    for d, _ in ds:
        assert d is None or (_rows(d) and d.shape == residual.shape and d.dtype == out_dtype)
    y = torch.empty((t, n), dtype=out_dtype, device=residual.device) if want_out else None
    (d1, c1), (d2, c2) = ds
    o._check(o._kernels().vpsa_add_dyt(o._p(residual), o._p(d1), c_long(d1.stride(0) if d1 is not None else 0),
                                       c_float(c1), o._p(d2), c_long(d2.stride(0) if d2 is not None else 0), c_float(c2),
                                       o._p(weight), o._p(bias), o._p(alpha), o._p(y), c_int(t), c_int(n),
                                       c_int(_DT[out_dtype]), o._stream()), "add_dyt_norm")
    return y


SCAN_FOLD_MIN_DECAY = 0.1    # decay^-16 stays below 1e16
SCAN_PIECE_MIN_ROWS = 128   # sequences of a step shorter than this are walked in one go
SCAN_PIECES_TARGET = 96     # pieces per launch that fill the chip (times heads and column blocks)


def build_scan_pieces(q_lens, target: int = SCAN_PIECES_TARGET):
    """Cuts the sequences of a step into pieces the recurrence kernels run side by side.  Returns None when
    no sequence is long enough to pay for it, else (pieces int32 [n, 3] = (sequence, first row, rows),
    seq_pieces int32 [S + 1] = a sequence's first piece)."""
    import numpy as np

    if not q_lens or max(q_lens) < SCAN_PIECE_MIN_ROWS:
        return None
    total = sum(q_lens)
    size = min(512, max(64, (total // target + 15) // 16 * 16))
    pieces, first, row = [], [0], 0
    for i, n in enumerate(q_lens):
        for k in range(0, n, size):
            pieces.append((i, row + k, min(size, n - k)))
        row += n
        first.append(len(pieces))
    return np.asarray(pieces, dtype=np.int32).reshape(-1, 3), np.asarray(first, dtype=np.int32)


def recurrent_scan(proj, q_col: int, k_col: int, v_col: int, heads: int, dim: int, vdim: int, state, state_off: int,
                   seq_cu, seq_state, positions, *, decay=None, cos_sin=None, rot_dims: int = 0, layout: int = 0,
                   k_scale: float = 1.0, gate_bias=None, gate_lower=None, pieces=None, min_decay: float = 0.0,
                   act: bool = False):
    """Per sequence and head, over the sequence's rows in order: S <- a_t (.) S + k_t v_t^T, o_t = S^T q_t
    with S [dim, vdim] carried in the sequence's state slot.  q, k and v are column ranges of ``proj``
    [T, cols] (heads side by side).

    ``decay`` (fp32 [heads]): a_t = decay[head] for every row of S; q and k turn by the rotary table
    ``cos_sin`` over their first ``rot_dims`` channels (``layout`` 0: pairs (i, i + rot_dims / 2), 1: pairs
    (2 i, 2 i + 1)) and k is multiplied by ``k_scale`` afterwards.

    ``min_decay``: the smallest of the decays as the host knows it; from ``SCAN_FOLD_MIN_DECAY`` up the kernel
    folds the decay into the staged keys and queries of a 16-token block (two operations per state element and
    token instead of three).

    ``act`` (with ``decay``, no rotation): q, k and v pass through silu first.

    ``gate_bias`` / ``gate_lower`` (fp32 [heads * dim]) instead: the k columns hold gate logits,
    a_t = lower + (1 - lower) sigmoid(logit + bias) per row of S, k_t = 1 - a_t, q = silu(q).

    ``pieces``: device copies of ``build_scan_pieces`` for steps with long chunks: the pieces' end states
    from zero are computed side by side, chained per sequence (the recurrence is linear in S), and the
    outputs of all pieces are computed side by side from their start states.

    Returns o fp32 [T, heads, vdim]."""
    gated = decay is None
    if not proj.is_cuda:
        return reference.recurrent_scan(proj, q_col, k_col, v_col, heads, dim, vdim, gated, state, state_off, seq_cu,
                                        seq_state, positions, decay, cos_sin, rot_dims, layout, k_scale, gate_bias,
                                        gate_lower, act)
    o = _ops()
    _f32(state, decay, cos_sin, gate_bias, gate_lower)
    _i32(seq_cu, seq_state, positions)
    assert _rows(proj) and max(q_col, k_col) + heads * dim <= proj.shape[1] and v_col + heads * vdim <= proj.shape[1]
    assert state_off + heads * dim * vdim <= state.shape[1] and seq_cu.numel() == seq_state.numel() + 1
    assert (gate_bias is not None and gate_lower is not None) if gated else (rot_dims == 0 or cos_sin.shape[1] == rot_dims)
    assert rot_dims <= dim and rot_dims % 2 == 0 and not (act and (gated or rot_dims))
    out = torch.empty((proj.shape[0], heads, vdim), dtype=torch.float32, device=proj.device)
    # what enters the recurrence besides v, prepared in fp32 by a pass of its own: q' | k' (| gates)
    prep = torch.empty((proj.shape[0], heads, 3 if gated else 2, dim), dtype=torch.float32, device=proj.device)
    pc = sp = ws_state = ws_decay = None
    n_pieces = 0
    if pieces is not None:
        pc, sp = pieces
        _i32(pc, sp)
        n_pieces = pc.shape[0]
        assert pc.shape[1] == 3 and sp.numel() == seq_cu.numel()
        ws_state = torch.empty((n_pieces, heads, dim, vdim), dtype=torch.float32, device=proj.device)
        ws_decay = torch.empty((n_pieces, heads, dim), dtype=torch.float32, device=proj.device)
    o._check(o._kernels().vpsa_recurrent_scan(
        o._p(proj), c_long(proj.stride(0)), c_int(q_col), c_int(k_col), c_int(v_col), c_int(heads), c_int(dim),
        c_int(vdim), _at(state, state_off), c_long(state.stride(0)), o._p(seq_cu), o._p(seq_state),
        c_int(seq_state.numel()), o._p(positions), o._p(decay), o._p(cos_sin), c_int(rot_dims), c_int(layout),
        c_float(k_scale), o._p(gate_bias), o._p(gate_lower), o._p(out), c_int(1 if gated else 0), o._p(pc), o._p(sp),
        c_int(n_pieces), o._p(ws_state), o._p(ws_decay), o._p(prep), c_int(proj.shape[0]),
        c_int(1 if (not gated and min_decay >= SCAN_FOLD_MIN_DECAY) else 0), c_int(1 if act else 0), c_int(_dt(proj)),
        o._stream()), "recurrent_scan")
    return out


def gla_prepare(proj, q_col: int, k_col: int, z, z_bias, heads: int, dim: int, q_scale: float, tau: float):
    """What a gated-linear-attention recurrence takes besides v, fp32 [T, heads, 3, dim]: q * q_scale | k | a with
    the decay a = sigmoid(z + z_bias)^(1 / tau) per head and key channel.  q and k are column ranges of ``proj``,
    ``z`` [T, heads * dim] the decay's pre-activation (activation dtype), ``z_bias`` fp32."""
    if not proj.is_cuda:
        return reference.gla_prepare(proj, q_col, k_col, z, z_bias, heads, dim, q_scale, tau)
    o = _ops()
    _f32(z_bias)
    t = proj.shape[0]
    assert _rows(proj) and _rows(z) and z.shape == (t, heads * dim) and max(q_col, k_col) + heads * dim <= proj.shape[1]
    prep = torch.empty((t, heads, 3, dim), dtype=torch.float32, device=proj.device)
    o._check(o._kernels().vpsa_gla_prepare(o._p(proj), c_long(proj.stride(0)), c_int(q_col), c_int(k_col), o._p(z),
                                           c_long(z.stride(0)), o._p(z_bias), c_int(heads), c_int(dim), c_float(q_scale),
                                           c_float(tau), o._p(prep), c_int(t), c_int(_dt(proj, z)), o._stream()),
             "gla_prepare")
    return prep


def mlstm_prepare(proj, q_col: int, k_col: int, gate_logits, bias_i, bias_f, cap: float, heads: int, dim: int,
                  q_scale: float, state, m_off: int, seq_cu, seq_state, positions):
    """Gates of a matrix memory with exponential gating.  ``gate_logits`` fp32 [T, 2 heads] = input | forget gate
    pre-activations (biases apart); i = cap tanh((x_i + b_i) / cap), f = logsigmoid(cap tanh((x_f + b_f) / cap)).
    The running maximum m_t = max(f_t + m_(t-1), i_t) starts at 0 with the sequence and is carried in the
    sequence's state slot (``heads`` floats at ``m_off``).  Returns (prep fp32 [T, heads, 3, dim] =
    q * q_scale | k * exp(i_t - m_t) | exp(f_t + m_(t-1) - m_t), m fp32 [T, heads])."""
    if not proj.is_cuda:
        return reference.mlstm_prepare(proj, q_col, k_col, gate_logits, bias_i, bias_f, cap, heads, dim, q_scale, state,
                                       m_off, seq_cu, seq_state, positions)
    o = _ops()
    _f32(gate_logits, bias_i, bias_f, state)
    _i32(seq_cu, seq_state, positions)
    t = proj.shape[0]
    assert _rows(proj) and gate_logits.shape == (t, 2 * heads) and max(q_col, k_col) + heads * dim <= proj.shape[1]
    assert m_off + heads <= state.shape[1] and seq_cu.numel() == seq_state.numel() + 1
    prep = torch.empty((t, heads, 3, dim), dtype=torch.float32, device=proj.device)
    ab = torch.empty((t, heads, 2), dtype=torch.float32, device=proj.device)
    mrow = torch.empty((t, heads), dtype=torch.float32, device=proj.device)
    o._check(o._kernels().vpsa_mlstm_prepare(
        o._p(proj), c_long(proj.stride(0)), c_int(q_col), c_int(k_col), o._p(gate_logits), o._p(bias_i), o._p(bias_f),
        c_float(cap), c_int(heads), c_int(dim), c_float(q_scale), _at(state, m_off), c_long(state.stride(0)), o._p(seq_cu),
        o._p(seq_state), c_int(seq_state.numel()), o._p(positions), o._p(ab), o._p(mrow), o._p(prep), c_int(t),
        c_int(_dt(proj)), o._stream()), "mlstm_prepare")
    return prep, mrow


def scan_state_cols(vdim: int, unit_col: bool = False) -> int:
    """Columns per key channel of a prepared recurrence's state: the values, one more for the normaliser when
    ``unit_col``, rounded up to whole float4."""
    return (vdim + 4) // 4 * 4 if unit_col else vdim


def prepared_scan(prep, proj, v_col: int, heads: int, dim: int, vdim: int, state, state_off: int, seq_cu, seq_state,
                  positions, *, unit_col: bool = False, pieces=None):
    """``recurrent_scan`` over rows a caller prepared: prep fp32 [T, heads, 3, dim] = q' | k' | a (per row, head and
    key channel), S <- diag(a_t) S + k'_t v_t^T, o_t = S^T q'_t, with S carried in the sequence's state slot.
    v is a column range of ``proj``.  ``unit_col``: the state gets one more value column that is fed with ones, so
    that it accumulates n_t = a_t n_(t-1) + k'_t and its read-out is n_t . q'_t (a normaliser); the state then
    has ``scan_state_cols(vdim, True)`` columns.  Returns o fp32 [T, heads, state columns]."""
    cols = scan_state_cols(vdim, unit_col)
    if not proj.is_cuda:
        return reference.prepared_scan(prep, proj, v_col, heads, dim, vdim, cols, unit_col, state, state_off, seq_cu,
                                       seq_state, positions)
    o = _ops()
    _f32(prep, state)
    _i32(seq_cu, seq_state, positions)
    t = proj.shape[0]
    assert _rows(proj) and v_col + heads * vdim <= proj.shape[1] and prep.shape == (t, heads, 3, dim)
    assert state_off + heads * dim * cols <= state.shape[1] and seq_cu.numel() == seq_state.numel() + 1
    out = torch.empty((t, heads, cols), dtype=torch.float32, device=proj.device)
    pc = sp = ws_state = ws_decay = None
    n_pieces = 0
    if pieces is not None:
        pc, sp = pieces
        _i32(pc, sp)
        n_pieces = pc.shape[0]
        assert pc.shape[1] == 3 and sp.numel() == seq_cu.numel()
        ws_state = torch.empty((n_pieces, heads, dim, cols), dtype=torch.float32, device=proj.device)
        ws_decay = torch.empty((n_pieces, heads, dim), dtype=torch.float32, device=proj.device)
    o._check(o._kernels().vpsa_prepared_scan(
        o._p(proj), c_long(proj.stride(0)), c_int(v_col), c_int(vdim), c_int(1 if unit_col else 0), c_int(heads),
        c_int(dim), c_int(cols), o._p(prep), _at(state, state_off), c_long(state.stride(0)), o._p(seq_cu),
        o._p(seq_state), c_int(seq_state.numel()), o._p(positions), o._p(out), o._p(pc), o._p(sp), c_int(n_pieces),
        o._p(ws_state), o._p(ws_decay), c_int(t), c_int(_dt(proj)), o._stream()), "prepared_scan")
    return out


GATE_ACTS = {"silu": 0, "sigmoid": 1}


def head_finish(o_heads, eps: float, out_dtype, *, vdim: int | None = None, stab=None, unit: bool = True, weight=None,
                gate=None, gate_act: str = "silu"):
    """Head outputs o fp32 [T, heads, cols] (the first ``vdim`` columns count) -> [T, heads * vdim] in ``out_dtype``.
    In this order, each part optional: ``stab`` (fp32 [T, heads], the gates' running maximum m): column ``vdim`` of o
    is a normaliser's read-out n . q and the output is divided by max(|n . q|, exp(-m)) + 1e-6; ``unit``: every head
    divided by its root mean square (eps inside the root); ``weight`` fp32 [vdim] (shared by the heads) or
    [heads * vdim]; ``gate`` (a [T, heads * vdim] view of a wider projection) through silu or sigmoid."""
    t, heads, cols = o_heads.shape
    vdim = cols if vdim is None else vdim
    if not o_heads.is_cuda:
        return reference.head_finish(o_heads, eps, out_dtype, vdim, stab, unit, weight, gate, gate_act)
    o = _ops()
    _f32(o_heads, weight, stab)
    assert gate is None or (_rows(gate) and gate.shape == (t, heads * vdim) and gate.dtype == out_dtype)
    assert weight is None or weight.numel() in (vdim, heads * vdim)
    assert stab is None or (stab.shape == (t, heads) and cols > vdim)
    y = torch.empty((t, heads * vdim), dtype=out_dtype, device=o_heads.device)
    o._check(o._kernels().vpsa_head_finish(
        o._p(o_heads), c_int(cols), o._p(stab), c_int(1 if unit else 0), o._p(weight),
        c_int(1 if (weight is not None and weight.numel() != vdim) else 0), o._p(gate),
        c_long(gate.stride(0) if gate is not None else 0), c_int(GATE_ACTS[gate_act]), o._p(y), c_int(t), c_int(heads),
        c_int(vdim), c_float(eps), c_int(_DT[out_dtype]), o._stream()), "head_finish")
    return y


def qk_norm_write(proj, heads: int, kv_heads: int, dim: int, vdim: int, positions, slots, pool, cache_off: int,
                  eps: float, temp_coef: float = 0.0, temp_every: float = 1.0, own: bool = True, *,
                  v_heads: int | None = None, q_weight=None, k_weight=None, cos_sin=None, rot_dims: int = 0,
                  layout: int = 0):
    """Rows of a fused projection, q | k | v (``own``) or q alone (a layer that reads another layer's cache
    entries): every q and k head is divided by its root mean square (eps inside the root), multiplied by
    ``q_weight`` / ``k_weight`` (fp32 [dim], shared by the heads) where given, and turned by the rotary table
    ``cos_sin`` over its first ``rot_dims`` channels (``layout`` 0: pairs (i, i + rot_dims / 2), 1: pairs
    (2 i, 2 i + 1)); q at position p is then multiplied by 1 + temp_coef ln(floor((p + 1) / temp_every) + 1).
    k and v go to the paged cache at ``slots`` (< 0: not cached) in the layout ``window_attention`` reads;
    ``v_heads``: value heads, when fewer than the ``kv_heads`` key heads (several key maps per value head).
    Returns q [T, heads, dim]."""
    v_heads = kv_heads if v_heads is None else v_heads
    if not proj.is_cuda:
        return reference.qk_norm_write(proj, heads, kv_heads, dim, vdim, positions, slots, pool, cache_off, eps,
                                       temp_coef, temp_every, own, v_heads, q_weight, k_weight, cos_sin, rot_dims, layout)
    o = _ops()
    _i32(positions)
    _f32(q_weight, k_weight, cos_sin)
    t = proj.shape[0]
    chans = heads * dim + (kv_heads * dim + v_heads * vdim if own else 0)
    assert _rows(proj) and proj.shape[1] >= chans and slots.dtype == torch.int64
    assert pool.dim() == 2 and pool.stride(1) == 1
    assert cache_off + window_cache_elems(kv_heads, dim, vdim, v_heads) <= pool.shape[1]
    assert rot_dims == 0 or (cos_sin is not None and cos_sin.shape[1] == rot_dims and rot_dims <= dim)
    assert all(w is None or w.numel() == dim for w in (q_weight, k_weight))
    q = torch.empty((t, heads, dim), dtype=proj.dtype, device=proj.device)
    o._check(o._kernels().vpsa_qk_norm_write(
        o._p(proj), c_long(proj.stride(0)), c_int(heads), c_int(kv_heads), c_int(dim), c_int(vdim), c_int(1 if own else 0),
        o._p(positions), o._p(slots), c_float(eps), c_float(temp_coef), c_float(temp_every), o._p(q), _at(pool, cache_off),
        c_long(pool.stride(0)), c_int(t), c_int(v_heads), o._p(q_weight), o._p(k_weight), o._p(cos_sin), c_int(rot_dims),
        c_int(layout), c_int(_dt(proj, pool)), o._stream()), "qk_norm_write")
    return q


def pool_blocks(pool, cache_off: int, pool_off: int, kv_heads: int, dim: int, vdim: int, block_tables, row_seq,
                positions, slots, block: int):
    """Pooled entries of a windowed attention that sees one mean key and value per block of ``block`` tokens
    before its window.  For every row of the step that completes a block (position p with (p + 1) % block == 0,
    cached), the block's keys and values are read back from the pages, averaged in fp32 in position order, and
    stored as entry b % PAGE of the pooled region (``pool_off`` elements behind the layer's token region, same
    layout) of the sequence's page b / PAGE, b = p // block.  Call it after the step's keys and values are written
    and before its attention."""
    if positions.numel() == 0:
        return
    if not pool.is_cuda:
        return reference.pool_blocks(pool, cache_off, pool_off, kv_heads, dim, vdim, block_tables, row_seq, positions,
                                     slots, block)
    o = _ops()
    _i32(positions, row_seq)
    assert block_tables.dtype == torch.int32 and block_tables.stride(1) == 1 and slots.dtype == torch.int64
    assert block >= 1 and pool_off >= window_cache_elems(kv_heads, dim, vdim)
    assert cache_off + pool_off + window_cache_elems(kv_heads, dim, vdim) <= pool.shape[1]
    o._check(o._kernels().vpsa_pool_blocks(
        _at(pool, cache_off), c_long(pool.stride(0)), c_long(pool_off), o._p(block_tables), c_int(block_tables.stride(0)),
        o._p(row_seq), o._p(positions), o._p(slots), c_int(positions.numel()), c_int(kv_heads * dim),
        c_int(kv_heads * vdim), c_int(block), c_int(_dt(pool)), o._stream()), "pool_blocks")


def diff_heads(u, kv_heads: int, lam: float, eps: float, post: float, out_dtype):
    """Differential attention's combination.  u fp32 [T, 2 heads, vdim] holds, per key/value group, the first
    map's outputs of the group's query heads and then the second map's.  Per head o = a1 - lam * a2, divided by its
    root mean square (eps inside the root), times ``post``; returns [T, heads * vdim] in ``out_dtype``, heads in
    their natural order."""
    if not u.is_cuda:
        return reference.diff_heads(u, kv_heads, lam, eps, post, out_dtype)
    o = _ops()
    _f32(u)
    t, h2, vdim = u.shape
    assert h2 % 2 == 0 and (h2 // 2) % kv_heads == 0
    y = torch.empty((t, h2 // 2 * vdim), dtype=out_dtype, device=u.device)
    o._check(o._kernels().vpsa_diff_heads(o._p(u), o._p(y), c_int(t), c_int(h2 // 2), c_int(kv_heads), c_int(vdim),
                                          c_float(lam), c_float(eps), c_float(post), c_int(_DT[out_dtype]), o._stream()),
             "diff_heads")
    return y


def head_rms_norm(o_heads, eps: float, out_dtype, weight=None, gate=None):
    """o fp32 [T, heads, vdim] -> [T, heads * vdim] in ``out_dtype``: every head divided by its root mean
    square (eps inside the root), times ``weight`` (fp32 [vdim], shared by the heads) and times
    silu(``gate``) (a [T, heads * vdim] view of a wider projection) where given."""
    if not o_heads.is_cuda:
        return reference.head_rms_norm(o_heads, eps, weight, gate, out_dtype)
    o = _ops()
    _f32(o_heads, weight)
    t, heads, vdim = o_heads.shape
    assert gate is None or (_rows(gate) and gate.shape == (t, heads * vdim) and gate.dtype == out_dtype)
    y = torch.empty((t, heads * vdim), dtype=out_dtype, device=o_heads.device)
    o._check(o._kernels().vpsa_head_rms(o._p(o_heads), o._p(weight), o._p(gate),
                                        c_long(gate.stride(0) if gate is not None else 0), o._p(y), c_int(t),
                                        c_int(heads), c_int(vdim), c_float(eps), c_int(_DT[out_dtype]), o._stream()),
             "head_rms_norm")
    return y


def window_cache_elems(kv_heads: int, dim: int, vdim: int, v_heads: int | None = None) -> int:
    """Elements a windowed-attention layer keeps per page (one region: the tokens', or the pooled blocks')."""
    return PAGE * (kv_heads * dim + (kv_heads if v_heads is None else v_heads) * vdim)


def short_conv_qkv(proj, conv_w, heads: int, kv_heads: int, dim: int, vdim: int, state, state_off: int, row_seq, seq_cu,
                   seq_state, positions, slots, cos_sin, rot_dims: int, layout: int, pool, cache_off: int):
    """The fused q | k | v projection rows ``proj`` [T, >= channels] through a causal convolution over
    time on every channel (``conv_w`` fp32 [channels, taps]: y_t = sum_j w[:, j] u_(t - taps + 1 + j), zeros
    before position 0; the rows before a chunk come from the sequence's state slot, which afterwards
    holds the chunk's last taps - 1 rows), then the rotary table on q and k.  k and v go to the paged
    cache at ``slots`` (< 0: not cached); returns q [T, heads, dim]."""
    if not proj.is_cuda:
        return reference.short_conv_qkv(proj, conv_w, heads, kv_heads, dim, vdim, state, state_off, seq_cu, seq_state,
                                        positions, slots, cos_sin, rot_dims, layout, pool, cache_off)
    o = _ops()
    _f32(state, conv_w, cos_sin)
    _i32(row_seq, seq_cu, seq_state, positions)
    t = proj.shape[0]
    chans = heads * dim + kv_heads * (dim + vdim)
    taps = conv_w.shape[1]
    assert _rows(proj) and proj.shape[1] >= chans and conv_w.shape[0] == chans and slots.dtype == torch.int64
    assert state_off + (taps - 1) * chans <= state.shape[1] and (rot_dims == 0 or cos_sin.shape[1] == rot_dims)
    assert pool.dim() == 2 and pool.stride(1) == 1 and cache_off + window_cache_elems(kv_heads, dim, vdim) <= pool.shape[1]
    assert row_seq is None or row_seq.numel() == t
    q = torch.empty((t, heads, dim), dtype=proj.dtype, device=proj.device)
    o._check(o._kernels().vpsa_short_conv_qkv(
        o._p(proj), c_long(proj.stride(0)), o._p(conv_w), c_int(taps), c_int(heads), c_int(kv_heads), c_int(dim),
        c_int(vdim), _at(state, state_off), c_long(state.stride(0)), o._p(row_seq), o._p(seq_cu), o._p(seq_state),
        c_int(seq_state.numel()), o._p(positions), o._p(slots), o._p(cos_sin), c_int(rot_dims), c_int(layout), o._p(q),
        _at(pool, cache_off), c_long(pool.stride(0)), c_int(t), c_int(_dt(proj, pool)), o._stream()), "short_conv_qkv")
    return q


def window_tile_slots() -> int:
    """(row, query head) pairs of one prefill tile of the matrix-core kernel."""
    return int(_ops()._kernels().vpsa_window_tile_slots())


WINDOW_MFMA = True      # False: every call takes the plain kernel (A/B runs, tests of the plain kernel)


def window_mfma_supported(heads: int, kv_heads: int, dim: int, vdim: int, own_values: bool = False) -> bool:
    return bool(_ops()._kernels().vpsa_window_mfma_supported(c_int(heads), c_int(kv_heads), c_int(dim), c_int(vdim),
                                                             c_int(1 if own_values else 0)))


def build_window_tiles(q_lens, ctx_lens, heads: int, kv_heads: int, chunk: int = 0):
    """Work list of the matrix-core kernel for the prefill part of a batch: int32 rows (sequence, first
    query row, rows, position of the first row); a tile holds consecutive rows of one sequence, as many as
    fit the kernel's slots ((row, query head of one KV group) pairs).  Latest rows first (they visit the most pages);
    with ``chunk`` (rows that see their own chunk of positions only) the rows deepest into their chunk first."""
    import numpy as np

    per = max(1, window_tile_slots() // (heads // kv_heads))
    parts = []
    row = 0
    for i, (n, ctx) in enumerate(zip(q_lens, ctx_lens)):
        k = np.arange(0, n, per, dtype=np.int64)
        parts.append(np.stack([np.full_like(k, i), row + k, np.minimum(per, n - k), ctx - n + k], axis=1))
        row += n
    if not parts:
        return np.zeros((0, 4), dtype=np.int32)
    tiles = np.concatenate(parts)
    work = tiles[:, 3] % chunk if chunk else tiles[:, 3]
    return tiles[np.argsort(-work, kind="stable")].astype(np.int32)


def window_decode_splits(rows: int, kv_heads: int, window: int, keep_first: int, max_ctx: int) -> int:
    """Key ranges per decode row: enough workgroups (rows x KV groups x splits) for about two per CU, none
    shorter than two pages."""
    pages = (min(window, max_ctx) + PAGE - 1) // PAGE + 1 + (keep_first + PAGE - 1) // PAGE
    want = max(1, 512 // max(1, rows * kv_heads))
    return max(1, min(want, pages // 2, 8))


def window_attention(q, pool, cache_off: int, kv_heads: int, vdim: int, block_tables, row_seq, positions, window: int,
                     keep_first: int, scale: float, softcap: float, sink, out=None, tiles=None, splits: int = 1,
                     own_values: bool = False, *, chunked: bool = False, pool_block: int = 0, pool_off: int = 0,
                     maps: int = 1):
    """Query rows q [T, heads, dim] over their sequences' cached keys: row i at position p sees key j when
    j <= p and (p - j < window or j < keep_first).  score = cap * tanh(q . k * scale / cap) (cap 0: none);
    softmax with ``sink`` [heads] (fp32, or None) in the denominator.  ``chunked``: ``window`` is a chunk size
    instead, and a row sees the keys of its own chunk (counted from position 0) up to itself.  ``pool_block`` P > 0:
    beside its window the row also sees the pooled entries (``pool_blocks``, ``pool_off`` elements behind the token
    region) of every block of P tokens that lies wholly before the window, in the same softmax.  ``maps`` > 1 (with
    ``own_values``): ``kv_heads`` counts key heads, of which ``maps`` neighbours share one value head.
    Returns u fp32 [T, heads, kv_heads, vdim]:
    each head's weights applied to the values of every KV head (``mix_heads`` picks and mixes).  With
    ``own_values`` only those of the head's own KV head: u fp32 [T, heads, 1, vdim], the attention output of designs
    without head mixing (a window of at least the context length makes it plain causal attention).

    bf16 rows of a shape the matrix-core kernel tiles take it: decode batches (``row_seq`` None) as they
    are (with ``splits`` key ranges per row, merged by a second launch), prefill rows when ``tiles`` (the
    device copy of ``build_window_tiles``) describes them.  Everything else takes the plain kernel."""
    t, heads, dim = q.shape
    vsets = 1 if own_values else kv_heads
    if out is None:
        out = torch.empty((t, heads, vsets, vdim), dtype=torch.float32, device=q.device)
    if t == 0:
        return out
    assert maps == 1 or (own_values and kv_heads % maps == 0)
    assert not pool_block or (keep_first == 0 and not chunked)
    if not q.is_cuda:
        return reference.window_attention(q, pool, cache_off, kv_heads, vdim, block_tables, row_seq, positions, window,
                                          keep_first, scale, softcap, sink, out, own_values, 1 if chunked else 0,
                                          pool_block, pool_off, maps)
    o = _ops()
    _f32(sink, out)
    _i32(row_seq, positions)
    assert q.is_contiguous() and block_tables.dtype == torch.int32 and block_tables.stride(1) == 1
    region = window_cache_elems(kv_heads, dim, vdim, kv_heads // maps)
    assert heads % kv_heads == 0 and cache_off + (pool_off if pool_block else 0) + region <= pool.shape[1]
    assert not pool_block or (pool_off >= region and (pool_off * pool.element_size()) % 16 == 0)
    extra = (c_int(1 if chunked else 0), c_int(pool_block), c_long(pool_off), c_int(maps))
    esz = pool.element_size()
    assert (cache_off * esz) % 16 == 0 and (pool.stride(0) * esz) % 16 == 0 and pool.data_ptr() % 16 == 0
    dt = _dt(q, pool)
    own = c_int(1 if own_values else 0)
    if (WINDOW_MFMA and dt == 0 and (tiles is not None or row_seq is None)
            and window_mfma_supported(heads, kv_heads, dim, vdim, own_values)
            and q.data_ptr() % 16 == 0 and out.data_ptr() % 16 == 0):
        ws_o = ws_ml = None
        if tiles is not None:
            assert tiles.dtype == torch.int32 and tiles.is_contiguous() and tiles.shape[1] == 4
            splits = 1
        elif splits > 1:
            assert out.is_contiguous()
            ws_o = torch.empty((t * heads * splits * vsets * vdim,), dtype=torch.float32, device=q.device)
            ws_ml = torch.empty((t * heads * splits * 2,), dtype=torch.float32, device=q.device)
        o._check(o._kernels().vpsa_window_attention_mfma(
            o._p(q), c_long(q.stride(0)), _at(pool, cache_off), c_long(pool.stride(0)), o._p(block_tables),
            c_int(block_tables.stride(0)), o._p(tiles), o._p(positions), o._p(sink), o._p(out),
            c_int(tiles.shape[0] if tiles is not None else t), c_int(heads), c_int(kv_heads), c_int(dim), c_int(vdim),
            c_int(window), c_int(keep_first), c_float(scale), c_float(softcap), c_int(splits), o._p(ws_o), o._p(ws_ml),
            own, *extra, o._stream()), "window_attention_mfma")
        return out
    o._check(o._kernels().vpsa_window_attention(
        o._p(q), c_long(q.stride(0)), _at(pool, cache_off), c_long(pool.stride(0)), o._p(block_tables),
        c_int(block_tables.stride(0)), o._p(row_seq), o._p(positions), o._p(sink), o._p(out), c_int(t), c_int(heads),
        c_int(kv_heads), c_int(dim), c_int(vdim), c_int(window), c_int(keep_first), c_float(scale), c_float(softcap),
        own, *extra, c_int(dt), o._stream()), "window_attention")
    return out


def mix_heads(u, talk, out_dtype):
    """u fp32 [T, heads, kv_heads, vdim], talk fp32 [heads, heads] -> [T, heads * vdim]:
    out[t, h] = sum_g talk[h, g] * u[t, g, kv head of h] (softmax weights mixed across heads, each head
    keeping its own values)."""
    if not u.is_cuda:
        return reference.mix_heads(u, talk, out_dtype)
    o = _ops()
    _f32(u, talk)
    t, heads, kv_heads, vdim = u.shape
    y = torch.empty((t, heads * vdim), dtype=out_dtype, device=u.device)
    o._check(o._kernels().vpsa_mix_heads(o._p(u), o._p(talk), o._p(y), c_int(t), c_int(heads), c_int(kv_heads),
                                         c_int(vdim), c_int(_DT[out_dtype]), o._stream()), "mix_heads")
    return y


def xielu(x, act):
    """z > 0: act[0] z^2 + z / 2; else act[1] (exp(z) - 1 - z) + z / 2.  ``act`` fp32 [2] on the device
    (softplus of the first learned number, 1/2 + softplus of the second)."""
    if not x.is_cuda:
        return reference.xielu(x, act)
    o = _ops()
    _f32(act)
    assert x.is_contiguous()
    y = torch.empty_like(x)
    o._check(o._kernels().vpsa_xielu(o._p(x), o._p(y), c_long(x.numel()), o._p(act), c_int(_dt(x)), o._stream()),
             "xielu")
    return y


def up_xielu(x, w_up, act, act_host=None):
    """xielu(x @ W.T), in the prefill GEMM's epilogue when that kernel takes the shape (``act_host``: the two
    numbers of ``act`` on the host, which the launch then carries as arguments)."""
    o = _ops()
    rows = o.tile_rows(x, w_up) if (x.is_cuda and act_host is not None) else 0
    if rows:
        return o.tile_gemm(x, w_up, xielu=act_host)
    return xielu(o.linear(x, w_up), act)
