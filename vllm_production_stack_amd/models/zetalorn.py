"""Zetalorn: a decoder whose layers, listed one by one in the configuration, are pre-norm with a gated
residual: ``x += sigmoid(W_g h + b) * sublayer(h)`` with ``h = rmsnorm(x) * g`` (one learned number g per norm),
first around a mixer, then around an optional mixture of experts.  The residual stream is fp32.

A run of neighbouring layers may loop: it is executed several times in a row with the same weights, every pass
with cache entries and recurrent state of its own; before every pass a learned vector of that pass is added to
the stream, and before every pass but the first the embedding output as well.  The model therefore works on
layer RUNS: a run has the weights of its layer and its own part of a pool page and of a state slot.

Mixers:

- ``attention``: differential grouped-query attention.  Every head has two query / key maps over the same values;
  q | k | v | residual-gate logits come from one fused projection, q and k maps are RMS-normed (a weight vector each),
  rotated (pairs (2 i, 2 i + 1), frequencies divided by a scaling factor) and k and v go to the paged pool; both maps
  run through the windowed-attention kernels as heads of their own (the query rows of the projection are ordered
  group, map, head at load so that a map's heads are neighbours over one key head; two key heads share a value
  head), masked to the query's chunk of positions; ``a1 - lambda a2`` is brought to unit RMS per head.
- ``parallel``: two mixers on the same input through one fused projection.  Left: grouped-query attention with
  normed, rotated q and k (pairs (i, i + dims / 2)) over a sliding window and, in the same softmax, one mean
  key / value per block of tokens that lies wholly before the window (the pooled entries live in a second region
  of the sequence's pages, written when a block's last token is).  Right: linear attention with a fixed decay per
  head on silu'd q, k and v, state in the sequence's slot; heads normed together, gated by sigmoid(W_g h).  The
  layer's result is half the sum of the two outputs, each RMS-normed over the model width with its own weight.

Feed-forward: a mixture of clamped gated units chosen by group-limited sigmoid routing, weights renormalised over
the chosen units.  Logits come from an output matrix of their own, times ``logit_scale``.
"""

from __future__ import annotations

import torch
import torch.nn.functional as F

from .. import ops
from ..engine.config import DiffAttentionSpec, FeedForwardSpec, ModelConfig, ParallelMixerSpec
from ..ops.reference import PAGE
from ..parallel.state import get_pp, get_tp
from .batch import BatchMeta

LAYOUTS = {"half": 0, "pairs": 1}
GLU_ALPHA = 1.702   # the gated unit: g sigmoid(1.702 g) (u + 1) on clamped g and u
GLU_UP_BIAS = 1.0


class ZetalornLayer:
    __slots__ = ("spec", "norm1", "norm2", "w_in", "rg1_b", "q_norm", "k_norm", "w_o", "lam_vecs", "lam", "cos_sin",
                 "wr_o", "r_norm", "left_out", "right_out", "decay", "router", "w13", "w2", "rg2", "rg2_b")

    def __init__(self, spec):
        for s in self.__slots__:
            setattr(self, s, None)
        self.spec = spec


class Pending:
    """A sublayer's result that the next norm adds to the stream: up to two (delta, norm weight, factor) triples,
    the residual gate's logits (a view of the sublayer's input projection) and their bias."""
    __slots__ = ("deltas", "gate", "bias")

    def __init__(self, deltas, gate, bias):
        self.deltas, self.gate, self.bias = deltas, gate, bias

    def rows(self, idx):
        return Pending([(d.index_select(0, idx), w, c) for d, w, c in self.deltas], self.gate.index_select(0, idx), self.bias)


class ZetalornModel:
    stateful = True  # sequences carry state slots; a prefix's pages alone do not restore a sequence

    def __init__(self, cfg: ModelConfig, dtype: torch.dtype, device: torch.device, max_model_len: int):
        if get_tp().size != 1 or get_pp().size != 1:
            raise ValueError("Zetalorn runs on single-GPU replicas (no tensor / pipeline parallel layout yet)")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Zetalorn runs in bfloat16 or float32")
        self.cfg = cfg
        self.dtype = dtype
        self.device = device
        self.max_model_len = max_model_len
        self.specs = cfg.layer_specs
        self.n_q = cfg.num_heads
        self.n_kv = cfg.num_kv_heads
        self.head_dim = cfg.head_dim
        self.tp_size = 1
        self.lora = None
        self.layers: list[ZetalornLayer] = []
        self.embed = self.norm = self.lm_head = self.loop_step = None
        self.state: torch.Tensor | None = None  # [slots, state_elems] fp32, bound by the runner
        self.layer_probe = None  # callable(run index, fp32 residual stream after the run) for tests
        # the layer runs, and where each run's part of a pool page and of a state slot starts, in elements
        self.runs = cfg.layer_runs()
        self.cache_offsets: list[int] = []
        self.state_offsets: list[int | None] = []
        c_off = s_off = 0
        for li, _ in self.runs:
            m = self.specs[li].mixer
            self.cache_offsets.append(c_off)
            if isinstance(m, ParallelMixerSpec):
                c_off += PAGE * m.left.cache_elems()
                self.state_offsets.append(s_off)
                s_off += (m.right.state_elems() + 3) // 4 * 4  # parts start on 16-byte boundaries
            else:
                c_off += PAGE * m.cache_elems()
                self.state_offsets.append(None)
        self.page_elems = max(c_off, 8)
        self.state_elems = max(s_off, 8)
        self._tables: dict[tuple, torch.Tensor] = {}

    @property
    def graph_capturable(self) -> bool:
        """Decode steps can be captured when no layer's mixture falls back to the per-unit loop, which reads
        the row counts on the host (shapes the grouped GEMM does not tile, fp32)."""
        probe = torch.empty((1, self.cfg.hidden_size), dtype=self.dtype, device=self.device)
        return self.dtype == torch.bfloat16 and self.device.type == "cuda" and all(
            lw.w13 is None or ops.moe_glu_grouped_supported(probe, lw.w13, lw.w2) for lw in self.layers)

    # ------------------------------------------------------------------ stores
    def kv_page_shape(self) -> tuple:
        """Shape of one page of the KV pool (the runner allocates [pages, *shape])."""
        return (self.page_elems,)

    def state_shape(self) -> tuple:
        """Shape of one sequence's state slot (the runner allocates fp32 [slots, *shape])."""
        return (self.state_elems,)

    def bind_state(self, state: torch.Tensor | None) -> None:
        self.state = state

    def _cos_sin(self, rot) -> torch.Tensor | None:
        if rot.dims == 0:
            return None
        key = (rot.base, rot.dims, rot.linear)
        t = self._tables.get(key)
        if t is None:
            t = self._tables[key] = ops.build_cos_sin(rot.dims, self.max_model_len, rot.base, rot.table_scaling(),
                                                      device=self.device)
        return t

    # ------------------------------------------------------------------ weights
    def _alloc(self, gen, *shape, std=None, dtype=None, mean=0.0):
        dtype = dtype or self.dtype
        t = torch.empty(shape, dtype=torch.float32, device=self.device)
        t.normal_(mean, std if std is not None else shape[-1] ** -0.5, generator=gen)
        return t.to(dtype)

    def in_rows(self, spec) -> dict:
        """Row ranges of a layer's fused input projection, by the part's name."""
        m = spec.mixer
        w = self.cfg.hidden_size
        if isinstance(m, DiffAttentionSpec):
            parts = [("q", 2 * m.heads * m.dim), ("k", 2 * m.kv_heads * m.dim), ("v", m.kv_heads * m.vdim)]
        else:
            a, r = m.left, m.right
            parts = [("left.q", a.heads * a.dim), ("left.k", a.kv_heads * a.dim), ("left.v", a.kv_heads * a.vdim),
                     ("right.q", r.heads * r.dim), ("right.k", r.heads * r.dim), ("right.v", r.heads * r.vdim),
                     ("right.g", r.heads * r.vdim)]
        out, at = {}, 0
        for name, n in parts + [("rg1", w)]:
            out[name] = (at, at + n)
            at += n
        out["end"] = (at, at)
        return out

    def init_random(self, seed: int = 0) -> None:
        """Allocates every tensor in the layout the forward pass uses; a checkpoint overwrites them."""
        cfg = self.cfg
        w = cfg.hidden_size
        g = torch.Generator(device=self.device).manual_seed(seed)
        f32 = torch.float32
        self.embed = self._alloc(g, cfg.vocab_size, w, std=1.0)
        self.lm_head = self._alloc(g, cfg.vocab_size, w)
        times = cfg.layer_loop[2] if cfg.layer_loop else 0
        self.loop_step = self._alloc(g, times, w, std=0.1, dtype=f32) if times else None
        self.layers = []
        for s in self.specs:
            m, f = s.mixer, s.mlp
            lw = ZetalornLayer(s)
            lw.norm1 = torch.ones(w, dtype=f32, device=self.device)
            lw.w_in = self._alloc(g, self.in_rows(s)["end"][0], w)
            lw.rg1_b = self._alloc(g, w, std=0.5, dtype=f32)
            if isinstance(m, DiffAttentionSpec):
                att = m
                lw.lam_vecs = self._alloc(g, 4, m.dim, std=0.2, dtype=f32)
                self.set_lambda(lw)
            else:
                att, r = m.left, m.right
                lw.wr_o = self._alloc(g, w, r.heads * r.vdim)
                lw.r_norm = self._alloc(g, r.heads * r.vdim, std=0.1, dtype=f32, mean=1.0)
                lw.left_out = self._alloc(g, w, std=0.1, dtype=f32, mean=1.0)
                lw.right_out = self._alloc(g, w, std=0.1, dtype=f32, mean=1.0)
                lw.decay = torch.tensor(r.decay, dtype=f32, device=self.device)
            lw.q_norm = self._alloc(g, att.dim, std=0.1, dtype=f32, mean=1.0)
            lw.k_norm = self._alloc(g, att.dim, std=0.1, dtype=f32, mean=1.0)
            lw.w_o = self._alloc(g, w, att.heads * att.vdim)
            lw.cos_sin = self._cos_sin(att.rot)
            if f is not None:
                lw.norm2 = torch.ones(w, dtype=f32, device=self.device)
                lw.router = self._alloc(g, f.experts, w, dtype=f32)
                lw.w13 = self._alloc(g, f.experts, 2 * f.ff, w)
                lw.w2 = self._alloc(g, f.experts, w, f.ff)
                lw.rg2 = self._alloc(g, w, w)
                lw.rg2_b = self._alloc(g, w, std=0.5, dtype=f32)
            self.layers.append(lw)
        self.norm = torch.ones(w, dtype=f32, device=self.device)

    def set_lambda(self, lw: ZetalornLayer) -> None:
        """The layer's lambda from its four vectors lq1 | lk1 | lq2 | lk2 (a launch argument of the combining kernel)."""
        v = lw.lam_vecs.double().cpu()
        lw.lam = float(torch.exp((v[0] * v[1]).sum()) - torch.exp((v[2] * v[3]).sum()) + lw.spec.mixer.diff)

    def weight_tensors(self):
        for t in (self.embed, self.lm_head, self.norm, self.loop_step):
            if t is not None:
                yield t
        for lw in self.layers:
            for s in ZetalornLayer.__slots__:
                t = getattr(lw, s)
                if s != "cos_sin" and isinstance(t, torch.Tensor):
                    yield t

    def weight_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.weight_tensors())

    # ------------------------------------------------------------------ batch description
    def _tile_keys(self):
        keys = set()
        for s in self.specs:
            m = s.mixer
            k = ((2 * m.heads, 2 * m.kv_heads, m.dim, m.vdim, m.chunk) if isinstance(m, DiffAttentionSpec)
                 else (m.left.heads, m.left.kv_heads, m.left.dim, m.left.vdim, 0))
            if ops.window_mfma_supported(*k[:4], True):
                keys.add((k[0], k[1], k[4]))   # heads, key heads, chunk size (0: a window)
        return sorted(keys)

    def plan_batch(self, meta: BatchMeta, plan: dict, to_dev) -> None:
        """Sequences of the step for the kernels that walk them: decode rows (one row each), then the
        prefill chunks; every sequence with its state slot."""
        nd = plan["num_decode"]
        q_lens = [1] * nd + list(plan.get("q_lens", []))
        cu, seq = [0], []
        for i, n in enumerate(q_lens):
            cu.append(cu[-1] + n)
            seq.extend([i] * n)
        meta.seq_cu = to_dev(cu, torch.int32)
        meta.seq_state = to_dev(plan["state_slots"], torch.int32)
        meta.row_seq = to_dev(seq, torch.int32)
        cut = ops.build_scan_pieces(q_lens) if self.device.type == "cuda" else None
        if cut is not None:
            meta.scan_pieces = tuple(torch.from_numpy(a).pin_memory().to(self.device, non_blocking=True) for a in cut)
        if plan["num_prefill"]:
            meta.pre_row_seq = to_dev([s - nd for s in seq[nd:]], torch.int32)
            meta.pre_win_tiles = {}
            if self.device.type == "cuda" and self.dtype == torch.bfloat16:
                for key in self._tile_keys():
                    tiles = ops.build_window_tiles(plan["q_lens"], plan["pre_ctx"], *key)
                    meta.pre_win_tiles[key] = torch.from_numpy(tiles).pin_memory().to(self.device, non_blocking=True)

    def plan_decode_graph(self, meta: BatchMeta, bsz: int, state_slots: torch.Tensor) -> None:
        """The same for a captured decode step of ``bsz`` rows: ``state_slots`` is a graph input."""
        meta.seq_cu = torch.arange(bsz + 1, dtype=torch.int32, device=self.device)
        meta.seq_state = state_slots
        meta.row_seq = None

    # ------------------------------------------------------------------ mixers
    def _attend(self, q, pool, cache_off, heads, kv_heads, vdim, window, scale, meta: BatchMeta, chunk=0, **how):
        """The windowed-attention kernels over the decode rows and the prefill rows of the step:
        u fp32 [T, heads, vdim], each head on its own value head."""
        t, nd = q.shape[0], meta.num_decode
        u = torch.empty((t, heads, 1, vdim), dtype=torch.float32, device=q.device)
        if nd > 0:
            # the split count follows the batch rounded up to a power of two, which an eager step and the
            # captured step of its batch bucket share: both then sum in the same order
            reach = self.max_model_len if how.get("pool_block") else min(window, self.max_model_len)
            splits = ops.window_decode_splits(1 << (nd - 1).bit_length(), kv_heads, reach, 0, self.max_model_len)
            ops.window_attention(q[:nd], pool, cache_off, kv_heads, vdim, meta.dec_block_tables, None, meta.positions[:nd],
                                 window, 0, scale, 0.0, None, out=u[:nd], splits=splits, own_values=True, **how)
        if meta.num_prefill_seqs > 0:
            ops.window_attention(q[nd:], pool, cache_off, kv_heads, vdim, meta.pre_block_tables, meta.pre_row_seq,
                                 meta.positions[nd:], window, 0, scale, 0.0, None, out=u[nd:],
                                 tiles=(meta.pre_win_tiles or {}).get((heads, kv_heads, chunk)), own_values=True, **how)
        return u.view(t, heads, vdim)

    def _attention(self, lw: ZetalornLayer, proj: torch.Tensor, pool, cache_off: int, meta: BatchMeta) -> torch.Tensor:
        m: DiffAttentionSpec = lw.spec.mixer
        eps = self.cfg.norm_eps
        q = ops.qk_norm_write(proj, 2 * m.heads, 2 * m.kv_heads, m.dim, m.vdim, meta.positions, meta.slots, pool,
                              cache_off, eps, v_heads=m.kv_heads, q_weight=lw.q_norm, k_weight=lw.k_norm,
                              cos_sin=lw.cos_sin, rot_dims=m.rot.dims, layout=LAYOUTS[m.rot.layout])
        if m.chunk:
            u = self._attend(q, pool, cache_off, 2 * m.heads, 2 * m.kv_heads, m.vdim, m.chunk, m.scale, meta,
                             chunk=m.chunk, chunked=True, maps=2)
        else:
            u = self._attend(q, pool, cache_off, 2 * m.heads, 2 * m.kv_heads, m.vdim, 1 << 30, m.scale, meta, maps=2)
        y = ops.diff_heads(u, m.kv_heads, lw.lam, eps, 1.0 - m.diff, self.dtype)
        return ops.linear(y, lw.w_o)

    def _parallel(self, lw: ZetalornLayer, proj: torch.Tensor, pool, cache_off: int, state_off: int, meta: BatchMeta):
        m: ParallelMixerSpec = lw.spec.mixer
        a, r = m.left, m.right
        eps = self.cfg.norm_eps
        rows = self.in_rows(lw.spec)
        t, nd = proj.shape[0], meta.num_decode
        q = ops.qk_norm_write(proj, a.heads, a.kv_heads, a.dim, a.vdim, meta.positions, meta.slots, pool, cache_off, eps,
                              q_weight=lw.q_norm, k_weight=lw.k_norm, cos_sin=lw.cos_sin, rot_dims=a.rot.dims,
                              layout=LAYOUTS[a.rot.layout])
        how = {}
        if a.pool:
            region = ops.window_cache_elems(a.kv_heads, a.dim, a.vdim)
            how = {"pool_block": a.pool, "pool_off": region}
            if nd > 0:
                ops.pool_blocks(pool, cache_off, region, a.kv_heads, a.dim, a.vdim, meta.dec_block_tables, None,
                                meta.positions[:nd], meta.slots[:nd], a.pool)
            if meta.num_prefill_seqs > 0:
                ops.pool_blocks(pool, cache_off, region, a.kv_heads, a.dim, a.vdim, meta.pre_block_tables,
                                meta.pre_row_seq, meta.positions[nd:], meta.slots[nd:], a.pool)
        u = self._attend(q, pool, cache_off, a.heads, a.kv_heads, a.vdim, a.window, a.scale, meta, **how)
        left = ops.linear(ops.head_finish(u, eps, self.dtype, unit=False), lw.w_o)
        o = ops.recurrent_scan(proj, rows["right.q"][0], rows["right.k"][0], rows["right.v"][0], r.heads, r.dim, r.vdim,
                               self.state, state_off, meta.seq_cu, meta.seq_state, meta.positions, decay=lw.decay,
                               pieces=meta.scan_pieces, min_decay=min(r.decay), act=True)
        g0, g1 = rows["right.g"]
        y = ops.head_finish(o.view(t, 1, r.heads * r.vdim), eps, self.dtype, weight=lw.r_norm, gate=proj[:, g0:g1],
                            gate_act="sigmoid")
        right = ops.linear(y, lw.wr_o)
        return [(left, lw.left_out, m.left_scale), (right, lw.right_out, m.right_scale)]

    # ------------------------------------------------------------------ feed-forward
    def _moe(self, lw: ZetalornLayer, h: torch.Tensor) -> torch.Tensor:
        """The mixture's output for rows h, fp32."""
        f: FeedForwardSpec = lw.spec.mlp
        t = h.shape[0]
        logits = F.linear(h.float(), lw.router)  # a true fp32 product
        w, ids, _ = ops.group_topk(logits, f.experts, f.groups, f.keep, f.top, 1.0, normalize=f.norm_topk)
        out = torch.empty((t, h.shape[1]), dtype=torch.float32, device=h.device)
        if ops.moe_glu_grouped_supported(h, lw.w13, lw.w2):
            ys, pos = ops.moe_glu_grouped(h, lw.w13, lw.w2, ids, f.limit, GLU_ALPHA, GLU_UP_BIAS)
            return ops.moe_finish(out, ys, w, pos, overwrite=True)
        # the CPU, fp32, and shapes the grouped kernel does not tile: unit by unit on the sorted rows
        offsets, pos, sorted_tok = ops.moe_align(ids, f.experts)
        xs = ops.gather_rows(h, sorted_tok)
        ys = torch.empty((t * f.top, h.shape[1]), dtype=h.dtype, device=h.device)
        off = offsets.tolist()
        for e in range(f.experts):
            a, b = off[e], off[e + 1]
            if b > a:
                act = ops.glu_clamp(F.linear(xs[a:b], lw.w13[e]), f.limit, GLU_ALPHA, GLU_UP_BIAS)
                torch.matmul(act, lw.w2[e].t(), out=ys[a:b])
        return ops.moe_finish(out, ys, w, pos, overwrite=True)

    # ------------------------------------------------------------------ forward
    def _norm(self, x, pending: Pending | None, weight, **extras):
        if pending is None:
            return ops.gated_add_rms_norm(x, [], None, None, weight, self.cfg.norm_eps, self.dtype, **extras)
        return ops.gated_add_rms_norm(x, pending.deltas, pending.gate, pending.bias, weight, self.cfg.norm_eps, self.dtype,
                                      **extras)

    def forward(self, input_ids: torch.Tensor, pool: torch.Tensor, meta: BatchMeta) -> torch.Tensor:
        """Final-normed hidden states of ``meta.logits_rows`` ([num_out, width], activation dtype)."""
        x = ops.embed_scale(input_ids, self.embed, 1.0)  # fp32 residual stream
        looped = self.cfg.layer_loop is not None
        emb = x.clone() if looped and self.cfg.layer_loop[2] > 1 else None
        pending: Pending | None = None
        for run, (li, pass_no) in enumerate(self.runs):
            lw = self.layers[li]
            extras = {}
            if pass_no is not None:  # the run starts a pass of the loop
                extras = {"extra": emb if pass_no > 0 else None, "extra_vec": self.loop_step[pass_no]}
            h = self._norm(x, pending, lw.norm1, **extras)
            proj = ops.linear(h, lw.w_in)  # the mixer's projections | residual-gate logits
            g0, g1 = self.in_rows(lw.spec)["rg1"]
            if lw.spec.type == "attention":
                deltas = [(self._attention(lw, proj, pool, self.cache_offsets[run], meta), None, 1.0)]
            else:
                deltas = self._parallel(lw, proj, pool, self.cache_offsets[run], self.state_offsets[run], meta)
            pending = Pending(deltas, proj[:, g0:g1], lw.rg1_b)
            if lw.spec.mlp is not None:
                h = self._norm(x, pending, lw.norm2)
                pending = Pending([(self._moe(lw, h), None, 1.0)], ops.linear(h, lw.rg2), lw.rg2_b)
            if self.layer_probe is not None:
                self._norm(x, pending, None, want_out=False)
                pending = None
                self.layer_probe(run, x)
        if meta.logits_rows is not None:
            x = x.index_select(0, meta.logits_rows)
            pending = None if pending is None else pending.rows(meta.logits_rows)
        return self._norm(x, pending, self.norm)

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        logits = ops.linear(hidden, self.lm_head)
        if self.cfg.logit_scale != 1.0:
            logits = logits.float() * self.cfg.logit_scale
        return logits
