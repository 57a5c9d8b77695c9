"""Pelatar: a decoder whose layers, listed one by one in the configuration, put their norm on the
sublayer's OUTPUT: ``x += norm1(mixer(x))``, then ``x += norm2(ff(x))`` (RMS norms).  The residual
stream is fp32; a sublayer reads the stream itself (rounded to the activation dtype for its projections,
as it is for the routers' and gates' fp32 products).

Mixers:

- ``attention``: grouped-query softmax attention without rotation.  q | k | v | gate logits come from one
  fused projection; q and k heads are brought to unit root mean square (no weight), q grows with the
  logarithm of the position, k and v go to the paged pool, a per-head sink logit joins the softmax
  denominator, the heads are gated by sigmoid(W_g h).  A layer with ``kv_from`` projects q and gate logits only
  and reads the pool entries of the layer it names.
- ``mlstm``: a matrix memory with exponential input / forget gates and a running maximum of their logarithms.
  The gates' pre-activations are a true fp32 product; the gate kernel turns them into one decay and one write
  strength per token and head (the maximum is carried in the sequence's state slot), and the recurrence kernel
  of the other linear-attention mixers runs over these prepared rows with one more value column of ones, whose
  read-out is the normaliser's dot product.
- ``gla``: linear attention with a decay per key channel from a low-rank pair of projections (the first of them
  fused into the input projection).

Feed-forwards: a dense gated unit with the tanh form of gelu, or a mixture of silu gated units routed by
softmax scores with a selection bias, group-limited, with identity experts (their output is the token
itself) that never reach the expert products.

Attention layers that own keys and values share the pool's pages (layer after layer inside a page); the
recurrences live in the per-sequence state slot.  A chunk that starts at position 0 starts from zero state,
so slots need no clearing.  Logits come from the embedding table.
"""

from __future__ import annotations

import torch
import torch.nn.functional as F

from .. import ops
from ..engine.config import FeedForwardSpec, GatedLinearSpec, MatrixMemorySpec, ModelConfig, NormedAttentionSpec
from ..ops.reference import PAGE
from ..parallel.state import get_pp, get_tp
from .batch import BatchMeta

NO_WINDOW = 1 << 30   # the windowed-attention kernels with a window no context reaches: plain causal attention


class PelatarLayer:
    __slots__ = ("spec", "norm1", "norm2", "w_in", "w_o", "sink", "w_if", "b_i", "b_f", "h_norm", "w_a2", "a2_b",
                 "w_gu", "w_down", "router", "correction", "w13", "w2", "cache_off", "state_off", "m_off")

    def __init__(self, spec):
        for s in self.__slots__:
            setattr(self, s, None)
        self.spec = spec


class PelatarModel:
    def __init__(self, cfg: ModelConfig, dtype: torch.dtype, device: torch.device, max_model_len: int):
        if get_tp().size != 1 or get_pp().size != 1:
            raise ValueError("Pelatar runs on single-GPU replicas (no tensor / pipeline parallel layout yet)")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Pelatar runs in bfloat16 or float32")
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
        self.layers: list[PelatarLayer] = []
        self.embed = self.norm = None
        self.state: torch.Tensor | None = None  # [slots, state_elems] fp32, bound by the runner
        self.layer_probe = None  # callable(layer index, fp32 residual stream after the layer) for tests
        # where each layer's part of a pool page and of a state slot starts, in elements
        self.cache_offsets: dict[int, int] = {}
        self.state_offsets: dict[int, tuple] = {}
        c_off = s_off = 0

        def up4(n):  # parts of a slot start on 16-byte boundaries (the kernels then move whole float4)
            return (n + 3) // 4 * 4

        for i, s in enumerate(self.specs):
            m = s.mixer
            if isinstance(m, NormedAttentionSpec):
                if m.kv_from is None:
                    self.cache_offsets[i] = c_off
                    c_off += PAGE * m.cache_elems()
            elif isinstance(m, MatrixMemorySpec):
                cols = ops.scan_state_cols(m.vdim, True)
                self.state_offsets[i] = (s_off, s_off + m.heads * m.dim * cols)  # the matrix, then the running maxima
                s_off += m.heads * m.dim * cols + up4(m.heads)
            else:
                self.state_offsets[i] = (s_off, None)
                s_off += up4(m.heads * m.dim * m.vdim)
        self.page_elems = max(c_off, 8)   # a model of recurrences only still names (empty) pages
        self.state_elems = max(s_off, 8)

    @property
    def graph_capturable(self) -> bool:
        """Decode steps can be captured when no layer's mixture falls back to the per-unit loop, which reads
        the row counts on the host (shapes the grouped GEMMs do not tile, fp32)."""
        return self.dtype == torch.bfloat16 and self.device.type == "cuda" and all(
            lw.w13 is None or self._grouped(lw) for lw in self.layers)

    # ------------------------------------------------------------------ stores
    def kv_page_shape(self) -> tuple:
        """Shape of one page of the KV pool (the runner allocates [pages, *shape])."""
        return (self.page_elems,)

    def state_shape(self) -> tuple:
        """Shape of one sequence's state slot (the runner allocates fp32 [slots, *shape])."""
        return (self.state_elems,)

    def bind_state(self, state: torch.Tensor | None) -> None:
        self.state = state

    # ------------------------------------------------------------------ weights
    def _alloc(self, gen, *shape, std=None, dtype=None, mean=0.0):
        dtype = dtype or self.dtype
        t = torch.empty(shape, dtype=torch.float32, device=self.device)
        t.normal_(mean, std if std is not None else shape[-1] ** -0.5, generator=gen)
        return t.to(dtype)

    def init_random(self, seed: int = 0) -> None:
        """Allocates every tensor in the layout the forward pass uses; a checkpoint overwrites them."""
        cfg = self.cfg
        w = cfg.hidden_size
        g = torch.Generator(device=self.device).manual_seed(seed)
        f32 = torch.float32
        self.embed = self._alloc(g, cfg.vocab_size, w, std=1.0)
        self.layers = []
        for i, s in enumerate(self.specs):
            m, f = s.mixer, s.mlp
            lw = PelatarLayer(s)
            lw.norm1 = self._alloc(g, w, std=0.1, dtype=f32, mean=1.0)
            hv = m.heads * m.vdim
            if isinstance(m, NormedAttentionSpec):
                own = m.kv_from is None
                lw.w_in = self._alloc(g, m.heads * m.dim + (m.kv_heads * (m.dim + m.vdim) if own else 0) + hv, w)
                lw.sink = self._alloc(g, m.heads, std=1.0, dtype=f32)
                lw.cache_off = self.cache_offsets[i if own else m.kv_from]
            elif isinstance(m, MatrixMemorySpec):
                lw.w_in = self._alloc(g, 2 * m.heads * m.dim + 2 * hv, w)
                lw.w_if = self._alloc(g, 2 * m.heads, w, dtype=f32)
                lw.b_i = self._alloc(g, m.heads, std=1.0, dtype=f32)
                lw.b_f = self._alloc(g, m.heads, std=1.0, dtype=f32, mean=2.0)
                lw.h_norm = self._alloc(g, hv, std=0.1, dtype=f32, mean=1.0)
                lw.state_off, lw.m_off = self.state_offsets[i]
            else:
                self.set_decay_rank(lw, m.decay_rank, g)
                lw.a2_b = self._alloc(g, m.heads * m.dim, std=1.0, dtype=f32, mean=2.0)
                lw.h_norm = self._alloc(g, m.vdim, std=0.1, dtype=f32, mean=1.0)
                lw.state_off = self.state_offsets[i][0]
            lw.w_o = self._alloc(g, w, hv)
            if f is not None:
                lw.norm2 = self._alloc(g, w, std=0.1, dtype=f32, mean=1.0)
                if f.kind == "dense":
                    lw.w_gu = self._alloc(g, 2 * f.ff, w)
                    lw.w_down = self._alloc(g, w, f.ff)
                else:
                    n = f.experts + f.identity
                    lw.router = self._alloc(g, n, w, dtype=f32)
                    lw.correction = self._alloc(g, n, std=0.02, dtype=f32)
                    lw.w13 = self._alloc(g, f.experts, 2 * f.ff, w)
                    lw.w2 = self._alloc(g, f.experts, w, f.ff)
            self.layers.append(lw)
        self.norm = self._alloc(g, w, std=0.1, dtype=f32, mean=1.0)

    def set_decay_rank(self, lw: PelatarLayer, rank: int, gen=None) -> None:
        """(Re)allocates a gla layer's input projection q | k | v | gate | decay-down and its decay-up matrix
        for a low-rank decay of ``rank`` (a checkpoint's tensors decide the rank)."""
        m: GatedLinearSpec = lw.spec.mixer
        gen = gen or torch.Generator(device=self.device).manual_seed(0)
        w = self.cfg.hidden_size
        lw.w_in = self._alloc(gen, 2 * m.heads * m.dim + 2 * m.heads * m.vdim + rank, w)
        lw.w_a2 = self._alloc(gen, m.heads * m.dim, rank)

    @property
    def lm_head(self) -> torch.Tensor:  # the embedding table is the output matrix
        return self.embed

    def weight_tensors(self):
        for t in (self.embed, self.norm):
            if t is not None:
                yield t
        for lw in self.layers:
            for s in PelatarLayer.__slots__:
                t = getattr(lw, s)
                if isinstance(t, torch.Tensor):
                    yield t

    def weight_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.weight_tensors())

    # ------------------------------------------------------------------ batch description
    def _tile_keys(self):
        return sorted({(s.mixer.heads, s.mixer.kv_heads) for s in self.specs
                       if isinstance(s.mixer, NormedAttentionSpec)
                       and ops.window_mfma_supported(s.mixer.heads, s.mixer.kv_heads, s.mixer.dim, s.mixer.vdim, True)})

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
    def _attention(self, lw: PelatarLayer, h: torch.Tensor, pool, meta: BatchMeta) -> torch.Tensor:
        m: NormedAttentionSpec = lw.spec.mixer
        own = m.kv_from is None
        proj = ops.linear(h, lw.w_in)  # q | k | v | gate logits (q | gate logits when the entries are another layer's)
        q = ops.qk_norm_write(proj, m.heads, m.kv_heads, m.dim, m.vdim, meta.positions, meta.slots, pool, lw.cache_off,
                              self.cfg.norm_eps, m.temp_coef, m.temp_every, own)
        t, nd = h.shape[0], meta.num_decode
        u = torch.empty((t, m.heads, 1, m.vdim), dtype=torch.float32, device=h.device)
        if nd > 0:
            # the split count follows the batch rounded up to a power of two, which an eager step and the
            # captured step of its batch bucket share: both then sum in the same order
            splits = ops.window_decode_splits(1 << (nd - 1).bit_length(), m.kv_heads, NO_WINDOW, 0, self.max_model_len)
            ops.window_attention(q[:nd], pool, lw.cache_off, m.kv_heads, m.vdim, meta.dec_block_tables, None,
                                 meta.positions[:nd], NO_WINDOW, 0, m.scale, 0.0, lw.sink, out=u[:nd], splits=splits,
                                 own_values=True)
        if meta.num_prefill_seqs > 0:
            ops.window_attention(q[nd:], pool, lw.cache_off, m.kv_heads, m.vdim, meta.pre_block_tables,
                                 meta.pre_row_seq, meta.positions[nd:], NO_WINDOW, 0, m.scale, 0.0, lw.sink, out=u[nd:],
                                 tiles=(meta.pre_win_tiles or {}).get((m.heads, m.kv_heads)), own_values=True)
        g0 = lw.w_in.shape[0] - m.heads * m.vdim
        y = ops.head_finish(u.view(t, m.heads, m.vdim), self.cfg.norm_eps, self.dtype, unit=False,
                            gate=proj[:, g0:], gate_act="sigmoid")
        return ops.linear(y, lw.w_o)

    def _mlstm(self, lw: PelatarLayer, x: torch.Tensor, h: torch.Tensor, meta: BatchMeta) -> torch.Tensor:
        m: MatrixMemorySpec = lw.spec.mixer
        hd, hv = m.heads * m.dim, m.heads * m.vdim
        proj = ops.linear(h, lw.w_in)  # q | k | v | gate logits
        gates = F.linear(x, lw.w_if)   # input | forget pre-activations: a true fp32 product of the stream
        prep, top = ops.mlstm_prepare(proj, 0, hd, gates, lw.b_i, lw.b_f, m.gate_cap, m.heads, m.dim, m.dim ** -0.5,
                                      self.state, lw.m_off, meta.seq_cu, meta.seq_state, meta.positions)
        o = ops.prepared_scan(prep, proj, 2 * hd, m.heads, m.dim, m.vdim, self.state, lw.state_off, meta.seq_cu,
                              meta.seq_state, meta.positions, unit_col=True, pieces=meta.scan_pieces)
        y = ops.head_finish(o, self.cfg.norm_eps, self.dtype, vdim=m.vdim, stab=top, weight=lw.h_norm,
                            gate=proj[:, 2 * hd + hv:2 * hd + 2 * hv], gate_act="sigmoid")
        return ops.linear(y, lw.w_o)

    def _gla(self, lw: PelatarLayer, h: torch.Tensor, meta: BatchMeta) -> torch.Tensor:
        m: GatedLinearSpec = lw.spec.mixer
        hd, hv = m.heads * m.dim, m.heads * m.vdim
        proj = ops.linear(h, lw.w_in)  # q | k | v | gate logits | decay-down
        z = ops.linear(proj[:, 2 * hd + 2 * hv:].contiguous(), lw.w_a2)
        prep = ops.gla_prepare(proj, 0, hd, z, lw.a2_b, m.heads, m.dim, m.dim ** -0.5, m.tau)
        o = ops.prepared_scan(prep, proj, 2 * hd, m.heads, m.dim, m.vdim, self.state, lw.state_off, meta.seq_cu,
                              meta.seq_state, meta.positions, pieces=meta.scan_pieces)
        y = ops.head_finish(o, self.cfg.norm_eps, self.dtype, weight=lw.h_norm, gate=proj[:, 2 * hd + hv:2 * hd + 2 * hv],
                            gate_act="silu")
        return ops.linear(y, lw.w_o)

    # ------------------------------------------------------------------ feed-forwards
    def _grouped(self, lw: PelatarLayer) -> bool:
        """Do the grouped matrix-core GEMMs take this layer's units?"""
        return (self.device.type == "cuda" and self.dtype == torch.bfloat16
                and ops.grouped_gemm_supported(lw.w13.shape[1], lw.w13.shape[2], True)
                and ops.grouped_gemm_supported(lw.w2.shape[1], lw.w2.shape[2]))

    def _moe(self, lw: PelatarLayer, x: torch.Tensor, h: torch.Tensor) -> torch.Tensor:
        """The mixture's output for rows h, fp32."""
        f: FeedForwardSpec = lw.spec.mlp
        t, width = h.shape
        logits = F.linear(x, lw.router)  # a true fp32 product of the stream
        w, ids, gate = ops.route_softmax(logits, f.experts + f.identity, f.experts, f.groups, f.keep, f.top,
                                         lw.correction, 1.0, park_in_bucket=True)
        out = torch.zeros((t, width), dtype=torch.float32, device=h.device)
        bucket = f.identity > 0
        if self._grouped(lw):
            if t <= ops.MOE_MFMA_MAX_TOKENS and ops.moe_mfma_supported(width, f.ff):
                ys, pos = ops.moe_experts_grouped(h, lw.w13, lw.w2, ids, w, foreign=bucket, combine=False)
            else:
                ys, pos = ops.moe_experts_prefill(h, lw.w13, lw.w2, ids, w, foreign=bucket, combine=False)
        else:
            # the CPU, fp32, and shapes the grouped kernels do not tile: unit by unit on the sorted rows
            offsets, pos, sorted_tok = ops.moe_align(ids, f.experts + (1 if bucket else 0))
            xs = ops.gather_rows(h, sorted_tok)
            ys = torch.empty((t * f.top, width), dtype=h.dtype, device=h.device)
            off = offsets.tolist()
            for e in range(f.experts):
                a, b = off[e], off[e + 1]
                if b > a:
                    torch.matmul(ops.glu_act(F.linear(xs[a:b], lw.w13[e]), f.act), lw.w2[e].t(), out=ys[a:b])
        return ops.moe_finish(out, ys, w, pos, h if gate is not None else None, gate)

    # ------------------------------------------------------------------ forward
    def forward(self, input_ids: torch.Tensor, pool: torch.Tensor, meta: BatchMeta) -> torch.Tensor:
        """Final-normed hidden states of ``meta.logits_rows`` ([num_out, width], activation dtype)."""
        eps = self.cfg.norm_eps
        x = ops.embed_scale(input_ids, self.embed, 1.0)  # fp32 residual stream
        h = x if self.dtype == torch.float32 else x.to(self.dtype)
        for i, lw in enumerate(self.layers):
            kind = lw.spec.type
            if kind == "attention":
                y = self._attention(lw, h, pool, meta)
            elif kind == "mlstm":
                y = self._mlstm(lw, x, h, meta)
            else:
                y = self._gla(lw, h, meta)
            h = ops.rms_norm_add(x, y, lw.norm1, eps, self.dtype)
            f = lw.spec.mlp
            if f is not None:
                if f.kind == "dense":
                    y = ops.linear(ops.gate_up_act(h, lw.w_gu, f.act), lw.w_down)
                else:
                    y = self._moe(lw, x, h)
                h = ops.rms_norm_add(x, y, lw.norm2, eps, self.dtype)
            if self.layer_probe is not None:
                self.layer_probe(i, x)
        if meta.logits_rows is not None:
            x = x.index_select(0, meta.logits_rows)
        return ops.add_rms_norm(x, None, self.norm, eps, self.dtype)

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        return ops.linear(hidden, self.embed)
