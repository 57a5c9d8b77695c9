"""Cases for Pelatar: every op against its float64 definition, and the engine on small random checkpoints
against the float64 oracle.  The CPU and the GPU test files call them with their device, dtype and tolerance."""

from __future__ import annotations

import math
import tempfile

import torch

import pelatar_oracle as po
from vllm_production_stack_amd import ops
from vllm_production_stack_amd.engine.config import EngineConfig
from vllm_production_stack_amd.engine.llm_engine import LLMEngine
from vllm_production_stack_amd.engine.request import SamplingParams
from vllm_production_stack_amd.ops import reference

PAGE = 64
F64 = torch.float64
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}
NO_WINDOW = 1 << 30


def close(got, want, tol, what=""):
    err = (got.double().cpu() - want).abs().max().item()
    lim = tol * max(1.0, want.abs().max().item())
    assert err <= lim, f"{what}: off by {err:.3g} (allowed {lim:.3g})"


def i32(x, dev):
    return torch.tensor(x, dtype=torch.int32, device=dev)


# ----------------------------------------------------------------------------- configurations
def config_a():
    """Every kind of layer and feed-forward, sizes that differ from one another wherever they can, a layer that
    reads its neighbour's keys and values, identity experts, two groups of which one is kept."""
    return po.make_config([
        po.mlstm_layer(heads=2, dim=8, vdim=12, cap=12.0, mlp=po.dense(40)),
        po.gla_layer(heads=2, dim=12, vdim=8, tau=8.0, rank=4, mlp=po.moe(24, 6, 3, groups=2, keep=1, identity=2)),
        po.attention_layer(heads=4, kv_heads=2, dim=12, vdim=20, every=16, mlp=po.dense(32)),
        po.attention_layer(heads=4, kv_heads=2, dim=12, vdim=20, every=16, kv_from=2, mlp=po.moe(16, 4, 2)),
    ], vocab=70, width=32)


def config_b():
    """Other corners: attention first and read two layers later, one KV head per query head and a single KV head,
    a single recurrent head, value sizes that are no multiple of 4, top 1, groups of one expert, all groups kept,
    no temperature in one layer, a period of one position in another, layers without a feed-forward, eps 1e-3."""
    return po.make_config([
        po.attention_layer(heads=3, kv_heads=3, dim=8, vdim=10, coef=0.0, scale=0.7, mlp=po.moe(16, 3, 1, groups=4, keep=2, identity=1)),
        po.gla_layer(heads=1, dim=20, vdim=6, tau=4.0, rank=3),
        po.attention_layer(heads=3, kv_heads=3, dim=8, vdim=10, coef=0.25, every=1, scale=0.2, kv_from=0),
        po.mlstm_layer(heads=1, dim=24, vdim=10, cap=6.0),
        po.attention_layer(heads=4, kv_heads=1, dim=16, vdim=8, coef=1.5, every=70, mlp=po.moe(8, 5, 2, groups=1, keep=1)),
    ], vocab=50, width=24, eps=1e-3)


def config_c():
    """Head sizes the matrix-core attention kernel tiles, unit sizes the grouped GEMMs tile, chunks long enough to be
    cut into pieces by the recurrence kernels."""
    return po.make_config([
        po.mlstm_layer(heads=2, dim=32, vdim=64, mlp=po.dense(128)),
        po.attention_layer(heads=4, kv_heads=2, dim=64, vdim=128, every=100, mlp=po.moe(64, 6, 2, groups=2, keep=1, identity=2)),
        po.gla_layer(heads=2, dim=64, vdim=32, rank=16, mlp=po.dense(128)),
        po.attention_layer(heads=4, kv_heads=2, dim=64, vdim=128, every=100, kv_from=1, mlp=po.moe(64, 4, 2)),
    ], vocab=200, width=128)


def config_d():
    """Recurrences only (the pool's pages stay empty), no feed-forward anywhere."""
    return po.make_config([po.gla_layer(heads=2, dim=8, vdim=10, rank=2), po.mlstm_layer(heads=3, dim=8, vdim=6, cap=30.0)],
                          vocab=40, width=24)


def config_e():
    """Unit widths the decode-sized matrix-core mixture kernels stream (with identity experts parked behind the last
    unit), beside a mixture without identity experts."""
    return po.make_config([
        po.gla_layer(heads=1, dim=32, vdim=32, rank=4, mlp=po.moe(512, 4, 2, groups=2, keep=1, identity=2)),
        po.attention_layer(heads=2, kv_heads=1, dim=64, vdim=128, every=9, mlp=po.moe(512, 3, 2)),
    ], vocab=120, width=128)


def config_f():
    """Sizes that are multiples of nothing: odd head sizes, a width and a vocabulary that are no multiple of 8."""
    return po.make_config([
        po.attention_layer(heads=6, kv_heads=2, dim=6, vdim=5, every=7, mlp=po.moe(9, 5, 2, groups=2, keep=2, identity=1)),
        po.mlstm_layer(heads=3, dim=5, vdim=7, cap=10.0, mlp=po.dense(13)),
        po.gla_layer(heads=2, dim=7, vdim=3, tau=2.0, rank=1),
        po.attention_layer(heads=6, kv_heads=2, dim=6, vdim=5, coef=0.3, every=2.5, kv_from=0, mlp=po.dense(11)),
    ], vocab=45, width=20)


# ----------------------------------------------------------------------------- mechanisms
def case_norm_on_output(dev, dtype, tol):
    dt = DTYPES[dtype]
    g = torch.Generator().manual_seed(0)
    for n in (5, 48, 300):
        res = torch.randn(7, n, generator=g) * 2
        w = torch.rand(n, generator=g) + 0.5
        for delta in ((torch.randn(7, n, generator=g) * 3).to(dt), torch.randn(7, n, generator=g) * 1e-3):  # in dtype, in fp32
            r = res.clone().to(dev)
            y = ops.rms_norm_add(r, delta.to(dev), w.to(dev), 1e-5, dt)
            want = res.double() + po.unit_rms(delta.double(), 1e-5) * w.double()
            close(r, want, 1e-6, "stream")
            close(y, want, tol, "rounded stream")
    z = torch.zeros(3, 16)  # a sublayer that returns nothing adds nothing (eps keeps the root away from zero)
    r = torch.ones(3, 16, device=dev)
    ops.rms_norm_add(r, z.to(dt).to(dev), torch.ones(16, device=dev), 1e-5, dt)
    close(r, torch.ones(3, 16, dtype=F64), 1e-7, "zero delta")


def case_gated_units(dev, dtype, tol):
    dt = DTYPES[dtype]
    g = torch.Generator().manual_seed(1)
    x = (torch.randn(9, 2 * 37, generator=g) * 3).to(dt)
    gate, up = x[:, :37].double(), x[:, 37:].double()
    close(ops.glu_act(x.to(dev), "gelu_tanh"), po.gelu_tanh(gate) * up, tol, "gelu gate")
    close(ops.glu_act(x.to(dev), "silu"), po.silu(gate) * up, tol, "silu gate")
    w = (torch.randn(2 * 24, 40, generator=g) * 0.2).to(dt)
    h = torch.randn(5, 40, generator=g).to(dt)
    want = po.gelu_tanh(h.double() @ w[:24].double().T) * (h.double() @ w[24:].double().T)
    close(ops.gate_up_act(h.to(dev), w.to(dev), "gelu_tanh"), want, max(tol, 2e-2 if dt == torch.bfloat16 else 0), "fused projection")
    if dt == torch.bfloat16 and torch.device(dev).type == "cuda":  # the same unit in the prefill GEMM's epilogue
        w = (torch.randn(2 * 96, 128, generator=g) * 0.3).to(dt)
        h = torch.randn(300, 128, generator=g).to(dt)
        want = po.gelu_tanh(h.double() @ w[:96].double().T) * (h.double() @ w[96:].double().T)
        close(ops.tile_gemm(h.to(dev), w.to(dev), gelu_mul=True), want, 2e-2, "epilogue of the prefill GEMM")


def case_routing(dev):
    """Softmax scores, a bias that only selects (and makes choice scores negative), groups scored by their best
    member, identity experts that leave the pair list."""
    g = torch.Generator().manual_seed(2)
    for n, experts, groups, keep, top in ((8, 6, 2, 1, 3), (18, 15, 3, 1, 4), (12, 12, 4, 2, 3), (5, 5, 1, 1, 1), (6, 3, 6, 3, 2),
                                          (9, 4, 3, 3, 9)):
        logits = torch.randn(33, n + 2, generator=g) * 3
        bias = torch.randn(n, generator=g) * 0.3 - 0.4          # most choice scores are below zero
        ids, wts = po.choose(logits[:, :n].double(), bias.double(), groups, keep, top)
        for park in (True, False):
            w, got, gate = ops.route_softmax(logits.to(dev), n, experts, groups, keep, top, bias.to(dev), 1.0, park)
            w, got = w.cpu(), got.cpu().long()
            ident = ids >= experts
            assert torch.equal(torch.where(ident, torch.full_like(ids, experts if park else 0), ids), got)
            close(w, torch.where(ident, torch.zeros_like(wts), wts), 1e-6, "weights")
            if experts < n:
                close(gate, torch.where(ident, wts, torch.zeros_like(wts)).sum(-1), 1e-6, "identity gate")
            else:
                assert gate is None
    # an output outside the kept group is never chosen, however large its own score
    logits = torch.tensor([[0.0, 0.1, 9.0, -9.0]])
    bias = torch.tensor([0.0, 0.0, -5.0, 6.0])  # group 1 = {2, 3}: its best biased score (output 3) wins the group
    w, ids, _ = ops.route_softmax(logits.to(dev), 4, 4, 2, 1, 2, bias.to(dev))
    assert sorted(ids.cpu().tolist()[0]) == [2, 3]
    close(w.cpu().sort().values, torch.softmax(logits.double(), -1)[0, [3, 2]][None], 1e-6, "weights are the unbiased scores")


def case_qk_norm(dev, dtype, tol):
    """Unit RMS of q and k heads, the temperature at the edges of its steps, cache entries, rows that are not cached."""
    dt = DTYPES[dtype]
    g = torch.Generator().manual_seed(3)
    for heads, kv_heads, dim, vdim, coef, every, eps in ((4, 2, 12, 20, 0.4, 16, 1e-5), (3, 3, 8, 10, 0.0, 1, 1e-3),
                                                         (2, 1, 70, 6, 1.5, 3, 1e-5), (4, 1, 64, 128, 0.25, 1, 1e-6)):
        pos = [0, 1, every - 2, every - 1, every, 2 * every - 2, 2 * every - 1, 100, 127, 128]
        pos = sorted({p for p in pos if p >= 0})
        t = len(pos)
        chans = heads * dim + kv_heads * (dim + vdim)
        proj = (torch.randn(t, chans + 7, generator=g) * 2).to(dt)
        pool = torch.zeros(4, 16 + ops.window_cache_elems(kv_heads, dim, vdim), dtype=dt, device=dev)
        pages = [3, 1, 2]
        slots = [pages[p // PAGE] * PAGE + p % PAGE for p in pos]
        slots[1] = -1                                                   # a row that is not cached
        q = ops.qk_norm_write(proj.to(dev), heads, kv_heads, dim, vdim, i32(pos, dev),
                              torch.tensor(slots, dtype=torch.int64, device=dev), pool, 16, eps, coef, float(every))
        nq, nk = heads * dim, kv_heads * dim
        temp = po.temperature(pos, {"coef": coef, "every": every} if coef else None)
        close(q, po.unit_rms(proj[:, :nq].double().view(t, heads, dim), eps) * temp[:, None, None], tol, "q")
        kc, vc = reference.window_cache_views(pool.cpu(), 16, kv_heads, dim, vdim)
        want_k = po.unit_rms(proj[:, nq:nq + nk].double().view(t, kv_heads, dim), eps)
        for r, p in enumerate(pos):
            pg = pages[p // PAGE]
            if slots[r] < 0:
                assert kc[pg, p % PAGE].abs().max() == 0 and vc[pg, p % PAGE].abs().max() == 0
                continue
            close(kc[pg, p % PAGE], want_k[r], tol, "cached k")
            close(vc[pg, p % PAGE], proj[r, nq + nk:nq + nk + kv_heads * vdim].double().view(kv_heads, vdim), 1e-6, "cached v")
        # a layer that reads another layer's entries projects q only and writes nothing
        pool2 = torch.zeros_like(pool)
        q2 = ops.qk_norm_write(proj[:, :nq + 3].contiguous().to(dev), heads, kv_heads, dim, vdim, i32(pos, dev),
                               torch.tensor(slots, dtype=torch.int64, device=dev), pool2, 16, eps, coef, float(every), own=False)
        close(q2, q.double().cpu(), 1e-6, "q alone")
        assert pool2.abs().max() == 0


def _fill_cache(dev, dt, k, v, order, n_pages, off):
    """Keys / values of one sequence into pages ``order`` of a pool of ``n_pages``."""
    n, kv_heads, dim = k.shape
    vdim = v.shape[2]
    pool = torch.zeros(n_pages, off + ops.window_cache_elems(kv_heads, dim, vdim), dtype=dt)
    kc, vc = reference.window_cache_views(pool, off, kv_heads, dim, vdim)
    idx = torch.arange(n)
    pg = torch.tensor(order)[idx // PAGE]
    kc[pg, idx % PAGE] = k.to(dt)
    vc[pg, idx % PAGE] = v.to(dt)
    return pool.to(dev)


def case_attention(dev, dtype, tol, shapes=None):
    """Plain causal attention through the windowed-attention kernels with each head on its own KV head's values:
    one score made to stand out per row (a far key, a page's first and last key, the row itself, key 0), sinks from
    negligible to dominant, prefill rows (tiles and plain) and decode rows (whole and in key ranges)."""
    dt = DTYPES[dtype]
    g = torch.Generator().manual_seed(4)
    for heads, kv_heads, dim, vdim in shapes or ((4, 2, 12, 20), (3, 3, 8, 10), (4, 1, 16, 6)):
        rep = heads // kv_heads
        n_keys = 300
        k = po.unit_rms(torch.randn(n_keys, kv_heads, dim, generator=g).double(), 1e-5).to(dt)
        v = torch.randn(n_keys, kv_heads, vdim, generator=g).to(dt)
        order = [5, 2, 7, 0, 3]
        pool = _fill_cache(dev, dt, k, v, order, 8, 32)
        bt = i32([[1, 1, 1, 1, 1], order], dev)
        sink = torch.tensor([-30.0, 0.0, 2.0, 9.0][:heads] + [0.5] * max(0, heads - 4))
        scale = 0.3
        chunks = [(150, 50), (255, 45)]       # (first position, rows) of two portions of sequence 1
        pos_q, seqs = [], []
        for p0, n in chunks:
            pos_q += list(range(p0, p0 + n))
            seqs += [1] * n
        t = len(pos_q)
        q = torch.randn(t, heads, dim, generator=g) * 0.3
        for r, p in enumerate(pos_q):
            cand = [j for j in (p, p - 1, 0, 1, 63, 64, 127, 128, 191, 192, p - 100, p // 2) if 0 <= j <= p]
            j = cand[r % len(cand)]
            q[r] += 25.0 * k[j, torch.arange(heads) // rep].float()
        q = q.to(dt)
        want = po.sink_softmax_attention(q.double(), k.double(), v.double(), pos_q, range(n_keys), rep, scale, sink.double())
        args = (pool, 32, kv_heads, vdim)
        plain = ops.window_attention(q.to(dev), *args, bt, i32(seqs, dev), i32(pos_q, dev), NO_WINDOW, 0, scale, 0.0,
                                     sink.to(dev), own_values=True)
        assert plain.shape == (t, heads, 1, vdim)
        close(plain.view(t, heads, vdim), want, tol, "prefill rows, plain kernel")
        tiles = torch.from_numpy(ops.build_window_tiles([n for _, n in chunks], [p0 + n for p0, n in chunks], heads,
                                                        kv_heads)).to(dev)
        tiles[:, 0] = 1
        u = ops.window_attention(q.to(dev), *args, bt, i32(seqs, dev), i32(pos_q, dev), NO_WINDOW, 0, scale, 0.0,
                                 sink.to(dev), tiles=tiles, own_values=True)
        close(u.view(t, heads, vdim), want, tol, "prefill rows, tiles")
        rows = list(range(0, t, 6))
        for splits in (1, 2, 5):
            u = ops.window_attention(q[rows].to(dev), *args, i32([order] * len(rows), dev), None,
                                     i32([pos_q[r] for r in rows], dev), NO_WINDOW, 0, scale, 0.0, sink.to(dev),
                                     splits=splits, own_values=True)
            close(u.view(len(rows), heads, vdim), want[rows], tol, f"decode rows in {splits} key ranges")
        # the sink alone: a head whose sink dwarfs every score returns almost nothing
        big = torch.full((heads,), 2000.0)
        u = ops.window_attention(q[:4].to(dev), *args, bt, i32(seqs[:4], dev), i32(pos_q[:4], dev), NO_WINDOW, 0, scale, 0.0,
                                 big.to(dev), own_values=True)
        assert u.abs().max().item() < 1e-6


def _feed(dev, n_rows, chunks, fn):
    """Call ``fn(first row, rows, seq_cu, positions)`` for consecutive portions of one sequence."""
    outs, at = [], 0
    for n in chunks:
        outs.append(fn(at, n, i32([0, n], dev), i32(list(range(at, at + n)), dev)))
        at += n
    assert at == n_rows
    return torch.cat(outs)


def case_matrix_memory(dev, dtype, tol):
    """Gates, running maximum, normaliser and read-out of the matrix memory: whole against portions (down to one
    row), a slot that held something else, gates that saturate at the cap, long sequences (the maximum keeps the
    exponentials in range), two sequences in one launch."""
    dt = DTYPES[dtype]
    g = torch.Generator().manual_seed(5)
    for heads, dim, vdim, cap, t in ((2, 8, 12, 12.0, 45), (1, 24, 10, 6.0, 45), (3, 40, 7, 30.0, 200), (2, 64, 64, 20.0, 70)):
        hd, hv = heads * dim, heads * vdim
        proj = torch.randn(t, 2 * hd + 2 * hv + 3, generator=g).to(dt)
        logits = torch.randn(t, 2 * heads, generator=g) * 8        # some gates reach the cap
        logits[:, heads:] += 3.0
        b_i, b_f = torch.randn(heads, generator=g), torch.randn(heads, generator=g)
        norm_w = torch.rand(hv, generator=g) + 0.5
        q = proj[:, :hd].double().view(t, heads, dim) * dim ** -0.5
        k = proj[:, hd:2 * hd].double().view(t, heads, dim)
        v = proj[:, 2 * hd:2 * hd + hv].double().view(t, heads, vdim)
        gi, gf = po.capped_gates(logits[:, :heads].double() + b_i.double(), logits[:, heads:].double() + b_f.double(), cap)
        cells, tops = po.matrix_memory(q, k, v, gi, gf)
        gate = proj[:, 2 * hd + hv:2 * hd + 2 * hv]
        want = po.unit_rms(cells, 1e-5).reshape(t, hv) * norm_w.double() * torch.sigmoid(gate.double())
        cols = ops.scan_state_cols(vdim, True)
        assert cols > vdim and cols % 4 == 0
        n_state = heads * dim * cols
        for chunks in ([t], [1, 1, 2, 1, t - 10, 2, 3]):
            state = torch.full((3, 4 + n_state + heads), float("nan"), device=dev)   # slots hold rubbish before they are used
            state[1] = 7.0

            def step(at, n, cu, pos):
                rows = proj[at:at + n].contiguous().to(dev)
                prep, top = ops.mlstm_prepare(rows, 0, hd, logits[at:at + n].contiguous().to(dev), b_i.to(dev), b_f.to(dev), cap,
                                              heads, dim, dim ** -0.5, state, 4 + n_state, cu, i32([1], dev), pos)
                close(top, tops[at:at + n], 1e-5, "running maximum")
                o = ops.prepared_scan(prep, rows, 2 * hd, heads, dim, vdim, state, 4, cu, i32([1], dev), pos, unit_col=True)
                return ops.head_finish(o, 1e-5, dt, vdim=vdim, stab=top, weight=norm_w.to(dev),
                                       gate=rows[:, 2 * hd + hv:2 * hd + 2 * hv], gate_act="sigmoid")

            close(_feed(dev, t, chunks, step), want, tol, f"{len(chunks)} portions, heads {heads} x {dim} x {vdim}")
            close(state[1, 4 + n_state:], tops[-1], 1e-5, "maximum left in the slot")
            assert torch.isnan(state[0]).all() and torch.isnan(state[2]).all() and (state[1, :4] == 7.0).all()
    # two sequences and a row of no sequence in one launch
    heads, dim, vdim, t = 2, 8, 12, 30
    hd, hv = heads * dim, heads * vdim
    proj = torch.randn(t, 2 * hd + hv, generator=g).to(dt)
    logits = torch.randn(t, 2 * heads, generator=g) * 3
    zero = torch.zeros(heads)
    cols = ops.scan_state_cols(vdim, True)
    state = torch.zeros((2, heads * dim * cols + heads), device=dev)
    cu, slots = i32([0, 1, 12, 30], dev), i32([-1, 1, 0], dev)
    pos = i32([5] + list(range(11)) + list(range(18)), dev)
    prep, top = ops.mlstm_prepare(proj.to(dev), 0, hd, logits.to(dev), zero.to(dev), zero.to(dev), 9.0, heads, dim, 1.0, state,
                                  heads * dim * cols, cu, slots, pos)
    o = ops.prepared_scan(prep, proj.to(dev), 2 * hd, heads, dim, vdim, state, 0, cu, slots, pos, unit_col=True)
    assert o[0].abs().max() == 0
    for r0, r1 in ((1, 12), (12, 30)):
        q = proj[r0:r1, :hd].double().view(-1, heads, dim)
        k = proj[r0:r1, hd:2 * hd].double().view(-1, heads, dim)
        v = proj[r0:r1, 2 * hd:].double().view(-1, heads, vdim)
        gi, gf = po.capped_gates(logits[r0:r1, :heads].double(), logits[r0:r1, heads:].double(), 9.0)
        cells, _ = po.matrix_memory(q, k, v, gi, gf)
        got = ops.head_finish(o[r0:r1].contiguous(), 1e-5, torch.float32, vdim=vdim, stab=top[r0:r1].contiguous(), unit=False)
        close(got.view(-1, heads, vdim), cells, max(tol, 1e-4), "sequences side by side")


def case_decayed_memory(dev, dtype, tol):
    """Per-channel decays from their pre-activations, the recurrence, the shared norm weight and the silu gate: whole
    against portions, a slot that held something else."""
    dt = DTYPES[dtype]
    g = torch.Generator().manual_seed(6)
    for heads, dim, vdim, tau, t in ((2, 12, 8, 8.0, 45), (1, 20, 6, 4.0, 45), (2, 64, 32, 12.0, 160), (3, 8, 70, 1.0, 33)):
        hd, hv = heads * dim, heads * vdim
        proj = torch.randn(t, 2 * hd + 2 * hv + 5, generator=g).to(dt)
        z = (torch.randn(t, hd, generator=g) * 3).to(dt)
        z_bias = torch.randn(hd, generator=g) + 2
        norm_w = torch.rand(vdim, generator=g) + 0.5
        q = proj[:, :hd].double().view(t, heads, dim) * dim ** -0.5
        k = proj[:, hd:2 * hd].double().view(t, heads, dim)
        v = proj[:, 2 * hd:2 * hd + hv].double().view(t, heads, vdim)
        alpha = po.channel_decay(z.double() + z_bias.double(), tau).view(t, heads, dim)
        cells = po.decayed_memory(q, k, v, alpha)
        gate = proj[:, 2 * hd + hv:2 * hd + 2 * hv].double()
        want = (po.unit_rms(cells, 1e-5) * norm_w.double()).reshape(t, hv) * po.silu(gate)
        n_state = heads * dim * vdim
        for chunks in ([t], [2, 1, 1, t - 9, 3, 2]):
            state = torch.full((2, 8 + n_state), float("nan"), device=dev)
            state[0] = -3.0

            def step(at, n, cu, pos):
                rows = proj[at:at + n].contiguous().to(dev)
                prep = ops.gla_prepare(rows, 0, hd, z[at:at + n].contiguous().to(dev), z_bias.to(dev), heads, dim, dim ** -0.5, tau)
                o = ops.prepared_scan(prep, rows, 2 * hd, heads, dim, vdim, state, 8, cu, i32([0], dev), pos)
                return ops.head_finish(o, 1e-5, dt, weight=norm_w.to(dev), gate=rows[:, 2 * hd + hv:2 * hd + 2 * hv],
                                       gate_act="silu")

            close(_feed(dev, t, chunks, step), want, tol, f"{len(chunks)} portions, heads {heads} x {dim} x {vdim}")
            assert torch.isnan(state[1]).all() and (state[0, :8] == -3.0).all()


def case_scan_pieces(dev, dtype, tol):
    """Long chunks cut into pieces that run side by side give what the walk in one go gives, for both recurrences."""
    dt = DTYPES[dtype]
    g = torch.Generator().manual_seed(7)
    heads, dim, vdim = 2, 32, 64
    hd, hv = heads * dim, heads * vdim
    lens = [300, 1, 140]
    t = sum(lens)
    cu = [0, 300, 301, 441]
    pos = list(range(300)) + [9] + list(range(50, 190))
    proj = (torch.randn(t, 2 * hd + hv, generator=g) * 0.5).to(dt).to(dev)
    z = torch.randn(t, hd, generator=g).to(dt).to(dev)
    logits = (torch.randn(t, 2 * heads, generator=g) * 2).to(dev)
    zero_h, zb = torch.zeros(heads, device=dev), torch.full((hd,), 2.0, device=dev)
    pieces = tuple(torch.from_numpy(a).to(dev) for a in ops.build_scan_pieces(lens, target=8))
    assert pieces[0].shape[0] > 4
    for unit in (False, True):
        cols = ops.scan_state_cols(vdim, unit)
        outs, states = [], []
        start = torch.randn(3, heads * dim * cols + heads, generator=g)   # what the going-on sequences left in their slots
        for pc in (None, pieces):
            state = start.clone().to(dev)
            if unit:
                prep, _ = ops.mlstm_prepare(proj, 0, hd, logits, zero_h, zero_h, 9.0, heads, dim, 1.0, state,
                                            heads * dim * cols, i32(cu, dev), i32([2, 0, 1], dev), i32(pos, dev))
            else:
                prep = ops.gla_prepare(proj, 0, hd, z, zb, heads, dim, 1.0, 8.0)
            outs.append(ops.prepared_scan(prep, proj, 2 * hd, heads, dim, vdim, state, 0, i32(cu, dev), i32([2, 0, 1], dev),
                                          i32(pos, dev), unit_col=unit, pieces=pc))
            states.append(state)
        close(outs[1], outs[0].double().cpu(), tol, "outputs")
        close(states[1][[2, 1]], states[0][[2, 1]].double().cpu(), tol, "states of the sequences that started or went on")


# ----------------------------------------------------------------------------- the engine
def make_engine(cfg, w, device, dtype, pages=12, slots=4, budget=None, eager=True):
    folder = str(po.write_checkpoint(tempfile.mkdtemp(prefix="px-"), cfg, w))
    ec = EngineConfig(model=folder, dtype=dtype, device=device, max_model_len=pages * PAGE, max_num_seqs=slots,
                      max_num_batched_tokens=budget or pages * PAGE, num_gpu_blocks_override=pages,
                      enable_prefix_caching=True, enforce_eager=eager, capture_graphs_at_start=False)
    return LLMEngine(ec)


def tokens(cfg, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


def replay(engine, rid, toks, cuts, end=True):
    """Feed ``toks`` in portions of the sizes ``cuts`` (the rest one by one), all rows wanted -> logits [T, vocab]."""
    out, at = [], 0
    sizes = list(cuts)
    while at < len(toks):
        n = min(sizes.pop(0) if sizes else 1, len(toks) - at)
        last = at + n == len(toks)
        out.append(engine.forced_step([(rid, toks[at:at + n], list(range(n)))], [rid] if last and end else []))
        at += n
    return torch.cat(out).cpu()


def check_rows(got, want, tol, what, loose=0):
    """Every row within ``tol``; with ``loose`` (16-bit runs) that many rows may miss it: a routing decision that
    rounding turns over changes a row, and says nothing about the kernels."""
    assert got.shape == want.shape, f"{what}: shape {tuple(got.shape)} != {tuple(want.shape)}"
    err = po.row_errors(got, want)
    bad = int((err >= tol).sum())
    loose = max(loose, int(loose / 100 * got.shape[0]))   # from 100 rows on, that many per cent
    assert err.median().item() < tol and bad <= loose, f"{what}: {bad} rows off, the worst (row {int(err.argmax())}) by {err.max().item():.3g} (allowed {tol})"
    assert torch.isfinite(err).all(), what


def check_cuts(device, dtype, tol, cfg, w, n, cuts_list, seed=1, pages=12, loose=0):
    toks = tokens(cfg, n, seed)
    want = po.forward(cfg, w, toks)
    eng = make_engine(cfg, w, device, dtype, pages=pages)
    for k, cuts in enumerate(cuts_list):
        check_rows(replay(eng, f"r{k}", toks, cuts), want, tol, f"cuts {cuts[:6]}", loose)
    assert eng.bm.num_free() == pages and eng.scheduler.state_slots.num_free() == 4  # pages and slots came back
    eng.shutdown()


def check_layers(device, dtype, tol, cfg, w, n=37):
    """The residual stream after every layer."""
    toks = tokens(cfg, n, 5)
    want = []
    po.forward(cfg, w, toks, probe=lambda i, x: want.append(x.clone()))
    eng = make_engine(cfg, w, device, dtype)
    got = {}
    eng.runner.model.layer_probe = lambda i, x: got.__setitem__(i, x.detach().double().cpu().clone())
    eng.forced_step([("a", toks, [n - 1])], ["a"])
    for i in range(len(want)):
        err = ((got[i] - want[i]).pow(2).mean(-1).sqrt() / want[i].pow(2).mean(-1).sqrt()).median().item()
        assert err < tol, f"layer {i}: error {err:.3g}"
    eng.shutdown()


def check_batches(device, dtype, tol, cfg, w, loose=0):
    """Unequal requests in the same steps (portions beside single tokens); pages and state slots are used
    again, by requests that start while others are in the middle of theirs."""
    lens = [150, 3, 70, 1, 129, 66, 40]
    reqs = {f"q{i}": tokens(cfg, n, 20 + i) for i, n in enumerate(lens)}
    want = {k: po.forward(cfg, w, v) for k, v in reqs.items()}
    pages = 8  # 512 tokens: less than the sum of all requests
    eng = make_engine(cfg, w, device, dtype, pages=pages, slots=3)
    at = {k: 0 for k in reqs}
    got = {k: [] for k in reqs}
    chunk = {"q0": [31, 2, 64, 1, 1, 33], "q1": [2], "q2": [5, 59, 2], "q3": [1], "q4": [64, 2, 61], "q5": [66],
             "q6": [3, 30]}
    live, waiting = [], list(reqs)
    used_slots = []
    guard = 0
    while live or waiting:
        guard += 1
        assert guard < 400
        while waiting and len(live) < 3:
            need = (len(reqs[waiting[0]]) + PAGE - 1) // PAGE
            held = sum((len(reqs[k]) + PAGE - 1) // PAGE for k in live)
            if held + need > pages:
                break
            live.append(waiting.pop(0))
        entries, end = [], []
        for k in live:
            n = min(chunk[k].pop(0) if chunk[k] else 1, len(reqs[k]) - at[k])
            entries.append((k, reqs[k][at[k]:at[k] + n], list(range(n))))
            at[k] += n
            if at[k] == len(reqs[k]):
                end.append(k)
        logits = eng.forced_step(entries, end).cpu()
        used_slots += [r.state_slot for r in eng.scheduler.running]
        row = 0
        for k, t, _ in entries:
            got[k].append(logits[row:row + len(t)])
            row += len(t)
        live = [k for k in live if k not in end]
    for k in reqs:
        check_rows(torch.cat(got[k]), want[k], tol, f"{k} ({len(reqs[k])} tokens)", loose)
    assert eng.bm.num_free() == pages and not eng.scheduler.running and eng.scheduler.state_slots.num_free() == 3
    assert len(reqs) > 3 >= len(set(used_slots))  # seven requests went through three slots
    eng.shutdown()


def check_generate(device, dtype, cfg, w, n_new=10, eager=True):
    """Greedy generation through the engine's own entry point: scheduler, chunked prefill, sampler."""
    prompts = [tokens(cfg, n, 40 + n) for n in (90, 5, 1, 66, 30)]
    eng = make_engine(cfg, w, device, dtype, pages=10, slots=3, budget=48, eager=eager)  # prompts are cut at 48 rows
    outs = eng.generate(prompts, SamplingParams(max_tokens=n_new, temperature=0.0, ignore_eos=True))
    for p, o in zip(prompts, outs):
        assert o == po.greedy(cfg, w, p, n_new), f"prompt of {len(p)} tokens"
    assert eng.scheduler.state_slots.num_free() == 3 and eng.bm.num_free() == 10
    eng.shutdown()


def check_preemption(device, dtype, cfg, w):
    """A pool too small for all running sequences: the scheduler preempts, the victim gives its slot and
    pages back and is recomputed from its first token; the tokens do not change."""
    prompts = [tokens(cfg, n, 70 + n) for n in (60, 61, 62)]
    n_new = 20
    eng = make_engine(cfg, w, device, dtype, pages=3, slots=3, budget=64)
    outs = eng.generate(prompts, SamplingParams(max_tokens=n_new, temperature=0.0, ignore_eos=True))
    assert eng.scheduler.num_preemptions > 0
    for p, o in zip(prompts, outs):
        assert o == po.greedy(cfg, w, p, n_new)
    eng.shutdown()


def check_far_token(device, dtype, cfg, w, tol):
    """A token far back decides the answer: the same long prompt twice, different in one early token only.  The
    logits hundreds of tokens later must differ from each other and match the oracle for both."""
    n = 330
    a = tokens(cfg, n, 90)
    b = list(a)
    b[3] = (a[3] + 1) % cfg["vocab"]
    eng = make_engine(cfg, w, device, dtype, pages=12)
    rows = [n - 70, n - 1]
    want = {"a": po.forward(cfg, w, a)[rows], "b": po.forward(cfg, w, b)[rows]}
    assert po.row_errors(want["a"], want["b"]).min().item() > 1e-3          # the early token matters to the answer
    for name, toks in (("a", a), ("b", b)):
        eng.forced_step([(name, toks[:200], [])], [])
        got = eng.forced_step([(name, toks[200:], [r - 200 for r in rows])], [name]).cpu()
        check_rows(got, want[name], tol, f"prompt {name}")
        other = want["b" if name == "a" else "a"]
        assert (po.row_errors(got, want[name]) < po.row_errors(got, other)).all()  # and it is seen
    eng.shutdown()
