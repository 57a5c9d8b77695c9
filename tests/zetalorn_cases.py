"""Cases for Zetalorn: every op against its float64 definition, and the engine on small random checkpoints
against the float64 oracle.  The CPU and the GPU test files call them with their device, dtype and tolerance."""

from __future__ import annotations

import tempfile

import torch

import zetalorn_oracle as zo
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
    """Both kinds of layer, a loop of three passes over the middle layers that ends before the last layer, sizes that
    differ from one another wherever they can, a layer without feed-forward, blocks that straddle pages."""
    return zo.make_config([
        zo.parallel_spec(heads=4, kv_heads=2, dim=12, vdim=20, window=40, pool=5, rot_dims=8, r_heads=3, r_dim=8, r_vdim=12)
        | {"mlp": zo.moe_spec(experts=6, top=2, count=3, keep=2, ff=20, limit=1.5)},
        zo.attention_spec(heads=4, kv_heads=2, dim=16, vdim=12, chunk=70, rot_dims=8, factor=4.0, diff=0.2)
        | {"mlp": zo.moe_spec(experts=4, top=2, count=2, keep=1, ff=16, limit=0.7)},
        zo.parallel_spec(heads=2, kv_heads=1, dim=8, vdim=8, window=33, pool=11, rot_dims=8, r_heads=2, r_dim=12, r_vdim=6)
        | {"mlp": None},
        zo.attention_spec(heads=2, kv_heads=1, dim=8, vdim=20, chunk=64, rot_dims=8, factor=1.5, diff=0.45)
        | {"mlp": zo.moe_spec(experts=5, top=3, count=1, keep=1, ff=12, limit=2.0)},
    ], width=48, vocab=97, loop=(1, 3, 3), eps=1e-5, logit_scale=0.5)


def config_b():
    """Other corners: attention first, no loop, one KV head per query head, no rotation in one layer and no
    scaling in another, chunks of 5 and 180 and a window of 7, blocks of one token and blocks longer than a page, groups of
    one expert, top 1, a single recurrent head, a decay of 1 and a tiny one, eps 1e-3, logits unscaled."""
    return zo.make_config([
        zo.attention_spec(heads=3, kv_heads=3, dim=8, vdim=10, chunk=5, rot_dims=0, factor=0, diff=0.1, scale=0.9)
        | {"mlp": zo.moe_spec(experts=4, top=1, count=4, keep=2, ff=16, limit=1.0)},
        zo.parallel_spec(heads=2, kv_heads=2, dim=10, vdim=6, window=7, pool=1, rot_dims=10, r_heads=1, r_dim=20, r_vdim=6,
                         decay=[1.0]) | {"mlp": None},
        zo.attention_spec(heads=4, kv_heads=1, dim=12, vdim=8, chunk=180, rot_dims=12, factor=0, diff=0.35)
        | {"mlp": zo.moe_spec(experts=3, top=3, count=1, keep=1, ff=24, limit=3.0)},
        zo.parallel_spec(heads=3, kv_heads=1, dim=6, vdim=14, window=20, pool=70, rot_dims=2, r_heads=2, r_dim=6, r_vdim=10,
                         decay=[0.03, 0.9]) | {"mlp": zo.moe_spec(experts=8, top=2, count=2, keep=2, ff=8, limit=0.5)},
    ], width=24, vocab=50, eps=1e-3, logit_scale=1.0)


def config_c():
    """Head sizes the matrix-core attention kernel tiles, unit sizes the grouped GEMMs tile, a loop that starts at
    layer 0 with two passes, chunks long enough to be cut into pieces by the recurrence kernel."""
    return zo.make_config([
        zo.attention_spec(heads=4, kv_heads=2, dim=64, vdim=128, chunk=150, rot_dims=32, factor=2.5, diff=0.25)
        | {"mlp": zo.moe_spec(experts=6, top=2, count=2, keep=1, ff=64, limit=1.0)},
        zo.parallel_spec(heads=4, kv_heads=2, dim=64, vdim=128, window=100, pool=9, rot_dims=64, r_heads=2, r_dim=32,
                         r_vdim=64) | {"mlp": zo.moe_spec(experts=4, top=2, count=1, keep=1, ff=128, limit=2.0)},
        zo.parallel_spec(heads=2, kv_heads=1, dim=128, vdim=128, window=64, pool=64, rot_dims=32, r_heads=1, r_dim=64,
                         r_vdim=64) | {"mlp": None},
    ], width=128, vocab=200, loop=(0, 2, 2), eps=2e-6, logit_scale=0.4)


def config_d():
    """Sizes that are multiples of nothing: odd head sizes, a width and a vocabulary that are no multiple of 8; a
    loop of one pass over a single layer."""
    return zo.make_config([
        zo.parallel_spec(heads=6, kv_heads=2, dim=6, vdim=5, window=13, pool=3, rot_dims=4, r_heads=3, r_dim=5, r_vdim=7)
        | {"mlp": zo.moe_spec(experts=9, top=2, count=3, keep=2, ff=9, limit=1.0)},
        zo.attention_spec(heads=6, kv_heads=3, dim=6, vdim=7, chunk=17, rot_dims=6, factor=3.0, diff=0.6)
        | {"mlp": zo.moe_spec(experts=5, top=2, count=1, keep=1, ff=11, limit=1.0)},
    ], width=20, vocab=45, loop=(1, 2, 1), eps=1e-5, logit_scale=2.0)


def config_e():
    """Attention layers only (the state slots stay empty)."""
    return zo.make_config([
        zo.attention_spec(heads=2, kv_heads=2, dim=8, vdim=8, chunk=30, rot_dims=4, factor=8.0, diff=0.3) | {"mlp": None},
        zo.attention_spec(heads=2, kv_heads=1, dim=16, vdim=4, chunk=9, rot_dims=16, factor=0, diff=0.05)
        | {"mlp": zo.moe_spec(experts=2, top=1, count=2, keep=1, ff=8, limit=1.0)},
    ], width=16, vocab=40, loop=(0, 2, 2), eps=1e-6, logit_scale=1.0)


# ----------------------------------------------------------------------------- mechanisms
def case_gated_residual(dev, dtype, tol):
    """residual += sigmoid(gate + b) * sum c_i n_i(d_i) + extra + vector, then the pre-norm: every part alone and together."""
    dt = DTYPES[dtype]
    g = torch.Generator().manual_seed(0)
    eps = 1e-5
    for n in (5, 48, 300, 2304, 4104):   # widths that take 16-byte loads (in one, two and four runs per thread) and not
        at = 8 if n % 8 == 0 else 3
        res = torch.randn(7, n, generator=g) * 2
        w = torch.rand(n, generator=g) + 0.5
        d1 = (torch.randn(7, n, generator=g) * 3).to(dt)
        d2 = (torch.randn(7, n, generator=g) * 0.1).to(dt)
        w1, w2 = torch.rand(n, generator=g) + 0.5, torch.rand(n, generator=g) + 0.5
        wide = (torch.randn(7, 2 * n + 8, generator=g) * 2).to(dt)   # the gate is a view of a wider projection
        bias = torch.randn(n, generator=g)
        extra, vec = torch.randn(7, n, generator=g), torch.randn(n, generator=g)
        sg = zo.sigmoid(wide[:, at:at + n].double() + bias.double())
        cases = {
            "one gated delta": ([(d1, None, 1.0)], True, None, None, sg * d1.double()),
            "a delta in 32 bits": ([(d1.float() * 1e-3, None, 1.0)], True, None, None, sg * d1.float().double() * 1e-3),
            "two normed deltas": ([(d1, w1, 0.5), (d2, w2, 0.5)], True, None, None,
                                  sg * 0.5 * (zo.rms(d1.double(), eps) * w1.double() + zo.rms(d2.double(), eps) * w2.double())),
            "no gate": ([(d1, None, 2.0)], False, None, None, 2.0 * d1.double()),
            "extras only": ([], False, extra, vec, extra.double() + vec.double()),
            "everything": ([(d1, w1, 0.5), (d2, None, 0.25)], True, extra, vec,
                           sg * (0.5 * zo.rms(d1.double(), eps) * w1.double() + 0.25 * d2.double()) + extra.double() + vec.double()),
            "nothing": ([], False, None, None, torch.zeros(7, n, dtype=F64)),
        }
        for name, (deltas, gated, ex, ve, add) in cases.items():
            r = res.clone().to(dev)
            deltas = [(d.to(dev), None if nw is None else nw.to(dev), c) for d, nw, c in deltas]
            y = ops.gated_add_rms_norm(r, deltas, wide.to(dev)[:, at:at + n] if gated else None, bias.to(dev) if gated else None,
                                       w.to(dev), eps, dt, extra=None if ex is None else ex.to(dev),
                                       extra_vec=None if ve is None else ve.to(dev))
            want = res.double() + add
            close(r, want, 2e-6, f"{name}: stream, width {n}")
            close(y, zo.rms(want, eps) * w.double(), tol, f"{name}: normed, width {n}")
            r2 = res.clone().to(dev)
            assert ops.gated_add_rms_norm(r2, deltas, wide.to(dev)[:, at:at + n] if gated else None,
                                          bias.to(dev) if gated else None, None, eps, dt,
                                          extra=None if ex is None else ex.to(dev),
                                          extra_vec=None if ve is None else ve.to(dev), want_out=False) is None
            close(r2, want, 2e-6, f"{name}: stream without output")


def case_routing(dev):
    """Sigmoid scores, groups by the sum of their two largest, top-k inside the kept groups, weights over their sum."""
    g = torch.Generator().manual_seed(1)
    for experts, count, keep, top in ((10, 2, 1, 2), (6, 3, 2, 2), (4, 4, 2, 1), (5, 1, 1, 3), (8, 2, 2, 2), (9, 3, 1, 3),
                                      (2, 2, 1, 1), (3, 1, 1, 3)):
        logits = torch.randn(40, experts + 2, generator=g) * 2
        w, ids, _ = ops.group_topk(logits.to(dev), experts, count, keep, top, 1.0, normalize=True)
        scores = zo.sigmoid(logits[:, :experts].double())
        for t in range(40):
            want = zo.choose_experts(scores[t], top, count, keep)
            assert ids[t].tolist() == want, (experts, count, keep, top, t)
            ws = scores[t, want] / (scores[t, want].sum() + 1e-20)
            close(w[t], ws, 1e-6, "weights")
        plain, _, _ = ops.group_topk(logits.to(dev), experts, count, keep, top, 2.5)   # the form without the division
        close(plain, 2.5 * torch.gather(scores, 1, ids.long().cpu()), 1e-6, "scores times a scale")
    # an expert outside the kept group is never chosen, however large: group 0 holds the largest single score,
    # group 1 the largest pair
    z = torch.tensor([[4.0, -4.0, -4.0, 2.0, 2.0, 1.0]])
    _, ids, _ = ops.group_topk(z.to(dev), 6, 2, 1, 2, 1.0, normalize=True)
    assert sorted(ids[0].tolist()) == [3, 4]


def _pages(dev, dt, n_pages, elems):
    return torch.zeros(n_pages, elems, dtype=dt, device=dev)


def case_qk_norm_rotation(dev, dtype, tol):
    """Per-head RMS norm with a weight, rotation in both pair layouts over part of the head, frequencies divided by a
    factor, fewer value heads than key heads; q returned, k and v in the pages."""
    dt = DTYPES[dtype]
    g = torch.Generator().manual_seed(2)
    eps = 1e-5
    for heads, k_heads, v_heads, dim, vdim, rot_dims, layout, factor in (
            (4, 2, 2, 12, 20, 8, 0, None), (8, 4, 2, 16, 12, 8, 1, 4.0), (3, 3, 3, 8, 10, 0, 0, None),
            (2, 1, 1, 70, 5, 70, 1, 1.5), (6, 2, 2, 6, 5, 4, 0, 3.0)):
        t = 23
        pos = torch.tensor([0, 1, 2, 63, 64, 65, 127, 128, 700] + list(range(300, 314)))
        rot = {"base": 700.0, "dims": rot_dims}
        if factor:
            rot["scaling"] = {"factor": factor}
        table = (ops.build_cos_sin(rot_dims, 1024, 700.0, {"rope_type": "linear", "factor": factor} if factor else None,
                                   device=dev) if rot_dims else None)
        nq, nk, nv = heads * dim, k_heads * dim, v_heads * vdim
        proj = (torch.randn(t, nq + nk + nv + 7, generator=g) * 2).to(dt)
        qw, kw = torch.rand(dim, generator=g) + 0.5, torch.rand(dim, generator=g) + 0.5
        region = ops.window_cache_elems(k_heads, dim, vdim, v_heads)
        pool = _pages(dev, dt, 16, 8 + region)
        slots = torch.tensor([(int(p) // PAGE + 2) * PAGE + int(p) % PAGE for p in pos], dtype=torch.int64)
        slots[5] = -1   # a row that is not cached
        q = ops.qk_norm_write(proj.to(dev), heads, k_heads, dim, vdim, pos.int().to(dev), slots.to(dev), pool, 8, eps,
                              v_heads=v_heads, q_weight=qw.to(dev), k_weight=kw.to(dev), cos_sin=table, rot_dims=rot_dims,
                              layout=layout)
        pd = proj.double()
        want_q = zo.rotate(zo.rms(pd[:, :nq].view(t, heads, dim), eps) * qw.double(), pos, rot, layout == 1)
        want_k = zo.rotate(zo.rms(pd[:, nq:nq + nk].view(t, k_heads, dim), eps) * kw.double(), pos, rot, layout == 1)
        close(q, want_q, tol, f"q, layout {layout}, {rot_dims} of {dim}")
        kc, vc = reference.window_cache_views(pool.cpu(), 8, k_heads, dim, vdim, v_heads)
        for r in range(t):
            pg, off = int(slots[r]) // PAGE, int(slots[r]) % PAGE
            if slots[r] < 0:
                continue
            close(kc[pg, off], want_k[r], tol, "k in the page")
            close(vc[pg, off], pd[r, nq + nk:nq + nk + nv].view(v_heads, vdim), 1e-6, "v in the page")
        assert float(pool[:, :8].abs().sum()) == 0 and float(pool[0].abs().sum()) == 0  # nothing outside its place


def _attention_oracle(q, k, v, pos_of_row, scale, seen_tokens, seen_blocks, block, maps):
    """q [R, heads, dim] at positions pos_of_row over k [T, k_heads, dim], v [T, v_heads, vdim] of the whole sequence;
    seen_tokens(i) -> bool [T], seen_blocks(i) -> number of pooled blocks seen."""
    rows, heads, _ = q.shape
    k_heads, v_heads = k.shape[1], v.shape[1]
    rep = heads // k_heads
    out = torch.zeros(rows, heads, v.shape[2], dtype=F64)
    for r in range(rows):
        i = int(pos_of_row[r])
        tok = seen_tokens(i)
        nb = seen_blocks(i)
        for h in range(heads):
            kh = h // rep
            keys, vals = k[tok, kh], v[tok, kh // maps]
            if nb:
                keys = torch.cat([k[:nb * block, kh].view(nb, block, -1).mean(1), keys])
                vals = torch.cat([v[:nb * block, kh // maps].view(nb, block, -1).mean(1), vals])
            wts = torch.softmax((keys @ q[r, h]) * scale, 0)
            out[r, h] = wts @ vals
    return out


def _run_attention(dev, dt, q, k, v, cuts, scale, how, window, tiles_for=None, splits=1):
    """Feeds a sequence's q / k / v rows through qk_norm_write (weights of one, no rotation: the rows go in as
    they are, up to the norm), pool_blocks and window_attention in portions; pages in scrambled order."""
    t, heads, dim = q.shape
    k_heads, v_heads, vdim = k.shape[1], v.shape[1], v.shape[2]
    maps = k_heads // v_heads
    region = ops.window_cache_elems(k_heads, dim, vdim, v_heads)
    block = how.get("pool_block", 0)
    elems = 16 + region * (2 if block else 1)
    n_pages = (t + PAGE - 1) // PAGE
    pool = _pages(dev, dt, n_pages + 3, elems)
    pool[:] = 3.0  # pages hold something finite from an earlier use
    order = [(7 * p + 2) % (n_pages + 3) for p in range(n_pages)]
    assert len(set(order)) == n_pages
    bt = i32([order + [0]], dev)
    proj = torch.cat([q.reshape(t, -1), k.reshape(t, -1), v.reshape(t, -1)], 1).to(dt)
    out, at = [], 0
    sizes = list(cuts)
    while at < t:
        n = min(sizes.pop(0) if sizes else 1, t - at)
        pos = torch.arange(at, at + n, dtype=torch.int32, device=dev)
        slots = torch.tensor([order[p // PAGE] * PAGE + p % PAGE for p in range(at, at + n)], dtype=torch.int64, device=dev)
        qq = ops.qk_norm_write(proj[at:at + n].contiguous().to(dev), heads, k_heads, dim, vdim, pos, slots, pool, 16, 1e-12,
                               v_heads=v_heads)
        decode = n == 1 and at > 0
        row_seq = None if decode else torch.zeros(n, dtype=torch.int32, device=dev)
        if block:
            ops.pool_blocks(pool, 16, region, k_heads, dim, vdim, bt, row_seq, pos, slots, block)
        tiles = None
        if tiles_for is not None and not decode:
            tiles = torch.from_numpy(ops.build_window_tiles([n], [at + n], heads, k_heads)).to(dev)
        u = ops.window_attention(qq, pool, 16, k_heads, vdim, bt, row_seq, pos, window, 0, scale, 0.0, None, tiles=tiles,
                                 splits=splits if decode else 1, own_values=True, maps=maps,
                                 **({"pool_off": region} if block else {}), **how)
        out.append(u[:, :, 0].double().cpu())
        at += n
    return torch.cat(out)


def case_masks(dev, dtype, tol, tiled=False):
    """Chunked, windowed and pooled attention with one key made to stand out: a key just inside and just outside the
    chunk or the window, a block that is just seen and one that is not yet, keys at page borders and hundreds back,
    the first tokens; whole, in portions that cut blocks, chunks and pages, and as single decode rows."""
    dt = DTYPES[dtype]
    g = torch.Generator().manual_seed(3)
    heads, k_heads, dim, vdim = (4, 2, 64, 128) if tiled else (4, 2, 12, 10)
    t = 330
    scale = 40.0 / dim   # an aligned pair scores 40, a random one about 40 / sqrt(dim)
    hot = torch.zeros(dim)
    hot[dim - 1] = 1.0

    def sequence(hot_keys, maps=1):
        q = torch.randn(t, heads * maps, dim, generator=g) * 0.05 + hot    # every query looks for the hot keys
        k = torch.randn(t, k_heads * maps, dim, generator=g)
        k[:, :, dim - 1] = 0.0
        v = torch.randn(t, k_heads, vdim, generator=g)
        for j in hot_keys:
            k[j] = hot * 3.0
            v[j] = 5.0 + j / 10.0   # what comes out says which key was seen

        def unit(x):  # what the write kernel makes of a row: the rounded input to unit RMS, rounded again
            x = x.to(dt).float()
            return (x / x.pow(2).mean(-1, keepdim=True).sqrt()).to(dt).double()

        return q, k, v, unit(q), unit(k), v.to(dt).double()

    cuts_list = [[t], [100, 2, 3, 64, 61, 2, 38], [200] + [1] * 130] if not tiled else [[t], [129, 2, 64, 70], [250] + [1] * 80]
    kw = {"tiles_for": True} if tiled else {}
    rows = torch.arange(t)
    # a chunk of 70 (not a page's multiple): a hot key at the chunk's first position, its last, and in the middle
    for size, hots in ((70, [70, 139, 175]), (64, [63, 64, 300]), (1000, [0, 5])):
        q, k, v, qn, kn, vn = sequence(hots, maps=2)
        want = _attention_oracle(qn, kn, vn, rows, scale, lambda i: (rows <= i) & (rows // size == i // size), lambda i: 0, 0, 2)
        for cuts in cuts_list:
            got = _run_attention(dev, dt, q, k, v, cuts, scale, {"chunked": True}, size, splits=2 if len(cuts) > 50 else 1, **kw)
            close(got, want, tol, f"chunk {size}, hot {hots}, {len(cuts)} portions")
    # a window: the hot key leaves it, is unseen for a while, and comes back inside its pooled block
    for window, block, hots in ((40, 5, [10, 11, 12, 13, 14, 201]), (33, 11, [0, 127, 128]), (64, 64, list(range(64, 128))),
                                (20, 70, [3]), (7, 1, [100, 250]), (50, 0, [60, 61]), (NO_WINDOW, 0, [2])):
        q, k, v, qn, kn, vn = sequence(hots)
        seen_b = (lambda i: max(0, (i - window + 1) // block)) if block else (lambda i: 0)
        want = _attention_oracle(qn, kn, vn, rows, scale, lambda i: (rows <= i) & (i - rows < window), seen_b, block, 1)
        for cuts in cuts_list:
            got = _run_attention(dev, dt, q, k, v, cuts, scale, {"pool_block": block} if block else {}, window,
                                 splits=3 if len(cuts) > 50 else 1, **kw)
            close(got, want, tol, f"window {window}, blocks of {block}, hot {hots[:3]}, {len(cuts)} portions")


def case_differential(dev, dtype, tol):
    dt = DTYPES[dtype]
    g = torch.Generator().manual_seed(4)
    for heads, kv_heads, vdim, lam, diff in ((4, 2, 12, 0.7, 0.2), (3, 3, 70, -0.4, 0.5), (6, 1, 5, 1.3, 0.05)):
        rep = heads // kv_heads
        a = torch.randn(9, heads, 2, vdim, generator=g)   # per head: the first map's output, the second's
        u = a.view(9, kv_heads, rep, 2, vdim).permute(0, 1, 3, 2, 4).reshape(9, 2 * heads, vdim).contiguous()
        y = ops.diff_heads(u.to(dev), kv_heads, lam, 1e-5, 1.0 - diff, dt)
        o = a[:, :, 0].double() - lam * a[:, :, 1].double()
        close(y, (zo.rms(o, 1e-5) * (1.0 - diff)).reshape(9, heads * vdim), tol, f"{heads} heads on {kv_heads}")


def case_lightning(dev, dtype, tol):
    """The decayed recurrence on silu'd q, k and v: whole against portions down to one row, a slot that held
    something else, two sequences side by side, the norm over all heads with the sigmoid gate."""
    dt = DTYPES[dtype]
    g = torch.Generator().manual_seed(5)
    for heads, dim, vdim, decay, t in ((3, 8, 12, [0.5, 0.9, 0.999], 45), (1, 20, 6, [1.0], 45), (2, 64, 32, [0.03, 0.97], 160),
                                       (2, 5, 7, [0.6, 0.7], 33)):
        hd, hv = heads * dim, heads * vdim
        proj = torch.randn(t, 2 * hd + 2 * hv + 5, generator=g).to(dt)
        norm_w = torch.rand(hv, generator=g) + 0.5
        m = {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay}
        pd = proj.double()
        want = _lightning(pd[:, :hd], pd[:, hd:2 * hd], pd[:, 2 * hd:2 * hd + hv], pd[:, 2 * hd + hv:2 * hd + 2 * hv], m,
                          norm_w.double())
        n_state = heads * dim * vdim
        dec = torch.tensor(decay, dtype=torch.float32, device=dev)
        for chunks in ([t], [2, 1, 1, t - 9, 3, 2]):
            state = torch.full((2, 8 + n_state), float("nan"), device=dev)
            state[0] = -3.0
            out, at = [], 0
            for n in chunks:
                rows = proj[at:at + n].contiguous().to(dev)
                o = ops.recurrent_scan(rows, 0, hd, 2 * hd, heads, dim, vdim, state, 8, i32([0, n], dev), i32([0], dev),
                                       torch.arange(at, at + n, dtype=torch.int32, device=dev), decay=dec,
                                       min_decay=min(decay), act=True)
                out.append(ops.head_finish(o.view(n, 1, hv), 1e-5, dt, weight=norm_w.to(dev),
                                           gate=rows[:, 2 * hd + hv:2 * hd + 2 * hv], gate_act="sigmoid").double().cpu())
                at += n
            close(torch.cat(out), want, tol, f"{len(chunks)} portions, heads {heads} x {dim} x {vdim}")
            assert torch.isnan(state[1]).all() and (state[0, :8] == -3.0).all()


def _lightning(q, k, v, gate, m, norm_w):
    t = q.shape[0]
    n, d, dv = m["heads"], m["dim"], m["vdim"]
    q, k, v = zo.silu(q).view(t, n, d), zo.silu(k).view(t, n, d), zo.silu(v).view(t, n, dv)
    out = torch.zeros(t, n, dv, dtype=F64)
    for head in range(n):
        state = torch.zeros(d, dv, dtype=F64)
        for i in range(t):
            state = m["decay"][head] * state + torch.outer(k[i, head], v[i, head])
            out[i, head] = state.T @ q[i, head]
    return zo.rms(out.reshape(t, n * dv), 1e-5) * norm_w * zo.sigmoid(gate)


def case_scan_pieces(dev, dtype, tol):
    """Long chunks cut into pieces that run side by side give what the walk in one go gives."""
    dt = DTYPES[dtype]
    g = torch.Generator().manual_seed(7)
    heads, dim, vdim = 2, 32, 64
    hd, hv = heads * dim, heads * vdim
    lens = [300, 1, 140]
    cu = [0, 300, 301, 441]
    pos = list(range(300)) + [9] + list(range(50, 190))
    proj = (torch.randn(sum(lens), 2 * hd + hv, generator=g)).to(dt).to(dev)
    pieces = tuple(torch.from_numpy(a).to(dev) for a in ops.build_scan_pieces(lens, target=8))
    for decay in ([0.97, 0.5], [0.05, 1.0]):
        dec = torch.tensor(decay, dtype=torch.float32, device=dev)
        start = torch.randn(3, heads * dim * vdim, generator=g)
        outs, states = [], []
        for pc in (None, pieces):
            state = start.clone().to(dev)
            outs.append(ops.recurrent_scan(proj, 0, hd, 2 * hd, heads, dim, vdim, state, 0, i32(cu, dev), i32([2, 0, 1], dev),
                                           i32(pos, dev), decay=dec, min_decay=min(decay), act=True, pieces=pc))
            states.append(state)
        close(outs[1], outs[0].double().cpu(), tol, "outputs")
        close(states[1][[2, 1]], states[0][[2, 1]].double().cpu(), tol, "states")


# ----------------------------------------------------------------------------- the engine
def make_engine(cfg, w, device, dtype, pages=12, slots=4, budget=None, eager=True):
    folder = zo.save_checkpoint(tempfile.mkdtemp(prefix="zx-"), cfg, w)
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
    err = zo.row_errors(got, want)
    bad = int((err >= tol).sum())
    loose = max(loose, int(loose / 100 * got.shape[0]))   # from 100 rows on, that many per cent
    assert err.median().item() < tol and bad <= loose, \
        f"{what}: {bad} rows off, the worst (row {int(err.argmax())}) by {err.max().item():.3g} (allowed {tol})"
    assert torch.isfinite(err).all(), what


def check_cuts(device, dtype, tol, cfg, w, n, cuts_list, seed=1, pages=12, loose=0):
    toks = tokens(cfg, n, seed)
    want = zo.forward(cfg, w, toks)
    eng = make_engine(cfg, w, device, dtype, pages=pages)
    for k, cuts in enumerate(cuts_list):
        check_rows(replay(eng, f"r{k}", toks, cuts), want, tol, f"cuts {cuts[:6]}", loose)
    assert eng.bm.num_free() == pages and eng.scheduler.state_slots.num_free() == 4  # pages and slots came back
    eng.shutdown()


def check_layers(device, dtype, tol, cfg, w, n=37):
    """The residual stream after every layer run."""
    toks = tokens(cfg, n, 5)
    want = zo.run(cfg, w, toks)[1]
    eng = make_engine(cfg, w, device, dtype)
    got = {}
    eng.runner.model.layer_probe = lambda i, x: got.__setitem__(i, x.detach().double().cpu().clone())
    eng.forced_step([("a", toks, [n - 1])], ["a"])
    assert len(got) == want.shape[0] == len(zo.layer_runs(cfg))
    for i in range(want.shape[0]):
        err = ((got[i] - want[i]).pow(2).mean(-1).sqrt() / want[i].pow(2).mean(-1).sqrt()).median().item()
        assert err < tol, f"run {i}: error {err:.3g}"
    eng.shutdown()


def check_batches(device, dtype, tol, cfg, w, loose=0):
    """Unequal requests in the same steps (portions beside single tokens); pages and state slots are used
    again, by requests that start while others are in the middle of theirs."""
    lens = [150, 3, 70, 1, 129, 66, 40]
    reqs = {f"q{i}": tokens(cfg, n, 20 + i) for i, n in enumerate(lens)}
    want = {k: zo.forward(cfg, w, v) for k, v in reqs.items()}
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
        assert o == zo.greedy(cfg, w, p, n_new), f"prompt of {len(p)} tokens"
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
        assert o == zo.greedy(cfg, w, p, n_new)
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
    want = {"a": zo.forward(cfg, w, a)[rows], "b": zo.forward(cfg, w, b)[rows]}
    assert zo.row_errors(want["a"], want["b"]).min().item() > 1e-4          # the early token matters to the answer
    for name, toks in (("a", a), ("b", b)):
        eng.forced_step([(name, toks[:200], [])], [])
        got = eng.forced_step([(name, toks[200:], [r - 200 for r in rows])], [name]).cpu()
        check_rows(got, want[name], tol, f"prompt {name}")
        other = want["b" if name == "a" else "a"]
        apart = zo.row_errors(want[name], other) > 4 * tol   # (16-bit rounding may be larger than a faint trace)
        assert (zo.row_errors(got, want[name]) < zo.row_errors(got, other))[apart].all()  # and it is seen
    eng.shutdown()


def check_graph_decode(device, dtype, cfg, w, tol):
    """Decode steps replayed from HIP graphs give what eager steps give, over several replays with prefill between."""
    prompts = [tokens(cfg, n, 60 + n) for n in (70, 3, 130)]
    outs = []
    for eager in (True, False):
        eng = make_engine(cfg, w, device, dtype, pages=12, slots=3, eager=eager)
        outs.append(eng.generate(prompts, SamplingParams(max_tokens=24, temperature=0.0, ignore_eos=True)))
        eng.shutdown()
    same = sum(a == b for a, b in zip(*outs))
    assert same == len(prompts), f"{len(prompts) - same} of {len(prompts)} generations differ between graph and eager steps"
