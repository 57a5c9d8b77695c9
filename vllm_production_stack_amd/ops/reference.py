"""Plain PyTorch (fp32 math) definitions of every engine op.

These are the numerical oracles for the HIP kernels in ``csrc/kernels`` and the execution
path for CPU tensors (unit tests, CPU-only plumbing replicas).  They share the paged
KV-cache layout with the kernels:

    pool[page, layer, 0, kv_head]  viewed as  [head_dim / 32, PAGE, 32]   (K: channel block, key, channel)
    pool[page, layer, 1, kv_head]  viewed as  [PAGE / 32, head_dim, 32]   (V: key half, channel, key)

(blocks of 32 = 64 bytes, so that a 16-row MFMA fragment load of the decode kernel is one
contiguous KiB; head sizes that are not a multiple of 32 use one block of the whole head).
``_kv_views`` presents both as [.., PAGE, head_dim] / [.., head_dim, PAGE] whatever the blocks.
"""

from __future__ import annotations

import math

import torch

PAGE = 64


def rms_norm(x, weight, eps, residual=None):
    if residual is not None:
        s = x.float() + residual.float()
        residual.copy_(s.to(residual.dtype))
        xf = residual.float()
    else:
        xf = x.float()
    var = xf.pow(2).mean(-1, keepdim=True)
    return (xf * torch.rsqrt(var + eps) * weight.float()).to(x.dtype)


def layer_norm(x, weight, bias, eps):
    return torch.nn.functional.layer_norm(x.float(), (x.shape[-1],), weight.float(), bias.float(), eps).to(x.dtype)


def build_cos_sin(head_dim: int, max_pos: int, theta: float, scaling: dict | None = None, device="cpu"):
    """[max_pos, head_dim] fp32 table: cos for the head_dim/2 frequencies, then sin."""
    half = head_dim // 2
    inv = 1.0 / (theta ** (torch.arange(0, half, dtype=torch.float64) / half))
    if scaling and scaling.get("rope_type", scaling.get("type")) == "llama3":
        factor = scaling.get("factor", 8.0)
        lo = scaling.get("low_freq_factor", 1.0)
        hi = scaling.get("high_freq_factor", 4.0)
        orig = scaling.get("original_max_position_embeddings", 8192)
        wavelen = 2 * torch.pi / inv
        smooth = ((orig / wavelen) - lo) / (hi - lo)
        scaled = torch.where(wavelen > orig / lo, inv / factor, inv)
        mid = (1 - smooth) * inv / factor + smooth * inv
        is_mid = (wavelen <= orig / lo) & (wavelen >= orig / hi)
        inv = torch.where(is_mid, mid, scaled)
    if scaling and scaling.get("rope_type", scaling.get("type")) == "linear":
        inv = inv / float(scaling["factor"])  # position interpolation: every frequency divided by the factor
    mag = 1.0
    if scaling and scaling.get("rope_type", scaling.get("type")) == "ramp":
        # frequencies divided by ``factor`` behind a linear ramp over the pair index, between the pairs
        # that make ``fast`` and ``slow`` turns over ``original`` positions; cos and sin grow by
        # 0.1 ln(factor) + 1
        import math

        factor, orig = float(scaling["factor"]), float(scaling["original"])

        def pair_of(turns):
            return head_dim * math.log(orig / (2 * math.pi * turns)) / (2 * math.log(theta))

        lo = max(math.floor(pair_of(float(scaling["fast"]))), 0)
        hi = min(math.ceil(pair_of(float(scaling["slow"]))), head_dim - 1)
        ramp = ((torch.arange(0, half, dtype=torch.float64) - lo) / max(hi - lo, 0.001)).clamp(0, 1)
        inv = inv / factor * ramp + inv * (1 - ramp)
        mag = 0.1 * math.log(factor) + 1.0
    ang = torch.arange(max_pos, dtype=torch.float64)[:, None] * inv[None, :]
    return (torch.cat([ang.cos(), ang.sin()], dim=-1) * mag).float().to(device)


def _kv_views(pool, layer, n_kv, head_dim):
    """K as [pages, n_kv, PAGE, head_dim] and V as [pages, n_kv, head_dim, PAGE]: permuted views of
    the pool (reads and indexed writes go through to it)."""
    cb = 32 if head_dim % 32 == 0 else head_dim
    n = pool.shape[0]
    k = pool[:, layer, 0].view(n, n_kv, head_dim // cb, PAGE, cb).permute(0, 1, 3, 2, 4)
    v = pool[:, layer, 1].view(n, n_kv, PAGE // 32, head_dim, 32).permute(0, 1, 3, 2, 4)
    return k, v  # [n, n_kv, PAGE, blocks, cb], [n, n_kv, head_dim, 2, 32]


def rope_and_cache(qkv, positions, slots, cos_sin, pool, layer, n_q, n_kv, head_dim, rotary=True):
    """Rotate Q and K heads of ``qkv`` in place (NeoX pairing) and write K/V into the pool."""
    t = qkv.shape[0]
    if t == 0:
        return
    half = head_dim // 2
    x = qkv.view(t, n_q + 2 * n_kv, head_dim)
    if rotary:
        cs = cos_sin[positions.long()]
        cos, sin = cs[:, None, :half], cs[:, None, half:]
        qk = x[:, : n_q + n_kv].float()
        a, b = qk[..., :half], qk[..., half:]
        rot = torch.cat([a * cos - b * sin, b * cos + a * sin], dim=-1)
        x[:, : n_q + n_kv] = rot.to(qkv.dtype)
    if slots is None:
        return
    kview, vview = _kv_views(pool, layer, n_kv, head_dim)
    ok = slots >= 0
    s = slots[ok].long()
    page, off = s // PAGE, s % PAGE
    cb = kview.shape[-1]
    kview[page, :, off] = x[ok, n_q : n_q + n_kv].reshape(-1, n_kv, head_dim // cb, cb)
    vview[page, :, :, off // 32, off % 32] = x[ok, n_q + n_kv :]


def _gather_kv(pool, layer, n_kv, head_dim, block_row, length):
    kview, vview = _kv_views(pool, layer, n_kv, head_dim)
    npages = (length + PAGE - 1) // PAGE
    pages = block_row[:npages].long()
    k = kview[pages].reshape(npages, n_kv, PAGE, head_dim).permute(1, 0, 2, 3).reshape(
        n_kv, npages * PAGE, head_dim)[:, :length]
    v = vview[pages].reshape(npages, n_kv, head_dim, PAGE).permute(1, 2, 0, 3).reshape(
        n_kv, head_dim, npages * PAGE)[:, :, :length]
    return k.float(), v.float().transpose(1, 2)


def paged_prefill(q, out, pool, layer, block_tables, cu_q, ctx_lens, n_q, n_kv, head_dim, scale):
    """Causal attention of each sequence's new rows against its cached prefix + new keys."""
    g = n_q // n_kv
    cu = cu_q.tolist()
    for s in range(len(cu) - 1):
        r0, r1 = cu[s], cu[s + 1]
        ql = r1 - r0
        if ql == 0:
            continue
        ctx = int(ctx_lens[s])
        k, v = _gather_kv(pool, layer, n_kv, head_dim, block_tables[s], ctx)
        qs = q[r0:r1].view(ql, n_kv, g, head_dim).float()
        sc = torch.einsum("qhgd,hkd->hgqk", qs, k) * scale
        qpos = torch.arange(ctx - ql, ctx, device=q.device)[:, None]
        kpos = torch.arange(ctx, device=q.device)[None, :]
        sc = sc.masked_fill(kpos > qpos, float("-inf"))
        p = torch.softmax(sc, dim=-1)
        o = torch.einsum("hgqk,hkd->qhgd", p, v)
        out[r0:r1] = o.reshape(ql, n_q * head_dim).to(out.dtype)


def paged_decode(q, out, pool, layer, block_tables, ctx_lens, n_q, n_kv, head_dim, scale):
    g = n_q // n_kv
    for s in range(q.shape[0]):
        ctx = int(ctx_lens[s])
        if ctx == 0:
            out[s] = 0
            continue
        k, v = _gather_kv(pool, layer, n_kv, head_dim, block_tables[s], ctx)
        qs = q[s].view(n_kv, g, head_dim).float()
        sc = torch.einsum("hgd,hkd->hgk", qs, k) * scale
        p = torch.softmax(sc, dim=-1)
        o = torch.einsum("hgk,hkd->hgd", p, v)
        out[s] = o.reshape(n_q * head_dim).to(out.dtype)


def silu_and_mul(x):
    inter = x.shape[-1] // 2
    g, u = x[..., :inter].float(), x[..., inter:].float()
    return (torch.nn.functional.silu(g) * u).to(x.dtype)


def argmax(logits):
    return torch.argmax(logits.float(), dim=-1)


def moe_topk_softmax(logits, topk, renorm=True):
    p = torch.softmax(logits.float(), dim=-1)
    w, ids = torch.topk(p, topk, dim=-1)
    if renorm:
        w = w / w.sum(-1, keepdim=True)
    return w, ids.int()


def cachegen_encode(staging, levels, unit_elems, n_layers):
    """Reference of the codec front end: returns (int8 symbols, fp32 scales)."""
    flat = staging.reshape(-1).float()
    n_groups = flat.numel() // 64
    gpu = unit_elems // 64
    x = flat.view(n_groups, 64)
    gidx = torch.arange(n_groups, device=flat.device)
    unit = gidx // gpu
    gin = gidx % gpu
    is_k = (unit % 2) == 0
    lv = torch.as_tensor(levels, device=flat.device, dtype=torch.float32)[(unit // 2) % n_layers][:, None]
    tok = torch.where(is_k, gin % 32, torch.zeros_like(gin))  # key pair within the channel block
    anchor = x[gidx - tok]
    amax = anchor.abs().amax(-1, keepdim=True)
    sa = torch.where(amax > 0, amax / lv, torch.ones_like(amax))
    qa = torch.round(anchor / sa)
    d = x - qa * sa
    dmax = d.abs().amax(-1, keepdim=True)
    sd = torch.where(dmax > 0, dmax / lv, torch.ones_like(dmax))
    qd = torch.round(d / sd)
    first = (tok == 0)[:, None]
    sym = torch.where(first, qa, qd).to(torch.int8)
    scales = torch.where(first, sa, sd).squeeze(-1)
    return sym.view(-1), scales


def cachegen_decode(symbols, scales, unit_elems, dtype=torch.bfloat16):
    n_groups = scales.numel()
    gpu = unit_elems // 64
    q = symbols.view(n_groups, 64).float()
    gidx = torch.arange(n_groups, device=symbols.device)
    unit = gidx // gpu
    gin = gidx % gpu
    is_k = (unit % 2) == 0
    tok = torch.where(is_k, gin % 32, torch.zeros_like(gin))
    a = gidx - tok
    base = q[a] * scales[a][:, None]
    delta = torch.where((tok == 0)[:, None], torch.zeros_like(q), q * scales[:, None])
    return (base + delta).to(dtype).view(-1)


def moe_experts(x, w13, w2, ids, weights):
    """out[t] = sum_k weights[t,k] * W2[e] . (silu(Wg[e] x) * (Wu[e] x)),  e = ids[t,k]."""
    t, k = ids.shape
    inter = w2.shape[2]
    out = torch.zeros((t, x.shape[1]), dtype=torch.float32, device=x.device)
    for ti in range(t):
        for ki in range(k):
            e = int(ids[ti, ki])
            gu = (w13[e].float() @ x[ti].float()).to(x.dtype).float()
            a = (torch.nn.functional.silu(gu[:inter]) * gu[inter:]).to(x.dtype).float()
            out[ti] += float(weights[ti, ki]) * (w2[e].float() @ a).to(x.dtype).float()
    return out.to(x.dtype)


def lora_shrink(x, a, slots):
    """h[t] = A[slots[t]] @ x[t]; rows without an adapter (slot < 0) give zeros."""
    h = torch.zeros((x.shape[0], a.shape[1]), dtype=x.dtype, device=x.device)
    for s in torch.unique(slots).tolist():
        if s < 0:
            continue
        rows = (slots == s).nonzero(as_tuple=True)[0]
        h[rows] = (x[rows].float() @ a[s].float().t()).to(x.dtype)
    return h


def lora_expand(h, h_off, b, slots, y, y_off):
    out_dim, r_pad = b.shape[1], b.shape[2]
    for s in torch.unique(slots).tolist():
        if s < 0:
            continue
        rows = (slots == s).nonzero(as_tuple=True)[0]
        delta = h[rows, h_off:h_off + r_pad].float() @ b[s].float().t()
        y[rows, y_off:y_off + out_dim] = (y[rows, y_off:y_off + out_dim].float() + delta).to(y.dtype)
    return y


# --------------------------------------------------------------------------- rANS entropy stage
# NumPy definition of the interleaved rANS coder of csrc/kernels/rans.hip (same tables, same
# stream layout, same bytes): the oracle of the GPU kernels and the codec of CPU-only hosts.
RANS_BITS = 12
RANS_M = 1 << RANS_BITS
RANS_LOW = 1 << 23


def rans_tables(sym, n_ctx: int):
    """-> (freq [n_ctx, 256] uint16 summing to 4096 per row, cum [n_ctx, 256] uint32)."""
    import numpy as np

    sym = np.asarray(sym).view(np.uint8).reshape(n_ctx, -1)
    total = sym.shape[1]
    freq = np.zeros((n_ctx, 256), dtype=np.int64)
    for c in range(n_ctx):
        cnt = np.bincount(sym[c], minlength=256).astype(np.int64)
        f = np.where(cnt > 0, np.maximum(1, (cnt * RANS_M + total // 2) // total), 0)
        i = int(np.argmax(f))  # first index among equals
        f[i] += RANS_M - int(f.sum())
        if f[i] < 1:
            raise ValueError("frequency table cannot be normalised")
        freq[c] = f
    cum = np.cumsum(freq, axis=1) - freq
    return freq.astype(np.uint16), cum.astype(np.uint32)


def rans_encode(sym, n_ctx: int, spc: int):
    """-> (freq uint16 [n_ctx, 256], states uint32 [n_ctx * spc], sizes uint16, coded uint8)."""
    import numpy as np

    sym = np.asarray(sym).view(np.uint8).reshape(n_ctx, -1)
    ctx_len = sym.shape[1]
    length = ctx_len // spc
    cap = 2 * length
    freq, cum = rans_tables(sym, n_ctx)
    n_streams = n_ctx * spc
    buf = np.zeros((n_streams, cap), dtype=np.uint8)
    pos = np.full(n_streams, cap, dtype=np.int64)
    x = np.full(n_streams, RANS_LOW, dtype=np.uint64)
    ctx_of = np.repeat(np.arange(n_ctx), spc)
    rows = np.arange(n_streams)
    per = sym.reshape(n_ctx, length, spc)  # [ctx, k, j]
    for k in range(length - 1, -1, -1):
        s = per[:, k, :].reshape(-1)
        f = freq[ctx_of, s].astype(np.uint64)
        c = cum[ctx_of, s].astype(np.uint64)
        x_max = np.uint64((RANS_LOW >> RANS_BITS) << 8) * f
        while True:
            m = x >= x_max
            if not m.any():
                break
            pos[m] -= 1
            buf[rows[m], pos[m]] = (x[m] & np.uint64(0xFF)).astype(np.uint8)
            x[m] >>= np.uint64(8)
        x = ((x // f) << np.uint64(RANS_BITS)) + (x % f) + c
    sizes = (cap - pos).astype(np.uint16)
    coded = np.concatenate([buf[i, pos[i]:] for i in range(n_streams)]) if n_streams else np.zeros(0, np.uint8)
    return freq, x.astype(np.uint32), sizes, coded


def rans_decode(freq, states, sizes, coded, n: int, n_ctx: int, spc: int):
    """-> uint8 symbols [n]."""
    import numpy as np

    freq = np.asarray(freq, dtype=np.uint16).reshape(n_ctx, 256)
    cum = (np.cumsum(freq.astype(np.int64), axis=1) - freq).astype(np.int64)
    ctx_len = n // n_ctx
    length = ctx_len // spc
    n_streams = n_ctx * spc
    slot2sym = np.zeros((n_ctx, RANS_M), dtype=np.uint8)
    for c in range(n_ctx):
        slot2sym[c] = np.repeat(np.arange(256, dtype=np.uint8), freq[c].astype(np.int64))[:RANS_M]
    ctx_of = np.repeat(np.arange(n_ctx), spc)
    sizes64 = np.asarray(sizes).astype(np.int64)
    rp = np.cumsum(sizes64) - sizes64
    x = np.asarray(states).astype(np.uint64).copy()
    coded = np.concatenate([np.asarray(coded, dtype=np.uint8), np.zeros(8, np.uint8)])
    limit = coded.size - 8
    out = np.zeros((n_ctx, length, spc), dtype=np.uint8)
    f64 = freq.astype(np.uint64)
    for k in range(length):
        slot = (x & np.uint64(RANS_M - 1)).astype(np.int64)
        s = slot2sym[ctx_of, slot]
        out[:, k, :] = s.reshape(n_ctx, spc)
        x = f64[ctx_of, s] * (x >> np.uint64(RANS_BITS)) + slot.astype(np.uint64) - cum[ctx_of, s].astype(np.uint64)
        while True:
            m = x < np.uint64(RANS_LOW)
            if not m.any():
                break
            b = np.where(rp[m] < limit, coded[np.minimum(rp[m], limit)], 0).astype(np.uint64)
            x[m] = (x[m] << np.uint64(8)) | b
            rp[m] += 1
    return out.reshape(-1)


# --------------------------------------------------------------------------- 32-bit residual stream, latent attention, group routing
# (PyTorch definitions of csrc/kernels/latent.hip; fp32 math, results rounded to the activation dtype)
def embed_scale(ids, embed, scale):
    return embed[ids.long()].float() * scale


def add_rms_norm(residual, delta, weight, eps, out_dtype, want_out=True):
    if delta is not None:
        residual.add_(delta.float())
    if not want_out:
        return None
    inv = torch.rsqrt(residual.pow(2).mean(-1, keepdim=True) + eps)
    return (residual * inv * weight).to(out_dtype)


def gated_add_rms_norm(residual, deltas, gate, gate_bias, extra, extra_vec, weight, eps, out_dtype, want_out=True):
    total = None
    for d, w, c in deltas:
        d = d.float()
        if w is not None:
            d = d * torch.rsqrt(d.pow(2).mean(-1, keepdim=True) + eps) * w
        total = d * c if total is None else total + d * c
    if total is not None:
        if gate is not None:
            total = total * torch.sigmoid(gate.float() + (gate_bias if gate_bias is not None else 0.0))
        residual.add_(total)
    if extra is not None:
        residual.add_(extra)
    if extra_vec is not None:
        residual.add_(extra_vec)
    if not want_out:
        return None
    return (residual * torch.rsqrt(residual.pow(2).mean(-1, keepdim=True) + eps) * weight).to(out_dtype)


def rms_norm_add(residual, delta, weight, eps, out_dtype, want_out=True):
    d = delta.float()
    residual.add_(d * torch.rsqrt(d.pow(2).mean(-1, keepdim=True) + eps) * weight)
    return residual.to(out_dtype) if want_out else None


def glu_act(x, act):
    inter = x.shape[1] // 2
    g, u = x[:, :inter].float(), x[:, inter:].float()
    a = torch.nn.functional.silu(g) if act == "silu" else torch.nn.functional.gelu(g, approximate="tanh")
    return (a * u).to(x.dtype)


def route_softmax(logits, n, experts, groups, keep, topk, bias, route_scale, park_in_bucket):
    t = logits.shape[0]
    s = torch.softmax(logits[:, :n].float(), dim=-1)
    c = s + bias if bias is not None else s.clone()
    per = n // groups
    score = c.view(t, groups, per).max(-1).values
    order = torch.sort(score, dim=-1, descending=True, stable=True).indices[:, :keep]
    allowed = torch.zeros((t, groups), dtype=torch.bool)
    allowed.scatter_(1, order, True)
    c = torch.where(allowed[:, :, None].expand(t, groups, per).reshape(t, n), c, torch.full_like(c, -math.inf))
    ids = torch.sort(c, dim=-1, descending=True, stable=True).indices[:, :topk]
    w = s.gather(1, ids) * route_scale
    if experts == n:
        return w, ids.int(), None
    ident = ids >= experts
    gate = torch.where(ident, w, torch.zeros_like(w)).sum(-1)
    ids = torch.where(ident, torch.full_like(ids, experts if park_in_bucket else 0), ids)
    return torch.where(ident, torch.zeros_like(w), w), ids.int(), gate


def rms_norm_rows(x, weight, eps):
    xf = x.float()
    return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * weight).to(x.dtype)


def _rotate_pairs(x, cs, dims):
    """x [..., n] float: the first ``dims`` columns rotate in pairs (2i, 2i+1); cs [..., dims] = cos | sin."""
    half = dims // 2
    c, s = cs[..., :half], cs[..., half:]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def latent_cache_view(pool, offset, entry):
    """A layer's part of a [pages, page_elems] pool as [pages, PAGE, entry]."""
    return pool[:, offset:offset + PAGE * entry].view(pool.shape[0], PAGE, entry)


def latent_kv_write(x, weight, positions, slots, cos_sin, pool, offset, rank, rot, rot_dims, eps):
    xf = x.float()
    c = xf[:, :rank]
    c = c * torch.rsqrt(c.pow(2).mean(-1, keepdim=True) + eps) * weight
    r = _rotate_pairs(xf[:, rank:rank + rot], cos_sin[positions.long()], rot_dims)
    view = latent_cache_view(pool, offset, rank + rot)
    ok = slots >= 0
    s = slots[ok].long()
    view[s // PAGE, s % PAGE] = torch.cat([c, r], dim=-1)[ok].to(pool.dtype)


def rope_pairs(q, positions, cos_sin, col0, rot_dims):
    """q [T, heads, d]: columns [col0, col0 + rot_dims) of every head, in place."""
    part = q[:, :, col0:col0 + rot_dims].float()
    q[:, :, col0:col0 + rot_dims] = _rotate_pairs(part, cos_sin[positions.long()][:, None, :], rot_dims).to(q.dtype)


def latent_attention(q_lat, q_rot, pool, offset, block_tables, row_seq, positions, sink, scale, out):
    t, heads, rank = q_lat.shape
    rot = q_rot.shape[2]
    view = latent_cache_view(pool, offset, rank + rot)
    seqs = row_seq.long() if row_seq is not None else torch.arange(t)
    for s in torch.unique(seqs).tolist():
        rows = (seqs == s).nonzero(as_tuple=True)[0]
        pos = positions[rows].long()
        ctx = int(pos.max()) + 1
        pages = block_tables[s, :(ctx + PAGE - 1) // PAGE].long()
        kv = view[pages].reshape(-1, rank + rot)[:ctx].float()
        q = torch.cat([q_lat[rows].float(), q_rot[rows].float()], dim=-1) * scale
        sc = torch.einsum("qhd,kd->qhk", q, kv)
        sc = sc.masked_fill(torch.arange(ctx)[None, None, :] > pos[:, None, None], float("-inf"))
        m = sc.max(-1).values
        if sink is not None:
            m = torch.maximum(m, sink[None, :])
        e = torch.exp(sc - m[..., None])
        den = e.sum(-1)
        if sink is not None:
            den = den + torch.exp(sink[None, :] - m)
        o = torch.einsum("qhk,kd->qhd", e, kv[:, :rank]) / den[..., None]
        out[rows] = o.to(out.dtype)
    return out


def sigmoid_gate(y, g):
    y.copy_((y.float() * torch.sigmoid(g.float())[..., None]).to(y.dtype))
    return y


def relu_sq(x):
    return torch.relu(x.float()).pow(2).to(x.dtype)


def glu_clamp(x, limit, alpha, up_bias):
    inter = x.shape[-1] // 2
    g = x[..., :inter].float().clamp(max=limit)
    u = x[..., inter:].float().clamp(-limit, limit)
    return (g * torch.sigmoid(alpha * g) * (u + up_bias)).to(x.dtype)


def group_topk(logits, experts, groups, keep, topk, route_scale, extra, normalize=False):
    t = logits.shape[0]
    s = torch.sigmoid(logits[:, :experts].float())
    per = experts // groups
    gs = s.view(t, groups, per)
    score = gs.topk(min(2, per), dim=-1).values.sum(-1)
    # stable descending order: ties go to the lower index
    order = torch.sort(score, dim=-1, descending=True, stable=True).indices[:, :keep]
    allowed = torch.zeros((t, groups), dtype=torch.bool)
    allowed.scatter_(1, order, True)
    masked = torch.where(allowed[:, :, None].expand(t, groups, per).reshape(t, experts), s, torch.full_like(s, -1.0))
    ids = torch.sort(masked, dim=-1, descending=True, stable=True).indices[:, :topk]
    w = s.gather(1, ids)
    if normalize:
        w = w / (w.sum(-1, keepdim=True) + 1e-20)
    w = w * route_scale
    ex = torch.sigmoid(logits[:, experts].float()) if extra else None
    return w, ids.int(), ex


def moe_finish(residual, y, weights, pos, shared, gate):
    t, k = weights.shape
    if k:  # a pair of weight 0 is skipped, as in the kernel: its row of y may never have been written
        rows = torch.where((weights != 0)[:, :, None], y[pos.long()].view(t, k, -1).float(), 0.0)
        residual.add_((rows * weights[:, :, None]).sum(1))
    if shared is not None:
        residual.add_(shared.float() * (gate[:, None] if gate is not None else 1.0))
    return residual


# --------------------------------------------------------------------------- recurrent mixers, windowed attention, Dynamic Tanh
def add_dyt_norm(residual, deltas, weight, bias, alpha, out_dtype, want_out=True):
    for d, scale in deltas:
        residual.add_(d.float() * scale)
    if not want_out:
        return None
    return (torch.tanh(residual * alpha) * weight + bias).to(out_dtype)


def _rotate_rows(x, pos, cos_sin, dims, layout):
    """x fp32 [T, heads, d]: the first ``dims`` channels of every head turn by the table row of the
    token's position; pairs (i, i + dims / 2) for layout 0, (2 i, 2 i + 1) for layout 1."""
    if dims == 0:
        return x
    cs = cos_sin[pos.long()]
    c, s = cs[:, None, :dims // 2], cs[:, None, dims // 2:]
    out = x.clone()
    if layout == 0:
        u, v = x[..., :dims // 2], x[..., dims // 2:dims]
        out[..., :dims // 2] = u * c - v * s
        out[..., dims // 2:dims] = v * c + u * s
    else:
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = u * c - v * s
        out[..., 1:dims:2] = v * c + u * s
    return out


def recurrent_scan(proj, q_col, k_col, v_col, heads, dim, vdim, gated, state, state_off, seq_cu, seq_state, positions,
                   decay, cos_sin, rot_dims, layout, k_scale, gate_bias, gate_lower, act=False):
    t = proj.shape[0]
    out = torch.zeros((t, heads, vdim), dtype=torch.float32)
    q = proj[:, q_col:q_col + heads * dim].float().view(t, heads, dim)
    k = proj[:, k_col:k_col + heads * dim].float().view(t, heads, dim)
    v = proj[:, v_col:v_col + heads * vdim].float().view(t, heads, vdim)
    if gated:
        q = torch.nn.functional.silu(q)
        lower = gate_lower.view(1, heads, dim)
        a = lower + (1 - lower) * torch.sigmoid(k + gate_bias.view(1, heads, dim))
        k = 1 - a
    else:
        if act:
            q, k, v = (torch.nn.functional.silu(x) for x in (q, k, v))
        q = _rotate_rows(q, positions, cos_sin, rot_dims, layout)
        k = _rotate_rows(k, positions, cos_sin, rot_dims, layout) * k_scale
        a = decay.view(1, heads, 1).expand(t, heads, dim)
    cu, slots = seq_cu.tolist(), seq_state.tolist()
    for s, slot in enumerate(slots):
        r0, r1 = cu[s], cu[s + 1]
        if slot < 0 or r1 <= r0:
            continue
        S = state[slot, state_off:state_off + heads * dim * vdim].view(heads, dim, vdim)
        if int(positions[r0]) == 0:
            S.zero_()
        for r in range(r0, r1):
            S.mul_(a[r].unsqueeze(-1)).add_(k[r].unsqueeze(-1) * v[r].unsqueeze(1))
            out[r] = torch.einsum("hdv,hd->hv", S, q[r])
    return out


def gla_prepare(proj, q_col, k_col, z, z_bias, heads, dim, q_scale, tau):
    t = proj.shape[0]
    q = proj[:, q_col:q_col + heads * dim].float() * q_scale
    k = proj[:, k_col:k_col + heads * dim].float()
    a = torch.exp(torch.nn.functional.logsigmoid(z.float() + z_bias) / tau)
    return torch.stack([q.view(t, heads, dim), k.view(t, heads, dim), a.view(t, heads, dim)], dim=2).contiguous()


def mlstm_prepare(proj, q_col, k_col, gate_logits, bias_i, bias_f, cap, heads, dim, q_scale, state, m_off, seq_cu,
                  seq_state, positions):
    t = proj.shape[0]
    q = proj[:, q_col:q_col + heads * dim].float().view(t, heads, dim) * q_scale
    k = proj[:, k_col:k_col + heads * dim].float().view(t, heads, dim)
    gi = cap * torch.tanh((gate_logits[:, :heads] + bias_i) / cap)
    gf = torch.nn.functional.logsigmoid(cap * torch.tanh((gate_logits[:, heads:] + bias_f) / cap))
    dec = torch.zeros((t, heads), dtype=torch.float32)
    wr = torch.zeros((t, heads), dtype=torch.float32)
    mrow = torch.zeros((t, heads), dtype=torch.float32)
    cu, slots = seq_cu.tolist(), seq_state.tolist()
    for s, slot in enumerate(slots):
        r0, r1 = cu[s], cu[s + 1]
        if slot < 0 or r1 <= r0:
            continue
        m = state[slot, m_off:m_off + heads]
        if int(positions[r0]) == 0:
            m.zero_()
        for r in range(r0, r1):
            new = torch.maximum(gf[r] + m, gi[r])
            dec[r] = torch.exp(gf[r] + m - new)
            wr[r] = torch.exp(gi[r] - new)
            mrow[r] = new
            m.copy_(new)
    prep = torch.stack([q, k * wr[:, :, None], dec[:, :, None].expand(t, heads, dim)], dim=2).contiguous()
    return prep, mrow


def prepared_scan(prep, proj, v_col, heads, dim, vdim, cols, unit_col, state, state_off, seq_cu, seq_state, positions):
    t = proj.shape[0]
    out = torch.zeros((t, heads, cols), dtype=torch.float32)
    v = torch.zeros((t, heads, cols), dtype=torch.float32)
    v[:, :, :vdim] = proj[:, v_col:v_col + heads * vdim].float().view(t, heads, vdim)
    if unit_col:
        v[:, :, vdim] = 1.0
    cu, slots = seq_cu.tolist(), seq_state.tolist()
    for s, slot in enumerate(slots):
        r0, r1 = cu[s], cu[s + 1]
        if slot < 0 or r1 <= r0:
            continue
        S = state[slot, state_off:state_off + heads * dim * cols].view(heads, dim, cols)
        if int(positions[r0]) == 0:
            S.zero_()
        for r in range(r0, r1):
            S.mul_(prep[r, :, 2].unsqueeze(-1)).add_(prep[r, :, 1].unsqueeze(-1) * v[r].unsqueeze(1))
            out[r] = torch.einsum("hdv,hd->hv", S, prep[r, :, 0])
    return out


def head_finish(o, eps, out_dtype, vdim, stab, unit, weight, gate, gate_act):
    t, heads, _ = o.shape
    y = o[:, :, :vdim]
    if stab is not None:
        y = y / (torch.maximum(o[:, :, vdim].abs(), torch.exp(-stab)) + 1e-6)[:, :, None]
    if unit:
        y = y * torch.rsqrt(y.pow(2).mean(-1, keepdim=True) + eps)
    if weight is not None:
        y = y * (weight if weight.numel() == vdim else weight.view(heads, vdim))
    y = y.reshape(t, heads * vdim)
    if gate is not None:
        g = gate.float()
        y = y * (torch.nn.functional.silu(g) if gate_act == "silu" else torch.sigmoid(g))
    return y.to(out_dtype)


def qk_norm_write(proj, heads, kv_heads, dim, vdim, positions, slots, pool, cache_off, eps, temp_coef, temp_every, own,
                  v_heads=None, q_weight=None, k_weight=None, cos_sin=None, rot_dims=0, layout=0):
    t = proj.shape[0]
    nq, nk = heads * dim, kv_heads * dim
    v_heads = kv_heads if v_heads is None else v_heads

    def unit(x, w):
        x = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)
        if w is not None:
            x = x * w
        return _rotate_rows(x, positions, cos_sin, rot_dims, layout) if rot_dims else x

    q = unit(proj[:, :nq].float().view(t, heads, dim), q_weight)
    if temp_coef != 0.0:
        steps = torch.floor((positions.double() + 1.0) / temp_every).float()
        q = q * (1.0 + temp_coef * torch.log(steps + 1.0))[:, None, None]
    if own:
        k = unit(proj[:, nq:nq + nk].float().view(t, kv_heads, dim), k_weight).to(pool.dtype)
        v = proj[:, nq + nk:nq + nk + v_heads * vdim].reshape(t, v_heads, vdim).to(pool.dtype)
        kc, vc = window_cache_views(pool, cache_off, kv_heads, dim, vdim, v_heads)
        ok = slots >= 0
        pg, off = (slots[ok] // PAGE).long(), (slots[ok] % PAGE).long()
        kc[pg, off] = k[ok]
        vc[pg, off] = v[ok]
    return q.to(proj.dtype)


def head_rms_norm(o, eps, weight, gate, out_dtype):
    t, heads, vdim = o.shape
    y = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps)
    if weight is not None:
        y = y * weight
    y = y.reshape(t, heads * vdim)
    if gate is not None:
        y = y * torch.nn.functional.silu(gate.float())
    return y.to(out_dtype)


def window_cache_views(pool, cache_off, kv_heads, dim, vdim, v_heads=None):
    """K [pages, PAGE, kv_heads, dim] and V [pages, PAGE, kv_heads, vdim] of one layer: views of the pool
    (indexed reads and writes go through).  In a page, K is stored key by key ([PAGE][kv_heads * dim]) and V
    transposed ([kv_heads * vdim][PAGE]: a channel's 64 keys are contiguous, which is what the second matrix
    product of the attention kernels reads)."""
    v_heads = kv_heads if v_heads is None else v_heads  # fewer when several key maps share a value head
    nk, nv = PAGE * kv_heads * dim, PAGE * v_heads * vdim
    k = pool[:, cache_off:cache_off + nk].view(pool.shape[0], PAGE, kv_heads, dim)
    v = pool[:, cache_off + nk:cache_off + nk + nv].view(pool.shape[0], v_heads, vdim, PAGE).permute(0, 3, 1, 2)
    return k, v


def pool_blocks(pool, cache_off, pool_off, kv_heads, dim, vdim, block_tables, row_seq, positions, slots, block):
    kc, vc = window_cache_views(pool, cache_off, kv_heads, dim, vdim)
    pk, pv = window_cache_views(pool, cache_off + pool_off, kv_heads, dim, vdim)
    for r in range(positions.numel()):
        p = int(positions[r])
        if int(slots[r]) < 0 or (p + 1) % block:
            continue
        s = r if row_seq is None else int(row_seq[r])
        b = p // block
        idx = torch.arange(b * block, p + 1)
        pages = block_tables[s].long()[idx // PAGE]
        dst = int(block_tables[s, b // PAGE])
        pk[dst, b % PAGE] = (kc[pages, idx % PAGE].float().sum(0) / block).to(pool.dtype)
        pv[dst, b % PAGE] = (vc[pages, idx % PAGE].float().sum(0) / block).to(pool.dtype)


def diff_heads(u, kv_heads, lam, eps, post, out_dtype):
    t, h2, vdim = u.shape
    heads = h2 // 2
    a = u.view(t, kv_heads, 2, heads // kv_heads, vdim)
    o = (a[:, :, 0] - lam * a[:, :, 1]).reshape(t, heads, vdim)
    o = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps) * post
    return o.reshape(t, heads * vdim).to(out_dtype)


def short_conv_qkv(proj, conv_w, heads, kv_heads, dim, vdim, state, state_off, seq_cu, seq_state, positions, slots,
                   cos_sin, rot_dims, layout, pool, cache_off):
    t = proj.shape[0]
    taps = conv_w.shape[1]
    chans = heads * dim + kv_heads * (dim + vdim)
    u = proj[:, :chans].float()
    y = torch.zeros((t, chans), dtype=torch.float32)
    cu, st = seq_cu.tolist(), seq_state.tolist()
    for s, slot in enumerate(st):
        r0, r1 = cu[s], cu[s + 1]
        if slot < 0 or r1 <= r0:
            continue
        tail = state[slot, state_off:state_off + (taps - 1) * chans].view(taps - 1, chans)
        if int(positions[r0]) == 0:
            tail.zero_()
        ext = torch.cat([tail, u[r0:r1]], dim=0)  # the rows before the chunk, then the chunk
        n = r1 - r0
        for j in range(taps):
            y[r0:r1] += conv_w[:, j] * ext[j:j + n]
        if taps > 1:
            tail.copy_(ext[n:n + taps - 1].clone())
    y = y.to(proj.dtype).float()
    nq, nk = heads * dim, kv_heads * dim
    q = _rotate_rows(y[:, :nq].reshape(t, heads, dim), positions, cos_sin, rot_dims, layout).to(proj.dtype)
    k = _rotate_rows(y[:, nq:nq + nk].reshape(t, kv_heads, dim), positions, cos_sin, rot_dims, layout).to(pool.dtype)
    v = y[:, nq + nk:].reshape(t, kv_heads, vdim).to(pool.dtype)
    kc, vc = window_cache_views(pool, cache_off, kv_heads, dim, vdim)
    ok = slots >= 0
    pg, off = (slots[ok] // PAGE).long(), (slots[ok] % PAGE).long()
    kc[pg, off] = k[ok]
    vc[pg, off] = v[ok]
    return q


def window_attention(q, pool, cache_off, kv_heads, vdim, block_tables, row_seq, positions, window, keep_first, scale,
                     softcap, sink, out, own_values=False, mode=0, pool_block=0, pool_off=0, maps=1):
    t, heads, dim = q.shape
    kc, vc = window_cache_views(pool, cache_off, kv_heads, dim, vdim, kv_heads // maps)
    if pool_block:
        pk, pv = window_cache_views(pool, cache_off + pool_off, kv_heads, dim, vdim, kv_heads // maps)
    rep = heads // kv_heads
    for r in range(t):
        s = r if row_seq is None else int(row_seq[r])
        p = int(positions[r])
        lo = p - p % window if mode == 1 else max(0, p - window + 1)
        keys = list(range(min(keep_first, lo))) + list(range(lo, p + 1))
        idx = torch.tensor(keys)
        pages = block_tables[s].long()[idx // PAGE]
        kk = kc[pages, idx % PAGE].float()       # [keys, kv_heads, dim]
        vv = vc[pages, idx % PAGE].float()       # [keys, value heads, vdim]
        nb = max(0, (p - window + 1) // pool_block) if pool_block else 0
        if nb:  # one pooled entry per block of tokens that lies wholly before the window
            idx = torch.arange(nb)
            pages = block_tables[s].long()[idx // PAGE]
            kk = torch.cat([pk[pages, idx % PAGE].float(), kk])
            vv = torch.cat([pv[pages, idx % PAGE].float(), vv])
        sc = torch.einsum("hd,khd->hk", q[r].float(), kk.repeat_interleave(rep, dim=1)) * scale
        if softcap > 0:
            sc = softcap * torch.tanh(sc / softcap)
        if sink is None:
            w = torch.softmax(sc, dim=-1)
        else:
            mx = torch.maximum(sc.max(-1).values, sink)
            e = torch.exp(sc - mx[:, None])
            w = e / (e.sum(-1) + torch.exp(sink - mx))[:, None]
        if own_values:
            out[r, :, 0] = torch.einsum("hk,khv->hv", w, vv.repeat_interleave(rep * maps, dim=1))
        else:
            out[r] = torch.einsum("hk,kgv->hgv", w, vv)
    return out


def mix_heads(u, talk, out_dtype):
    t, heads, kv_heads, vdim = u.shape
    rep = heads // kv_heads
    own = torch.arange(heads) // rep
    # out[t, h] = sum_g talk[h, g] u[t, g, kv(h)]
    sel = u[:, :, own, :]                          # [t, g, h, vdim]
    return torch.einsum("hg,tghv->thv", talk, sel).reshape(t, heads * vdim).to(out_dtype)


def xielu(x, act):
    z = x.float()
    pos = act[0] * z * z + 0.5 * z
    neg = act[1] * (torch.expm1(z) - z) + 0.5 * z
    return torch.where(z > 0, pos, neg).to(x.dtype)
