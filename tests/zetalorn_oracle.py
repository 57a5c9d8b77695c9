"""Zetalorn in float64, written from the design's equations: one function per mechanism, whole
sequences recomputed from their first token, keys and values per head in plain tensors.  Nothing here is
shared with the engine, its ops or its reference definitions.  Also makers of small random checkpoints.

A checkpoint is (config dict, {tensor name: tensor}); ``run`` returns the logits of every position and the
residual stream after every layer run (a looped layer counts once per pass).
"""

from __future__ import annotations

import json
import math
import os

import torch

F64 = torch.float64


# ------------------------------------------------------------------ small parts
def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def scalar_norm(x, g, eps):
    return rms(x, eps) * g


def sigmoid(x):
    return 1.0 / (1.0 + torch.exp(-x))


def silu(x):
    return x * sigmoid(x)


def frequencies(rot):
    dims = rot["dims"]
    f = torch.tensor([rot["base"] ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F64)
    scaling = rot.get("scaling")
    if scaling:
        f = f / scaling["factor"]
    return f


def rotate(x, pos, rot, interleaved):
    """x [T, heads, dim]; the first rot['dims'] channels of every head turn by pos * f_i."""
    dims = rot["dims"]
    if dims == 0:
        return x
    ang = pos.to(F64)[:, None] * frequencies(rot)[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    out = x.clone()
    if interleaved:
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = u * c - v * s
        out[..., 1:dims:2] = v * c + u * s
    else:
        u, v = x[..., :dims // 2], x[..., dims // 2:dims]
        out[..., :dims // 2] = u * c - v * s
        out[..., dims // 2:dims] = v * c + u * s
    return out


def softmax_rows(scores, seen):
    """scores [T, K], seen bool [T, K] -> weights, rows that see nothing are zero."""
    s = scores.masked_fill(~seen, -math.inf)
    m = s.max(-1, keepdim=True).values
    m = torch.where(torch.isinf(m), torch.zeros_like(m), m)
    e = torch.exp(s - m)
    e = torch.where(seen, e, torch.zeros_like(e))
    return e / e.sum(-1, keepdim=True).clamp_min(1e-300)


def chunk_mask(t, size):
    i = torch.arange(t)[:, None]
    j = torch.arange(t)[None, :]
    return (j <= i) & (i // size == j // size)


def window_mask(t, size):
    i = torch.arange(t)[:, None]
    j = torch.arange(t)[None, :]
    return (j <= i) & (i - j < size)


def block_mask(t, size, pool):
    """[T, blocks]: block b is seen by position i when its last token is at or before i - size."""
    nb = t // pool
    i = torch.arange(t)[:, None]
    b = torch.arange(nb)[None, :]
    return b * pool + pool - 1 <= i - size


# ------------------------------------------------------------------ mixers
def differential_attention(h, m, w, eps, prefix):
    t = h.shape[0]
    hq, g, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(t)
    q = (h @ w[prefix + "q"].T).view(t, hq * 2, d)
    k = (h @ w[prefix + "k"].T).view(t, g * 2, d)
    v = (h @ w[prefix + "v"].T).view(t, g, dv)
    q = rotate(rms(q, eps) * w[prefix + "q.norm"], pos, m["rot"], True)
    k = rotate(rms(k, eps) * w[prefix + "k.norm"], pos, m["rot"], True)
    lam = (torch.exp((w[prefix + "lq1"] * w[prefix + "lk1"]).sum())
           - torch.exp((w[prefix + "lq2"] * w[prefix + "lk2"]).sum()) + m["diff"])
    mask = m.get("mask")
    seen = chunk_mask(t, mask["size"]) if mask else window_mask(t, t + 1)
    outs = []
    for head in range(hq):
        kv = head // (hq // g)
        a = []
        for which in range(2):
            s = (q[:, 2 * head + which] @ k[:, 2 * kv + which].T) * m["scale"]
            a.append(softmax_rows(s, seen) @ v[:, kv])
        o = a[0] - lam * a[1]
        outs.append(rms(o, eps) * (1.0 - m["diff"]))
    return torch.cat(outs, -1) @ w[prefix + "o"].T


def pooled_window_attention(h, m, w, eps, prefix):
    t = h.shape[0]
    hq, g, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(t)
    q = (h @ w[prefix + "q"].T).view(t, hq, d)
    k = (h @ w[prefix + "k"].T).view(t, g, d)
    v = (h @ w[prefix + "v"].T).view(t, g, dv)
    q = rotate(rms(q, eps) * w[prefix + "q.norm"], pos, m["rot"], False)
    k = rotate(rms(k, eps) * w[prefix + "k.norm"], pos, m["rot"], False)
    mask = m.get("mask") or {}
    size = mask.get("size", t + 1)
    pool = mask.get("pool", 0)
    seen = window_mask(t, size)
    nb = t // pool if pool else 0
    if nb:
        seen = torch.cat([seen, block_mask(t, size, pool)], 1)
    outs = []
    for head in range(hq):
        kv = head // (hq // g)
        keys, vals = k[:, kv], v[:, kv]
        if nb:
            keys = torch.cat([keys, keys[:nb * pool].view(nb, pool, d).mean(1)], 0)
            vals = torch.cat([vals, vals[:nb * pool].view(nb, pool, dv).mean(1)], 0)
        s = (q[:, head] @ keys.T) * m["scale"]
        outs.append(softmax_rows(s, seen) @ vals)
    return torch.cat(outs, -1) @ w[prefix + "o"].T


def lightning_attention(h, m, w, eps, prefix):
    t = h.shape[0]
    n, d, dv = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ w[prefix + "q"].T).view(t, n, d)
    k = silu(h @ w[prefix + "k"].T).view(t, n, d)
    v = silu(h @ w[prefix + "v"].T).view(t, n, dv)
    out = torch.zeros(t, n, dv, dtype=F64)
    for head in range(n):
        state = torch.zeros(d, dv, dtype=F64)
        for i in range(t):
            state = m["decay"][head] * state + torch.outer(k[i, head], v[i, head])
            out[i, head] = state.T @ q[i, head]
    y = rms(out.reshape(t, n * dv), eps) * w[prefix + "norm"]
    return (y * sigmoid(h @ w[prefix + "g"].T)) @ w[prefix + "o"].T


def parallel_mixer(h, m, w, eps, prefix):
    left = pooled_window_attention(h, m["left"], w, eps, prefix + "left.")
    right = lightning_attention(h, m["right"], w, eps, prefix + "right.")
    return 0.5 * (rms(left, eps) * w[prefix + "left.out"] + rms(right, eps) * w[prefix + "right.out"])


# ------------------------------------------------------------------ feed-forward
def choose_experts(scores, top, count, keep):
    """scores [E] -> the chosen expert indices (sorting, ties to the lower index)."""
    e = scores.numel()
    per = e // count
    group = []
    for gi in range(count):
        part = sorted(scores[gi * per:(gi + 1) * per].tolist(), reverse=True)
        group.append(sum(part[:2]))
    kept = sorted(range(count), key=lambda gi: (-group[gi], gi))[:keep]
    allowed = [i for i in range(e) if i // per in kept]
    return sorted(allowed, key=lambda i: (-scores[i].item(), i))[:top]


def expert(h, w, prefix, limit):
    gate = torch.clamp(h @ w[prefix + "gate"].T, max=limit)
    up = torch.clamp(h @ w[prefix + "up"].T, -limit, limit)
    return (gate * sigmoid(1.702 * gate) * (up + 1.0)) @ w[prefix + "down"].T


def mixture(h, f, w, prefix):
    r = f["router"]
    groups = r.get("groups") or {"count": 1, "keep": 1}
    scores = sigmoid(h @ w[prefix + "router"].T)
    out = torch.zeros_like(h)
    for i in range(h.shape[0]):
        ids = choose_experts(scores[i], r["top"], groups["count"], groups["keep"])
        total = sum(scores[i, e] for e in ids) + 1e-20
        for e in ids:
            out[i] += scores[i, e] / total * expert(h[i:i + 1], w, "%se%d." % (prefix, e), f["expert"]["limit"])[0]
    return out


# ------------------------------------------------------------------ the model
def layer_runs(cfg):
    """The layer index of every run, and the pass (None outside the loop) whose start it is."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    runs = [(i, None) for i in range(loop["start"])]
    for t in range(loop["times"]):
        for i in range(loop["start"], loop["stop"]):
            runs.append((i, t if i == loop["start"] else None))
    runs += [(i, None) for i in range(loop["stop"], n)]
    return runs


def run(cfg, weights, tokens):
    w = {k: v.to(F64) for k, v in weights.items() if v.dtype != torch.int32}
    eps = cfg["norm"]["eps"]
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    emb = x.clone()
    after = []
    for li, start_of in layer_runs(cfg):
        if start_of is not None:
            if start_of > 0:
                x = x + emb
            x = x + w["loop.step"][start_of]
        spec = cfg["layers"][li]
        p = "l%d." % li
        h = scalar_norm(x, w[p + "norm1"], eps)
        if spec["type"] == "attention":
            y = differential_attention(h, spec["mixer"], w, eps, p + "mix.")
        else:
            y = parallel_mixer(h, spec["mixer"], w, eps, p + "mix.")
        x = x + y * sigmoid(h @ w[p + "rg1"].T + w[p + "rg1.b"])
        if spec.get("mlp") is not None:
            h = scalar_norm(x, w[p + "norm2"], eps)
            y = mixture(h, spec["mlp"], w, p + "mlp.")
            x = x + y * sigmoid(h @ w[p + "rg2"].T + w[p + "rg2.b"])
        after.append(x.clone())
    logits = (scalar_norm(x, w["final.norm"], eps) @ w["head"].T) * cfg.get("logit_scale", 1.0)
    return logits, torch.stack(after)


# ------------------------------------------------------------------ checkpoints
def attention_spec(heads=2, kv_heads=1, dim=16, vdim=24, chunk=70, rot_dims=8, base=500.0, factor=4.0, diff=0.2,
                   scale=None):
    rot = {"base": base, "dims": rot_dims}
    if factor:
        rot["scaling"] = {"factor": factor}
    return {"type": "attention",
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "diff": diff, "rot": rot,
                      "mask": {"size": chunk}, "scale": scale if scale is not None else dim ** -0.5}}


def parallel_spec(heads=2, kv_heads=2, dim=16, vdim=8, window=40, pool=5, rot_dims=16, base=3000.0, r_heads=3,
                  r_dim=8, r_vdim=12, decay=None, scale=None):
    decay = decay or [0.5 + 0.49 * (i + 1) / r_heads for i in range(r_heads)]
    return {"type": "parallel",
            "mixer": {"left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
                               "mask": {"size": window, "pool": pool}, "rot": {"base": base, "dims": rot_dims},
                               "scale": scale if scale is not None else dim ** -0.5},
                      "right": {"heads": r_heads, "dim": r_dim, "vdim": r_vdim, "decay": decay}}}


def moe_spec(experts=6, top=2, count=3, keep=2, ff=20, limit=1.5):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit},
            "router": {"experts": experts, "top": top, "groups": {"count": count, "keep": keep}}}


def make_config(layers, width=48, vocab=97, loop=None, eps=1e-5, logit_scale=0.5):
    cfg = {"architecture": "Zetalorn", "layers": layers, "logit_scale": logit_scale, "norm": {"eps": eps},
           "vocab": vocab, "width": width}
    if loop:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


def make_weights(cfg, seed=0, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    width = cfg["width"]
    w = {}

    def mat(name, out, inp, gain=1.0):
        w[name] = (torch.randn(out, inp, generator=g) * gain * inp ** -0.5).to(dtype)

    def vec(name, n, mean=1.0, std=0.1):
        w[name] = (mean + std * torch.randn(n, generator=g)).to(dtype)

    w["embed"] = torch.randn(cfg["vocab"], width, generator=g).to(dtype)
    if cfg.get("loop"):
        w["loop.step"] = (0.3 * torch.randn(cfg["loop"]["times"], width, generator=g)).to(dtype)
    for i, spec in enumerate(cfg["layers"]):
        p = "l%d." % i
        w[p + "norm1"] = (1.0 + 0.1 * torch.randn((), generator=g)).to(dtype)
        m = spec["mixer"]
        if spec["type"] == "attention":
            mat(p + "mix.q", m["heads"] * 2 * m["dim"], width, 2.0)
            mat(p + "mix.k", m["kv_heads"] * 2 * m["dim"], width, 2.0)
            mat(p + "mix.v", m["kv_heads"] * m["vdim"], width)
            vec(p + "mix.q.norm", m["dim"], 1.5, 0.3)
            vec(p + "mix.k.norm", m["dim"], 1.5, 0.3)
            for n in ("lq1", "lk1", "lq2", "lk2"):
                vec(p + "mix." + n, m["dim"], 0.0, 0.25)
            mat(p + "mix.o", width, m["heads"] * m["vdim"])
        else:
            a, r = m["left"], m["right"]
            mat(p + "mix.left.q", a["heads"] * a["dim"], width, 2.0)
            mat(p + "mix.left.k", a["kv_heads"] * a["dim"], width, 2.0)
            mat(p + "mix.left.v", a["kv_heads"] * a["vdim"], width)
            vec(p + "mix.left.q.norm", a["dim"], 1.5, 0.3)
            vec(p + "mix.left.k.norm", a["dim"], 1.5, 0.3)
            mat(p + "mix.left.o", width, a["heads"] * a["vdim"])
            mat(p + "mix.right.q", r["heads"] * r["dim"], width)
            mat(p + "mix.right.k", r["heads"] * r["dim"], width)
            mat(p + "mix.right.v", r["heads"] * r["vdim"], width)
            mat(p + "mix.right.g", r["heads"] * r["vdim"], width)
            mat(p + "mix.right.o", width, r["heads"] * r["vdim"])
            vec(p + "mix.right.norm", r["heads"] * r["vdim"])
            vec(p + "mix.left.out", width)
            vec(p + "mix.right.out", width)
        mat(p + "rg1", width, width)
        vec(p + "rg1.b", width, 0.0, 0.5)
        f = spec.get("mlp")
        if f is not None:
            w[p + "norm2"] = (1.0 + 0.1 * torch.randn((), generator=g)).to(dtype)
            for e in range(f["router"]["experts"]):
                mat("%smlp.e%d.gate" % (p, e), f["expert"]["ff"], width, 1.5)
                mat("%smlp.e%d.up" % (p, e), f["expert"]["ff"], width, 1.5)
                mat("%smlp.e%d.down" % (p, e), width, f["expert"]["ff"])
            mat(p + "mlp.router", f["router"]["experts"], width, 2.0)
            mat(p + "rg2", width, width)
            vec(p + "rg2.b", width, 0.0, 0.5)
    w["final.norm"] = (1.0 + 0.1 * torch.randn((), generator=g)).to(dtype)
    mat("head", cfg["vocab"], width)
    return w


def save_checkpoint(path, cfg, weights):
    from safetensors.torch import save_file

    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in weights.items()}, os.path.join(path, "model.safetensors"))
    return path


# ------------------------------------------------------------------ helpers of the tests
def forward(cfg, weights, tokens):
    return run(cfg, weights, tokens)[0]


def greedy(cfg, weights, prompt, n_new):
    toks = list(prompt)
    for _ in range(n_new):
        toks.append(int(forward(cfg, weights, toks)[-1].argmax()))
    return toks[len(prompt):]


def row_errors(got, want):
    """Per row: root mean square of the difference (its mean taken off) over that of the wanted row."""
    d = got.double() - want.double()
    d = d - d.mean(-1, keepdim=True)
    w = want.double() - want.double().mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / w.pow(2).mean(-1).sqrt().clamp_min(1e-30)
