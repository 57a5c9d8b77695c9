"""A slow float64 implementation of the Pelatar decoder, one function per mechanism, written from the
design's equations and sharing no code with the framework.  It walks whole sequences (no cache, no
state slots, no batches) and is what the engine tests compare against.

Weights are a dict name -> tensor with the checkpoint's names ("embed", "l<i>.norm1", "l<i>.mix.q", ...);
the configuration is the dict of a config.json.
"""

from __future__ import annotations

import math

import torch

F64 = torch.float64


def unit_rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def log_sigmoid(z):
    return -torch.nn.functional.softplus(-z)


def attention_keys_values(w, pre, h, m, eps):
    """Keys (unit RMS per head) and values a layer would cache: [T, G, dim], [T, G, vdim]."""
    t = h.shape[0]
    k = (h @ w[pre + "k"].T).view(t, m["kv_heads"], m["dim"])
    v = (h @ w[pre + "v"].T).view(t, m["kv_heads"], m["vdim"])
    return unit_rms(k, eps), v


def temperature(positions, temp):
    """1 + coef ln(floor((p + 1) / every) + 1), or 1 without a temperature."""
    p = torch.as_tensor(positions, dtype=F64)
    if not temp:
        return torch.ones_like(p)
    return 1.0 + temp["coef"] * torch.log(torch.floor((p + 1) / temp["every"]) + 1.0)


def sink_softmax_attention(q, k, v, pos_q, pos_k, rep, scale, sink):
    """q [Tq, H, d] at positions pos_q over k [Tk, G, d], v [Tk, G, dv] at pos_k (causal); the sink is one
    more term exp(sink_h) of every denominator, with no value.  -> [Tq, H, dv]"""
    tq, hq, _ = q.shape
    out = torch.zeros(tq, hq, v.shape[2], dtype=F64)
    hidden = torch.as_tensor(pos_k)[None, :] > torch.as_tensor(pos_q)[:, None]
    for a in range(hq):
        s = (q[:, a] @ k[:, a // rep].T) * scale
        s = s.masked_fill(hidden, -math.inf)
        big = torch.maximum(s.max(-1).values, sink[a])
        e = torch.exp(s - big[:, None])
        den = e.sum(-1) + torch.exp(sink[a] - big)
        out[:, a] = (e / den[:, None]) @ v[:, a // rep]
    return out


def attention(w, pre, h, m, eps, kv):
    """Softmax attention of h [T, width] over keys / values ``kv`` (its own, or another layer's)."""
    t = h.shape[0]
    hq, g, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = unit_rms((h @ w[pre + "q"].T).view(t, hq, d), eps) * temperature(range(t), m.get("q_temp"))[:, None, None]
    k, v = kv
    out = sink_softmax_attention(q, k, v, range(t), range(t), hq // g, m["scale"], w[pre + "sink"])
    gate = torch.sigmoid(h @ w[pre + "g"].T)
    return (out.reshape(t, hq * dv) * gate) @ w[pre + "o"].T


def capped_gates(xi, xf, cap):
    """Log input gate and log forget gate from their pre-activations."""
    return cap * torch.tanh(xi / cap), log_sigmoid(cap * torch.tanh(xf / cap))


def matrix_memory(q, k, v, gi, gf):
    """q, k [T, H, d] (q already scaled), v [T, H, dv], log gates [T, H] -> ([T, H, dv], the running maxima [T, H]).
    The maximum starts at zero."""
    t, nh, d = q.shape
    dv = v.shape[2]
    out = torch.zeros(t, nh, dv, dtype=F64)
    tops = torch.zeros(t, nh, dtype=F64)
    for a in range(nh):
        mem = torch.zeros(d, dv, dtype=F64)
        nrm = torch.zeros(d, dtype=F64)
        top = 0.0
        for s in range(t):
            new = max(float(gf[s, a]) + top, float(gi[s, a]))
            keep, put = math.exp(float(gf[s, a]) + top - new), math.exp(float(gi[s, a]) - new)
            mem = keep * mem + put * torch.outer(k[s, a], v[s, a])
            nrm = keep * nrm + put * k[s, a]
            top = new
            tops[s, a] = top
            out[s, a] = (mem.T @ q[s, a]) / (max(abs(float(nrm @ q[s, a])), math.exp(-top)) + 1e-6)
    return out, tops


def mlstm(w, pre, h, m, eps):
    """Matrix memory with exponential gates and a running maximum that starts at zero."""
    t = h.shape[0]
    nh, d, dv, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    q = (h @ w[pre + "q"].T).view(t, nh, d) * d ** -0.5
    k = (h @ w[pre + "k"].T).view(t, nh, d)
    v = (h @ w[pre + "v"].T).view(t, nh, dv)
    gi, gf = capped_gates(h @ w[pre + "i"].T + w[pre + "i.b"], h @ w[pre + "f"].T + w[pre + "f.b"], cap)
    out, _ = matrix_memory(q, k, v, gi, gf)
    y = unit_rms(out, eps).reshape(t, nh * dv) * w[pre + "norm"] * torch.sigmoid(h @ w[pre + "g"].T)
    return y @ w[pre + "o"].T


def decayed_memory(q, k, v, alpha):
    """S <- diag(alpha_t) S + k_t v_t^T, o_t = S^T q_t per head; alpha [T, H, d] acts on the rows of key channels."""
    t, nh, d = q.shape
    out = torch.zeros(t, nh, v.shape[2], dtype=F64)
    for a in range(nh):
        mem = torch.zeros(d, v.shape[2], dtype=F64)
        for s in range(t):
            mem = alpha[s, a][:, None] * mem + torch.outer(k[s, a], v[s, a])
            out[s, a] = mem.T @ q[s, a]
    return out


def channel_decay(z, tau):
    return torch.exp(log_sigmoid(z) / tau)


def gla(w, pre, h, m, eps):
    """Linear attention whose state rows decay by a per-channel gate."""
    t = h.shape[0]
    nh, d, dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ w[pre + "q"].T).view(t, nh, d) * d ** -0.5
    k = (h @ w[pre + "k"].T).view(t, nh, d)
    v = (h @ w[pre + "v"].T).view(t, nh, dv)
    z = (h @ w[pre + "a1"].T) @ w[pre + "a2"].T + w[pre + "a2.b"]
    out = decayed_memory(q, k, v, channel_decay(z, m["tau"]).view(t, nh, d))
    y = unit_rms(out, eps) * w[pre + "norm"]
    return (y.reshape(t, nh * dv) * silu(h @ w[pre + "g"].T)) @ w[pre + "o"].T


def dense_ff(w, pre, h):
    return (gelu_tanh(h @ w[pre + "gate"].T) * (h @ w[pre + "up"].T)) @ w[pre + "down"].T


def choose(logits, bias, n_groups, keep, top):
    """Softmax scores; the ``top`` largest of score + bias among the outputs of the ``keep`` groups whose largest
    biased score is largest -> (ids [T, top], scores of the chosen [T, top])."""
    s = torch.softmax(logits, -1)
    choice = s + bias
    per = logits.shape[1] // n_groups
    best = choice.view(-1, n_groups, per).max(-1).values
    kept = best.topk(keep, dim=-1).indices
    allowed = torch.zeros(logits.shape[0], n_groups, dtype=torch.bool)
    allowed.scatter_(1, kept, True)
    choice = choice.masked_fill(~allowed.repeat_interleave(per, dim=1), -math.inf)
    ids = choice.topk(top, dim=-1).indices
    return ids, s.gather(1, ids)


def route(w, pre, h, r):
    """(chosen ids [T, top], their weights [T, top]); ids >= experts are identity experts."""
    groups = r.get("groups") or {"count": 1, "keep": 1}
    return choose(h @ w[pre + "router"].T, w[pre + "correction"], groups["count"], groups["keep"], r["top"])


def moe_ff(w, pre, h, f):
    r = f["router"]
    ids, wts = route(w, pre, h, r)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, c in zip(ids[t].tolist(), wts[t].tolist()):
            if e >= r["experts"]:
                out[t] += c * h[t]
            else:
                p = f"{pre}e{e}."
                out[t] += c * ((silu(h[t] @ w[p + "gate"].T) * (h[t] @ w[p + "up"].T)) @ w[p + "down"].T)
    return out


def forward(cfg, weights, tokens, probe=None):
    """Logits [T, vocab] of one sequence; ``probe(i, x)`` sees the residual stream after every layer."""
    w = {k: v.to(F64) for k, v in weights.items()}
    eps = cfg["norm"]["eps"]
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    held = {}
    for i, layer in enumerate(cfg["layers"]):
        m, pre = layer["mixer"], f"l{i}.mix."
        if layer["type"] == "attention":
            src = m.get("kv_from")
            held[i] = held[src] if src is not None else attention_keys_values(w, pre, x, m, eps)
            y = attention(w, pre, x, m, eps, held[i])
        elif layer["type"] == "mlstm":
            y = mlstm(w, pre, x, m, eps)
        elif layer["type"] == "gla":
            y = gla(w, pre, x, m, eps)
        else:
            raise ValueError(layer["type"])
        x = x + unit_rms(y, eps) * w[f"l{i}.norm1"]
        f = layer.get("mlp")
        if f is not None:
            y = dense_ff(w, f"l{i}.mlp.", x) if f["kind"] == "dense" else moe_ff(w, f"l{i}.mlp.", x, f)
            x = x + unit_rms(y, eps) * w[f"l{i}.norm2"]
        if probe is not None:
            probe(i, x)
    return (unit_rms(x, eps) * w["final.norm"]) @ w["embed"].T


# ----------------------------------------------------------------------------- configurations and weights for tests
def attention_layer(heads=4, kv_heads=2, dim=16, vdim=24, scale=None, coef=0.4, every=16, kv_from=None, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else dim ** -0.5}
    if coef:
        m["q_temp"] = {"coef": coef, "every": every}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m, "mlp": mlp}


def mlstm_layer(heads=2, dim=16, vdim=24, cap=12.0, mlp=None):
    return {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}, "mlp": mlp}


def gla_layer(heads=2, dim=16, vdim=24, tau=8.0, rank=8, mlp=None):
    # the rank is no key of the configuration: the shape of the first decay projection carries it
    return {"type": "gla", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau}, "mlp": mlp, "_rank": rank}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(ff, experts, top, groups=1, keep=1, identity=0):
    r = {"experts": experts, "top": top, "groups": {"count": groups, "keep": keep}}
    if identity:
        r["identity"] = identity
    return {"kind": "moe", "expert": {"ff": ff}, "router": r}


def make_config(layers, vocab=96, width=48, eps=1e-5):
    ranks = [layer.pop("_rank", None) for layer in layers]
    return {"architecture": "Pelatar", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers,
            "_ranks": ranks}


def random_weights(cfg, seed=0, router_gain=4.0):
    """bfloat16-valued weights (so that both number formats load the same model)."""
    g = torch.Generator().manual_seed(seed)
    w = {}
    width = cfg["width"]

    def lin(name, out, inp, gain=1.0):
        w[name] = (torch.randn(out, inp, generator=g) * gain * inp ** -0.5).bfloat16()

    def vec(name, n, mean=0.0, std=1.0):
        w[name] = (mean + std * torch.randn(n, generator=g)).bfloat16()

    w["embed"] = torch.randn(cfg["vocab"], width, generator=g).bfloat16()
    for i, layer in enumerate(cfg["layers"]):
        m, p = layer["mixer"], f"l{i}.mix."
        vec(f"l{i}.norm1", width, 1.0, 0.2)
        hd, hv = m["heads"] * m["dim"], m["heads"] * m["vdim"]
        lin(p + "q", hd, width)
        lin(p + "g", hv, width)
        lin(p + "o", width, hv)
        if layer["type"] == "attention":
            vec(p + "sink", m["heads"])
            if m.get("kv_from") is None:
                lin(p + "k", m["kv_heads"] * m["dim"], width)
                lin(p + "v", m["kv_heads"] * m["vdim"], width)
        else:
            lin(p + "k", hd, width)
            lin(p + "v", hv, width)
            if layer["type"] == "mlstm":
                vec(p + "norm", hv, 1.0, 0.2)
                lin(p + "i", m["heads"], width, 2.0)
                lin(p + "f", m["heads"], width, 2.0)
                vec(p + "i.b", m["heads"])
                vec(p + "f.b", m["heads"], 3.0)
            else:
                rank = cfg["_ranks"][i] or 8
                vec(p + "norm", m["vdim"], 1.0, 0.2)
                lin(p + "a1", rank, width)
                lin(p + "a2", hd, rank, 2.0)
                vec(p + "a2.b", hd, 2.0)
        f = layer.get("mlp")
        if f is None:
            continue
        vec(f"l{i}.norm2", width, 1.0, 0.2)
        q = f"l{i}.mlp."
        if f["kind"] == "dense":
            lin(q + "gate", f["ff"], width)
            lin(q + "up", f["ff"], width)
            lin(q + "down", width, f["ff"])
        else:
            r = f["router"]
            n = r["experts"] + r.get("identity", 0)
            lin(q + "router", n, width, router_gain)   # far-apart scores: no routing decision is a close call
            vec(q + "correction", n, 0.0, 0.05)
            for e in range(r["experts"]):
                lin(f"{q}e{e}.gate", f["expert"]["ff"], width)
                lin(f"{q}e{e}.up", f["expert"]["ff"], width)
                lin(f"{q}e{e}.down", width, f["expert"]["ff"])
    vec("final.norm", width, 1.0, 0.2)
    return w


def write_checkpoint(path, cfg, weights):
    import json
    from pathlib import Path

    from safetensors.torch import save_file

    path = Path(path)
    path.mkdir(parents=True, exist_ok=True)
    (path / "config.json").write_text(json.dumps({k: v for k, v in cfg.items() if not k.startswith("_")}))
    save_file({k: v.contiguous().clone() for k, v in weights.items()}, str(path / "model.safetensors"))
    return path


def greedy(cfg, weights, prompt, n_new):
    ids = list(prompt)
    for _ in range(n_new):
        ids.append(int(forward(cfg, weights, ids)[-1].argmax()))
    return ids[len(prompt):]


def row_errors(got, want):
    """Per row: root mean square of the difference (means taken off) over that of the wanted row."""
    d = got.double() - want.double()
    d = d - d.mean(-1, keepdim=True)
    ref = want.double() - want.double().mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / ref.pow(2).mean(-1).sqrt().clamp_min(1e-12)


def check_rows(got, want, tol, what=""):
    assert got.shape == want.shape, f"{what}: shape {tuple(got.shape)} != {tuple(want.shape)}"
    err = row_errors(got, want)
    bad = int(err.argmax())
    assert err.max().item() < tol, f"{what}: row {bad} is off by {err.max().item():.3g} (allowed {tol})"
