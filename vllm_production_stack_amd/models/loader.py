"""Model construction: random init (no checkpoint on disk) or HF safetensors loading.

Checkpoint tensors are streamed shard by shard straight into the fused / TP-sharded
layout the engine uses (QKV and gate|up fused, column shards by head, row shards by
channel), so the host never holds more than one checkpoint tensor at a time.
"""

from __future__ import annotations

import json
import re
from pathlib import Path

import torch

from ..engine.config import ModelConfig
from ..parallel.state import get_tp
from .opt import OPTModel
from .transformer import LayerWeights, TransformerModel
from .pelatar import PelatarModel
from .revelix import RevelixModel
from .zetalorn import ZetalornModel
from .zururax import ZururaxModel


def build_model(cfg: ModelConfig, dtype: torch.dtype, device: torch.device, max_model_len: int,
                ckpt_dir: Path | None = None, seed: int = 0, load_format: str = "auto",
                expert_parallel: bool = False):
    if cfg.architecture in ("opt", "gpt2"):
        model = OPTModel(cfg, dtype, device, max_model_len)
    elif cfg.architecture == "zururax":
        model = ZururaxModel(cfg, dtype, device, max_model_len)
    elif cfg.architecture == "revelix":
        model = RevelixModel(cfg, dtype, device, max_model_len)
    elif cfg.architecture == "pelatar":
        model = PelatarModel(cfg, dtype, device, max_model_len)
    elif cfg.architecture == "zetalorn":
        model = ZetalornModel(cfg, dtype, device, max_model_len)
    else:
        model = TransformerModel(cfg, dtype, device, max_model_len, expert_parallel=expert_parallel)
    has_weights = ckpt_dir is not None and any(Path(ckpt_dir).glob("*.safetensors"))
    if has_weights and load_format != "dummy":
        model.init_random(seed)  # allocates every tensor; checkpoint values overwrite them
        load_hf_weights(model, Path(ckpt_dir))
    else:
        model.init_random(seed)
    return model


def _iter_safetensors(ckpt_dir: Path):
    from safetensors import safe_open

    index = ckpt_dir / "model.safetensors.index.json"
    if index.exists():
        with open(index) as f:
            files = sorted(set(json.load(f)["weight_map"].values()))
    else:
        files = sorted(p.name for p in ckpt_dir.glob("*.safetensors"))
    for fn in files:
        with safe_open(str(ckpt_dir / fn), framework="pt", device="cpu") as f:
            for k in f.keys():
                yield k, f.get_tensor(k)


def load_hf_weights(model, ckpt_dir: Path) -> None:
    if isinstance(model, OPTModel):
        (_load_gpt2 if model.cfg.architecture == "gpt2" else _load_opt)(model, ckpt_dir)
    elif isinstance(model, ZururaxModel):
        _load_zururax(model, ckpt_dir)
    elif isinstance(model, RevelixModel):
        _load_revelix(model, ckpt_dir)
    elif isinstance(model, PelatarModel):
        _load_pelatar(model, ckpt_dir)
    elif isinstance(model, ZetalornModel):
        _load_zetalorn(model, ckpt_dir)
    else:
        _load_llama(model, ckpt_dir)


def _shard_rows(t: torch.Tensor, rank: int, size: int) -> torch.Tensor:
    n = t.shape[0] // size
    return t[rank * n:(rank + 1) * n]


def _shard_cols(t: torch.Tensor, rank: int, size: int) -> torch.Tensor:
    n = t.shape[1] // size
    return t[:, rank * n:(rank + 1) * n]


def _load_llama(model: TransformerModel, ckpt_dir: Path) -> None:
    cfg = model.cfg
    tp = get_tp()
    r, s = tp.rank, tp.size
    d = cfg.head_dim
    nq, nkv, inter = model.n_q, model.n_kv, model.inter
    pat = re.compile(r"model\.layers\.(\d+)\.(.+)")
    for name, t in _iter_safetensors(ckpt_dir):
        t = t.to(model.dtype)
        if name == "model.embed_tokens.weight":
            if model.embed is None:
                continue
            model.embed.copy_(t)
            if model.lm_head is not model.embed and cfg.tie_word_embeddings:
                model.lm_head[: min(model.vocab_shard, t.shape[0] - r * model.vocab_shard)].copy_(
                    t[r * model.vocab_shard:(r + 1) * model.vocab_shard])
            continue
        if name == "model.norm.weight":
            if model.norm is not None:
                model.norm.copy_(t)
            continue
        if name == "lm_head.weight":
            if model.lm_head is not None and model.lm_head is not model.embed:
                rows = t[r * model.vocab_shard:(r + 1) * model.vocab_shard]
                model.lm_head[: rows.shape[0]].copy_(rows)
            continue
        m = pat.match(name)
        if not m:
            continue
        li, sub = int(m.group(1)), m.group(2)
        if not (model.first_layer <= li < model.last_layer):
            continue  # another pipeline stage's layer
        lw: LayerWeights = model.layers[li - model.first_layer]
        if sub == "input_layernorm.weight":
            lw.ln1.copy_(t)
        elif sub == "post_attention_layernorm.weight":
            lw.ln2.copy_(t)
        elif sub == "self_attn.q_proj.weight":
            lw.wqkv[: nq * d].copy_(_shard_rows(t, r, s))
        elif sub == "self_attn.k_proj.weight":
            lw.wqkv[nq * d:(nq + nkv) * d].copy_(_shard_rows(t, r, s))
        elif sub == "self_attn.v_proj.weight":
            lw.wqkv[(nq + nkv) * d:].copy_(_shard_rows(t, r, s))
        elif sub == "self_attn.q_proj.bias" and lw.bqkv is not None:
            lw.bqkv[: nq * d].copy_(_shard_rows(t, r, s))
        elif sub == "self_attn.k_proj.bias" and lw.bqkv is not None:
            lw.bqkv[nq * d:(nq + nkv) * d].copy_(_shard_rows(t, r, s))
        elif sub == "self_attn.v_proj.bias" and lw.bqkv is not None:
            lw.bqkv[(nq + nkv) * d:].copy_(_shard_rows(t, r, s))
        elif sub == "self_attn.o_proj.weight":
            lw.wo.copy_(_shard_cols(t, r, s))
        elif sub == "mlp.gate_proj.weight":
            lw.w_gate_up[:inter].copy_(_shard_rows(t, r, s))
        elif sub == "mlp.up_proj.weight":
            lw.w_gate_up[inter:].copy_(_shard_rows(t, r, s))
        elif sub == "mlp.down_proj.weight":
            lw.w_down.copy_(_shard_cols(t, r, s))
        elif sub == "block_sparse_moe.gate.weight":
            lw.router.copy_(t)
        else:
            me = re.match(r"block_sparse_moe\.experts\.(\d+)\.(w[123])\.weight", sub)
            if me:
                ex, which = int(me.group(1)), me.group(2)
                if model.ep:  # whole experts, this rank's range of them
                    ex -= model.first_expert
                    if 0 <= ex < model.local_experts:
                        full = cfg.intermediate_size
                        if which == "w1":
                            lw.w13[ex, :full].copy_(t)
                        elif which == "w3":
                            lw.w13[ex, full:].copy_(t)
                        else:
                            lw.w2[ex].copy_(t)
                elif which == "w1":
                    lw.w13[ex, :inter].copy_(_shard_rows(t, r, s))
                elif which == "w3":
                    lw.w13[ex, inter:].copy_(_shard_rows(t, r, s))
                else:
                    lw.w2[ex].copy_(_shard_cols(t, r, s))


def _load_opt(model: OPTModel, ckpt_dir: Path) -> None:
    h = model.cfg.hidden_size
    pat = re.compile(r"(?:model\.)?decoder\.layers\.(\d+)\.(.+)")
    for name, t in _iter_safetensors(ckpt_dir):
        t = t.to(model.dtype)
        base = name.removeprefix("model.")
        if base == "decoder.embed_tokens.weight":
            model.embed.copy_(t)
        elif base == "decoder.embed_positions.weight":
            n = min(t.shape[0], model.pos_embed.shape[0])
            model.pos_embed[:n].copy_(t[:n])
        elif base == "decoder.final_layer_norm.weight":
            model.final_ln[0].copy_(t)
        elif base == "decoder.final_layer_norm.bias":
            model.final_ln[1].copy_(t)
        else:
            m = pat.match(name)
            if not m:
                continue
            lw = model.layers[int(m.group(1))]
            sub = m.group(2)
            table = {
                "self_attn_layer_norm.weight": ("ln1_w", None), "self_attn_layer_norm.bias": ("ln1_b", None),
                "self_attn.q_proj.weight": ("wqkv", 0), "self_attn.k_proj.weight": ("wqkv", 1),
                "self_attn.v_proj.weight": ("wqkv", 2), "self_attn.q_proj.bias": ("bqkv", 0),
                "self_attn.k_proj.bias": ("bqkv", 1), "self_attn.v_proj.bias": ("bqkv", 2),
                "self_attn.out_proj.weight": ("wo", None), "self_attn.out_proj.bias": ("bo", None),
                "final_layer_norm.weight": ("ln2_w", None), "final_layer_norm.bias": ("ln2_b", None),
                "fc1.weight": ("fc1", None), "fc1.bias": ("b1", None),
                "fc2.weight": ("fc2", None), "fc2.bias": ("b2", None),
            }
            if sub in table:
                key, part = table[sub]
                if part is None:
                    lw[key].copy_(t)
                else:
                    lw[key][part * h:(part + 1) * h].copy_(t)


def _load_gpt2(model: OPTModel, ckpt_dir: Path) -> None:
    """GPT-2 checkpoints: ``wte / wpe / h.N.{ln_1, attn.c_attn, attn.c_proj, ln_2, mlp.c_fc,
    mlp.c_proj} / ln_f``; the Conv1D projections store [in, out] and are transposed here."""
    pat = re.compile(r"(?:transformer\.)?h\.(\d+)\.(.+)")
    table = {
        "ln_1.weight": ("ln1_w", False), "ln_1.bias": ("ln1_b", False),
        "attn.c_attn.weight": ("wqkv", True), "attn.c_attn.bias": ("bqkv", False),
        "attn.c_proj.weight": ("wo", True), "attn.c_proj.bias": ("bo", False),
        "ln_2.weight": ("ln2_w", False), "ln_2.bias": ("ln2_b", False),
        "mlp.c_fc.weight": ("fc1", True), "mlp.c_fc.bias": ("b1", False),
        "mlp.c_proj.weight": ("fc2", True), "mlp.c_proj.bias": ("b2", False),
    }
    for name, t in _iter_safetensors(ckpt_dir):
        t = t.to(model.dtype)
        base = name.removeprefix("transformer.")
        if base == "wte.weight":
            model.embed.copy_(t)
        elif base == "wpe.weight":
            n = min(t.shape[0], model.pos_embed.shape[0])
            model.pos_embed[:n].copy_(t[:n])
        elif base == "ln_f.weight":
            model.final_ln[0].copy_(t)
        elif base == "ln_f.bias":
            model.final_ln[1].copy_(t)
        else:
            m = pat.match(name)
            if m and m.group(2) in table:
                key, transpose = table[m.group(2)]
                model.layers[int(m.group(1))][key].copy_(t.t() if transpose else t)


def _load_zururax(model: ZururaxModel, ckpt_dir: Path) -> None:
    """Zururax checkpoints: ``embed``, ``l<i>.norm1|norm2``, ``l<i>.mix.{dq, dq.norm, uq, dkv, dkv.norm, uk, uv,
    sink, g, o}``, ``l<i>.mlp.{up, down}`` or ``l<i>.mlp.{router, e<k>.{gate, up, down}, shared.{gate, up, down,
    sg}}``, ``final.norm``, ``head``; linear weights are [out, in].  Every tensor the model holds must
    be found, and every tensor of the file must have a place."""
    pat = re.compile(r"l(\d+)\.(.+)")
    expert = re.compile(r"mlp\.e(\d+)\.(gate|up|down)")
    seen: set[str] = set()

    def put(dst: torch.Tensor, src: torch.Tensor, what: str) -> None:
        if tuple(dst.shape) != tuple(src.shape):
            raise ValueError(f"{what}: checkpoint shape {tuple(src.shape)}, model expects {tuple(dst.shape)}")
        dst.copy_(src.to(dst.dtype))

    for name, t in _iter_safetensors(ckpt_dir):
        seen.add(name)
        if name == "embed":
            put(model.embed, t, name)
        elif name == "head":
            put(model.lm_head, t, name)
        elif name == "final.norm":
            put(model.norm, t, name)
        else:
            mt = pat.match(name)
            if not mt or int(mt.group(1)) >= len(model.layers):
                raise ValueError(f"unexpected tensor {name!r}")
            lw = model.layers[int(mt.group(1))]
            sub = mt.group(2)
            m, f = lw.spec.mixer, lw.spec.mlp
            own = m.kv_from is None
            me = expert.fullmatch(sub)
            if sub == "norm1":
                put(lw.norm1, t, name)
            elif sub == "norm2" and f is not None:
                put(lw.norm2, t, name)
            elif sub == "mix.dq":
                put(lw.w_in[:m.q_rank], t, name)
            elif sub == "mix.dkv" and own:
                put(lw.w_in[m.q_rank:m.q_rank + m.entry], t, name)
            elif sub == "mix.g" and m.out_gate:
                put(lw.w_in[lw.w_in.shape[0] - m.heads:], t, name)
            elif sub == "mix.dq.norm":
                put(lw.dq_norm, t, name)
            elif sub == "mix.dkv.norm" and own:
                put(lw.dkv_norm, t, name)
            elif sub == "mix.uq":
                put(lw.w_uq, t, name)
            elif sub == "mix.uk":
                put(lw.w_uk.view(m.heads * m.dim, m.kv_rank), t, name)
            elif sub == "mix.uv":
                put(lw.w_uv.view(m.heads * m.vdim, m.kv_rank), t, name)
            elif sub == "mix.sink" and m.sink:
                put(lw.sink, t, name)
            elif sub == "mix.o":
                put(lw.w_o, t, name)
            elif sub == "mlp.up" and f is not None and f.kind == "dense":
                put(lw.w_up, t, name)
            elif sub == "mlp.down" and f is not None and f.kind == "dense":
                put(lw.w_down, t, name)
            elif sub == "mlp.router" and f is not None and f.kind == "moe":
                put(lw.router[:f.experts], t, name)
            elif me and f is not None and f.kind == "moe" and int(me.group(1)) < f.experts:
                e, which = int(me.group(1)), me.group(2)
                if which == "gate":
                    put(lw.w13[e, :f.ff], t, name)
                elif which == "up":
                    put(lw.w13[e, f.ff:], t, name)
                else:
                    put(lw.w2[e], t, name)
            elif sub.startswith("mlp.shared.") and f is not None and f.shared_ff:
                which = sub[len("mlp.shared."):]
                if which == "gate":
                    put(lw.w_sh13[:f.shared_ff], t, name)
                elif which == "up":
                    put(lw.w_sh13[f.shared_ff:], t, name)
                elif which == "down":
                    put(lw.w_sh2, t, name)
                elif which == "sg":
                    put(lw.router[f.experts:], t, name)
                else:
                    raise ValueError(f"unexpected tensor {name!r}")
            else:
                raise ValueError(f"unexpected tensor {name!r}")
    want = {"embed", "head", "final.norm"}
    for i, lw in enumerate(model.layers):
        m, f = lw.spec.mixer, lw.spec.mlp
        want |= {f"l{i}.norm1", f"l{i}.mix.dq", f"l{i}.mix.dq.norm", f"l{i}.mix.uq", f"l{i}.mix.uk", f"l{i}.mix.uv",
                 f"l{i}.mix.o"}
        if m.kv_from is None:
            want |= {f"l{i}.mix.dkv", f"l{i}.mix.dkv.norm"}
        if m.sink:
            want.add(f"l{i}.mix.sink")
        if m.out_gate:
            want.add(f"l{i}.mix.g")
        if f is not None:
            want.add(f"l{i}.norm2")
            if f.kind == "dense":
                want |= {f"l{i}.mlp.up", f"l{i}.mlp.down"}
            else:
                want.add(f"l{i}.mlp.router")
                want |= {f"l{i}.mlp.e{e}.{k}" for e in range(f.experts) for k in ("gate", "up", "down")}
                if f.shared_ff:
                    want |= {f"l{i}.mlp.shared.{k}" for k in ("gate", "up", "down", "sg")}
    if want - seen:
        raise ValueError(f"checkpoint lacks {sorted(want - seen)[:8]}")


def _load_revelix(model: RevelixModel, ckpt_dir: Path) -> None:
    """Revelix checkpoints: ``embed``; per layer ``l<i>.norm1|norm2`` with ``.b`` and ``.alpha``;
    ``l<i>.mix.{q, k, v, g, o}`` (retention) or ``l<i>.mix.left.{q, k, v (each with .b and .conv), talk, sink, o}``
    and ``l<i>.mix.right.{q, f, f.b, lower, v, norm, o}`` (parallel); ``l<i>.mlp.{up, down, act}``;
    ``final.norm`` (+ ``.b``, ``.alpha``).  Linear weights are [out, in]; the input projections of a
    mixer are fused row-wise here.  Every tensor the model holds must be found, and every tensor of the
    file must have a place."""
    from ..engine.config import ParallelMixerSpec

    pat = re.compile(r"l(\d+)\.(.+)")
    seen: set[str] = set()

    def put(dst: torch.Tensor, src: torch.Tensor, what: str) -> None:
        if tuple(dst.shape) != tuple(src.shape):
            raise ValueError(f"{what}: checkpoint shape {tuple(src.shape)}, model expects {tuple(dst.shape)}")
        dst.copy_(src.to(dst.dtype))

    def put_norm(norm: list, which: str, src: torch.Tensor, what: str) -> bool:
        i = {"": 0, ".b": 1, ".alpha": 2}.get(which)
        if i is None:
            return False
        put(norm[i], src.reshape(norm[i].shape) if i == 2 and src.numel() == 1 else src, what)
        return True

    for name, t in _iter_safetensors(ckpt_dir):
        seen.add(name)
        if name == "embed":
            put(model.embed, t, name)
            continue
        if name.startswith("final.norm"):
            if not put_norm(model.norm, name[len("final.norm"):], t, name):
                raise ValueError(f"unexpected tensor {name!r}")
            continue
        mt = pat.match(name)
        if not mt or int(mt.group(1)) >= len(model.layers):
            raise ValueError(f"unexpected tensor {name!r}")
        lw = model.layers[int(mt.group(1))]
        sub = mt.group(2)
        m, f = lw.spec.mixer, lw.spec.mlp
        ok = False
        if sub.startswith("norm1"):
            ok = put_norm(lw.norm1, sub[5:], t, name)
        elif sub.startswith("norm2") and f is not None:
            ok = put_norm(lw.norm2, sub[5:], t, name)
        elif sub.startswith("mlp.") and f is not None:
            ok = True
            if sub == "mlp.up":
                put(lw.w_up, t, name)
            elif sub == "mlp.down":
                put(lw.w_down, t, name)
            elif sub == "mlp.act":
                p = t.double()
                if p.numel() != 2:
                    raise ValueError(f"{name}: two numbers expected")
                sp = torch.nn.functional.softplus(p)
                model.set_activation(lw, float(sp[0]), float(0.5 + sp[1]))
            else:
                ok = False
        elif not isinstance(m, ParallelMixerSpec):
            hd, hv = m.heads * m.dim, m.heads * m.vdim
            rows = {"mix.q": (0, hd), "mix.k": (hd, 2 * hd), "mix.v": (2 * hd, 2 * hd + hv),
                    "mix.g": (2 * hd + hv, 2 * hd + 2 * hv)}
            if sub in rows:
                a, b = rows[sub]
                put(lw.w_in[a:b], t, name)
                ok = True
            elif sub == "mix.o":
                put(lw.w_o, t, name)
                ok = True
        else:
            a, r = m.left, m.right
            nq, nk, nv = a.heads * a.dim, a.kv_heads * a.dim, a.kv_heads * a.vdim
            c0, rd = a.channels, r.heads * r.dim
            left = {"q": (0, nq), "k": (nq, nq + nk), "v": (nq + nk, nq + nk + nv)}
            right = {"q": (c0, c0 + rd), "f": (c0 + rd, c0 + 2 * rd), "v": (c0 + 2 * rd, c0 + 2 * rd + r.heads * r.vdim)}
            ok = True
            parts = sub.split(".")
            if sub.startswith("mix.left.") and len(parts) >= 3 and parts[2] in left:
                lo, hi = left[parts[2]]
                rest = ".".join(parts[3:])
                if rest == "":
                    put(lw.w_in[lo:hi], t, name)
                elif rest == "b":
                    put(lw.b_in[lo:hi], t, name)
                elif rest == "conv":
                    put(lw.conv_w[lo:hi], t, name)
                else:
                    ok = False
            elif sub == "mix.left.talk":
                put(lw.talk, t, name)
            elif sub == "mix.left.sink":
                put(lw.sink, t, name)
            elif sub == "mix.left.o":
                put(lw.w_o, t, name)
            elif sub.startswith("mix.right.") and len(parts) == 3 and parts[2] in right:
                lo, hi = right[parts[2]]
                put(lw.w_in[lo:hi], t, name)
            elif sub == "mix.right.f.b":
                put(lw.gate_bias, t, name)
            elif sub == "mix.right.lower":
                put(lw.gate_lower, t, name)
            elif sub == "mix.right.norm":
                put(lw.r_norm, t, name)
            elif sub == "mix.right.o":
                put(lw.wr_o, t, name)
            else:
                ok = False
        if not ok:
            raise ValueError(f"unexpected tensor {name!r}")
    want = {"embed"} | {"final.norm" + x for x in ("", ".b", ".alpha")}
    for i, lw in enumerate(model.layers):
        m, f = lw.spec.mixer, lw.spec.mlp
        want |= {f"l{i}.norm1{x}" for x in ("", ".b", ".alpha")}
        if isinstance(m, ParallelMixerSpec):
            for k in ("q", "k", "v"):
                want |= {f"l{i}.mix.left.{k}", f"l{i}.mix.left.{k}.b", f"l{i}.mix.left.{k}.conv"}
            want |= {f"l{i}.mix.left.{k}" for k in ("talk", "sink", "o")}
            want |= {f"l{i}.mix.right.{k}" for k in ("q", "f", "f.b", "lower", "v", "norm", "o")}
        else:
            want |= {f"l{i}.mix.{k}" for k in ("q", "k", "v", "g", "o")}
        if f is not None:
            want |= {f"l{i}.norm2{x}" for x in ("", ".b", ".alpha")}
            want |= {f"l{i}.mlp.{k}" for k in ("up", "down", "act")}
    if want - seen:
        raise ValueError(f"checkpoint lacks {sorted(want - seen)[:8]}")


def _load_pelatar(model: PelatarModel, ckpt_dir: Path) -> None:
    """Pelatar checkpoints: ``embed``; per layer ``l<i>.norm1|norm2``; ``l<i>.mix.{q, k, v, sink, g, o}`` (attention; no
    k and v with ``kv_from``), ``l<i>.mix.{q, k, v, g, o, norm, i, i.b, f, f.b}`` (mlstm), ``l<i>.mix.{q, k, v, g, o, norm,
    a1, a2, a2.b}`` (gla, whose low rank is the shape of ``a1``); ``l<i>.mlp.{gate, up, down}`` or ``l<i>.mlp.{router,
    correction, e<k>.{gate, up, down}}``; ``final.norm``.  Linear weights are [out, in]; the input projections of a
    mixer are fused row-wise here.  Every tensor the model holds must be found, and every tensor of the file must
    have a place."""
    from ..engine.config import GatedLinearSpec, MatrixMemorySpec, NormedAttentionSpec

    pat = re.compile(r"l(\d+)\.(.+)")
    expert = re.compile(r"mlp\.e(\d+)\.(gate|up|down)")
    seen: set[str] = set()

    def put(dst: torch.Tensor, src: torch.Tensor, what: str) -> None:
        if tuple(dst.shape) != tuple(src.shape):
            raise ValueError(f"{what}: checkpoint shape {tuple(src.shape)}, model expects {tuple(dst.shape)}")
        dst.copy_(src.to(dst.dtype))

    tensors = list(_iter_safetensors(ckpt_dir))
    for name, t in tensors:  # the decays' low rank first: it sizes the fused input projection
        mt = pat.match(name)
        if mt and mt.group(2) == "mix.a1" and int(mt.group(1)) < len(model.layers):
            lw = model.layers[int(mt.group(1))]
            if isinstance(lw.spec.mixer, GatedLinearSpec) and t.dim() == 2 and lw.w_a2.shape[1] != t.shape[0]:
                model.set_decay_rank(lw, t.shape[0])
    for name, t in tensors:
        seen.add(name)
        if name == "embed":
            put(model.embed, t, name)
            continue
        if name == "final.norm":
            put(model.norm, t, name)
            continue
        mt = pat.match(name)
        if not mt or int(mt.group(1)) >= len(model.layers):
            raise ValueError(f"unexpected tensor {name!r}")
        lw = model.layers[int(mt.group(1))]
        sub = mt.group(2)
        m, f = lw.spec.mixer, lw.spec.mlp
        me = expert.fullmatch(sub)
        hd, hv = m.heads * m.dim, m.heads * m.vdim
        rows: dict[str, tuple] = {}
        if isinstance(m, NormedAttentionSpec):
            kd, kv = m.kv_heads * m.dim, m.kv_heads * m.vdim
            if m.kv_from is None:
                rows = {"mix.q": (0, hd), "mix.k": (hd, hd + kd), "mix.v": (hd + kd, hd + kd + kv),
                        "mix.g": (hd + kd + kv, hd + kd + kv + hv)}
            else:
                rows = {"mix.q": (0, hd), "mix.g": (hd, hd + hv)}
        else:
            rows = {"mix.q": (0, hd), "mix.k": (hd, 2 * hd), "mix.v": (2 * hd, 2 * hd + hv),
                    "mix.g": (2 * hd + hv, 2 * hd + 2 * hv)}
            if isinstance(m, GatedLinearSpec):
                rows["mix.a1"] = (2 * hd + 2 * hv, lw.w_in.shape[0])
        if sub == "norm1":
            put(lw.norm1, t, name)
        elif sub == "norm2" and f is not None:
            put(lw.norm2, t, name)
        elif sub in rows:
            a, b = rows[sub]
            put(lw.w_in[a:b], t, name)
        elif sub == "mix.o":
            put(lw.w_o, t, name)
        elif sub == "mix.sink" and isinstance(m, NormedAttentionSpec):
            put(lw.sink, t, name)
        elif sub == "mix.norm" and not isinstance(m, NormedAttentionSpec):
            put(lw.h_norm, t, name)
        elif sub == "mix.i" and isinstance(m, MatrixMemorySpec):
            put(lw.w_if[:m.heads], t, name)
        elif sub == "mix.f" and isinstance(m, MatrixMemorySpec):
            put(lw.w_if[m.heads:], t, name)
        elif sub == "mix.i.b" and isinstance(m, MatrixMemorySpec):
            put(lw.b_i, t, name)
        elif sub == "mix.f.b" and isinstance(m, MatrixMemorySpec):
            put(lw.b_f, t, name)
        elif sub == "mix.a2" and isinstance(m, GatedLinearSpec):
            put(lw.w_a2, t, name)
        elif sub == "mix.a2.b" and isinstance(m, GatedLinearSpec):
            put(lw.a2_b, t, name)
        elif sub == "mlp.gate" and f is not None and f.kind == "dense":
            put(lw.w_gu[:f.ff], t, name)
        elif sub == "mlp.up" and f is not None and f.kind == "dense":
            put(lw.w_gu[f.ff:], t, name)
        elif sub == "mlp.down" and f is not None and f.kind == "dense":
            put(lw.w_down, t, name)
        elif sub == "mlp.router" and f is not None and f.kind == "moe":
            put(lw.router, t, name)
        elif sub == "mlp.correction" and f is not None and f.kind == "moe":
            put(lw.correction, t, name)
        elif me and f is not None and f.kind == "moe" and int(me.group(1)) < f.experts:
            e, which = int(me.group(1)), me.group(2)
            if which == "gate":
                put(lw.w13[e, :f.ff], t, name)
            elif which == "up":
                put(lw.w13[e, f.ff:], t, name)
            else:
                put(lw.w2[e], t, name)
        else:
            raise ValueError(f"unexpected tensor {name!r}")
    want = {"embed", "final.norm"}
    for i, lw in enumerate(model.layers):
        m, f = lw.spec.mixer, lw.spec.mlp
        want |= {f"l{i}.norm1", f"l{i}.mix.q", f"l{i}.mix.g", f"l{i}.mix.o"}
        if isinstance(m, NormedAttentionSpec):
            want.add(f"l{i}.mix.sink")
            if m.kv_from is None:
                want |= {f"l{i}.mix.k", f"l{i}.mix.v"}
        else:
            want |= {f"l{i}.mix.k", f"l{i}.mix.v", f"l{i}.mix.norm"}
            want |= ({f"l{i}.mix.{k}" for k in ("i", "i.b", "f", "f.b")} if isinstance(m, MatrixMemorySpec)
                     else {f"l{i}.mix.{k}" for k in ("a1", "a2", "a2.b")})
        if f is not None:
            want.add(f"l{i}.norm2")
            if f.kind == "dense":
                want |= {f"l{i}.mlp.{k}" for k in ("gate", "up", "down")}
            else:
                want |= {f"l{i}.mlp.router", f"l{i}.mlp.correction"}
                want |= {f"l{i}.mlp.e{e}.{k}" for e in range(f.experts) for k in ("gate", "up", "down")}
    if want - seen:
        raise ValueError(f"checkpoint lacks {sorted(want - seen)[:8]}")


def _load_zetalorn(model: ZetalornModel, ckpt_dir: Path) -> None:
    """Zetalorn checkpoints: ``embed``, ``head``, ``final.norm``, ``loop.step`` (models with a layer loop); per layer
    ``l<i>.norm1|norm2`` (one number each), ``l<i>.rg1|rg2`` with ``.b`` (the residual gates), ``l<i>.mix.{q, k, v,
    q.norm, k.norm, lq1, lk1, lq2, lk2, o}`` (attention) or ``l<i>.mix.left.{q, k, v, q.norm, k.norm, o, out}`` and
    ``l<i>.mix.right.{q, k, v, g, norm, o, out}`` (parallel), ``l<i>.mlp.router`` and ``l<i>.mlp.e<j>.{gate, up, down}``.
    Linear weights are [out, in]; a mixer's input projections and the mixer's residual gate are fused row-wise
    here, the units stacked, the norms' single numbers spread over the width.  The query rows of a differential
    attention (stored head by head as map 1 | map 2) are reordered to group, map, head in group.  Every tensor
    the model holds must be found, and every tensor of the file must have a place."""
    from ..engine.config import DiffAttentionSpec

    pat = re.compile(r"l(\d+)\.(.+)")
    unit = re.compile(r"mlp\.e(\d+)\.(gate|up|down)")
    seen: set[str] = set()

    def put(dst: torch.Tensor, src: torch.Tensor, what: str) -> None:
        if tuple(dst.shape) != tuple(src.shape):
            raise ValueError(f"{what}: checkpoint shape {tuple(src.shape)}, model expects {tuple(dst.shape)}")
        dst.copy_(src.to(dst.dtype))

    def put_scalar(dst: torch.Tensor, src: torch.Tensor, what: str) -> None:
        if src.numel() != 1:
            raise ValueError(f"{what}: one number expected, checkpoint shape {tuple(src.shape)}")
        dst.fill_(float(src.float().reshape(())))

    for name, t in _iter_safetensors(ckpt_dir):
        seen.add(name)
        if name == "embed":
            put(model.embed, t, name)
            continue
        if name == "head":
            put(model.lm_head, t, name)
            continue
        if name == "final.norm":
            put_scalar(model.norm, t, name)
            continue
        if name == "loop.step" and model.loop_step is not None:
            put(model.loop_step, t, name)
            continue
        mt = pat.match(name)
        if not mt or int(mt.group(1)) >= len(model.layers):
            raise ValueError(f"unexpected tensor {name!r}")
        lw = model.layers[int(mt.group(1))]
        sub = mt.group(2)
        m, f = lw.spec.mixer, lw.spec.mlp
        rows = model.in_rows(lw.spec)
        diff = isinstance(m, DiffAttentionSpec)
        ok = True
        um = unit.fullmatch(sub)
        if sub == "norm1":
            put_scalar(lw.norm1, t, name)
        elif sub == "rg1":
            put(lw.w_in[rows["rg1"][0]:rows["rg1"][1]], t, name)
        elif sub == "rg1.b":
            put(lw.rg1_b, t, name)
        elif f is not None and sub == "norm2":
            put_scalar(lw.norm2, t, name)
        elif f is not None and sub == "rg2":
            put(lw.rg2, t, name)
        elif f is not None and sub == "rg2.b":
            put(lw.rg2_b, t, name)
        elif f is not None and sub == "mlp.router":
            put(lw.router, t, name)
        elif f is not None and um and int(um.group(1)) < f.experts:
            e, which = int(um.group(1)), um.group(2)
            if which == "down":
                put(lw.w2[e], t, name)
            else:
                put(lw.w13[e, :f.ff] if which == "gate" else lw.w13[e, f.ff:], t, name)
        elif diff and sub == "mix.q":
            a, b = rows["q"]
            if tuple(t.shape) != (b - a, lw.w_in.shape[1]):
                raise ValueError(f"{name}: checkpoint shape {tuple(t.shape)}, model expects {(b - a, lw.w_in.shape[1])}")
            rep = m.heads // m.kv_heads
            t = t.view(m.kv_heads, rep, 2, m.dim, -1).permute(0, 2, 1, 3, 4).reshape(b - a, -1)
            put(lw.w_in[a:b], t, name)
        elif diff and sub in ("mix.k", "mix.v"):
            a, b = rows[sub[4:]]
            put(lw.w_in[a:b], t, name)
        elif diff and sub in ("mix.lq1", "mix.lk1", "mix.lq2", "mix.lk2"):
            put(lw.lam_vecs[("lq1", "lk1", "lq2", "lk2").index(sub[4:])], t, name)
        elif not diff and sub.startswith("mix.") and sub[4:] in rows and sub[4:] != "rg1":
            a, b = rows[sub[4:]]
            put(lw.w_in[a:b], t, name)
        elif sub in ("mix.q.norm", "mix.left.q.norm") and diff == (sub == "mix.q.norm"):
            put(lw.q_norm, t, name)
        elif sub in ("mix.k.norm", "mix.left.k.norm") and diff == (sub == "mix.k.norm"):
            put(lw.k_norm, t, name)
        elif sub in ("mix.o", "mix.left.o") and diff == (sub == "mix.o"):
            put(lw.w_o, t, name)
        elif not diff and sub == "mix.right.o":
            put(lw.wr_o, t, name)
        elif not diff and sub == "mix.right.norm":
            put(lw.r_norm, t, name)
        elif not diff and sub == "mix.left.out":
            put(lw.left_out, t, name)
        elif not diff and sub == "mix.right.out":
            put(lw.right_out, t, name)
        else:
            ok = False
        if not ok:
            raise ValueError(f"unexpected tensor {name!r}")
    want = {"embed", "head", "final.norm"} | ({"loop.step"} if model.loop_step is not None else set())
    for i, lw in enumerate(model.layers):
        m, f = lw.spec.mixer, lw.spec.mlp
        want |= {f"l{i}.{k}" for k in ("norm1", "rg1", "rg1.b")}
        if isinstance(m, DiffAttentionSpec):
            want |= {f"l{i}.mix.{k}" for k in ("q", "k", "v", "q.norm", "k.norm", "lq1", "lk1", "lq2", "lk2", "o")}
            model.set_lambda(lw)
        else:
            want |= {f"l{i}.mix.left.{k}" for k in ("q", "k", "v", "q.norm", "k.norm", "o", "out")}
            want |= {f"l{i}.mix.right.{k}" for k in ("q", "k", "v", "g", "norm", "o", "out")}
        if f is not None:
            want |= {f"l{i}.{k}" for k in ("norm2", "rg2", "rg2.b", "mlp.router")}
            want |= {f"l{i}.mlp.e{e}.{k}" for e in range(f.experts) for k in ("gate", "up", "down")}
    if want - seen:
        raise ValueError(f"checkpoint lacks {sorted(want - seen)[:8]}")
