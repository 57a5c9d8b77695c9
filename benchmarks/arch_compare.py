"""Prefill and decode throughput of one decoder design beside the closest existing one at equal size.

    python bench.py --arch-compare zururax|revelix|pelatar|zetalorn [--arch-sizes s,m] [--arch-prompt 4096] [--arch-batch 32]

Random weights at layer shapes of real models (a few layers each); both models run through the same
engine (scheduler, paged pool, HIP-graph decode).  Prefill: prompts of --arch-prompt tokens in chunks of
--max-num-batched-tokens, tokens per second until every prompt has its first token.  Decode:
--arch-batch sequences with --arch-context tokens of context each, tokens per second over the timed
decode steps.  One JSON line per (size, model), then one summary line.
"""

from __future__ import annotations

import json
import time

import torch

SIZES = {
    # width, layers, heads, experts, unit width, units per token, shared / dense width
    "s": dict(width=2048, layers=4, heads=16, experts=16, ff=1024, top=4, shared=1024, q_rank=768),
    "m": dict(width=4096, layers=4, heads=32, experts=32, ff=2048, top=4, shared=2048, q_rank=1536),
}
VOCAB = 32000


def _configs(design: str, size: str):
    from vllm_production_stack_amd.engine.config import ModelConfig, zururax_config

    z = SIZES[size]
    if design == "revelix":
        return _revelix_configs(size)
    if design == "pelatar":
        return _pelatar_configs(size)
    if design == "zetalorn":
        return _zetalorn_configs(size)
    if design != "zururax":
        raise SystemExit(f"--arch-compare: unknown design {design!r}")

    def mixer(i):
        m = {"heads": z["heads"], "dim": 128, "rot_dim": 64, "vdim": 128, "kv_rank": 512, "q_rank": z["q_rank"],
             "rot": {"base": 10000.0, "dims": 64}, "scale": 192 ** -0.5}
        if i % 2:
            m["kv_from"] = i - 1  # every second layer reads its neighbour's entries
        return m

    moe = {"kind": "moe", "expert": {"ff": z["ff"], "limit": 7.0},
           "router": {"experts": z["experts"], "top": z["top"], "groups": {"count": 4, "keep": 2}, "scale": 2.5},
           "shared": {"ff": z["shared"], "limit": 7.0}}
    dense = {"kind": "dense", "ff": z["top"] * z["ff"] + z["shared"]}
    new = zururax_config(f"zururax-{size}", VOCAB, z["width"],
                         [{"type": "latent_attention", "mixer": mixer(i), "mlp": dense if i == 0 else moe}
                          for i in range(z["layers"])], max_position_embeddings=32768)
    # the closest existing design: grouped-query attention + top-k softmax mixture, same width, depth,
    # heads, unit count and unit width
    old = ModelConfig(name=f"mixtral-{size}", architecture="mixtral", vocab_size=VOCAB, hidden_size=z["width"],
                      intermediate_size=z["ff"], num_layers=z["layers"], num_heads=z["heads"],
                      num_kv_heads=max(1, z["heads"] // 4), head_dim=128, num_experts=z["experts"],
                      num_experts_per_tok=z["top"], max_position_embeddings=32768)
    return new, old


def _revelix_configs(size: str):
    """Revelix (retention | parallel | parallel | retention, every layer with a feed-forward of four times the
    width) beside the closest existing design: a dense grouped-query decoder of the same width, depth, heads
    and feed-forward parameter count."""
    from vllm_production_stack_amd.engine.config import ModelConfig, revelix_config

    z = SIZES[size]
    w, heads = z["width"], z["heads"]
    ff = 4 * w
    mlp = {"kind": "dense", "ff": ff}
    retention = {"type": "retention", "mlp": mlp,
                 "mixer": {"heads": heads, "dim": 128, "vdim": 256, "rot": {"base": 10000.0, "dims": 128},
                           "decay": [1 - 2.0 ** (-5 - 3 * i / heads) for i in range(heads)]}}
    parallel = {"type": "parallel", "mlp": mlp,
                "mixer": {"left": {"heads": heads, "kv_heads": heads // 4, "dim": 128, "vdim": 128, "conv": 4,
                                   "mask": {"size": 1024, "keep_first": 4},
                                   "rot": {"base": 1e6, "dims": 128,
                                           "scaling": {"factor": 8.0, "original": 4096, "fast": 32.0, "slow": 1.0}},
                                   "scale": 128 ** -0.5, "softcap": 50.0},
                          "right": {"heads": heads // 2, "dim": 128, "vdim": 128},
                          "left_scale": 0.7, "right_scale": 0.7}}
    new = revelix_config(f"revelix-{size}", VOCAB, w, [retention, parallel, parallel, retention], logit_scale=0.5,
                         max_position_embeddings=32768)
    old = ModelConfig(name=f"llama-{size}", architecture="llama", vocab_size=VOCAB, hidden_size=w,
                      intermediate_size=(2 * ff // 3 + 255) // 256 * 256, num_layers=4, num_heads=heads,
                      num_kv_heads=heads // 4, head_dim=128, max_position_embeddings=32768)
    return new, old


def _pelatar_configs(size: str):
    """Pelatar (matrix memory | gated linear attention | attention | attention on its neighbour's keys and values;
    dense gated gelu units and routed silu units with identity experts in turn) beside the closest existing design,
    Revelix at the same width, depth and head shapes: its recurrences run the same scan kernel, its attention the
    same tile kernel (there with a window and head mixing), its feed-forward holds the parameters of the dense
    gated unit here."""
    from vllm_production_stack_amd.engine.config import pelatar_config, pelatar_stack

    z = SIZES[size]
    w = z["width"]
    ff = (8 * w // 3 + 255) // 256 * 256
    new = pelatar_config(f"pelatar-{size}", VOCAB, w,
                         pelatar_stack(w, z["heads"], ff, z["experts"] - 4, z["ff"], z["top"], 4),
                         max_position_embeddings=32768)
    return new, _revelix_configs(size)[0]


def _zetalorn_configs(size: str):
    """Zetalorn (a differential attention layer over chunks of 2048 positions and a parallel layer: a window of 1024
    positions with pooled blocks of 16 tokens before it, beside a lightning recurrence; routed clamped units behind
    both; the pair runs twice, so four layer runs) beside the closest existing design, Pelatar at the same width,
    depth and head shapes: its attention runs the same tile kernel (one map per head, plain causal), its
    recurrences the same scan kernel, its routed units the same grouped GEMMs."""
    from vllm_production_stack_amd.engine.config import zetalorn_config, zetalorn_stack

    z = SIZES[size]
    new = zetalorn_config(f"zetalorn-{size}", VOCAB, z["width"],
                          zetalorn_stack(z["width"], z["heads"], z["experts"], z["ff"], z["top"]),
                          loop={"start": 0, "stop": 2, "times": 2}, logit_scale=0.5, max_position_embeddings=32768)
    return new, _pelatar_configs(size)[0]


def _measure(cfg, a) -> dict:
    from vllm_production_stack_amd.engine.config import PRESETS, EngineConfig
    from vllm_production_stack_amd.engine.llm_engine import LLMEngine
    from vllm_production_stack_amd.engine.request import SamplingParams

    PRESETS[cfg.name] = cfg
    page = 64
    need = max(a.arch_prompts * (a.arch_prompt + 2 * page), a.arch_batch * (a.arch_context + a.arch_decode_steps + 2 * page))
    eng = LLMEngine(EngineConfig(model=cfg.name, dtype="bfloat16", max_model_len=32768, max_num_seqs=max(a.arch_batch, 8),
                                 max_num_batched_tokens=a.max_num_batched_tokens, num_gpu_blocks_override=need // page + 8,
                                 enable_prefix_caching=False, prefill_step_ms=0.0))
    g = torch.Generator().manual_seed(0)

    def prompts(n, length):
        return [torch.randint(10, VOCAB - 10, (length,), generator=g).tolist() for _ in range(n)]

    def run_until_first_tokens(ps, max_tokens):
        reqs = [eng.add_request(p, SamplingParams(max_tokens=max_tokens, temperature=0.0, ignore_eos=True)) for p in ps]
        while any(not r.output_ids for r in reqs):
            eng.step()
        return reqs

    def drain():
        while eng.has_work():
            eng.step()

    out = {"model": cfg.name, "params_b": round(cfg.num_params() / 1e9, 2)}
    # prefill
    run_until_first_tokens(prompts(1, a.arch_prompt), 1)  # warm-up: library plans, lazy buffers
    drain()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    run_until_first_tokens(prompts(a.arch_prompts, a.arch_prompt), 1)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    drain()
    out["prefill_tok_s"] = round(a.arch_prompts * a.arch_prompt / dt, 1)
    # decode
    reqs = run_until_first_tokens(prompts(a.arch_batch, a.arch_context), a.arch_decode_steps + 9)
    for _ in range(4):
        eng.step()
    torch.cuda.synchronize()
    n0 = sum(len(r.output_ids) for r in reqs)
    t0 = time.perf_counter()
    for _ in range(a.arch_decode_steps):
        eng.step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    out["decode_tok_s"] = round((sum(len(r.output_ids) for r in reqs) - n0) / dt, 1)
    out["decode_ms_per_step"] = round(1e3 * dt / a.arch_decode_steps, 3)
    out["decode_steps_by_kind"] = dict(eng.runner.step_kinds)
    drain()
    eng.shutdown()
    return out


def main(a) -> None:
    torch.cuda.set_device(0)
    results = []
    for size in [s for s in a.arch_sizes.split(",") if s]:
        for cfg in _configs(a.arch_compare, size):
            r = {"size": size, **_measure(cfg, a)}
            print(json.dumps(r), flush=True)
            results.append(r)
    summary = {"metric": "arch_compare", "design": a.arch_compare, "prompt": a.arch_prompt, "prompts": a.arch_prompts,
               "batch": a.arch_batch, "context": a.arch_context, "dtype": "bf16", "data": "synthetic", "n_gpus": 1,
               "ratios": {}}
    for size in {r["size"] for r in results}:
        new, old = [r for r in results if r["size"] == size]
        summary["ratios"][size] = {"prefill": round(new["prefill_tok_s"] / old["prefill_tok_s"], 3),
                                   "decode": round(new["decode_tok_s"] / old["decode_tok_s"], 3)}
    print(json.dumps(summary), flush=True)
