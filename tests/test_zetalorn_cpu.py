"""Zetalorn on the CPU (the PyTorch definitions of the ops, fp32): every mechanism against its float64
definition, then the engine (scheduler, pages, state slots, batch assembly, model) against the oracle."""

import json
import os
import subprocess
import sys
import tempfile

import pytest
import torch

import zetalorn_cases as zc
import zetalorn_oracle as zo
from vllm_production_stack_amd.engine.config import (PRESETS, DiffAttentionSpec, LightningSpec, ParallelMixerSpec,
                                                     PooledWindowSpec, resolve_model, zetalorn_config, zetalorn_layers)

DEV = torch.device("cpu")
TOL = 2e-5


@pytest.fixture(scope="module")
def model_a():
    cfg = zc.config_a()
    return cfg, zo.make_weights(cfg, seed=3)


@pytest.fixture(scope="module")
def model_b():
    cfg = zc.config_b()
    return cfg, zo.make_weights(cfg, seed=4)


def test_gated_residual_and_norm():
    zc.case_gated_residual(DEV, "float32", 1e-5)


def test_routing():
    zc.case_routing(DEV)


def test_query_key_norm_and_rotation():
    zc.case_qk_norm_rotation(DEV, "float32", 1e-5)


def test_chunk_window_and_pooled_blocks():
    zc.case_masks(DEV, "float32", 2e-5)


def test_differential_combination():
    zc.case_differential(DEV, "float32", 1e-5)


def test_lightning_recurrence():
    zc.case_lightning(DEV, "float32", 2e-5)


def test_config_reader(model_a):
    cfg, _ = model_a
    specs = zetalorn_layers(json.loads(json.dumps(cfg["layers"])))
    assert [type(s.mixer) for s in specs] == [ParallelMixerSpec, DiffAttentionSpec, ParallelMixerSpec, DiffAttentionSpec]
    left, right = specs[0].mixer.left, specs[0].mixer.right
    assert isinstance(left, PooledWindowSpec) and isinstance(right, LightningSpec) and specs[0].mixer.normed
    assert (left.window, left.pool, left.rot.layout, left.rot.linear) == (40, 5, "half", None)
    assert specs[1].mixer.chunk == 70 and specs[1].mixer.rot.layout == "pairs" and specs[1].mixer.rot.linear == 4.0
    assert specs[2].mlp is None and specs[3].mlp.norm_topk and specs[3].mlp.groups == 1
    mc = zetalorn_config("x", cfg["vocab"], cfg["width"], cfg["layers"], loop=cfg["loop"], logit_scale=cfg["logit_scale"])
    assert mc.layer_runs() == [(0, None), (1, 0), (2, None), (1, 1), (2, None), (1, 2), (2, None), (3, None)]
    assert mc.num_params() > 0 and mc.prefill_flops()[0] > 0 and not mc.tie_word_embeddings
    for path, value in ((("mixer", "left", "kv_heads"), 3), (("mixer", "right", "decay"), [0.5]),
                        (("mlp", "router", "groups", "count"), 4), (("mixer", "left", "rot", "dims"), 14)):
        bad = json.loads(json.dumps(cfg["layers"]))
        at = bad[0]
        for k in path[:-1]:
            at = at[k]
        at[path[-1]] = value
        with pytest.raises(ValueError):
            zetalorn_layers(bad)
    with pytest.raises(ValueError):
        zetalorn_config("x", 10, 8, cfg["layers"], loop={"start": 2, "stop": 2, "times": 2})
    assert PRESETS["tiny-zetalorn"].architecture == "zetalorn" and PRESETS["tiny-zetalorn"].num_params() > 0


def test_loader_refuses_what_does_not_fit(model_a):
    cfg, w = model_a
    from vllm_production_stack_amd.models.loader import build_model

    def load(weights):
        folder = zo.save_checkpoint(tempfile.mkdtemp(prefix="zx-"), cfg, weights)
        mc, where = resolve_model(folder)
        return build_model(mc, torch.float32, DEV, 256, ckpt_dir=where)

    model = load(w)
    assert model.layers[1].lam == pytest.approx(float(
        torch.exp((w["l1.mix.lq1"].double() * w["l1.mix.lk1"].double()).sum())
        - torch.exp((w["l1.mix.lq2"].double() * w["l1.mix.lk2"].double()).sum()) + 0.2), rel=1e-6)
    lacking = {k: v for k, v in w.items() if k != "l2.mix.right.out"}
    with pytest.raises(ValueError, match="lacks"):
        load(lacking)
    with pytest.raises(ValueError, match="unexpected"):
        load({**w, "l2.norm2": torch.ones(())})   # a layer without a feed-forward has no second norm
    with pytest.raises(ValueError, match="shape"):
        load({**w, "l1.mix.k": w["l1.mix.k"][:-1]})
    with pytest.raises(ValueError, match="one number"):
        load({**w, "final.norm": torch.ones(3)})


def test_residual_stream_after_every_run(model_a, model_b):
    zc.check_layers("cpu", "float32", 1e-5, *model_a)
    zc.check_layers("cpu", "float32", 1e-5, *model_b)


def test_whole_prompt_token_by_token_and_portions(model_a):
    cfg, w = model_a
    # 150 tokens: portions that end at and around the page border, inside blocks, chunks and windows; down to two tokens
    zc.check_cuts("cpu", "float32", TOL, cfg, w, 150, [[150], [], [64, 64, 22], [63, 2, 5, 58, 2, 2, 18], [3, 2, 2, 130]])


def test_other_corners(model_b):
    cfg, w = model_b
    zc.check_cuts("cpu", "float32", TOL, cfg, w, 160, [[160], [5, 2, 7, 1, 70, 2, 64], [128, 2]], seed=2)


def test_first_tokens(model_a, model_b):
    for cfg, w in (model_a, model_b):
        zc.check_cuts("cpu", "float32", TOL, cfg, w, 1, [[1]])
        zc.check_cuts("cpu", "float32", TOL, cfg, w, 3, [[3], [], [2, 1]])


def test_sizes_that_are_multiples_of_nothing():
    cfg = zc.config_d()
    zc.check_cuts("cpu", "float32", TOL, cfg, zo.make_weights(cfg, seed=8), 100, [[100], [66, 2, 1, 20], [1, 1, 3]])


def test_attention_layers_only():
    cfg = zc.config_e()
    zc.check_cuts("cpu", "float32", TOL, cfg, zo.make_weights(cfg, seed=9), 70, [[70], [29, 2, 33], [1, 1, 3]])


def test_long_decoding(model_b):
    cfg, w = model_b
    zc.check_cuts("cpu", "float32", TOL, cfg, w, 200, [[60]], seed=4)   # 140 tokens one by one, across three pages


def test_batches_of_unequal_requests(model_a):
    zc.check_batches("cpu", "float32", TOL, *model_a)


def test_a_token_far_back(model_a):
    cfg, w = model_a
    zc.check_far_token("cpu", "float32", cfg, w, TOL)


def test_generation_through_the_engine(model_a):
    zc.check_generate("cpu", "float32", *model_a, n_new=6)


def test_preemption(model_b):
    zc.check_preemption("cpu", "float32", *model_b)


def test_replay_command(model_a):
    """The replay program on a checkpoint directory: steps on stdin, logits files, one 'done' line per step."""
    cfg, w = model_a
    folder = zo.save_checkpoint(tempfile.mkdtemp(prefix="zx-"), cfg, w)
    out = tempfile.mkdtemp(prefix="zx-out-")
    toks = zc.tokens(cfg, 70, 9)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": toks[:40], "want": [0, 39]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": toks[40:69], "want": []}, {"id": "b", "tokens": toks[:2], "want": [1]}],
              "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": toks[69:], "want": [0]}], "end": ["a"]}]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", "float32",
                        "--out", out, "--max-tokens", "192", "--device", "cpu"],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [ln for ln in r.stdout.splitlines() if ln.startswith("done")] == ["done 0", "done 1", "done 2"]
    want = zo.forward(cfg, w, toks)
    import numpy as np

    got0 = torch.from_numpy(np.fromfile(os.path.join(out, "0.f32"), dtype="<f4").reshape(2, -1))
    got1 = torch.from_numpy(np.fromfile(os.path.join(out, "1.f32"), dtype="<f4").reshape(1, -1))
    got2 = torch.from_numpy(np.fromfile(os.path.join(out, "2.f32"), dtype="<f4").reshape(1, -1))
    zc.check_rows(got0, want[[0, 39]], TOL, "step 0")
    zc.check_rows(got1, want[[1]], TOL, "step 1")
    zc.check_rows(got2, want[[69]], TOL, "step 2")
