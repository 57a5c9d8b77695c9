"""Zetalorn on the GPU: the HIP kernels one by one against float64 definitions in both activation dtypes,
then the engine in fp32 and in bf16 against the float64 oracle (same cases as on the CPU), and HIP-graph
decode steps against eager ones."""

import pytest
import torch

import zetalorn_cases as zc
import zetalorn_oracle as zo
from vllm_production_stack_amd import ops
from vllm_production_stack_amd.engine.request import SamplingParams

pytestmark = pytest.mark.gpu

# 16-bit runs: a routing decision that rounding turns over changes a row and says nothing about the kernels, so a few
# rows may miss the bound there; fp32 is the sharp run
MODES = [("float32", 5e-5, 0), ("bfloat16", 8e-2, 8)]
KERNEL_TOL = {"float32": 2e-5, "bfloat16": 2e-2}
DEV = torch.device("cuda")


@pytest.fixture(scope="module")
def model_a():
    cfg = zc.config_a()
    return cfg, zo.make_weights(cfg, seed=3)


@pytest.fixture(scope="module")
def model_b():
    cfg = zc.config_b()
    return cfg, zo.make_weights(cfg, seed=4)


@pytest.fixture(scope="module")
def model_c():
    cfg = zc.config_c()
    return cfg, zo.make_weights(cfg, seed=5)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_gated_residual_and_norm(dtype):
    zc.case_gated_residual(DEV, dtype, KERNEL_TOL[dtype])
    assert ops.native_loaded()


def test_routing():
    zc.case_routing(DEV)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_query_key_norm_and_rotation(dtype):
    zc.case_qk_norm_rotation(DEV, dtype, KERNEL_TOL[dtype])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_chunk_window_and_pooled_blocks(dtype):
    zc.case_masks(DEV, dtype, 2e-5 if dtype == "float32" else 2e-2)   # pooled entries are rounded to the cache's 16 bits


def test_masks_on_the_matrix_cores():
    assert ops.window_mfma_supported(8, 4, 64, 128, True)
    zc.case_masks(DEV, "bfloat16", 3e-2, tiled=True)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_differential_combination(dtype):
    zc.case_differential(DEV, dtype, KERNEL_TOL[dtype])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_lightning_recurrence(dtype):
    zc.case_lightning(DEV, dtype, KERNEL_TOL[dtype])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_recurrence_in_pieces(dtype):
    zc.case_scan_pieces(DEV, dtype, 5e-5)


@pytest.mark.parametrize("dtype,tol,loose", MODES)
def test_layers(dtype, tol, loose, model_a, model_b):
    zc.check_layers("cuda", dtype, tol, *model_a)
    zc.check_layers("cuda", dtype, tol, *model_b)


@pytest.mark.parametrize("dtype,tol,loose", MODES)
def test_whole_decode_and_portions(dtype, tol, loose, model_a):
    zc.check_cuts("cuda", dtype, tol, *model_a, 150, [[150], [118], [64, 64], [63, 2, 63, 2], [2, 2, 2, 58, 1, 64],
                                                      [1, 1, 1, 25, 23, 2]], loose=loose)


@pytest.mark.parametrize("dtype,tol,loose", MODES)
def test_other_sizes_and_first_tokens(dtype, tol, loose, model_b):
    tol = tol if dtype == "float32" else 0.15   # a width of 24 averages bf16 rounding over few terms
    zc.check_cuts("cuda", dtype, tol, *model_b, 160, [[160], [1], [2, 1, 2], [5, 2, 7, 1, 70, 2, 64], [128, 2]], loose=loose)
    zc.check_cuts("cuda", dtype, tol, *model_b, 3, [[3], [1, 2]], loose=loose)


@pytest.mark.parametrize("dtype,tol,loose", MODES)
def test_tiled_kernels_and_pieces_in_the_engine(dtype, tol, loose, model_c):
    cfg, w = model_c
    assert ops.window_mfma_supported(8, 4, 64, 128, True) and ops.window_mfma_supported(2, 1, 128, 128, True)
    assert ops.build_scan_pieces([300]) is not None
    zc.check_cuts("cuda", dtype, tol, cfg, w, 300, [[300], [200, 100], [130, 1, 1, 168], [290]], loose=loose)


@pytest.mark.parametrize("dtype,tol,loose", MODES)
def test_sizes_that_are_multiples_of_nothing(dtype, tol, loose):
    cfg = zc.config_d()
    tol = tol if dtype == "float32" else 0.15   # a width of 20 averages bf16 rounding over few terms
    zc.check_cuts("cuda", dtype, tol, cfg, zo.make_weights(cfg, seed=8), 100, [[100], [66, 2, 1, 20], [1, 1, 3]], loose=loose)
    if dtype == "float32":  # (in 16 bits a width of 20 turns routing decisions over in too many rows to say anything)
        zc.check_batches("cuda", dtype, tol, cfg, zo.make_weights(cfg, seed=8))


@pytest.mark.parametrize("dtype,tol,loose", MODES)
def test_attention_layers_only(dtype, tol, loose):
    cfg = zc.config_e()
    tol = tol if dtype == "float32" else 0.15
    zc.check_cuts("cuda", dtype, tol, cfg, zo.make_weights(cfg, seed=9), 70, [[70], [29, 2, 33], [1, 1, 3]], loose=loose)


@pytest.mark.parametrize("dtype,tol,loose", MODES)
def test_long_decode(dtype, tol, loose, model_a):
    zc.check_cuts("cuda", dtype, tol, *model_a, 330, [[20]], pages=6, loose=loose)


@pytest.mark.parametrize("dtype,tol,loose", MODES)
def test_batches_and_reuse(dtype, tol, loose, model_a):
    zc.check_batches("cuda", dtype, tol, *model_a, loose=loose)


@pytest.mark.parametrize("dtype,tol,loose", MODES)
def test_a_token_far_back(dtype, tol, loose, model_a):
    zc.check_far_token("cuda", dtype, *model_a, tol)


def test_greedy_generation(model_a, model_b):
    zc.check_generate("cuda", "float32", *model_a)
    zc.check_generate("cuda", "float32", *model_b)
    zc.check_preemption("cuda", "float32", *model_a)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_graphs_match_eager(dtype, model_c):
    """Decode steps replayed from HIP graphs (state slots, positions and pages are graph inputs) give the
    tokens of eager steps, replay after replay, with eager prefill steps of new requests in between."""
    cfg, w = model_c
    prompts = [zc.tokens(cfg, n, 90 + n) for n in (70, 3, 33, 64, 20, 9)]
    params = SamplingParams(max_tokens=24, temperature=0.0, ignore_eos=True)
    outs = {}
    for eager in (True, False):
        eng = zc.make_engine(cfg, w, "cuda", dtype, pages=12, slots=3, budget=64, eager=eager)
        outs[eager] = eng.generate(prompts, params)
        if not eager and dtype == "bfloat16":
            assert eng.runner.model.graph_capturable and eng.runner.step_kinds["decode_graph"] > 20
        eng.shutdown()
    assert outs[True] == outs[False]
    if dtype == "float32":
        assert outs[True][0] == zo.greedy(cfg, w, prompts[0], 24)


def test_preset_at_random_weights_generates():
    from vllm_production_stack_amd.engine.config import EngineConfig
    from vllm_production_stack_amd.engine.llm_engine import LLMEngine

    eng = LLMEngine(EngineConfig(model="tiny-zetalorn", dtype="bfloat16", max_model_len=512, max_num_seqs=4,
                                 num_gpu_blocks_override=16, enable_prefix_caching=False))
    outs = eng.generate([[5, 6, 7] * 30, [9] * 3], SamplingParams(max_tokens=8, temperature=0.0, ignore_eos=True))
    assert [len(o) for o in outs] == [8, 8]
    assert eng.sleep(1) > 0 and eng.runner.state_pool is None
    eng.wake_up()
    assert eng.generate([[5, 6, 7] * 30, [9] * 3], SamplingParams(max_tokens=8, temperature=0.0, ignore_eos=True)) == outs
    eng.shutdown()
