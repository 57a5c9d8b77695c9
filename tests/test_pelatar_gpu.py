"""Pelatar on the GPU: the HIP kernels one by one against float64 definitions in both activation dtypes,
then the engine in fp32 and in bf16 against the float64 oracle (same cases as on the CPU), and HIP-graph
decode steps against eager ones."""

import pytest
import torch

import pelatar_cases as pc
import pelatar_oracle as po
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
    cfg = pc.config_a()
    return cfg, po.random_weights(cfg, seed=3)


@pytest.fixture(scope="module")
def model_b():
    cfg = pc.config_b()
    return cfg, po.random_weights(cfg, seed=4)


@pytest.fixture(scope="module")
def model_c():
    cfg = pc.config_c()
    return cfg, po.random_weights(cfg, seed=5)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_norm_on_the_sublayer_output(dtype):
    pc.case_norm_on_output(DEV, dtype, KERNEL_TOL[dtype])
    assert ops.native_loaded()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_gated_units(dtype):
    pc.case_gated_units(DEV, dtype, KERNEL_TOL[dtype])


def test_routing():
    pc.case_routing(DEV)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_unit_rms_queries_keys_and_temperature(dtype):
    pc.case_qk_norm(DEV, dtype, KERNEL_TOL[dtype])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_attention_with_sink(dtype):
    pc.case_attention(DEV, dtype, 2e-5)  # scores, weights and their sums are fp32 in both


@pytest.mark.parametrize("heads,kv_heads,dim,vdim", [(4, 2, 64, 128), (8, 2, 128, 128), (3, 1, 64, 256), (16, 4, 128, 128),
                                                      (4, 4, 128, 512), (6, 3, 128, 384)])
def test_attention_on_the_matrix_cores(heads, kv_heads, dim, vdim):
    assert ops.window_mfma_supported(heads, kv_heads, dim, vdim, True)
    pc.case_attention(DEV, "bfloat16", 1.5e-2, shapes=[(heads, kv_heads, dim, vdim)])  # weights enter the second product in bf16


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_matrix_memory(dtype):
    pc.case_matrix_memory(DEV, dtype, KERNEL_TOL[dtype])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decayed_memory(dtype):
    pc.case_decayed_memory(DEV, dtype, KERNEL_TOL[dtype])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_recurrences_in_pieces(dtype):
    pc.case_scan_pieces(DEV, dtype, 5e-5)


@pytest.mark.parametrize("dtype,tol,loose", MODES)
def test_layers(dtype, tol, loose, model_a, model_b):
    pc.check_layers("cuda", dtype, tol, *model_a)
    pc.check_layers("cuda", dtype, tol, *model_b)


@pytest.mark.parametrize("dtype,tol,loose", MODES)
def test_whole_decode_and_portions(dtype, tol, loose, model_a):
    pc.check_cuts("cuda", dtype, tol, *model_a, 150, [[150], [118], [64, 64], [63, 2, 63, 2], [2, 2, 2, 58, 1, 64],
                                                      [1, 1, 1, 25, 23, 2]], loose=loose)


@pytest.mark.parametrize("dtype,tol,loose", MODES)
def test_other_sizes_and_first_tokens(dtype, tol, loose, model_b):
    pc.check_cuts("cuda", dtype, tol, *model_b, 140, [[140], [1], [2, 1, 2], [3, 61, 64], [70, 5, 60]], loose=loose)
    pc.check_cuts("cuda", dtype, tol, *model_b, 3, [[3], [1, 2]], loose=loose)


@pytest.mark.parametrize("dtype,tol,loose", MODES)
def test_tiled_kernels_and_pieces_in_the_engine(dtype, tol, loose, model_c):
    cfg, w = model_c
    assert ops.window_mfma_supported(4, 2, 64, 128, True) and ops.build_scan_pieces([300]) is not None
    pc.check_cuts("cuda", dtype, tol, cfg, w, 300, [[300], [200, 100], [130, 1, 1, 168], [290]], loose=loose)


@pytest.mark.parametrize("dtype,tol,loose", MODES)
def test_decode_sized_mixture_kernels(dtype, tol, loose):
    cfg = pc.config_e()
    assert ops.moe_mfma_supported(128, 512)
    pc.check_cuts("cuda", dtype, tol, cfg, po.random_weights(cfg, seed=7), 120, [[120], [70, 40, 3], [30, 2, 2]], loose=loose)


@pytest.mark.parametrize("dtype,tol,loose", MODES)
def test_sizes_that_are_multiples_of_nothing(dtype, tol, loose):
    cfg = pc.config_f()
    tol = tol if dtype == "float32" else 0.15   # a width of 20 averages bf16 rounding over few terms
    pc.check_cuts("cuda", dtype, tol, cfg, po.random_weights(cfg, seed=8), 100, [[100], [66, 2, 1, 20], [1, 1, 3]], loose=loose)
    if dtype == "float32":  # (in 16 bits a width of 20 turns routing decisions over in too many rows to say anything)
        pc.check_batches("cuda", dtype, tol, cfg, po.random_weights(cfg, seed=8))


@pytest.mark.parametrize("dtype,tol,loose", MODES)
def test_recurrences_only(dtype, tol, loose):
    cfg = pc.config_d()
    tol = tol if dtype == "float32" else 0.15   # a width of 24 averages bf16 rounding over few terms
    pc.check_cuts("cuda", dtype, tol, cfg, po.random_weights(cfg, seed=6), 130, [[130], [66, 2, 1, 61], [1, 1, 1, 1, 3]])


@pytest.mark.parametrize("dtype,tol,loose", MODES)
def test_long_decode(dtype, tol, loose, model_b):
    pc.check_cuts("cuda", dtype, tol, *model_b, 330, [[20]], pages=6, loose=loose)


@pytest.mark.parametrize("dtype,tol,loose", MODES)
def test_batches_and_reuse(dtype, tol, loose, model_a):
    pc.check_batches("cuda", dtype, tol, *model_a, loose=loose)


@pytest.mark.parametrize("dtype,tol,loose", MODES)
def test_a_token_far_back(dtype, tol, loose, model_a):
    pc.check_far_token("cuda", dtype, *model_a, tol)


def test_greedy_generation(model_a, model_b):
    pc.check_generate("cuda", "float32", *model_a)
    pc.check_generate("cuda", "float32", *model_b)
    pc.check_preemption("cuda", "float32", *model_a)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_graphs_match_eager(dtype, model_c):
    """Decode steps replayed from HIP graphs (state slots, positions and pages are graph inputs) give the
    tokens of eager steps, replay after replay, with eager prefill steps of new requests in between."""
    cfg, w = model_c
    prompts = [pc.tokens(cfg, n, 90 + n) for n in (70, 3, 33, 64, 20, 9)]
    params = SamplingParams(max_tokens=24, temperature=0.0, ignore_eos=True)
    outs = {}
    for eager in (True, False):
        eng = pc.make_engine(cfg, w, "cuda", dtype, pages=12, slots=3, budget=64, eager=eager)
        outs[eager] = eng.generate(prompts, params)
        if not eager and dtype == "bfloat16":
            assert eng.runner.model.graph_capturable and eng.runner.step_kinds["decode_graph"] > 20
        eng.shutdown()
    assert outs[True] == outs[False]
    if dtype == "float32":
        assert outs[True][0] == po.greedy(cfg, w, prompts[0], 24)


def test_preset_at_random_weights_generates():
    from vllm_production_stack_amd.engine.config import EngineConfig
    from vllm_production_stack_amd.engine.llm_engine import LLMEngine

    eng = LLMEngine(EngineConfig(model="tiny-pelatar", dtype="bfloat16", max_model_len=512, max_num_seqs=4,
                                 num_gpu_blocks_override=16, enable_prefix_caching=False))
    outs = eng.generate([[5, 6, 7] * 30, [9] * 3], SamplingParams(max_tokens=8, temperature=0.0, ignore_eos=True))
    assert [len(o) for o in outs] == [8, 8]
    assert eng.sleep(1) > 0 and eng.runner.state_pool is None
    eng.wake_up()
    assert eng.generate([[5, 6, 7] * 30, [9] * 3], SamplingParams(max_tokens=8, temperature=0.0, ignore_eos=True)) == outs
    eng.shutdown()
