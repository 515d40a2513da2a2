"""Revelix on the GPU: the HIP kernels one by one against float64 definitions in both activation dtypes,
then the engine in fp32 and in bf16 against the float64 oracle (same cases as on the CPU), and HIP-graph
decode steps against eager ones."""

import pytest
import torch

import revelix_cases as rc
import revelix_oracle as ro
from vllm_production_stack_amd import ops
from vllm_production_stack_amd.engine.request import SamplingParams

pytestmark = pytest.mark.gpu

MODES = [("float32", 5e-5), ("bfloat16", 6e-2)]
KERNEL_TOL = {"float32": 2e-5, "bfloat16": 2e-2}
DEV = torch.device("cuda")


@pytest.fixture(scope="module")
def model_a():
    cfg = rc.config_a()
    return cfg, ro.random_weights(cfg, seed=3)


@pytest.fixture(scope="module")
def model_b():
    cfg = rc.config_b()
    return cfg, ro.random_weights(cfg, seed=4)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_norm_and_activation(dtype):
    rc.case_dyt_and_xielu(DEV, dtype, KERNEL_TOL[dtype])
    assert ops.native_loaded()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_recurrences(dtype):
    rc.case_recurrences(DEV, dtype, 2e-5)  # fp32 inside whatever the activations


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_recurrence_in_pieces(dtype):
    rc.case_recurrence_pieces(DEV, dtype, 2e-5)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_head_norm(dtype):
    rc.case_head_norm(DEV, dtype, KERNEL_TOL[dtype])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_short_convolution(dtype):
    rc.case_short_conv(DEV, dtype, KERNEL_TOL[dtype])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_window_edges(dtype):
    rc.case_window_edges(DEV, dtype, 2e-5)  # scores, weights and their sums are fp32 in both
    rc.case_far_keys(DEV, dtype, 2e-5)


@pytest.mark.parametrize("heads,kv_heads,dim,vdim,size,keep", [(4, 2, 64, 64, 70, 3), (8, 2, 128, 128, 100, 0),
                                                                (3, 1, 64, 128, 64, 65), (16, 4, 128, 128, 129, 4),
                                                                (4, 4, 128, 64, 1000, 2), (16, 8, 64, 128, 90, 5),
                                                                (6, 3, 128, 128, 70, 1)])
def test_window_attention_on_the_matrix_cores(heads, kv_heads, dim, vdim, size, keep):
    rc.case_window_tiles(DEV, heads, kv_heads, dim, vdim, size, keep)


@pytest.mark.parametrize("dtype,tol", MODES)
def test_layers(dtype, tol, model_a, model_b):
    rc.check_layers("cuda", dtype, tol, *model_a)
    rc.check_layers("cuda", dtype, tol, *model_b)


@pytest.mark.parametrize("dtype,tol", MODES)
def test_whole_decode_and_portions(dtype, tol, model_a):
    rc.check_cuts("cuda", dtype, tol, *model_a, 150, [[150], [118], [64, 64], [63, 2, 63, 2], [2, 2, 2, 58, 1, 64],
                                                      [1, 1, 1, 25, 23, 2]])


@pytest.mark.parametrize("dtype,tol", MODES)
def test_other_sizes_and_first_tokens(dtype, tol, model_b):
    rc.check_cuts("cuda", dtype, tol, *model_b, 140, [[140], [1], [2, 1, 2], [3, 61, 64], [70, 5, 60]])
    rc.check_cuts("cuda", dtype, tol, *model_b, 3, [[3], [1, 2]])


@pytest.mark.parametrize("dtype,tol", MODES)
def test_tiled_attention_and_pieces_in_the_engine(dtype, tol):
    cfg = rc.config_c()
    w = ro.random_weights(cfg, seed=5)
    assert ops.window_mfma_supported(4, 2, 64, 64) and ops.build_scan_pieces([300]) is not None
    rc.check_cuts("cuda", dtype, tol, cfg, w, 300, [[300], [200, 100], [130, 1, 1, 168], [290]])


@pytest.mark.parametrize("dtype,tol", MODES)
def test_one_kind_of_layer_only(dtype, tol):
    # widths of 16 and 24 average bf16 rounding over few terms: fp32 is the sharp run, bf16 a sanity bound
    tol = tol if dtype == "float32" else 0.15
    for cfg in (rc.config_d(), rc.config_e()):
        rc.check_cuts("cuda", dtype, tol, cfg, ro.random_weights(cfg, seed=6), 130, [[130], [66, 2, 1, 61], [1, 1, 1, 1, 3]])


@pytest.mark.parametrize("dtype,tol", MODES)
def test_long_decode(dtype, tol, model_b):
    rc.check_cuts("cuda", dtype, tol, *model_b, 330, [[20]], pages=6)


@pytest.mark.parametrize("dtype,tol", MODES)
def test_batches_and_reuse(dtype, tol, model_a):
    rc.check_batches("cuda", dtype, tol, *model_a)


def test_greedy_generation(model_a, model_b):
    rc.check_generate("cuda", "float32", *model_a)
    rc.check_generate("cuda", "float32", *model_b)
    rc.check_preemption("cuda", "float32", *model_a)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_graphs_match_eager(dtype, model_a):
    """Decode steps replayed from HIP graphs (state slots, positions and pages are graph inputs) give the
    tokens of eager steps, replay after replay, with eager prefill steps of new requests in between."""
    cfg, w = model_a
    prompts = [rc.tokens(cfg, n, 90 + n) for n in (70, 3, 33, 64, 20, 9)]
    params = SamplingParams(max_tokens=24, temperature=0.0, ignore_eos=True)
    outs = {}
    for eager in (True, False):
        eng = rc.make_engine(cfg, w, "cuda", dtype, pages=12, slots=3, budget=64, eager=eager)
        outs[eager] = eng.generate(prompts, params)
        if not eager:
            assert eng.runner.step_kinds["decode_graph"] > 20
        eng.shutdown()
    assert outs[True] == outs[False]
    if dtype == "float32":
        assert outs[True][0] == ro.greedy(cfg, w, prompts[0], 24)


def test_sleep_and_wake_keep_the_tokens(model_a):
    """The state pool leaves with the KV pool and comes back; stochastic sampling takes the fp32 logits."""
    cfg, w = model_a
    eng = rc.make_engine(cfg, w, "cuda", "bfloat16", pages=8, slots=3, eager=False)
    prompts = [rc.tokens(cfg, n, 200 + n) for n in (50, 3, 70)]
    greedy = SamplingParams(max_tokens=12, temperature=0.0, ignore_eos=True)
    first = eng.generate(prompts, greedy)
    sampled = eng.generate(prompts[:2], SamplingParams(max_tokens=8, temperature=0.9, top_p=0.9, seed=3, ignore_eos=True))
    assert [len(o) for o in sampled] == [8, 8]
    assert eng.sleep(1) > 0 and eng.runner.state_pool is None
    eng.wake_up()
    assert eng.generate(prompts, greedy) == first
    eng.shutdown()
