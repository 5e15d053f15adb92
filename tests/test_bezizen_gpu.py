"""Bezizen family on an MI355X: the HIP kernels, in exact fp32 mode and in
the bf16 serving mode, against the plain model in bezizen_oracle.py."""
import os
import sys

import pytest

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import bezizen_cases as cases  # noqa: E402

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
BOTH = pytest.mark.parametrize("dtype", ["fp32", "bf16"])


def test_kernel_group_is_loaded():
    from kukeon_amd import ops
    assert ops.strm_available(), "kukeon_amd/_C_strm.so is not built"


@BOTH
def test_op_streams(dtype):
    cases.case_op_streams(DEV, dtype)


@BOTH
def test_op_shift(dtype):
    cases.case_op_shift(DEV, dtype)


@BOTH
@pytest.mark.parametrize("mode", [0, 1])
def test_op_scan(mode, dtype):
    cases.case_op_scan(DEV, dtype, mode=mode)
    cases.case_op_scan(DEV, dtype, mode=mode, H=2, d=40, dv=3,
                       cuts=(1, 1, 20, 2))
    # state rows over several lanes, more than one tile of tokens
    cases.case_op_scan(DEV, dtype, mode=mode, H=2, d=128, dv=64,
                       cuts=(37, 1, 3))
    # 32 rows per thread
    cases.case_op_scan(DEV, dtype, mode=mode, H=1, d=128, dv=128,
                       cuts=(5, 18))
    cases.case_op_scan(DEV, dtype, mode=mode, H=3, d=64, dv=24,
                       cuts=(2, 30, 1, 1))


def test_op_router():
    cases.case_op_router(DEV)


@BOTH
@pytest.mark.parametrize("name", sorted(cases.CONFIGS))
def test_whole_prompt(name, dtype):
    cases.case_whole(name, DEV, dtype)


@BOTH
def test_residual_after_every_layer(dtype):
    cases.case_layers(DEV, dtype)


@BOTH
@pytest.mark.parametrize("name", ["hybrid", "aligned", "plain", "one_stream"])
def test_prefill_against_token_by_token(name, dtype):
    cases.case_prefill_vs_decode(name, DEV, dtype)


@BOTH
@pytest.mark.parametrize("sizes", [(2,), (3, 2, 7), (16, 1, 5)])
def test_portions(sizes, dtype):
    cases.case_portions("hybrid", DEV, dtype, sizes)
    cases.case_portions("aligned", DEV, dtype, sizes)


@BOTH
@pytest.mark.parametrize("name", ["hybrid", "aligned", "plain"])
def test_unequal_batch(name, dtype):
    cases.case_batch(name, DEV, dtype)


@BOTH
def test_pages_and_slots_reused(dtype):
    cases.case_reuse(DEV, dtype)


@BOTH
def test_first_tokens(dtype):
    cases.case_first_tokens(DEV, dtype)


@BOTH
def test_long_decode(dtype):
    cases.case_long_decode(DEV, dtype)


@BOTH
def test_long_window(dtype):
    cases.case_long_window(DEV, dtype)


@BOTH
def test_long_portions(dtype):
    cases.case_long_portions(DEV, dtype)


@BOTH
def test_long_portions_sort_rows_by_expert(dtype):
    cases.case_sorted_experts(DEV, dtype)


@BOTH
@pytest.mark.parametrize("decode", [False, True])
def test_window_edges(decode, dtype):
    cases.case_window_edges(DEV, dtype, decode)


@BOTH
def test_state_is_carried(dtype):
    cases.case_state_carry(DEV, dtype)


@BOTH
def test_router(dtype):
    cases.case_router(DEV, dtype)


@BOTH
@pytest.mark.parametrize("graphs", [False, True])
def test_greedy_generation(graphs, dtype):
    cases.case_generate(DEV, dtype, use_graphs=graphs)


@BOTH
def test_multi_turn_and_eviction(dtype):
    cases.case_multi_turn(DEV, dtype)


def test_checkpoint_folder(tmp_path):
    cases.case_registry(tmp_path, DEV, "bf16")


@BOTH
def test_trace_runner(tmp_path, dtype):
    cases.case_trace_runner(tmp_path, DEV, dtype)


def test_modelhub_server():
    cases.case_modelhub(DEV)


def test_real_sizes():
    def say(s):
        print("real sizes:", s, flush=True)
    cases.case_real_sizes(DEV, say)
