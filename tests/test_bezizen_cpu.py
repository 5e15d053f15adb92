"""Bezizen family on the CPU path (reference ops, fp32) against the plain
model in bezizen_oracle.py: the engine's batching, paging, state slots and
scheduler with this family, and every mechanism by itself."""
import os
import sys

import pytest

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import bezizen_cases as cases  # noqa: E402

DEV, DT = "cpu", "fp32"


@pytest.mark.parametrize("name", sorted(set(cases.CONFIGS) - {"tiles"}))
def test_whole_prompt(name):
    cases.case_whole(name, DEV, DT)


def test_whole_prompt_wide_heads():
    cases.case_whole("tiles", DEV, DT, n=19)


def test_residual_after_every_layer():
    cases.case_layers(DEV, DT)


@pytest.mark.parametrize("name", ["hybrid", "plain", "one_stream"])
def test_prefill_against_token_by_token(name):
    cases.case_prefill_vs_decode(name, DEV, DT)


@pytest.mark.parametrize("sizes", [(2,), (3, 2, 7), (16, 1, 5)])
def test_portions(sizes):
    cases.case_portions("hybrid", DEV, DT, sizes)


def test_unequal_batch():
    cases.case_batch("hybrid", DEV, DT)
    cases.case_batch("plain", DEV, DT)


def test_pages_and_slots_reused():
    cases.case_reuse(DEV, DT)


def test_first_tokens():
    cases.case_first_tokens(DEV, DT)


def test_long_decode():
    cases.case_long_decode(DEV, DT)


def test_long_window():
    cases.case_long_window(DEV, DT)


def test_long_portions_sort_rows_by_expert():
    cases.case_sorted_experts(DEV, DT)


@pytest.mark.parametrize("decode", [False, True])
def test_window_edges(decode):
    cases.case_window_edges(DEV, DT, decode)


def test_state_is_carried():
    cases.case_state_carry(DEV, DT)


def test_router():
    cases.case_router(DEV, DT)


def test_greedy_generation():
    cases.case_generate(DEV, DT)


def test_multi_turn_and_eviction():
    cases.case_multi_turn(DEV, DT)


def test_op_streams():
    cases.case_op_streams(DEV, DT)


def test_op_shift():
    cases.case_op_shift(DEV, DT)


@pytest.mark.parametrize("mode", [0, 1])
def test_op_scan(mode):
    cases.case_op_scan(DEV, DT, mode=mode)


def test_op_router():
    cases.case_op_router(DEV)


def test_presets_and_registry():
    from kukeon_amd.models import registry
    cfg = registry.preset("tiny-bezizen")
    assert cfg.family == "bezizen" and registry.family_of(cfg) == "bezizen"
    model = registry.build_model(cfg, "cpu", dtype="fp32")
    assert len(model.layers) == cfg.num_layers
    assert registry.OP_GROUPS["bezizen"] == ("strm",)
    big = registry.preset("bezizen-8b-like")
    assert big.width == 4096 and big.num_layers == 32


def test_config_rejects_unknown_kinds():
    cfg = cases.CONFIGS["hybrid"]()
    cfg["layers"][0]["type"] = "other"
    with pytest.raises(ValueError):
        cases.BezizenConfig.from_json(cfg)
    cfg = cases.CONFIGS["hybrid"]()
    cfg["layers"][0]["mlp"]["kind"] = "dense"
    with pytest.raises(ValueError):
        cases.BezizenConfig.from_json(cfg)


def test_checkpoint_folder(tmp_path):
    cases.case_registry(tmp_path, DEV, DT)


def test_trace_runner(tmp_path):
    cases.case_trace_runner(tmp_path, DEV, DT)


def test_modelhub_server():
    cases.case_modelhub(DEV)


def test_bench_stack_shapes():
    """The throughput stack at several sizes builds its configuration (no
    weights): every layer has ff active rows, the last layer of a short stack
    is a parallel one."""
    from kukeon_amd.models.bezizen import bezizen_bench, tensor_shapes
    for W, hq, hk, ff, nl in ((2048, 16, 4, 8192, 4), (8192, 64, 8, 28672, 2)):
        cfg = bezizen_bench(width=W, layers=nl, heads=hq, kv_heads=hk, ff=ff,
                            vocab=1000, max_positions=64)
        assert cfg.layers[-1].type == "parallel"
        for L in cfg.layers:
            f = L.mlp
            assert abs(f.shared_ff + f.top * f.ff - ff) <= 16
        assert "l0.hc1.mix" in tensor_shapes(cfg)
