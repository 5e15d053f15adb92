"""Dumovik family on the CPU path (fp32 reference ops through the engine)
against the plain model in dumovik_oracle.py."""
import os
import sys

import pytest

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import dumovik_cases as cases  # noqa: E402

DEV, DT = "cpu", "fp32"


@pytest.mark.parametrize("name", sorted(cases.CONFIGS))
def test_whole_prompt(name):
    cases.case_whole(name, DEV, DT)


def test_residual_after_every_layer():
    cases.case_layers(DEV, DT)


@pytest.mark.parametrize("name", ["hybrid", "plain"])
def test_prefill_against_token_by_token(name):
    cases.case_prefill_vs_decode(name, DEV, DT)


@pytest.mark.parametrize("sizes", [(2,), (3, 2, 7), (16, 1, 5)])
def test_portions(sizes):
    cases.case_portions("hybrid", DEV, DT, sizes)


def test_unequal_batch():
    cases.case_batch("hybrid", DEV, DT)


def test_pages_and_slots_reused():
    cases.case_reuse(DEV, DT)


def test_first_tokens():
    cases.case_first_tokens(DEV, DT)


def test_long_decode():
    cases.case_long_decode(DEV, DT)


def test_long_chunk():
    cases.case_long_chunk(DEV, DT)


def test_long_portions():
    cases.case_long_portions(DEV, DT)


def test_long_portions_sort_rows_by_expert():
    cases.case_sorted_experts(DEV, DT)


def test_greedy_generation():
    cases.case_generate(DEV, DT)


def test_multi_turn_and_eviction():
    cases.case_multi_turn(DEV, DT)


def test_modelhub_serves_the_family():
    cases.case_modelhub(DEV)


def test_checkpoint_folder(tmp_path):
    cases.case_registry(tmp_path, DEV, DT)


def test_trace_runner(tmp_path):
    cases.case_trace_runner(tmp_path, DEV, DT)


@pytest.mark.parametrize("decode", [False, True])
def test_chunk_edges(decode):
    cases.case_chunk_edges(DEV, DT, decode)


@pytest.mark.parametrize("decode", [False, True])
def test_far_key_in_the_latent_cache(decode):
    cases.case_far_latent_key(DEV, DT, decode)


def test_state_is_carried():
    cases.case_state_carry(DEV, DT)


def test_router():
    cases.case_router(DEV, DT)


def test_op_layer_norm():
    cases.case_op_layer_norm(DEV, DT)


def test_op_gated():
    cases.case_op_gated(DEV, DT)


def test_op_scan():
    cases.case_op_scan(DEV, DT)
    cases.case_op_scan(DEV, DT, H=2, d=40, dv=3, cuts=(1, 1, 20, 2))


def test_op_router():
    cases.case_op_router(DEV, DT)


def test_presets_build_through_the_registry():
    from kukeon_amd.models import registry
    assert "dumovik-8b-like" in registry.preset_names()
    cfg = registry.preset("tiny-dumovik")
    model = registry.build_model(cfg, "cpu", dtype="fp32")
    assert model.family == "dumovik" and len(model.layers) == 8
    kinds = [type(L.mixer).__name__ for L in model.layers]
    assert kinds.count("LightningMixer") == 4
    assert kinds.count("ChunkedAttention") == 2
    assert model.layers[4].kv_layer == 0


def test_config_rejects_unknown_parts():
    from kukeon_amd.models.dumovik import DumovikConfig, DumovikModel
    cfg = cases.CONFIGS["hybrid"]()
    cfg["layers"][0]["type"] = "other"
    with pytest.raises(ValueError):
        DumovikConfig.from_json(cfg)
    cfg = cases.CONFIGS["hybrid"]()
    cfg["layers"][0]["mlp"]["kind"] = "other"
    with pytest.raises(ValueError):
        DumovikConfig.from_json(cfg)
    # keys can only come from an earlier layer that has its own
    cfg = cases.CONFIGS["hybrid"]()
    cfg["layers"][3]["mixer"]["kv_from"] = 2
    with pytest.raises(ValueError):
        DumovikModel(DumovikConfig.from_json(cfg), device="cpu",
                     dtype="fp32")
