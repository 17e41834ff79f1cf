"""Rasesun family on the CPU path (fp32 reference ops through the engine)
against the plain model in rasesun_oracle.py."""
import os
import sys

import pytest

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import rasesun_cases as cases  # noqa: E402

DEV, DT = "cpu", "fp32"


@pytest.mark.parametrize("name", sorted(cases.CONFIGS))
def test_whole_prompt(name):
    cases.case_whole(name, DEV, DT)


def test_residual_after_every_layer_run():
    cases.case_layers(DEV, DT)


@pytest.mark.parametrize("name", ["hybrid", "looped"])
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


def test_long_portions_sort_rows_by_expert():
    cases.case_grouped_experts(DEV, DT)


def test_long_portions():
    cases.case_long_portions(DEV, DT)


def test_greedy_generation():
    cases.case_greedy(DEV, DT)


def test_checkpoint_folder(tmp_path):
    cases.case_registry(tmp_path, DEV, DT)


def test_multi_turn_and_eviction():
    cases.case_multi_turn(DEV, DT)


def test_modelhub_serves_the_family():
    cases.case_modelhub(DEV)


def test_presets_build_through_the_registry():
    from kukeon_amd.models import registry
    assert "rasesun-8b-like" in registry.preset_names()
    cfg = registry.preset("tiny-rasesun")
    model = registry.build_model(cfg, "cpu", dtype="fp32")
    assert model.family == "rasesun" and len(model.runs) == 4
    kinds = [type(L.mixer).__name__ for L in model.layers]
    assert kinds.count("LatentAttention") == 1


def test_trace_runner(tmp_path):
    cases.case_trace_runner(tmp_path, DEV, DT)


def test_op_sandwich_norm():
    cases.case_op_sandwich_norm(DEV, DT)


@pytest.mark.parametrize("taps", [1, 2, 4])
def test_op_conv(taps):
    cases.case_op_conv(DEV, DT, taps=taps)


def test_op_scan():
    cases.case_op_scan(DEV, DT)
    cases.case_op_scan(DEV, DT, H=4, P=3, N=40, G=1, cuts=(1, 1, 20, 2))


def test_op_gated_norm():
    cases.case_op_gated_norm(DEV, DT)


def test_op_activations():
    cases.case_op_activations(DEV, DT)


@pytest.mark.parametrize("top", [1, 2, 3])
def test_op_table_moe(top):
    cases.case_op_table_moe(DEV, DT, top=top)


def test_op_latent_append():
    cases.case_op_latent_append(DEV, DT)


def test_op_latent_attention():
    cases.case_op_latent_attention(DEV, DT, ctx=120, window=40)


def test_config_rejects_unknown_parts():
    from kukeon_amd.models.rasesun import RasesunConfig
    cfg = cases.CONFIGS["hybrid"]()
    cfg["layers"][0]["type"] = "other"
    with pytest.raises(ValueError):
        RasesunConfig.from_json(cfg)
    cfg = cases.CONFIGS["hybrid"]()
    cfg["layers"][0]["mlp"]["kind"] = "other"
    with pytest.raises(ValueError):
        RasesunConfig.from_json(cfg)


def test_layer_runs_follow_the_loop():
    from kukeon_amd.models.rasesun import RasesunConfig
    c = RasesunConfig.from_json(cases.CONFIGS["hybrid"]())
    assert c.runs() == [0, 1, 2, 1, 2, 1, 2, 3]
    c = RasesunConfig.from_json(cases.CONFIGS["wide"]())
    assert c.runs() == [0, 1]
