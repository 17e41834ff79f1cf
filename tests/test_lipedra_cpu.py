"""Lipedra family on the CPU path (engine + fp32 reference ops) against the
plain model in lipedra_oracle.py."""
import os
import sys

import pytest

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import lipedra_cases as cases  # noqa: E402

DEV, DT = "cpu", "fp32"


@pytest.mark.parametrize("name", sorted(cases.CONFIGS))
def test_whole_prompt(name):
    cases.case_whole(name, DEV, DT)


def test_residual_after_every_layer():
    cases.case_layers(DEV, DT)


@pytest.mark.parametrize("name", ["mixed", "gqa"])
def test_prefill_against_token_by_token(name):
    cases.case_prefill_vs_decode(name, DEV, DT)


@pytest.mark.parametrize("sizes", [(2,), (3, 2, 7), (16, 1, 5), (2, 1)])
def test_portions(sizes):
    cases.case_portions("mixed", DEV, DT, sizes)


def test_portions_long_taps():
    cases.case_portions("gqa", DEV, DT, (2, 3))


@pytest.mark.parametrize("name", ["mixed", "odd", "narrow"])
def test_unequal_batch(name):
    cases.case_batch(name, DEV, DT)


def test_long_prompts_and_tile_edges():
    cases.case_tiles(DEV, DT)


def test_pages_and_slots_reused():
    cases.case_reuse(DEV, DT)


def test_first_tokens():
    cases.case_first_tokens(DEV, DT)


def test_long_decode():
    cases.case_long_decode(DEV, DT)


def test_greedy_generation():
    cases.case_greedy(DEV, DT)


def test_multi_turn_and_eviction():
    cases.case_multi_turn(DEV, DT)


def test_presets_and_registry():
    from kukeon_amd.models import registry
    assert "lipedra-8b-like" in registry.preset_names()
    cfg = registry.preset("tiny-lipedra")
    assert registry.family_of(cfg) == "lipedra"
    model = registry.build_model(cfg, "cpu", dtype="fp32")
    assert len(model.kv_specs()) == cfg.num_layers
    assert model.kv_specs()[2].share_from == 1
    assert registry.family_of(registry.preset("tiny-llama")) == "llama"


def test_norm_op():
    cases.case_op_norm(DEV, DT)


def test_glu_op():
    cases.case_op_glu(DEV, DT)


def test_angle_tables():
    cases.case_op_angles()


@pytest.mark.parametrize("taps", [1, 2, 4])
def test_conv_rotary_append_op(taps):
    cases.case_op_conv_rope(DEV, DT, taps=taps)
    cases.case_op_conv_rope(DEV, DT, taps=taps, aligned=True)


def test_attention_far_keys_and_page_borders():
    cases.case_op_attention_far(DEV, DT, ctx=150, BS=16)
    cases.case_op_attention_far(DEV, DT, ctx=70, BS=4)


def test_config_reader_rejects_unknown_parts():
    from kukeon_amd.models.lipedra import LipedraConfig
    c = cases.CONFIGS["mixed"]()
    c["layers"][0]["type"] = "something"
    with pytest.raises(ValueError):
        LipedraConfig.from_json(c)
    c = cases.CONFIGS["mixed"]()
    c["layers"][2]["mlp"]["kind"] = "other"
    with pytest.raises(ValueError):
        LipedraConfig.from_json(c)


def test_shared_cache_must_point_back():
    import torch
    from kukeon_amd.engine.kv_cache import LayerKVSpec, LayeredKVCache
    with pytest.raises(ValueError):
        LayeredKVCache([LayerKVSpec(1, 8, 4, share_from=1),
                        LayerKVSpec(1, 8, 4)], 4, 4, "cpu", torch.float32)
    kv = LayeredKVCache([LayerKVSpec(1, 8, 4), LayerKVSpec(1, 8, 4, 0)],
                        4, 4, "cpu", torch.float32)
    assert kv.k[1] is kv.k[0] and kv.v[1] is kv.v[0]


def test_checkpoint_roundtrip(tmp_path):
    """Weights written as a safetensors file load through the registry."""
    import json
    import struct
    import torch
    from kukeon_amd.models.registry import load_checkpoint
    cfg = cases.CONFIGS["odd"]()
    W = cases.weights(cfg, 11)
    header, blobs, at = {}, [], 0
    for k, t in W.items():
        raw = t.contiguous().view(torch.int16).numpy().tobytes()
        header[k] = {"dtype": "BF16", "shape": list(t.shape),
                     "data_offsets": [at, at + len(raw)]}
        blobs.append(raw)
        at += len(raw)
    hj = json.dumps(header).encode()
    with open(tmp_path / "model.safetensors", "wb") as f:
        f.write(struct.pack("<Q", len(hj)) + hj + b"".join(blobs))
    with open(tmp_path / "config.json", "w") as f:
        json.dump(cfg, f)
    mcfg, model = load_checkpoint(str(tmp_path), device="cpu", dtype="fp32")
    assert mcfg.num_layers == 2 and mcfg.layers[1].mixer.conv == 5
    assert torch.equal(model.lm_head.cpu(), W["head"].float())
