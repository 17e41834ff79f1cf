"""Lipedra family on an MI355X: the HIP kernels, in exact fp32 mode and in
the bf16 serving mode, against the plain model in lipedra_oracle.py."""
import os
import sys

import pytest

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import lipedra_cases as cases  # noqa: E402

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
BOTH = pytest.mark.parametrize("dtype", ["fp32", "bf16"])


def test_kernel_group_is_loaded():
    from kukeon_amd import ops
    assert ops.mix_available(), "kukeon_amd/_C_mix.so is not built"


@BOTH
@pytest.mark.parametrize("name", sorted(cases.CONFIGS))
def test_whole_prompt(name, dtype):
    cases.case_whole(name, DEV, dtype)


@BOTH
def test_residual_after_every_layer(dtype):
    cases.case_layers(DEV, dtype)


@BOTH
@pytest.mark.parametrize("name", ["mixed", "gqa"])
def test_prefill_against_token_by_token(name, dtype):
    cases.case_prefill_vs_decode(name, DEV, dtype)


@BOTH
@pytest.mark.parametrize("sizes", [(2,), (3, 2, 7), (16, 1, 5), (2, 1)])
def test_portions(sizes, dtype):
    cases.case_portions("mixed", DEV, dtype, sizes)


@BOTH
def test_portions_long_taps(dtype):
    cases.case_portions("gqa", DEV, dtype, (2, 3))


@BOTH
@pytest.mark.parametrize("name", ["mixed", "odd", "narrow"])
def test_unequal_batch(name, dtype):
    cases.case_batch(name, DEV, dtype)


@BOTH
def test_long_prompts_and_tile_edges(dtype):
    cases.case_tiles(DEV, dtype)


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
@pytest.mark.parametrize("graphs", [False, True])
def test_greedy_generation(dtype, graphs):
    cases.case_greedy(DEV, dtype, graphs=graphs)


def test_multi_turn_and_eviction():
    cases.case_multi_turn(DEV, "fp32")


@BOTH
def test_norm_op(dtype):
    cases.case_op_norm(DEV, dtype)


@BOTH
def test_glu_op(dtype):
    cases.case_op_glu(DEV, dtype)


@BOTH
@pytest.mark.parametrize("taps", [1, 2, 4])
def test_conv_rotary_append_op(taps, dtype):
    cases.case_op_conv_rope(DEV, dtype, taps=taps)
    cases.case_op_conv_rope(DEV, dtype, taps=taps, aligned=True)


@BOTH
@pytest.mark.parametrize("taps", [2, 3, 4])
def test_conv_long_portions(taps, dtype):
    """Portions long enough for the sliding-window form, a second sequence
    starting inside a thread's run of rows, then a continuation."""
    cases.case_op_conv_rope(DEV, dtype, taps=taps, aligned=True,
                            cuts=((2101, 3), (150, 70)), pages=1200)


@BOTH
def test_attention_far_keys_and_page_borders(dtype):
    cases.case_op_attention_far(DEV, dtype, ctx=700, BS=16)
    cases.case_op_attention_far(DEV, dtype, ctx=70, BS=4)
    # sizes of the matrix-core and split kernels; groups of 2, 1 and 4
    cases.case_op_attention_far(DEV, dtype, ctx=330, BS=16, H=4, G=2,
                                dim=16, vdim=32)
    cases.case_op_attention_far(DEV, dtype, ctx=200, BS=8, H=2, G=2,
                                dim=32, vdim=64)
    cases.case_op_attention_far(DEV, dtype, ctx=130, BS=16, H=8, G=2,
                                dim=64, vdim=128)
    cases.case_op_attention_far(DEV, dtype, ctx=100, BS=16, H=3, G=1,
                                dim=64, vdim=64)
    cases.case_op_attention_far(DEV, dtype, ctx=90, BS=32, H=2, G=1,
                                dim=128, vdim=128)
    cases.case_op_attention_far(DEV, dtype, ctx=75, BS=16, H=16, G=2,
                                dim=32, vdim=32)
