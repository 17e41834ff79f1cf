"""Rasesun family on an MI355X: the HIP kernels, in exact fp32 mode and in
the bf16 serving mode, against the plain model in rasesun_oracle.py."""
import os
import sys

import pytest

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import rasesun_cases as cases  # noqa: E402

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
BOTH = pytest.mark.parametrize("dtype", ["fp32", "bf16"])


def test_kernel_group_is_loaded():
    from kukeon_amd import ops
    assert ops.recur_available(), "kukeon_amd/_C_recur.so is not built"


@BOTH
def test_op_sandwich_norm(dtype):
    cases.case_op_sandwich_norm(DEV, dtype)


@BOTH
@pytest.mark.parametrize("taps", [1, 2, 4])
def test_op_conv(taps, dtype):
    cases.case_op_conv(DEV, dtype, taps=taps)
    # eight channels per thread
    cases.case_op_conv(DEV, dtype, taps=taps, C=40, col0=8, ld=64)
    cases.case_op_conv(DEV, dtype, taps=taps, C=2560, col0=16, ld=2600)


@BOTH
def test_op_scan(dtype):
    cases.case_op_scan(DEV, dtype)
    cases.case_op_scan(DEV, dtype, H=4, P=3, N=40, G=1, cuts=(1, 1, 20, 2))
    # state rows over 8 lanes, a full wave of columns, more than one tile
    cases.case_op_scan(DEV, dtype, H=2, P=64, N=128, G=2, cuts=(37, 1, 3))
    # 32 rows per thread
    cases.case_op_scan(DEV, dtype, H=1, P=128, N=200, G=1, cuts=(5, 18))


@BOTH
def test_op_gated_norm(dtype):
    cases.case_op_gated_norm(DEV, dtype)


@BOTH
def test_op_activations(dtype):
    cases.case_op_activations(DEV, dtype)


@BOTH
@pytest.mark.parametrize("top", [1, 2, 3])
def test_op_table_moe(top, dtype):
    cases.case_op_table_moe(DEV, dtype, top=top)
    cases.case_op_table_moe(DEV, dtype, E=7, top=top, W=136, ff=70, V=19)
    # whole 16-byte chunks both ways: the expert-major kernels
    cases.case_op_table_moe(DEV, dtype, E=7, top=top, W=136, ff=72, V=19)
    # whole 128-element blocks: the matrix-core kernels in bf16; an expert
    # with more pairs than one tile holds, row counts that end inside a tile
    cases.case_op_table_moe(DEV, dtype, E=3, top=top, W=256, ff=136,
                            V=19, rows=45)
    cases.case_op_table_moe(DEV, dtype, E=6, top=top, W=128, ff=384, V=8,
                            rows=5)
    # rows longer than one register segment
    cases.case_op_table_moe(DEV, dtype, E=4, top=top, W=8200, ff=16, V=9)


@BOTH
def test_op_latent_append(dtype):
    cases.case_op_latent_append(DEV, dtype)


@BOTH
def test_op_latent_attention(dtype):
    cases.case_op_latent_attention(DEV, dtype)
    # a window longer than one pass over the keys, a latent wider than a
    # workgroup
    cases.case_op_latent_attention(DEV, dtype, ctx=700, BS=16, H=3, R=300,
                                   dr=8, window=600)
    # whole 16-byte chunks: the vector form, one and several key chunks
    cases.case_op_latent_attention(DEV, dtype, ctx=300, BS=16, H=5, R=64,
                                   dr=8, window=40)
    cases.case_op_latent_attention(DEV, dtype, ctx=700, BS=8, H=9, R=512,
                                   dr=64, window=600)
    # sizes of the matrix-core form; two head tiles, the second partly filled
    cases.case_op_latent_attention(DEV, dtype, ctx=600, BS=16, H=20, R=128,
                                   dr=32, window=100)
    cases.case_op_latent_attention(DEV, dtype, ctx=520, BS=4, H=3, R=256,
                                   dr=64, window=33)


@BOTH
@pytest.mark.parametrize("name", sorted(cases.CONFIGS))
def test_whole_prompt(name, dtype):
    cases.case_whole(name, DEV, dtype)


@BOTH
def test_residual_after_every_layer_run(dtype):
    cases.case_layers(DEV, dtype)


@BOTH
@pytest.mark.parametrize("name", ["hybrid", "looped"])
def test_prefill_against_token_by_token(name, dtype):
    cases.case_prefill_vs_decode(name, DEV, dtype)


@BOTH
@pytest.mark.parametrize("sizes", [(2,), (3, 2, 7), (16, 1, 5), (2, 1)])
def test_portions(sizes, dtype):
    cases.case_portions("hybrid", DEV, dtype, sizes)


@BOTH
@pytest.mark.parametrize("name", ["hybrid", "wide", "looped", "aligned"])
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
def test_window_longer_than_a_key_chunk(dtype):
    cases.case_window_chunks(DEV, dtype)


@BOTH
def test_long_portions_on_the_matrix_cores(dtype):
    cases.case_long_portions(DEV, dtype)


@BOTH
def test_long_portions_sort_rows_by_expert(dtype):
    cases.case_grouped_experts(DEV, dtype)


@BOTH
@pytest.mark.parametrize("graphs", [False, True])
def test_greedy_generation(dtype, graphs):
    cases.case_greedy(DEV, dtype, graphs=graphs)


def test_multi_turn_and_eviction():
    cases.case_multi_turn(DEV, "fp32")


@BOTH
def test_checkpoint_folder(tmp_path, dtype):
    cases.case_registry(tmp_path, DEV, dtype)


@BOTH
def test_trace_runner(tmp_path, dtype):
    cases.case_trace_runner(tmp_path, DEV, dtype)
