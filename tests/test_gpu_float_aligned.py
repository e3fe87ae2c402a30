"""Every operand only float-aligned: whole parity tests run again with each device buffer 1, 2 or 3
floats into its allocation.

The library takes pointers with no more than a float's alignment (views into a larger buffer, as
custos' `Buffer` slices are).  Its kernels read and write 16-byte vectors wherever they can, so
each of them has a way of dealing with a base, a row pitch or a tail that is off that grid; the
tests here send the operands of the ordinary parity tests through those ways, with the same bars:
the test functions are the ones of the other files, called with the facade switched to handing
out misplaced buffers.
"""
import sys

import pytest

import test_gpu_fusion as fusion
import test_gpu_parity as parity
import test_gpu_random_shapes as shapes
import test_gpu_special_values as special

pytestmark = pytest.mark.gpu


@pytest.fixture
def misplaced(hip):
    hip.operands_off_the_vector_grid(True)
    yield
    hip.operands_off_the_vector_grid(False)


def cases():
    out = []

    def add(fn, **kw):
        tag = ",".join("x".join(map(str, v)) if isinstance(v, tuple) else str(v) for v in kw.values())
        out.append(pytest.param(fn, kw, id=fn.__name__[5:60] + ("[" + tag.replace(" ", "_")[:40] + "]" if tag else "")))

    for fn in (shapes.test_random_gemm_shapes, shapes.test_random_linear_fwd_shapes, shapes.test_random_matrix_op_shapes,
               parity.test_gemm_split_k_and_large_tiles, parity.test_gemm_spread_tail, parity.test_gemm_skinny_kernels,
               parity.test_gemm_rows_narrow_kernel, parity.test_gemm_tall_kernel,
               parity.test_gemm_transposed_tall_operand_with_narrow_b, parity.test_gemm_narrow_b_stored_transposed,
               parity.test_gemm_with_a_row_vector_runs_as_matrix_times_column, parity.test_gemm_few_rows_times_a_large_matrix,
               parity.test_gemm_small_tile, parity.test_gemm_eight_wave_tile,
               parity.test_sgemm_relu_mask_equals_gemm_then_relu_grad, parity.test_gemm_grad_matches_oracle,
               parity.test_linear_fwd_fused_equals_gemm_bias_relu, parity.test_linear_grad_one_launch_equals_the_three_ops,
               parity.test_max_is_bit_exact_with_injected_ties_and_negatives, parity.test_max_grads_tie_rules,
               parity.test_broadcast_grads_are_bit_exact, parity.test_row_op_and_bias_grad, parity.test_cce_and_onehot,
               parity.test_tanh_sigmoid_diagflat_onehot_grad, parity.test_relu_mask_as_bits_equals_the_float_mask,
               special.test_softmax_gradient_and_losses_on_special_operands,
               special.test_set_semantics_of_the_other_ops_with_an_output_full_of_nan):
        add(fn)
    for shape in parity.GEMM_SHAPES:
        for form in ("gemm", "gemmT", "Tgemm"):
            add(parity.test_gemm_forms, shape=shape, form=form)
    for shape in parity.RED_SHAPES:
        add(parity.test_reductions, shape=shape)
    for shape in parity.SOFTMAX_SHAPES:
        add(parity.test_softmax_forward_backward, shape=shape)
    for shape in parity.TR_SHAPES:
        add(parity.test_transpose_bit_exact, shape=shape)
    for n in (1, 3, 4, 5, 1023, 4096, 100003, 1 << 20):
        add(parity.test_elementwise_ops, n=n)
    for shape in [(1, 1), (3, 5), (64, 10), (257, 129), (4096, 33), (5, 70000), (2000, 2048), (5000, 1), (3000, 7), (1, 5000),
                  (20000, 2), (1500, 64), (40, 4099)]:
        for kind in ("row_op", "col_op"):
            add(parity.test_broadcast_ops_with_op_code, shape=shape, kind=kind)
    for n in (1, 5, 1024, 4099, 1 << 20, 3000001):
        add(parity.test_fused_mse_against_the_op_chain, n=n)
    for shape in [(1, 1), (7, 3), (8192, 10), (300, 1000), (5, 70001), (3000, 100), (70000, 7), (9000, 512), (1100, 4099)]:
        add(parity.test_fused_softmax_cross_entropy_against_the_op_chain, shape=shape)
    for shape in special.SHAPES:
        add(special.test_nan_and_inf_land_where_the_reference_puts_them, shape=shape)
        add(special.test_subnormals_are_not_flushed, shape=shape)
    for shape in special.SET_SHAPES:
        add(special.test_beta_zero_overwrites_whatever_the_output_held, shape=shape)
    for name in fusion.PROGRAMS:
        add(fusion.test_program_equals_the_ops_one_by_one, name=name)
    return out


@pytest.mark.parametrize("fn,kw", cases())
def test_with_every_operand_off_the_vector_grid(hip, orc, misplaced, fn, kw):
    print("misplaced operands:", fn.__name__, kw, flush=True)
    sys.stdout.flush()
    names = fn.__code__.co_varnames[:fn.__code__.co_argcount]
    fixtures = {"hip": hip, "orc": orc}
    fn(**{k: fixtures[k] for k in names if k in fixtures}, **kw)
