"""The table tests of `test_jit.py` (the reference's nn / numpy / lax-linalg / random tables replayed through traced
programs) run again with the hip backend in place of the CPU checker: same programs, same expected values, every
kernel and routine on the GPU (Wasm-faithful numerics, so the tables' own tolerances apply unchanged)."""
import pytest

import test_jit as T
from gpu_util import WARM_ONLY, backend

pytestmark = pytest.mark.gpu

# Tests of test_jit.py that only look at program structure (no backend involved) are left out.
TABLE_TESTS = [
    "test_elementwise_chain_is_one_kernel", "test_reduction_fuses_unary_and_literal_epilogue",
    "test_reduction_epilogue_stops_at_broadcasting_operand_and_second_use", "test_two_reductions_never_share_a_kernel",
    "test_dot_operand_with_reuse_is_materialised", "test_row_softmax_argmax_program_is_four_row_reductions_plus_one_constant",
    "test_max_args_splits_wide_expressions", "test_softmax_table", "test_gelu_tables", "test_tanh_matches_libm_and_saturates",
    "test_standardize_table", "test_attention_tables", "test_causal_attention_closed_form", "test_matmul_integer_cases_are_exact",
    "test_einsum_layouts_of_attention", "test_gpt2_block_program_structure_and_values_f32",
    "test_routine_outputs_and_operands_are_dispatch_boundaries", "test_solve_is_lu_plus_two_triangular_solves",
    "test_triangular_solve_variants_match_the_reference_tables", "test_cholesky_upper_eigh_and_fft_along_an_axis",
    "test_eigh_svd_and_diagonal_reference_tables", "test_random_bits_and_split_match_jax", "test_uniform_and_normal_distributions",
    "test_gather_take_and_take_along_axis", "test_concatenate_stack_and_split",
    "test_output_returned_twice_carries_two_references", "test_input_returned_twice_beside_a_result",
    "test_count_nonzero_any_all_tables", "test_prod_ptp_var_std_average_tables", "test_cumsum_cumprod_tables_and_the_two_stage_scan",
    "test_diff_tables", "test_flip_rot90_roll_tables", "test_sign_and_float_class_predicates", "test_trapezoid_tables",
    "test_matvec_vecmat_tensordot_outer_inner_tables", "test_min_max_fmin_fmax_abs_signbit_tables", "test_division_family_tables",
    "test_exponential_and_power_tables", "test_trigonometric_and_hyperbolic_tables", "test_nan_to_num_rounding_and_copysign_tables",
    "test_logical_and_bitwise_tables", "test_creation_tables", "test_diag_family_tables",
    "test_where_select_equality_and_membership_tables", "test_pad_and_split_family_tables", "test_joins_repeats_and_reshapes_tables",
    "test_polynomial_convolution_and_statistics_tables", "test_unwrap_tables", "test_reductions_views_dot_and_sort_tables",
    "test_activation_tables", "test_top_k_tables", "test_numpy_linalg_tables", "test_numpy_fft_tables", "test_random_distribution_tables",
    "test_einsum_tables", "test_dtype_promotion_and_half_double_tables", "test_cholesky_lu_eigvalsh_and_argreduce_tables",
    "test_frexp_ldexp_and_flips", "test_jit_cases_of_the_tracing_suite", "test_array_suite_tables",
]


_shared = None


def _hip():
    """One backend object for all table tests (each test releases its own slots, so its leak check still holds)."""
    global _shared
    if _shared is None:
        from jaxjs_hip.backend import HipBackend
        backend()  # device up
        _shared = HipBackend(numerics="wasm")
    return _shared


class _CompileOnly(T.OracleBackend):
    """Warm-up stand-in: compiles what the hip backend would run into the on-disk cache, computes on the CPU checker."""

    def prepareKernelSync(self, kernel):
        from jaxjs_hip.kernelgen import generate
        from jaxjs_hip.runtime import compile_source
        for src in generate(kernel, "wasm").sources:
            compile_source(src)
        return super().prepareKernelSync(kernel)

    def prepareRoutineSync(self, routine):
        from jaxjs_hip.routinegen import generateRoutine
        from jaxjs_hip.runtime import compile_source
        for src in generateRoutine(routine, "wasm").sources:
            compile_source(src)
        return super().prepareRoutineSync(routine)


@pytest.mark.parametrize("name", TABLE_TESTS)
def test_table_on_the_gpu(name, monkeypatch):
    monkeypatch.setattr(T, "OracleBackend", _CompileOnly if WARM_ONLY else (lambda *a, **kw: _hip()))
    getattr(T, name)()


# The reference's convolution tables (tests/test_conv.py) on the GPU, the same way.
CONV_TABLE_TESTS = [
    "test_1d_convolution_tables", "test_same_and_same_lower_padding", "test_2d_convolution_table", "test_transposed_convolution_table",
    "test_transposed_convolution_downstream_ops_and_integer_dtype", "test_zero_dimensional_grouped_and_conv_transpose_tables",
    "test_pooling_and_window_reductions",
]


@pytest.mark.parametrize("name", CONV_TABLE_TESTS)
def test_convolution_table_on_the_gpu(name, monkeypatch):
    import test_conv as C
    monkeypatch.setattr(C, "OracleBackend", _CompileOnly if WARM_ONLY else (lambda *a, **kw: _hip()))
    getattr(C, name)()


def test_transposed_1d_lowering_cases_on_the_gpu(monkeypatch):
    import test_conv as C
    monkeypatch.setattr(C, "OracleBackend", _CompileOnly if WARM_ONLY else (lambda *a, **kw: _hip()))
    for case in C.TRANSPOSED_1D:
        C.test_transposed_1d_convolution_lowering_matches_direct_loops(*case)
