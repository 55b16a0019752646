"""Kernel forms that the library only chooses for large arrays, or that a knob switches off,
run on the ordinary suites' small inputs in child processes:
  CUMO_HIP_NT=1            every kernel's non-temporal form, and with it the lean two-dimensional
                           row kernel (two rows per lane, operand mode chosen per block), the
                           non-temporal gather / scatter, mulsum, scans and fused rows;
  CUMO_HIP_RED_POLL=0      split reductions with tickets instead of the hand-over words;
  CUMO_HIP_SCAN_CHAIN=0    long runs scanned by the three launches instead of the one pass;
  CUMO_HIP_SCAN_CHAIN_WAVES=4 the one pass over one long run by blocks of four waves at every size (4097 tiles: the
                           second supergroup);
  CUMO_HIP_SCAN_COLS_CHAIN=0  long runs across memory scanned in two passes over segments;
  CUMO_HIP_SCAN_KEEP_WORDS=0  the one-pass scans with their words from the pool, cleared by a kernel
                           before each launch (what a stream under capture gets);
  CUMO_HIP_EW_LEAN_ROWS=0  (with CUMO_HIP_NT=1) the general row kernel in its non-temporal forms;
  CUMO_HIP_BIT_VEC_GRID=1  (with CUMO_HIP_NT=1) the Bit vector kernels with one block per compute unit, whose lanes
                           then loop over the result's vectors (what an array beyond 2^37 bits gets) and carry a
                           vector's row and column from turn to turn.
Each child runs the same parity tests against the oracle as the main suite does."""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

ELEMENTWISE = ["tests/test_gpu_elementwise.py::test_float_binary_over_views", "tests/test_gpu_elementwise.py::test_broadcast_shapes",
               "tests/test_gpu_elementwise.py::test_three_dimensions_with_an_operand_repeating_along_one",
               "tests/test_gpu_elementwise.py::test_inputs_that_start_off_a_16_byte_boundary",
               "tests/test_gpu_elementwise.py::test_rows_that_run_backwards_in_memory",
               "tests/test_gpu_elementwise.py::test_many_dims_and_permuted_views", "tests/test_gpu_elementwise.py::test_sizes_and_tails",
               "tests/test_gpu_elementwise.py::test_unary_and_rounding", "tests/test_gpu_elementwise.py::test_int32_arithmetic",
               "tests/test_gpu_elementwise.py::test_int32_error_flags", "tests/test_gpu_elementwise.py::test_casts_and_copies",
               "tests/test_gpu_elementwise.py::test_compare_into_bit", "tests/test_gpu_elementwise.py::test_nmath"]
REDUCE = ["tests/test_gpu_reduce.py::test_float_reductions_every_axis", "tests/test_gpu_reduce.py::test_random_float_sums",
          "tests/test_gpu_reduce.py::test_nan_rules", "tests/test_gpu_reduce.py::test_int32_reductions",
          "tests/test_gpu_reduce.py::test_min_max_keep_the_zero_that_came_first"]
ADJACENT = ["tests/test_gpu_adjacent.py::test_clip_parity_over_views", "tests/test_gpu_adjacent.py::test_float_pow_parity",
            "tests/test_gpu_adjacent.py::test_cumsum_cumprod_parity", "tests/test_gpu_adjacent.py::test_cum_along_contiguous_runs_of_whole_chunks",
            "tests/test_gpu_adjacent.py::test_one_long_run_in_one_pass",
            "tests/test_gpu_adjacent.py::test_cum_along_columns_of_tall_wide_and_stacked_arrays", "tests/test_gpu_adjacent.py::test_mulsum_parity"]
OTHERS = ["tests/test_gpu_index.py::test_gather_and_scatter_between_view_and_buffer", "tests/test_gpu_index.py::test_getitem_with_index_arrays",
          "tests/test_gpu_index.py::test_setitem_with_index_arrays_and_slices", "tests/test_gpu_fused.py", "tests/test_gpu_configs.py"]


def run_child(env_extra, picked):
    env = dict(os.environ, **env_extra)
    p = subprocess.run([sys.executable, "-m", "pytest", "-x", "-q", "-m", "gpu", "-p", "no:cacheprovider", "--timeout", "120",
                        "--timeout-method", "thread"] + picked, cwd=ROOT, env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=900)
    tail = "\n".join(p.stdout.strip().splitlines()[-15:])
    assert p.returncode == 0, tail
    assert " passed" in tail and "failed" not in tail, tail


def test_suites_with_the_non_temporal_forms_forced():
    run_child({"CUMO_HIP_NT": "1"}, ELEMENTWISE + REDUCE + ADJACENT + OTHERS)


def test_row_kernels_without_the_lean_form():
    run_child({"CUMO_HIP_NT": "1", "CUMO_HIP_EW_LEAN_ROWS": "0"}, ELEMENTWISE[:5])


def test_reductions_with_tickets():
    run_child({"CUMO_HIP_RED_POLL": "0"}, REDUCE)


def test_long_runs_scanned_by_three_launches():
    run_child({"CUMO_HIP_SCAN_CHAIN": "0", "CUMO_HIP_SCAN_COLS_CHAIN": "0"},
              ["tests/test_gpu_adjacent.py::test_one_long_run_in_one_pass", "tests/test_gpu_adjacent.py::test_cumsum_cumprod_parity",
               "tests/test_gpu_adjacent.py::test_long_columns_in_one_pass"])


def test_one_pass_scans_with_cleared_words_from_the_pool():
    run_child({"CUMO_HIP_SCAN_KEEP_WORDS": "0"},
              ["tests/test_gpu_adjacent.py::test_one_long_run_in_one_pass", "tests/test_gpu_adjacent.py::test_long_columns_in_one_pass"])


def test_one_long_run_by_blocks_of_four_waves():
    run_child({"CUMO_HIP_SCAN_CHAIN_WAVES": "4"}, ["tests/test_gpu_adjacent.py::test_one_long_run_in_one_pass"])


def test_bit_vector_kernels_with_lanes_that_loop():
    run_child({"CUMO_HIP_BIT_VEC_GRID": "1", "CUMO_HIP_NT": "1"},
              ["tests/test_gpu_bit.py::test_rows_of_bits_in_views_word_by_word", "tests/test_gpu_bit.py::test_long_runs_of_bits_by_whole_vectors",
               "tests/test_gpu_bit.py::test_windows_of_a_large_matrix_into_a_fresh_result", "tests/test_gpu_bit.py::test_long_arrays_and_views",
               "tests/test_gpu_bit.py::test_all_any_along_word_aligned_rows"])


def test_table_operators_with_blocks_that_take_many_tiles():
    """Operators that fill tables in LDS run a capped grid whose blocks take a tile after the other: with two blocks every
    block loops wherever a launch has three tiles or more."""
    run_child({"CUMO_HIP_EW_TABLE_BLOCKS": "2"},
              ["tests/test_gpu_nmath_vectors.py", "tests/test_gpu_elementwise.py::test_nmath",
               "tests/test_gpu_elementwise.py::test_dfloat_power_of_arrays_with_every_kind_of_argument",
               "tests/test_gpu_adjacent.py::test_float_pow_parity"])
