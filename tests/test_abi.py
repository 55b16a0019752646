"""The drop-in boundary, checked without a GPU: descriptor layouts match the
reference's structs byte for byte, the library loads, and every symbol that
the headers under include/ declare is exported."""
import ctypes as C
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADERS = sorted(os.path.join(ROOT, "include", n) for n in os.listdir(os.path.join(ROOT, "include")) if n.endswith(".h"))


def test_descriptor_layouts():
    # sizes stated beside the reference's definitions (ext/cumo/include/cumo/indexer.h:16-68)
    from cumo_amd import _lib
    assert C.sizeof(_lib.Indexer) == 216
    assert C.sizeof(_lib.IArray) == 104
    assert C.sizeof(_lib.BitIArray) == 112
    assert C.sizeof(_lib.IArrayStridx) == 104
    assert C.sizeof(_lib.BitIArrayStridx) == 112
    assert C.sizeof(_lib.ReductionArg) == 640
    assert _lib.Indexer.total_size.offset == 8
    assert _lib.Indexer.shape.offset == 16
    assert _lib.Indexer.index.offset == 112
    assert _lib.Indexer.raw_index.offset == 208
    assert _lib.IArray.step.offset == 8
    assert _lib.BitIArray.pos.offset == 8 and _lib.BitIArray.step.offset == 16
    assert _lib.ReductionArg.out.offset == 104
    assert _lib.ReductionArg.in_indexer.offset == 208
    assert _lib.ReductionArg.out_indexer.offset == 424


def test_header_layouts_compile_to_the_same_numbers(tmp_path):
    src = tmp_path / "layout.c"
    src.write_text(
        '#include <stdio.h>\n#include <stddef.h>\n#include "cumo_hip.h"\n'
        "int main(void){printf(\"%zu %zu %zu %zu %zu %zu %zu %zu\\n\", sizeof(cumo_na_indexer_t), sizeof(cumo_na_iarray_t),"
        "sizeof(cumo_na_bit_iarray_t), sizeof(cumo_na_reduction_arg_t), offsetof(cumo_na_indexer_t, shape),"
        "offsetof(cumo_na_reduction_arg_t, out_indexer), sizeof(cumo_na_iarray_stridx_t), sizeof(cumo_stridx_t));return 0;}\n")
    exe = tmp_path / "layout"
    subprocess.run(["gcc", "-std=c11", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], check=True, stdout=subprocess.PIPE, text=True).stdout.split()
    assert [int(x) for x in out] == [216, 104, 112, 640, 16, 424, 104, 8]


def declared_symbols():
    """Function names in the preprocessed header."""
    names = set()
    for header in HEADERS:
        txt = subprocess.run(["gcc", "-E", "-P", "-I", os.path.join(ROOT, "include"), header], check=True, stdout=subprocess.PIPE, text=True).stdout
        names |= set(re.findall(r"\b(cumo_[a-z0-9_]+)\s*\(", txt))
    names.discard("cumo_hip_error_handler_t")
    return sorted(names)


def test_every_declared_symbol_is_exported():
    from cumo_amd import _lib
    names = declared_symbols()
    assert len(names) > 300, len(names)
    missing = [n for n in names if not hasattr(_lib.lib, n)]
    assert not missing, missing


def test_nothing_but_the_declared_interface_is_exported():
    """The library shares a process with Ruby and the extension: it must export the
    C-ABI of the two headers and nothing else (no kernel stubs, no C++ internals,
    no unprefixed helpers that another library's symbols could interpose)."""
    from cumo_amd import _lib
    out = subprocess.run(["nm", "-D", "--defined-only", _lib.LIB_PATH], check=True, stdout=subprocess.PIPE, text=True).stdout
    exported = {line.split()[2] for line in out.splitlines() if len(line.split()) == 3}
    assert exported, "nm found no exported symbols"
    stray = sorted(n for n in exported if not n.startswith("cumo_"))
    assert not stray, stray[:20]
    undeclared = sorted(exported - set(declared_symbols()))
    assert not undeclared, undeclared[:20]


def test_expected_launcher_names_present():
    names = set(declared_symbols())
    for n in ["cumo_iter_sfloat_add_kernel_launch", "cumo_iter_sfloat_mul_s_kernel_launch", "cumo_iter_dfloat_math_s_exp_kernel_launch",
              "cumo_iter_int32_left_shift_s_kernel_launch", "cumo_iter_sfloat_gt_s_kernel_launch", "cumo_sfloat_sum_kernel_launch",
              "cumo_dfloat_kahan_sum_nan_kernel_launch", "cumo_sfloat_argmax_int32_kernel_launch", "cumo_int32_max_index_int64_kernel_launch",
              "cumo_sfloat_minmax_kernel_launch", "cumo_iter_bit_count_true_stride_kernel_launch", "cumo_iter_bit_and_contiguous_kernel_launch",
              "cumo_iter_copy_bytes_indexer_kernel_launch", "cumo_iter_int32_store_dfloat_kernel_launch", "cumo_cuda_runtime_malloc",
              "cumo_cuda_runtime_check_kernel_launch", "cumo_cuda_runtime_error_flag_new"]:
        assert n in names, n


def test_errors_latch_without_a_handler():
    from cumo_amd import _lib
    # a pointer the pool does not own
    assert _lib.lib.cumo_hip_pool_free(C.c_void_p(0x1000)) == 3
    msg = C.c_char_p()
    assert _lib.lib.cumo_hip_last_error(C.byref(msg)) == 0


def test_missing_library_fails_loudly(tmp_path):
    # the product path has no CPU fallback: without the built library the import raises
    code = (
        "import importlib.util, sys, os\n"
        "spec = importlib.util.spec_from_file_location('lib_copy', %r)\n"
        "m = importlib.util.module_from_spec(spec)\n"
        "try:\n    spec.loader.exec_module(m)\nexcept ImportError as e:\n    print('IMPORTERROR', e); sys.exit(0)\nsys.exit(1)\n")
    src = open(os.path.join(ROOT, "cumo_amd", "_lib.py")).read()
    p = tmp_path / "_lib.py"
    p.write_text(src)
    r = subprocess.run(["python", "-c", code % str(p)], stdout=subprocess.PIPE, text=True)
    assert r.returncode == 0 and "IMPORTERROR" in r.stdout
