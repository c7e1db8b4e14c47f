"""The C-ABI shared library loads without a GPU and exports every function include/*.h declares;
pure-constant entry points answer; bench.py refuses more than one GPU."""
import ctypes
import os
import re
import subprocess
import sys

import pytest

from aspen_amd import api

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INCLUDE = os.path.join(ROOT, "include")


def declared_functions(path):
    text = open(path).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    text = re.sub(r"^\s*#.*$", "", text, flags=re.M)
    names = set()
    for stmt in text.split(";"):
        stmt = " ".join(stmt.split())
        if "(" not in stmt or stmt.startswith("typedef") or "{" in stmt:
            continue
        m = re.match(r"^(?:extern \"C\" )?[\w\s\*]+?[\s\*](\w+) ?\(", stmt)
        if m:
            names.add(m.group(1))
    return names


def test_headers_declare_what_the_library_exports():
    lib = ctypes.CDLL(api.LIB_PATH)
    total = 0
    for h in sorted(os.listdir(INCLUDE)):
        names = declared_functions(os.path.join(INCLUDE, h))
        assert names, h
        missing = [n for n in sorted(names) if not hasattr(lib, n)]
        assert not missing, (h, missing)
        total += len(names)
    assert total >= 70


def test_reference_api_names_present():
    """The names a reference user calls (every function of reference include/aspen.h:90-133)."""
    lib = api.lib()
    names = """apu_create_dnn apu_destroy_dnn apu_save_dnn_to_file apu_load_dnn_from_file apu_generate_nasm
        apu_generate_transformer_nasm apu_create_nasm apu_create_transformer_nasm apu_destroy_nasm apu_load_nasm_from_file
        apu_save_nasm_to_file apu_reset_nasm rpool_init rpool_destroy rpool_add_nasm_raw_input rpool_add_nasm
        rpool_reset_queue rpool_reset_nasm dse_group_init dse_group_set_rpool dse_group_destroy dse_group_run
        dse_group_stop dse_group_run_until_nasm_completion dse_wait_for_nasm_completion dse_check_nasm_completion
        dse_get_ldata_result dse_get_nasm_result aspen_flush_dynamic_memory print_aspen_build_info print_dnn_info
        print_layer_info print_tensor_info print_nasm_info print_ldata_info print_ninst_info print_rpool_queue_info
        print_rpool_queue_group_info print_rpool_info""".split()
    for n in names:
        assert hasattr(lib, n), n


def test_tile_shapes_are_constants():
    s = (ctypes.c_uint32 * 9)()
    api.lib().aspen_hip_tile_shapes(s)
    shapes = list(s)
    for v in range(3):
        assert shapes[2 * v] in (64, 128) and shapes[2 * v + 1] in (64, 128)
    assert shapes[6] in (64, 128) and shapes[7] > 0 and shapes[8] in (2, 4)


def test_bench_refuses_more_than_one_gpu():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0 and "ONE GPU" in r.stderr and r.stdout.strip() == ""
