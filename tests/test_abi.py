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
    s = (ctypes.c_uint32 * 13)()
    api.lib().aspen_hip_tile_shapes(s)
    shapes = list(s)
    for v in range(3):
        assert shapes[2 * v] in (64, 128) and shapes[2 * v + 1] in (64, 128)
    assert shapes[6] in (32, 64, 128) and shapes[7] > 0 and shapes[8] in (2, 4)
    assert (shapes[9], shapes[10]) == (32, 32) and (shapes[11], shapes[12]) == (128, 32)      # the narrow and the tall shape


def test_bench_refuses_more_than_one_gpu():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0 and "ONE GPU" in r.stderr and r.stdout.strip() == ""


def test_error_conventions_of_the_reference_api(tmp_path, capfd):
    """Constructors return NULL on failure, read-outs return -1 on NULL arguments, other calls print and
    return (reference main.c:67-71, src/apu.c:229-238); an object that is still referenced is not
    destroyed (reference src/apu.c:49-54, src/rpool.c:62-66).  No call here touches the GPU."""
    import ctypes as C
    from aspen_amd import models as M
    from tests import helpers as H
    L = api.lib()
    assert not L.apu_create_dnn(None, None)
    assert not L.apu_create_dnn(b"/nonexistent/net.cfg", None)
    assert not L.apu_create_dnn(b"/nonexistent/net.txt", None)          # only .cfg descriptions are read
    assert not L.apu_create_nasm(None, 8, 1)
    assert not L.apu_load_dnn_from_file(None) and not L.apu_load_nasm_from_file(None, None)
    out = C.c_void_p()
    assert L.dse_get_nasm_result(None, None, C.byref(out)) == -1
    assert L.dse_get_ldata_result(None, 0, None, C.byref(out)) == -1
    assert L.dse_check_nasm_completion(None) == 0
    for call in (lambda: L.rpool_add_nasm_raw_input(None, None, None), lambda: L.dse_group_run(None),
                 lambda: L.dse_group_stop(None), lambda: L.dse_group_set_rpool(None, None),
                 lambda: L.rpool_reset_nasm(None, None), lambda: L.apu_destroy_nasm(None), lambda: L.apu_destroy_dnn(None),
                 lambda: L.rpool_destroy(None), lambda: L.dse_group_destroy(None), lambda: L.apu_save_nasm_to_file(None, None)):
        call()                                                           # must return, not crash
    cfg, layers, tens, x, batch, seq = H.tiny_case()
    wp = str(tmp_path / "w.bin")
    M.write_aspen_data(wp, tens)
    d = api.Dnn(cfg, wp)
    assert not L.apu_create_nasm(d.h, 0, batch)                          # min_ninst_per_ldata must be at least 1
    n = api.Nasm(d, batch, seq, 8)
    L.apu_destroy_dnn(d.h)                                               # refused: a nasm still references it
    assert "still referencing" in capfd.readouterr().err
    assert api.Nasm(d, batch, seq, 8).num_ninst == n.num_ninst           # ... and the dnn is still usable
    assert L.dse_get_ldata_result(n.h, 10 ** 6, None, C.byref(out)) == -1   # layer index out of range
    assert L.dse_get_nasm_result(n.h, None, C.byref(out)) == -1          # never run: nothing on the device
    rp, g = L.rpool_init(), L.dse_group_init(4)
    L.dse_group_set_rpool(g, rp)
    L.rpool_destroy(rp)                                                  # refused: an engine group still references it
    assert "still referencing" in capfd.readouterr().err
    L.dse_group_run(g)                                                   # nothing attached: returns without a launch
    L.rpool_reset_nasm(rp, n.h)                                          # not in this pool: prints
    assert "not in rpool" in capfd.readouterr().err
    L.dse_group_destroy(g)
    L.rpool_destroy(rp)
