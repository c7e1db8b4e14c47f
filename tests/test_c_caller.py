"""The public header is enough for a C caller: the reference's own driver and example programs compile
against include/aspen.h, and a C program written here links against the shared library and runs."""
import glob
import os
import subprocess

import numpy as np
import pytest

from aspen_amd import api, models as M
from tests import helpers as H

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INCLUDE = os.path.join(ROOT, "include")
CALLER_SRC = os.path.join(ROOT, "tests", "c", "caller.c")
REFERENCE = "/root/reference"


def build_caller(out_dir):
    exe = os.path.join(str(out_dir), "caller")
    lib_dir = os.path.dirname(api.LIB_PATH)
    subprocess.check_call(["gcc", "-O1", "-Wall", "-Wextra", "-Werror", "-I", INCLUDE, CALLER_SRC, "-o", exe,
                           "-L", lib_dir, "-laspen_amd", f"-Wl,-rpath,{lib_dir}", "-Wl,-rpath,/opt/rocm/lib", "-lm"])
    return exe


@pytest.mark.skipif(not os.path.isdir(REFERENCE), reason="the reference tree is not mounted here")
def test_reference_callers_compile_against_the_header():
    """reference main.c and examples/*/aspen_*.c include only aspen.h; every function, type, enumerator and
    system facility they use must come through include/aspen.h."""
    sources = [os.path.join(REFERENCE, "main.c")] + sorted(glob.glob(os.path.join(REFERENCE, "examples", "*", "aspen_*.c")))
    assert len(sources) >= 4
    for src in sources:
        r = subprocess.run(["gcc", "-fsyntax-only", "-Wall", "-Werror=implicit-function-declaration", "-I", INCLUDE, src],
                           capture_output=True, text=True)
        assert r.returncode == 0, (src, r.stderr)
        assert "error" not in r.stderr, (src, r.stderr)


def test_reference_header_macros_and_tables_for_c_callers(tmp_path):
    """Enumerator name tables and the console macros of the reference header (include/aspen.h:34-48,65-73),
    used from C; also under SUPPRESS_OUTPUT."""
    src = tmp_path / "names.c"
    src.write_text('#include "aspen.h"\n'
                   "int main (void) {\n"
                   '  PRTF ("%s %s %s %s %s %s %s\\n", ninst_state_str[NINST_COMPLETED], layer_type_str[V_ATTENTION_LAYER],\n'
                   "    param_type_str[FORM_BYTES], tensor_type_str[BN_WEIGHT_TENSOR], parent_type_str[PARENT_WEIGHT],\n"
                   "    activation_type_str[GELU_ACCURATE], rpool_cond_str[RPOOL_DSE]);\n"
                   '  GREEN_PRTF ("%d", 1); RED_PRTF ("%d", 2); YELLOW_PRTF ("%d", 3); BLUE_PRTF ("%d", 4);\n'
                   "  if (NUM_RPOOL_CONDS != 5) return 3;\n"
                   "  return 0; }\n")
    lib_dir = os.path.dirname(api.LIB_PATH)
    for extra, expect in ((["-DSUPPRESS_OUTPUT=0"], True), (["-DSUPPRESS_OUTPUT=1"], False)):
        exe = str(tmp_path / "names")
        subprocess.check_call(["gcc", "-Wall", "-Werror", "-I", INCLUDE, str(src), "-o", exe, "-L", lib_dir, "-laspen_amd",
                               f"-Wl,-rpath,{lib_dir}", "-Wl,-rpath,/opt/rocm/lib"] + extra)
        out = subprocess.run([exe], capture_output=True, text=True, check=True).stdout
        if expect:
            assert "NINST_COMPLETED V_ATTENTION_LAYER FORM_BYTES BN_WEIGHT_TENSOR PARENT_WEIGHT GELU_ACCURATE RPOOL_DSE" in out
            assert "\033[0;32m1\033[0m" in out
        else:
            assert out == ""


def test_c_caller_compiles_and_links(tmp_path):
    exe = build_caller(tmp_path)
    r = subprocess.run([exe], capture_output=True, text=True)
    assert r.returncode == 2 and "usage" in r.stderr


@pytest.mark.gpu
def test_c_caller_runs_a_network_and_matches_the_reference_fixture(gpu, tmp_path):
    """The compiled C program end to end on the GPU (cfg + weights -> .aspen -> graph -> three inferences ->
    result file) against the compiled reference's output for the same network, weights and input."""
    name = "custom_b3"
    cfg, layers, tens, x, batch, seq = H.build_case(H.micro_cases()[name])
    gold = np.load(os.path.join(H.GOLDEN, f"micro_{name}.npz"))
    exe = build_caller(tmp_path)
    cfg_path, w_path, in_path, out_path = (str(tmp_path / n) for n in ("net.cfg", "net.bin", "in.bin", "out.bin"))
    open(cfg_path, "w").write(cfg)
    M.write_aspen_data(w_path, tens)
    chw = [l for l in layers if l["type"] == "input"][0]
    nchw = np.ascontiguousarray(x, dtype=np.float32).reshape(batch, chw["H"], chw["W"], chw["C"]).transpose(0, 3, 1, 2)
    np.ascontiguousarray(nchw).tofile(in_path)
    print("running", exe, flush=True)
    r = subprocess.run([exe, cfg_path, w_path, in_path, str(batch), "64", "3", out_path, str(tmp_path / "net.aspen")],
                       capture_output=True, text=True, timeout=100)
    assert r.returncode == 0, r.stderr[-2000:]
    want = gold[f"layer{len(layers) - 1}"]                       # [batch][classes]
    got = np.fromfile(out_path, dtype=np.float32).reshape(want.shape)
    assert H.rel_l2(got, want) <= H.REL_L2_TOL
    assert (got.argmax(1) == want.argmax(1)).all()
