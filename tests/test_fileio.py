"""The reference's container formats (.aspen model files, .nasm graph files; reference
src/apu_file_io.c:434-1093): files written by the compiled reference (tests/golden/tiny_ref.*, made by
tests/golden/make_file_fixtures.py) load here, and what this library writes is what the reference writes."""
import os

import numpy as np
import pytest

from aspen_amd import api, models as M
from tests import helpers as H

REF_ASPEN = os.path.join(H.GOLDEN, "tiny_ref.aspen")
REF_NASM = os.path.join(H.GOLDEN, "tiny_ref_b2.nasm")


def lines_except_header(path):
    """File bytes with the two free-text header lines (build id, model name) blanked."""
    out = []
    with open(path, "rb") as f:
        for i, line in enumerate(f.read().split(b"\n")):
            out.append(b"" if line.startswith((b"ASPEN_BUILD:", b"DNN_NAME:")) and i < 4 else line)
    return out


def dnn_from_cfg(tmp_path):
    cfg, layers, tens, x, batch, seq = H.tiny_case()
    wp = str(tmp_path / "w.bin")
    M.write_aspen_data(wp, tens)
    return api.Dnn(cfg, wp)


def test_aspen_file_written_here_equals_the_reference_file(tmp_path):
    """Model built from cfg + ASPEN_DATA weights, saved: byte-identical (but for build id and name) to the
    file the reference wrote for the same model -- same layer records, same packed [M/8][K][8] tensors."""
    d = dnn_from_cfg(tmp_path)
    mine = str(tmp_path / "mine.aspen")
    api.lib().apu_save_dnn_to_file(d.h, mine.encode())
    assert lines_except_header(mine) == lines_except_header(REF_ASPEN)
    d.destroy()


def test_aspen_file_from_the_reference_loads(tmp_path):
    """Load the reference's file, save it again: round trip is lossless, and the graph of the loaded
    model is the graph of the cfg-built model."""
    L = api.lib()
    h = L.apu_load_dnn_from_file(REF_ASPEN.encode())
    assert h
    again = str(tmp_path / "again.aspen")
    L.apu_save_dnn_to_file(h, again.encode())
    assert lines_except_header(again) == lines_except_header(REF_ASPEN)
    loaded = api.Dnn.__new__(api.Dnn); loaded.h = h
    n1 = api.Nasm(loaded, 2, 0, 8)
    d = dnn_from_cfg(tmp_path)
    n2 = api.Nasm(d, 2, 0, 8)
    assert n1.num_ninst == n2.num_ninst and n1.total_flops == n2.total_flops
    for a, b in zip(n1.graph(), n2.graph()):
        assert np.array_equal(a, b)
    n1.destroy(); n2.destroy(); d.destroy(); L.apu_destroy_dnn(h)


def test_aspen_file_errors(tmp_path, capfd):
    L = api.lib()
    assert not L.apu_load_dnn_from_file(b"/nonexistent.aspen")
    raw = open(REF_ASPEN, "rb").read()
    cut = tmp_path / "cut.aspen"
    cut.write_bytes(raw[: len(raw) // 2])                      # truncated inside a tensor
    assert not L.apu_load_dnn_from_file(str(cut).encode())
    bad = tmp_path / "bad.aspen"
    bad.write_bytes(raw.replace(b"LAYER_PARAMS_END", b"LAYER_PARAMS_ENX", 1))
    assert not L.apu_load_dnn_from_file(str(bad).encode())
    assert capfd.readouterr().err != ""


@pytest.mark.parametrize("field, value", [(b"LAYER_TYPE:", b"99"), (b"LAYER_TYPE:", b"-3"), (b"LAYER_ACTIVATION:", b"42")])
def test_aspen_file_with_unknown_ids_is_rejected(tmp_path, field, value, capfd):
    """A model file whose second layer names a layer type or activation the enumerations do not have
    (they index the tables of the print_* dumps and select device code) does not load."""
    raw = open(REF_ASPEN, "rb").read()
    first = raw.index(field)
    at = raw.index(field, first + 1) + len(field)
    end = raw.index(b"\n", at)
    bad = tmp_path / "bad.aspen"
    bad.write_bytes(raw[:at] + value + raw[end:])
    assert not api.lib().apu_load_dnn_from_file(str(bad).encode())
    assert "unknown" in capfd.readouterr().err


def test_nasm_file_round_trip_and_cross_check(tmp_path, capfd):
    L = api.lib()
    d = dnn_from_cfg(tmp_path)
    n = api.Nasm(d, 2, 0, 8)
    path = str(tmp_path / "g.nasm")
    L.apu_save_nasm_to_file(n.h, path.encode())
    text = open(path).read()
    assert text.startswith("ASPEN_NASM\n") and text.endswith("NASM_NINSTS_END\nASPEN_NASM_END\n")
    assert text.count("\tNINST_IDX:") == n.num_ninst and f"TOTAL_FLOPS:{n.total_flops}\n" in text
    h = L.apu_load_nasm_from_file(path.encode(), d.h)
    assert h and L.aspen_nasm_num_ninst(h) == n.num_ninst and L.aspen_nasm_num_edges(h) == n.num_edges
    L.apu_destroy_nasm(h)
    assert "another tile grid" not in capfd.readouterr().out
    # a file whose dependency lists were tampered with is refused
    tl, npar, off, idx = n.graph()
    t = int(np.argmax(npar > 0))                               # first tile with a parent
    marker = f"\tNINST_IDX:{t}\n"
    i = text.index(marker)
    j = text.index("\tPARENT_NINSTS:\n", i) + len("\tPARENT_NINSTS:\n")
    k = text.index("\n", j)
    first = text[j:k].split()
    tampered = text[:j] + f"\t\t{first[0]} {int(first[1]) + 1}" + text[k:]
    bad = tmp_path / "bad.nasm"
    bad.write_text(tampered)
    assert not L.apu_load_nasm_from_file(str(bad).encode(), d.h)
    # wrong model / batch: FLOP total does not match
    bad.write_text(text.replace(f"TOTAL_FLOPS:{n.total_flops}", f"TOTAL_FLOPS:{n.total_flops + 2}"))
    assert not L.apu_load_nasm_from_file(str(bad).encode(), d.h)
    assert not L.apu_load_nasm_from_file(b"/nonexistent.nasm", d.h)
    assert not L.apu_load_nasm_from_file(path.encode(), None)
    capfd.readouterr()
    n.destroy(); d.destroy()


def test_nasm_file_from_the_reference_loads(tmp_path, capfd):
    """The reference's file describes its CPU tile grid: the header (batch, tiles per layer, FLOPs) is
    taken, the graph is rebuilt on this build's grid."""
    L = api.lib()
    d = dnn_from_cfg(tmp_path)
    h = L.apu_load_nasm_from_file(REF_NASM.encode(), d.h)
    assert h
    assert "another tile grid" in capfd.readouterr().out
    ref_hdr = dict(l.split(":", 1) for l in open(REF_NASM).read().split("NASM_NINSTS:")[0].strip().split("\n")[1:])
    assert L.aspen_nasm_total_flops(h) == int(ref_hdr["TOTAL_FLOPS"])
    a = (api.C.c_uint * 20)()
    L.aspen_nasm_ldata_info(h, 0, a)
    assert a[3] == int(ref_hdr["NUM_BATCH"]) * 8 * 8
    L.apu_destroy_nasm(h)
    d.destroy()


@pytest.mark.skipif(not os.path.exists("/root/reference/files/resnet50/resnet50_B1.nasm"), reason="reference tree not mounted")
def test_shipped_resnet50_nasm_header_matches_model(capfd):
    """The graph file the reference ships for ResNet-50 batch 1 loads against this build's ResNet-50:
    its TOTAL_FLOPS header must equal the model's FLOP count or the load is refused."""
    L = api.lib()
    d = api.Dnn(M.resnet50_cfg(), None)
    h = L.apu_load_nasm_from_file(b"/root/reference/files/resnet50/resnet50_B1.nasm", d.h)
    assert h and L.aspen_nasm_total_flops(h) == 8185945088
    L.apu_destroy_nasm(h)
    h = L.apu_load_nasm_from_file(b"/root/reference/files/vgg16/vgg16_B1.nasm", d.h)     # VGG graph, ResNet model
    assert not h
    capfd.readouterr()
    d.destroy()


def _with_layer_param(raw: bytes, layer: int, param: int, value: int) -> bytes:
    """The model file with parameter `param` of layer `layer` set to `value` (records are "\\t\\t<index> <value>")."""
    at = -1
    for _ in range(layer + 1):
        at = raw.index(b"\tLAYER_PARAMS:\n", at + 1)
    key = b"\t\t%d " % param
    i = raw.index(key, at)
    j = raw.index(b"\n", i)
    return raw[:i] + key + b"%d" % value + raw[j:]


@pytest.mark.parametrize("layer, param, value", [
    (1, api.STRIDE, 7),             # window geometry no longer gives the stated output size
    (1, api.OUT_H, 4000),           # output taller than its parent allows
    (1, api.IN_C, 64),              # more input channels than the parent has
    (1, api.PADDING, 1 << 30),      # absurd value
    (2, api.IN_H, 1),               # pool reading a parent of another height
    (4, api.IN_W, 9),               # FC layer over a wider image than its parent
])
def test_aspen_file_with_inconsistent_parameters_is_rejected(tmp_path, layer, param, value, capfd):
    """The loader derives every layer's geometry from its parents and window, as the cfg parser does, and
    refuses a file that states something else: tensors are sized and kernels index with these numbers."""
    raw = open(REF_ASPEN, "rb").read()
    assert api.lib().apu_load_dnn_from_file(str(REF_ASPEN).encode())     # untouched: loads
    bad = tmp_path / "bad.aspen"
    bad.write_bytes(_with_layer_param(raw, layer, param, value))
    assert not api.lib().apu_load_dnn_from_file(str(bad).encode())
    err = capfd.readouterr().err
    assert "inconsistent parameters" in err


def test_weight_file_cannot_ask_for_arbitrary_memory(tmp_path, capfd):
    """ASPEN_DATA: a tensor's size is checked against the layer BEFORE anything is allocated."""
    cfg, layers, tens, x, batch, seq = H.tiny_case()
    wp = str(tmp_path / "w.bin")
    M.write_aspen_data(wp, tens)
    raw = open(wp, "rb").read()
    i = raw.index(b"DATA_SIZE:") + len(b"DATA_SIZE:")
    j = raw.index(b"\n", i)
    huge = tmp_path / "huge.bin"
    huge.write_bytes(raw[:i] + b"%d" % (1 << 46) + raw[j:])
    d = api.Dnn(cfg, str(huge))                                    # prints, keeps the seeded weights (as the reference does)
    assert "size mismatch" in capfd.readouterr().err
    d.destroy()


def test_reloading_weights_marks_device_graphs_stale(tmp_path):
    """apu_load_dnn_data_from_file on a model advances its device generation only when device copies existed;
    without a GPU no copies exist and the call just replaces the host weights."""
    cfg, layers, tens, x, batch, seq = H.tiny_case()
    wp = str(tmp_path / "w.bin")
    M.write_aspen_data(wp, tens)
    d = api.Dnn(cfg, wp)
    before = str(tmp_path / "a.aspen"); after = str(tmp_path / "b.aspen")
    api.lib().apu_save_dnn_to_file(d.h, before.encode())
    tens2 = [(i, k, (a * 2).astype(np.float32)) for i, k, a in tens]
    wp2 = str(tmp_path / "w2.bin")
    M.write_aspen_data(wp2, tens2)
    assert api.lib().aspen_dnn_device_generation(d.h) == 0
    api.lib().apu_load_dnn_data_from_file(d.h, wp2.encode())
    assert api.lib().aspen_dnn_device_generation(d.h) == 0          # nothing was on a device
    api.lib().apu_save_dnn_to_file(d.h, after.encode())
    assert lines_except_header(before) != lines_except_header(after)
    d.destroy()
