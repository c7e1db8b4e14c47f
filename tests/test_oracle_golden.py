"""The oracle against the vectors the compiled reference produced (tests/golden, written by
tests/golden/make_golden.py), and against the compiled reference itself where oracle/_ref exists."""
import os

import numpy as np
import pytest

from aspen_amd import models as M
from oracle import cpu, ref
from tests import helpers as H


@pytest.mark.parametrize("name", list(H.micro_cases()))
def test_oracle_reproduces_reference_fixture(name):
    cfg, layers, tens, x, batch, seq = H.build_case(H.micro_cases()[name])
    gold = np.load(os.path.join(H.GOLDEN, f"micro_{name}.npz"))
    outs = cpu.run_network(layers, tens, x, batch, seq)
    assert len(outs) == len(gold.files)
    for l, o in enumerate(outs):
        g = gold[f"layer{l}"]
        assert o.shape == g.shape
        assert H.rel_l2(o, g) <= 1e-6, (name, l, layers[l]["type"])
    assert (outs[-1].argmax(1) == gold[f"layer{len(outs) - 1}"].argmax(1)).all()


def test_oracle_resnet50_b1_summary():
    """Full ResNet-50 batch 1 against the reference's per-layer summaries."""
    cfg, layers, tens, x, batch, seq = H.full_config("resnet50_b1")
    gold = np.load(os.path.join(H.GOLDEN, "resnet50_b1.npz"))
    outs = cpu.run_network(layers, tens, x, batch, seq)
    for l, o in enumerate(outs):
        flat = o.reshape(-1)
        ref_val = gold[f"val{l}"].astype(np.float64)
        err = np.linalg.norm(flat[gold[f"idx{l}"]] - ref_val) / max(np.linalg.norm(ref_val), 1e-30)
        assert err <= 1e-5, (l, layers[l]["type"], err)
        assert abs(float(np.sqrt((flat.astype(np.float64) ** 2).sum())) - float(gold[f"l2_{l}"])) <= 1e-5 * float(gold[f"l2_{l}"])
    assert (outs[-1].argmax(1) == gold["argmax"]).all()


@pytest.mark.skipif(not ref.available(), reason="oracle/_ref (reference build) not present")
@pytest.mark.parametrize("name", ["custom_b3", "bert_mini_b2_s24", "activation_zoo"])
def test_oracle_matches_compiled_reference(name, tmp_path):
    """Layer by layer against the reference's own tiled_* kernels, including its packed weights
    and its result unpacker.  "activation_zoo" runs every activation of naive_activate and padded pools
    through the reference, with inputs of both signs (without the closing [softmax] layer: the reference's
    tiler divides by zero on a softmax layer outside a transformer; the oracle's softmax is pinned by torch;
    64 channels in front of each connected layer, whose reference kernel assumes that its parent's column
    stride equals its channel count)."""
    if name == "activation_zoo":
        cfg = H.activation_zoo_cfg(softmax=False, filters=64, hidden=64)
        layers = M.parse_cfg(cfg)
        tens = M.synth_weights(layers, 21, "he")
        batch, seq = 3, 0
        x = (M.synth_input(layers, 21, batch, 0, "token_ids") * 2.0 - 1.0).astype(np.float32)
    else:
        cfg, layers, tens, x, batch, seq = H.build_case(H.micro_cases()[name])
    wp = str(tmp_path / "w.bin")
    M.write_aspen_data(wp, tens)
    net = ref.RefNet(cfg, wp, batch, seq, threads=2)
    try:
        net.set_input(x)
        net.forward()
        outs = cpu.run_network(layers, tens, x, batch, seq)
        for l in range(net.num_layers):
            assert H.rel_l2(outs[l], net.layer(l)) <= 1e-6, (l, layers[l]["type"])
        # packed weights: the oracle's [M/8][K][8] layout is the reference's
        widx = 0
        for l, L in enumerate(layers):
            if L["type"] not in ("conv", "fc", "matmul"):
                widx += L["type"] == "layernorm"
                continue
            widx += 1
            w = [t for t in tens if t[0] == widx and t[1] == "WEIGHT"][0][2]
            if L["type"] == "conv":
                mine = cpu.pack_weight(cpu.conv_weight_to_hwc(w))
            elif L["type"] == "fc":
                mine = cpu.pack_weight(np.ascontiguousarray(w.transpose(0, 2, 3, 1)).reshape(w.shape[0], -1))
            else:
                mine = cpu.pack_weight(w)
            theirs = net.weight(l, 3)          # WEIGHT_TENSOR
            assert np.array_equal(mine[: theirs.size], theirs), (l, L["type"])
    finally:
        net.close()
