"""Migration helpers (aspen_amd/export.py): a PyTorch model exported to an ASPEN_DATA file must give
PyTorch's own outputs when the CPU oracle runs the cfg on that file, which pins batch-norm folding,
tensor order and the connected layer's C,H,W flattening against a library implementation rather than
against this repository's own conventions.  The GPU run of the same file is in test_gpu_parity.py."""
import numpy as np
import pytest
import torch

from aspen_amd import export, models as M
from oracle import cpu as O
from tests import helpers as H


def test_fold_batchnorm_matches_torch():
    torch.manual_seed(1)
    conv, bn = torch.nn.Conv2d(3, 5, 3, padding=1, bias=True), torch.nn.BatchNorm2d(5)
    bn.running_mean.uniform_(-1, 1); bn.running_var.uniform_(0.5, 2); bn.weight.data.uniform_(0.5, 1.5); bn.bias.data.uniform_(-1, 1)
    bn.eval()
    x = torch.randn(2, 3, 6, 6)
    w, b = export.fold_batchnorm(conv.weight, conv.bias, bn.weight, bn.bias, bn.running_mean, bn.running_var, bn.eps)
    want = bn(conv(x)).detach()
    got = torch.nn.functional.conv2d(x, torch.from_numpy(w), torch.from_numpy(b), padding=1)
    assert torch.allclose(got, want, atol=2e-6, rtol=1e-5)


def test_exported_model_runs_like_torch(tmp_path):
    net, cfg, entries = H.export_example_model()
    path = str(tmp_path / "w.bin")
    written = export.export_weights(path, cfg, net.state_dict(), entries, eps=1e-5)
    # the file holds what was written, record by record
    back = export.read_aspen_data(path)
    assert [(i, k) for i, k, _ in back] == [(i, k) for i, k, _ in written]
    for (_, _, a), (_, _, b) in zip(back, written):
        assert np.array_equal(a, np.asarray(b, dtype=np.float32).reshape(-1))
    x = torch.rand(3, 3, 16, 16)
    want = net(x).detach().numpy()                              # [batch, 10]
    layers = M.parse_cfg(cfg)
    tens = [(i, k, a) for i, k, a in back]
    # reshape flat arrays to PyTorch shapes for the oracle's layer functions
    shaped, wl = [], [L for L in layers if L["type"] in export.WEIGHT_LAYERS]
    for i, k, a in tens:
        L = wl[i - 1]
        if k == "WEIGHT" and L["type"] == "conv":
            a = a.reshape(L["C"], L["inC"], L["size"], L["size"])
        elif k == "WEIGHT" and L["type"] == "fc":
            a = a.reshape(L["C"], L["inC"], L["inH"], L["inW"])
        shaped.append((i, k, a))
    outs = O.run_network(layers, shaped, export.nchw_to_dense(x.numpy()), 3, 0)
    got = outs[-1].reshape(3, -1)
    assert np.linalg.norm(got - want) / np.linalg.norm(want) < 1e-5
    assert (got.argmax(1) == want.argmax(1)).all()


def test_export_checks_shapes(tmp_path):
    net, cfg, entries = H.export_example_model()
    sd = dict(net.state_dict())
    with pytest.raises(ValueError):
        export.export_weights(str(tmp_path / "w.bin"), cfg, sd, entries[:-1])
    sd["conv2.weight"] = sd["conv2.weight"][:, :4]
    with pytest.raises(ValueError):
        export.export_weights(str(tmp_path / "w.bin"), cfg, sd, entries)


def test_preprocess_image_closed_forms(tmp_path):
    # a 256 x 256 image needs no resampling: the result is the normalised centre crop
    rng = np.random.default_rng(3)
    img = rng.integers(0, 256, size=(256, 256, 3), dtype=np.uint8)
    out = export.preprocess_image(img)
    want = (img[16:240, 16:240].astype(np.float32) / 255.0 - np.array(export.IMAGENET_MEAN, dtype=np.float32)) / np.array(export.IMAGENET_STD, dtype=np.float32)
    assert out.shape == (3, 224, 224)
    assert np.allclose(out, want.transpose(2, 0, 1), atol=1e-5)
    # a constant image of any size stays constant
    flat = np.full((300, 517, 3), 128, dtype=np.uint8)
    out = export.preprocess_image(flat)
    for c in range(3):
        assert np.allclose(out[c], (128 / 255.0 - export.IMAGENET_MEAN[c]) / export.IMAGENET_STD[c], atol=1e-5)
    # input file: raw NCHW floats, and the dense matrix is its channel-minor transpose
    batch = np.stack([out, out * 0.5])
    p = str(tmp_path / "in.bin")
    export.write_input_file(p, batch)
    assert np.array_equal(np.fromfile(p, dtype=np.float32).reshape(batch.shape), batch)
    dense = export.nchw_to_dense(batch)
    assert dense.shape == (2 * 224 * 224, 3) and dense[224 * 224 + 5 * 224 + 7, 1] == batch[1, 1, 5, 7]
