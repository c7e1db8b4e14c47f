"""Shared test plumbing: run a network through the C-ABI library, compare with oracle / fixtures."""
import os
import tempfile

import numpy as np

from aspen_amd import api, models as M

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
REL_L2_TOL = 1e-4          # per-layer relative L2 bound of the parity contract


def rel_l2(a, b):
    a = np.asarray(a, dtype=np.float64).ravel()
    b = np.asarray(b, dtype=np.float64).ravel()
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))


class GpuNet:
    """dnn + nasm + rpool + dse group of one network, driven in the reference's call order."""

    def __init__(self, cfg, tensors, batch, seq=0, min_ninst=512, mode=api.MODE_DATAFLOW, workgroups=0):
        self.wpath = None
        if tensors is not None:
            self.wpath = tempfile.mktemp(suffix=".bin")
            M.write_aspen_data(self.wpath, tensors)
        self.dnn = api.Dnn(cfg, self.wpath)
        if self.wpath:
            os.unlink(self.wpath)
        self.nasm = api.Nasm(self.dnn, batch, seq, min_ninst)
        self.rpool = api.RPool()
        self.dse = api.DseGroup(1, mode, workgroups)
        self.dse.set_rpool(self.rpool)
        self.first = True

    def run(self, x):
        if self.first:
            self.rpool.add_nasm_raw_input(self.nasm, x)
            self.first = False
        else:
            self.rpool.reset_queue()
            self.rpool.reset_nasm(self.nasm)
            if x is not None:
                self.rpool.add_nasm_raw_input(self.nasm, x)
        self.dse.run()
        self.dse.wait(self.nasm)
        self.dse.stop()

    def layer(self, l):
        return self.nasm.layer_output(l)

    def close(self):
        self.dse.destroy()
        self.rpool.destroy()
        self.nasm.destroy()
        self.dnn.destroy()


def micro_cases():
    # name -> (cfg, style, batch, seq, seed, input kind); must match tests/golden/make_golden.py
    return {
        "custom_b3": (M.custom_cifar_cfg(), "he", 3, 0, 7, None),
        "resnet_mini_b2": (M.resnet50_cfg(64, 64, 10, (16, 32, 64, 128), (1, 2, 1, 1), 16), "he", 2, 0, 8, None),
        "vgg_mini_b5": (M.vgg16_cfg(32, 32, 10, (8, "M", 16, "M", 64, 64, "M"), (128,)), "he", 5, 0, 9, None),
        "bert_mini_b2_s24": (M.bert_cfg(2, 128, 2, 256), "gpt", 2, 24, 10, "embeddings"),
        "gpt_mini_b2_s20": (M.gpt2_cfg(2, 128, 2, 256), "gpt", 2, 20, 11, "token_ids"),
        "yolo_mini_b2": (M.yolo_mini_cfg(), "he", 2, 0, 12, None),
    }


def build_case(case):
    cfg, style, batch, seq, seed, kind = case
    layers = M.parse_cfg(cfg)
    tens = M.synth_weights(layers, seed, style)
    x = M.synth_input(layers, seed, batch, seq, kind or "token_ids")
    return cfg, layers, tens, x, batch, seq


_CONFIG_CACHE = {}


def full_config(name):
    """(cfg, layers, tensors, input, batch, seq) of a named benchmark configuration; weights are
    cached per (generator, seed) because several configurations share a network."""
    gen, style, batch, seq, seed, kind = M.CONFIGS[name]
    key = (gen.__name__, style, seed)
    if key not in _CONFIG_CACHE:
        cfg = gen()
        layers = M.parse_cfg(cfg)
        _CONFIG_CACHE.clear()          # keep at most one big weight set alive
        _CONFIG_CACHE[key] = (cfg, layers, M.synth_weights(layers, seed, style))
    cfg, layers, tens = _CONFIG_CACHE[key]
    x = M.synth_input(layers, seed, batch, seq, kind or "token_ids")
    return cfg, layers, tens, x, batch, seq


def check_against_summary(net, gold, layers, label):
    """Per-layer comparison with a summary fixture (norm, sum, strided samples, final argmax)."""
    n = int(gold["num_layers"])
    assert n == net.nasm.num_ldata
    worst = 0.0
    for l in range(n):
        got = net.layer(l)
        h, w = (int(v) for v in gold[f"hw{l}"])
        assert got.shape == (w, h), (label, l, got.shape, (w, h))
        flat = got.reshape(-1)
        ref_val = gold[f"val{l}"].astype(np.float64)
        got_val = flat[gold[f"idx{l}"]].astype(np.float64)
        ref_l2 = float(gold[f"l2_{l}"])
        # relative L2 over the sampled entries, scaled by the layer's RMS so that near-zero samples do not dominate
        rms = ref_l2 / np.sqrt(flat.size)
        err = np.linalg.norm(got_val - ref_val) / max(np.linalg.norm(ref_val), rms * np.sqrt(ref_val.size) * 1e-3, 1e-30)
        worst = max(worst, err)
        assert err <= REL_L2_TOL, f"{label} layer {l} ({layers[l]['type']}): sampled rel L2 {err:.3g}"
        got_l2 = float(np.sqrt((flat.astype(np.float64) ** 2).sum()))
        assert abs(got_l2 - ref_l2) <= REL_L2_TOL * ref_l2, f"{label} layer {l}: norm {got_l2} vs {ref_l2}"
        got_sum = float(flat.astype(np.float64).sum())
        assert abs(got_sum - float(gold[f"sum{l}"])) <= REL_L2_TOL * ref_l2 * np.sqrt(flat.size), f"{label} layer {l}: sum"
    final = net.layer(n - 1)
    assert (final.argmax(axis=1) == gold["argmax"]).all(), f"{label}: argmax differs"
    return worst


def activation_zoo_cfg(softmax=True, filters=24, hidden=40):
    """Every activation the reference's naive_activate knows (reference src/naive_kernels.c:11-57) on a
    contraction epilogue or a shortcut, a padded max pool and average pool, a [softmax] layer at the end."""
    s = "[net]\nheight=12\nwidth=12\nchannels=5\n\n"
    for act in ("logistic", "tanh", "elu", "selu", "leaky", "gelu", "gelu_acc", "relu", "linear"):
        s += f"[convolutional]\nfilters={filters}\nsize=3\nstride=1\npad=1\nactivation={act}\n\n"
    s += "[shortcut]\nfrom=-3\nactivation=tanh\n\n"
    s += "[maxpool]\nsize=3\nstride=2\npad=1\n\n"
    s += "[avgpool]\nsize=3\nstride=1\npad=1\n\n"
    s += f"[connected]\noutput={hidden}\nactivation=logistic\n\n[connected]\noutput=17\nactivation=linear\n\n"
    if softmax:
        s += "[softmax]\n\n"
    return s


def tiny_cfg():
    """A few-kilobyte network for file-format fixtures: odd channel counts exercise the padding of the
    reference's 8-row weight interleave (the layer in front of the FC layer has 64 channels:
    the reference requires the FC parent's column stride to equal its channel count)."""
    return ("[net]\nheight=8\nwidth=8\nchannels=3\n\n"
            "[convolutional]\nfilters=5\nsize=3\nstride=1\npad=1\nactivation=relu\n\n"
            "[maxpool]\nsize=2\nstride=2\n\n"
            "[convolutional]\nfilters=64\nsize=1\nstride=1\npad=0\nactivation=leaky\n\n"
            "[connected]\noutput=10\nactivation=linear\n\n")


def tiny_case():
    cfg = tiny_cfg()
    layers = M.parse_cfg(cfg)
    tens = M.synth_weights(layers, 77, "he")
    x = M.synth_input(layers, 77, 2, 0, "embeddings")
    return cfg, layers, tens, x, 2, 0


def export_example_model():
    """A small PyTorch network with batch-norm after its convolutions, its cfg, and the state-dict
    entries of its tensor-owning layers in cfg order (for aspen_amd.export.export_weights)."""
    import torch

    class Net(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.conv1 = torch.nn.Conv2d(3, 8, 3, padding=1, bias=False)
            self.bn1 = torch.nn.BatchNorm2d(8)
            self.conv2 = torch.nn.Conv2d(8, 16, 3, stride=2, padding=1, bias=True)
            self.bn2 = torch.nn.BatchNorm2d(16)
            self.conv3 = torch.nn.Conv2d(16, 64, 1, bias=True)
            self.fc1 = torch.nn.Linear(64 * 4 * 4, 32)
            self.fc2 = torch.nn.Linear(32, 10)

        def forward(self, x):
            x = torch.relu(self.bn1(self.conv1(x)))
            x = torch.nn.functional.max_pool2d(x, 2, 2)
            x = torch.nn.functional.leaky_relu(self.bn2(self.conv2(x)), 0.1)
            x = torch.relu(self.conv3(x))
            x = torch.relu(self.fc1(torch.flatten(x, 1)))
            return self.fc2(x)

    torch.manual_seed(5)
    net = Net()
    for bn in (net.bn1, net.bn2):
        bn.running_mean.uniform_(-0.5, 0.5); bn.running_var.uniform_(0.5, 2.0)
        bn.weight.data.uniform_(0.5, 1.5); bn.bias.data.uniform_(-0.5, 0.5)
    net.eval()
    cfg = ("[net]\nheight=16\nwidth=16\nchannels=3\n\n"
           "[convolutional]\nfilters=8\nsize=3\nstride=1\npad=1\nactivation=relu\n\n"
           "[maxpool]\nsize=2\nstride=2\n\n"
           "[convolutional]\nfilters=16\nsize=3\nstride=2\npad=1\nactivation=leaky\n\n"
           "[convolutional]\nfilters=64\nsize=1\nstride=1\npad=0\nactivation=relu\n\n"
           "[connected]\noutput=32\nactivation=relu\n\n"
           "[connected]\noutput=10\nactivation=linear\n\n")
    entries = [("conv1", "bn1"), ("conv2", "bn2"), "conv3", "fc1", "fc2"]
    return net, cfg, entries
