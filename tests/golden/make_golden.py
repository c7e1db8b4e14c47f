"""Regenerates tests/golden/*.npz by running the COMPILED REFERENCE (oracle/_ref, built from
/root/reference by oracle/Makefile) on the seeded synthetic configurations.

Only runs where the reference tree is mounted.  Fixtures are data only:
  <config>.npz     per layer: H, W, l2 (float64 norm), sum (float64), 256 strided samples + their
                   flat indices into the dense [W][H] matrix; final layer: argmax per column
  micro_<name>.npz full dense per-layer tensors of small nets

usage: python tests/golden/make_golden.py [config ...]
"""
import os
import sys
import tempfile
import time

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from aspen_amd import models as M  # noqa: E402
from oracle import ref  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))
NSAMP = 256

MICRO = {
    # name: (cfg, style, batch, seq, seed, kind)
    "custom_b3": (M.custom_cifar_cfg(), "he", 3, 0, 7, None),
    "resnet_mini_b2": (M.resnet50_cfg(64, 64, 10, (16, 32, 64, 128), (1, 2, 1, 1), 16), "he", 2, 0, 8, None),
    "vgg_mini_b5": (M.vgg16_cfg(32, 32, 10, (8, "M", 16, "M", 64, 64, "M"), (128,)), "he", 5, 0, 9, None),
    "bert_mini_b2_s24": (M.bert_cfg(2, 128, 2, 256), "gpt", 2, 24, 10, "embeddings"),
    "gpt_mini_b2_s20": (M.gpt2_cfg(2, 128, 2, 256), "gpt", 2, 20, 11, "token_ids"),
    "yolo_mini_b2": (M.yolo_mini_cfg(), "he", 2, 0, 12, None),
}


def sample_idx(n):
    return np.unique(np.linspace(0, n - 1, NSAMP).astype(np.int64))


def run_ref(cfg, layers, tens, x, batch, seq):
    wp = tempfile.mktemp(suffix=".bin")
    M.write_aspen_data(wp, tens)
    r = ref.RefNet(cfg, wp, batch, seq)
    os.unlink(wp)
    r.set_input(x)
    r.forward()
    return r


def main(argv):
    assert ref.build() and ref.available(), "reference build unavailable"
    names = argv or list(M.CONFIGS) + ["micro"]
    for name in names:
        if name == "micro":
            for mname, (cfg, style, batch, seq, seed, kind) in MICRO.items():
                layers = M.parse_cfg(cfg)
                tens = M.synth_weights(layers, seed, style)
                x = M.synth_input(layers, seed, batch, seq, kind)
                r = run_ref(cfg, layers, tens, x, batch, seq)
                d = {f"layer{l}": r.layer(l) for l in range(r.num_layers)}
                np.savez_compressed(os.path.join(HERE, f"micro_{mname}.npz"), **d)
                r.close()
                print("micro", mname, "done", flush=True)
            continue
        t0 = time.time()
        cfg, layers, tens, x, batch, seq = M.make_config(name)
        r = run_ref(cfg, layers, tens, x, batch, seq)
        d = {"num_layers": np.int64(r.num_layers)}
        for l in range(r.num_layers):
            a = r.layer(l)
            flat = a.reshape(-1)
            idx = sample_idx(flat.size)
            a64 = flat.astype(np.float64)
            d[f"hw{l}"] = np.array([a.shape[1], a.shape[0]], dtype=np.int64)
            d[f"l2_{l}"] = np.float64(np.sqrt((a64 * a64).sum()))
            d[f"sum{l}"] = np.float64(a64.sum())
            d[f"idx{l}"] = idx
            d[f"val{l}"] = flat[idx].copy()
        last = r.layer(r.num_layers - 1)
        d["argmax"] = last.argmax(axis=1).astype(np.int32)
        d["final_head"] = last[: min(4, last.shape[0])].copy()
        np.savez_compressed(os.path.join(HERE, f"{name}.npz"), **d)
        r.close()
        print(name, "done in %.1fs" % (time.time() - t0), flush=True)


if __name__ == "__main__":
    main(sys.argv[1:])
