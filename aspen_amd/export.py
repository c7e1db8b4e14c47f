"""Migration helpers: bring a trained PyTorch model and its input images to the files this library
(and the reference) load.

* ``export_weights``   PyTorch tensors -> ``ASPEN_DATA`` weight file, batch-norm folded into the
                       preceding convolution (the file format is the one spelled out in the reference's
                       ``examples/3. custom_example/instructions.txt:29-48`` and parsed by
                       ``src/apu_file_io.c:48-432``; the reference's loaders expect folded weights)
* ``read_aspen_data``  the inverse, for checking a file
* ``preprocess_image`` the usual ImageNet preprocessing (shorter side to 256, centre crop 224, scale to
                       [0, 1], normalise) that the reference's examples apply before inference
                       (``examples/1. resnet50_example/preprocess_image.py:21-31``), on a decoded image array
* ``write_input_file`` a batch of NCHW float32 images as the raw file ``rpool_add_nasm`` reads
                       (reference ``src/apu.c:638``, ``src/util.c:311-343``)

Nothing here runs on the GPU; PyTorch is used on the CPU for resampling only.
"""
from typing import Dict, Iterable, List, Optional, Sequence, Tuple

import numpy as np

from .models import Tensor, parse_cfg, write_aspen_data

WEIGHT_LAYERS = ("conv", "fc", "matmul", "layernorm")     # the layer kinds that own tensors, in file order


def _np(t) -> np.ndarray:
    if hasattr(t, "detach"):
        t = t.detach().cpu().numpy()
    return np.ascontiguousarray(t, dtype=np.float32)


def fold_batchnorm(weight, bias, gamma, beta, mean, var, eps: float = 1e-5) -> Tuple[np.ndarray, np.ndarray]:
    """conv -> batch-norm (inference) as one convolution: scale every output channel's filter by
    gamma / sqrt(var + eps) and move the shift into the bias."""
    w = _np(weight).astype(np.float64)
    scale = _np(gamma).astype(np.float64) / np.sqrt(_np(var).astype(np.float64) + eps)
    b = np.zeros(w.shape[0]) if bias is None else _np(bias).astype(np.float64)
    w = w * scale.reshape((-1,) + (1,) * (w.ndim - 1))
    b = _np(beta).astype(np.float64) + (b - _np(mean).astype(np.float64)) * scale
    return w.astype(np.float32), b.astype(np.float32)


def export_weights(path: str, cfg_text: str, state: Dict, entries: Sequence, eps: float = 1e-5) -> List[Tensor]:
    """Writes the ``ASPEN_DATA`` file for the network ``cfg_text`` describes.

    ``entries`` names, for every tensor-owning layer of the cfg in order (convolutional, connected,
    matmul, layernorm sections), where its tensors are in ``state`` (a ``state_dict`` or any mapping of
    names to arrays): a module prefix ``"conv1"`` (reads ``conv1.weight`` and, if present, ``conv1.bias``)
    or a pair ``("layer1.0.conv1", "layer1.0.bn1")`` whose second module is a batch-norm to fold in
    (``.weight .bias .running_mean .running_var``).  Shapes are checked against the cfg: a convolution's
    weight is ``[filters, in_channels, size, size]``, a connected layer's ``[outputs, inputs]`` (flattened
    in PyTorch's C,H,W order, which is what the library expects), a matmul's ``[M, K]``.
    Returns the tensor list that was written.
    """
    layers = [L for L in parse_cfg(cfg_text) if L["type"] in WEIGHT_LAYERS]
    if len(entries) != len(layers):
        raise ValueError(f"cfg has {len(layers)} tensor-owning layers, {len(entries)} entries given")
    out: List[Tensor] = []
    for widx, (L, ent) in enumerate(zip(layers, entries), start=1):
        conv, bn = (ent, None) if isinstance(ent, str) else ent
        w = _np(state[conv + ".weight"])
        b = _np(state[conv + ".bias"]) if conv + ".bias" in state else None
        if bn is not None:
            w, b = fold_batchnorm(w, b, state[bn + ".weight"], state[bn + ".bias"],
                                  state[bn + ".running_mean"], state[bn + ".running_var"], eps)
        rows = L["C"] if L["type"] in ("conv", "fc") else L["M"]
        if w.shape[0] != rows:
            raise ValueError(f"layer {L['idx']} ({L['type']}): cfg wants {rows} output rows, '{conv}.weight' has {w.shape[0]}")
        if L["type"] == "conv" and (w.ndim != 4 or w.shape[1] != L["inC"] or w.shape[2] != L["size"] or w.shape[3] != L["size"]):
            raise ValueError(f"layer {L['idx']}: convolution weight {w.shape} does not match the cfg "
                             f"([{rows}, {L['inC']}, {L['size']}, {L['size']}])")
        if L["type"] == "fc" and w.size != rows * L["inC"] * L["inH"] * L["inW"]:
            raise ValueError(f"layer {L['idx']}: connected weight {w.shape} does not match {L['inC']}x{L['inH']}x{L['inW']} inputs")
        out.append((widx, "WEIGHT", w))
        if b is not None:
            out.append((widx, "BIAS", b))
    write_aspen_data(path, out)
    return out


def read_aspen_data(path: str) -> List[Tensor]:
    """Parses an ``ASPEN_DATA`` file into ``(layer index, tensor type, flat float32 array)`` records."""
    raw = open(path, "rb").read()
    if not raw.startswith(b"ASPEN_DATA\n"):
        raise ValueError("not an ASPEN_DATA file")
    pos, out = len(b"ASPEN_DATA\n"), []

    def line():
        nonlocal pos
        end = raw.index(b"\n", pos)
        s = raw[pos:end].decode()
        pos = end + 1
        return s

    while pos < len(raw):
        head = line()
        if not head:
            continue
        if not head.startswith("LAYER:"):
            raise ValueError(f"expected LAYER:, found {head!r}")
        widx = int(head[6:])
        kind = line().split(":", 1)[1]
        size = int(line().split(":", 1)[1])
        if line() != "DATA_START:":
            raise ValueError("expected DATA_START:")
        arr = np.frombuffer(raw, dtype=np.float32, count=size // 4, offset=pos).copy()
        pos += size
        if line() != "DATA_END" or line() != "LAYER_END":
            raise ValueError("expected DATA_END / LAYER_END")
        out.append((widx, kind, arr))
    return out


IMAGENET_MEAN = (0.485, 0.456, 0.406)
IMAGENET_STD = (0.229, 0.224, 0.225)


def preprocess_image(img: np.ndarray, resize: int = 256, crop: int = 224,
                     mean: Iterable[float] = IMAGENET_MEAN, std: Iterable[float] = IMAGENET_STD) -> np.ndarray:
    """``img``: decoded image, ``[H, W, 3]`` uint8 (or float in [0, 255]).  Returns ``[3, crop, crop]``
    float32: shorter side resized to ``resize`` (bilinear, antialiased), centre crop, /255, normalised."""
    import torch
    import torch.nn.functional as F

    if img.ndim != 3 or img.shape[2] != 3:
        raise ValueError("expected an [H, W, 3] image")
    t = torch.from_numpy(np.ascontiguousarray(img, dtype=np.float32)).permute(2, 0, 1).unsqueeze(0)
    h, w = t.shape[2:]
    if h <= w:
        nh, nw = resize, max(resize, int(resize * w / h))
    else:
        nh, nw = max(resize, int(resize * h / w)), resize
    t = F.interpolate(t, size=(nh, nw), mode="bilinear", align_corners=False, antialias=True)
    top, left = int(round((nh - crop) / 2.0)), int(round((nw - crop) / 2.0))
    t = t[0, :, top:top + crop, left:left + crop] / 255.0
    m = torch.tensor(list(mean), dtype=torch.float32).view(3, 1, 1)
    s = torch.tensor(list(std), dtype=torch.float32).view(3, 1, 1)
    return ((t - m) / s).numpy().astype(np.float32)


def write_input_file(path: str, batch_nchw: np.ndarray) -> None:
    """Raw float32 ``[batch, C, H, W]`` file, the layout ``rpool_add_nasm`` converts to the library's
    channel-minor input matrix."""
    a = np.ascontiguousarray(batch_nchw, dtype=np.float32)
    if a.ndim != 4:
        raise ValueError("expected [batch, C, H, W]")
    a.tofile(path)


def nchw_to_dense(batch_nchw: np.ndarray) -> np.ndarray:
    """The same conversion on the Python side: ``[batch, C, H, W]`` -> ``[batch*H*W, C]``, the matrix
    ``rpool_add_nasm_raw_input`` takes."""
    a = np.ascontiguousarray(batch_nchw, dtype=np.float32)
    return np.ascontiguousarray(a.transpose(0, 2, 3, 1)).reshape(-1, a.shape[1])
