"""Model descriptions (Darknet-style ``.cfg`` text) and seeded synthetic tensors.

The cfg dialect is the one the reference parses (reference
``src/darknet_parser.c:410-486``): ``[net]`` is the input layer, ``parent=`` /
``from=`` are relative layer offsets, ``M/K/n_head/n_embd/masked`` describe the
transformer layers.  The generators below emit that text from the network's
arithmetic description, so any depth/width can be produced for tests.

Synthetic tensors come from a counter-based splitmix64 stream so that the same
(seed, tensor id, element index) gives the same float on every machine and for
every consumer (the HIP library, the CPU oracle, the reference build).
Tensors are produced in PyTorch element order -- the order the reference's
weight file holds (reference ``src/apu_file_io.c:240-262``).
"""
from __future__ import annotations

import math
from typing import Dict, List, Tuple

import numpy as np

# ----------------------------------------------------------------------------
# cfg generators
# ----------------------------------------------------------------------------


def _conv(filters, size, stride, pad, act, parent=None):
    s = "[convolutional]\n"
    if parent is not None:
        s += f"parent={parent}\n"
    s += f"filters={filters}\nsize={size}\nstride={stride}\npad={pad}\nactivation={act}\n\n"
    return s


def resnet50_cfg(height=224, width=224, classes=1000, widths=(64, 128, 256, 512),
                 blocks=(3, 4, 6, 3), stem=64) -> str:
    """ResNet-50 v1.5 (stride 2 on the 3x3 conv); head = 7x7 avgpool + 1x1 conv."""
    s = f"[net]\nheight={height}\nwidth={width}\nchannels=3\n\n"
    s += _conv(stem, 7, 2, 3, "relu")
    s += "[maxpool]\nsize=3\nstride=2\npad=1\n\n"
    for stage, (w, nb) in enumerate(zip(widths, blocks)):
        for b in range(nb):
            stride = 2 if (b == 0 and stage > 0) else 1
            s += _conv(w, 1, 1, 0, "relu")
            s += _conv(w, 3, stride, 1, "relu")
            s += _conv(4 * w, 1, 1, 0, "linear")
            if b == 0:
                s += _conv(4 * w, 1, stride, 0, "linear", parent=-4)
                s += "[shortcut]\nfrom=-2\nactivation=relu\n\n"
            else:
                s += "[shortcut]\nfrom=-4\nactivation=relu\n\n"
    final_hw = height // 32
    s += f"[avgpool]\nsize={final_hw}\nstride=1\n\n"
    s += _conv(classes, 1, 1, 0, "linear")
    return s


def vgg16_cfg(height=224, width=224, classes=1000,
              plan=(64, 64, "M", 128, 128, "M", 256, 256, 256, "M", 512, 512, 512, "M", 512, 512, 512, "M"),
              fc=(4096, 4096)) -> str:
    s = f"[net]\nheight={height}\nwidth={width}\nchannels=3\n\n"
    for p in plan:
        if p == "M":
            s += "[maxpool]\nsize=2\nstride=2\n\n"
        else:
            s += _conv(p, 3, 1, 1, "relu")
    for f in fc:
        s += f"[connected]\noutput={f}\nactivation=relu\n\n"
    s += f"[connected]\noutput={classes}\nactivation=linear\n\n"
    return s


def _attn_block(n_embd, n_head, masked):
    hd = n_embd // n_head
    s = ""
    for parent in (None, -2, -3):  # Key, Query, Value all read the block input
        s += "[matmul]\n"
        if parent is not None:
            s += f"parent={parent}\n"
        s += f"M={n_embd}\nn_head={n_head}\nn_embd={n_embd}\n\n"
    s += f"[attention_k]\nparent=-2\nfrom=-3\nM=1\nK={hd}\nn_head={n_head}\nn_embd={n_embd}\n"
    if masked:
        s += "masked=1\n"
    s += "\n"
    s += f"[attention_v]\nfrom=-2\nM={n_embd}\nn_head={n_head}\nn_embd={n_embd}\n\n"
    s += f"[matmul]\nM={n_embd}\n\n"
    return s


def bert_cfg(n_layer=12, n_embd=768, n_head=12, ffn=3072) -> str:
    """Post-LN encoder: K,Q,V -> attn_k -> attn_v -> proj -> +x -> LN -> FFN -> +x -> LN."""
    s = f"[net]\nM={n_embd}\nheight=1\nfilters={n_embd}\n\n"
    for _ in range(n_layer):
        s += _attn_block(n_embd, n_head, masked=False)
        s += f"[shortcut]\nfrom=-7\nM={n_embd}\n\n"
        s += f"[layernorm]\nM={n_embd}\n\n"
        s += f"[matmul]\nM={ffn}\nactivation=gelu\n\n"
        s += f"[matmul]\nM={n_embd}\n\n"
        s += f"[shortcut]\nfrom=-3\nM={n_embd}\n\n"
        s += f"[layernorm]\nM={n_embd}\n\n"
    return s


def gpt2_cfg(n_layer=12, n_embd=768, n_head=12, ffn=3072) -> str:
    """Pre-LN causal decoder; no final LN, no LM head (as the reference's cfg)."""
    s = f"[net]\nM={n_embd}\nheight=1\nfilters={n_embd}\n\n"
    for _ in range(n_layer):
        s += f"[layernorm]\nM={n_embd}\n\n"
        s += _attn_block(n_embd, n_head, masked=True)
        s += f"[shortcut]\nfrom=-8\nM={n_embd}\n\n"
        s += f"[layernorm]\nM={n_embd}\n\n"
        s += f"[matmul]\nM={ffn}\nactivation=gelu_acc\n\n"
        s += f"[matmul]\nM={n_embd}\n\n"
        s += f"[shortcut]\nfrom=-4\nM={n_embd}\n\n"
    return s


def yolo_mini_cfg(size=32, classes=3) -> str:
    """A two-scale detector in the style of the reference's YOLO-v3 cfg (files/yolov3/yolov3_aspen.cfg):
    leaky convolutions, a detection head, a branch that is upsampled and appended to an earlier
    feature map, a second head."""
    rows = 3 * (classes + 5)
    anchors = "10,13,  16,30,  33,23,  30,61,  62,45,  59,119,  116,90,  156,198,  373,326"
    s = f"[net]\nheight={size}\nwidth={size}\nchannels=3\n\n"
    s += _conv(16, 3, 1, 1, "leaky") + _conv(32, 3, 2, 1, "leaky")          # 1, 2: size/2
    s += _conv(64, 3, 2, 1, "leaky") + _conv(32, 1, 1, 0, "leaky")          # 3, 4: size/4
    s += _conv(rows, 1, 1, 0, "linear")                                     # 5
    s += f"[yolo]\nmask = 6,7,8\nstride = 4\nanchors = {anchors}\nclasses={classes}\nnum=9\n\n"   # 6
    s += "[convolutional]\nparent=-3\nfilters=16\nsize=1\nstride=1\npad=0\nactivation=leaky\n\n"  # 7 (from 4)
    s += "[append]\nstride=2\nparent=-1\nfrom=-6\n\n"                    # 8: upsample 7, concat with 2
    s += _conv(32, 3, 1, 1, "leaky") + _conv(rows, 1, 1, 0, "linear")       # 9, 10
    s += f"[yolo]\nmask = 3,4,5\nstride = 2\nanchors = {anchors}\nclasses={classes}\nnum=9\n\n"   # 11
    return s


def yolov3_cfg(size=416, classes=80) -> str:
    """YOLO-v3: Darknet-53 backbone (1, 2, 8, 8, 4 residual blocks after the five stride-2 convolutions),
    three detection heads at strides 32 / 16 / 8; the two finer heads take a 1x1-reduced branch of the
    previous head, upsampled and appended to the backbone map of their scale.  Same section sequence as
    the reference's files/yolov3/yolov3_aspen.cfg ([append] instead of darknet's route + upsample)."""
    rows = 3 * (classes + 5)
    anchors = "10,13,  16,30,  33,23,  30,61,  62,45,  59,119,  116,90,  156,198,  373,326"
    s = f"[net]\nheight={size}\nwidth={size}\nchannels=3\n\n"
    s += _conv(32, 3, 1, 1, "leaky")
    n = 1                                   # sections so far after [net] = index of the next layer
    scale_end = {}                          # filters -> index of the last backbone layer at that width
    for f, blocks in ((64, 1), (128, 2), (256, 8), (512, 8), (1024, 4)):
        s += _conv(f, 3, 2, 1, "leaky"); n += 1
        for _ in range(blocks):
            s += _conv(f // 2, 1, 1, 0, "leaky") + _conv(f, 3, 1, 1, "leaky")
            s += "[shortcut]\nfrom=-3\nactivation=linear\n\n"
            n += 3
        scale_end[f] = n - 1
    for head, (f, mask, stride) in enumerate(((512, "6,7,8", 32), (256, "3,4,5", 16), (128, "0,1,2", 8))):
        if head > 0:
            # branch from the fifth convolution of the previous head (4 sections back), reduced,
            # upsampled twice and appended to the backbone map that has this head's resolution
            s += _conv(f, 1, 1, 0, "leaky", parent=-4); n += 1
            s += f"[append]\nstride=2\nparent=-1\nfrom={scale_end[2 * f] - n}\n\n"; n += 1
        for _ in range(3):
            s += _conv(f, 1, 1, 0, "leaky") + _conv(2 * f, 3, 1, 1, "leaky"); n += 2
        s += _conv(rows, 1, 1, 0, "linear"); n += 1
        s += f"[yolo]\nmask = {mask}\nstride = {stride}\nanchors = {anchors}\nclasses={classes}\nnum=9\n\n"; n += 1
    return s


def custom_cifar_cfg() -> str:
    """The small CIFAR-10 net of the reference's third example (conv5/pool/conv3/pool/3 FC)."""
    s = "[net]\nheight=32\nwidth=32\nchannels=3\n\n"
    s += _conv(32, 5, 1, 2, "relu") + "[maxpool]\nsize=2\nstride=2\n\n"
    s += _conv(64, 3, 1, 1, "relu") + "[maxpool]\nsize=2\nstride=2\n\n"
    s += "[connected]\noutput=256\nactivation=relu\n\n[connected]\noutput=128\nactivation=relu\n\n"
    s += "[connected]\noutput=10\nactivation=linear\n\n"
    return s


# ----------------------------------------------------------------------------
# cfg -> layer list (host-side mirror of the parser, used to size synthetic tensors)
# ----------------------------------------------------------------------------

_TYPES = {
    "[net]": "input", "[network]": "input", "[conv]": "conv", "[convolutional]": "conv",
    "[shortcut]": "residual", "[max]": "maxpool", "[maxpool]": "maxpool", "[avg]": "avgpool",
    "[avgpool]": "avgpool", "[conn]": "fc", "[connected]": "fc", "[soft]": "softmax",
    "[softmax]": "softmax", "[matmul]": "matmul", "[attention_k]": "attn_k",
    "[attention_v]": "attn_v", "[layernorm]": "layernorm", "[yolo]": "yolo", "[append]": "append",
}


def parse_cfg(text: str) -> List[Dict]:
    """Layer dictionaries with resolved parents and in/out shapes
    (reference ``src/darknet_parser.c:455-486`` and ``src/input_parser.c:35-127``)."""
    layers: List[Dict] = []
    cur = None
    for raw in text.splitlines():
        line = raw.strip()
        if not line or line[0] in "#;":
            continue
        if line.startswith("["):
            if line not in _TYPES:
                cur = None  # unsupported sections are dropped
                continue
            cur = {"type": _TYPES[line], "opts": {}}
            layers.append(cur)
        elif cur is not None and "=" in line:
            k, v = line.split("=", 1)
            cur["opts"][k.strip()] = v.strip()
    for i, L in enumerate(layers):
        o = L["opts"]
        gi = lambda k, d=0: int(o.get(k, d))
        L["idx"] = i
        L["act"] = o.get("activation", "none")
        L["p0"] = None if L["type"] == "input" else (i + gi("parent") if gi("parent") else i - 1)
        L["p1"] = i + gi("from") if gi("from") else None
        L["size"], L["stride"], L["pad"] = gi("size"), max(gi("stride"), 1), gi("pad")
        L["M"], L["K"] = gi("M"), gi("K")
        L["n_head"], L["n_embd"], L["masked"] = gi("n_head"), gi("n_embd"), gi("masked")
        if L["type"] == "input":
            if L["M"]:
                L["C"], L["H"], L["W"] = L["M"], 1, 0
            else:
                L["C"], L["H"], L["W"] = gi("channels"), gi("height"), gi("width")
            continue
        P = layers[L["p0"]]
        L["inC"], L["inH"], L["inW"] = P["C"], P["H"], P["W"]
        t = L["type"]
        if t == "conv":
            L["C"] = gi("filters")
            L["H"] = (P["H"] + 2 * L["pad"] - (L["size"] - 1) - 1) // L["stride"] + 1
            L["W"] = (P["W"] + 2 * L["pad"] - (L["size"] - 1) - 1) // L["stride"] + 1
        elif t in ("maxpool", "avgpool"):
            L["C"] = P["C"]
            L["H"] = (P["H"] + 2 * L["pad"] - (L["size"] - 1) - 1) // L["stride"] + 1
            L["W"] = (P["W"] + 2 * L["pad"] - (L["size"] - 1) - 1) // L["stride"] + 1
        elif t == "yolo":
            # rows = classes + 5; one output column per (anchor, cell); the layer's three anchors are
            # picked from the anchor list by `mask` (reference src/darknet_parser.c:487-545)
            L["C"] = gi("classes") + 5
            L["H"], L["W"] = 1, P["H"] * P["W"] * (P["C"] // L["C"])
            mask = [int(v) for v in o["mask"].split(",")]
            anch = [float(v) for v in o["anchors"].split(",")]
            L["anchors"] = np.array([anch[2 * m + k] for m in mask[:3] for k in (0, 1)], dtype=np.float32)
        elif t == "append":
            Q = layers[L["p1"]]
            L["C"], L["H"], L["W"] = P["C"] + Q["C"], P["H"] * L["stride"], P["W"] * L["stride"]
        elif t == "fc":
            L["C"], L["H"], L["W"] = gi("output") or gi("filters"), 1, 1
        elif t == "softmax":
            L["C"], L["H"], L["W"] = P["C"], 1, 1
        elif t == "residual":
            L["C"], L["H"], L["W"] = (L["M"], 1, 0) if L["M"] else (P["C"], P["H"], P["W"])
        elif t in ("matmul", "layernorm", "attn_v"):
            L["C"], L["H"], L["W"] = L["M"], 1, 0
            if t == "matmul":
                L["K"] = P["M"] if P["type"] != "input" else P["C"]
        elif t == "attn_k":
            L["C"], L["H"], L["W"] = 0, 1, 0  # rows = seq_len, known at graph build
            L["K"] = L["n_embd"] // L["n_head"]
    return layers


# ----------------------------------------------------------------------------
# deterministic tensors
# ----------------------------------------------------------------------------

_U64 = np.uint64
_GOLD = _U64(0x9E3779B97F4A7C15)


def _mix(x: np.ndarray) -> np.ndarray:
    with np.errstate(over="ignore"):
        z = x + _GOLD
        z = (z ^ (z >> _U64(30))) * _U64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> _U64(27))) * _U64(0x94D049BB133111EB)
        return z ^ (z >> _U64(31))


def _stream(seed: int, tensor_id: int, n: int, lane: int) -> np.ndarray:
    """n uniform floats in [0,1) with 24 random bits each (exactly representable in fp32)."""
    with np.errstate(over="ignore"):
        base = _mix(np.array([seed], dtype=_U64) * _U64(0xD1342543DE82EF95)
                    + _U64(tensor_id) * _U64(0xA0761D6478BD642F) + _U64(lane))
        z = _mix(base + np.arange(n, dtype=_U64) * _GOLD)
    return ((z >> _U64(40)).astype(np.float64) * (1.0 / (1 << 24))).astype(np.float32)


def uniform(seed: int, tensor_id: int, shape) -> np.ndarray:
    n = int(np.prod(shape))
    return _stream(seed, tensor_id, n, 0).reshape(shape)


def normal(seed: int, tensor_id: int, shape, std: float, mean: float = 0.0) -> np.ndarray:
    n = int(np.prod(shape))
    u1 = _stream(seed, tensor_id, n, 1).astype(np.float64)
    u2 = _stream(seed, tensor_id, n, 2).astype(np.float64)
    r = np.sqrt(-2.0 * np.log(1.0 - u1))  # 1-u1 in (0,1]
    z = r * np.cos(2.0 * math.pi * u2)
    return (mean + std * z).astype(np.float32).reshape(shape)


Tensor = Tuple[int, str, np.ndarray]  # (1-based weighted-layer index, "WEIGHT"/"BIAS", data)


def synth_weights(layers: List[Dict], seed: int, style: str) -> List[Tensor]:
    """style "he": conv/FC ~ N(0, 2/fan_in), bias ~ N(0, 0.01^2) (stands in for folded BN);
    style "yolo": the same with two damped kinds of convolution, see below;
    style "gpt": matmul W,b ~ N(0, 0.02^2), layernorm w = 1 + N(0, 0.02^2), b ~ N(0, 0.02^2)."""
    out: List[Tensor] = []
    widx = 0
    for L in layers:
        t = L["type"]
        if t not in ("conv", "fc", "matmul", "layernorm"):
            continue
        widx += 1
        tid = 2 * widx
        if t == "conv":
            shp = (L["C"], L["inC"], L["size"], L["size"])
            fan = L["inC"] * L["size"] * L["size"]
        elif t == "fc":
            shp = (L["C"], L["inC"], L["inH"], L["inW"])
            fan = L["inC"] * L["inH"] * L["inW"]
        elif t == "matmul":
            shp = (L["M"], L["K"])
            fan = L["K"]
        else:
            shp = (L["M"],)
            fan = 1
        if t == "layernorm":
            w = normal(seed, tid, shp, 0.02, 1.0)
            b = normal(seed, tid + 1, shp, 0.02)
        elif style in ("he", "yolo"):
            gain = 1.0
            if style == "yolo":
                # 23 unnormalised residual additions would double the variance 23 times and the box decode
                # exponentiates its input: damp the branch that closes a residual block and the
                # convolution that feeds a detection layer
                nxt = layers[L["idx"] + 1]["type"] if L["idx"] + 1 < len(layers) else None
                gain = 0.3 if nxt == "residual" else (0.1 if nxt == "yolo" else 1.0)
            w = normal(seed, tid, shp, gain * math.sqrt(2.0 / fan))
            b = normal(seed, tid + 1, (shp[0],), 0.01)
        elif style == "gpt":
            w = normal(seed, tid, shp, 0.02)
            b = normal(seed, tid + 1, (shp[0],), 0.02)
        else:
            raise ValueError(style)
        out.append((widx, "WEIGHT", w))
        out.append((widx, "BIAS", b))
    return out


def write_aspen_data(path: str, tensors: List[Tensor]) -> None:
    """``ASPEN_DATA`` weight file (format: reference ``src/apu_file_io.c:48-432``)."""
    with open(path, "wb") as f:
        f.write(b"ASPEN_DATA\n")
        for widx, kind, arr in tensors:
            raw = np.ascontiguousarray(arr, dtype=np.float32).tobytes()
            f.write(f"LAYER:{widx}\nTENSOR_TYPE:{kind}\nDATA_SIZE:{len(raw)}\nDATA_START:\n".encode())
            f.write(raw)
            f.write(b"DATA_END\nLAYER_END\n")


# ----------------------------------------------------------------------------
# the five benchmark configurations
# ----------------------------------------------------------------------------

CONFIGS = {
    # name: (cfg generator, weight style, batch, seq, seed, transformer input kind)
    "resnet50_b1": (resnet50_cfg, "he", 1, 0, 101, None),
    "resnet50_b32": (resnet50_cfg, "he", 32, 0, 101, None),
    "vgg16_b32": (vgg16_cfg, "he", 32, 0, 202, None),
    "resnet50_b16": (resnet50_cfg, "he", 16, 0, 101, None),
    "vgg16_b16": (vgg16_cfg, "he", 16, 0, 202, None),
    "yolov3_b1": (yolov3_cfg, "yolo", 1, 0, 505, None),
    "yolov3_b8": (yolov3_cfg, "yolo", 8, 0, 505, None),
    "bert_base_b8_s128": (bert_cfg, "gpt", 8, 128, 303, "embeddings"),
    "gpt2_b4_s512": (gpt2_cfg, "gpt", 4, 512, 404, "token_ids"),
}

# The graphs the benchmark times AND the full-size parity tests check (one table, so they cannot drift apart):
#   name: (configurations co-run in one ready pool, unit, units per step, tiles wanted per layer, engine)
# The last two entries are what the library's timing tuner (apu_generate_nasm: candidate tile counts on both
# engines) settles on for the configuration, fixed here so that a run does not spend its time tuning; the
# reference ships its tile graphs tuned per model and batch in the same way.
WORKLOADS = {
    "resnet50_b32": (["resnet50_b32"], "img/s", 32, 1536, "dataflow"),
    "resnet50_b1": (["resnet50_b1"], "img/s", 1, 256, "dataflow"),
    "vgg16_b32": (["vgg16_b32"], "img/s", 32, 1536, "dataflow"),
    "co_resnet50_vgg16_b16": (["resnet50_b16", "vgg16_b16"], "img/s", 32, 1536, "dataflow"),
    # the two halves of the co-scheduled pair on their own: what back-to-back runs would take
    "resnet50_b16": (["resnet50_b16"], "img/s", 16, 1536, "dataflow"),
    "vgg16_b16": (["vgg16_b16"], "img/s", 16, 1536, "dataflow"),
    "bert_base_b8_s128": (["bert_base_b8_s128"], "tokens/s", 8 * 128, 192, "dataflow"),
    "gpt2_b4_s512": (["gpt2_b4_s512"], "tokens/s", 4 * 512, 384, "dataflow"),
    # (engine "dataflow-ordered": the persistent kernel, its ordered mode asked for with Nasm.set_ordered)
    "yolov3_b1": (["yolov3_b1"], "img/s", 1, 768, "dataflow-ordered"),
    "yolov3_b8": (["yolov3_b8"], "img/s", 8, 1536, "dataflow"),
}


def make_config(name: str):
    """(cfg text, parsed layers, weight tensors, dense input, batch, seq) of a named configuration."""
    gen, style, batch, seq, seed, kind = CONFIGS[name]
    cfg = gen()
    layers = parse_cfg(cfg)
    return cfg, layers, synth_weights(layers, seed, style), synth_input(layers, seed, batch, seq, kind), batch, seq


def synth_input(layers: List[Dict], seed: int, batch: int, seq: int, kind: str = "token_ids") -> np.ndarray:
    """Dense network input in the layout ``rpool_add_nasm_raw_input`` takes:
    NHWC for images (uniform [0,1)), ``[batch][seq][M]`` for transformers.

    Transformer kind "embeddings": rows ~ N(0, 0.02^2) fed directly.  Kind
    "token_ids": ids uniform in [0, 50257) select rows of a seeded N(0, 0.02^2) table (wte) and a position
    table (wpe) is added; the lookup happens here, outside the graph, because
    the reference graph starts at the float matrix (its cfg has no embedding)."""
    L0 = layers[0]
    if L0["M"]:
        M = L0["M"]
        if kind == "embeddings":
            return normal(seed, 1_000_004, (batch, seq, M), 0.02)
        ids = (uniform(seed, 1_000_001, (batch, seq)).astype(np.float64) * 50257).astype(np.int64)
        # wte rows generated on demand: row r = normal stream with tensor id derived from r
        uniq, inv = np.unique(ids, return_inverse=True)
        rows = np.stack([normal(seed, 2_000_000 + int(r), (M,), 0.02) for r in uniq])
        wpe = normal(seed, 1_000_002, (seq, M), 0.02)
        x = rows[inv.reshape(-1)].reshape(batch, seq, M) + wpe[None]
        return np.ascontiguousarray(x, dtype=np.float32)
    nchw = uniform(seed, 1_000_003, (batch, L0["C"], L0["H"], L0["W"]))
    return np.ascontiguousarray(nchw.transpose(0, 2, 3, 1))
