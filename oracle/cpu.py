"""ctypes binding of oracle/aspen_oracle.c plus a whole-network walker (test infrastructure).

The walker interprets the parsed cfg layer list (aspen_amd.models.parse_cfg) with the oracle's
per-layer functions and keeps every layer's dense output ``[W][H]`` (columns x channels), the
un-padded region of the reference's out_mat.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from typing import Dict, List

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_HERE, "_build", "liboracle.so")

ACT = {"none": 0, "linear": 0, "logistic": 1, "tanh": 3, "relu": 4, "leaky": 5, "elu": 6,
       "selu": 7, "gelu": 8, "gelu_acc": 9}

_fp = C.POINTER(C.c_float)
_u = C.c_uint


def build(force: bool = False) -> str:
    if force or not os.path.exists(_LIB) or os.path.getmtime(_LIB) < os.path.getmtime(
            os.path.join(_HERE, "aspen_oracle.c")):
        subprocess.check_call(["make", "-s", "-C", _HERE, "oracle"] + (["-B"] if force else []))
    return _LIB


_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = C.CDLL(build())
    return _lib


def _p(a: np.ndarray):
    assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(_fp)


def activate(x: np.ndarray, act: int) -> np.ndarray:
    y = np.ascontiguousarray(x, dtype=np.float32).copy()
    lib().oracle_activate(_p(y), _u(y.size), C.c_int(act))
    return y


def pack_weight(w: np.ndarray) -> np.ndarray:
    M, K = w.shape
    w = np.ascontiguousarray(w, dtype=np.float32)
    out = np.empty(((M + 7) // 8) * K * 8, dtype=np.float32)
    lib().oracle_pack_weight(_p(w), _p(out), _u(M), _u(K))
    return out


def conv_weight_to_hwc(w: np.ndarray) -> np.ndarray:
    OC, IC, KH, KW = w.shape
    w = np.ascontiguousarray(w, dtype=np.float32)
    out = np.empty((OC, KH * KW * IC), dtype=np.float32)
    lib().oracle_conv_weight_to_hwc(_p(w), _p(out), _u(OC), _u(IC), _u(KH), _u(KW))
    return out


def sgemm_packed(Ap: np.ndarray, B: np.ndarray, M: int, C0: np.ndarray = None) -> np.ndarray:
    N, K = B.shape
    out = np.zeros((N, M), dtype=np.float32) if C0 is None else C0.copy()
    lib().oracle_sgemm_packed(_u(M), _u(N), _u(K), _p(Ap), _u(K), _p(B), _u(K), _p(out), _u(M))
    return out


def conv2d(x, w_oihw, bias, B, IH, IW, stride, pad, act):
    OC, IC, KH, KW = w_oihw.shape
    Wp = pack_weight(conv_weight_to_hwc(w_oihw))
    OH = (IH + 2 * pad - KH) // stride + 1
    OW = (IW + 2 * pad - KW) // stride + 1
    out = np.empty((B * OH * OW, OC), dtype=np.float32)
    lib().oracle_conv2d(_p(x), _u(IC), _p(Wp), _p(bias) if bias is not None else None, _p(out), _u(OC),
                        _u(B), _u(IH), _u(IW), _u(IC), _u(OC), _u(KH), _u(KW), _u(stride), _u(pad), C.c_int(act))
    return out


def matmul(x, w, bias, act):
    M, K = w.shape
    N = x.shape[0]
    Wp = pack_weight(w)
    out = np.empty((N, M), dtype=np.float32)
    lib().oracle_matmul(_p(x), _u(K), _p(Wp), _p(bias) if bias is not None else None, _p(out), _u(M),
                        _u(M), _u(N), _u(K), C.c_int(act))
    return out


def fc(x, w_ochw, bias, B, act):
    OC, IC, IH, IW = w_ochw.shape
    w = np.ascontiguousarray(w_ochw.transpose(0, 2, 3, 1)).reshape(OC, IH * IW * IC)  # (h, w, c) flatten
    Wp = pack_weight(w)
    out = np.empty((B, OC), dtype=np.float32)
    lib().oracle_fc(_p(x), _u(IC), _p(Wp), _p(bias) if bias is not None else None, _p(out), _u(OC),
                    _u(B), _u(IH * IW), _u(IC), _u(OC), C.c_int(act))
    return out


def pool(kind, x, B, IH, IW, Cc, size, stride, pad, act):
    OH = (IH + 2 * pad - size) // stride + 1
    OW = (IW + 2 * pad - size) // stride + 1
    out = np.empty((B * OH * OW, Cc), dtype=np.float32)
    fn = lib().oracle_maxpool2d if kind == "maxpool" else lib().oracle_avgpool2d
    fn(_p(x), _u(Cc), _p(out), _u(Cc), _u(B), _u(IH), _u(IW), _u(Cc), _u(size), _u(size), _u(stride), _u(pad),
       C.c_int(act))
    return out


def residual(a, b, act):
    N, M = a.shape
    out = np.empty((N, M), dtype=np.float32)
    lib().oracle_residual(_p(a), _u(M), _p(b), _u(M), _p(out), _u(M), _u(M), _u(N), C.c_int(act))
    return out


def yolo(x, anchors, B, IH, IW, rows, stride):
    IC = x.shape[1]
    A = IC // rows
    out = np.empty((B * IH * IW * A, rows), dtype=np.float32)
    anchors = np.ascontiguousarray(anchors, dtype=np.float32)
    lib().oracle_yolo(_p(x), _u(IC), _p(out), _u(rows), _p(anchors), _u(B), _u(IH), _u(IW), _u(IC), _u(rows), _u(stride))
    return out


def append(a, b, B, OH, OW, stride):
    C0, C1 = a.shape[1], b.shape[1]
    out = np.empty((B * OH * OW, C0 + C1), dtype=np.float32)
    lib().oracle_append(_p(a), _u(C0), _p(b), _u(C1), _p(out), _u(C0 + C1), _u(B), _u(OH), _u(OW), _u(C0), _u(C1), _u(stride))
    return out


def softmax(x):
    N, M = x.shape
    out = np.empty((N, M), dtype=np.float32)
    lib().oracle_softmax(_p(x), _u(M), _p(out), _u(M), _u(M), _u(N))
    return out


def layernorm(x, w, b):
    N, M = x.shape
    out = np.empty((N, M), dtype=np.float32)
    lib().oracle_layernorm(_p(x), _u(M), _p(w), _p(b) if b is not None else None, _p(out), _u(M), _u(M), _u(N))
    return out


def k_attention(q, k, B, H, S, masked):
    hd = q.shape[1] // H
    out = np.empty((B * H * S, S), dtype=np.float32)
    lib().oracle_k_attention(_p(q), _u(q.shape[1]), _p(k), _u(k.shape[1]), _p(out), _u(S),
                             _u(B), _u(H), _u(S), _u(hd), C.c_int(masked))
    return out


def v_attention(p, v, B, H, S):
    hd = v.shape[1] // H
    out = np.empty((B * S, v.shape[1]), dtype=np.float32)
    lib().oracle_v_attention(_p(p), _u(S), _p(v), _u(v.shape[1]), _p(out), _u(v.shape[1]),
                             _u(B), _u(H), _u(S), _u(hd))
    return out


def run_network(layers: List[Dict], tensors, x_dense: np.ndarray, batch: int, seq: int,
                keep_all: bool = True) -> List[np.ndarray]:
    """Walk the layer list; returns per-layer dense outputs (None for freed ones when keep_all=False)."""
    wmap: Dict = {}
    for widx, kind, arr in tensors:
        wmap[(widx, kind)] = np.ascontiguousarray(arr, dtype=np.float32)
    outs: List[np.ndarray] = []
    widx = 0
    last_use = {}
    for L in layers:
        for p in (L.get("p0"), L.get("p1")):
            if p is not None:
                last_use[p] = L["idx"]
    for L in layers:
        t = L["type"]
        act = ACT[L["act"]]
        if t in ("conv", "fc", "matmul", "layernorm"):
            widx += 1
            w, b = wmap[(widx, "WEIGHT")], wmap.get((widx, "BIAS"))
        p0 = outs[L["p0"]] if L["p0"] is not None else None
        p1 = outs[L["p1"]] if L["p1"] is not None else None
        if t == "input":
            M = L["M"] or L["C"]
            o = np.ascontiguousarray(x_dense, dtype=np.float32).reshape(-1, M)
        elif t == "conv":
            o = conv2d(p0, w, b, batch, L["inH"], L["inW"], L["stride"], L["pad"], act)
        elif t in ("maxpool", "avgpool"):
            o = pool(t, p0, batch, L["inH"], L["inW"], L["inC"], L["size"], L["stride"], L["pad"], act)
        elif t == "yolo":
            o = yolo(p0, L["anchors"], batch, L["inH"], L["inW"], L["C"], L["stride"])
        elif t == "append":
            o = append(p0, p1, batch, L["H"], L["W"], L["stride"])
        elif t == "fc":
            o = fc(p0, w, b, batch, act)
        elif t == "residual":
            o = residual(p0, p1, act)
        elif t == "softmax":
            o = softmax(p0)
        elif t == "matmul":
            o = matmul(p0, w, b, act)
        elif t == "layernorm":
            o = layernorm(p0, w, b)
        elif t == "attn_k":
            o = k_attention(p0, p1, batch, L["n_head"], seq, L["masked"])
        elif t == "attn_v":
            o = v_attention(p0, p1, batch, L["n_head"], seq)
        else:
            raise ValueError(t)
        outs.append(o)
        if not keep_all:
            for p, lu in last_use.items():
                if lu == L["idx"] and p != len(layers) - 1:
                    outs[p] = None
    return outs
