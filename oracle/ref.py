"""ctypes binding of oracle/_ref/libaspen_ref.so: the reference's own sources compiled in place
(see oracle/Makefile) behind oracle/ref_glue.c.  Test infrastructure; optional -- ``available()``
is False wherever the library was not built."""
from __future__ import annotations

import ctypes as C
import os
import subprocess
import tempfile

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_HERE, "_ref", "libaspen_ref.so")
_fp = C.POINTER(C.c_float)


def build() -> bool:
    """Compile the reference where it lies; only possible where /root/reference is mounted."""
    if not os.path.isdir("/root/reference/src"):
        return os.path.exists(_LIB)
    subprocess.check_call(["make", "-s", "-C", _HERE, "ref", "-j8"])
    return True


def available() -> bool:
    return os.path.exists(_LIB)


_lib = None


def lib():
    global _lib
    if _lib is None:
        L = C.CDLL(_LIB)
        L.refglue_open.restype = C.c_void_p
        L.refglue_open.argtypes = [C.c_char_p, C.c_char_p, C.c_uint, C.c_uint, C.c_uint, C.c_int]
        L.refglue_num_layers.argtypes = [C.c_void_p]
        L.refglue_num_ninst.argtypes = [C.c_void_p]
        L.refglue_layer_info.argtypes = [C.c_void_p, C.c_int, C.POINTER(C.c_uint)]
        L.refglue_set_input.argtypes = [C.c_void_p, _fp]
        L.refglue_forward.argtypes = [C.c_void_p]
        L.refglue_layer_copy.argtypes = [C.c_void_p, C.c_int, _fp]
        L.refglue_time_forward.argtypes = [C.c_void_p, C.c_int]
        L.refglue_time_forward.restype = C.c_double
        L.refglue_layer_weight.argtypes = [C.c_void_p, C.c_int, C.c_int, _fp, C.c_long]
        L.refglue_layer_weight.restype = C.c_long
        L.refglue_result.argtypes = [C.c_void_p, C.c_int, C.POINTER(C.c_int), C.c_int, _fp, C.c_long]
        L.refglue_result.restype = C.c_long
        L.refglue_save_dnn.argtypes = [C.c_void_p, C.c_char_p]
        L.refglue_save_nasm.argtypes = [C.c_void_p, C.c_uint, C.c_uint, C.c_uint, C.c_char_p]
        L.refglue_time_dse.argtypes = [C.c_void_p, C.c_uint, C.c_uint, C.c_uint, _fp, C.c_int, C.c_int, C.c_int, _fp, C.c_long]
        L.refglue_time_dse.restype = C.c_double
        L.refglue_close.argtypes = [C.c_void_p]
        _lib = L
    return _lib


class RefNet:
    """One reference dnn + nasm, executed layer-synchronously with the reference's tiled_* kernels."""

    def __init__(self, cfg_text: str, weight_path: str, batch: int, seq: int = 0, min_ninst: int = 100,
                 threads: int = 8):
        self._tmp = tempfile.NamedTemporaryFile("w", suffix=".cfg", delete=False)
        self._tmp.write(cfg_text)
        self._tmp.close()
        self.h = lib().refglue_open(self._tmp.name.encode(), weight_path.encode() if weight_path else None,
                                    batch, seq, min_ninst, threads)
        if not self.h:
            raise RuntimeError("reference failed to create the dnn")
        self.num_layers = lib().refglue_num_layers(self.h)
        self.num_ninst = lib().refglue_num_ninst(self.h)

    def info(self, l: int) -> dict:
        a = (C.c_uint * 10)()
        lib().refglue_layer_info(self.h, l, a)
        keys = ["type", "act", "H", "W", "stride", "num_ninst", "tile_H", "tile_W", "p0", "p1"]
        return dict(zip(keys, [int(v) for v in a]))

    def set_input(self, x: np.ndarray):
        x = np.ascontiguousarray(x, dtype=np.float32)
        i = self.info(0)
        assert x.size == i["H"] * i["W"], (x.size, i)
        lib().refglue_set_input(self.h, x.ctypes.data_as(_fp))

    def forward(self):
        lib().refglue_forward(self.h)

    def layer(self, l: int) -> np.ndarray:
        i = self.info(l)
        out = np.empty((i["W"], i["H"]), dtype=np.float32)
        lib().refglue_layer_copy(self.h, l, out.ctypes.data_as(_fp))
        return out

    def save_dnn(self, path: str):
        """The reference's apu_save_dnn_to_file."""
        lib().refglue_save_dnn(self.h, path.encode())

    def save_nasm(self, path: str, batch: int, seq: int, min_ninst: int) -> int:
        """apu_create_nasm (full dependency search) + apu_save_nasm_to_file; returns the tile count."""
        return lib().refglue_save_nasm(self.h, batch, seq, min_ninst, path.encode())

    def weight(self, l: int, tensor_type: int) -> np.ndarray:
        n = lib().refglue_layer_weight(self.h, l, tensor_type, None, 0)
        out = np.empty(n, dtype=np.float32)
        if n:
            lib().refglue_layer_weight(self.h, l, tensor_type, out.ctypes.data_as(_fp), n)
        return out

    def result(self, l: int, order) -> np.ndarray:
        i = self.info(l)
        out = np.empty(i["W"] * i["H"], dtype=np.float32)
        arr = (C.c_int * len(order))(*order)
        lib().refglue_result(self.h, l, arr, len(order), out.ctypes.data_as(_fp), out.nbytes)
        return out

    def time_forward(self, iters: int) -> float:
        return float(lib().refglue_time_forward(self.h, iters))

    def time_dse(self, x: np.ndarray, batch: int, seq: int, min_ninst: int, num_dse: int, warmup: int, iters: int):
        """The reference's own scheduler: apu_create_nasm (full dependency search) + the run loop of its main.c on
        num_dse DSE threads.  Returns (seconds per inference, final layer as [columns][rows])."""
        x = np.ascontiguousarray(x, dtype=np.float32)
        i = self.info(self.num_layers - 1)
        out = np.zeros((i["W"], i["H"]), dtype=np.float32)
        sec = float(lib().refglue_time_dse(self.h, batch, seq, min_ninst, x.ctypes.data_as(_fp), num_dse, warmup, iters,
                                           out.ctypes.data_as(_fp), out.size))
        if sec < 0:
            raise RuntimeError("the reference could not build the graph")
        return sec, out

    def close(self):
        if self.h:
            lib().refglue_close(self.h)
            self.h = None
            os.unlink(self._tmp.name)
