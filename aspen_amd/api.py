"""ctypes mirror of ``include/aspen.h`` (+ ``aspen_ext.h`` / ``aspen_hip.h``).

Function names, argument order and ownership are those of the C API, which in turn are those of
the reference's ``aspen.h``; the small classes below only pair every ``*_create``/``*_init`` with
its ``*_destroy`` and turn result buffers into numpy arrays.  There is no CPU fallback: every
compute call goes through ``libaspen_amd.so`` and raises if the library is missing.
"""
from __future__ import annotations

import ctypes as C
import os
import tempfile
from typing import Optional, Sequence

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("ASPEN_AMD_LIB", os.path.join(_HERE, "libaspen_amd.so"))

# enum values of include/aspen.h
(OUT_W, OUT_H, OUT_C, BATCH, IN_W, IN_H, IN_C, WEIGHT_W, WEIGHT_H, SUB_C, STRIDE, PADDING, DILATION, GROUPS,
 NUM_HIDDEN, NUM_HEAD, NUM_SEQ, MAT_M, MAT_N, MAT_K, SUB_M, MASKED, FORM_BYTES, NUM_PARAM_ELEMENTS) = range(24)
(NO_LAYER_TYPE, INPUT_LAYER, CONV_LAYER, FC_LAYER, RESIDUAL_LAYER, BATCHNORM_LAYER, YOLO_LAYER, APPEND_LAYER,
 ACTIVATION_LAYER, MAXPOOL_LAYER, AVGPOOL_LAYER, ROUTE_LAYER, SOFTMAX_LAYER, MATMUL_LAYER, LAYERNORM_LAYER,
 K_ATTENTION_LAYER, V_ATTENTION_LAYER) = range(17)
LAYER_TYPE_NAMES = ["none", "input", "conv", "fc", "residual", "batchnorm", "yolo", "append", "activation",
                    "maxpool", "avgpool", "route", "softmax", "matmul", "layernorm", "attn_k", "attn_v"]
(NO_ACTIVATION, SIGMOID, LINEAR, TANH, RELU, LEAKY_RELU, ELU, SELU, GELU, GELU_ACCURATE) = range(10)

MODE_LAYERS, MODE_DATAFLOW, MODE_AUTO = 0, 1, 2

_vp = C.c_void_p
_fp = C.POINTER(C.c_float)
_u32p = C.POINTER(C.c_uint32)
_lib = None


def lib() -> C.CDLL:
    """Loads the in-tree shared library; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(f"{LIB_PATH} is missing: run `python -m aspen_amd.build` (or __graft_entry__.build())")
    L = C.CDLL(LIB_PATH)
    sig = {
        "apu_create_dnn": (_vp, [C.c_char_p, C.c_char_p]),
        "apu_destroy_dnn": (None, [_vp]),
        "apu_create_nasm": (_vp, [_vp, C.c_uint, C.c_uint]),
        "apu_create_transformer_nasm": (_vp, [_vp, C.c_uint, C.c_uint, C.c_uint]),
        "apu_generate_nasm": (_vp, [_vp, C.c_uint, C.c_uint]),
        "apu_generate_transformer_nasm": (_vp, [_vp, C.c_uint, C.c_uint, C.c_uint]),
        "apu_destroy_nasm": (None, [_vp]),
        "apu_reset_nasm": (None, [_vp]),
        "apu_load_nasm_from_file": (_vp, [C.c_char_p, _vp]),
        "apu_save_nasm_to_file": (None, [_vp, C.c_char_p]),
        "apu_save_dnn_to_file": (None, [_vp, C.c_char_p]),
        "apu_load_dnn_from_file": (_vp, [C.c_char_p]),
        "rpool_init": (_vp, []),
        "rpool_destroy": (None, [_vp]),
        "rpool_add_nasm_raw_input": (None, [_vp, _vp, _vp]),
        "rpool_add_nasm": (None, [_vp, _vp, C.c_char_p]),
        "rpool_reset_queue": (None, [_vp]),
        "rpool_reset_nasm": (None, [_vp, _vp]),
        "dse_group_init": (_vp, [C.c_uint]),
        "dse_group_set_rpool": (None, [_vp, _vp]),
        "dse_group_destroy": (None, [_vp]),
        "dse_group_run": (None, [_vp]),
        "dse_group_stop": (None, [_vp]),
        "dse_group_run_until_nasm_completion": (None, [_vp, _vp]),
        "dse_wait_for_nasm_completion": (None, [_vp]),
        "dse_check_nasm_completion": (C.c_uint, [_vp]),
        "dse_get_ldata_result": (C.c_ssize_t, [_vp, C.c_uint, C.POINTER(C.c_int), C.POINTER(_vp)]),
        "dse_get_nasm_result": (C.c_ssize_t, [_vp, C.POINTER(C.c_int), C.POINTER(_vp)]),
        "aspen_flush_dynamic_memory": (None, []),
        "print_nasm_info": (None, [_vp, C.c_int, C.c_int]),
        "print_dnn_info": (None, [_vp, C.c_int]),
        "print_rpool_info": (None, [_vp]),
        # aspen_ext.h
        "aspen_dse_group_set_mode": (None, [_vp, C.c_int]),
        "aspen_dse_group_last_mode": (C.c_int, [_vp]),
        "aspen_dse_group_last_run_ordered": (C.c_int, [_vp]),
        "aspen_nasm_set_ordered": (None, [_vp, C.c_int]),
        "aspen_dse_group_set_spin_limit": (None, [_vp, C.c_uint64]),
        "aspen_dse_group_set_workgroups": (None, [_vp, C.c_uint]),
        "aspen_keep_layer_outputs": (None, [C.c_int]),
        "apu_load_dnn_data_from_file": (None, [_vp, C.c_char_p]),
        "aspen_dnn_device_generation": (C.c_uint, [_vp]),
        "aspen_nasm_num_ldata": (C.c_uint, [_vp]),
        "aspen_nasm_num_ninst": (C.c_uint, [_vp]),
        "aspen_nasm_num_edges": (C.c_uint, [_vp]),
        "aspen_nasm_total_flops": (C.c_uint64, [_vp]),
        "aspen_nasm_ldata_flops": (C.c_uint64, [_vp, C.c_uint]),
        "aspen_nasm_ldata_info": (None, [_vp, C.c_uint, C.POINTER(C.c_uint)]),
        "aspen_nasm_graph": (None, [_vp, C.POINTER(_u32p), C.POINTER(_u32p), C.POINTER(_u32p), C.POINTER(_u32p)]),
        "aspen_nasm_tile_range": (None, [_vp, C.c_uint, C.POINTER(C.c_uint)]),
        "aspen_rpool_run_stats": (C.c_int, [_vp, _u32p, _u32p, _u32p]),
        "aspen_rpool_num_ninst": (C.c_uint, [_vp]),
        "aspen_rpool_profile_layers": (C.c_int, [_vp, C.c_uint, _fp]),
        "aspen_rpool_dataflow_profile": (C.c_int, [_vp, C.POINTER(C.c_uint64), C.c_int]),
        "aspen_rpool_dataflow_trace": (C.c_int, [_vp, _vp]),
        "aspen_rpool_debug_set_epoch": (C.c_int, [_vp, C.c_uint32]),
        "aspen_rpool_dataflow_trace_phases": (C.c_int, [_vp, _vp]),
        # aspen_hip.h
        "aspen_hip_init": (C.c_int, []),
        "aspen_hip_last_error": (C.c_char_p, []),
        "aspen_hip_device_info": (C.c_int, [C.POINTER(C.c_int), C.POINTER(C.c_int), C.POINTER(C.c_size_t), C.c_char_p, C.c_int]),
        "aspen_hip_alloc": (_vp, [C.c_size_t]),
        "aspen_hip_free": (None, [_vp]),
        "aspen_hip_h2d": (C.c_int, [_vp, _vp, C.c_size_t]),
        "aspen_hip_d2h": (C.c_int, [_vp, _vp, C.c_size_t]),
        "aspen_hip_copy": (C.c_int, [_vp, _vp, C.c_size_t]),
        "aspen_hip_zero": (C.c_int, [_vp, C.c_size_t]),
        "aspen_hip_sync": (C.c_int, []),
        "aspen_hip_graph_sync": (C.c_int, [_vp]),
        "aspen_hip_set_flags": (None, [C.c_uint32]),
        "aspen_hip_idle": (C.c_int, []),
        "aspen_hip_event_record": (C.c_int, [C.c_int]),
        "aspen_hip_event_elapsed_ms": (C.c_int, [C.c_int, C.c_int, _fp]),
        "aspen_hip_sgemm": (C.c_int, [C.c_uint32, C.c_uint32, C.c_uint32, _vp, C.c_uint32, _vp, C.c_uint32, _vp,
                                      C.c_uint32, _vp, C.c_int]),
        "aspen_hip_sgemm_static": (C.c_int, [C.c_uint32, C.c_uint32, C.c_uint32, _vp, C.c_uint32, _vp, C.c_uint32, _vp,
                                             C.c_uint32, _vp, C.c_int]),
        "aspen_hip_sgemm_static_max_bytes": (C.c_size_t, []),
    }
    for name, (res, args) in sig.items():
        fn = getattr(L, name)
        fn.restype = res
        fn.argtypes = args
    libc = C.CDLL(None)
    libc.free.argtypes = [_vp]
    L._free = libc.free
    _lib = L
    return L


def gpu_available() -> bool:
    """True when the library loads and finds a HIP device."""
    try:
        return lib().aspen_hip_init() == 0
    except (OSError, RuntimeError):
        return False


def device_info() -> dict:
    cu, khz, mem = C.c_int(), C.c_int(), C.c_size_t()
    name = C.create_string_buffer(256)
    if lib().aspen_hip_device_info(C.byref(cu), C.byref(khz), C.byref(mem), name, 256):
        raise RuntimeError(lib().aspen_hip_last_error().decode())
    return {"name": name.value.decode(), "compute_units": cu.value, "clock_khz": khz.value, "memory_bytes": mem.value}


class Dnn:
    """``aspen_dnn_t`` -- ``apu_create_dnn`` / ``apu_destroy_dnn``."""

    def __init__(self, cfg_text: Optional[str] = None, weight_path: Optional[str] = None, cfg_path: Optional[str] = None):
        self._tmp = None
        if cfg_path is None:
            f = tempfile.NamedTemporaryFile("w", suffix=".cfg", delete=False)
            f.write(cfg_text)
            f.close()
            cfg_path = self._tmp = f.name
        self.h = lib().apu_create_dnn(cfg_path.encode(), weight_path.encode() if weight_path else None)
        if self._tmp:
            os.unlink(self._tmp)
        if not self.h:
            raise ValueError("apu_create_dnn failed")

    def destroy(self):
        if self.h:
            lib().apu_destroy_dnn(self.h)
            self.h = None


class Nasm:
    """``nasm_t`` -- ``apu_create_nasm`` / ``apu_create_transformer_nasm`` / ``apu_destroy_nasm``."""

    def __init__(self, dnn: Dnn, batch: int, seq: int = 0, min_ninst: int = 512, generate_iters: Optional[int] = None):
        """``generate_iters`` not None: ``apu_generate_nasm`` / ``apu_generate_transformer_nasm`` (the tile count
        is chosen by timing that many candidates beyond the default on the GPU) instead of ``min_ninst``."""
        self.dnn = dnn
        if generate_iters is not None:
            self.h = (lib().apu_generate_transformer_nasm(dnn.h, batch, seq, generate_iters) if seq
                      else lib().apu_generate_nasm(dnn.h, batch, generate_iters))
        elif seq:
            self.h = lib().apu_create_transformer_nasm(dnn.h, min_ninst, batch, seq)
        else:
            self.h = lib().apu_create_nasm(dnn.h, min_ninst, batch)
        if not self.h:
            raise ValueError("apu_create_nasm failed")
        self.batch, self.seq = batch, seq
        self.num_ldata = lib().aspen_nasm_num_ldata(self.h)
        self.num_ninst = lib().aspen_nasm_num_ninst(self.h)
        self.num_edges = lib().aspen_nasm_num_edges(self.h)
        self.total_flops = lib().aspen_nasm_total_flops(self.h)

    def info(self, l: int) -> dict:
        a = (C.c_uint * 20)()
        lib().aspen_nasm_ldata_info(self.h, l, a)
        keys = ["type", "act", "H", "W", "stride", "num_ninst", "tile_H", "tile_W", "p0", "p1", "ninst_start", "variant",
                "fused_into", "fused_residual", "splits", "tiles_H", "kiters_per_split", "discarded", "fused_attention", "folded_norm"]
        d = dict(zip(keys, [int(v) for v in a]))
        for k in ("fused_into", "fused_residual", "fused_attention", "folded_norm"):
            d[k] = -1 if d[k] == 0xffffffff else d[k]
        d["flops"] = int(lib().aspen_nasm_ldata_flops(self.h, l))
        return d

    def set_ordered(self, ordered: int):
        """1 / 0: runs on the persistent kernel use / do not use its ordered mode; -1: the engine decides."""
        lib().aspen_nasm_set_ordered(self.h, ordered)

    def graph(self):
        """(tile -> layer, parent counts, child offsets, child indices) as numpy copies."""
        p = [_u32p() for _ in range(4)]
        lib().aspen_nasm_graph(self.h, *[C.byref(x) for x in p])
        n, e = self.num_ninst, self.num_edges
        mk = lambda ptr, cnt: np.ctypeslib.as_array(ptr, shape=(max(cnt, 1),))[:cnt].copy()
        return mk(p[0], n), mk(p[1], n), mk(p[2], n + 1), mk(p[3], e)

    def tile_range(self, idx: int):
        a = (C.c_uint * 4)()
        lib().aspen_nasm_tile_range(self.h, idx, a)
        return tuple(int(v) for v in a)

    def layer_output(self, l: int, order: Optional[Sequence[int]] = None) -> np.ndarray:
        """``dse_get_ldata_result``; default = native order, returned as [columns][rows]."""
        i = self.info(l)
        out = _vp()
        arr = (C.c_int * 8)(*(list(order) + [0] * (8 - len(order)))) if order is not None else None
        n = lib().dse_get_ldata_result(self.h, l, arr, C.byref(out))
        if n < 0:
            raise RuntimeError("dse_get_ldata_result failed")
        a = np.ctypeslib.as_array(C.cast(out, _fp), shape=(n // 4,)).copy()
        lib()._free(out)
        return a.reshape(i["W"], i["H"]) if order is None else a

    def result(self, order: Optional[Sequence[int]] = None) -> np.ndarray:
        return self.layer_output(self.num_ldata - 1, order)

    def destroy(self):
        if self.h:
            lib().apu_destroy_nasm(self.h)
            self.h = None


class RPool:
    def __init__(self):
        self.h = lib().rpool_init()

    def add_nasm_raw_input(self, nasm: Nasm, x: Optional[np.ndarray]):
        if x is not None:
            x = np.ascontiguousarray(x, dtype=np.float32)
            i = nasm.info(0)
            if x.size != i["H"] * i["W"]:
                raise ValueError(f"input has {x.size} floats, layer 0 holds {i['H'] * i['W']}")
        lib().rpool_add_nasm_raw_input(self.h, nasm.h, x.ctypes.data_as(_vp) if x is not None else None)

    def reset_queue(self):
        lib().rpool_reset_queue(self.h)

    def reset_nasm(self, nasm: Nasm):
        lib().rpool_reset_nasm(self.h, nasm.h)

    def run_stats(self) -> dict:
        a, b, c = C.c_uint32(), C.c_uint32(), C.c_uint32()
        if lib().aspen_rpool_run_stats(self.h, C.byref(a), C.byref(b), C.byref(c)):
            raise RuntimeError("no dataflow run to report on")
        return {"executed": a.value, "double_runs": b.value, "aborted": c.value}

    def debug_set_epoch(self, epoch: int):
        if lib().aspen_rpool_debug_set_epoch(self.h, epoch):
            raise RuntimeError("the pool has no device graph yet")

    def dataflow_profile(self, reset: bool = True) -> dict:
        """Summed workgroup time of dataflow runs since the last reset, in seconds (profile flag 4)."""
        t = (C.c_uint64 * 16)()
        if lib().aspen_rpool_dataflow_profile(self.h, t, 1 if reset else 0):
            raise RuntimeError("no dataflow profile")
        d = {k: t[i] * 1e-8 for i, k in enumerate(["tile", "drain", "sched", "total", "publish", "ticket", "slot_wait"])}
        for i, k in enumerate(["gemm_first_loads", "gemm_kloop", "gemm_epilogue", "gemm_splitk", "gemm_init"]):
            d[k] = t[8 + i] * 1e-8
        d["engine_clock_mhz"] = t[7] / max(t[3], 1) * 100.0
        return d

    def dataflow_trace(self) -> np.ndarray:
        """[tiles][2] start / end stamps (100 MHz ticks) of the last run made with the trace flag (8)."""
        n = lib().aspen_rpool_num_ninst(self.h)
        t = np.zeros((n, 2), dtype=np.uint64)
        if lib().aspen_rpool_dataflow_trace(self.h, t.ctypes.data):
            raise RuntimeError("no dataflow trace: " + lib().aspen_hip_last_error().decode())
        return t

    def dataflow_trace_phases(self) -> np.ndarray:
        """[tiles][2] end-of-K-loop / stores-issued stamps of the contraction tiles of the same traced run."""
        n = lib().aspen_rpool_num_ninst(self.h)
        t = np.zeros((n, 2), dtype=np.uint64)
        if lib().aspen_rpool_dataflow_trace_phases(self.h, t.ctypes.data):
            raise RuntimeError("no dataflow trace: " + lib().aspen_hip_last_error().decode())
        return t

    def profile_layers(self, num_layers: int, iters: int = 5) -> np.ndarray:
        """Per-layer kernel time in ms (layer-launch mode, HIP events); the pool must have run once."""
        ms = np.zeros(num_layers, dtype=np.float32)
        if lib().aspen_rpool_profile_layers(self.h, iters, ms.ctypes.data_as(_fp)):
            raise RuntimeError("profile_layers failed: " + lib().aspen_hip_last_error().decode())
        return ms

    def destroy(self):
        if self.h:
            lib().rpool_destroy(self.h)
            self.h = None


class DseGroup:
    def __init__(self, num_dse: int = 1, mode: Optional[int] = None, workgroups: int = 0):
        self.h = lib().dse_group_init(num_dse)
        if mode is not None:
            lib().aspen_dse_group_set_mode(self.h, mode)
        if workgroups:
            lib().aspen_dse_group_set_workgroups(self.h, workgroups)

    def set_mode(self, mode: int):
        lib().aspen_dse_group_set_mode(self.h, mode)

    def last_mode(self) -> int:
        """The engine the last run() used: MODE_LAYERS or MODE_DATAFLOW (-1 before the first run)."""
        return lib().aspen_dse_group_last_mode(self.h)

    def last_run_ordered(self) -> bool:
        return lib().aspen_dse_group_last_run_ordered(self.h) == 1

    def set_rpool(self, rpool: RPool):
        lib().dse_group_set_rpool(self.h, rpool.h)

    def run(self):
        lib().dse_group_run(self.h)

    def stop(self):
        lib().dse_group_stop(self.h)

    @staticmethod
    def wait(nasm: Nasm):
        lib().dse_wait_for_nasm_completion(nasm.h)

    @staticmethod
    def check(nasm: Nasm) -> bool:
        """``dse_check_nasm_completion``: True once THIS nasm has finished, whatever the pool's others do."""
        return lib().dse_check_nasm_completion(nasm.h) == 1

    def destroy(self):
        if self.h:
            lib().dse_group_destroy(self.h)
            self.h = None
