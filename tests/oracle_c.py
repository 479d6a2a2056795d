"""ctypes view of oracle/liberi_oracle.so for the tests (the checker, never the product)."""
import ctypes as C
import json
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
BLOCK = 2048
MODE_ERI, MODE_L2, MODE_BNB = 0, 1, 2
DT_F32, DT_BF16 = 0, 2


class Hyper(C.Structure):
    _fields_ = [("beta1", C.c_float), ("beta2", C.c_float), ("omb1", C.c_float),
                ("omb2", C.c_float), ("eps", C.c_float), ("weight_decay", C.c_float),
                ("step_size", C.c_float), ("bc1", C.c_float), ("bc2", C.c_float),
                ("grad_scale", C.c_float), ("mode", C.c_int32), ("use_grad_scale", C.c_int32)]


def load_maps():
    with open(os.path.join(ROOT, "tests", "golden", "dynamic_maps.json")) as f:
        j = json.load(f)
    s = np.array([int(x, 16) for x in j["signed"]], dtype=np.uint32).view(np.float32)
    u = np.array([int(x, 16) for x in j["unsigned"]], dtype=np.uint32).view(np.float32)
    return s, u


_lib = None


def lib():
    global _lib
    if _lib is None:
        so = os.path.join(ORACLE_DIR, "liberi_oracle.so")
        if not os.path.exists(so):
            subprocess.check_call(["make", "-C", ORACLE_DIR, "-s"])
        L = C.CDLL(so)
        L.eri_oracle_bf16_to_f32.restype = C.c_float
        L.eri_oracle_bf16_to_f32.argtypes = [C.c_uint16]
        L.eri_oracle_f32_to_bf16.restype = C.c_uint16
        L.eri_oracle_f32_to_bf16.argtypes = [C.c_float]
        L.eri_oracle_nearest_index.restype = C.c_int
        L.eri_oracle_nearest_index.argtypes = [C.c_void_p, C.c_float]
        L.eri_oracle_midpoints.argtypes = [C.c_void_p, C.c_void_p]
        L.eri_oracle_hyper_pack.argtypes = [C.c_double] * 5 + [C.c_uint64, C.c_int, C.POINTER(Hyper)]
        L.eri_oracle_step_tensor.restype = C.c_int
        L.eri_oracle_step_tensor.argtypes = [C.c_void_p] * 6 + [C.c_uint64, C.c_int, C.POINTER(Hyper),
                                                               C.c_void_p, C.c_void_p, C.c_int]
        L.eri_oracle_step_tensor_g.restype = C.c_int
        L.eri_oracle_step_tensor_g.argtypes = [C.c_void_p] * 6 + [C.c_uint64, C.c_int, C.c_int, C.POINTER(Hyper),
                                                                 C.c_void_p, C.c_void_p, C.c_int]
        L.eri_oracle_state_init.argtypes = [C.c_void_p] * 4 + [C.c_uint64]
        L.eri_oracle_dequantize.argtypes = [C.c_void_p] * 3 + [C.c_uint64, C.c_void_p]
        L.eri_oracle_quantize.argtypes = [C.c_void_p] * 2 + [C.c_uint64, C.c_void_p, C.c_void_p]
        L.eri_oracle_adamw32_step.argtypes = [C.c_void_p] * 4 + [C.c_uint64, C.c_int] + [C.c_float] * 5 + [C.c_void_p]
        L.eri_oracle_adamw32_step_scaled.argtypes = [C.c_void_p] * 4 + [C.c_uint64, C.c_int] + [C.c_float] * 5 + [C.c_void_p, C.c_float]
        L.eri_oracle_ema_update.argtypes = [C.c_void_p] * 2 + [C.c_uint64, C.c_int, C.c_float]
        L.eri_oracle_num_threads.restype = C.c_int
        _lib = L
    return _lib


def ptr(a):
    return a.ctypes.data_as(C.c_void_p)


def hyper_pack(lr, b1, b2, eps, wd, step, mode=MODE_ERI, grad_scale=None):
    h = Hyper()
    lib().eri_oracle_hyper_pack(lr, b1, b2, eps, wd, step, mode, C.byref(h))
    if grad_scale is not None:
        h.grad_scale = grad_scale
        h.use_grad_scale = 1
    return h


def midpoints(table):
    out = np.empty(255, np.float32)
    lib().eri_oracle_midpoints(ptr(np.ascontiguousarray(table, np.float32)), ptr(out))
    return out


def state_init(numel):
    nb = (numel + BLOCK - 1) // BLOCK
    m = np.empty(numel, np.uint8)
    v = np.empty(numel, np.uint8)
    am = np.empty(nb, np.float32)
    av = np.empty(nb, np.float32)
    lib().eri_oracle_state_init(ptr(m), ptr(v), ptr(am), ptr(av), numel)
    return m, v, am, av


def step_tensor(p, g, m, v, am, av, h, maps, dtype, threads=1, g_dtype=None):
    """In place on p, m, v, am, av (NumPy arrays: float32, or uint16 bit patterns for bf16).
    g_dtype: storage type of g when it differs from the parameter's (float32 gradients for bf16 parameters)."""
    s, u = maps
    for a in (p, g, m, v, am, av):
        assert a.flags["C_CONTIGUOUS"]
    return lib().eri_oracle_step_tensor_g(ptr(p), ptr(g), ptr(m), ptr(v), ptr(am), ptr(av), m.size, dtype,
                                          dtype if g_dtype is None else g_dtype, C.byref(h), ptr(s), ptr(u), threads)
