"""ctypes binding of liberi_optim8.so (the C ABI declared in include/eri_optim8.h).

The library is built in-tree by `make -C eridiffusion_amd/csrc` (or __graft_entry__.build()).
There is no fallback: if the shared object is missing or a call fails, this module raises.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "liberi_optim8.so")

BLOCK = 2048
DTYPE_F32, DTYPE_F16, DTYPE_BF16, DTYPE_I32 = 0, 1, 2, 3
MODE_ERI, MODE_L2, MODE_BNB = 0, 1, 2
FLAG_GRAD_SCALE, FLAG_EXACT_PARAM, FLAG_BSEARCH, FLAG_NO_PIPELINE, FLAG_CLIP_FROM_TABLE, FLAG_ONE_WAVE, FLAG_EMA = 1, 2, 4, 8, 16, 32, 64


class Hyper(C.Structure):
    _fields_ = [("beta1", C.c_float), ("beta2", C.c_float), ("omb1", C.c_float), ("omb2", C.c_float),
                ("eps", C.c_float), ("weight_decay", C.c_float), ("step_size", C.c_float),
                ("bc1", C.c_float), ("bc2", C.c_float), ("grad_scale", C.c_float),
                ("mode", C.c_int32), ("flags", C.c_uint32), ("ema_decay", C.c_float), ("reserved", C.c_uint32)]


class TensorRow(C.Structure):
    _fields_ = [("p", C.c_void_p), ("g", C.c_void_p), ("m", C.c_void_p), ("v", C.c_void_p),
                ("absmax_m", C.c_void_p), ("absmax_v", C.c_void_p), ("numel", C.c_uint64),
                ("block_start", C.c_uint64), ("dtype_tag", C.c_int32), ("grad_scale", C.c_float),
                ("p_src", C.c_void_p), ("grad_f32", C.c_int32), ("reserved", C.c_int32), ("ema_shadow", C.c_void_p)]


class Adam8bitConfigC(C.Structure):
    _fields_ = [("lr", C.c_double), ("beta1", C.c_double), ("beta2", C.c_double), ("eps", C.c_double),
                ("weight_decay", C.c_double), ("amsgrad", C.c_int32), ("block_wise", C.c_int32),
                ("percentile_clipping", C.c_uint64)]


class AdamW32Row(C.Structure):
    _fields_ = [("p", C.c_void_p), ("g", C.c_void_p), ("m", C.c_void_p), ("v", C.c_void_p), ("master", C.c_void_p),
                ("numel", C.c_uint64), ("dtype_tag", C.c_int32), ("grad_scale", C.c_float)]


class AdamW32Hyper(C.Structure):
    _fields_ = [("lr", C.c_float), ("beta1", C.c_float), ("beta2", C.c_float), ("eps", C.c_float),
                ("weight_decay", C.c_float)]


class EmaRow(C.Structure):
    _fields_ = [("shadow", C.c_void_p), ("p", C.c_void_p), ("numel", C.c_uint64), ("dtype_tag", C.c_int32),
                ("reserved", C.c_int32)]


class MemoryReportC(C.Structure):
    _fields_ = [("num_params", C.c_uint64), ("param_memory_gb", C.c_double), ("state_memory_gb", C.c_double),
                ("total_memory_gb", C.c_double), ("memory_reduction_percent", C.c_double), ("has_reduction", C.c_int32),
                ("description", C.c_char * 44)]


class EriError(RuntimeError):
    def __init__(self, what, code, message):
        super().__init__("%s failed with code %d: %s" % (what, code, message))
        self.code = code
        self.message = message


EXPORTS = {
    # name: (restype, argtypes)
    "eri_last_error": (C.c_char_p, []),
    "eri_set_last_error": (None, [C.c_char_p]),
    "eri_hip_get_device": (C.c_int, [C.POINTER(C.c_int)]),
    "eri_hip_device_count": (C.c_int, [C.POINTER(C.c_int)]),
    "eri_hip_set_device": (C.c_int, [C.c_int]),
    "eri_hip_malloc_zeroed": (C.c_int, [C.c_int, C.c_size_t, C.POINTER(C.c_void_p)]),
    "eri_hip_free": (C.c_int, [C.c_void_p]),
    "eri_hip_host_alloc": (C.c_void_p, [C.c_size_t]),
    "eri_hip_host_free": (C.c_int, [C.c_void_p]),
    "eri_hip_memcpy_async": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int, C.c_void_p]),
    "eri_hip_memset_async": (C.c_int, [C.c_void_p, C.c_int, C.c_size_t, C.c_void_p]),
    "eri_hip_stream_create": (C.c_int, [C.POINTER(C.c_void_p)]),
    "eri_hip_stream_sync": (C.c_int, [C.c_void_p]),
    "eri_hip_stream_destroy": (C.c_int, [C.c_void_p]),
    "eri_hip_mem_info": (C.c_int, [C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]),
    "eri_hip_pointer_kind": (C.c_int, [C.c_void_p, C.POINTER(C.c_int)]),
    "eri_hip_pool_create": (C.c_int, [C.c_int, C.c_size_t, C.c_uint32, C.POINTER(C.c_void_p)]),
    "eri_hip_pool_alloc_zeroed": (C.c_int, [C.c_void_p, C.c_uint32, C.c_size_t, C.POINTER(C.c_void_p)]),
    "eri_hip_pool_alloc_zeroed_async": (C.c_int, [C.c_void_p, C.c_uint32, C.c_size_t, C.c_void_p, C.POINTER(C.c_void_p)]),
    "eri_hip_pool_release": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t]),
    "eri_hip_pool_retain": (C.c_int, [C.c_void_p]),
    "eri_hip_pool_unretain": (C.c_int, [C.c_void_p]),
    "eri_hip_pool_info": (C.c_int, [C.c_void_p, C.POINTER(C.c_uint32), C.POINTER(C.c_size_t)]),
    "eri_hip_pool_lane_used": (C.c_int, [C.c_void_p, C.c_uint32, C.POINTER(C.c_size_t)]),
    "eri_hip_pool_reset": (C.c_int, [C.c_void_p]),
    "eri_hip_pool_destroy": (C.c_int, [C.c_void_p]),
    "eri_adam8_init": (C.c_int, []),
    "eri_adam8_get_maps": (C.c_int, [C.c_void_p, C.c_void_p]),
    "eri_adam8_table_image": (C.c_int, [C.c_void_p, C.c_size_t, C.POINTER(C.c_size_t), C.POINTER(C.c_uint32)]),
    "eri_adam8_hyper_pack": (C.c_int, [C.c_double] * 5 + [C.c_uint64, C.c_int, C.c_uint32, C.POINTER(Hyper)]),
    "eri_adam8_state_init": (C.c_int, [C.c_void_p] * 4 + [C.c_uint64, C.c_void_p]),
    "eri_adam8_table_create": (C.c_int, [C.POINTER(TensorRow), C.c_uint32, C.c_void_p, C.POINTER(C.c_void_p)]),
    "eri_adam8_table_update": (C.c_int, [C.c_void_p, C.POINTER(TensorRow), C.c_uint32, C.c_void_p]),
    "eri_adam8_table_destroy": (C.c_int, [C.c_void_p]),
    "eri_adam8_table_info": (C.c_int, [C.c_void_p, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]),
    "eri_adam8_step_table": (C.c_int, [C.c_void_p, C.POINTER(Hyper), C.c_void_p]),
    "eri_adam8_grad_norm": (C.c_int, [C.c_void_p, C.c_float, C.c_float, C.c_void_p]),
    "eri_adam8_grad_table_create": (C.c_int, [C.POINTER(TensorRow), C.c_uint32, C.c_void_p, C.POINTER(C.c_void_p)]),
    "eri_adam8_grad_norm_joint": (C.c_int, [C.c_void_p, C.c_void_p, C.c_float, C.c_float, C.c_void_p]),
    "eri_adam8_grad_norm_scale_ptr": (C.c_int, [C.c_void_p, C.POINTER(C.c_void_p)]),
    "eri_adam8_grad_norm_static": (C.c_int, [C.c_void_p, C.c_float, C.c_float, C.c_void_p, C.c_void_p]),
    "eri_adam8_grad_norm_read": (C.c_int, [C.c_void_p, C.POINTER(C.c_float), C.POINTER(C.c_float), C.c_void_p]),
    "eri_adam8_grad_nonfinite_read": (C.c_int, [C.c_void_p, C.POINTER(C.c_uint64), C.c_void_p]),
    "eri_adam8_traffic_probe": (C.c_int, [C.c_void_p, C.c_void_p]),
    "eri_adam8_quant_error": (C.c_int, [C.c_void_p, C.POINTER(Hyper), C.c_void_p]),
    "eri_adam8_quant_error_read": (C.c_int, [C.c_void_p, C.POINTER(C.c_float), C.POINTER(C.c_float), C.c_void_p]),
    "eri_adam8_step_multi": (C.c_int, [C.POINTER(TensorRow), C.c_uint32, C.POINTER(Hyper), C.c_void_p]),
    "eri_adam8_dequantize": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_uint64, C.c_void_p, C.c_void_p]),
    "eri_adam8_quantize": (C.c_int, [C.c_void_p, C.c_int, C.c_uint64, C.c_void_p, C.c_void_p, C.c_void_p]),
    "eri_adamw32_step_multi": (C.c_int, [C.POINTER(AdamW32Row), C.c_uint32, C.POINTER(AdamW32Hyper), C.c_void_p]),
    "eri_adamw32_step_multi_scaled": (C.c_int, [C.POINTER(AdamW32Row), C.c_uint32, C.POINTER(AdamW32Hyper), C.c_float,
                                              C.c_void_p, C.c_void_p]),
    "eri_ema_update_multi": (C.c_int, [C.POINTER(EmaRow), C.c_uint32, C.c_float, C.c_void_p]),
    # ---- include/eri_adam8bit.h
    "eri_param_create": (C.c_int, [C.c_void_p, C.c_uint64, C.c_int, C.POINTER(C.c_void_p)]),
    "eri_param_set_grad": (C.c_int, [C.c_void_p, C.c_void_p]),
    "eri_param_set_grad_typed": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int]),
    "eri_param_set_data": (C.c_int, [C.c_void_p, C.c_void_p]),
    "eri_param_retain": (C.c_int, [C.c_void_p]),
    "eri_param_release": (C.c_int, [C.c_void_p]),
    "eri_adam8bit_config_default": (None, [C.POINTER(Adam8bitConfigC)]),
    "eri_adam8bit_new": (C.c_int, [C.POINTER(C.c_void_p), C.c_uint32, C.POINTER(Adam8bitConfigC), C.c_void_p,
                                   C.POINTER(C.c_void_p)]),
    "eri_adam8bit_destroy": (C.c_int, [C.c_void_p]),
    "eri_adam8bit_step": (C.c_int, [C.c_void_p, C.POINTER(C.c_uint32)]),
    "eri_adam8bit_zero_grad": (C.c_int, [C.c_void_p]),
    "eri_adam8bit_current_lr": (C.c_double, [C.c_void_p]),
    "eri_adam8bit_set_learning_rate": (C.c_int, [C.c_void_p, C.c_double]),
    "eri_adam8bit_quantized_memory_usage": (C.c_uint64, [C.c_void_p]),
    "eri_adam8bit_get_step": (C.c_uint64, [C.c_void_p]),
    "eri_adam8bit_set_grad_scale": (C.c_int, [C.c_void_p, C.c_float]),
    "eri_adam8bit_set_param_grad_scale": (C.c_int, [C.c_void_p, C.c_uint32, C.c_float]),
    "eri_adam8bit_attach_ema": (C.c_int, [C.c_void_p, C.c_void_p, C.POINTER(C.c_char_p), C.c_uint32]),
    "eri_adam8bit_set_min_8bit_size": (C.c_int, [C.c_void_p, C.c_uint64]),
    "eri_adam8bit_set_state_pool": (C.c_int, [C.c_void_p, C.c_void_p, C.c_uint32]),
    "eri_adam8bit_state32_ptrs": (C.c_int, [C.c_void_p, C.c_uint32, C.POINTER(C.c_void_p), C.POINTER(C.c_void_p)]),
    "eri_adam8bit_set_max_grad_norm": (C.c_int, [C.c_void_p, C.c_float, C.c_float]),
    "eri_ema_new": (C.c_int, [C.c_float, C.c_int, C.c_float, C.c_void_p, C.POINTER(C.c_void_p)]),
    "eri_ema_destroy": (C.c_int, [C.c_void_p]),
    "eri_ema_init_from_params": (C.c_int, [C.c_void_p, C.POINTER(C.c_char_p), C.POINTER(C.c_void_p), C.c_uint32]),
    "eri_ema_update": (C.c_int, [C.c_void_p, C.POINTER(C.c_char_p), C.POINTER(C.c_void_p), C.c_uint32]),
    "eri_ema_copy_to": (C.c_int, [C.c_void_p, C.POINTER(C.c_char_p), C.POINTER(C.c_void_p), C.c_uint32]),
    "eri_ema_step": (C.c_uint64, [C.c_void_p]),
    "eri_ema_set_step": (C.c_int, [C.c_void_p, C.c_uint64]),
    "eri_ema_current_decay": (C.c_float, [C.c_void_p]),
    "eri_ema_num_shadows": (C.c_uint32, [C.c_void_p]),
    "eri_ema_shadow": (C.c_int, [C.c_void_p, C.c_char_p, C.POINTER(C.c_void_p), C.POINTER(C.c_uint64), C.POINTER(C.c_int)]),
    "eri_analyze_optimizer_memory": (C.c_int, [C.c_uint64, C.c_char_p, C.POINTER(MemoryReportC)]),
    "eri_ema_decay_from_half_life": (C.c_float, [C.c_uint64]),
    "eri_ema_decay_from_window": (C.c_float, [C.c_uint64]),
    "eri_ema_effective_decay": (C.c_float, [C.c_float, C.c_uint64, C.c_float, C.c_int]),
    "eri_adam8bit_set_mode": (C.c_int, [C.c_void_p, C.c_int]),
    "eri_adam8bit_last_grad_norm": (C.c_int, [C.c_void_p, C.POINTER(C.c_float), C.POINTER(C.c_float)]),
    "eri_adam8bit_last_nonfinite_grads": (C.c_int, [C.c_void_p, C.POINTER(C.c_uint64)]),
    "eri_adam8bit_track_quantization_error": (C.c_int, [C.c_void_p, C.c_int]),
    "eri_adam8bit_quantization_stats": (C.c_int, [C.c_void_p, C.POINTER(C.c_float), C.POINTER(C.c_float)]),
    "eri_adam8bit_set_flags": (C.c_int, [C.c_void_p, C.c_uint32]),
    "eri_adam8bit_save_state": (C.c_int, [C.c_void_p, C.c_char_p]),
    "eri_adam8bit_load_state": (C.c_int, [C.c_void_p, C.c_char_p]),
    "eri_adam8bit_load_legacy_state": (C.c_int, [C.c_void_p, C.c_char_p]),
    "eri_adam8bit_state_ptrs": (C.c_int, [C.c_void_p, C.c_uint32] + [C.POINTER(C.c_void_p)] * 4),
    "eri_adam8bit_fn_with_params": (C.c_int, [C.c_double] * 5 + [C.c_void_p, C.POINTER(C.c_void_p)]),
    "eri_adam8bit_fn_destroy": (C.c_int, [C.c_void_p]),
    "eri_adam8bit_fn_update": (C.c_int, [C.c_void_p, C.c_char_p, C.c_void_p, C.c_void_p, C.c_uint64, C.c_int, C.c_int, C.c_void_p]),
    "eri_adam8bit_fn_set_batching": (C.c_int, [C.c_void_p, C.c_int]),
    "eri_adam8bit_fn_set_state_pool": (C.c_int, [C.c_void_p, C.c_void_p, C.c_uint32]),
    "eri_adam8bit_fn_flush": (C.c_int, [C.c_void_p]),
    "eri_adam8bit_fn_update_many": (C.c_int, [C.c_void_p, C.POINTER(C.c_char_p), C.POINTER(C.c_void_p), C.POINTER(C.c_void_p),
                                              C.POINTER(C.c_uint64), C.POINTER(C.c_int32), C.POINTER(C.c_int32),
                                              C.POINTER(C.c_void_p), C.c_uint32]),
    "eri_adam8bit_fn_step": (C.c_int, [C.c_void_p]),
    "eri_adam8bit_fn_set_lr": (C.c_int, [C.c_void_p, C.c_float]),
    "eri_adam8bit_fn_get_step": (C.c_uint64, [C.c_void_p]),
    "eri_adam8bit_fn_table_stats": (C.c_int, [C.c_void_p, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]),
    "eri_adam8bit_fn_memory_stats": (C.c_int, [C.c_void_p, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]),
    "eri_adam8bit_fn_state_numel": (C.c_int, [C.c_void_p, C.c_char_p, C.POINTER(C.c_uint64)]),
    "eri_adam8bit_fn_get_state_fp32": (C.c_int, [C.c_void_p, C.c_char_p, C.c_void_p, C.c_void_p]),
    "eri_adam8bit_fn_load_state_fp32": (C.c_int, [C.c_void_p, C.c_char_p, C.c_void_p, C.c_void_p, C.c_uint64]),
}

_lib = None


def lib():
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("%s is missing: build it with `make -C eridiffusion_amd/csrc` "
                               "(there is no CPU or PyTorch fallback)" % LIB_PATH)
        try:  # PyTorch ships its own copy of the HIP runtime: when both live in one process the library
            import torch  # noqa: F401  must bind to that copy, so torch is loaded first (two runtimes crash)
        except ImportError:
            pass
        L = C.CDLL(LIB_PATH)
        for name, (res, args) in EXPORTS.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def check(code, what):
    if code != 0:
        raise EriError(what, code, lib().eri_last_error().decode("utf-8", "replace"))


def hyper_pack(lr, beta1, beta2, eps, weight_decay, step, mode=MODE_ERI, flags=0, grad_scale=None):
    h = Hyper()
    check(lib().eri_adam8_hyper_pack(lr, beta1, beta2, eps, weight_decay, step, mode, flags, C.byref(h)),
          "eri_adam8_hyper_pack")
    if grad_scale is not None:
        h.grad_scale = grad_scale
        h.flags |= FLAG_GRAD_SCALE
    return h
