"""Python face of the optimizer objects declared in include/eri_adam8bit.h.

`Adam8bit` keeps the method set of EriDiffusion's list-of-parameters optimizer
(src/trainers/adam8bit_enhanced.rs:160-369: new / step / zero_grad / current_lr /
set_learning_rate / quantized_memory_usage / save_state / load_state), `Adam8bitConfig` its
configuration (:372-395), and `Adam8bitFunctional` the per-tensor flavour
(src/trainers/adam8bit.rs:49-345: with_params / update / step / set_lr / get_step / memory_stats /
get_state_as_tensors / load_state_from_tensors).  Every method forwards to the C functions of the
same name; torch supplies device memory and the current stream, nothing else.
"""
import ctypes as C
from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

import torch

from ._lib import DTYPE_BF16, DTYPE_F32, Adam8bitConfigC, check, lib


def _dtype_tag(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return DTYPE_F32
    if t.dtype == torch.bfloat16:
        return DTYPE_BF16
    raise TypeError("Unsupported: 8-bit Adam takes float32 or bfloat16 parameters, got %s" % t.dtype)


def _usable_grad(g: torch.Tensor, p: torch.Tensor) -> torch.Tensor:
    """The gradient as the step reads it.  A float32 gradient of a bfloat16 parameter goes in as it is: the
    reference casts gradients to F32 and never rounds them (adam8bit_enhanced.rs:231-235).  Any other
    mismatch is cast to the parameter's dtype, which for bf16 -> f32 is exact."""
    if g.dtype != p.dtype and not (p.dtype == torch.bfloat16 and g.dtype == torch.float32):
        g = g.to(p.dtype)
    return g.contiguous()


def _stream_ptr() -> int:
    return torch.cuda.current_stream().cuda_stream


class DevicePool:
    """One device allocation cut into equal lanes (eri_hip_pool_*): tensors of different kinds taken from
    different lanes lie far apart in device memory, which is what the optimizer step wants of its 8-bit states
    and the parameters.  alloc_ptr() returns the device address of zero-filled, 256-byte aligned pool memory; the
    pool must outlive every use of it (an optimizer given the pool keeps it alive)."""

    def __init__(self, nbytes: int = 0, lanes: int = 0, device: int = 0):
        self._pool = C.c_void_p()
        check(lib().eri_hip_pool_create(device, nbytes, lanes, C.byref(self._pool)), "eri_hip_pool_create")
        n, b = C.c_uint32(), C.c_size_t()
        check(lib().eri_hip_pool_info(self._pool, C.byref(n), C.byref(b)), "eri_hip_pool_info")
        self.lanes, self.lane_bytes = n.value, b.value

    def alloc_ptr(self, lane: int, nbytes: int) -> int:
        out = C.c_void_p()
        check(lib().eri_hip_pool_alloc_zeroed(self._pool, lane, nbytes, C.byref(out)), "eri_hip_pool_alloc_zeroed")
        return out.value

    def reset(self) -> None:
        check(lib().eri_hip_pool_reset(self._pool), "eri_hip_pool_reset")

    def close(self) -> None:
        if self._pool:
            lib().eri_hip_pool_destroy(self._pool)
            self._pool = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


@dataclass
class Adam8bitConfig:
    """adam8bit_enhanced.rs:372-395; amsgrad, block_wise and percentile_clipping are carried only."""
    lr: float = 1e-3
    betas: Tuple[float, float] = (0.9, 0.999)
    eps: float = 1e-8
    weight_decay: float = 0.01
    amsgrad: bool = False
    block_wise: bool = True
    percentile_clipping: int = 99
    min_8bit_size: int = 0  # pipeline_flux_lora_1024.rs:451 passes 4096; 0 keeps every parameter 8-bit


class Adam8bit:
    """`step()` over a list of tensors that carry their gradients in `.grad`."""

    def __init__(self, params: List[torch.Tensor], config: Optional[Adam8bitConfig] = None, flags: Optional[int] = None):
        config = config or Adam8bitConfig()
        self.params = list(params)
        for p in self.params:
            if not p.is_contiguous():
                raise ValueError("parameters must be contiguous")
        self._handles = (C.c_void_p * len(self.params))()
        for i, p in enumerate(self.params):
            h = C.c_void_p()
            check(lib().eri_param_create(p.data_ptr(), p.numel(), _dtype_tag(p), C.byref(h)), "eri_param_create")
            self._handles[i] = h
        cfg = Adam8bitConfigC(config.lr, config.betas[0], config.betas[1], config.eps, config.weight_decay,
                              int(config.amsgrad), int(config.block_wise), config.percentile_clipping)
        self._opt = C.c_void_p()
        check(lib().eri_adam8bit_new(self._handles, len(self.params), C.byref(cfg), _stream_ptr(),
                                     C.byref(self._opt)), "eri_adam8bit_new")
        if flags is not None:  # None keeps the library's default, FLAG_EXACT_PARAM; 0 selects the faster arithmetic
            check(lib().eri_adam8bit_set_flags(self._opt, flags), "eri_adam8bit_set_flags")
        if config.min_8bit_size:
            check(lib().eri_adam8bit_set_min_8bit_size(self._opt, config.min_8bit_size), "eri_adam8bit_set_min_8bit_size")
        self._live = []

    def step(self) -> int:
        """One optimizer step; returns how many parameters were skipped for lack of a gradient."""
        live = []
        for i, p in enumerate(self.params):
            g = p.grad
            if g is not None:
                g = _usable_grad(g, p)
                live.append(g)
            check(lib().eri_param_set_data(self._handles[i], p.data_ptr()), "eri_param_set_data")
            if g is None:
                check(lib().eri_param_set_grad(self._handles[i], None), "eri_param_set_grad")
            else:
                check(lib().eri_param_set_grad_typed(self._handles[i], g.data_ptr(), _dtype_tag(g)),
                      "eri_param_set_grad_typed")
        self._live = live  # cast gradients must outlive the launch
        skipped = C.c_uint32()
        check(lib().eri_adam8bit_step(self._opt, C.byref(skipped)), "eri_adam8bit_step")
        return skipped.value

    def zero_grad(self) -> None:
        check(lib().eri_adam8bit_zero_grad(self._opt), "eri_adam8bit_zero_grad")
        for p in self.params:
            p.grad = None

    def current_lr(self) -> float:
        return lib().eri_adam8bit_current_lr(self._opt)

    def set_learning_rate(self, lr: float) -> None:
        check(lib().eri_adam8bit_set_learning_rate(self._opt, lr), "eri_adam8bit_set_learning_rate")

    def set_grad_scale(self, scale: float) -> None:
        check(lib().eri_adam8bit_set_grad_scale(self._opt, scale), "eri_adam8bit_set_grad_scale")

    def set_mode(self, mode: int) -> None:
        """MODE_ERI (the reference's update, default) or MODE_BNB."""
        check(lib().eri_adam8bit_set_mode(self._opt, mode), "eri_adam8bit_set_mode")

    def set_state_pool(self, pool: Optional[DevicePool], lane: int = 0) -> None:
        """States created from now on (at the first step of their parameter) come out of `lane` of the pool."""
        check(lib().eri_adam8bit_set_state_pool(self._opt, pool._pool if pool else None, lane), "eri_adam8bit_set_state_pool")
        self._pool = pool  # keeps the pool alive as long as the optimizer

    def attach_ema(self, ema: Optional["EMAModel"], names: Optional[List[str]] = None) -> None:
        """From now on every step() also performs ema.update() over this optimizer's parameters (names[i] is the
        model's name for parameter i): one launch instead of two sweeps.  attach_ema(None) detaches."""
        if ema is None:
            check(lib().eri_adam8bit_attach_ema(self._opt, None, None, 0), "eri_adam8bit_attach_ema")
            self._ema = None
            return
        arr = (C.c_char_p * len(self.params))(*[n.encode() for n in names])
        check(lib().eri_adam8bit_attach_ema(self._opt, ema._ema, arr, len(self.params)), "eri_adam8bit_attach_ema")
        self._ema = ema  # keeps the model alive as long as it is attached

    def set_max_grad_norm(self, max_norm: float, denom_eps: float = 0.0) -> None:
        """Global-norm clipping inside step(): norm on the device, factor applied by the step kernel
        (clip_gradients, src/trainers/pipeline_flux_lora_sequential.rs:1198-1213).  <= 0 switches it off."""
        check(lib().eri_adam8bit_set_max_grad_norm(self._opt, max_norm, denom_eps), "eri_adam8bit_set_max_grad_norm")

    def last_grad_norm(self) -> Tuple[float, float]:
        """(norm, clip factor) of the last step that clipped; waits for the stream."""
        n, s = C.c_float(), C.c_float()
        check(lib().eri_adam8bit_last_grad_norm(self._opt, C.byref(n), C.byref(s)), "eri_adam8bit_last_grad_norm")
        return n.value, s.value

    def last_nonfinite_grads(self) -> int:
        """NaN / infinite gradient elements seen by the norm pass of the last step that clipped."""
        c = C.c_uint64()
        check(lib().eri_adam8bit_last_nonfinite_grads(self._opt, C.byref(c)), "eri_adam8bit_last_nonfinite_grads")
        return c.value

    def track_quantization_error(self, enabled: bool = True) -> None:
        check(lib().eri_adam8bit_track_quantization_error(self._opt, int(enabled)),
              "eri_adam8bit_track_quantization_error")

    def quantization_stats(self) -> Tuple[float, float]:
        """adam8bit_enhanced.rs:318-327: mean absolute quantisation error of (first, second) moments."""
        m, v = C.c_float(), C.c_float()
        check(lib().eri_adam8bit_quantization_stats(self._opt, C.byref(m), C.byref(v)),
              "eri_adam8bit_quantization_stats")
        return m.value, v.value

    def quantized_memory_usage(self) -> int:
        return lib().eri_adam8bit_quantized_memory_usage(self._opt)

    def get_step(self) -> int:
        return lib().eri_adam8bit_get_step(self._opt)

    def save_state(self, path: str) -> None:
        check(lib().eri_adam8bit_save_state(self._opt, str(path).encode()), "eri_adam8bit_save_state")

    def load_state(self, path: str) -> None:
        check(lib().eri_adam8bit_load_state(self._opt, str(path).encode()), "eri_adam8bit_load_state")

    def close(self) -> None:
        if self._opt:
            lib().eri_adam8bit_destroy(self._opt)
            self._opt = C.c_void_p()
            for h in self._handles:
                lib().eri_param_release(h)

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Adam8bitFunctional:
    """Per-tensor flavour keyed by name: update() returns the new parameter tensor, step() ends the step
    (adam8bit.rs:89-92,101-208).

    batched=False: every update() is one kernel launch and its result is valid at once.
    batched=True: update() queues, and one launch over everything queued runs at step() / flush(); the
    tensors update() returned are filled then.  Inputs are kept alive until that launch."""

    def __init__(self, learning_rate=1e-4, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.01, batched=False):
        self._opt = C.c_void_p()
        check(lib().eri_adam8bit_fn_with_params(learning_rate, beta1, beta2, eps, weight_decay, _stream_ptr(),
                                                C.byref(self._opt)), "eri_adam8bit_fn_with_params")
        self._names: List[str] = []
        self._live: List[torch.Tensor] = []
        self._launched = False
        self._batched = bool(batched)
        if batched:
            check(lib().eri_adam8bit_fn_set_batching(self._opt, 1), "eri_adam8bit_fn_set_batching")

    @classmethod
    def with_params(cls, learning_rate, beta1, beta2, eps, weight_decay):
        return cls(learning_rate, beta1, beta2, eps, weight_decay)

    def set_state_pool(self, pool: Optional[DevicePool], lane: int = 0) -> None:
        """States of names not seen yet come out of `lane` of the pool."""
        check(lib().eri_adam8bit_fn_set_state_pool(self._opt, pool._pool if pool else None, lane), "eri_adam8bit_fn_set_state_pool")
        self._pool = pool

    def step(self) -> None:
        check(lib().eri_adam8bit_fn_step(self._opt), "eri_adam8bit_fn_step")
        self._launched = True

    def flush(self) -> None:
        check(lib().eri_adam8bit_fn_flush(self._opt), "eri_adam8bit_fn_flush")
        self._launched = True

    def set_lr(self, lr: float) -> None:
        check(lib().eri_adam8bit_fn_set_lr(self._opt, lr), "eri_adam8bit_fn_set_lr")
        self._launched = True

    def _keep(self, tensors) -> None:
        """What a launch reads and writes stays referenced until the first update after that launch: the launch is
        asynchronous (and, batched, still to come), and nothing it touches may go back to the allocator under it."""
        if self._launched:
            self._live = []
            self._launched = False
        self._live += tensors

    def get_step(self) -> int:
        return lib().eri_adam8bit_fn_get_step(self._opt)

    def update(self, name: str, param: torch.Tensor, grad: torch.Tensor) -> torch.Tensor:
        p = param.detach().contiguous()
        g = _usable_grad(grad, p)
        out = torch.empty_like(p)
        check(lib().eri_adam8bit_fn_update(self._opt, name.encode(), p.data_ptr(), g.data_ptr(), p.numel(),
                                           _dtype_tag(p), _dtype_tag(g), out.data_ptr()), "eri_adam8bit_fn_update")
        self._keep([p, g, out])
        if not self._batched:
            self._launched = True  # ran at once; released when the next update arrives
        if name not in self._names:
            self._names.append(name)
        return out

    def update_many(self, params: Dict[str, torch.Tensor], grads: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
        """Every named parameter that has a gradient, in one launch; returns the new tensors by name."""
        names = [n for n in params if n in grads]
        k = len(names)
        ps = [params[n].detach().contiguous() for n in names]
        gs = [_usable_grad(grads[n], p) for n, p in zip(names, ps)]
        outs = [torch.empty_like(p) for p in ps]
        c_names = (C.c_char_p * k)(*[n.encode() for n in names])
        arr = lambda ts: (C.c_void_p * k)(*[t.data_ptr() for t in ts])
        check(lib().eri_adam8bit_fn_update_many(self._opt, c_names, arr(ps), arr(gs),
                                                (C.c_uint64 * k)(*[p.numel() for p in ps]),
                                                (C.c_int32 * k)(*[_dtype_tag(p) for p in ps]),
                                                (C.c_int32 * k)(*[_dtype_tag(g) for g in gs]), arr(outs), k),
              "eri_adam8bit_fn_update_many")
        self._keep(ps + gs + outs)
        self._launched = True
        for n in names:
            if n not in self._names:
                self._names.append(n)
        return dict(zip(names, outs))

    def memory_stats(self) -> Tuple[int, int]:
        n, b = C.c_uint64(), C.c_uint64()
        check(lib().eri_adam8bit_fn_memory_stats(self._opt, C.byref(n), C.byref(b)), "eri_adam8bit_fn_memory_stats")
        return n.value, b.value

    def get_state_as_tensors(self) -> Dict[str, Tuple[torch.Tensor, torch.Tensor]]:
        out = {}
        for name in self._names:
            numel = C.c_uint64()
            check(lib().eri_adam8bit_fn_state_numel(self._opt, name.encode(), C.byref(numel)), "state_numel")
            m = torch.empty(numel.value, dtype=torch.float32, device="cuda")
            v = torch.empty_like(m)
            check(lib().eri_adam8bit_fn_get_state_fp32(self._opt, name.encode(), m.data_ptr(), v.data_ptr()),
                  "eri_adam8bit_fn_get_state_fp32")
            out[name] = (m, v)
        return out

    def load_state_from_tensors(self, state: Dict[str, Tuple[torch.Tensor, torch.Tensor]]) -> None:
        for name, (m, v) in state.items():
            m = m.detach().to(torch.float32).contiguous().view(-1)
            v = v.detach().to(torch.float32).contiguous().view(-1)
            check(lib().eri_adam8bit_fn_load_state_fp32(self._opt, name.encode(), m.data_ptr(), v.data_ptr(),
                                                        m.numel()), "eri_adam8bit_fn_load_state_fp32")
            if name not in self._names:
                self._names.append(name)

    def close(self) -> None:
        if self._opt:
            lib().eri_adam8bit_fn_destroy(self._opt)
            self._opt = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class EMAModel:
    """src/trainers/ema_enhanced.rs:12-204 over torch tensors: named shadow copies updated by one launch.
    `params` is a dict name -> tensor (float32 or bfloat16, contiguous)."""

    def __init__(self, decay: float, use_bias_correction: bool = True, power: float = 1.0):
        self._ema = C.c_void_p()
        check(lib().eri_ema_new(decay, int(use_bias_correction), power, _stream_ptr(), C.byref(self._ema)), "eri_ema_new")
        self._handles: Dict[str, Tuple[C.c_void_p, int, int]] = {}

    def _pack(self, params: Dict[str, torch.Tensor]):
        names = (C.c_char_p * len(params))()
        hs = (C.c_void_p * len(params))()
        for i, (name, t) in enumerate(params.items()):
            if not t.is_contiguous():
                raise ValueError("parameters must be contiguous")
            key = (t.data_ptr(), t.numel())
            h = self._handles.get(name)
            if h is None or (h[1], h[2]) != key:
                if h is not None:
                    lib().eri_param_release(h[0])
                hnd = C.c_void_p()
                check(lib().eri_param_create(t.data_ptr(), t.numel(), _dtype_tag(t), C.byref(hnd)), "eri_param_create")
                h = (hnd, *key)
                self._handles[name] = h
            names[i] = name.encode()
            hs[i] = h[0]
        return names, hs, len(params)

    def init_from_params(self, params: Dict[str, torch.Tensor]) -> None:
        check(lib().eri_ema_init_from_params(self._ema, *self._pack(params)), "eri_ema_init_from_params")

    def update(self, params: Dict[str, torch.Tensor]) -> None:
        check(lib().eri_ema_update(self._ema, *self._pack(params)), "eri_ema_update")

    def copy_to(self, params: Dict[str, torch.Tensor]) -> None:
        check(lib().eri_ema_copy_to(self._ema, *self._pack(params)), "eri_ema_copy_to")

    def step(self) -> int:
        return lib().eri_ema_step(self._ema)

    def set_step(self, step: int) -> None:
        check(lib().eri_ema_set_step(self._ema, step), "eri_ema_set_step")

    def current_decay(self) -> float:
        return lib().eri_ema_current_decay(self._ema)

    def shadow_params(self, like: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
        """Copies of the shadows of the names in `like` (torch cannot wrap foreign device memory)."""
        out = {}
        for name, t in like.items():
            ptr, numel, tag = C.c_void_p(), C.c_uint64(), C.c_int()
            check(lib().eri_ema_shadow(self._ema, name.encode(), C.byref(ptr), C.byref(numel), C.byref(tag)), "eri_ema_shadow")
            dst = torch.empty(numel.value, dtype=torch.float32 if tag.value == DTYPE_F32 else torch.bfloat16, device=t.device)
            check(lib().eri_hip_memcpy_async(dst.data_ptr(), ptr.value, dst.numel() * dst.element_size(), 3, _stream_ptr()), "memcpy")
            out[name] = dst
        return out

    def __contains__(self, name: str) -> bool:
        return lib().eri_ema_shadow(self._ema, name.encode(), None, None, None) == 0

    def close(self) -> None:
        if self._ema:
            lib().eri_ema_destroy(self._ema)
            self._ema = C.c_void_p()
            for h in self._handles.values():
                lib().eri_param_release(h[0])
            self._handles = {}

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def update_params_8bit(optimizer: Adam8bitFunctional, params: Dict[str, torch.Tensor],
                       grads: Dict[str, torch.Tensor]) -> None:
    """adam8bit.rs:333-345: every named parameter that has a gradient is replaced by its update
    (one launch for all of them instead of the reference's loop of update() calls)."""
    params.update(optimizer.update_many(params, grads))


def create_optimizer(optimizer_type: str, params: List[torch.Tensor], learning_rate=1e-4, weight_decay=0.01,
                     betas=(0.9, 0.999), eps=1e-8):
    """String-keyed factory (src/trainers/training/optimization.rs:30-58,
    src/optimizers/memory_efficient_optimizers.rs:285-308)."""
    if optimizer_type in ("adam8bit", "adamw8bit", "adamw_8bit"):
        return Adam8bit(params, Adam8bitConfig(lr=learning_rate, betas=betas, eps=eps, weight_decay=weight_decay))
    raise ValueError("InvalidOperation: Unknown optimizer: %s" % optimizer_type)
