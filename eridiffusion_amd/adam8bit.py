"""Python mirror of the reference's 8-bit Adam surface, on top of the C ABI.

`Adam8bit` keeps the method set of EriDiffusion's list-of-parameters optimizer
(src/trainers/adam8bit_enhanced.rs:160-369: new / step / zero_grad / current_lr /
set_learning_rate / quantized_memory_usage), `Adam8bitConfig` its configuration
(:372-395), and `Adam8bitFunctional` the per-tensor flavour
(src/trainers/adam8bit.rs:49-345: with_params / update / step / set_lr / get_step /
get_state_as_tensors / load_state_from_tensors).  torch is used for device memory and the current
stream only; every update runs in the library's HIP kernel.
"""
import ctypes as C
from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

import torch

from . import _lib
from ._lib import BLOCK, DTYPE_BF16, DTYPE_F32, MODE_ERI, MODE_L2, TensorRow, check, hyper_pack, lib


def _dtype_tag(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return DTYPE_F32
    if t.dtype == torch.bfloat16:
        return DTYPE_BF16
    raise TypeError("Unsupported: 8-bit Adam takes float32 or bfloat16 parameters, got %s" % t.dtype)


def _stream_ptr() -> int:
    return torch.cuda.current_stream().cuda_stream


class State8:
    """uint8 codes + per-block absmax of both moments for one tensor."""

    def __init__(self, numel: int, device):
        nb = (numel + BLOCK - 1) // BLOCK
        self.m = torch.empty(numel, dtype=torch.uint8, device=device)
        self.v = torch.empty(numel, dtype=torch.uint8, device=device)
        self.absmax_m = torch.empty(nb, dtype=torch.float32, device=device)
        self.absmax_v = torch.empty(nb, dtype=torch.float32, device=device)
        check(lib().eri_adam8_state_init(self.m.data_ptr(), self.v.data_ptr(), self.absmax_m.data_ptr(),
                                         self.absmax_v.data_ptr(), numel, _stream_ptr()), "eri_adam8_state_init")

    def nbytes(self) -> int:
        return self.m.numel() + self.v.numel() + 4 * (self.absmax_m.numel() + self.absmax_v.numel())


def build_rows(params, grads, states, grad_scales=None):
    """ctypes array of launch-table rows for parallel lists of tensors and states."""
    n = len(params)
    rows = (TensorRow * n)()
    start = 0
    for i, (p, g, s) in enumerate(zip(params, grads, states)):
        if g.dtype != p.dtype or g.numel() != p.numel():
            raise ValueError("gradient %d does not match its parameter in dtype or size" % i)
        if not (p.is_contiguous() and g.is_contiguous()):
            raise ValueError("parameter/gradient %d is not contiguous" % i)
        r = rows[i]
        r.p, r.g = p.data_ptr(), g.data_ptr()
        r.m, r.v = s.m.data_ptr(), s.v.data_ptr()
        r.absmax_m, r.absmax_v = s.absmax_m.data_ptr(), s.absmax_v.data_ptr()
        r.numel = p.numel()
        r.block_start = start
        r.dtype_tag = _dtype_tag(p)
        r.grad_scale = 1.0 if grad_scales is None else float(grad_scales[i])
        start += (p.numel() + BLOCK - 1) // BLOCK
    return rows


class LaunchTable:
    """Device-resident launch table (eri_adam8_table_*)."""

    def __init__(self, rows):
        self.n = len(rows)
        self._h = C.c_void_p()
        check(lib().eri_adam8_table_create(rows, self.n, _stream_ptr(), C.byref(self._h)), "eri_adam8_table_create")
        self._key = bytes(rows)

    def update(self, rows):
        key = bytes(rows)
        if key != self._key:
            check(lib().eri_adam8_table_update(self._h, rows, len(rows), _stream_ptr()), "eri_adam8_table_update")
            self._key = key

    def step(self, hyper):
        check(lib().eri_adam8_step_table(self._h, C.byref(hyper), _stream_ptr()), "eri_adam8_step_table")

    def info(self) -> Tuple[int, int]:
        a, b = C.c_uint64(), C.c_uint64()
        check(lib().eri_adam8_table_info(self._h, C.byref(a), C.byref(b)), "eri_adam8_table_info")
        return a.value, b.value

    def close(self):
        if self._h:
            lib().eri_adam8_table_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


@dataclass
class Adam8bitConfig:
    """adam8bit_enhanced.rs:372-395.  amsgrad, block_wise and percentile_clipping are carried for
    interface compatibility; the blockwise format has no clipping and is always block-wise."""
    lr: float = 1e-3
    betas: Tuple[float, float] = (0.9, 0.999)
    eps: float = 1e-8
    weight_decay: float = 0.01
    amsgrad: bool = False
    block_wise: bool = True
    percentile_clipping: int = 99


class Adam8bit:
    """`step()` over a list of parameters that carry their gradients (`.grad`)."""

    def __init__(self, params: List[torch.Tensor], config: Optional[Adam8bitConfig] = None, flags: int = 0):
        config = config or Adam8bitConfig()
        self.params = list(params)
        self.learning_rate = float(config.lr)
        self.beta1, self.beta2 = map(float, config.betas)
        self.epsilon = float(config.eps)
        self.weight_decay = float(config.weight_decay)
        self.step_count = 0
        self.flags = flags
        self.grad_scale = None  # set to a float to fold a clip factor into the step
        self._states: Dict[int, State8] = {}
        self._table: Optional[LaunchTable] = None
        self._table_ids: Optional[Tuple[int, ...]] = None
        lib()  # fail now, not at the first step, if the HIP library is missing

    def step(self) -> None:
        """adam8bit_enhanced.rs:202-291; parameters without a gradient are skipped with a warning."""
        self.step_count += 1
        idx, ps, gs = [], [], []
        for i, p in enumerate(self.params):
            g = p.grad
            if g is None:
                print("Warning: No gradient for param_%d" % i)
                continue
            if p.numel() == 0:
                raise RuntimeError("InvalidOperation: Empty tensor for quantization")
            if i not in self._states:
                self._states[i] = State8(p.numel(), p.device)
            idx.append(i)
            ps.append(p.data)
            gs.append(g if g.dtype == p.dtype else g.to(p.dtype))
        if not idx:
            return
        rows = build_rows(ps, gs, [self._states[i] for i in idx])
        ids = tuple(idx)
        if self._table is None or self._table_ids != ids:
            if self._table is not None:
                self._table.close()
            self._table = LaunchTable(rows)
            self._table_ids = ids
        else:
            self._table.update(rows)
        self._live = gs  # keep cast gradients alive until the stream has consumed them
        h = hyper_pack(self.learning_rate, self.beta1, self.beta2, self.epsilon, self.weight_decay,
                       self.step_count, MODE_ERI, self.flags, self.grad_scale)
        self._table.step(h)

    def zero_grad(self) -> None:
        for p in self.params:
            p.grad = None

    def current_lr(self) -> float:
        return self.learning_rate

    def set_learning_rate(self, lr: float) -> None:
        self.learning_rate = float(lr)

    def quantized_memory_usage(self) -> int:
        return sum(s.nbytes() for s in self._states.values())

    def state(self, index: int) -> State8:
        return self._states[index]


class Adam8bitFunctional:
    """Per-tensor flavour keyed by name (adam8bit.rs): update() returns the new parameter tensor,
    step() only bumps the counter."""

    def __init__(self, learning_rate=1e-4, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.01, flags=0):
        self.learning_rate, self.beta1, self.beta2 = float(learning_rate), float(beta1), float(beta2)
        self.eps, self.weight_decay = float(eps), float(weight_decay)
        self.step_count = 0
        self.flags = flags
        self._states: Dict[str, State8] = {}
        lib()

    @classmethod
    def with_params(cls, learning_rate, beta1, beta2, eps, weight_decay):
        return cls(learning_rate, beta1, beta2, eps, weight_decay)

    def step(self) -> None:
        self.step_count += 1

    def set_lr(self, lr: float) -> None:
        self.learning_rate = float(lr)

    def get_step(self) -> int:
        return self.step_count

    def update(self, name: str, param: torch.Tensor, grad: torch.Tensor) -> torch.Tensor:
        if param.numel() == 0:
            raise RuntimeError("InvalidOperation: Empty tensor for quantization")
        new = param.detach().clone()
        g = grad if grad.dtype == param.dtype else grad.to(param.dtype)
        if name not in self._states:
            self._states[name] = State8(param.numel(), param.device)
        rows = build_rows([new], [g.contiguous()], [self._states[name]])
        h = hyper_pack(self.learning_rate, self.beta1, self.beta2, self.eps, self.weight_decay,
                       self.step_count, MODE_L2, self.flags)
        check(lib().eri_adam8_step_multi(rows, 1, C.byref(h), _stream_ptr()), "eri_adam8_step_multi")
        return new

    def memory_stats(self) -> Tuple[int, int]:
        return len(self._states), sum(s.nbytes() for s in self._states.values())

    def get_state_as_tensors(self) -> Dict[str, Tuple[torch.Tensor, torch.Tensor]]:
        out = {}
        for name, s in self._states.items():
            m = torch.empty(s.m.numel(), dtype=torch.float32, device=s.m.device)
            v = torch.empty_like(m)
            check(lib().eri_adam8_dequantize(s.m.data_ptr(), s.absmax_m.data_ptr(), 1, m.numel(), m.data_ptr(),
                                             _stream_ptr()), "eri_adam8_dequantize")
            check(lib().eri_adam8_dequantize(s.v.data_ptr(), s.absmax_v.data_ptr(), 0, v.numel(), v.data_ptr(),
                                             _stream_ptr()), "eri_adam8_dequantize")
            out[name] = (m, v)
        return out

    def load_state_from_tensors(self, state: Dict[str, Tuple[torch.Tensor, torch.Tensor]]) -> None:
        self._states.clear()
        for name, (m, v) in state.items():
            m = m.detach().to(torch.float32).contiguous().view(-1)
            v = v.detach().to(torch.float32).contiguous().view(-1)
            s = State8(m.numel(), m.device)
            check(lib().eri_adam8_quantize(m.data_ptr(), 1, m.numel(), s.m.data_ptr(), s.absmax_m.data_ptr(),
                                           _stream_ptr()), "eri_adam8_quantize")
            check(lib().eri_adam8_quantize(v.data_ptr(), 0, v.numel(), s.v.data_ptr(), s.absmax_v.data_ptr(),
                                           _stream_ptr()), "eri_adam8_quantize")
            self._states[name] = s


def update_params_8bit(optimizer: Adam8bitFunctional, params: Dict[str, torch.Tensor],
                       grads: Dict[str, torch.Tensor]) -> None:
    """adam8bit.rs:333-345."""
    for name in list(params.keys()):
        if name in grads:
            params[name] = optimizer.update(name, params[name], grads[name])
