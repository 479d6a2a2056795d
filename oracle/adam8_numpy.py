"""Second, independent CPU restatement of the blockwise 8-bit AdamW step, in NumPy.

TEST INFRASTRUCTURE ONLY.  It exists so that two separately written restatements (this one,
vectorised float32 NumPy; the other, scalar C in adam8_oracle.c) can be required to agree bit for
bit; the shipped library and the Python package never import it.

It follows the same two reference functions as the C oracle:
  * mode "eri": Adam8bit::step, src/trainers/adam8bit_enhanced.rs:202-291
  * mode "l2" : Adam8bit::update, src/trainers/adam8bit.rs:101-208
  * mode "bnb": parameter update and sign rule of bitsandbytes' 8-bit blockwise Adam (the library the
    state format comes from; not installed here, not used by the reference)
with the state kept as uint8 codes into the bitsandbytes dynamic maps plus one fp32 absmax per
2048-element block.  Every NumPy float32 operation below rounds once, which is the rounding
behaviour of the reference's chain of separate tensor operations.
"""
import math

import numpy as np

BLOCK = 2048
F32 = np.float32


def bf16_to_f32(h):
    """uint16 bf16 bit patterns -> float32."""
    return (np.asarray(h, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(F32)


def f32_to_bf16(x):
    """float32 -> uint16 bf16 bit patterns, round to nearest even; NaN keeps a set quiet bit."""
    u = np.ascontiguousarray(x, dtype=F32).view(np.uint32)
    nan = (u & np.uint32(0x7FFFFFFF)) > np.uint32(0x7F800000)
    r = (u + (np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1)))) >> np.uint32(16)
    r = np.where(nan, (u >> np.uint32(16)) | np.uint32(0x40), r)
    return r.astype(np.uint16)


def midpoints(table):
    t = np.asarray(table, dtype=F32)
    return ((t[:-1] + t[1:]) * F32(0.5)).astype(F32)


def nearest_index(mid, x):
    """Count of midpoints strictly below x (lower index on a tie); NaN -> 0."""
    x = np.asarray(x, dtype=F32)
    idx = np.searchsorted(mid, x, side="left")
    return np.where(np.isnan(x), 0, idx).astype(np.uint8)


def hyper_pack(lr, beta1, beta2, eps, wd, step, mode="eri"):
    """Per-step scalars with the reference's cast points.

    eri: adam8bit_enhanced.rs:203-215 (f64 bias corrections, one cast of the step size),
         :256/:260 (`1.0 - beta as f32` is an fp32 subtraction).
    l2 : adam8bit.rs:139-178 (`(1.0 - beta) as f32` is an f64 subtraction; s = max(step, 1)).
    """
    h = {"mode": mode, "beta1": F32(beta1), "beta2": F32(beta2), "eps": F32(eps),
         "wd": F32(wd), "grad_scale": None}
    if mode == "l2":
        s = max(int(step), 1)
        h["omb1"] = F32(1.0 - beta1)
        h["omb2"] = F32(1.0 - beta2)
        h["bc1"] = F32(1.0 - beta1 ** s)
        h["bc2"] = F32(1.0 - beta2 ** s)
        h["step_size"] = F32(lr)
    else:
        t = float(step)
        bc1 = 1.0 - math.pow(beta1, t)
        bc2 = 1.0 - math.pow(beta2, t)
        h["omb1"] = F32(1.0) - F32(beta1)
        h["omb2"] = F32(1.0) - F32(beta2)
        h["bc1"] = F32(bc1)
        h["bc2"] = F32(bc2)
        h["step_size"] = F32(lr * (math.sqrt(bc2) / bc1))
        if mode == "bnb":  # eps rides on sqrt(bc2); the decay becomes a factor applied after the Adam term
            h["eps"] = F32(eps * math.sqrt(bc2))
            h["wd"] = F32(1.0 - lr * wd)
    return h


def state_init(numel):
    nb = (numel + BLOCK - 1) // BLOCK
    return (np.full(numel, 127, np.uint8), np.zeros(numel, np.uint8),
            np.zeros(nb, F32), np.zeros(nb, F32))


def _blockwise(x, numel):
    nb = (numel + BLOCK - 1) // BLOCK
    pad = nb * BLOCK - numel
    return np.concatenate([x, np.zeros(pad, x.dtype)]).reshape(nb, BLOCK), nb


def step_tensor(p, g, m_code, v_code, absmax_m, absmax_v, h, map_s, map_u, bf16=False, grad_bf16=None):
    """Returns (p_new, m_code_new, v_code_new, absmax_m_new, absmax_v_new); inputs untouched.

    p and g are float32 arrays, or uint16 bf16 bit patterns when bf16=True.  grad_bf16=False with bf16=True
    is a float32 gradient for bf16 parameters: the reference casts every gradient to F32 and never rounds it
    (adam8bit_enhanced.rs:231-235).
    """
    if grad_bf16 is None:
        grad_bf16 = bf16
    numel = int(np.asarray(m_code).size)
    if numel == 0:
        raise ValueError("Empty tensor for quantization")
    map_s = np.asarray(map_s, F32)
    map_u = np.asarray(map_u, F32)
    pf = bf16_to_f32(p) if bf16 else np.asarray(p, F32)
    gf = bf16_to_f32(g) if grad_bf16 else np.asarray(g, F32)
    blk = np.arange(numel) // BLOCK
    with np.errstate(all="ignore"):
        m_old = map_s[m_code] * absmax_m[blk]
        v_old = map_u[v_code] * absmax_v[blk]
        if h.get("grad_scale") is not None:
            gf = gf * F32(h["grad_scale"])
        if h["mode"] == "l2" and h["wd"] > 0:
            gf = gf + pf * h["wd"]
        m = m_old * h["beta1"] + gf * h["omb1"]
        v = v_old * h["beta2"] + (gf * gf) * h["omb2"]
        if h["mode"] == "l2":
            mh = m / h["bc1"]
            vh = np.fmax(v / h["bc2"], F32(0))
            us = (mh / (np.sqrt(vh) + h["eps"])) * h["step_size"]
            if bf16:
                us = bf16_to_f32(f32_to_bf16(us))
            pn = pf - us
        elif h["mode"] == "bnb":
            pn = pf - (m / (np.sqrt(v) + h["eps"])) * h["step_size"]
            if h["wd"] != F32(1.0):
                pn = pn * h["wd"]
        else:
            r = m / (np.sqrt(v) + h["eps"])
            u = r + pf * h["wd"] if h["wd"] > 0 else r
            pn = pf - u * h["step_size"]
        mb, nb = _blockwise(np.abs(m), numel)
        vb, _ = _blockwise(np.abs(v), numel)
        am = np.fmax.reduce(mb, axis=1, initial=F32(0)).astype(F32)
        av = np.fmax.reduce(vb, axis=1, initial=F32(0)).astype(F32)
        am_e = am[blk]
        av_e = av[blk]
        xm = np.where(am_e == 0, F32(0), m / np.where(am_e == 0, F32(1), am_e)).astype(F32)
        xv = np.where(av_e == 0, F32(0), v / np.where(av_e == 0, F32(1), av_e)).astype(F32)
    mc = nearest_index(midpoints(map_s), xm)
    vc = nearest_index(midpoints(map_u), xv)
    if h["mode"] == "bnb":  # a code whose map value has the other sign than the moment moves toward the moment
        flip = (np.signbit(map_s[mc]) != np.signbit(m)) & (am_e != 0) & np.isfinite(m)
        mc = np.where(flip, np.where(m > 0, mc.astype(np.int32) + 1, mc.astype(np.int32) - 1), mc).astype(np.uint8)
    p_out = f32_to_bf16(pn) if bf16 else pn.astype(F32)
    return p_out, mc, vc, am, av
