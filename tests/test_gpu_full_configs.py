"""The two LoRA configurations of the benchmark at their full size, every element against the oracle.

Config 2 (SDXL LoRA rank 16: 1,400 tensors, 44.8e6 bf16 parameters) and config 3 (FLUX LoRA rank 32: 608
tensors, 153e6 parameters) run a hundred steps with fresh gradients each step, as the benchmark prescribes,
on two device copies of the same table:

  exact    ERI_ADAM8_FLAG_EXACT_PARAM.  Parameters, codes and absmax must equal the oracle's bit for bit
           at every checkpoint, the last being step 100 (nothing is ever re-synchronised).
  default  flags = 0, the arithmetic the benchmark times (hardware square root and reciprocal, two fused
           multiply-adds).  Its states must equal the oracle's bit for bit at every checkpoint: in this
           mode the moments do not depend on the parameters.  Its parameters are
           (a) compared after every step (config 2: all hundred, config 3: the first ten) with one
               oracle step taken from the device's own parameters of the step before: at most one bf16
               step apart, counted;
           (b) never re-synchronised with the oracle's trajectory, and the distance to it after 10 and
               after 100 steps is measured, printed and bounded (see DRIFT below).

Gradients are drawn on the device (seeded) and read back for the oracle, so both sides see the same bits;
the oracle runs one tensor per host thread.
"""
import ctypes as C
from concurrent.futures import ThreadPoolExecutor

import numpy as np
import pytest

import harness as hs
import oracle_c as oc

pytestmark = pytest.mark.gpu
LR, B1, B2, EPS, WD = 1e-4, 0.9, 0.999, 1e-8, 0.01
BLOCK = 2048
GUARD = 256  # poisoned bytes behind every tensor in every arena

# DRIFT.  What the default chain guarantees is local: from identical inputs it lands on the exact chain's
# bf16 result or on its neighbour (the one-ulp bar, checked in (a)); call the second a flip (measured:
# 6e-6 per element and step on config 2).  What happens to a flipped parameter afterwards belongs to bf16
# arithmetic, not to the kernel, and it is not a contraction:
#   * LoRA weights are of the size of their updates, so a parameter can shrink by several binades in one
#     step (p - update cancels), and the same absolute distance is then many steps of the smaller value
#     (17 after two steps of config 2, thousands later).  Distances are therefore measured in bf16 steps of
#     the largest magnitude the parameter has had on the oracle's trajectory so far ("history steps").
#   * Two trajectories one step apart on either side of a power of two live on grids of different pitch:
#     an update between half a fine step and half a coarse step moves the lower one and leaves the upper
#     one where it is, every step, for as long as the update keeps that size.  The exact chain started
#     one bf16 step off shows the same divergence.
# So the distance of a single parameter has no small a-priori bound (4.5 history steps were seen among the
# 153e6 of config 3 after 100 steps), and the assertions are on the population: at most one parameter in a
# thousand off the oracle's trajectory at any checkpoint (a flip rate of 1e-5 and 100 steps allow that), a
# mean distance below a thousandth of a history step, and no parameter further than 16 history steps.
DRIFT_MAX_FRACTION_OFF = 1e-3
DRIFT_MAX_MEAN_HISTORY_STEPS = 1e-3
DRIFT_MAX_HISTORY_STEPS = 16.0


class Arena:
    """One flat device buffer of one kind (p, g, m, v, absmax) with a host mirror for the oracle."""

    def __init__(self, torch, counts, itemsize, poison):
        self.itemsize = itemsize
        self.offs, tot = [], 0
        for n in counts:
            self.offs.append(tot)
            tot += (n * itemsize + GUARD + 255) // 256 * 256
        self.counts = counts
        self.dev = torch.full((tot,), poison, dtype=torch.uint8, device="cuda:0")
        self.poison = poison

    def ptr(self, i):
        return self.dev.data_ptr() + self.offs[i]

    def host(self):
        return self.dev.cpu().numpy()

    def views(self, raw, dtype):
        return [raw[o:o + n * self.itemsize].view(dtype) for o, n in zip(self.offs, self.counts)]

    def guards_intact(self, raw):
        for o, n in zip(self.offs, self.counts):
            if not np.all(raw[o + n * self.itemsize:o + n * self.itemsize + GUARD] == self.poison):
                return False
        return True


class DeviceCopy:
    def __init__(self, torch, L, sizes, p_host_raw, arenas_like=None):
        nbs = [(n + BLOCK - 1) // BLOCK for n in sizes]
        self.p = Arena(torch, sizes, 2, 0xFF)
        self.m = Arena(torch, sizes, 1, 0xEE)
        self.v = Arena(torch, sizes, 1, 0xEE)
        self.am = Arena(torch, nbs, 4, 0xFF)
        self.av = Arena(torch, nbs, 4, 0xFF)
        self.p.dev.copy_(torch.from_numpy(p_host_raw))
        self.sizes = sizes
        self.table = C.c_void_p()
        self.L = L

    def make_table(self, g_arena, stream):
        L = self.L
        rows = (L.TensorRow * len(self.sizes))()
        start = 0
        for i, n in enumerate(self.sizes):
            r = rows[i]
            r.p, r.g, r.m, r.v = self.p.ptr(i), g_arena.ptr(i), self.m.ptr(i), self.v.ptr(i)
            r.absmax_m, r.absmax_v = self.am.ptr(i), self.av.ptr(i)
            r.numel, r.block_start, r.dtype_tag, r.grad_scale = n, start, L.DTYPE_BF16, 1.0
            start += (n + BLOCK - 1) // BLOCK
            L.check(L.lib().eri_adam8_state_init(r.m, r.v, r.absmax_m, r.absmax_v, n, stream), "state_init")
        L.check(L.lib().eri_adam8_table_create(rows, len(rows), stream, C.byref(self.table)), "table_create")

    def destroy(self):
        self.L.lib().eri_adam8_table_destroy(self.table)


def _oracle_step(pool, ps, gs, states, step):
    h = oc.hyper_pack(LR, B1, B2, EPS, WD, step)

    def one(i):
        return oc.step_tensor(ps[i], gs[i], *states[i], h, hs.MAPS, oc.DT_BF16, 1)

    assert all(rc == 0 for rc in pool.map(one, range(len(ps))))


def _states_equal(copy, states, label):
    raws = [copy.m.host(), copy.v.host(), copy.am.host(), copy.av.host()]
    arenas = [copy.m, copy.v, copy.am, copy.av]
    for k, (raw, arena) in enumerate(zip(raws, arenas)):
        assert arena.guards_intact(raw), label + ": a guard band behind a state buffer was overwritten"
        dt = np.uint8 if k < 2 else np.uint32
        for i, got in enumerate(arena.views(raw, dt)):
            want = states[i][k].view(dt)
            if not np.array_equal(got, want):
                bad = int(np.flatnonzero(got != want)[0])
                raise AssertionError("%s: %s of tensor %d differs first at %d (got %r, oracle %r)" %
                                     (label, ("m codes", "v codes", "absmax_m", "absmax_v")[k], i, bad, got[bad], want[bad]))


def _bf16_to_f32(x):
    return (x.astype(np.uint32) << 16).view(np.float32)


def _history_distance(got_views, want_views, runmax_views):
    """Largest and mean |got - want| in bf16 steps of the running maximum magnitude, and how many differ."""
    worst, total, dist_sum, off = 0.0, 0, 0.0, 0
    for g, w, r in zip(got_views, want_views, runmax_views):
        differ = np.flatnonzero(g != w)
        total += g.size
        if differ.size == 0:
            continue
        off += differ.size
        e = (r[differ] >> 7).astype(np.int32)  # exponent field of the running maximum
        step = np.ldexp(np.float64(1.0), np.maximum(e, 1) - 127 - 7)
        d = np.abs(_bf16_to_f32(g[differ]).astype(np.float64) - _bf16_to_f32(w[differ]).astype(np.float64)) / step
        worst = max(worst, float(d.max()))
        dist_sum += float(d.sum())
    return worst, off, total, dist_sum


def _ulp_stats(got_views, want_views):
    worst, off, total, dist_sum = 0, 0, 0, 0
    for g, w in zip(got_views, want_views):
        d = hs.bf16_ulp_distance(g, w)
        worst = max(worst, int(d.max(initial=0)))
        off += int((d != 0).sum())
        dist_sum += int(d.sum())
        total += d.size
    return worst, off, total, dist_sum


def _run_config(tensors, seed, steps, checkpoints, one_step_checks):
    import torch
    from eridiffusion_amd import _lib as L
    from eridiffusion_amd import workloads as W

    sizes = [W.numel(s) for _, s in tensors]
    n_params = sum(sizes)
    dev = torch.device("cuda:0")
    stream = torch.cuda.current_stream().cuda_stream
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed)

    # parameters as the configuration prescribes: A ~ N(0, 1/in), B = 0 + N(0, 1e-4)
    g_arena = Arena(torch, sizes, 2, 0xFF)
    p_seed = Arena(torch, sizes, 2, 0xFF)
    for i, (name, shape) in enumerate(tensors):
        n = sizes[i]
        is_a = name.endswith("down") or name.endswith("lora_A")
        std = (1.0 / shape[1]) ** 0.5 if is_a else 1e-4
        p_seed.dev[p_seed.offs[i]:p_seed.offs[i] + 2 * n].view(torch.bfloat16).copy_(
            torch.randn(n, device=dev, generator=gen).mul_(std))
    p_raw = p_seed.host()
    exact = DeviceCopy(torch, L, sizes, p_raw)
    dflt = DeviceCopy(torch, L, sizes, p_raw)
    del p_seed
    exact.make_table(g_arena, stream)
    dflt.make_table(g_arena, stream)

    p_flat = p_raw.copy()  # the oracle's trajectory, one flat array so that the running maximum is one operation
    ps = exact.p.views(p_flat, np.uint16)
    runmax_flat = p_flat.view(np.uint16) & np.uint16(0x7FFF)
    runmax = [runmax_flat[o // 2:o // 2 + n] for o, n in zip(exact.p.offs, sizes)]
    states = [list(oc.state_init(n)) for n in sizes]
    flips = 0
    report = []
    with ThreadPoolExecutor(16) as pool:
        for t in range(1, steps + 1):
            for i, n in enumerate(sizes):  # fresh gradients ~ N(0, 1e-4), drawn on the device
                g_arena.dev[g_arena.offs[i]:g_arena.offs[i] + 2 * n].view(torch.bfloat16).copy_(
                    torch.randn(n, device=dev, generator=gen).mul_(1e-4))
            gs = g_arena.views(g_arena.host(), np.uint16)
            one_step_check = t <= one_step_checks
            if one_step_check:  # (a): one oracle step from the default copy's own parameters
                own = [a.copy() for a in dflt.p.views(dflt.p.host(), np.uint16)]
                own_states = [[a.copy() for a in st] for st in states]
                _oracle_step(pool, own, gs, own_states, t)
            _oracle_step(pool, ps, gs, states, t)
            np.maximum(runmax_flat, p_flat.view(np.uint16) & np.uint16(0x7FFF), out=runmax_flat)
            for copy, flags in ((exact, L.FLAG_EXACT_PARAM), (dflt, 0)):
                h = L.hyper_pack(LR, B1, B2, EPS, WD, t, L.MODE_ERI, flags)
                L.check(L.lib().eri_adam8_step_table(copy.table, C.byref(h), stream), "step_table")
            torch.cuda.synchronize()
            if one_step_check:
                raw = dflt.p.host()
                assert dflt.p.guards_intact(raw)
                worst, off, total, _ = _ulp_stats(dflt.p.views(raw, np.uint16), own)
                assert worst <= 1, "step %d: default path more than one bf16 step from the oracle's step" % t
                flips += off
            if t in checkpoints:
                label = "step %d" % t
                raw = exact.p.host()
                assert exact.p.guards_intact(raw)
                for i, (got, want) in enumerate(zip(exact.p.views(raw, np.uint16), ps)):
                    assert np.array_equal(got, want), "%s: exact parameters of tensor %d differ" % (label, i)
                _states_equal(exact, states, label + " exact")
                _states_equal(dflt, states, label + " default")
                got = dflt.p.views(dflt.p.host(), np.uint16)
                worst, off, total, dist_sum = _history_distance(got, ps, runmax)
                now_worst = _ulp_stats(got, ps)[0]
                report.append((t, worst, off, total, dist_sum, now_worst))
                assert worst <= DRIFT_MAX_HISTORY_STEPS, \
                    "%s: default path drifted %.2f history steps from the oracle's trajectory" % (label, worst)
                assert off <= DRIFT_MAX_FRACTION_OFF * total, "%s: %d of %d parameters off the oracle's trajectory" % (label, off, total)
                assert dist_sum <= DRIFT_MAX_MEAN_HISTORY_STEPS * total, "%s: mean distance %.3e history steps" % (label, dist_sum / total)
    print("%d tensors, %d params: default path, one-step flips in steps 1-%d: %d of %d (%.2e per element and step)" %
          (len(sizes), n_params, one_step_checks, flips, one_step_checks * n_params,
           flips / (float(one_step_checks) * n_params)), flush=True)
    for t, worst, off, total, dist_sum, now_worst in report:
        print("  after %3d unsynchronised steps: %d of %d parameters off the oracle's trajectory (%.2e); distance in "
              "history steps: max %.2f, mean over all parameters %.2e (in steps of the current value: max %d)" %
              (t, off, total, off / total, worst, dist_sum / total, now_worst), flush=True)
    exact.destroy()
    dflt.destroy()
    return report


def test_c2_sdxl_lora_full_size_hundred_steps():
    from eridiffusion_amd import workloads as W
    tensors = W.c2_sdxl_lora()
    assert len(tensors) == 1400 and W.total_params(tensors) == 44_813_312
    _run_config(tensors, 0xE21D + 2, 100, {1, 2, 3, 5, 10, 30, 100}, one_step_checks=100)


def test_c3_flux_lora_full_size_hundred_steps():
    from eridiffusion_amd import workloads as W
    tensors = W.c3_flux_lora()
    assert len(tensors) == 608 and W.total_params(tensors) == 153_157_632
    _run_config(tensors, 0xE21D + 3, 100, {1, 2, 5, 10, 100}, one_step_checks=10)
