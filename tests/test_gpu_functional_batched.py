"""The functional update(name, param, grad) path in one launch, rows that read their parameters from one
tensor and write them to another, and F32 gradients for BF16 parameters.

The reference's LoRA trainers call update() once per tensor, 600 to 1,400 times per step
(src/trainers/pipeline_flux_lora_sequential.rs:749-794, pipeline_sdxl_lora.rs:696-728); here those calls
become one row each of one launch table.  Everything is compared with the oracle bit for bit: the
functional update always takes the IEEE chain.
"""
import ctypes as C
from concurrent.futures import ThreadPoolExecutor

import numpy as np
import pytest

import harness as hs
import oracle_c as oc
from oracle import adam8_numpy as onp

pytestmark = pytest.mark.gpu
LR, B1, B2, EPS, WD = 1e-4, 0.9, 0.999, 1e-8, 0.01
BLOCK = 2048


def _L():
    from eridiffusion_amd import _lib
    return _lib


def _dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a).view(np.uint8).reshape(-1).copy()).to("cuda:0")


def _bits(t, dtype):
    return t.cpu().numpy().view(dtype)


def test_sdxl_lora_list_through_update_many_in_one_launch():
    """Config 2 at full size (1,400 tensors, 44.8e6 bf16 parameters) through eri_adam8bit_fn_update_many,
    four steps, each writing into fresh output tensors (update() returns a new tensor), against the oracle's
    functional update: parameters, codes and absmax bit for bit."""
    import torch
    from eridiffusion_amd import workloads as W
    L = _L()
    tensors = W.c2_sdxl_lora()
    sizes = [W.numel(s) for _, s in tensors]
    n = len(sizes)
    assert n == 1400
    rng = np.random.default_rng(0xE21D + 2)
    ps = [onp.f32_to_bf16((rng.standard_normal(k) * (0.02 if i % 2 == 0 else 1e-4)).astype(np.float32)) for i, k in enumerate(sizes)]
    states = hs.oracle_states(sizes)
    cur = [_dev(p) for p in ps]
    opt = C.c_void_p()
    stream = torch.cuda.current_stream().cuda_stream
    L.check(L.lib().eri_adam8bit_fn_with_params(LR, B1, B2, EPS, WD, stream, C.byref(opt)), "with_params")
    names = (C.c_char_p * n)(*[t[0].encode() for t in tensors])
    numels = (C.c_uint64 * n)(*sizes)
    tags = (C.c_int32 * n)(*([L.DTYPE_BF16] * n))
    keep = []
    with ThreadPoolExecutor(16) as pool:
        for step in range(4):
            gs = hs.fresh_grads(sizes, True, 7000 + step, 1e-4)
            g_dev = [_dev(g) for g in gs]
            outs = [torch.empty_like(c) for c in cur]
            arr = lambda ts: (C.c_void_p * n)(*[t.data_ptr() for t in ts])
            L.check(L.lib().eri_adam8bit_fn_update_many(opt, names, arr(cur), arr(g_dev), numels, tags, None, arr(outs), n),
                    "update_many")
            L.check(L.lib().eri_adam8bit_fn_step(opt), "fn_step")
            keep += [cur, g_dev]
            cur = outs
            h = oc.hyper_pack(LR, B1, B2, EPS, WD, step, oc.MODE_L2)  # the counter as it stood during the updates
            rcs = pool.map(lambda i: oc.step_tensor(ps[i], gs[i], *states[i], h, hs.MAPS, oc.DT_BF16, 1), range(n))
            assert all(rc == 0 for rc in rcs)
    torch.cuda.synchronize()
    for i in range(n):
        assert np.array_equal(_bits(cur[i], np.uint16), ps[i]), "parameters of tensor %d (%s)" % (i, tensors[i][0])
    # the states, through the fp32 export, for a sample of names
    for i in (0, 1, 17, 700, 1399):
        k = sizes[i]
        m_out = torch.empty(k, dtype=torch.float32, device="cuda:0")
        v_out = torch.empty(k, dtype=torch.float32, device="cuda:0")
        L.check(L.lib().eri_adam8bit_fn_get_state_fp32(opt, names[i], m_out.data_ptr(), v_out.data_ptr()), "get_state")
        torch.cuda.synchronize()
        blk = np.arange(k) // BLOCK
        assert np.array_equal(m_out.cpu().numpy(), hs.MAPS[0][states[i][0]] * states[i][2][blk])
        assert np.array_equal(v_out.cpu().numpy(), hs.MAPS[1][states[i][1]] * states[i][3][blk])
    assert L.lib().eri_adam8bit_fn_get_step(opt) == 4
    L.lib().eri_adam8bit_fn_destroy(opt)


@pytest.mark.parametrize("mixed", [False, True])
def test_batched_updates_equal_immediate_updates(mixed):
    """The same sequence of update() / step() calls on two optimizers, one batching, one not: identical
    parameters and states after every step.  The sequence has a name updated twice inside one step (the
    first update must run before the second is queued), a change of the set of names between steps, a
    learning-rate change, and with `mixed` F32 tensors, BF16 tensors and BF16 tensors with F32 gradients."""
    import torch
    L = _L()
    spec = [("a.down", 2048 * 3 + 5, 2, 2), ("a.up", 640, 2, 2), ("b.down", 4096, 2, 0 if mixed else 2),
            ("b.up", 2048 * 2, 0 if mixed else 2, 0 if mixed else 2), ("c.bias", 77, 2, 0 if mixed else 2)]
    opts = []
    for batching in (0, 1):
        o = C.c_void_p()
        L.check(L.lib().eri_adam8bit_fn_with_params(LR, B1, B2, EPS, WD, None, C.byref(o)), "with_params")
        L.check(L.lib().eri_adam8bit_fn_set_batching(o, batching), "set_batching")
        opts.append(o)
    rng = np.random.default_rng(5)

    def host(k, tag, std):
        x = (rng.standard_normal(k) * std).astype(np.float32)
        return onp.f32_to_bf16(x) if tag == 2 else x

    cur = [[_dev(host(k, pt, 0.02)) for _, k, pt, _ in spec] for _ in range(2)]
    for b in range(len(spec)):
        cur[1][b].copy_(cur[0][b])
    keep = []
    for step in range(4):
        order = list(range(len(spec)))
        if step == 1:
            order = [0, 1, 0, 2]      # "a.down" twice, "b.up" and "c.bias" without a gradient this step
        if step == 2:
            order = [4, 3, 2, 1, 0]   # another order
        grads = [_dev(host(spec[b][1], spec[b][3], 1e-3)) for b in order]
        for which, o in enumerate(opts):
            for g, b in zip(grads, order):
                name, k, pt, gt = spec[b]
                out = torch.empty_like(cur[which][b])
                L.check(L.lib().eri_adam8bit_fn_update(o, name.encode(), cur[which][b].data_ptr(), g.data_ptr(), k, pt, gt,
                                                       out.data_ptr()), "fn_update")
                keep.append(cur[which][b])
                cur[which][b] = out
            if step == 2:
                L.check(L.lib().eri_adam8bit_fn_set_lr(o, 3e-4), "set_lr")  # runs what is queued under the old rate
            L.check(L.lib().eri_adam8bit_fn_step(o), "fn_step")
        keep.append(grads)
        torch.cuda.synchronize()
        for b in range(len(spec)):
            assert torch.equal(cur[0][b], cur[1][b]), (step, spec[b][0])
    for name, k, _, _ in spec:
        got = []
        for o in opts:
            m_out = torch.empty(k, dtype=torch.float32, device="cuda:0")
            v_out = torch.empty(k, dtype=torch.float32, device="cuda:0")
            L.check(L.lib().eri_adam8bit_fn_get_state_fp32(o, name.encode(), m_out.data_ptr(), v_out.data_ptr()), "get_state")
            got.append((m_out, v_out))
        torch.cuda.synchronize()
        assert torch.equal(got[0][0], got[1][0]) and torch.equal(got[0][1], got[1][1]), name
    for o in opts:
        L.lib().eri_adam8bit_fn_destroy(o)


@pytest.mark.parametrize("flags_name", ["default-kernels", "one-wave", "plain"])
@pytest.mark.parametrize("mode", [0, 1, 2])
def test_rows_that_write_to_another_tensor(mode, flags_name):
    """p_src: the old parameters are read from one tensor and the new ones written to another, on every
    step kernel (four waves per block, prefetching, plain), full and partial blocks, both dtypes.  The
    source must be left as it was, the result must equal the oracle's."""
    import torch
    L = _L()
    extra = {"default-kernels": 0, "one-wave": L.FLAG_ONE_WAVE, "plain": L.FLAG_NO_PIPELINE}[flags_name]
    for bf16 in (True, False):
        sizes = [2048 * 7 + 24, 2048 * 2, 9, 2048 + 1000]
        ps, gs = hs.make_inputs(sizes, bf16, 40 + mode)
        states = hs.oracle_states(sizes)
        gt = hs.GpuTensors(ps, gs, states, bf16)
        src = [_dev(p) for p in ps]
        rows = gt.rows()
        for r, s in zip(rows, src):
            r.p_src = s.data_ptr()
        for buf in gt.p:
            buf[0].fill_(0x55)  # whatever the destination held is irrelevant
        table = C.c_void_p()
        L.check(L.lib().eri_adam8_table_create(rows, len(rows), None, C.byref(table)), "table_create")
        step = 0 if mode == 1 else 1
        h = L.hyper_pack(LR, B1, B2, EPS, WD, step, mode, L.FLAG_EXACT_PARAM | extra)
        L.check(L.lib().eri_adam8_step_table(table, C.byref(h), None), "step_table")
        torch.cuda.synchronize()
        want_src = [p.copy() for p in ps]
        hs.oracle_step(ps, gs, states, (LR, B1, B2, EPS, WD, step), bf16, {0: oc.MODE_ERI, 1: oc.MODE_L2, 2: oc.MODE_BNB}[mode])
        for s, w in zip(src, want_src):
            assert np.array_equal(_bits(s, np.uint8), w.view(np.uint8)), "the source tensor was written"
        # the guard bands of GpuTensors.p were filled with 0x55 above, so only the payload is compared
        for buf, w in zip(gt.p, ps):
            t, dt, k, _ = buf
            got = t.cpu().numpy()[gt.GUARD * dt.itemsize:(gt.GUARD + k) * dt.itemsize]
            assert np.array_equal(got, w.view(np.uint8)), (mode, flags_name, bf16)
            lo = t.cpu().numpy()[:gt.GUARD * dt.itemsize]
            hi = t.cpu().numpy()[(gt.GUARD + k) * dt.itemsize:]
            assert np.all(lo == 0x55) and np.all(hi == 0x55), "written outside the destination"
        L.lib().eri_adam8_table_destroy(table)
    # a source that overlaps its destination without being equal to it is refused
    rows = gt.rows()
    rows[0].p_src = rows[0].p + 32
    table = C.c_void_p()
    assert L.lib().eri_adam8_table_create(rows, len(rows), None, C.byref(table)) == -6


@pytest.mark.parametrize("kernels", ["default-kernels", "one-wave", "plain"])
@pytest.mark.parametrize("mode,flags", [(0, 2), (0, 0), (1, 2), (2, 2), (2, 0)])
def test_f32_gradients_for_bf16_parameters_in_a_mixed_table(mode, flags, kernels):
    """One table with all three layouts -- F32, BF16, and BF16 parameters with F32 gradients -- ragged sizes,
    three steps.  The F32 gradients are not representable in BF16 (their low mantissa bits are set), so a
    kernel that rounded them first would produce other moments than the oracle, which uses them as they are
    (the reference casts gradients to F32 and never rounds them, adam8bit_enhanced.rs:231-235).  Small tables
    take the four-waves-per-block kernel; "one-wave" runs the kernels that the largest tables take (with the
    next block's loads in flight), "plain" the one-wave kernel without them, which mid-size tables take."""
    import torch
    L = _L()
    flags |= {"default-kernels": 0, "one-wave": L.FLAG_ONE_WAVE, "plain": L.FLAG_NO_PIPELINE}[kernels]
    sizes = [2048 * 4 + 12, 2048 * 3, 100, 2048 * 9 + 1, 640 * 16, 2048 * 2 + 1023, 5]
    p_tags = [2, 0, 2, 2, 0, 2, 2]
    g_tags = [0, 0, 0, 2, 0, 0, 2]  # rows 0, 2, 5: BF16 parameters with F32 gradients
    rng = np.random.default_rng(99 + mode)

    def host(k, tag, std):
        x = (rng.standard_normal(k) * std).astype(np.float32)
        return onp.f32_to_bf16(x) if tag == 2 else x

    ps = [host(k, t, 0.02) for k, t in zip(sizes, p_tags)]
    states = hs.oracle_states(sizes)
    p_dev = [_dev(p) for p in ps]
    st_dev = [[_dev(a) for a in st] for st in states]
    omode = {0: oc.MODE_ERI, 1: oc.MODE_L2, 2: oc.MODE_BNB}[mode]
    table = C.c_void_p()
    flips = 0
    for step in range(1, 4):
        gs = [host(k, t, 1e-3) for k, t in zip(sizes, g_tags)]
        assert any((g.view(np.uint32) & 0xFFFF).any() for g, t in zip(gs, g_tags) if t == 0)
        g_dev = [_dev(g) for g in gs]
        rows = (L.TensorRow * len(sizes))()
        start = 0
        for i, k in enumerate(sizes):
            r = rows[i]
            r.p, r.g = p_dev[i].data_ptr(), g_dev[i].data_ptr()
            r.m, r.v, r.absmax_m, r.absmax_v = [a.data_ptr() for a in st_dev[i]]
            r.numel, r.block_start, r.dtype_tag, r.grad_scale = k, start, p_tags[i], 1.0
            r.grad_f32 = 1 if (p_tags[i] == 2 and g_tags[i] == 0) else 0
            start += (k + BLOCK - 1) // BLOCK
        if step == 1:
            L.check(L.lib().eri_adam8_table_create(rows, len(rows), None, C.byref(table)), "table_create")
        else:
            L.check(L.lib().eri_adam8_table_update(table, rows, len(rows), None), "table_update")
        t = step - 1 if mode == 1 else step
        # global gradient norm over the mixed table
        L.check(L.lib().eri_adam8_grad_norm(table, 1e9, 0.0, None), "grad_norm")
        norm, scale = C.c_float(), C.c_float()
        L.check(L.lib().eri_adam8_grad_norm_read(table, C.byref(norm), C.byref(scale), None), "norm_read")
        want = np.sqrt(sum(float(np.sum((onp.bf16_to_f32(g) if tg == 2 else g).astype(np.float64) ** 2)) for g, tg in zip(gs, g_tags)))
        assert abs(norm.value - want) <= 2e-6 * want and scale.value == 1.0
        h = L.hyper_pack(LR, B1, B2, EPS, WD, t, mode, flags)
        L.check(L.lib().eri_adam8_step_table(table, C.byref(h), None), "step_table")
        torch.cuda.synchronize()
        ho = oc.hyper_pack(LR, B1, B2, EPS, WD, t, omode)
        for i in range(len(sizes)):
            assert oc.step_tensor(ps[i], gs[i], *states[i], ho, hs.MAPS, p_tags[i], 2, g_dtype=g_tags[i]) == 0
        for i in range(len(sizes)):
            for k_, dt in enumerate((np.uint8, np.uint8, np.uint32, np.uint32)):
                assert np.array_equal(_bits(st_dev[i][k_], dt), states[i][k_].view(dt)), (step, i, k_)
            if p_tags[i] == 0:
                assert np.array_equal(_bits(p_dev[i], np.uint32), ps[i].view(np.uint32)), (step, i)
            else:
                got = _bits(p_dev[i], np.uint16)
                d = hs.bf16_ulp_distance(got, ps[i])
                exact = bool(flags & 2) or mode == 1
                assert d.max(initial=0) <= (0 if exact else 1), (step, i, int(d.max(initial=0)))
                flips += int((d != 0).sum())
                if not exact:  # the next step starts from the device's parameters (one-ulp bar per step)
                    ps[i][:] = got
    print("mixed table mode %d flags %d: bf16 parameters one step off: %d" % (mode, flags, flips), flush=True)
    # changing a row's layout is not an update of the same table
    rows[3].grad_f32 = 1
    assert L.lib().eri_adam8_table_update(table, rows, len(rows), None) == -6
    L.lib().eri_adam8_table_destroy(table)
    rows[1].grad_f32 = 1  # F32 parameters
    bad = C.c_void_p()
    assert L.lib().eri_adam8_table_create(rows, len(rows), None, C.byref(bad)) == -4


def test_python_face_batched_functional_and_f32_gradients():
    """Adam8bitFunctional(batched=True): update() returns tensors that step() fills; float32 gradients of
    bfloat16 parameters go in unrounded, through both optimizer objects."""
    import torch
    from eridiffusion_amd.adam8bit import Adam8bit, Adam8bitConfig, Adam8bitFunctional, update_params_8bit
    torch.manual_seed(3)
    dev = "cuda:0"
    shapes = {"x.down": (16, 640), "x.up": (1280, 16), "y.bias": (320,)}
    params = {k: (torch.randn(s, device=dev) * 0.02).to(torch.bfloat16) for k, s in shapes.items()}
    grads = {k: torch.randn(s, device=dev) * 1e-3 for k, s in shapes.items()}  # float32
    a = Adam8bitFunctional(LR, B1, B2, EPS, WD, batched=True)
    b = Adam8bitFunctional(LR, B1, B2, EPS, WD)
    outs_a = {k: a.update(k, params[k], grads[k]) for k in params}
    a.step()
    outs_b = {k: b.update(k, params[k], grads[k]) for k in params}
    b.step()
    c = Adam8bitFunctional(LR, B1, B2, EPS, WD)
    pc = dict(params)
    update_params_8bit(c, pc, grads)
    c.step()
    torch.cuda.synchronize()
    maps = hs.MAPS
    for k in params:
        assert torch.equal(outs_a[k], outs_b[k]) and torch.equal(outs_a[k], pc[k]), k
        n = params[k].numel()
        p_host = params[k].view(torch.int16).cpu().numpy().view(np.uint16).reshape(-1).copy()
        g_host = grads[k].cpu().numpy().reshape(-1).copy()
        st = list(oc.state_init(n))
        h = oc.hyper_pack(LR, B1, B2, EPS, WD, 0, oc.MODE_L2)
        assert oc.step_tensor(p_host, g_host, *st, h, maps, oc.DT_BF16, 1, g_dtype=oc.DT_F32) == 0
        assert np.array_equal(outs_a[k].view(torch.int16).cpu().numpy().view(np.uint16).reshape(-1), p_host), k
        # rounding the gradient first gives another result somewhere
    rounded = Adam8bitFunctional(LR, B1, B2, EPS, WD)
    differs = any(not torch.equal(rounded.update(k, params[k], grads[k].to(torch.bfloat16)), outs_a[k]) for k in params)
    torch.cuda.synchronize()
    assert differs
    # the list-of-parameters optimizer with float32 .grad on bfloat16 parameters
    plist = [params[k].clone() for k in params]
    for p, k in zip(plist, params):
        if hasattr(p, "grad_dtype"):
            p.grad_dtype = None  # newer torch versions refuse a gradient of another dtype otherwise
        p.grad = grads[k]
    opt = Adam8bit(plist, Adam8bitConfig(lr=LR, betas=(B1, B2), eps=EPS, weight_decay=WD), flags=2)
    assert opt.step() == 0
    torch.cuda.synchronize()
    for p, k in zip(plist, params):
        n = p.numel()
        p_host = params[k].view(torch.int16).cpu().numpy().view(np.uint16).reshape(-1).copy()
        g_host = grads[k].cpu().numpy().reshape(-1).copy()
        st = list(oc.state_init(n))
        assert oc.step_tensor(p_host, g_host, *st, oc.hyper_pack(LR, B1, B2, EPS, WD, 1), maps, oc.DT_BF16, 1, g_dtype=oc.DT_F32) == 0
        assert np.array_equal(p.view(torch.int16).cpu().numpy().view(np.uint16).reshape(-1), p_host), k
    for o in (a, b, c, rounded, opt):
        o.close()


def test_alternating_output_sets_stop_uploading_after_two_flushes():
    """update() returns a new tensor per call (adam8bit.rs:205-207), so a trainer's rows alternate between two sets of
    addresses.  The two launch tables kept serve every flush from the third on without an upload, and the results
    stay those of the oracle, bit for bit.  A third set of addresses costs one more upload."""
    import torch
    L = _L()
    sizes = [2048 * 3 + 8, 640 * 16, 2048, 4104]
    n = len(sizes)
    ps, _ = hs.make_inputs(sizes, True, 991)
    states = hs.oracle_states(sizes)
    bufs = [[_dev(p) for p in ps], [_dev(p) for p in ps]]  # the two sets a trainer's allocator hands back in turn
    g_dev = [_dev(np.zeros(k, np.uint16)) for k in sizes]   # gradient buffers are reused, refilled every step
    opt = C.c_void_p()
    stream = torch.cuda.current_stream().cuda_stream
    L.check(L.lib().eri_adam8bit_fn_with_params(LR, B1, B2, EPS, WD, stream, C.byref(opt)), "with_params")
    names = (C.c_char_p * n)(*[("w%d" % i).encode() for i in range(n)])
    numels = (C.c_uint64 * n)(*sizes)
    tags = (C.c_int32 * n)(*([L.DTYPE_BF16] * n))
    arr = lambda ts: (C.c_void_p * n)(*[t.data_ptr() for t in ts])
    flushes, uploads = C.c_uint64(), C.c_uint64()
    seen = []
    for step in range(6):
        gs = hs.fresh_grads(sizes, True, 8100 + step, 1e-3)
        for d, g in zip(g_dev, gs):
            d.copy_(_dev(g))
        src, dst = bufs[step & 1], bufs[1 - (step & 1)]
        L.check(L.lib().eri_adam8bit_fn_update_many(opt, names, arr(src), arr(g_dev), numels, tags, None, arr(dst), n), "update_many")
        L.check(L.lib().eri_adam8bit_fn_step(opt), "fn_step")
        hs.oracle_step(ps, gs, states, (LR, B1, B2, EPS, WD, step), True, oc.MODE_L2)
        L.check(L.lib().eri_adam8bit_fn_table_stats(opt, C.byref(flushes), C.byref(uploads)), "table_stats")
        seen.append((flushes.value, uploads.value))
    assert seen == [(1, 1), (2, 2), (3, 2), (4, 2), (5, 2), (6, 2)]
    torch.cuda.synchronize()
    for i in range(n):
        assert np.array_equal(_bits(bufs[0][i], np.uint16), ps[i])
    # addresses seen in neither of the last two flushes: one upload, into the table used longer ago
    third = [torch.empty_like(t) for t in bufs[0]]
    gs = hs.fresh_grads(sizes, True, 8200, 1e-3)
    for d, g in zip(g_dev, gs):
        d.copy_(_dev(g))
    L.check(L.lib().eri_adam8bit_fn_update_many(opt, names, arr(bufs[0]), arr(g_dev), numels, tags, None, arr(third), n), "update_many")
    L.check(L.lib().eri_adam8bit_fn_step(opt), "fn_step")
    hs.oracle_step(ps, gs, states, (LR, B1, B2, EPS, WD, 6), True, oc.MODE_L2)
    L.check(L.lib().eri_adam8bit_fn_table_stats(opt, C.byref(flushes), C.byref(uploads)), "table_stats")
    assert (flushes.value, uploads.value) == (7, 3)
    torch.cuda.synchronize()
    for i in range(n):
        assert np.array_equal(_bits(third[i], np.uint16), ps[i])
    L.check(L.lib().eri_adam8bit_fn_destroy(opt), "destroy")


def test_a_refused_update_many_runs_nothing_and_leaves_no_state_behind():
    """Every row is validated and every new state created before the first launch: a call with one bad row
    changes no parameter, creates no state and queues nothing, whether the bad row comes first or last, and also
    when a name repeats before it (which would otherwise split the call into two launches)."""
    import torch
    L = _L()
    sizes = [4096, 2048 + 8, 1024]
    n = len(sizes)
    ps, gs = hs.make_inputs(sizes, True, 77)
    p_dev = [_dev(p) for p in ps]
    g_dev = [_dev(g) for g in gs]
    outs = [torch.zeros_like(p) for p in p_dev]
    opt = C.c_void_p()
    L.check(L.lib().eri_adam8bit_fn_with_params(LR, B1, B2, EPS, WD, torch.cuda.current_stream().cuda_stream, C.byref(opt)), "with_params")
    cnt, nbytes = C.c_uint64(), C.c_uint64()

    def call(names, idx, tags=None, numels=None):
        k = len(idx)
        return L.lib().eri_adam8bit_fn_update_many(
            opt, (C.c_char_p * k)(*names), (C.c_void_p * k)(*[p_dev[i].data_ptr() for i in idx]),
            (C.c_void_p * k)(*[g_dev[i].data_ptr() for i in idx]), (C.c_uint64 * k)(*(numels or [sizes[i] for i in idx])),
            (C.c_int32 * k)(*(tags or [L.DTYPE_BF16] * k)), None, (C.c_void_p * k)(*[outs[i].data_ptr() for i in idx]), k)

    # a bad dtype tag in the last row
    assert call([b"a", b"b", b"c"], [0, 1, 2], tags=[L.DTYPE_BF16, L.DTYPE_BF16, 1]) == -4
    # a repeated name (which splits the call) followed by an empty tensor
    assert call([b"a", b"a", b"c"], [0, 0, 2], numels=[sizes[0], sizes[0], 0]) == -3
    L.check(L.lib().eri_adam8bit_fn_step(opt), "fn_step")
    torch.cuda.synchronize()
    L.check(L.lib().eri_adam8bit_fn_memory_stats(opt, C.byref(cnt), C.byref(nbytes)), "memory_stats")
    assert (cnt.value, nbytes.value) == (0, 0)
    assert all(int(o.count_nonzero()) == 0 for o in outs)
    # a state that exists with another size: refused before the new name of the same call gets a state
    L.check(call([b"a"], [0]), "update_many")
    assert call([b"d", b"a"], [1, 2]) == -6
    L.check(L.lib().eri_adam8bit_fn_memory_stats(opt, C.byref(cnt), C.byref(nbytes)), "memory_stats")
    assert cnt.value == 1
    assert int(outs[1].count_nonzero()) == 0
    L.check(L.lib().eri_adam8bit_fn_destroy(opt), "destroy")
