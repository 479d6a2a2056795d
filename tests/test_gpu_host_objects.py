"""GPU tests of the optimizer objects (include/eri_adam8bit.h) against the oracle: the list-of-
parameters step with a skipped parameter and folded gradient scales, save/load of the 8-bit state
(read back with the safetensors package), and the functional per-tensor flavour."""
import ctypes as C

import numpy as np
import pytest

import harness as hs
import oracle_c as oc
from oracle import adam8_numpy as onp

pytestmark = pytest.mark.gpu
LR, B1, B2, EPS, WD = 1e-3, 0.9, 0.999, 1e-8, 0.01


def _L():
    from eridiffusion_amd import _lib
    return _lib


def _sync():
    import torch
    torch.cuda.synchronize()


def _make(sizes, bf16, seed):
    ps, gs = hs.make_inputs(sizes, bf16, seed)
    states = hs.oracle_states(sizes)
    gt = hs.GpuTensors(ps, gs, states, bf16)
    return ps, gs, states, gt


def _new_optimizer(gt, stream=None, flags=2):
    L = _L()
    n = len(gt.p)
    handles = (C.c_void_p * n)()
    for i in range(n):
        h = C.c_void_p()
        L.check(L.lib().eri_param_create(gt.ptr(gt.p[i]), gt.p[i][2], 2 if gt.bf16 else 0, C.byref(h)), "param_create")
        handles[i] = h
    cfg = L.Adam8bitConfigC()
    L.lib().eri_adam8bit_config_default(C.byref(cfg))
    opt = C.c_void_p()
    L.check(L.lib().eri_adam8bit_new(handles, n, C.byref(cfg), stream, C.byref(opt)), "adam8bit_new")
    if flags is not None:
        L.check(L.lib().eri_adam8bit_set_flags(opt, flags), "set_flags")
    return opt, handles


def _fetch_states(opt, gt):
    import torch
    L = _L()
    out = []
    for i in range(len(gt.p)):
        ptrs = [C.c_void_p() for _ in range(4)]
        L.check(L.lib().eri_adam8bit_state_ptrs(opt, i, *[C.byref(p) for p in ptrs]), "state_ptrs")
        if not ptrs[0].value:
            out.append(None)
            continue
        n = gt.p[i][2]
        nb = (n + 2047) // 2048
        arrs = []
        for p, (cnt, dt) in zip(ptrs, ((n, np.uint8), (n, np.uint8), (nb, np.float32), (nb, np.float32))):
            host = np.empty(cnt, dt)
            L.check(L.lib().eri_hip_memcpy_async(host.ctypes.data, p.value, host.nbytes, 2, None), "d2h")
            L.check(L.lib().eri_hip_stream_sync(None), "sync")
            arrs.append(host)
        out.append(arrs)
    return out


@pytest.mark.parametrize("bf16", [True, False])
def test_step_over_parameter_list_with_a_missing_gradient(bf16, capfd):
    L = _L()
    sizes = [2048 * 3 + 11, 777, 2048 * 2, 5000]
    ps, gs, states, gt = _make(sizes, bf16, 41 + bf16)
    opt, handles = _new_optimizer(gt)
    live = [0, 2, 3]  # parameter 1 never gets a gradient
    for t in (1, 2, 3):
        g_t = hs.fresh_grads(sizes, bf16, 900 + t)
        gt.set_grads(g_t)
        for i in range(4):
            L.check(L.lib().eri_param_set_grad(handles[i], gt.ptr(gt.g[i]) if i in live else None), "set_grad")
        skipped = C.c_uint32()
        L.check(L.lib().eri_adam8bit_step(opt, C.byref(skipped)), "step")
        assert skipped.value == 1
        for i in live:
            hs.oracle_step([ps[i]], [g_t[i]], [states[i]], (LR, B1, B2, EPS, WD, t), bf16)
    _sync()
    assert "No gradient for param_1" in capfd.readouterr().err
    got_p = [gt.down(b) for b in gt.p]
    got_st = _fetch_states(opt, gt)
    assert got_st[1] is None  # no state was created for the parameter without gradients
    assert np.array_equal(got_p[1], ps[1])
    hs.compare([got_p[i] for i in live], [got_st[i] for i in live], [ps[i] for i in live],
               [states[i] for i in live], bf16, True, "host-step")
    want_bytes = sum(2 * sizes[i] + 8 * ((sizes[i] + 2047) // 2048) for i in live)
    assert L.lib().eri_adam8bit_quantized_memory_usage(opt) == want_bytes
    assert L.lib().eri_adam8bit_get_step(opt) == 3
    L.lib().eri_adam8bit_destroy(opt)


def test_a_new_optimizer_reproduces_bf16_parameters_bit_for_bit_without_any_flag_set():
    """24 million element-steps: the faster chain (flags 0) leaves a few dozen parameters one bf16 ulp
    away at this size, so the comparison passes only if the object starts in the exact arithmetic."""
    L = _L()
    sizes = [2048 * 1500 + 7, 2048 * 2000, 2048 * 500 + 1023]
    ps, gs, states, gt = _make(sizes, True, 47)
    opt, handles = _new_optimizer(gt, flags=None)
    for t in (1, 2, 3):
        g_t = hs.fresh_grads(sizes, True, 950 + t)
        gt.set_grads(g_t)
        for i in range(len(sizes)):
            L.check(L.lib().eri_param_set_grad(handles[i], gt.ptr(gt.g[i])), "set_grad")
        L.check(L.lib().eri_adam8bit_step(opt, None), "step")
        hs.oracle_step(ps, g_t, states, (LR, B1, B2, EPS, WD, t), True)
    _sync()
    hs.compare([gt.down(b) for b in gt.p], _fetch_states(opt, gt), ps, states, True, True, "host-default-flags")
    L.lib().eri_adam8bit_destroy(opt)


def test_clip_factor_and_per_parameter_multiplier_are_folded_in():
    L = _L()
    sizes = [2048 * 2 + 5, 4096]
    ps, gs, states, gt = _make(sizes, True, 51)
    opt, handles = _new_optimizer(gt)
    L.check(L.lib().eri_adam8bit_set_grad_scale(opt, 0.5), "grad_scale")
    L.check(L.lib().eri_adam8bit_set_param_grad_scale(opt, 1, 0.25), "param_scale")
    for i in range(2):
        L.check(L.lib().eri_param_set_grad(handles[i], gt.ptr(gt.g[i])), "set_grad")
    L.check(L.lib().eri_adam8bit_step(opt, None), "step")
    _sync()
    # the kernel multiplies by hyper.grad_scale * tensor.grad_scale, one product, one multiply
    for i, s in enumerate((np.float32(0.5) * np.float32(1.0), np.float32(0.5) * np.float32(0.25))):
        hs.oracle_step([ps[i]], [gs[i]], [states[i]], (LR, B1, B2, EPS, WD, 1), True, grad_scale=float(s))
    hs.compare([gt.down(b) for b in gt.p], _fetch_states(opt, gt), ps, states, True, True, "host-scales")
    L.lib().eri_adam8bit_destroy(opt)


def test_save_and_load_state_round_trip(tmp_path):
    from safetensors import safe_open
    L = _L()
    sizes = [2048 * 2 + 100, 300, 4096]
    ps, gs, states, gt = _make(sizes, True, 61)
    opt, handles = _new_optimizer(gt)
    for i in range(3):
        L.check(L.lib().eri_param_set_grad(handles[i], gt.ptr(gt.g[i])), "set_grad")
    for t in (1, 2):
        L.check(L.lib().eri_adam8bit_step(opt, None), "step")
        hs.oracle_step(ps, gs, states, (LR, B1, B2, EPS, WD, t), True)
    L.check(L.lib().eri_adam8bit_set_learning_rate(opt, 7e-4), "set_lr")
    path = str(tmp_path / "optimizer.safetensors")
    L.check(L.lib().eri_adam8bit_save_state(opt, path.encode()), "save_state")
    with safe_open(path, framework="np") as f:
        meta = f.metadata()
        assert meta["step"] == "2" and float(meta["learning_rate"]) == 7e-4 and meta["block_size"] == "2048"
        for i in range(3):
            base = "optimizer.param_%d" % i
            assert np.array_equal(f.get_tensor(base + ".m"), states[i][0])
            assert np.array_equal(f.get_tensor(base + ".v"), states[i][1])
            assert np.array_equal(f.get_tensor(base + ".absmax_m").view(np.uint32), states[i][2].view(np.uint32))
            assert np.array_equal(f.get_tensor(base + ".absmax_v").view(np.uint32), states[i][3].view(np.uint32))
    # a fresh optimizer over the same parameters resumes from the file and takes the same third step
    opt2, handles2 = _new_optimizer(gt)
    L.check(L.lib().eri_adam8bit_load_state(opt2, path.encode()), "load_state")
    assert L.lib().eri_adam8bit_get_step(opt2) == 2 and L.lib().eri_adam8bit_current_lr(opt2) == 7e-4
    for i in range(3):
        L.check(L.lib().eri_param_set_grad(handles2[i], gt.ptr(gt.g[i])), "set_grad")
    L.check(L.lib().eri_adam8bit_step(opt2, None), "step")
    _sync()
    hs.oracle_step(ps, gs, states, (7e-4, B1, B2, EPS, WD, 3), True)
    hs.compare([gt.down(b) for b in gt.p], _fetch_states(opt2, gt), ps, states, True, True, "resume")
    L.lib().eri_adam8bit_destroy(opt)
    L.lib().eri_adam8bit_destroy(opt2)


def test_state_larger_than_the_staging_buffer_round_trips(tmp_path):
    """The file is written and read in 32 MiB pieces through pinned memory; a 72 Mi-element state takes
    three pieces per moment, the last one partial, and a second small parameter follows it in the file.
    The device state is filled with a known byte pattern so that a misplaced piece shows."""
    import torch
    from safetensors import safe_open
    L = _L()
    big = 72 * (1 << 20) + 12345
    sizes = [big, 5000]
    dev = torch.device("cuda:0")
    p = [torch.zeros(n, dtype=torch.bfloat16, device=dev) for n in sizes]
    g = [torch.full((n,), 1e-3, dtype=torch.bfloat16, device=dev) for n in sizes]
    handles = (C.c_void_p * 2)()
    for i in range(2):
        h = C.c_void_p()
        L.check(L.lib().eri_param_create(p[i].data_ptr(), sizes[i], 2, C.byref(h)), "param_create")
        L.check(L.lib().eri_param_set_grad(h, g[i].data_ptr()), "set_grad")
        handles[i] = h

    def new_opt():
        opt = C.c_void_p()
        L.check(L.lib().eri_adam8bit_new(handles, 2, None, None, C.byref(opt)), "adam8bit_new")
        return opt

    def state_views(opt, i):
        ptrs = [C.c_void_p() for _ in range(4)]
        L.check(L.lib().eri_adam8bit_state_ptrs(opt, i, *[C.byref(q) for q in ptrs]), "state_ptrs")
        return ptrs

    opt = new_opt()
    L.check(L.lib().eri_adam8bit_step(opt, None), "step")  # creates the states
    _sync()
    want = []
    gen = torch.Generator(device=dev)
    gen.manual_seed(99)
    for i, n in enumerate(sizes):
        nb = (n + 2047) // 2048
        ptrs = state_views(opt, i)
        arrs = []
        for q, (nbytes, dt) in zip(ptrs, ((n, torch.uint8), (n, torch.uint8), (4 * nb, torch.float32), (4 * nb, torch.float32))):
            if dt is torch.uint8:
                src = torch.randint(0, 256, (nbytes,), dtype=torch.uint8, device=dev, generator=gen)
            else:
                src = torch.rand(nbytes // 4, dtype=torch.float32, device=dev, generator=gen)
            L.check(L.lib().eri_hip_memcpy_async(q.value, src.data_ptr(), nbytes, 3, None), "fill")
            arrs.append(src.cpu().numpy())
        want.append(arrs)
    _sync()
    path = str(tmp_path / "big.safetensors")
    L.check(L.lib().eri_adam8bit_save_state(opt, path.encode()), "save_state")
    with safe_open(path, framework="np") as f:
        for i in range(2):
            base = "optimizer.param_%d" % i
            for k, name in enumerate((".m", ".v", ".absmax_m", ".absmax_v")):
                got = f.get_tensor(base + name)
                assert np.array_equal(got.view(np.uint8), want[i][k].view(np.uint8)), base + name
    opt2 = new_opt()
    L.check(L.lib().eri_adam8bit_load_state(opt2, path.encode()), "load_state")
    assert L.lib().eri_adam8bit_get_step(opt2) == 1
    for i, n in enumerate(sizes):
        nb = (n + 2047) // 2048
        for q, w, nbytes in zip(state_views(opt2, i), want[i], (n, n, 4 * nb, 4 * nb)):
            back = torch.empty(nbytes, dtype=torch.uint8, device=dev)
            L.check(L.lib().eri_hip_memcpy_async(back.data_ptr(), q.value, nbytes, 3, None), "read")
            _sync()
            assert np.array_equal(back.cpu().numpy(), w.view(np.uint8))
    # a file cut inside the big tensor is refused and leaves the optimizer as it was
    cut = tmp_path / "cut.safetensors"
    with open(path, "rb") as f:
        blob = f.read(40 * (1 << 20))
    cut.write_bytes(blob)
    before = [q.value for q in state_views(opt2, 0)]
    assert L.lib().eri_adam8bit_load_state(opt2, str(cut).encode()) == -6
    assert [q.value for q in state_views(opt2, 0)] == before
    L.lib().eri_adam8bit_destroy(opt)
    L.lib().eri_adam8bit_destroy(opt2)
    for h in handles:
        L.lib().eri_param_release(h)


def test_functional_updates_of_several_names_in_turn():
    """Three names of different sizes and dtypes updated in turn for three rounds, each call writing
    into a fresh output buffer: every name keeps its own launch table, re-pointed when the addresses
    change."""
    import torch
    L = _L()
    names = [(b"a.lora_down", 2048 * 2 + 9, True), (b"b.lora_up", 700, True), (b"c.bias", 2048 * 5, False)]
    dev = torch.device("cuda:0")
    opt = C.c_void_p()
    L.check(L.lib().eri_adam8bit_fn_with_params(1e-4, B1, B2, EPS, WD, None, C.byref(opt)), "with_params")
    host = {}
    for k, (name, n, bf16) in enumerate(names):
        ps, gs = hs.make_inputs([n], bf16, 300 + k)
        host[name] = [ps, gs, hs.oracle_states([n]), torch.from_numpy(ps[0].view(np.uint8).copy()).to(dev)]
    keep = []
    for rnd in range(3):
        for name, n, bf16 in names:
            ps, gs, states, cur = host[name]
            g_dev = torch.from_numpy(gs[0].view(np.uint8).copy()).to(dev)
            out = torch.zeros(n * (2 if bf16 else 4), dtype=torch.uint8, device=dev)
            keep += [g_dev, out, cur]
            L.check(L.lib().eri_adam8bit_fn_update(opt, name, cur.data_ptr(), g_dev.data_ptr(), n, 2 if bf16 else 0,
                                                   2 if bf16 else 0, out.data_ptr()), "fn_update")
            host[name][3] = out
            hs.oracle_step(ps, gs, states, (1e-4, B1, B2, EPS, WD, rnd), bf16, mode=oc.MODE_L2)
        L.check(L.lib().eri_adam8bit_fn_step(opt), "fn_step")
    _sync()
    for name, n, bf16 in names:
        ps, gs, states, cur = host[name]
        bits = np.uint16 if bf16 else np.uint32
        assert np.array_equal(cur.cpu().numpy().view(bits), ps[0].view(bits)), name
    cnt, nbytes = C.c_uint64(), C.c_uint64()
    L.check(L.lib().eri_adam8bit_fn_memory_stats(opt, C.byref(cnt), C.byref(nbytes)), "memory_stats")
    assert cnt.value == 3
    L.lib().eri_adam8bit_fn_destroy(opt)


@pytest.mark.parametrize("bf16", [True, False])
def test_functional_update_returns_a_new_tensor(bf16):
    import torch
    L = _L()
    n = 2048 * 3 + 77
    ps, gs = hs.make_inputs([n], bf16, 71 + bf16)
    states = hs.oracle_states([n])
    dev = torch.device("cuda:0")
    item = 2 if bf16 else 4
    p_dev = torch.from_numpy(ps[0].view(np.uint8).copy()).to(dev)
    out_dev = torch.zeros(n * item, dtype=torch.uint8, device=dev)
    g_dev = torch.from_numpy(gs[0].view(np.uint8).copy()).to(dev)
    opt = C.c_void_p()
    L.check(L.lib().eri_adam8bit_fn_with_params(1e-4, B1, B2, EPS, WD, None, C.byref(opt)), "with_params")
    p0 = ps[0].copy()
    for call in range(3):  # update, update, step, update: calls 1 and 2 both see counter 0 -> s = 1
        src = p_dev if call == 0 else out_dev
        L.check(L.lib().eri_adam8bit_fn_update(opt, b"layer.lora_down", src.data_ptr(), g_dev.data_ptr(), n,
                                               2 if bf16 else 0, 2 if bf16 else 0, out_dev.data_ptr()), "fn_update")
        step = 0 if call < 2 else 1
        hs.oracle_step(ps, gs, states, (1e-4, B1, B2, EPS, WD, step), bf16, mode=oc.MODE_L2)
        if call == 1:
            L.check(L.lib().eri_adam8bit_fn_step(opt), "fn_step")
    _sync()
    dt = np.uint16 if bf16 else np.float32
    assert np.array_equal(p_dev.cpu().numpy().view(dt), p0)  # the input tensor is left alone
    got = out_dev.cpu().numpy().view(dt)
    assert np.array_equal(got.view(np.uint16 if bf16 else np.uint32), ps[0].view(np.uint16 if bf16 else np.uint32))
    # fp32 export equals the oracle's dequantisation; re-import quantises to the same codes
    m_out = torch.empty(n, dtype=torch.float32, device=dev)
    v_out = torch.empty(n, dtype=torch.float32, device=dev)
    L.check(L.lib().eri_adam8bit_fn_get_state_fp32(opt, b"layer.lora_down", m_out.data_ptr(), v_out.data_ptr()), "get")
    _sync()
    want_m = np.empty(n, np.float32)
    want_v = np.empty(n, np.float32)
    oc.lib().eri_oracle_dequantize(oc.ptr(states[0][0]), oc.ptr(states[0][2]), oc.ptr(hs.MAPS[0]), n, oc.ptr(want_m))
    oc.lib().eri_oracle_dequantize(oc.ptr(states[0][1]), oc.ptr(states[0][3]), oc.ptr(hs.MAPS[1]), n, oc.ptr(want_v))
    assert np.array_equal(m_out.cpu().numpy().view(np.uint32), want_m.view(np.uint32))
    assert np.array_equal(v_out.cpu().numpy().view(np.uint32), want_v.view(np.uint32))
    cnt, nbytes = C.c_uint64(), C.c_uint64()
    L.check(L.lib().eri_adam8bit_fn_memory_stats(opt, C.byref(cnt), C.byref(nbytes)), "memory_stats")
    assert (cnt.value, nbytes.value) == (1, 2 * n + 8 * ((n + 2047) // 2048))
    L.check(L.lib().eri_adam8bit_fn_load_state_fp32(opt, b"other", m_out.data_ptr(), v_out.data_ptr(), n), "load")
    numel = C.c_uint64()
    L.check(L.lib().eri_adam8bit_fn_state_numel(opt, b"other", C.byref(numel)), "numel")
    assert numel.value == n
    L.lib().eri_adam8bit_fn_destroy(opt)


def test_legacy_bincode_state_is_imported_and_requantised(tmp_path):
    import torch
    from test_host_objects_cpu import _bincode_state
    L = _L()
    n = 2048 + 500
    ps, gs, states, gt = _make([n], False, 81)
    rng = np.random.default_rng(4)
    qm = rng.integers(-128, 128, n).tolist()
    qv = rng.integers(-128, 128, n).tolist()
    sm, zm, sv, zv = 3e-5, -7, 2e-9, -128
    path = tmp_path / "optimizer.pt"
    path.write_bytes(_bincode_state(41, 3e-4, {"param_0": (qm, sm, zm, [n], 0.1)}, {"param_0": (qv, sv, zv, [n], 0.1)}))
    opt, handles = _new_optimizer(gt)
    L.check(L.lib().eri_adam8bit_load_legacy_state(opt, str(path).encode()), "load_legacy")
    assert L.lib().eri_adam8bit_get_step(opt) == 41 and L.lib().eri_adam8bit_current_lr(opt) == 3e-4
    got = _fetch_states(opt, gt)[0]
    for k, (q, scale, zp, table) in enumerate(((qm, sm, zm, hs.MAPS[0]), (qv, sv, zv, hs.MAPS[1]))):
        x = ((np.array(q, np.float32) - np.float32(zp)) * np.float32(scale)).astype(np.float32)  # (q - zp) * scale, :121
        codes = np.empty(n, np.uint8)
        absmax = np.empty(2, np.float32)
        oc.lib().eri_oracle_quantize(oc.ptr(x), oc.ptr(table), n, oc.ptr(codes), oc.ptr(absmax))
        assert np.array_equal(got[k], codes)
        assert np.array_equal(got[2 + k].view(np.uint32), absmax.view(np.uint32))
    L.lib().eri_adam8bit_destroy(opt)


def test_legacy_state_longer_than_one_staging_piece(tmp_path):
    """A tensor of 8 Mi + 5000 elements is dequantised in two pieces of pinned memory (the second partial)
    before it is quantised blockwise; a small second parameter follows."""
    import torch
    from test_host_objects_cpu import _bincode_state
    L = _L()
    sizes = [8 * (1 << 20) + 5000, 3000]
    dev = torch.device("cuda:0")
    p = [torch.zeros(n, dtype=torch.float32, device=dev) for n in sizes]
    handles = (C.c_void_p * 2)()
    for i in range(2):
        h = C.c_void_p()
        L.check(L.lib().eri_param_create(p[i].data_ptr(), sizes[i], 0, C.byref(h)), "param_create")
        handles[i] = h
    opt = C.c_void_p()
    L.check(L.lib().eri_adam8bit_new(handles, 2, None, None, C.byref(opt)), "adam8bit_new")
    rng = np.random.default_rng(12)
    q = {(i, k): rng.integers(-128, 128, n, dtype=np.int8) for i, n in enumerate(sizes) for k in (0, 1)}
    par = {(0, 0): (2e-5, 3), (0, 1): (4e-10, -128), (1, 0): (1e-4, -1), (1, 1): (7e-9, -128)}
    first = {"param_%d" % i: (q[i, 0].tobytes(), par[i, 0][0], par[i, 0][1], [n], 0.0) for i, n in enumerate(sizes)}
    second = {"param_%d" % i: (q[i, 1].tobytes(), par[i, 1][0], par[i, 1][1], [n], 0.0) for i, n in enumerate(sizes)}
    path = tmp_path / "optimizer.pt"
    path.write_bytes(_bincode_state(9, 1e-4, first, second))
    L.check(L.lib().eri_adam8bit_load_legacy_state(opt, str(path).encode()), "load_legacy")
    assert L.lib().eri_adam8bit_get_step(opt) == 9
    for i, n in enumerate(sizes):
        nb = (n + 2047) // 2048
        ptrs = [C.c_void_p() for _ in range(4)]
        L.check(L.lib().eri_adam8bit_state_ptrs(opt, i, *[C.byref(x) for x in ptrs]), "state_ptrs")
        for k in (0, 1):
            scale, zp = par[i, k]
            x = ((q[i, k].astype(np.float32) - np.float32(zp)) * np.float32(scale)).astype(np.float32)
            codes = np.empty(n, np.uint8)
            absmax = np.empty(nb, np.float32)
            oc.lib().eri_oracle_quantize(oc.ptr(x), oc.ptr(hs.MAPS[k]), n, oc.ptr(codes), oc.ptr(absmax))
            got_c = np.empty(n, np.uint8)
            got_a = np.empty(nb, np.float32)
            L.check(L.lib().eri_hip_memcpy_async(got_c.ctypes.data, ptrs[k].value, n, 2, None), "d2h")
            L.check(L.lib().eri_hip_memcpy_async(got_a.ctypes.data, ptrs[2 + k].value, 4 * nb, 2, None), "d2h")
            L.check(L.lib().eri_hip_stream_sync(None), "sync")
            assert np.array_equal(got_c, codes)
            assert np.array_equal(got_a.view(np.uint32), absmax.view(np.uint32))
    L.lib().eri_adam8bit_destroy(opt)
    for h in handles:
        L.lib().eri_param_release(h)


def test_min_8bit_size_keeps_short_tensors_in_fp32_moments(tmp_path):
    """Parameters below min_8bit_size take the same update with fp32 moments (one launch of the 32-bit step
    for all of them), the others the 8-bit step; both against their oracles over three steps, then a
    save / load round trip that carries both kinds of state, then two steps with loss scale, per-layer
    multipliers and clipping by the global norm of all gradients, and the refusal of another mode."""
    import torch
    L = _L()
    sizes = [2048 * 3 + 5, 300, 4095, 4096, 64, 2048 * 2]
    dts = [True, True, False, True, True, False]  # bf16?
    small = [n < 4096 for n in sizes]
    dev = torch.device("cuda:0")
    host_p, dev_p, handles = [], [], (C.c_void_p * len(sizes))()
    for i, (n, bf16) in enumerate(zip(sizes, dts)):
        ps, _ = hs.make_inputs([n], bf16, 900 + i)
        host_p.append(ps[0])
        dev_p.append(torch.from_numpy(ps[0].view(np.uint8).copy()).to(dev))
        h = C.c_void_p()
        L.check(L.lib().eri_param_create(dev_p[i].data_ptr(), n, 2 if bf16 else 0, C.byref(h)), "param_create")
        handles[i] = h
    cfg = L.Adam8bitConfigC(1e-4, B1, B2, EPS, WD, 0, 1, 100)

    def make():
        o = C.c_void_p()
        L.check(L.lib().eri_adam8bit_new(handles, len(sizes), C.byref(cfg), None, C.byref(o)), "new")
        L.check(L.lib().eri_adam8bit_set_flags(o, L.FLAG_EXACT_PARAM), "set_flags")
        L.check(L.lib().eri_adam8bit_set_min_8bit_size(o, 4096), "set_min_8bit_size")
        return o

    opt = make()
    states8 = [list(oc.state_init(n)) for n in sizes]
    states32 = [[np.zeros(n, np.float32), np.zeros(n, np.float32)] for n in sizes]
    keep = []

    def one_step(o, t):
        gs = [hs.fresh_grads([n], bf16, 100 * t + i)[0] for i, (n, bf16) in enumerate(zip(sizes, dts))]
        g_dev = [torch.from_numpy(g.view(np.uint8).copy()).to(dev) for g in gs]
        keep.append(g_dev)
        for i in range(len(sizes)):
            L.check(L.lib().eri_param_set_grad(handles[i], g_dev[i].data_ptr()), "set_grad")
        L.check(L.lib().eri_adam8bit_step(o, None), "step")
        h = oc.hyper_pack(1e-4, B1, B2, EPS, WD, t)
        for i, (n, bf16) in enumerate(zip(sizes, dts)):
            dt = oc.DT_BF16 if bf16 else oc.DT_F32
            if small[i]:
                oc.lib().eri_oracle_adamw32_step(oc.ptr(host_p[i]), oc.ptr(gs[i]), oc.ptr(states32[i][0]), oc.ptr(states32[i][1]),
                                                 n, dt, float(h.step_size), B1, B2, EPS, WD, None)
            else:
                assert oc.step_tensor(host_p[i], gs[i], *states8[i], h, hs.MAPS, dt, 2) == 0

    def check(o):
        _sync()
        for i, (n, bf16) in enumerate(zip(sizes, dts)):
            bits = np.uint16 if bf16 else np.uint32
            assert np.array_equal(dev_p[i].cpu().numpy().view(bits), host_p[i].view(bits)), i
            m32, v32 = C.c_void_p(), C.c_void_p()
            L.check(L.lib().eri_adam8bit_state32_ptrs(o, i, C.byref(m32), C.byref(v32)), "state32_ptrs")
            ptrs = [C.c_void_p() for _ in range(4)]
            L.check(L.lib().eri_adam8bit_state_ptrs(o, i, *[C.byref(q) for q in ptrs]), "state_ptrs")
            if small[i]:
                assert m32.value and v32.value and not ptrs[0].value
                for src, want in ((m32, states32[i][0]), (v32, states32[i][1])):
                    got = torch.empty(n, dtype=torch.float32, device=dev)
                    L.check(L.lib().eri_hip_memcpy_async(got.data_ptr(), src.value, 4 * n, 3, None), "memcpy")
                    _sync()
                    assert np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32)), i
            else:
                assert ptrs[0].value and not m32.value
                got = torch.empty(n, dtype=torch.uint8, device=dev)
                L.check(L.lib().eri_hip_memcpy_async(got.data_ptr(), ptrs[0].value, n, 3, None), "memcpy")
                _sync()
                assert np.array_equal(got.cpu().numpy(), states8[i][0]), i

    for t in (1, 2, 3):
        one_step(opt, t)
    check(opt)
    want_bytes = sum(8 * n if s else 2 * n + 8 * ((n + 2047) // 2048) for n, s in zip(sizes, small))
    assert L.lib().eri_adam8bit_quantized_memory_usage(opt) == want_bytes
    # save, load into a fresh optimizer, continue there: same trajectory
    path = tmp_path / "mixed_state.safetensors"
    L.check(L.lib().eri_adam8bit_save_state(opt, str(path).encode()), "save_state")
    _sync()
    L.lib().eri_adam8bit_destroy(opt)
    opt = make()
    L.check(L.lib().eri_adam8bit_load_state(opt, str(path).encode()), "load_state")
    assert L.lib().eri_adam8bit_get_step(opt) == 3
    one_step(opt, 4)
    check(opt)
    # loss scale, a per-layer multiplier on one tensor of either kind and clipping by the global norm, all inside
    # the step: the short tensors get the same factors as the 8-bit ones, and the norm covers every gradient
    # (the trainer that sets min_8bit_size clips all of them: pipeline_flux_lora_1024.rs:451,691-697)
    L.check(L.lib().eri_adam8bit_set_grad_scale(opt, 0.5), "set_grad_scale")
    L.check(L.lib().eri_adam8bit_set_param_grad_scale(opt, 1, 0.25), "param_scale")   # a short tensor
    L.check(L.lib().eri_adam8bit_set_param_grad_scale(opt, 3, 2.0), "param_scale")    # an 8-bit one
    L.check(L.lib().eri_adam8bit_set_max_grad_norm(opt, 0.01, 0.0), "set_max_grad_norm")
    per_param = [1.0, 0.25, 1.0, 2.0, 1.0, 1.0]
    for t in (5, 6):
        gs = [hs.fresh_grads([n], bf16, 100 * t + i)[0] for i, (n, bf16) in enumerate(zip(sizes, dts))]
        g_dev = [torch.from_numpy(g.view(np.uint8).copy()).to(dev) for g in gs]
        keep.append(g_dev)
        for i in range(len(sizes)):
            L.check(L.lib().eri_param_set_grad(handles[i], g_dev[i].data_ptr()), "set_grad")
        L.check(L.lib().eri_adam8bit_step(opt, None), "step")
        norm, scale = C.c_float(), C.c_float()
        L.check(L.lib().eri_adam8bit_last_grad_norm(opt, C.byref(norm), C.byref(scale)), "last_grad_norm")
        g64 = [(onp.bf16_to_f32(g) if bf16 else g).astype(np.float64) for g, bf16 in zip(gs, dts)]
        want = np.sqrt(sum(float((g * g).sum()) for g in g64))  # over all six gradients, unscaled as stored
        assert abs(norm.value - want) <= 2e-6 * want
        assert norm.value > 0.01 and scale.value == np.float32(0.01) / np.float32(norm.value)
        h = oc.hyper_pack(1e-4, B1, B2, EPS, WD, t)
        for i, (n, bf16) in enumerate(zip(sizes, dts)):
            dt = oc.DT_BF16 if bf16 else oc.DT_F32
            factor = float((np.float32(0.5) * np.float32(per_param[i])) * np.float32(scale.value))
            if small[i]:
                oc.lib().eri_oracle_adamw32_step_scaled(oc.ptr(host_p[i]), oc.ptr(gs[i]), oc.ptr(states32[i][0]), oc.ptr(states32[i][1]),
                                                        n, dt, float(h.step_size), B1, B2, EPS, WD, None, factor)
            else:
                hh = oc.hyper_pack(1e-4, B1, B2, EPS, WD, t, grad_scale=factor)
                assert oc.step_tensor(host_p[i], gs[i], *states8[i], hh, hs.MAPS, dt, 2) == 0
    check(opt)
    # the one refusal left: another arithmetic than the reference's own for the 8-bit tensors
    L.check(L.lib().eri_adam8bit_set_mode(opt, L.MODE_BNB), "set_mode")
    assert L.lib().eri_adam8bit_step(opt, None) == -6
    assert b"min_8bit_size" in L.lib().eri_last_error()
    assert L.lib().eri_adam8bit_get_step(opt) == 6  # a refused step counts for nothing
    L.lib().eri_adam8bit_destroy(opt)
    for h in handles:
        L.lib().eri_param_release(h)
