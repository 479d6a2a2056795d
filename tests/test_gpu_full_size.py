"""Parity at the full size of the two full fine-tune configurations: the FLUX-12B-shaped set (780 bf16
tensors, 11.9e9 parameters, ~72 GB resident) and the SDXL-UNet-shaped set (1,680 tensors from 4 to
29.5e6 elements, 2.57e9 parameters, 828 of them with a partial last block).  The oracle cannot sweep
those in reasonable time, so the check is
(a) the oracle on a sample of blocks -- first, last and partial blocks of tensors plus random ones --
whose inputs are copied out before the step, and (b) properties that hold for every block and are
cheap to evaluate on the device: each block's largest second moment carries code 255 and its largest
first moment code 0 or 255 (value / absmax = +-1 exactly), absmax is positive and finite, and no
code outside a tensor's extent was touched (guard values between tensors survive)."""
import ctypes as C

import numpy as np
import pytest

import harness as hs
import oracle_c as oc

pytestmark = pytest.mark.gpu
BLOCK = 2048


def test_flux12b_full_size_sampled_blocks_and_block_properties():
    from eridiffusion_amd import workloads as W
    _full_size(W.c5_flux_full(), 0xE21D + 5, 11_901_408_320, 5_811_496, 80e9)


def test_sdxl_unet_full_size_sampled_blocks_and_block_properties():
    from eridiffusion_amd import workloads as W
    _full_size(W.c4_sdxl_full(), 0xE21D + 4, 2_567_463_684, 1_254_022, 20e9)


def test_sdxl_unet_full_size_with_f32_gradients_for_bf16_parameters():
    """The same table with the gradients left in F32 (what the reference's upcast amounts to when autograd
    hands back F32 gradients): the prefetching kernel's two-waves-per-SIMD variant at its real size."""
    from eridiffusion_amd import workloads as W
    _full_size(W.c4_sdxl_full(), 0xE21D + 41, 2_567_463_684, 1_254_022, 26e9, layout="bf16_grad_f32")


def test_sdxl_unet_full_size_with_f32_parameters():
    from eridiffusion_amd import workloads as W
    _full_size(W.c4_sdxl_full(), 0xE21D + 42, 2_567_463_684, 1_254_022, 32e9, layout="f32")


def _full_size(tensors, seed, want_numel, want_blocks, need_bytes, layout="bf16"):
    import torch
    from eridiffusion_amd import _lib as L
    from eridiffusion_amd import workloads as W

    free, total = torch.cuda.mem_get_info()
    if free < need_bytes:
        pytest.skip("needs %.0f GB of free device memory" % (need_bytes / 1e9))
    sizes = [W.numel(s) for _, s in tensors]
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed)
    GUARD = 256  # poisoned bytes after every tensor's codes
    p_bf16 = layout != "f32"
    g_bf16 = layout == "bf16"
    psz, gsz = (2 if p_bf16 else 4), (2 if g_bf16 else 4)
    p_t = torch.bfloat16 if p_bf16 else torch.float32
    g_t = torch.bfloat16 if g_bf16 else torch.float32
    p_np = np.uint16 if p_bf16 else np.float32
    g_np = np.uint16 if g_bf16 else np.float32

    def arena(byte_sizes):
        offs, tot = [], 0
        for b in byte_sizes:
            offs.append(tot)
            tot += (b + GUARD + 255) // 256 * 256
        return torch.empty(tot, dtype=torch.uint8, device=dev), offs

    p_buf, p_off = arena([psz * n for n in sizes])
    g_buf, g_off = arena([gsz * n for n in sizes])
    m_buf, m_off = arena(sizes)
    v_buf, v_off = arena(sizes)
    nbs = [(n + BLOCK - 1) // BLOCK for n in sizes]
    am_buf, am_off = arena([4 * b for b in nbs])
    av_buf, av_off = arena([4 * b for b in nbs])
    m_buf.fill_(0xEE)
    v_buf.fill_(0xEE)
    stream = torch.cuda.current_stream().cuda_stream
    rows = (L.TensorRow * len(sizes))()
    start = 0
    for i, n in enumerate(sizes):
        p_buf[p_off[i]:p_off[i] + psz * n].view(p_t).copy_(torch.randn(n, device=dev, generator=gen).mul_(0.02))
        g_buf[g_off[i]:g_off[i] + gsz * n].view(g_t).copy_(torch.randn(n, device=dev, generator=gen).mul_(1e-3))
        r = rows[i]
        r.p, r.g = p_buf.data_ptr() + p_off[i], g_buf.data_ptr() + g_off[i]
        r.m, r.v = m_buf.data_ptr() + m_off[i], v_buf.data_ptr() + v_off[i]
        r.absmax_m, r.absmax_v = am_buf.data_ptr() + am_off[i], av_buf.data_ptr() + av_off[i]
        r.numel, r.block_start, r.dtype_tag, r.grad_scale = n, start, (L.DTYPE_BF16 if p_bf16 else L.DTYPE_F32), 1.0
        r.grad_f32 = 1 if layout == "bf16_grad_f32" else 0
        start += nbs[i]
        L.check(L.lib().eri_adam8_state_init(r.m, r.v, r.absmax_m, r.absmax_v, n, stream), "state_init")
    table = C.c_void_p()
    L.check(L.lib().eri_adam8_table_create(rows, len(rows), stream, C.byref(table)), "table_create")
    total_numel, total_blocks = C.c_uint64(), C.c_uint64()
    L.check(L.lib().eri_adam8_table_info(table, C.byref(total_numel), C.byref(total_blocks)), "table_info")
    assert total_numel.value == want_numel and total_blocks.value == want_blocks

    rng = np.random.default_rng(3)
    sample = set()
    for i in range(len(sizes)):
        sample.add((i, 0))
        sample.add((i, nbs[i] - 1))
    big = [i for i in range(len(sizes)) if nbs[i] > 4]
    for _ in range(400):
        i = int(rng.choice(big))
        sample.add((i, int(rng.integers(0, nbs[i]))))
    sample = sorted(sample)

    def grab():
        out = []
        for i, b in sample:
            lo = b * BLOCK
            n = min(BLOCK, sizes[i] - lo)
            out.append((p_buf[p_off[i] + psz * lo:p_off[i] + psz * (lo + n)].cpu().numpy().view(p_np).copy(),
                        g_buf[g_off[i] + gsz * lo:g_off[i] + gsz * (lo + n)].cpu().numpy().view(g_np).copy(),
                        m_buf[m_off[i] + lo:m_off[i] + lo + n].cpu().numpy().copy(),
                        v_buf[v_off[i] + lo:v_off[i] + lo + n].cpu().numpy().copy(),
                        am_buf[am_off[i] + 4 * b:am_off[i] + 4 * b + 4].cpu().numpy().view(np.float32).copy(),
                        av_buf[av_off[i] + 4 * b:av_off[i] + 4 * b + 4].cpu().numpy().view(np.float32).copy()))
        return out

    hyper = (1e-4, 0.9, 0.999, 1e-8, 0.01)
    flips = 0
    for t in (1, 2, 3, 4):  # two steps on the default arithmetic, then two with the IEEE chain
        exact = t > 2
        before = grab()
        h = L.hyper_pack(*hyper, t, L.MODE_ERI, L.FLAG_EXACT_PARAM if exact else 0)
        L.check(L.lib().eri_adam8_step_table(table, C.byref(h), stream), "step_table")
        torch.cuda.synchronize()
        after = grab()
        ho = oc.hyper_pack(*hyper, t)
        for (p, g, m, v, am, av), got in zip(before, after):
            rc = oc.step_tensor(p, g, m, v, am, av, ho, hs.MAPS, oc.DT_BF16 if p_bf16 else oc.DT_F32, 1,
                                g_dtype=oc.DT_BF16 if g_bf16 else oc.DT_F32)
            assert rc == 0
            assert np.array_equal(got[2], m) and np.array_equal(got[3], v)
            assert np.array_equal(got[4].view(np.uint32), am.view(np.uint32))
            assert np.array_equal(got[5].view(np.uint32), av.view(np.uint32))
            if p_bf16:
                d = hs.bf16_ulp_distance(got[0], p)
                assert d.max() <= (0 if exact else 1)
                flips += int((d != 0).sum())
            else:  # fp32 parameters take the IEEE chain whatever the flag says
                assert np.array_equal(got[0].view(np.uint32), p.view(np.uint32))
    print("full-size sample of %d tensors (%s): %d blocks x (2 default + 2 exact) steps, bf16 parameters one ulp off: %d" %
          (len(sizes), layout, len(sample), flips), flush=True)

    # properties of every block
    for i, n in enumerate(sizes):
        nf = n // BLOCK
        if nf:
            mv = m_buf[m_off[i]:m_off[i] + nf * BLOCK].view(nf, BLOCK)
            vv = v_buf[v_off[i]:v_off[i] + nf * BLOCK].view(nf, BLOCK)
            assert bool((vv.max(dim=1).values == 255).all())
            assert bool(((mv.max(dim=1).values == 255) | (mv.min(dim=1).values == 0)).all())
        am = am_buf[am_off[i]:am_off[i] + 4 * nbs[i]].view(torch.float32)
        av = av_buf[av_off[i]:av_off[i] + 4 * nbs[i]].view(torch.float32)
        assert bool(torch.isfinite(am).all()) and bool((am > 0).all()) and bool((av > 0).all())
        assert bool((m_buf[m_off[i] + n:m_off[i] + n + GUARD] == 0xEE).all())
        assert bool((v_buf[v_off[i] + n:v_off[i] + n + GUARD] == 0xEE).all())
    L.lib().eri_adam8_table_destroy(table)


def test_one_tensor_past_two_to_the_32_elements():
    """64-bit element offsets: a single bf16 tensor of 2**32 + 3*2048 + 5 elements (26 GB with its
    gradient and states).  Blocks on both sides of element 2**32, the first, the last full and the
    partial last block are checked against the oracle; every block must satisfy the code-255 property."""
    import torch
    from eridiffusion_amd import _lib as L

    free, _ = torch.cuda.mem_get_info()
    if free < 40e9:
        pytest.skip("needs ~30 GB of free device memory")
    n = (1 << 32) + 3 * BLOCK + 5
    nb = (n + BLOCK - 1) // BLOCK
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev)
    gen.manual_seed(99)
    p = torch.empty(n, dtype=torch.bfloat16, device=dev)
    g = torch.empty(n, dtype=torch.bfloat16, device=dev)
    step = 1 << 28
    for lo in range(0, n, step):  # fill in pieces: randn over 2**32 elements at once would need 17 GB of fp32
        hi = min(n, lo + step)
        p[lo:hi] = torch.randn(hi - lo, device=dev, generator=gen).mul_(0.02)
        g[lo:hi] = torch.randn(hi - lo, device=dev, generator=gen).mul_(1e-3)
    GUARD = 256
    m = torch.full((n + GUARD,), 0xEE, dtype=torch.uint8, device=dev)
    v = torch.full((n + GUARD,), 0xEE, dtype=torch.uint8, device=dev)
    am = torch.empty(nb, dtype=torch.float32, device=dev)
    av = torch.empty(nb, dtype=torch.float32, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    L.check(L.lib().eri_adam8_state_init(m.data_ptr(), v.data_ptr(), am.data_ptr(), av.data_ptr(), n, stream), "state_init")
    row = (L.TensorRow * 1)()
    r = row[0]
    r.p, r.g, r.m, r.v, r.absmax_m, r.absmax_v = p.data_ptr(), g.data_ptr(), m.data_ptr(), v.data_ptr(), am.data_ptr(), av.data_ptr()
    r.numel, r.block_start, r.dtype_tag, r.grad_scale = n, 0, L.DTYPE_BF16, 1.0
    table = C.c_void_p()
    L.check(L.lib().eri_adam8_table_create(row, 1, stream, C.byref(table)), "table_create")
    edge = (1 << 32) // BLOCK
    sample = [0, 1, edge - 2, edge - 1, edge, edge + 1, edge + 2, nb - 2, nb - 1, 12345, edge // 2, edge + 1 - 7]

    def grab():
        out = []
        for b in sample:
            lo = b * BLOCK
            k = min(BLOCK, n - lo)
            out.append((p[lo:lo + k].view(torch.int16).cpu().numpy().view(np.uint16).copy(),
                        g[lo:lo + k].view(torch.int16).cpu().numpy().view(np.uint16).copy(),
                        m[lo:lo + k].cpu().numpy().copy(), v[lo:lo + k].cpu().numpy().copy(),
                        am[b:b + 1].cpu().numpy().copy(), av[b:b + 1].cpu().numpy().copy()))
        return out

    hyper = (1e-4, 0.9, 0.999, 1e-8, 0.01)
    for t in (1, 2):
        before = grab()
        h = L.hyper_pack(*hyper, t, L.MODE_ERI, L.FLAG_EXACT_PARAM)
        L.check(L.lib().eri_adam8_step_table(table, C.byref(h), stream), "step_table")
        torch.cuda.synchronize()
        after = grab()
        ho = oc.hyper_pack(*hyper, t)
        for b, (pp, gg, mm, vv, a1, a2), got in zip(sample, before, after):
            assert oc.step_tensor(pp, gg, mm, vv, a1, a2, ho, hs.MAPS, oc.DT_BF16, 1) == 0
            assert np.array_equal(got[0], pp), b
            assert np.array_equal(got[2], mm) and np.array_equal(got[3], vv), b
            assert np.array_equal(got[4].view(np.uint32), a1.view(np.uint32)), b
            assert np.array_equal(got[5].view(np.uint32), a2.view(np.uint32)), b
    nf = n // BLOCK
    assert bool((v[:nf * BLOCK].view(nf, BLOCK).max(dim=1).values == 255).all())
    assert bool(torch.isfinite(am).all()) and bool((am > 0).all()) and bool((av > 0).all())
    assert bool((m[n:] == 0xEE).all()) and bool((v[n:] == 0xEE).all())
    # the gradient norm pass walks the same offsets
    L.check(L.lib().eri_adam8_grad_norm(table, 1.0, 0.0, stream), "grad_norm")
    norm, scale = C.c_float(), C.c_float()
    L.check(L.lib().eri_adam8_grad_norm_read(table, C.byref(norm), C.byref(scale), stream), "norm_read")
    want = 0.0
    for lo in range(0, n, step):
        want += float(g[lo:min(n, lo + step)].float().double().pow(2).sum())
    assert abs(norm.value - want ** 0.5) <= 2e-6 * want ** 0.5
    L.lib().eri_adam8_table_destroy(table)
