"""The steady-state step allocates nothing and synchronises nothing, so a caller can capture it in a HIP
graph (useful for the launch-bound LoRA-sized workloads).  The graph holds the gradient-norm pass and the
step that consumes its clip factor; it is replayed several times with eager work and synchronisations in
between, and every replay is checked against the same sequence issued eagerly on a second copy."""
import ctypes as C

import numpy as np
import pytest

import harness as hs

pytestmark = pytest.mark.gpu
LR, B1, B2, EPS, WD = 1e-4, 0.9, 0.999, 1e-8, 0.01


@pytest.mark.parametrize("bf16", [True, False])
def test_graph_replays_equal_eager_steps(bf16):
    import torch
    from eridiffusion_amd import _lib as L
    sizes = [2048 * 6 + 100, 640, 2048, 5120, 33]
    ps, gs = hs.make_inputs(sizes, bf16, 71 + bf16, g_std=1e-2)
    copies = []
    for _ in range(2):
        states = hs.oracle_states(sizes)
        gt = hs.GpuTensors([p.copy() for p in ps], [g.copy() for g in gs], states, bf16)
        rows = gt.rows()
        table = C.c_void_p()
        L.check(L.lib().eri_adam8_table_create(rows, len(rows), None, C.byref(table)), "table_create")
        copies.append((gt, table))
    (gt_e, tab_e), (gt_g, tab_g) = copies
    h = L.hyper_pack(LR, B1, B2, EPS, WD, 3, L.MODE_ERI, L.FLAG_CLIP_FROM_TABLE)

    def issue(table, stream):
        L.check(L.lib().eri_adam8_grad_norm(table, 0.05, 0.0, stream), "grad_norm")
        L.check(L.lib().eri_adam8_step_table(table, C.byref(h), stream), "step_table")

    # warm-up outside the capture: the first norm pass allocates the table's partial sums
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        issue(tab_g, side.cuda_stream)
    side.synchronize()
    issue(tab_e, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        issue(tab_g, torch.cuda.current_stream().cuda_stream)
    for replay in range(4):
        graph.replay()
        issue(tab_e, torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        pe, se = gt_e.fetch()
        pg, sg = gt_g.fetch()
        for a, b in zip(pe, pg):
            assert np.array_equal(a, b), replay
        for sa, sb in zip(se, sg):
            for a, b in zip(sa, sb):
                assert np.array_equal(a.view(np.uint8), b.view(np.uint8)), replay
        na, nb_ = C.c_float(), C.c_float()
        sc_a, sc_b = C.c_float(), C.c_float()
        L.check(L.lib().eri_adam8_grad_norm_read(tab_e, C.byref(na), C.byref(sc_a), None), "read")
        L.check(L.lib().eri_adam8_grad_norm_read(tab_g, C.byref(nb_), C.byref(sc_b), None), "read")
        assert na.value == nb_.value and sc_a.value == sc_b.value and sc_a.value < 1.0
        # eager work between replays: new gradients for both copies
        scratch = torch.randn(512, 512, device="cuda")
        scratch = (scratch @ scratch).sum()  # unrelated eager work, library reductions included
        fresh = hs.fresh_grads(sizes, bf16, 500 + replay, 1e-2)
        gt_e.set_grads(fresh)
        gt_g.set_grads(fresh)
        torch.cuda.synchronize()
    L.lib().eri_adam8_table_destroy(tab_e)
    L.lib().eri_adam8_table_destroy(tab_g)
