"""The lane pool of the storage seam and the optimizers' states inside it."""
import ctypes as C

import numpy as np
import pytest

import harness as hs
import oracle_c as oc
from oracle import adam8_numpy as onp

pytestmark = pytest.mark.gpu
LR, B1, B2, EPS, WD = 1e-3, 0.9, 0.999, 1e-8, 0.01
MiB = 1 << 20


def _L():
    from eridiffusion_amd import _lib
    return _lib


def _pool(nbytes, lanes):
    L = _L()
    h = C.c_void_p()
    L.check(L.lib().eri_hip_pool_create(0, nbytes, lanes, C.byref(h)), "pool_create")
    return h


def test_lanes_are_equal_parts_of_one_allocation_and_pieces_come_zeroed():
    import torch
    L = _L()
    pool = _pool(64 * MiB, 4)
    lanes, lane_bytes = C.c_uint32(), C.c_size_t()
    L.check(L.lib().eri_hip_pool_info(pool, C.byref(lanes), C.byref(lane_bytes)), "pool_info")
    assert lanes.value == 4 and lane_bytes.value == 16 * MiB
    a, b, c, d = (C.c_void_p() for _ in range(4))
    L.check(L.lib().eri_hip_pool_alloc_zeroed(pool, 0, 1000, C.byref(a)), "alloc")
    L.check(L.lib().eri_hip_pool_alloc_zeroed(pool, 0, 5, C.byref(b)), "alloc")
    L.check(L.lib().eri_hip_pool_alloc_zeroed(pool, 3, 4 * MiB, C.byref(c)), "alloc")
    L.check(L.lib().eri_hip_pool_alloc_zeroed(pool, 6, 256, C.byref(d)), "alloc")  # lane 6 of 4 is lane 2
    assert b.value - a.value == 1024 and a.value % 256 == 0          # 256-byte steps inside a lane
    assert c.value - a.value == 3 * lane_bytes.value                 # lanes are lane_bytes apart
    assert d.value - a.value == 2 * lane_bytes.value
    used = C.c_size_t()
    L.check(L.lib().eri_hip_pool_lane_used(pool, 0, C.byref(used)), "lane_used")
    assert used.value == 1024 + 256
    # dirty a piece, reset, take it again: zero-filled again
    host = np.full(4 * MiB, 0xAB, np.uint8)
    L.check(L.lib().eri_hip_memcpy_async(c.value, host.ctypes.data, host.size, 1, None), "memcpy")
    torch.cuda.synchronize()
    L.check(L.lib().eri_hip_pool_reset(pool), "reset")
    e = C.c_void_p()
    L.check(L.lib().eri_hip_pool_alloc_zeroed(pool, 3, 4 * MiB, C.byref(e)), "alloc")
    assert e.value == c.value
    back = np.empty(4 * MiB, np.uint8)
    L.check(L.lib().eri_hip_memcpy_async(back.ctypes.data, e.value, back.size, 2, None), "memcpy")
    torch.cuda.synchronize()
    assert not back.any()
    # a lane that is full says so and leaves the pool usable
    f = C.c_void_p()
    assert L.lib().eri_hip_pool_alloc_zeroed(pool, 3, 13 * MiB, C.byref(f)) == -6
    assert b"lane is full" in L.lib().eri_last_error()
    L.check(L.lib().eri_hip_pool_alloc_zeroed(pool, 3, 12 * MiB, C.byref(f)), "alloc")
    assert L.lib().eri_hip_pool_alloc_zeroed(None, 0, 16, C.byref(f)) == -1
    assert L.lib().eri_hip_pool_alloc_zeroed(pool, 0, 0, C.byref(f)) == -3
    L.check(L.lib().eri_hip_pool_destroy(pool), "destroy")


@pytest.mark.parametrize("bf16", [True, False])
def test_list_optimizer_with_pooled_states_matches_the_oracle(bf16):
    """The same steps as with states of its own allocation: bit-exact states and (exact flag) parameters; the state
    pointers lie inside the lane that was named."""
    import torch
    from eridiffusion_amd.adam8bit import Adam8bit, Adam8bitConfig, DevicePool
    L = _L()
    sizes = [2048 * 5 + 77, 300, 2048 * 2, 4099]
    ps, gs = hs.make_inputs(sizes, bf16, 321)
    states = hs.oracle_states(sizes)
    dt = torch.bfloat16 if bf16 else torch.float32
    to_t = lambda a: (torch.from_numpy(a.view(np.int16)).cuda().view(torch.bfloat16) if bf16 else torch.from_numpy(a.copy()).cuda())
    params = [to_t(p) for p in ps]
    pool = DevicePool(48 * MiB, 3)
    opt = Adam8bit(params, Adam8bitConfig(lr=LR, betas=(B1, B2), eps=EPS, weight_decay=WD), flags=L.FLAG_EXACT_PARAM)
    opt.set_state_pool(pool, 2)
    for t in (1, 2, 3):
        g_t = hs.fresh_grads(sizes, bf16, 400 + t, 1e-3)
        for p, g in zip(params, g_t):
            p.grad = to_t(g)
        opt.step()
        hs.oracle_step(ps, g_t, states, (LR, B1, B2, EPS, WD, t), bf16)
    torch.cuda.synchronize()
    lane0 = pool.alloc_ptr(0, 256)
    for i, n in enumerate(sizes):
        ptrs = [C.c_void_p() for _ in range(4)]
        L.check(L.lib().eri_adam8bit_state_ptrs(opt._opt, i, *[C.byref(q) for q in ptrs]), "state_ptrs")
        nb = (n + 2047) // 2048
        arrs = []
        for q, (cnt, dtp) in zip(ptrs, ((n, np.uint8), (n, np.uint8), (nb, np.float32), (nb, np.float32))):
            host = np.empty(cnt, dtp)
            L.check(L.lib().eri_hip_memcpy_async(host.ctypes.data, q.value, host.nbytes, 2, None), "d2h")
            L.check(L.lib().eri_hip_stream_sync(None), "sync")
            arrs.append(host)
        m, v, am, av = arrs
        assert np.array_equal(m, states[i][0]) and np.array_equal(v, states[i][1])
        assert np.array_equal(am.view(np.uint32), states[i][2].view(np.uint32))
        assert np.array_equal(av.view(np.uint32), states[i][3].view(np.uint32))
        got = params[i].view(torch.int16).cpu().numpy().view(np.uint16) if bf16 else params[i].cpu().numpy()
        assert np.array_equal(got.view(np.uint16 if bf16 else np.uint32), ps[i].view(np.uint16 if bf16 else np.uint32))
        ptr = ptrs[0].value
        assert lane0 + 2 * pool.lane_bytes <= ptr < lane0 + 3 * pool.lane_bytes
    del opt
    pool.close()


def test_functional_optimizer_with_pooled_states_matches_the_oracle():
    import torch
    from eridiffusion_amd.adam8bit import Adam8bitFunctional, DevicePool
    sizes = [2048 * 3 + 9, 640 * 16, 77]
    ps, _ = hs.make_inputs(sizes, True, 654)
    states = hs.oracle_states(sizes)
    to_t = lambda a: torch.from_numpy(a.view(np.int16)).cuda().view(torch.bfloat16)
    cur = {"t%d" % i: to_t(p) for i, p in enumerate(ps)}
    pool = DevicePool(32 * MiB, 2)
    opt = Adam8bitFunctional(LR, B1, B2, EPS, WD, batched=True)
    opt.set_state_pool(pool, 1)
    for t in range(3):
        g_t = hs.fresh_grads(sizes, True, 700 + t, 1e-3)
        grads = {"t%d" % i: to_t(g) for i, g in enumerate(g_t)}
        cur = opt.update_many(cur, grads)
        opt.step()
        hs.oracle_step(ps, g_t, states, (LR, B1, B2, EPS, WD, t), True, oc.MODE_L2)
    torch.cuda.synchronize()
    for i in range(len(sizes)):
        got = cur["t%d" % i].view(torch.int16).cpu().numpy().view(np.uint16)
        assert np.array_equal(got, ps[i])
    del opt
    pool.close()


def test_released_pieces_are_handed_out_again():
    """eri_hip_pool_release: the top piece lowers the lane's fill level (and takes released pieces right below it
    along), any other piece waits for the next request of exactly its size; the stream-ordered allocation hands out
    cleared memory; pieces that are not the pool's are refused."""
    import torch
    L = _L()
    pool = _pool(32 * MiB, 2)
    used = C.c_size_t()
    a, b, c, d = (C.c_void_p() for _ in range(4))
    stream = torch.cuda.current_stream().cuda_stream
    L.check(L.lib().eri_hip_pool_alloc_zeroed(pool, 0, 1000, C.byref(a)), "alloc")
    L.check(L.lib().eri_hip_pool_alloc_zeroed(pool, 0, 4096, C.byref(b)), "alloc")
    L.check(L.lib().eri_hip_pool_alloc_zeroed(pool, 0, 300, C.byref(c)), "alloc")
    L.check(L.lib().eri_hip_pool_lane_used(pool, 0, C.byref(used)), "lane_used")
    assert used.value == 1024 + 4096 + 512
    # dirty the middle piece, give it back, ask for its size again on a stream: the same piece, cleared
    L.check(L.lib().eri_hip_memset_async(b, 0xAB, 4096, stream), "memset")
    L.check(L.lib().eri_hip_pool_release(pool, b, 4096), "release")
    L.check(L.lib().eri_hip_pool_lane_used(pool, 0, C.byref(used)), "lane_used")
    assert used.value == 1024 + 4096 + 512  # not the top piece: the level stays
    L.check(L.lib().eri_hip_pool_alloc_zeroed_async(pool, 0, 2000, stream, C.byref(d)), "alloc_async")  # another size: from the top
    assert d.value == a.value + 1024 + 4096 + 512
    e = C.c_void_p()
    L.check(L.lib().eri_hip_pool_alloc_zeroed_async(pool, 0, 4000, stream, C.byref(e)), "alloc_async")  # 4000 rounds to 4096
    assert e.value == b.value
    host = np.full(4096, 7, np.uint8)
    L.check(L.lib().eri_hip_memcpy_async(host.ctypes.data, e, 4096, 2, stream), "d2h")
    L.check(L.lib().eri_hip_stream_sync(stream), "sync")
    assert not host.any()
    # top piece back: the level drops to its start; then the piece below it, and the released one under that goes along
    L.check(L.lib().eri_hip_pool_release(pool, d, 2000), "release")
    L.check(L.lib().eri_hip_pool_lane_used(pool, 0, C.byref(used)), "lane_used")
    assert used.value == 1024 + 4096 + 512
    L.check(L.lib().eri_hip_pool_release(pool, e, 4000), "release")
    L.check(L.lib().eri_hip_pool_release(pool, c, 300), "release")
    L.check(L.lib().eri_hip_pool_lane_used(pool, 0, C.byref(used)), "lane_used")
    assert used.value == 1024
    # a piece given back twice would be handed out twice: refused while it waits below the lane's level
    f, g = C.c_void_p(), C.c_void_p()
    L.check(L.lib().eri_hip_pool_alloc_zeroed(pool, 0, 4096, C.byref(f)), "alloc")
    L.check(L.lib().eri_hip_pool_alloc_zeroed(pool, 0, 256, C.byref(g)), "alloc")
    L.check(L.lib().eri_hip_pool_release(pool, f, 4096), "release")
    assert L.lib().eri_hip_pool_release(pool, f, 4096) == -6
    assert b"released already" in L.lib().eri_last_error()
    assert L.lib().eri_hip_pool_release(pool, C.c_void_p(f.value + 1024), 256) == -6  # a part of it
    L.check(L.lib().eri_hip_pool_release(pool, g, 256), "release")
    L.check(L.lib().eri_hip_pool_lane_used(pool, 0, C.byref(used)), "lane_used")
    assert used.value == 1024
    # not the pool's, or beyond the lane's level
    assert L.lib().eri_hip_pool_release(pool, C.c_void_p(a.value + 8 * MiB), 256) == -6
    assert L.lib().eri_hip_pool_release(pool, C.c_void_p(a.value + 100), 256) == -6
    assert L.lib().eri_hip_pool_release(pool, None, 256) == 0
    L.check(L.lib().eri_hip_pool_destroy(pool), "destroy")


def test_loading_a_checkpoint_again_does_not_grow_the_state_lane(tmp_path):
    """States that are replaced go back to the pool and the next load takes them: however often a checkpoint is
    loaded into an optimizer that has stepped, the lane never holds more than two sets of states."""
    import torch
    from eridiffusion_amd.adam8bit import Adam8bit, Adam8bitConfig, DevicePool
    L = _L()
    sizes = [2048 * 4 + 16, 5000, 2048]
    ps, gs = hs.make_inputs(sizes, True, 555)
    to_t = lambda a: torch.from_numpy(a.view(np.int16)).cuda().view(torch.bfloat16)
    params = [to_t(p) for p in ps]
    pool = DevicePool(16 * MiB, 2)
    opt = Adam8bit(params, Adam8bitConfig(lr=LR, betas=(B1, B2), eps=EPS, weight_decay=WD))
    opt.set_state_pool(pool, 1)
    for p, g in zip(params, gs):
        p.grad = to_t(g)
    opt.step()
    torch.cuda.synchronize()
    used = C.c_size_t()
    L.check(L.lib().eri_hip_pool_lane_used(pool._pool, 1, C.byref(used)), "lane_used")
    one_set = used.value
    assert one_set > 0
    path = str(tmp_path / "state.safetensors")
    opt.save_state(path)
    levels = []
    for _ in range(3):
        opt.load_state(path)
        L.check(L.lib().eri_hip_pool_lane_used(pool._pool, 1, C.byref(used)), "lane_used")
        levels.append(used.value)
    # a load builds the new states before it lets the old ones go (a load that fails changes nothing), so the
    # lane holds two sets at most; each load takes the pieces the load before it gave back
    assert max(levels) <= 2 * one_set and levels[2] == levels[0]
    opt.step()  # the loaded states are the ones that step
    torch.cuda.synchronize()
    # the pool's creator lets go first: the states keep the allocation alive and still return their pieces
    raw = C.c_void_p(pool._pool.value)
    pool.close()
    assert L.lib().eri_hip_pool_alloc_zeroed(raw, 0, 256, C.byref(C.c_void_p())) == -6  # alive, but hands out nothing more
    assert b"destroyed" in L.lib().eri_last_error()
    del opt


def test_parameters_and_gradients_in_lane_0_states_in_lane_2():
    """What a tensor runtime gets by backing its allocator with the pool and choosing the lane by dtype alone (U8 into
    lane 2, everything else into lane 0): parameters and gradients share a lane, the optimizer's states lie two
    lanes away.  The step over such a placement is checked against the oracle like any other, and the pieces are
    cleared on the optimizer's stream."""
    import torch
    L = _L()
    sizes = [2048 * 6 + 40, 4096, 333, 2048 * 3]
    ps, gs = hs.make_inputs(sizes, True, 8088)
    states = hs.oracle_states(sizes)
    stream = torch.cuda.current_stream().cuda_stream
    pool = _pool(96 * MiB, 3)
    lanes, lane_bytes = C.c_uint32(), C.c_size_t()
    L.check(L.lib().eri_hip_pool_info(pool, C.byref(lanes), C.byref(lane_bytes)), "pool_info")

    def place(lane, arr):
        out = C.c_void_p()
        L.check(L.lib().eri_hip_pool_alloc_zeroed_async(pool, lane, arr.nbytes, stream, C.byref(out)), "alloc_async")
        L.check(L.lib().eri_hip_memcpy_async(out, arr.ctypes.data, arr.nbytes, 1, stream), "h2d")
        return out.value

    rows = (L.TensorRow * len(sizes))()
    start = 0
    first = None
    for i, n in enumerate(sizes):
        r = rows[i]
        r.p, r.g = place(0, ps[i]), place(0, gs[i])               # BF16: lane 0
        r.m, r.v = place(2, states[i][0]), place(2, states[i][1])  # U8: lane 2
        r.absmax_m, r.absmax_v = place(2, states[i][2]), place(2, states[i][3])
        r.numel, r.block_start, r.dtype_tag, r.grad_scale = n, start, L.DTYPE_BF16, 1.0
        start += (n + 2047) // 2048
        first = first or r.p
        assert first <= r.p < first + lane_bytes.value and first <= r.g < first + lane_bytes.value
        assert first + 2 * lane_bytes.value <= r.m < first + 3 * lane_bytes.value
    L.check(L.lib().eri_hip_stream_sync(stream), "sync")  # the host arrays above were pageable
    table = C.c_void_p()
    L.check(L.lib().eri_adam8_table_create(rows, len(rows), stream, C.byref(table)), "table_create")
    for t in (1, 2):
        h = L.hyper_pack(LR, B1, B2, EPS, WD, t, L.MODE_ERI, L.FLAG_EXACT_PARAM)
        L.check(L.lib().eri_adam8_step_table(table, C.byref(h), stream), "step_table")
        hs.oracle_step(ps, gs, states, (LR, B1, B2, EPS, WD, t), True)
    L.check(L.lib().eri_hip_stream_sync(stream), "sync")
    for i, n in enumerate(sizes):
        for ptr, want in ((rows[i].p, ps[i]), (rows[i].m, states[i][0]), (rows[i].v, states[i][1]),
                          (rows[i].absmax_m, states[i][2]), (rows[i].absmax_v, states[i][3])):
            got = np.empty_like(want)
            L.check(L.lib().eri_hip_memcpy_async(got.ctypes.data, ptr, got.nbytes, 2, stream), "d2h")
            L.check(L.lib().eri_hip_stream_sync(stream), "sync")
            assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), i
    L.lib().eri_adam8_table_destroy(table)
    L.check(L.lib().eri_hip_pool_destroy(pool), "destroy")
