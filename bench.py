#!/usr/bin/env python3
"""Benchmark of the blockwise 8-bit AdamW step on one MI355X.

A step = one pass of the multi-tensor optimizer step over the whole parameter set, every input
already resident in HBM.  Default workload: the FLUX-12B-shaped full fine-tune set (780 bf16
tensors, 11,901,408,320 parameters, 8-bit m/v + fp32 absmax per 2048-block, ~72 GB resident).
Prints one JSON line: params/s, the HBM roofline fraction of the step kernel (algorithmic bytes /
measured launch duration / 8 TB/s) and, beside it, the CPU oracle timed on this host's cores.

The default command also times, after the headline and in the same process, the other benchmark
configurations and the other ways into the same step (the functional update the LoRA trainers call, the
bit-exact flag, one allocation per tensor) and reports them as `configs`: one row each with ms per step,
the kernel's duration and its roofline fraction.  Any other command line measures just what it names
(`--rows all` adds the rows, `--rows none` leaves them out).
"""
import argparse
import ctypes as C
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_HBM_GBPS = 8000.0
# algorithmic bytes per parameter: read p, g, m, v and write p, m, v, plus 16 bytes of absmax per block
BYTES_PER_PARAM = {"bf16": 2 + 2 + 1 + 1 + 2 + 1 + 1 + 16.0 / 2048, "f32": 4 + 4 + 1 + 1 + 4 + 1 + 1 + 16.0 / 2048}
# the type the arithmetic of each kernel is carried out in, whatever the parameters are stored as: every one of
# them widens its inputs to fp32 and rounds each operation to fp32 (the gradient norm adds its fp32 block sums in f64)
ARITHMETIC = {"adam8": "f32", "adam8_clip": "f32", "adam8_ema": "f32", "grad_norm": "f32", "adamw32": "f32", "ema": "f32",
              "traffic": "u8"}  # the traffic probe moves bytes and computes nothing

HEADLINE = dict(config="c5_flux12b_full", flags=0, kernel="adam8", mode="eri", api="table", param_dtype="config",
                grad_dtype="param", alloc="pool")
# (what changes against the headline's options, timed steps, warm-up steps); the LoRA sets run the 100 steps
# the benchmark configurations name
ROWS = [
    (dict(config="c1_flat_fp32"), 100, 10),
    (dict(config="c2_sdxl_lora_r16"), 100, 10),
    (dict(config="c2_sdxl_lora_r16", api="functional"), 100, 10),
    (dict(config="c2_sdxl_lora_r16", kernel="traffic"), 100, 10),
    (dict(config="c3_flux_lora_r32"), 100, 10),
    (dict(config="c3_flux_lora_r32", api="functional"), 100, 10),
    (dict(config="c3_flux_lora_r32", kernel="traffic"), 100, 10),
    (dict(config="c4_sdxl_unet_full"), 20, 3),
    (dict(config="c4_sdxl_unet_full", kernel="traffic"), 20, 3),
    (dict(config="c5_flux12b_full", flags=2), 20, 3),
    (dict(config="c5_flux12b_full", flags=2, api="object"), 20, 3),  # the list optimizer as a trainer gets it
    (dict(config="c5_flux12b_full", mode="l2"), 20, 3),
    (dict(config="c5_flux12b_full", kernel="traffic"), 20, 3),
    (dict(config="c5_flux12b_full", alloc="tensor"), 20, 3),
    # the sweeps that sit beside the step in a training iteration
    (dict(config="c5_flux12b_full", kernel="grad_norm"), 20, 3),
    (dict(config="c5_flux12b_full", kernel="adam8_clip"), 20, 3),
    (dict(config="c5_flux12b_full", kernel="adam8_ema"), 20, 3),
    (dict(config="c5_flux12b_full", kernel="ema"), 20, 3),
    (dict(config="c4_sdxl_unet_full", kernel="adamw32"), 20, 3),
]


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--config", default=HEADLINE["config"])
    ap.add_argument("--flags", type=int, default=0, help="ERI_ADAM8_FLAG_* bits for the step")
    ap.add_argument("--cpu-sample", type=int, default=1 << 30, help="parameters in the CPU baseline sample (0 = skip)")
    ap.add_argument("--kernel", choices=sorted(ARITHMETIC), default="adam8",
                    help="what one step is: the 8-bit AdamW step (headline), the same preceded by the device-side "
                         "gradient norm, the same with the EMA of the parameters taken inside it, the norm alone, "
                         "the 32-bit AdamW sibling, the EMA sweep, or the traffic probe (the step's reads and writes in "
                         "the step's launch shape with no arithmetic: what the memory system gives that mix of streams)")
    ap.add_argument("--mode", choices=["eri", "l2"], default="eri",
                    help="arithmetic of the table API's step: the list optimizer's (adam8bit_enhanced.rs) or the "
                         "functional update's (adam8bit.rs, what --api functional always runs)")
    ap.add_argument("--api", choices=["table", "object", "functional", "functional_update"], default="table",
                    help="table: eri_adam8_step_table on a launch table built once (headline).  object: the list "
                         "optimizer of the reference's API (eri_adam8bit_new over parameter handles, which owns its "
                         "states; one eri_adam8bit_step call per step).  functional: the "
                         "per-name optimizer, all tensors through one eri_adam8bit_fn_update_many call per step, "
                         "each step writing into the other of two output sets (update() returns a new tensor).  "
                         "functional_update: the same through one batched eri_adam8bit_fn_update call per tensor")
    ap.add_argument("--param-dtype", choices=["config", "bf16", "f32"], default="config",
                    help="parameter dtype: the one the configuration names, or an override (the shapes stay)")
    ap.add_argument("--grad-dtype", choices=["param", "f32"], default="param",
                    help="gradient dtype: the parameter's, or fp32 gradients (for bf16 parameters: read unrounded)")
    ap.add_argument("--alloc", choices=["pool", "arena", "tensor"], default="pool",
                    help="pool: one flat buffer per kind of array out of the library's lane pool (eri_hip_pool_*): "
                         "parameters, gradients and optimizer state each in a 48 GiB lane of their own, which keeps "
                         "the 8-bit states far from the parameters in device memory and the placement the same in "
                         "every process; if the pool cannot be created the run goes on "
                         "as arena and says so.  arena: the same flat buffers, each a device allocation of its own "
                         "(eri_hip_malloc_zeroed).  tensor: one torch allocation per tensor and buffer (how a tensor "
                         "runtime holds parameters and states)")
    ap.add_argument("--rows", choices=["auto", "all", "none"], default="auto",
                    help="the `configs` rows (the other configurations and entry points, timed after the headline in "
                         "the same process): auto = only when the command line is the default one")
    ap.add_argument("--rows-max-params", type=int, default=0,
                    help="leave out the `configs` rows of configurations with more parameters than this (0 = keep all)")
    ap.add_argument("--traffic-json", default=os.path.join(ROOT, "profiles", "traffic.json"),
                    help="HBM bytes per launch derived from rocprofv3 --pmc runs, if present")
    return ap.parse_args()


def align(n, a=256):
    return (n + a - 1) // a * a


class PerTensor:
    """One device allocation per tensor (how a tensor runtime holds parameters and states)."""

    def __init__(self, torch, sizes_bytes, lane=0):
        self.bufs = [torch.empty(max(b, 16), dtype=torch.uint8, device="cuda:0") for b in sizes_bytes]

    def ptr(self, i):
        return self.bufs[i].data_ptr()

    def fill(self, i, src, stream):
        self.bufs[i][:src.numel() * src.element_size()].copy_(src.view(-1).view(self.bufs[i].dtype))

    def free(self):
        self.bufs = []


class Arena:
    """One flat device allocation per kind of buffer, from the library's allocator
    (eri_hip_malloc_zeroed); every tensor starts on a 256-byte boundary."""

    def __init__(self, torch, sizes_bytes, lane=0):
        from eridiffusion_amd import _lib as L
        self.offsets = []
        total = 0
        for b in sizes_bytes:
            self.offsets.append(total)
            total += align(b)
        self.nbytes = max(total, 256)
        out = C.c_void_p()
        L.check(L.lib().eri_hip_malloc_zeroed(0, self.nbytes, C.byref(out)), "eri_hip_malloc_zeroed")
        self.base = out.value

    def ptr(self, i):
        return self.base + self.offsets[i]

    def fill(self, i, src, stream):
        """Device-to-device copy of a torch tensor's bytes into tensor i, on torch's current stream."""
        from eridiffusion_amd import _lib as L
        L.check(L.lib().eri_hip_memcpy_async(self.ptr(i), src.data_ptr(), src.numel() * src.element_size(), 3, stream),
                "eri_hip_memcpy_async")

    def free(self):
        from eridiffusion_amd import _lib as L
        L.lib().eri_hip_free(self.base)


class Pool(Arena):
    """The arenas of Arena out of the library's lane pool (eri_hip_pool_*): one device allocation, one 48 GiB lane
    per kind of tensor -- parameters, gradients, optimizer state, anything else -- so that the 8-bit states lie
    far from the parameters and gradients in device memory.  What a runtime with a pool allocator (the
    reference's MemoryPool) gets by backing it with that pool."""

    handle = None

    def __init__(self, torch, sizes_bytes, lane=0):
        from eridiffusion_amd import _lib as L
        cls = Pool
        self.offsets = []
        total = 0
        for b in sizes_bytes:
            self.offsets.append(total)
            total += align(b)
        self.nbytes = max(total, 256)
        if cls.handle is None:
            L.check(cls.open(), "eri_hip_pool_create")
        out = C.c_void_p()
        lanes = C.c_uint32()
        L.check(L.lib().eri_hip_pool_info(cls.handle, C.byref(lanes), None), "eri_hip_pool_info")
        for attempt in range(lanes.value):  # the lane of its kind, or the first one after it that still has room
            rc = L.lib().eri_hip_pool_alloc_zeroed(cls.handle, lane + attempt, self.nbytes, C.byref(out))
            if rc == 0:
                break
        L.check(rc, "eri_hip_pool_alloc_zeroed")
        self.base = out.value

    @classmethod
    def open(cls):
        """Creates the pool (nine tenths of the free device memory, 48 GiB lanes) unless it exists; the library's
        return code."""
        from eridiffusion_amd import _lib as L
        if cls.handle is not None:
            return 0
        handle = C.c_void_p()
        rc = L.lib().eri_hip_pool_create(0, 0, 0, C.byref(handle))
        if rc == 0:
            cls.handle = handle
        return rc

    @classmethod
    def close(cls):
        from eridiffusion_amd import _lib as L
        if cls.handle is not None:
            L.lib().eri_hip_pool_destroy(cls.handle)
            cls.handle = None

    def free(self):
        pass  # pieces go back when the pool is reset (after every measurement) or destroyed


def cpu_baseline(tensors, bf16, sample_params, hyper_args, reps=5, single_thread=True):
    """Times the C oracle (oracle/liberi_oracle.so) on a prefix of the same tensor list (the whole list when it
    has no more than `sample_params` parameters): one untimed step that warms the pages and gives the states real
    contents, then `reps` timed steps, the median reported."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import numpy as np

    import oracle_c as oc
    from eridiffusion_amd.workloads import numel

    threads = max(1, min(16, os.cpu_count() or 1))
    sizes, total = [], 0
    for _, shape in tensors:
        n = numel(shape)
        if total + n > sample_params and sizes:
            break
        n = min(n, sample_params)
        sizes.append(n)
        total += n
    whole = len(sizes) == len(tensors) and total == sum(numel(s) for _, s in tensors)
    rng = np.random.default_rng(7)
    tile = 1 << 22
    base_p = (rng.standard_normal(tile) * 0.02).astype(np.float32)
    base_g = (rng.standard_normal(tile) * 1e-3).astype(np.float32)
    if bf16:
        from oracle import adam8_numpy as onp
        base_p, base_g = onp.f32_to_bf16(base_p), onp.f32_to_bf16(base_g)
    maps = oc.load_maps()
    bufs = []
    for n in sizes:
        reps_n = (n + tile - 1) // tile
        bufs.append((np.tile(base_p, reps_n)[:n].copy(), np.tile(base_g, reps_n)[:n].copy(), list(oc.state_init(n))))
    dt_tag = oc.DT_BF16 if bf16 else oc.DT_F32
    times = []
    for rep in range(reps + 1):
        h = oc.hyper_pack(*hyper_args[:5], rep + 1)
        t0 = time.perf_counter()
        for p, g, st in bufs:
            oc.step_tensor(p, g, *st, h, maps, dt_tag, threads)
        if rep > 0:
            times.append(time.perf_counter() - t0)
    out = {"value": total / statistics.median(times), "unit": "params/s", "cores": threads, "host_cores": os.cpu_count(),
           "kind": "port",
           "sample": "%s (%d tensors, %d params), C oracle with OpenMP over blocks on %d threads, one warm-up step, "
                     "median of %d timed steps" % ("the whole workload" if whole else "the first tensors of the workload",
                                                   len(sizes), total, threads, reps)}
    if single_thread:  # the same code on one thread, on the largest tensor of the sample only
        big = max(range(len(sizes)), key=lambda i: sizes[i])
        p1, g1, st1 = bufs[big]
        n1 = min(sizes[big], 1 << 25)
        st1 = list(oc.state_init(n1))
        p1, g1 = p1[:n1].copy(), g1[:n1].copy()
        single = []
        for rep in range(4):  # the first step starts from the all-zero state and is not timed
            t0 = time.perf_counter()
            oc.step_tensor(p1, g1, *st1, oc.hyper_pack(*hyper_args[:5], rep + 1), maps, dt_tag, 1)
            if rep > 0:
                single.append(n1 / (time.perf_counter() - t0))
        out["single_thread_value"] = statistics.median(single)
        out["single_thread_sample"] = "%d params of the sample's largest tensor, median of steps 2-4" % n1
    return out


def measure(args, torch, separate_events=False):
    """One configuration: allocates, fills, times `args.steps` steps after `args.warmup`, frees; the JSON object of
    the run (without the CPU baseline).  separate_events: the wall clock is taken over steps without events around
    them and the kernel's duration over as many further steps with them (for steps of a few microseconds, where
    recording two events per step shows in the wall clock)."""
    from eridiffusion_amd import _lib as L
    from eridiffusion_amd import workloads as W

    fn, dt_name = W.CONFIGS[args.config]
    tensors = fn()
    if args.param_dtype != "config":
        dt_name = args.param_dtype
    bf16 = dt_name == "bf16"
    esz = 2 if bf16 else 4
    grad_f32 = bf16 and args.grad_dtype == "f32"
    gsz = 4 if grad_f32 else esz
    if grad_f32 and (args.kernel in ("adamw32",) or args.api not in ("table", "object")):
        sys.exit("--grad-dtype f32 is wired for the 8-bit step of the table and object APIs and for the gradient norm")
    sizes = [W.numel(s) for _, s in tensors]
    n_params = sum(sizes)
    n_blocks = sum((n + L.BLOCK - 1) // L.BLOCK for n in sizes)
    torch.cuda.set_device(0)
    stream = torch.cuda.current_stream().cuda_stream
    alloc = args.alloc

    if alloc == "pool" and args.kernel == "adamw32" and n_params * 4 > (20 << 30):
        # fp32 moments of the large sets fill a 48 GiB lane each and leave no room for the other arrays
        alloc = "arena"
    if alloc != "pool":
        Pool.close()  # the pool holds nine tenths of the device memory
    elif Pool.open() != 0:
        print("bench.py: no lane pool (%s); the flat buffers become allocations of their own (--alloc arena)"
              % L.lib().eri_last_error().decode("utf-8", "replace"), file=sys.stderr)
        alloc = "arena"
    if alloc == "pool":  # four lanes, each wide enough for its kind of tensor (little free memory gives fewer)
        lanes, lane_bytes = C.c_uint32(), C.c_size_t()
        L.check(L.lib().eri_hip_pool_info(Pool.handle, C.byref(lanes), C.byref(lane_bytes)), "eri_hip_pool_info")
        state_bytes = 2 * n_params + 8 * n_blocks + 1024 * len(sizes)
        widest = max(n_params * max(esz, gsz) + 256 * len(sizes), state_bytes)
        if args.api != "table":  # the flat states, unused by the optimizer objects, share the last lane
            widest = max(widest, state_bytes + (0 if args.api == "object" else n_params * esz + 256 * len(sizes)))
        if lanes.value < 4 or widest > lane_bytes.value:
            print("bench.py: the lane pool has %d lanes of %.1f GiB, too few or too narrow for this workload; the "
                  "flat buffers become allocations of their own (--alloc arena)" % (lanes.value, lane_bytes.value / 2**30),
                  file=sys.stderr)
            Pool.close()
            alloc = "arena"
    Alloc = {"arena": Arena, "tensor": PerTensor, "pool": Pool}[alloc]
    LANE_PARAM, LANE_GRAD, LANE_STATE, LANE_OTHER = 0, 1, 2, 3  # the pool's lanes, one per kind of tensor
    a_p = Alloc(torch, [n * esz for n in sizes], LANE_PARAM)
    a_g = Alloc(torch, [n * gsz for n in sizes], LANE_GRAD)
    # The optimizer objects allocate their states themselves, out of the state lane, as they would under a trainer;
    # the flat state arrays (which only the table API steps) then stay out of that lane.
    flat_lane = LANE_STATE if args.api == "table" else LANE_OTHER
    a_m = Alloc(torch, sizes, flat_lane)
    a_v = Alloc(torch, sizes, flat_lane)
    a_am = Alloc(torch, [((n + 2047) // 2048) * 4 for n in sizes], flat_lane)
    a_av = Alloc(torch, [((n + 2047) // 2048) * 4 for n in sizes], flat_lane)
    tdt = torch.bfloat16 if bf16 else torch.float32
    gen = torch.Generator(device="cuda:0")
    gen.manual_seed(0xE21D + 5)
    for i, (n, (name, shape)) in enumerate(zip(sizes, tensors)):  # synthetic data, the spread the configuration names
        p_std, g_std = W.init_std(args.config, name, shape)
        a_p.fill(i, torch.randn(n, device="cuda:0", generator=gen).mul_(p_std).to(tdt), stream)
        a_g.fill(i, torch.randn(n, device="cuda:0", generator=gen).mul_(g_std).to(torch.float32 if grad_f32 else tdt), stream)
        L.check(L.lib().eri_adam8_state_init(a_m.ptr(i), a_v.ptr(i), a_am.ptr(i), a_av.ptr(i), n, stream), "state_init")
    rows = (L.TensorRow * len(sizes))()
    start = 0
    for i, n in enumerate(sizes):
        r = rows[i]
        r.p, r.g, r.m, r.v, r.absmax_m, r.absmax_v = a_p.ptr(i), a_g.ptr(i), a_m.ptr(i), a_v.ptr(i), a_am.ptr(i), a_av.ptr(i)
        r.numel, r.block_start, r.dtype_tag, r.grad_scale = n, start, (L.DTYPE_BF16 if bf16 else L.DTYPE_F32), 1.0
        r.grad_f32 = 1 if grad_f32 else 0
        start += (n + L.BLOCK - 1) // L.BLOCK
    table = C.c_void_p()
    L.check(L.lib().eri_adam8_table_create(rows, len(rows), stream, C.byref(table)), "table_create")
    hyper_args = (1e-4, 0.9, 0.999, 1e-8, 0.01)
    bytes_per_param = BYTES_PER_PARAM[dt_name] + (gsz - esz)
    extra = []
    if args.kernel == "adamw32":
        a_m32 = Alloc(torch, [4 * n for n in sizes], LANE_STATE)
        a_v32 = Alloc(torch, [4 * n for n in sizes], LANE_OTHER)  # 32-bit moments are the bulk of the written bytes: a lane each
        extra += [a_m32, a_v32]
        rows32 = (L.AdamW32Row * len(sizes))()
        for i, n in enumerate(sizes):
            rows32[i].p, rows32[i].g, rows32[i].m, rows32[i].v = a_p.ptr(i), a_g.ptr(i), a_m32.ptr(i), a_v32.ptr(i)
            rows32[i].numel, rows32[i].dtype_tag = n, (L.DTYPE_BF16 if bf16 else L.DTYPE_F32)
        h32 = L.AdamW32Hyper(1e-4, 0.9, 0.999, 1e-8, 0.01)
        bytes_per_param = 3 * esz + 16
    elif args.kernel == "adam8_ema":
        a_sh = Alloc(torch, [n * esz for n in sizes], LANE_OTHER)
        extra.append(a_sh)
        for i in range(len(sizes)):
            rows[i].ema_shadow = a_sh.ptr(i)
        L.check(L.lib().eri_adam8_table_update(table, rows, len(rows), stream), "table_update")
        bytes_per_param += 2 * esz  # the shadow is read and written; the new parameter is still in registers
    elif args.kernel == "ema":
        a_sh = Alloc(torch, [n * esz for n in sizes], LANE_OTHER)
        extra.append(a_sh)
        rows_e = (L.EmaRow * len(sizes))()
        for i, n in enumerate(sizes):
            rows_e[i].shadow, rows_e[i].p, rows_e[i].numel = a_sh.ptr(i), a_p.ptr(i), n
            rows_e[i].dtype_tag = L.DTYPE_BF16 if bf16 else L.DTYPE_F32
        bytes_per_param = 3 * esz
    elif args.kernel == "grad_norm":
        bytes_per_param = gsz + 4.0 / 2048
    elif args.kernel == "adam8_clip":
        bytes_per_param += gsz + 4.0 / 2048

    fn_opt = None
    obj_opt, obj_params = None, []
    if args.api == "object":
        if args.kernel != "adam8" or args.mode != "eri":
            sys.exit("--api object runs the 8-bit step of the list optimizer only")
        cfg = L.Adam8bitConfigC()
        L.lib().eri_adam8bit_config_default(C.byref(cfg))
        cfg.lr, cfg.beta1, cfg.beta2, cfg.eps, cfg.weight_decay = hyper_args
        handles = (C.c_void_p * len(sizes))()
        for i, n in enumerate(sizes):
            hnd = C.c_void_p()
            L.check(L.lib().eri_param_create(a_p.ptr(i), n, L.DTYPE_BF16 if bf16 else L.DTYPE_F32, C.byref(hnd)), "param_create")
            L.check(L.lib().eri_param_set_grad_typed(hnd, a_g.ptr(i), L.DTYPE_F32 if gsz == 4 else L.DTYPE_BF16), "set_grad")
            handles[i] = hnd.value
            obj_params.append(hnd)
        obj_opt = C.c_void_p()
        L.check(L.lib().eri_adam8bit_new(handles, len(sizes), C.byref(cfg), stream, C.byref(obj_opt)), "adam8bit_new")
        # the object starts with ERI_ADAM8_FLAG_EXACT_PARAM; the bench times what --flags says, as for the table
        L.check(L.lib().eri_adam8bit_set_flags(obj_opt, args.flags), "set_flags")
        if alloc == "pool":  # the optimizer's own states out of the state lane
            L.check(L.lib().eri_adam8bit_set_state_pool(obj_opt, Pool.handle, LANE_STATE), "set_state_pool")
    elif args.api != "table":
        if args.kernel != "adam8":
            sys.exit("--api functional runs the 8-bit step only")
        n_t = len(sizes)
        a_p2 = Alloc(torch, [n * esz for n in sizes], LANE_OTHER)  # the other output set
        extra.append(a_p2)
        fn_opt = C.c_void_p()
        L.check(L.lib().eri_adam8bit_fn_with_params(*hyper_args, stream, C.byref(fn_opt)), "fn_with_params")
        L.check(L.lib().eri_adam8bit_fn_set_batching(fn_opt, 1), "fn_set_batching")
        if alloc == "pool":
            L.check(L.lib().eri_adam8bit_fn_set_state_pool(fn_opt, Pool.handle, LANE_STATE), "fn_set_state_pool")
        tag = L.DTYPE_BF16 if bf16 else L.DTYPE_F32
        fn_names = [name.encode() for name, _ in tensors]
        c_names = (C.c_char_p * n_t)(*fn_names)
        c_numels = (C.c_uint64 * n_t)(*sizes)
        c_tags = (C.c_int32 * n_t)(*([tag] * n_t))
        ptrs = lambda a: (C.c_void_p * n_t)(*[a.ptr(i) for i in range(n_t)])
        c_g = ptrs(a_g)
        sets = [(ptrs(a_p), ptrs(a_p2)), (ptrs(a_p2), ptrs(a_p))]  # (read from, write to), alternating
        raw = [([a_p.ptr(i) for i in range(n_t)], [a_p2.ptr(i) for i in range(n_t)]),
               ([a_p2.ptr(i) for i in range(n_t)], [a_p.ptr(i) for i in range(n_t)])]
        g_raw = [a_g.ptr(i) for i in range(n_t)]

    def step(t):
        if obj_opt is not None:
            L.check(L.lib().eri_adam8bit_step(obj_opt, None), "adam8bit_step")
            return
        if fn_opt is not None:
            if args.api == "functional":
                src, dst = sets[t & 1]
                L.check(L.lib().eri_adam8bit_fn_update_many(fn_opt, c_names, src, c_g, c_numels, c_tags, None, dst, n_t),
                        "fn_update_many")
            else:
                src, dst = raw[t & 1]
                upd = L.lib().eri_adam8bit_fn_update
                for i in range(n_t):
                    rc = upd(fn_opt, fn_names[i], src[i], g_raw[i], sizes[i], tag, tag, dst[i])
                    if rc:
                        L.check(rc, "fn_update")
            L.check(L.lib().eri_adam8bit_fn_step(fn_opt), "fn_step")
            return
        if args.kernel == "adamw32":
            L.check(L.lib().eri_adamw32_step_multi(rows32, len(sizes), C.byref(h32), stream), "adamw32")
            return
        if args.kernel == "ema":
            L.check(L.lib().eri_ema_update_multi(rows_e, len(sizes), 0.999, stream), "ema")
            return
        if args.kernel == "traffic":
            L.check(L.lib().eri_adam8_traffic_probe(table, stream), "traffic_probe")
            return
        flags = args.flags
        if args.kernel in ("grad_norm", "adam8_clip"):
            L.check(L.lib().eri_adam8_grad_norm(table, 1.0, 0.0, stream), "grad_norm")
            if args.kernel == "grad_norm":
                return
            flags |= L.FLAG_CLIP_FROM_TABLE
        if args.kernel == "adam8_ema":
            flags |= L.FLAG_EMA
        h = L.hyper_pack(*hyper_args, t, L.MODE_L2 if args.mode == "l2" else L.MODE_ERI, flags)
        h.ema_decay = 0.999
        L.check(L.lib().eri_adam8_step_table(table, C.byref(h), stream), "step_table")

    t = 0
    for _ in range(args.warmup):
        t += 1
        step(t)
    torch.cuda.synchronize()
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    if separate_events:
        t0 = time.perf_counter()
        for k in range(args.steps):
            t += 1
            step(t)
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        for k in range(args.steps):
            t += 1
            ev[k][0].record()
            step(t)
            ev[k][1].record()
        torch.cuda.synchronize()
    else:
        t0 = time.perf_counter()
        for k in range(args.steps):
            t += 1
            ev[k][0].record()
            step(t)
            ev[k][1].record()
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
    launch_ms = [a.elapsed_time(b) for a, b in ev]
    avg_launch_s = sum(launch_ms) / len(launch_ms) / 1e3

    algo_bytes = bytes_per_param * n_params
    achieved = algo_bytes / avg_launch_s / 1e9
    traffic = None
    if os.path.exists(args.traffic_json):
        try:
            with open(args.traffic_json) as f:
                key = "%s|%s|flags=%d" % (args.config, args.kernel, args.flags)
                if args.param_dtype != "config" and args.param_dtype != W.CONFIGS[args.config][1]:
                    key += "|param=" + args.param_dtype
                if grad_f32:
                    key += "|grad=f32"
                traffic = json.load(f).get(key) if args.api == "table" and args.mode == "eri" else None
        except Exception:
            traffic = None
    out = {
        "metric": "params/sec per 8-bit AdamW step" if args.kernel == "adam8" else "params/sec per %s step" % args.kernel,
        "value": n_params * args.steps / wall,
        "unit": "params/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": wall / args.steps * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": ARITHMETIC[args.kernel],
        "data": "synthetic",
        "config": {"workload": args.config, "tensors": len(sizes), "params": n_params, "blocks": n_blocks,
                   "kernel": args.kernel, "api": args.api, "alloc": alloc, "mode": args.mode if args.api in ("table", "object") else "l2",
                   "param_dtype": dt_name, "grad_dtype": "f32" if gsz == 4 else "bf16", "state": "uint8 m/v + fp32 absmax per 2048-block", "flags": args.flags,
                   "resident_gb": round((n_params * (esz + gsz + 2) + n_blocks * 8) / 1e9, 2)},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": PEAK_HBM_GBPS, "unit": "GB/s",
                     "frac": achieved / PEAK_HBM_GBPS, "traffic": traffic,
                     "traffic_source": None if traffic is None else "profiles/traffic.json: FETCH_SIZE and WRITE_SIZE of "
                                       "rocprofv3 --pmc runs of this command, not counted in this run",
                     "kernel_ms": avg_launch_s * 1e3, "kernel_ms_min": min(launch_ms), "kernel_ms_max": max(launch_ms),
                     "algorithmic_bytes": algo_bytes},
    }
    L.lib().eri_adam8_table_destroy(table)
    if fn_opt is not None:
        L.lib().eri_adam8bit_fn_destroy(fn_opt)
    if obj_opt is not None:
        L.lib().eri_adam8bit_destroy(obj_opt)
        for hnd in obj_params:
            L.lib().eri_param_release(hnd)
    for a in [a_p, a_g, a_m, a_v, a_am, a_av] + extra:
        a.free()
    if Pool.handle is not None:
        torch.cuda.synchronize()
        L.lib().eri_hip_pool_reset(Pool.handle)  # every piece of this measurement goes back
    torch.cuda.empty_cache()
    return out, tensors, bf16, hyper_args


def row_of(out):
    """The short form of a measurement for the `configs` list."""
    c, r = out["config"], out["roofline"]
    return {"workload": c["workload"], "kernel": c["kernel"], "api": c["api"], "mode": c["mode"], "flags": c["flags"], "alloc": c["alloc"],
            "param_dtype": c["param_dtype"], "params": c["params"], "tensors": c["tensors"], "steps": out["steps"],
            "warmup": out["warmup"], "ms_per_step": out["ms_per_step"], "params_per_s": out["value"],
            "kernel_ms": r["kernel_ms"], "kernel_ms_min": r["kernel_ms_min"], "frac": r["frac"],
            "frac_of_step": r["algorithmic_bytes"] / (out["ms_per_step"] * 1e-3) / 1e9 / PEAK_HBM_GBPS}


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU: the 8-bit AdamW step has no cross-GPU exchange and this build runs on "
              "a single MI355X; rerun with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch

    is_headline = all(getattr(args, k) == v for k, v in HEADLINE.items())
    out, tensors, bf16, hyper_args = measure(args, torch)
    if args.cpu_sample > 0:
        out["cpu_baseline"] = cpu_baseline(tensors, bf16, args.cpu_sample, hyper_args)
    if args.rows == "all" or (args.rows == "auto" and is_headline):
        from eridiffusion_amd import workloads as W
        rows = []
        for change, steps, warmup in ROWS:
            if args.rows_max_params and W.total_params(W.CONFIGS[change["config"]][0]()) > args.rows_max_params:
                continue
            a = argparse.Namespace(**vars(args))
            for k, v in HEADLINE.items():
                setattr(a, k, v)
            for k, v in change.items():
                setattr(a, k, v)
            a.steps, a.warmup = steps, warmup
            try:
                o, tens, b16, hy = measure(a, torch, separate_events=True)
            except SystemExit:
                raise
            except Exception as e:  # a row that cannot run must not take the headline with it
                rows.append({"workload": a.config, "api": a.api, "mode": a.mode, "flags": a.flags, "alloc": a.alloc,
                             "error": "%s: %s" % (type(e).__name__, e)})
                continue
            row = row_of(o)
            small = W.total_params(tens) <= (1 << 28)
            if args.cpu_sample > 0 and small and a.kernel == "adam8" and a.api == "table" and a.mode == "eri" and a.flags == 0:
                cb = cpu_baseline(tens, b16, 1 << 62, hy, single_thread=False)  # the whole configuration
                row["cpu_params_per_s"], row["cpu_sample"] = cb["value"], cb["sample"]
            rows.append(row)
        out["configs"] = rows
    Pool.close()
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
