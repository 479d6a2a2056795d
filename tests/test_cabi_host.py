"""CPU-only checks of the C ABI: every declared symbol is exported, argument validation answers
with the documented codes before any device is touched, the per-step scalars equal the oracle's,
and the kernel's slot lookup (replayed here from the library's own table image) equals a search."""
import ctypes as C
import os
import re

import numpy as np
import pytest

import oracle_c as oc
from eridiffusion_amd import _lib as L

ROOT = oc.ROOT


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "eri_optim8.h")).read() + \
        open(os.path.join(ROOT, "include", "eri_adam8bit.h")).read()
    declared = set(re.findall(r"\b(eri_[a-z0-9_]+)\s*\(", header)) - {"eri_last_error"} | {"eri_last_error"}
    assert declared, "no declarations parsed"
    lib = C.CDLL(L.LIB_PATH)
    for name in sorted(declared):
        assert hasattr(lib, name), name + " is declared in include/eri_optim8.h but not exported"
    assert declared == set(L.EXPORTS), "binding table and header disagree: %s" % (declared ^ set(L.EXPORTS))


def test_rust_binding_source_declares_every_symbol():
    """The Rust `extern "C"` block shipped as source must name exactly the header's functions."""
    header = open(os.path.join(ROOT, "include", "eri_optim8.h")).read() + \
        open(os.path.join(ROOT, "include", "eri_adam8bit.h")).read()
    declared = set(re.findall(r"\b(eri_[a-z0-9_]+)\s*\(", header))
    rust = open(os.path.join(ROOT, "eridiffusion_amd", "rust", "eri_optim8_sys.rs")).read()
    bound = set(re.findall(r"pub fn (eri_[a-z0-9_]+)\s*\(", rust))
    assert bound == declared, bound ^ declared


def test_build_rs_compiles_the_objects_of_the_makefile():
    """The crate's build script and csrc/Makefile must build the same objects from the same sources with
    the same defines: the Rust crate is never compiled here, so a file missing from its list would only
    show as an undefined symbol at the maintainer's link step."""
    csrc = os.path.join(ROOT, "eridiffusion_amd", "csrc")
    make = open(os.path.join(csrc, "Makefile")).read().replace("\\\n", " ")
    objs = re.search(r"^OBJS\s*:=(.*)$", make, re.M).group(1).split()
    want = set()
    for obj in objs:
        rule = re.search(r"^%s:\s*(\S+).*\n\t(.*)$" % re.escape(obj), make, re.M)
        assert rule, obj
        define = re.search(r"(-DERI_\w+=\w+)", rule.group(2))
        want.add((rule.group(1), define.group(1) if define else ""))
    assert len(want) == len(objs)
    rust = open(os.path.join(ROOT, "eridiffusion_amd", "rust", "build.rs")).read()
    got = set(re.findall(r'\("([\w.]+\.(?:hip|cpp))",\s*"\w+",\s*"([^"]*)",\s*(?:true|false)\)', rust))
    assert got == want, got ^ want
    for src, _ in want:
        assert os.path.exists(os.path.join(csrc, src)), src


def test_struct_layouts_match_the_header():
    assert C.sizeof(L.Hyper) == 56
    assert C.sizeof(L.TensorRow) == 96
    assert C.sizeof(L.AdamW32Row) == 56 and C.sizeof(L.EmaRow) == 32
    assert L.TensorRow.numel.offset == 48 and L.TensorRow.dtype_tag.offset == 64
    assert L.TensorRow.p_src.offset == 72 and L.TensorRow.grad_f32.offset == 80


def test_maps_equal_the_fixture():
    s = np.empty(256, np.float32)
    u = np.empty(256, np.float32)
    L.check(L.lib().eri_adam8_get_maps(s.ctypes.data, u.ctypes.data), "get_maps")
    fs, fu = oc.load_maps()
    assert np.array_equal(s.view(np.uint32), fs.view(np.uint32)) and np.array_equal(u.view(np.uint32), fu.view(np.uint32))


@pytest.mark.parametrize("mode", [0, 1, 2])
@pytest.mark.parametrize("step", [0, 1, 2, 11, 1000, 100000])
def test_hyper_pack_equals_the_oracle(mode, step):
    for lr, b1, b2, eps, wd in ((1e-4, 0.9, 0.999, 1e-8, 0.01), (1e-3, 0.95, 0.99, 1e-6, 0.0), (3e-5, 0.8, 0.9999, 1e-10, 0.1)):
        if mode != 1 and step == 0:
            continue
        h = L.hyper_pack(lr, b1, b2, eps, wd, step, mode)
        o = oc.hyper_pack(lr, b1, b2, eps, wd, step, mode)
        for f in ("beta1", "beta2", "omb1", "omb2", "eps", "weight_decay", "step_size", "bc1", "bc2"):
            assert getattr(h, f) == getattr(o, f), (f, mode, step)


def _row(**kw):
    r = L.TensorRow()
    r.p, r.g, r.m, r.v, r.absmax_m, r.absmax_v = 0x1000, 0x2000, 0x3000, 0x4000, 0x5000, 0x6000
    r.numel, r.block_start, r.dtype_tag, r.grad_scale = 4096, 0, L.DTYPE_BF16, 1.0
    for k, v in kw.items():
        setattr(r, k, v)
    return r


def _create(rows):
    arr = (L.TensorRow * len(rows))(*rows)
    out = C.c_void_p()
    rc = L.lib().eri_adam8_table_create(arr, len(rows), None, C.byref(out))
    return rc, L.lib().eri_last_error().decode()


def test_table_validation_codes():
    assert _create([_row(p=0)])[0] == -1
    assert _create([_row(absmax_v=0)])[0] == -1
    assert _create([_row(m=0x3008)])[0] == -2
    assert _create([_row(absmax_m=0x5002)])[0] == -2
    rc, msg = _create([_row(numel=0)])
    assert rc == -3 and "Empty tensor for quantization" in msg
    for tag in (L.DTYPE_F16, L.DTYPE_I32, 9):
        rc, msg = _create([_row(dtype_tag=tag)])
        assert rc == -4 and "dtype" in msg
    rc, msg = _create([_row(), _row(block_start=3)])
    assert rc == -5 and "expected 2" in msg
    # a ragged row counts its partial block: these rows pass validation (what remains is the device, absent here)
    assert _create([_row(numel=2049), _row(block_start=2)])[0] >= 0
    out = C.c_void_p()
    assert L.lib().eri_adam8_table_create(None, 1, None, C.byref(out)) == -1
    arr = (L.TensorRow * 1)(_row())
    assert L.lib().eri_adam8_table_create(arr, 0, None, C.byref(out)) == -6
    assert L.lib().eri_adam8_table_create(arr, 1, None, None) == -1


def test_other_argument_errors():
    lib = L.lib()
    h = L.Hyper()
    assert lib.eri_adam8_hyper_pack(1e-4, 0.9, 0.999, 1e-8, 0.01, 1, 7, 0, C.byref(h)) == -6
    assert lib.eri_adam8_hyper_pack(1e-4, 0.9, 0.999, 1e-8, 0.01, 1, 0, 0, None) == -1
    assert lib.eri_adam8_state_init(None, None, None, None, 10, None) == -1
    assert lib.eri_adam8_state_init(1, 1, 1, 1, 0, None) == -3
    assert lib.eri_adam8_step_table(None, C.byref(h), None) == -1
    assert lib.eri_adam8_dequantize(None, None, 1, 10, None, None) == -1
    assert lib.eri_adam8_quantize(1, 1, 0, 1, 1, None) == -3
    assert lib.eri_hip_memcpy_async(None, None, 16, 1, None) == -1
    with pytest.raises(L.EriError) as e:
        L.check(lib.eri_adam8_state_init(1, 1, 1, 1, 0, None), "eri_adam8_state_init")
    assert "failed with code -3" in str(e.value)


def _image():
    n = C.c_size_t()
    offs = (C.c_uint32 * 6)()
    L.check(L.lib().eri_adam8_table_image(None, 0, C.byref(n), offs), "table_image")
    buf = np.empty(n.value, np.uint8)
    L.check(L.lib().eri_adam8_table_image(buf.ctypes.data, buf.size, None, None), "table_image")
    return buf, list(offs)


KEY_SCALE = np.float32(4096.0)


def _replay(x, img, offs, signed):
    """The kernel's slot lookup (code_signed_key / code_unsigned_key), in NumPy: scale the quotient,
    convert to binary16 (rounded toward zero, as v_cvt_pkrtz_f16_f32 does), mask the pattern into a byte address."""
    xs = (x * KEY_SCALE).astype(np.float32)
    with np.errstate(over="ignore", invalid="ignore"):
        h16 = xs.astype(np.float16)  # nearest even; one pattern closer to zero wherever that rounded away from it
        away = np.abs(h16.astype(np.float32)) > np.abs(xs)
        h = (h16.view(np.uint16) - away.astype(np.uint16)).astype(np.uint32)
    addr = (h & 0xFFF0) if signed else (h & 0x7FF8)
    base = offs[4] if signed else offs[5]
    mid = np.empty(x.size, np.float32)
    lo = np.empty(x.size, np.uint32)
    words = img.view(np.uint32)
    idx = (base + addr) // 4
    mid = words[idx].copy().view(np.float32)
    lo = words[idx + 1]
    with np.errstate(invalid="ignore"):
        return (lo + (xs > mid)).astype(np.int64)


@pytest.mark.parametrize("signed", [True, False])
def test_slot_lookup_equals_search(signed):
    img, offs = _image()
    table = oc.load_maps()[0 if signed else 1]
    mid = oc.midpoints(table)
    assert np.array_equal(img[offs[2 if signed else 3]:][:255 * 4].view(np.float32), mid)
    rng = np.random.default_rng(13)
    near = np.concatenate([np.nextafter(mid, np.float32(-2)), mid, np.nextafter(mid, np.float32(2)),
                           np.nextafter(table, np.float32(-2)), table, np.nextafter(table, np.float32(2))])
    # every boundary between binary16 values of the scaled quotient, and its float32 neighbours
    halves = np.arange(0, 0x6C01, dtype=np.uint16).view(np.float16).astype(np.float32)  # 0 .. 4096
    ties = ((halves[:-1].astype(np.float64) + halves[1:].astype(np.float64)) / 2).astype(np.float32)
    edges = np.concatenate([halves, ties, np.nextafter(ties, np.float32(-1)), np.nextafter(ties, np.float32(1e9))])
    edges = (edges / KEY_SCALE).astype(np.float32)
    rnd = rng.integers(0, 0x3F800001, 4_000_000, dtype=np.uint32).view(np.float32)
    logu = (10.0 ** rng.uniform(-12, 0, 1_000_000)).astype(np.float32)
    xs = np.concatenate([near, edges, rnd, logu, np.array([0.0, 1.0, 1e-45, 1e-30], np.float32)]).astype(np.float32)
    xs = xs[(xs >= 0) & (xs <= 1)]
    if signed:
        xs = np.concatenate([xs, -xs])
    want = np.searchsorted(mid, xs, side="left")
    got = _replay(xs, img, offs, signed)
    assert np.array_equal(got, want)
    nan = np.array([np.nan, -np.nan], np.float32)
    assert np.array_equal(_replay(nan, img, offs, signed), [0, 0])


def test_package_refuses_to_work_without_the_library(monkeypatch):
    monkeypatch.setattr(L, "_lib", None)
    monkeypatch.setattr(L, "LIB_PATH", os.path.join(ROOT, "eridiffusion_amd", "no_such_library.so"))
    with pytest.raises(RuntimeError, match="no CPU or PyTorch fallback"):
        L.lib()


def test_headers_compile_as_c_and_cpp_and_agree_on_struct_sizes(tmp_path):
    """The two headers are the boundary: they must be valid C11 and C++17 on their own, and the struct sizes a
    C compiler sees must be the ones the ctypes table (and the Rust #[repr(C)] block) assume."""
    import subprocess
    inc = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include")
    src = tmp_path / "check.c"
    src.write_text('''
#include "eri_optim8.h"
#include "eri_adam8bit.h"
#include <stdio.h>
int main(void) {
    printf("%zu %zu %zu %zu %zu %zu %zu\\n", sizeof(EriAdam8Hyper), sizeof(EriAdam8Tensor), sizeof(EriAdamW32Tensor),
           sizeof(EriAdamW32Hyper), sizeof(EriEmaTensor), sizeof(EriAdam8bitConfig), sizeof(EriOptimizerMemoryReport));
    return 0;
}
''')
    exe = tmp_path / "check"
    subprocess.check_call(["gcc", "-std=c11", "-Wall", "-Wextra", "-pedantic", "-Werror", "-I", inc, str(src), "-o", str(exe)])
    got = [int(x) for x in subprocess.check_output([str(exe)]).split()]
    want = [C.sizeof(L.Hyper), C.sizeof(L.TensorRow), C.sizeof(L.AdamW32Row), C.sizeof(L.AdamW32Hyper), C.sizeof(L.EmaRow),
            C.sizeof(L.Adam8bitConfigC), C.sizeof(L.MemoryReportC)]
    assert got == want, (got, want)
    cpp = tmp_path / "check.cpp"
    cpp.write_text('#include "eri_optim8.h"\n#include "eri_adam8bit.h"\nint main() { return sizeof(EriAdam8Hyper) == 56 && sizeof(EriAdam8Tensor) == 96 ? 0 : 1; }\n')
    subprocess.check_call(["g++", "-std=c++17", "-Wall", "-Wextra", "-pedantic", "-Werror", "-I", inc, str(cpp), "-o", str(tmp_path / "checkpp")])
    assert subprocess.call([str(tmp_path / "checkpp")]) == 0
