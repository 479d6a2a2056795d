"""Pins the oracle's bf16 casts and its nearest-entry quantiser without retyping its formulas."""
import numpy as np
import torch

import oracle_c as oc
from oracle import adam8_numpy as onp


def test_bf16_to_f32_all_patterns_against_torch():
    h = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    want = torch.from_numpy(h.view(np.int16).copy()).view(torch.bfloat16).float().numpy()
    got_np = onp.bf16_to_f32(h)
    got_c = np.array([oc.lib().eri_oracle_bf16_to_f32(int(x)) for x in h[::7]], np.float32)
    assert np.array_equal(got_np.view(np.uint32), want.view(np.uint32))
    ok = ~np.isnan(want[::7])  # a NaN payload does not survive the float return of a C call
    assert np.array_equal(got_c.view(np.uint32)[ok], want[::7].view(np.uint32)[ok])
    assert np.all(np.isnan(got_c[~ok]))


def test_f32_to_bf16_rne_against_torch():
    rng = np.random.default_rng(5)
    # every high half, with low halves chosen to hit below / exactly at / above the rounding tie
    hi = np.arange(65536, dtype=np.uint32) << 16
    lows = np.array([0x0000, 0x0001, 0x7FFF, 0x8000, 0x8001, 0xFFFF], np.uint32)
    bits = (hi[:, None] | lows[None, :]).reshape(-1)
    bits = np.concatenate([bits, rng.integers(0, 2 ** 32, 200000, dtype=np.uint64).astype(np.uint32)])
    x = bits.view(np.float32)
    finite = np.isfinite(x)
    want = torch.from_numpy(x.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = onp.f32_to_bf16(x)
    assert np.array_equal(got[finite], want[finite])
    nan = np.isnan(x)
    assert np.all((got[nan] & 0x7F80) == 0x7F80) and np.all((got[nan] & 0x7F) != 0)
    sub = slice(0, None, 97)
    got_c = np.array([oc.lib().eri_oracle_f32_to_bf16(float(v)) for v in x[sub][np.isfinite(x[sub])]], np.uint16)
    assert np.array_equal(got_c, want[sub][np.isfinite(x[sub])])


def brute_nearest(table, x):
    """argmin |x - table[j]| in exact arithmetic (float64 holds fp32 differences exactly enough:
    both operands are fp32, the difference of two fp32 values is exact in float64)."""
    d = np.abs(x.astype(np.float64)[:, None] - table.astype(np.float64)[None, :])
    return np.argmin(d, axis=1)  # first minimum = lower index on a tie


def test_nearest_index_is_argmin_distance():
    rng = np.random.default_rng(11)
    for table, lo in zip(oc.load_maps(), (-1.0, 0.0)):
        mid = oc.midpoints(table)
        xs = np.concatenate([
            rng.uniform(lo, 1.0, 20000), lo + (1 - lo) * rng.random(5000) ** 6 * rng.choice([-1, 1], 5000) * (lo < 0),
            10.0 ** rng.uniform(-9, 0, 5000), table, np.nextafter(table, 2), np.nextafter(table, -2),
        ]).astype(np.float32)
        xs = xs[(xs >= lo) & (xs <= 1.0)]
        want = brute_nearest(table, xs)
        got_c = np.array([oc.lib().eri_oracle_nearest_index(oc.ptr(mid), float(x)) for x in xs])
        got_np = onp.nearest_index(onp.midpoints(table), xs)
        # the fp32 midpoint can sit one ulp off the true midpoint; only there may argmin differ
        true_mid = (table[:-1].astype(np.float64) + table[1:].astype(np.float64)) / 2
        near = np.min(np.abs(xs.astype(np.float64)[:, None] - true_mid[None, :]) /
                      np.spacing(np.abs(xs)).astype(np.float64)[:, None], axis=1) <= 1.0
        assert np.array_equal(got_c, got_np)
        assert np.array_equal(got_c[~near], want[~near])
        assert np.all(np.abs(got_c[near] - want[near]) <= 1)


def test_round_trip_every_code_and_tie_rule():
    for table in oc.load_maps():
        mid = oc.midpoints(table)
        codes = np.array([oc.lib().eri_oracle_nearest_index(oc.ptr(mid), float(x)) for x in table])
        assert np.array_equal(codes, np.arange(256))
        # exactly on a midpoint -> the lower index; one ulp above -> the upper
        on = np.array([oc.lib().eri_oracle_nearest_index(oc.ptr(mid), float(x)) for x in mid])
        up = np.array([oc.lib().eri_oracle_nearest_index(oc.ptr(mid), float(np.nextafter(x, np.float32(2))))
                       for x in mid])
        assert np.array_equal(on, np.arange(255)) and np.array_equal(up, np.arange(1, 256))
        assert oc.lib().eri_oracle_nearest_index(oc.ptr(mid), float("nan")) == 0
        assert np.array_equal(onp.nearest_index(mid, mid), np.arange(255))


def test_nearest_index_monotone():
    rng = np.random.default_rng(3)
    for table, lo in zip(oc.load_maps(), (-1.0, 0.0)):
        xs = np.sort(rng.uniform(lo, 1, 50000).astype(np.float32))
        idx = onp.nearest_index(onp.midpoints(table), xs).astype(int)
        assert np.all(np.diff(idx) >= 0)


def test_quantize_dequantize_blockwise():
    rng = np.random.default_rng(9)
    s, u = oc.load_maps()
    n = 3 * 2048 + 321
    x = (rng.standard_normal(n) * 1e-3).astype(np.float32)
    x[2048:4096] = 0.0  # an all-zero block
    codes = np.empty(n, np.uint8)
    absmax = np.empty(4, np.float32)
    oc.lib().eri_oracle_quantize(oc.ptr(x), oc.ptr(s), n, oc.ptr(codes), oc.ptr(absmax))
    want_abs = np.array([np.abs(x[i:i + 2048]).max() for i in range(0, n, 2048)], np.float32)
    assert np.array_equal(absmax, want_abs)
    assert np.all(codes[2048:4096] == 127)
    back = np.empty(n, np.float32)
    oc.lib().eri_oracle_dequantize(oc.ptr(codes), oc.ptr(absmax), oc.ptr(s), n, oc.ptr(back))
    # nearest entry: error bounded by half the widest gap of the map times absmax
    gap = np.diff(s).max() / 2
    assert np.all(np.abs(back - x) <= gap * np.repeat(want_abs, 2048)[:n] * 1.0001)
    # the block maximum itself is reproduced exactly when it is positive (x = 1.0 is an entry)
    for b in (0, 2, 3):
        seg = slice(b * 2048, min((b + 1) * 2048, n))
        i = np.argmax(np.abs(x[seg]))
        if x[seg][i] > 0:
            assert back[seg][i] == x[seg][i]


def test_quantization_as_in_the_reference():
    # adam8bit_enhanced.rs:486-498: a 10x10 tensor ~N(0, 1) is quantised and dequantised; the shape
    # survives and the mean absolute error is below 0.1.  The blockwise dynamic format is far inside that:
    # its relative step near full scale is 1/128 and finer below.
    rng = np.random.default_rng(486)
    s, _ = oc.load_maps()
    x = rng.standard_normal(100).astype(np.float32)
    codes, absmax, back = np.empty(100, np.uint8), np.empty(1, np.float32), np.empty(100, np.float32)
    oc.lib().eri_oracle_quantize(oc.ptr(x), oc.ptr(s), 100, oc.ptr(codes), oc.ptr(absmax))
    oc.lib().eri_oracle_dequantize(oc.ptr(codes), oc.ptr(absmax), oc.ptr(s), 100, oc.ptr(back))
    assert back.shape == x.shape
    err = np.abs(back - x).mean()
    assert err < 0.1 and err < 0.02
