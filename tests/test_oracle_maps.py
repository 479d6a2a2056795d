"""Pins the two dynamic maps: fixture invariants, a float64 closed form, and the product header."""
import os
import re

import numpy as np

from oracle_c import ROOT, load_maps, midpoints


def closed_form(signed):
    vals = []
    for i in range(7):
        k = 2 ** i if signed else 2 ** (i + 1)
        edges = np.linspace(0.1, 1.0, k + 1)
        mids = (edges[:-1] + edges[1:]) / 2
        vals += list(mids * 10.0 ** (i - 6))
        if signed:
            vals += list(-mids * 10.0 ** (i - 6))
    vals += [0.0, 1.0]
    return np.sort(np.array(vals))


def ulp_distance(a, b):
    ai = a.view(np.int32).astype(np.int64)
    bi = b.view(np.int32).astype(np.int64)
    ai = np.where(ai < 0, -(ai & 0x7FFFFFFF), ai)
    bi = np.where(bi < 0, -(bi & 0x7FFFFFFF), bi)
    return np.abs(ai - bi)


def test_fixture_invariants():
    s, u = load_maps()
    assert s.size == 256 and u.size == 256
    assert np.all(np.diff(s) > 0) and np.all(np.diff(u) > 0)
    assert s[127] == 0.0 and s[255] == 1.0 and u[0] == 0.0 and u[255] == 1.0
    assert s[0] == np.float32(-0.99296874)
    # antisymmetric apart from the extra +1.0 on the positive side
    assert np.array_equal(s[:127], -s[128:255][::-1])
    assert np.isclose(s[128], 5.5e-7, rtol=1e-6) and np.isclose(u[1], 3.25e-7, rtol=1e-6)
    # unsigned decade i holds 2**(i+1) entries, signed 2**i per sign
    assert np.sum((u > 0.1) & (u < 1.0)) == 128
    assert np.sum((s > 0.1) & (s < 1.0)) == 64


def test_fixture_matches_float64_closed_form():
    s, u = load_maps()
    for table, signed in ((s, True), (u, False)):
        ref = closed_form(signed).astype(np.float32)
        assert ulp_distance(table, ref).max() <= 2


def test_midpoints_strictly_increasing_and_between_entries():
    for table in load_maps():
        mid = midpoints(table)
        assert np.all(np.diff(mid) > 0)
        assert np.all(mid > table[:-1]) and np.all(mid < table[1:])
        ref = (table[:-1].astype(np.float64) + table[1:].astype(np.float64)) / 2
        assert np.all(np.abs(mid - ref) <= np.spacing(np.abs(mid)))


def test_product_header_holds_the_fixture_bits():
    text = open(os.path.join(ROOT, "eridiffusion_amd", "csrc", "eri_dynamic_maps.inc")).read()
    words = [int(w, 16) for w in re.findall(r"0x([0-9a-f]{8})u", text)]
    assert len(words) == 512
    s, u = load_maps()
    assert np.array_equal(np.array(words[:256], np.uint32), s.view(np.uint32))
    assert np.array_equal(np.array(words[256:], np.uint32), u.view(np.uint32))
