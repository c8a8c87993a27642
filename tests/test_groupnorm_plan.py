"""The launch plan of msd_groupnorm, checked on the CPU through msd_groupnorm_plan (host arithmetic).

A kernel that does not match its launch faults the GPU, so what the planner may hand to the
register kernel is pinned here: the vectors-per-lane values the kernels are built for, workgroup
sizes in whole wavefronts, slices that fit their workgroup and own at least one vector, the largest
vectors-per-lane value only on exact fits, power-of-two slice counts within the exchange scratch,
several writers only on whole units of at most 10 vectors per lane and never for a call in place.
The reference has no counterpart: its geometry is fixed (M/nn/GroupNorm.cpp:105-128)."""
import importlib
import random

import pytest

msd = importlib.import_module("mobile-stable-diffusion_amd")

K_VALUES = {1, 2, 3, 4, 5, 6, 8, 10, 12, 16, 20}
MAX_SPLIT, MAX_UNITS, STATIC_UNITS = 64, 8192, 1024


def _check(batch, channels, hw, groups, code, noalloc=False, in_place=False):
    split, threads, k, writers = msd.groupnorm_plan(batch, channels, hw, groups, code, noalloc, in_place)
    elt = 4 if code == msd.DTYPE_F32 else 2
    epv = 16 // elt
    unit = channels // groups * hw
    if split == 0:
        assert threads == 0 and k == 0 and writers == 1
        return split, threads, k, writers
    assert hw % epv == 0 and unit * elt < 2 ** 32          # what the register kernel assumes
    vecs = unit // epv
    assert split & (split - 1) == 0 and 1 <= split <= MAX_SPLIT
    if split > 1:
        assert batch * groups <= (STATIC_UNITS if noalloc else MAX_UNITS)
    assert threads % 64 == 0 and 64 <= threads <= 1024
    assert k in K_VALUES
    per_slice = -(-vecs // split)
    assert per_slice * (split - 1) < vecs                  # the last slice owns at least one vector
    assert k * threads >= per_slice                        # a slice fits its workgroup's registers
    assert (k - 1) * threads < per_slice or k == min(v for v in K_VALUES if v * threads >= per_slice)
    if k == 20:                                            # no masked code for the largest K
        assert per_slice * split == vecs and per_slice == 20 * threads
    if k > 6:                                              # gamma / beta of the group go through LDS
        assert channels // groups <= 1024
    assert writers in (1, 2, 4, 8, 16)
    if writers > 1:                                        # whole units, kernels built up to K = 10,
        assert split == 1 and k <= 10 and not in_place     # every writer owns a wavefront's vectors at least
        assert vecs >= writers * 64
    return split, threads, k, writers


UNET_SHAPES = [(1280, 64), (640, 256), (2560, 64), (320, 1024), (1280, 256), (1920, 256), (640, 1024), (2560, 256),
               (960, 1024), (320, 4096), (1280, 1024), (1920, 1024), (640, 4096), (960, 4096)]   # (channels, hw)


def _knobs(msd, **values):
    lib = msd.load_library()
    for name, value in values.items():
        assert lib.msd_set_tuning(getattr(msd, "TUNE_" + name), value) == 0


def test_the_rule_alone_plans_every_batch_and_never_leaves_cut_units_between_one_and_two_workgroups_per_cu():
    """With the table of measured plans switched off, every UNet shape at every batch from 1 to 40
    gets a launch that fits; and when the rule cuts units (it is not the registers of one workgroup
    that force it) the launch has at most one workgroup per CU or at least two, never one and a
    bit: such a launch runs as two rounds with the second mostly empty."""
    _knobs(msd, GN_PLAN_RULE_ONLY=1)
    try:
        for batch in range(1, 41):
            for channels, hw in UNET_SHAPES:
                for code, elt in ((msd.DTYPE_F16, 2), (msd.DTYPE_F32, 4)):
                    for in_place in (True, False):
                        split, threads, k, writers = _check(batch, channels, hw, 32, code, in_place=in_place)
                        units, vecs = batch * 32, channels // 32 * hw * elt // 16
                        if split > 1 and vecs <= 16 * 1024:
                            assert not 256 < units * split < 512, (batch, channels, hw, elt, split)
                        if writers > 1:
                            assert units * writers <= 256 and units % 8 == 0
    finally:
        _knobs(msd, GN_PLAN_RULE_ONLY=0)


def test_plans_follow_the_chip_that_is_reported():
    """CU and XCD counts come from the device (here: injected through the knobs).  The table of
    measured plans belongs to 256 CUs in 8 XCDs and is not consulted elsewhere; writers per unit
    follow the CU count, need the units in whole rows of a power-of-two XCD count, and a chip of
    one XCD needs no such rows."""
    f16 = msd.DTYPE_F16
    try:
        # the chip the table was measured on: the measured plan of 320 channels at 64 x 64, batch 2, in place
        assert msd.groupnorm_plan(2, 320, 4096, 32, f16, in_place=True) == (4, 640, 2, 1)
        _knobs(msd, DEVICE_CUS=64, DEVICE_XCDS=2)     # a quarter of the chip
        assert msd.groupnorm_plan(2, 320, 4096, 32, f16, in_place=True) == (1, 1024, 5, 1)   # 64 units on 64 CUs: whole
        assert msd.groupnorm_plan(1, 640, 1024, 32, f16)[3] == 2     # 32 units: two writers fill 64 CUs
        assert msd.groupnorm_plan(2, 640, 1024, 32, f16)[3] == 1     # 64 units: every CU has a unit already
        _knobs(msd, DEVICE_CUS=228, DEVICE_XCDS=6)    # not a power of two: no block-id stride keeps writers on one XCD
        assert msd.groupnorm_plan(1, 640, 1024, 32, f16)[3] == 1
        _knobs(msd, DEVICE_CUS=304, DEVICE_XCDS=8)    # more CUs than the table's chip: the rule, same shape of plan
        assert msd.groupnorm_plan(1, 640, 1024, 32, f16)[3] == 8 and msd.groupnorm_plan(4, 640, 1024, 32, f16)[3] == 2
        _knobs(msd, DEVICE_CUS=32, DEVICE_XCDS=1)     # one XCD (a partitioned device): no rows of units needed
        assert msd.groupnorm_plan(1, 24, 4096, 3, f16)[3] == 8       # 3 units, one L2 for everybody
        _knobs(msd, DEVICE_CUS=256, DEVICE_XCDS=8)
        assert msd.groupnorm_plan(3, 24, 4096, 3, f16)[3] == 1       # 9 units on 8 XCDs: the writers would sit apart
        for cus, xcds in ((16, 1), (64, 2), (120, 4), (228, 6), (1024, 16)):   # whatever the chip, a launch that fits
            _knobs(msd, DEVICE_CUS=cus, DEVICE_XCDS=xcds)
            for batch in (1, 2, 5, 32):
                for channels, hw in UNET_SHAPES:
                    _check(batch, channels, hw, 32, f16)
                    _check(batch, channels, hw, 32, msd.DTYPE_F32, in_place=True)
    finally:
        _knobs(msd, DEVICE_CUS=0, DEVICE_XCDS=0)


def test_plans_of_the_unet_shapes_at_batch_2_and_32():
    f16, f32 = msd.DTYPE_F16, msd.DTYPE_F32
    # a call in place (the reference's out-norms): one workgroup per unit or slices with an exchange
    in_place = {
        (2, 320, 4096, f16): (4, 640, 2, 1), (2, 640, 1024, f16): (1, 512, 5, 1), (2, 1280, 256, f16): (1, 512, 3, 1),
        (2, 1280, 64, f16): (1, 320, 1, 1), (2, 960, 1024, f16): (2, 960, 2, 1), (2, 1920, 256, f16): (1, 960, 2, 1),
        (1, 320, 4096, f32): (4, 640, 4, 1), (1, 640, 4096, f16): (4, 1024, 3, 1), (1, 960, 4096, f16): (8, 960, 2, 1),
        (2, 960, 4096, f32): (8, 960, 4, 1), (2, 640, 1024, f32): (1, 1024, 5, 1), (1, 640, 1024, f32): (4, 640, 2, 1),
        (4, 640, 4096, f32): (4, 512, 10, 1), (8, 640, 4096, f32): (2, 512, 20, 1), (2, 640, 256, f32): (1, 640, 2, 1),
        (32, 320, 4096, f16): (1, 256, 20, 1), (32, 640, 1024, f16): (1, 256, 10, 1), (32, 1280, 256, f16): (1, 256, 5, 1),
        (8, 320, 4096, f16): (1, 1024, 5, 1), (32, 960, 4096, f16): (8, 384, 5, 1),
    }
    for (batch, channels, hw, code), want in in_place.items():
        assert _check(batch, channels, hw, 32, code, in_place=True) == want, (batch, channels, hw, code)
    # output apart from the input: up to 256 workgroups share whole units of up to 5120 vectors
    # (10240 of 4-byte elements with up to four writers); larger units and batches plan as above
    apart = {
        (2, 320, 4096, f16): (1, 1024, 5, 4), (2, 640, 1024, f16): (1, 640, 4, 4), (2, 1280, 256, f16): (1, 512, 3, 4),
        (2, 1280, 64, f16): (1, 384, 1, 4), (2, 960, 1024, f16): (1, 1024, 4, 4), (2, 1920, 256, f16): (1, 512, 4, 4),
        (2, 1920, 1024, f16): (4, 960, 2, 1), (2, 640, 4096, f16): (4, 1024, 3, 1),
        (1, 320, 4096, f16): (1, 1024, 5, 8), (1, 1280, 64, f16): (1, 384, 1, 4), (4, 640, 1024, f16): (1, 1024, 3, 2),
        (1, 320, 4096, f32): (4, 640, 4, 1), (1, 640, 1024, f32): (1, 1024, 5, 8), (2, 320, 4096, f32): (1, 1024, 10, 4),
        # (960 channels at 32 x 32, fp32: 768 x 10 measured 5.84 us against 6.04 us for the 1024 x 8 it had before)
        (2, 960, 1024, f32): (1, 768, 10, 4), (2, 960, 4096, f32): (8, 960, 4, 1), (2, 1280, 256, f32): (1, 640, 4, 4),
        (8, 320, 4096, f16): (1, 1024, 5, 1), (32, 320, 4096, f16): (1, 256, 20, 1),
    }
    for (batch, channels, hw, code), want in apart.items():
        assert _check(batch, channels, hw, 32, code) == want, (batch, channels, hw, code)
    assert _check(3, 24, 4096, 3, f16)[3] == 1    # 9 units: not in whole rows of 8, the writers would sit on different XCDs


def test_shapes_the_register_kernel_cannot_take_go_to_the_general_kernel():
    assert msd.groupnorm_plan(2, 320, 4090, 32, msd.DTYPE_F16) == (0, 0, 0, 1)   # hw not in whole vectors
    assert msd.groupnorm_plan(2, 320, 4094, 32, msd.DTYPE_F32) == (0, 0, 0, 1)
    assert msd.groupnorm_plan(1, 32 * 1100, 32, 32, msd.DTYPE_F16)[2] <= 6         # wide groups: no LDS affine
    assert msd.groupnorm_plan(0, 320, 4096, 32, msd.DTYPE_F16) == (0, 0, 0, 1)     # nothing to do
    lib = msd.load_library()
    import ctypes
    o = [ctypes.c_int(7) for _ in range(4)]
    refs = [ctypes.byref(v) for v in o]
    assert lib.msd_groupnorm_plan(2, 320, 4096, 0, msd.DTYPE_F16, 0, 0, *refs) == 1   # no groups
    assert lib.msd_groupnorm_plan(2, 321, 4096, 32, msd.DTYPE_F16, 0, 0, *refs) == 1  # channels % groups
    assert lib.msd_groupnorm_plan(2, 320, 4096, 32, 5, 0, 0, *refs) == 1              # unknown dtype
    assert lib.msd_groupnorm_plan(2, 320, 4096, 32, msd.DTYPE_F16, 0, 0, None, None, None, None) == 1
    assert lib.msd_groupnorm_plan(33, 320, 4096, 32, msd.DTYPE_F16, 1, 0, *refs) == -2  # beyond the fixed scratch


@pytest.mark.parametrize("seed", range(6))
def test_random_shapes_always_get_a_launch_that_fits(seed):
    rng = random.Random(seed)
    lib = msd.load_library()
    knobs = [(0, 0, 0)] + [(rng.choice([0, 1, 2, 4, 8, 16, 32, 64]), rng.choice([0, 64, 128, 256, 320, 512, 640, 768, 1024]),
                            rng.choice([0, 0, 1, 2, 4, 8, 16])) for _ in range(4)]
    try:
        for split_knob, threads_knob, writers_knob in knobs:
            assert lib.msd_set_tuning(msd.TUNE_GN_SPLIT, split_knob) == 0
            assert lib.msd_set_tuning(msd.TUNE_GN_THREADS, threads_knob) == 0
            assert lib.msd_set_tuning(msd.TUNE_GN_WRITERS, writers_knob) == 0
            for _ in range(1500):
                groups = rng.choice([1, 2, 8, 32, 32, 32, 64])
                cpg = rng.choice([1, 2, 3, 5, 10, 20, 30, 40, 60, 80, 128, 1100])
                hw = rng.choice([8, 16, 24, 64, 72, 256, 1000, 1024, 4096, 4104, 16384, 65536, 262144])
                batch = rng.choice([1, 2, 2, 3, 8, 16, 32, 64, 300])
                code = rng.choice([msd.DTYPE_F16, msd.DTYPE_F32])
                if cpg * hw > 0x7FFFFFFF or batch * groups > 0x7FFFFFFF:
                    continue
                _check(batch, groups * cpg, hw, groups, code, noalloc=batch * groups <= STATIC_UNITS and rng.random() < 0.3,
                       in_place=rng.random() < 0.3)
    finally:
        lib.msd_set_tuning(msd.TUNE_GN_SPLIT, 0)
        lib.msd_set_tuning(msd.TUNE_GN_THREADS, 0)
        lib.msd_set_tuning(msd.TUNE_GN_WRITERS, 0)


def _table_rows():
    import os
    import re
    path = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "mobile-stable-diffusion_amd", "csrc",
                        "gn_plan_table.inc")
    rows = []
    for line in open(path):
        m = re.match(r"\s*\{(\d+),\s*(\d+),\s*(\d+),\s*(\d+),\s*(\d+),\s*(\d+),\s*(\d+)\}", line)
        if m:
            rows.append(tuple(int(v) for v in m.groups()))
    return rows


def test_every_row_of_the_table_of_measured_plans_is_the_plan_its_shape_gets():
    """The table is data written by gn_plan_table.py: each row must name a launch the kernels are
    built for, and gn_decide must hand exactly that launch to the shape the row is for (on the
    chip the table belongs to) - and something else, the rule's plan, when the table is off."""
    rows = _table_rows()
    assert 20 <= len(rows) <= 200 and len(set(r[:4] for r in rows)) == len(rows)   # one row per shape
    differs = 0
    for elt, apart, vectors, units, split, threads, writers in rows:
        code = msd.DTYPE_F16 if elt == 2 else msd.DTYPE_F32
        assert units % 32 == 0 and vectors % 10 == 0
        batch, channels, hw = units // 32, 320, vectors * (16 // elt) // 10      # 10 channels per group
        got = _check(batch, channels, hw, 32, code, in_place=not apart)
        assert (got[0], got[1], got[3]) == (split, threads, writers), (elt, apart, vectors, units, got)
        _knobs(msd, GN_PLAN_RULE_ONLY=1)
        try:
            differs += _check(batch, channels, hw, 32, code, in_place=not apart) != got
        finally:
            _knobs(msd, GN_PLAN_RULE_ONLY=0)
    assert differs == len(rows)          # a row exists only where the rule alone picks another plan


def test_table_generator_keeps_shipped_plans_within_three_percent_and_writes_rows_only_where_the_rule_differs(tmp_path):
    """gn_plan_table.py on a synthetic sweep: a shape whose shipped plan is within 3 % of the fastest
    keeps it, one whose shipped plan is further behind gets the fastest, and no row is written where
    the rule alone already picks the candidate; away from the tuned batches a rule plan within 1 %
    of the candidate needs no row either."""
    import importlib.util
    import json
    import os
    here = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    spec = importlib.util.spec_from_file_location("gn_plan_table", os.path.join(here, "mobile-stable-diffusion_amd", "csrc",
                                                                               "gn_plan_table.py"))
    gen = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(gen)

    def text(plan):
        return "%dx%dx%d" % plan[:3] + (" w%d" % plan[3] if plan[3] > 1 else "")

    def row(batch, c, hw, dtype, in_place, auto, variants):
        elt = 2 if dtype == "f16" else 4
        return {"batch": batch, "c": c, "hw": hw, "dtype": dtype, "in_place": in_place, "units": batch * 32,
                "vectors_per_unit": c // 32 * hw * elt // 16, "auto": text(auto), "variants": {text(p): us for p, us in variants.items()}}

    _knobs(msd, GN_PLAN_RULE_ONLY=1)
    try:
        rule_a = msd.groupnorm_plan(2, 320, 4096, 32, msd.DTYPE_F16, in_place=True)     # tuned batch
        rule_b = msd.groupnorm_plan(2, 640, 4096, 32, msd.DTYPE_F16, in_place=True)
        rule_c = msd.groupnorm_plan(4, 960, 4096, 32, msd.DTYPE_F16, in_place=True)     # batch 4: not a tuned batch
    finally:
        _knobs(msd, GN_PLAN_RULE_ONLY=0)
    shipped_a, fast_b, fast_c = (4, 768, 2, 1), (8, 640, 2, 1), (4, 960, 4, 1)
    assert shipped_a != rule_a and fast_b != rule_b and fast_c != rule_c
    sweep = [
        row(2, 320, 4096, "f16", True, shipped_a, {shipped_a: 6.10, rule_a: 6.00, (2, 1024, 3, 1): 6.05}),   # within 3 %: stays
        row(2, 640, 4096, "f16", True, rule_b, {rule_b: 7.50, fast_b: 7.00}),                                # 7 % behind: replaced
        row(4, 960, 4096, "f16", True, fast_c, {fast_c: 12.00, rule_c: 12.05}),                              # rule within 1 %: no row
        row(2, 1280, 256, "f16", True, msd.groupnorm_plan(2, 1280, 256, 32, msd.DTYPE_F16, in_place=True),
            {msd.groupnorm_plan(2, 1280, 256, 32, msd.DTYPE_F16, in_place=True): 3.5}),
    ]
    src = tmp_path / "sweep.json"
    src.write_text(json.dumps({"gn_plan_sweep": sweep}) + "\n")
    out = tmp_path / "table.inc"
    rows = gen.main([str(src)], str(out))
    body = [l for l in out.read_text().splitlines() if l.strip().startswith("{")]
    assert rows == body and len(body) in (2, 3)
    assert any("{2, 0,  5120,   64, 4,  768, 1}" in l for l in body)        # the shipped plan kept
    assert any("{2, 0, 10240,   64, 8,  640, 1}" in l for l in body)        # the faster plan taken
    assert not any(" 15360,  128," in l for l in body)                      # no row: the rule is as good
