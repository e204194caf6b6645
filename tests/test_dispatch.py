"""Host-only: which kernel, tile shape and split the launchers choose.
``int4mm_describe_launch`` runs the launchers' own decision code with the launches
switched off.  The benchmark configurations are pinned exactly -- an edit of a shape
rule that silently reroutes one of them fails here, without a GPU; every other shape
is held to properties: a kernel that exists, launched within its limits."""
import pytest

from int4matmul_kernels_amd import capi

K, S = 5120, 20480


def d(*a, **kw):
    return capi.describe_launch(*a, **kw)


def test_matvec_configurations():
    # C1: K = S = 1024, g = 64
    assert d("vec", 4, 1, 1, 1024, 1024, 64).startswith(
        "matvec_kernel<bits=4,dense,lane_groups=4,prefetch=0> strips=16 splits=4 waves=2 units_per_workgroup=5")
    # C2: 640 workgroups of four waves; the three writing splits take 23 units each, the summing one 11.
    # Its transposed shape has 8 splits, which share K equally
    assert d("vec", 4, 1, 1, K, S, 128).startswith(
        "matvec_kernel<bits=4,dense,lane_groups=2,prefetch=0> strips=160 splits=4 waves=4 units_per_workgroup=23")
    assert d("vec", 4, 1, 1, S, K, 128).startswith(
        "matvec_kernel<bits=4,dense,lane_groups=4,prefetch=0> strips=80 splits=8 waves=4 units_per_workgroup=40")
    # C4: 16:32 at K = S = 16384, g = 64
    assert d("vec", 4, 1, 1, 16384, 16384, 64, sparse=True).startswith(
        "matvec_kernel<bits=4,16:32,lane_groups=4,prefetch=1> strips=256 splits=3 waves=4 units_per_workgroup=103")
    # C5: int3 / int2 take the shape of C2
    for bits in (3, 2):
        assert d("vec", bits, 1, 1, K, S, 128).startswith(
            f"matvec_kernel<bits={bits},dense,lane_groups=2,prefetch=0> strips=160 splits=4 waves=4 units_per_workgroup=23")


@pytest.mark.parametrize("bits", [4, 3, 2])
def test_dense_matmul_m2048(bits):
    # 640 tiles of 256 x 256 in the two-phase order; the 128 tiles of the third round split in two along K
    want = (f"matmul_kernel_pipe<bits={bits},dense,tile=256x256,two-phase> tiles=640 ksplit=2 split_from=512 "
            "workgroups=768")
    assert d("mtx", bits, 1, 2048, K, S, 128).startswith(want)
    # without room for the partial tiles the last round stays whole
    assert "ksplit=1 split_from=0 workgroups=640" in d("mtx", bits, 1, 2048, K, S, 128, workspace_bytes=0)


def test_other_matmul_configurations():
    assert d("mtx", 4, 1, 2048, S, K, 128).startswith("matmul_kernel_pipe<bits=4,dense,tile=256x256,two-phase> tiles=160")
    # C3 small: one group, 16 tiles of the general kernel (the pipelined kernel's prologue would dominate)
    assert d("mtx", 4, 1, 2048, 128, 128, 128).startswith("matmul_kernel<bits=4,dense,tile=128x128> tiles=16")
    # C4: the 16:32 format keeps the plain order (its decode has no registers to spare)
    assert d("mtx", 4, 1, 2048, K, S, 64, sparse=True).startswith(
        "matmul_kernel_pipe<bits=4,16:32,tile=256x256,plain> tiles=640 ksplit=2 split_from=512 workgroups=768")


def test_baseline_shape_with_few_rows():
    # the few-row legs that bench.py reports at the benchmark shape (K=5120, S=20480): 2 rows through the matvec kernel (a row per
    # MFMA result register), 8 rows through the few-row kernel, 64 rows through the kernel with shared staging
    assert d("mtx", 4, 1, 2, K, S, 128).startswith("matvec_kernel<bits=4,dense,lane_groups=2,prefetch=0,rows=2> strips=160 splits=4")
    # (320 strips of 64 columns on 256 CUs: 256 workgroups share the strips' units evenly)
    shared = "skinny_kernel<bits=4,dense,columns_per_lane=4,row_tiles=1,balanced> strips=320 row_blocks=1 workgroups=256 waves=8"
    assert d("mtx", 4, 1, 8, K, S, 128).startswith(shared)
    assert d("vec", 4, 8, 1, K, S, 128).startswith(shared)
    assert d("mtx", 4, 1, 64, K, S, 128).startswith("wide_rows_kernel<bits=4,dense,row_tiles=4> strips=80 row_blocks=1 ksplit=3")
    # a single row through the matmul entry: the matvec kernel (all formats), the same launch as the matvec entry's
    for bits, sparse, g in ((4, False, 128), (3, False, 128), (2, False, 128), (4, True, 64)):
        assert d("mtx", bits, 1, 1, K, S, g, sparse) == d("vec", bits, 1, 1, K, S, g, sparse)
        assert d("mtx", bits, 1, 1, K, S, g, sparse).startswith("matvec_kernel<bits=%d," % bits)


# ---- every other shape: properties of the choice, not the choice itself (the shape rules are tuned on
# measurements and may move; what must hold is that a kernel that exists is launched within its limits)
KERNELS = ("matvec_kernel", "skinny_kernel", "wide_rows_kernel", "matmul_kernel_pipe", "matmul_kernel")
SHAPES = [(k, s) for k in (64, 512, 2048, 4096, 5120, 8192, 14336, 28672) for s in (64, 512, 2048, 4096, 5120, 11008, 20480, 32768)]
ROWS = (1, 2, 3, 4, 5, 8, 16, 17, 32, 33, 64, 65, 96, 128, 129, 192, 256, 257, 384, 512, 513, 1024, 1280, 2048, 4097)


def fields(line):
    """'name<template args> key=value key=value ...; ' -> (name, {key: int})"""
    import re
    head = line.split(";")[0]
    name = head.split("<")[0]
    return name, {k: int(v) for k, v in re.findall(r"(\w+)=(\d+)(?![x\d])", head)}, head


@pytest.mark.parametrize("fmt", [(4, False, 128), (3, False, 128), (2, False, -1), (4, True, 64)])
def test_every_shape_gets_a_kernel_within_its_limits(fmt):
    bits, sparse, g = fmt
    for k, s in SHAPES:
        for rows in ROWS:
            line = d("mtx", bits, 1, rows, k, s, g, sparse)
            name, f, head = fields(line)
            assert name in KERNELS, line
            assert f"bits={bits}," in head and ("16:32" in head) == sparse, line
            if name == "matvec_kernel":
                cols = 256 // f["lane_groups"]
                assert f["strips"] * cols >= s and (f["strips"] - 1) * cols < s, line
                nr = int(head.split(",rows=")[1][0]) if ",rows=" in head else 1
                assert 1 <= f["splits"] * nr <= 32 and 1 <= f["waves"] <= 8, line
                assert f["splits"] * f["units_per_workgroup"] >= k // 64 and f["units_per_workgroup"] * nr <= 224, line
                assert rows <= 4
            elif name in ("skinny_kernel", "wide_rows_kernel"):
                assert 2 <= rows <= 512 and f["strips"] >= 1, line
                assert f.get("ksplit", 1) >= 1 and f.get("row_blocks", 1) * 16 * f["row_tiles"] >= rows, line
            else:
                tm, tn = (int(v) for v in head.split("tile=")[1].split(",")[0].split(">")[0].split("x"))
                assert f["tiles"] >= -(-rows // tm) * -(-s // tn) // 1 and f["tiles"] >= 1, line
                assert 1 <= f.get("ksplit", 1) <= 8, line
            # without a workspace nothing may split K across workgroups
            bare = d("mtx", bits, 1, rows, k, s, g, sparse, workspace_bytes=0)
            n2, f2, _ = fields(bare)
            assert n2 in KERNELS and f2.get("ksplit", 1) == 1 and f2.get("splits", 1) == 1, bare


def evenly_shared(line):
    return "balanced" in line or "columns_per_lane=4+1" in line


def test_more_strips_than_cus_are_shared_out_evenly_within_limits():
    assert evenly_shared(d("mtx", 4, 1, 8, 12288, 28672, 128)) and evenly_shared(d("mtx", 4, 1, 16, 3072, 16448, 64, True))
    assert not evenly_shared(d("mtx", 4, 1, 17, 3072, 17408, 128))          # more than 16 rows
    assert not evenly_shared(d("mtx", 4, 1, 8, 2048, 20480, 128))           # a short K
    assert not evenly_shared(d("mtx", 4, 1, 8, 8192, 22016, 128))           # many more strips than CUs, K not long
    assert not evenly_shared(d("mtx", 4, 1, 8, 5120, 16384, 128))           # a strip per CU
    # without a workspace there is nowhere to sum a shared strip: a workgroup per strip; slivers need none
    assert not evenly_shared(d("mtx", 4, 1, 8, 5120, 20480, 128, False, 0))
    assert "columns_per_lane=4+1" in d("mtx", 3, 1, 8, 5120, 20480, 128, False, 0)
    # tuning key 9 = 1 switches both off
    capi.tune(9, 1)
    try:
        assert not evenly_shared(d("mtx", 4, 1, 8, K, S, 128)) and not evenly_shared(d("mtx", 3, 1, 8, K, S, 128))
    finally:
        capi.tune(9, 0)
    # the shared launch's partial tiles fit the workspace that the size query asks for
    for bits, sparse in ((4, False), (4, True)):
        for k, s in ((3072, 16448), (5120, 20480), (12288, 32704)):
            assert capi.matmul_workspace_bytes(1, 16, k, s, sparse) >= 2 * ((s // 64) * 2 * 8192), (k, s)


def test_workspace_sizes_are_consistent():
    lib = capi.lib()
    prev = 0
    for s in (64, 256, 1024, 4096, 20480, 32768, 131072):
        n = lib.int4mm_workspace_bytes(s)
        assert n >= prev and n >= 2 * (32 * 8 * s)              # 32 splits of {fp32, flag} per column, kept twice
        prev = n
        for k in (64, 4096, 28672):
            for rows in (1, 8, 64, 300, 2048):
                for sparse in (False, True):
                    assert capi.matmul_workspace_bytes(1, rows, k, s, sparse) >= n


def test_matvec_of_a_k_beyond_one_launch():
    # 32 x 224 units of 64 rows is what one launch covers: a longer K runs as several launches (one line each)
    line = d("vec", 4, 1, 1, 1 << 20, 256, 128)
    assert line.count("matvec_kernel<") == 3, line
    assert d("vec", 4, 1, 1, 458752, 256, 128).count("matvec_kernel<") == 1
    with pytest.raises(capi.Int4mmError):                     # a single group longer than a launch covers, on a longer K
        d("vec", 4, 1, 1, 1 << 20, 256, 1 << 19)
    assert d("vec", 4, 1, 1, 1 << 20, 256, -1).count("matvec_kernel<") == 3       # one group: any cut will do


def test_matvec_needs_its_workspace_whatever_the_shape():
    # K = 64: a single unit, nothing to hand over -- the documented rule holds all the same
    with pytest.raises(capi.Int4mmError) as e:
        d("vec", 4, 1, 1, 64, 64, 64, workspace_bytes=0)
    assert e.value.code == 6
    assert d("vec", 4, 1, 1, 64, 64, 64, workspace_bytes=capi.lib().int4mm_workspace_bytes(64)).startswith("matvec_kernel")


def test_tuning_is_per_thread_and_describe_leaves_no_trace():
    import threading
    capi.tune(3, 1)
    try:
        seen = {}
        t = threading.Thread(target=lambda: seen.setdefault("other", d("mtx", 4, 1, 2048, K, S, 128)))
        t.start()
        t.join()
        assert seen["other"].startswith("matmul_kernel_pipe")            # the other thread keeps the defaults
        assert d("mtx", 4, 1, 2048, K, S, 128).startswith("matmul_kernel<bits=4,dense,tile=128x128>")
    finally:
        capi.tune(3, 0)
    assert d("mtx", 4, 1, 2048, K, S, 128).startswith("matmul_kernel_pipe")
