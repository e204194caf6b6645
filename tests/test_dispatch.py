"""Host-only: which kernel, tile shape and split the launchers choose for every
benchmark configuration.  ``int4mm_describe_launch`` runs the launchers' own
decision code with the launches switched off, so an edit of a shape rule that
silently reroutes one of these shapes fails here, without a GPU."""
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


def test_long_k_on_a_narrow_output():
    # one round of unsplit 128 x 256 tiles loses to 256 x 128 tiles split three ways when the shares of K stay long
    assert d("mtx", 4, 1, 1024, S, K, 128).startswith("matmul_kernel_pipe<bits=4,dense,tile=256x128,plain> tiles=160 ksplit=3")
    assert d("mtx", 4, 1, 1280, S, K, 128).startswith("matmul_kernel_pipe<bits=4,dense,tile=128x256,plain> tiles=200 ksplit=1")
    assert d("mtx", 4, 1, 1024, 8192, 8192, 128).startswith("matmul_kernel_pipe<bits=4,dense,tile=128x256,plain> tiles=256 ksplit=1")
    # (without a workspace for the partial tiles: unsplit)
    assert "tile=128x256" in d("mtx", 4, 1, 1024, S, K, 128, workspace_bytes=0)


def test_two_to_four_rows_take_the_matvec_kernel_up_to_k_5120():
    assert d("mtx", 4, 1, 3, K, S, 128).startswith(
        "matvec_kernel<bits=4,dense,lane_groups=2,prefetch=0,rows=4> strips=160 splits=4 waves=4 units_per_workgroup=23 rows=3")
    assert d("vec", 3, 2, 1, K, S, 128).startswith("matvec_kernel<bits=3,dense,lane_groups=2,prefetch=0,rows=2>")
    assert d("mtx", 4, 2, 2, 4096, 22016, 128).startswith("matvec_kernel<bits=4,dense,lane_groups=2,prefetch=0,rows=4> strips=172 splits=")
    assert d("mtx", 4, 2, 2, 4096, 11008, 128).startswith("skinny_kernel")           # (one round of 64-column strips there)
    assert d("mtx", 4, 1, 3, 8192, 22016, 128).startswith("skinny_kernel")          # long K: the few-row kernel
    # narrow outputs stay with the few-row kernel: two rows below 8192 columns, three and four up to 16384
    assert d("mtx", 4, 1, 2, 4096, 4096, 128).startswith("skinny_kernel")
    assert d("mtx", 4, 1, 2, 4096, 8192, 128).startswith("matvec_kernel<bits=4,dense,lane_groups=4,prefetch=0,rows=2>")
    assert d("mtx", 4, 1, 4, 5120, 8192, 128).startswith("skinny_kernel")
    assert d("mtx", 4, 1, 4, 5120, 16384, 128).startswith("skinny_kernel")
    assert d("mtx", 4, 1, 2, 5120, 16384, 128).startswith("matvec_kernel")
    # a single row through the matmul entry: the matvec kernel (all formats), the same launch as the matvec entry's
    for bits, sparse, g in ((4, False, 128), (3, False, 128), (2, False, 128), (4, True, 64)):
        assert d("mtx", bits, 1, 1, K, S, g, sparse) == d("vec", bits, 1, 1, K, S, g, sparse)
        assert d("mtx", bits, 1, 1, K, S, g, sparse).startswith("matvec_kernel<bits=%d," % bits)
    assert d("mtx", 4, 1, 2, 8192, 22016, 128).startswith("matvec_kernel<bits=4,dense,lane_groups=2,prefetch=1,rows=2> strips=172 splits=4")
    assert d("mtx", 4, 1, 2, 14336, 4096, 128).startswith("skinny_kernel")          # ... two rows too when K is split ten ways
    assert d("mtx", 4, 1, 3, 2048, 32768, 128).startswith("skinny_kernel")          # short K: only two rows
    assert d("mtx", 4, 1, 2, 2048, 32768, 128).startswith("matvec_kernel")
    assert d("mtx", 4, 1, 5, K, S, 128).startswith("skinny_kernel")
    assert d("mtx", 4, 1, 3, K, S, 64, sparse=True).startswith("skinny_kernel<bits=4,16:32")
    assert d("mtx", 4, 1, 3, K, S, 128, workspace_bytes=0).startswith("skinny_kernel")  # no room for the hand-over


def test_few_rows_and_batches():
    assert d("mtx", 4, 1, 8, K, S, 128).startswith("skinny_kernel<bits=4,dense,columns_per_lane=4,row_tiles=1> strips=320")
    assert d("vec", 4, 8, 1, K, S, 128).startswith("skinny_kernel<bits=4,dense,columns_per_lane=4,row_tiles=1> strips=320")
    assert d("mtx", 4, 1, 64, K, S, 128).startswith("wide_rows_kernel<bits=4,dense,row_tiles=4> strips=80 row_blocks=1 ksplit=3")
    # 65 ... 128 rows in one block of six or eight 16-row tiles where K is split into long shares, in two blocks of
    # four where the split would have to be deeper or shorter
    assert d("mtx", 4, 1, 128, K, S, 128).startswith("wide_rows_kernel<bits=4,dense,row_tiles=8> strips=80 row_blocks=1 ksplit=3")
    assert d("mtx", 3, 1, 70, K, S, 128).startswith("wide_rows_kernel<bits=3,dense,row_tiles=6> strips=80 row_blocks=1 ksplit=3")
    assert d("mtx", 4, 1, 128, 8192, 8192, 128).startswith("wide_rows_kernel<bits=4,dense,row_tiles=4> strips=32 row_blocks=2 ksplit=4")
    assert d("mtx", 4, 1, 128, 2048, 16384, 64).startswith("wide_rows_kernel<bits=4,dense,row_tiles=4> strips=64 row_blocks=2 ksplit=2")
    assert d("mtx", 4, 1, 200, 28672, 8192, 128).startswith("wide_rows_kernel<bits=4,dense,row_tiles=8> strips=32 row_blocks=2 ksplit=4")
    assert d("mtx", 4, 1, 96, K, S, 64, sparse=True).startswith("wide_rows_kernel<bits=4,16:32,row_tiles=6> strips=80 row_blocks=1 ksplit=3")
    assert d("mtx", 4, 1, 128, K, S, 64, sparse=True).startswith("wide_rows_kernel<bits=4,16:32,row_tiles=8> strips=80 row_blocks=1 ksplit=3")
    # (16:32 against 4096 ... 8192 columns: block height and split from its own fitted cost model)
    assert d("mtx", 4, 1, 128, 8192, 8192, 64, sparse=True).startswith("wide_rows_kernel<bits=4,16:32,row_tiles=8> strips=32 row_blocks=1 ksplit=8")
    # 129 ... 192 rows: on any output up to 32768 columns, with the block height and split the cost model picks;
    # 193 ... 256 rows: up to 10240 columns, and wider ones on a K of at most 4096
    assert d("mtx", 4, 1, 192, 4096, 14336, 128).startswith("wide_rows_kernel<bits=4,dense,row_tiles=6> strips=56 row_blocks=2 ksplit=2")
    assert d("mtx", 4, 1, 256, 4096, 14336, 128).startswith("wide_rows_kernel<bits=4,dense,row_tiles=4> strips=56 row_blocks=4 ksplit=1")
    assert d("mtx", 4, 1, 192, 2048, 12288, 128).startswith("wide_rows_kernel<bits=4,dense,row_tiles=3> strips=48 row_blocks=4 ksplit=1")
    assert d("mtx", 4, 1, 192, K, S, 128).startswith("wide_rows_kernel<bits=4,dense,row_tiles=4> strips=80 row_blocks=3 ksplit=1")
    assert d("mtx", 4, 1, 256, K, S, 128).startswith("matmul_kernel_pipe<bits=4,dense,tile=256x128")
    assert d("mtx", 4, 1, 256, 8192, 14336, 128).startswith("matmul_kernel_pipe<bits=4,dense,tile=256x128")
    assert d("mtx", 4, 1, 192, 8192, 8192, 64, sparse=True).startswith("wide_rows_kernel<bits=4,16:32,row_tiles=6> strips=32 row_blocks=2 ksplit=4")
    # up to 512 rows on outputs of at most 8192 columns; wider outputs and the 16:32 format go to the tile kernels
    assert d("mtx", 4, 1, 384, 4096, 4096, 128).startswith("wide_rows_kernel<bits=4,dense,row_tiles=3> strips=16 row_blocks=8 ksplit=2")
    # (65 ... 512 rows against 4096 ... 8192 columns: block height and split from the fitted cost model -- a short K is
    # not split into shares of a few units, blocks of 48 rows where they fill the GPU better)
    assert d("mtx", 4, 1, 416, 2048, 8192, 128).startswith("wide_rows_kernel<bits=4,dense,row_tiles=4> strips=32 row_blocks=7 ksplit=1")
    assert d("mtx", 4, 1, 160, 4096, 8192, 128).startswith("wide_rows_kernel<bits=4,dense,row_tiles=3> strips=32 row_blocks=4 ksplit=2")
    assert d("mtx", 3, 1, 352, 8192, 8192, 128).startswith("wide_rows_kernel<bits=3,dense,row_tiles=6> strips=32 row_blocks=4 ksplit=2")
    assert d("mtx", 4, 1, 128, 8192, 8192, 128).startswith("wide_rows_kernel<bits=4,dense,row_tiles=4> strips=32 row_blocks=2 ksplit=4")
    assert d("mtx", 4, 1, 384, K, S, 128).startswith("matmul_kernel_pipe<bits=4,dense,tile=128x256")
    assert d("mtx", 4, 1, 384, 8192, 8192, 64, sparse=True).startswith("matmul_kernel_pipe<bits=4,16:32")
    assert d("mtx", 4, 1, 513, 4096, 4096, 128).startswith("matmul_kernel")
    assert d("mtx", 4, 1, 16, S, K, 128).startswith("skinny_kernel<bits=4,dense")
    # 33 ... 64 rows: the few-row kernel where its two row blocks per strip make one round of workgroups (strips cut for
    # that), the wide kernel on a longer K or where no strip width gives such a round
    assert d("mtx", 4, 1, 40, 2048, 8192, 128).startswith("skinny_kernel<bits=4,dense,columns_per_lane=4,row_tiles=4> strips=128 row_blocks=2")
    assert d("mtx", 4, 1, 64, 8192, 4096, 128).startswith("skinny_kernel<bits=4,dense,columns_per_lane=2,row_tiles=4> strips=128 row_blocks=2")
    assert d("mtx", 4, 1, 64, 8192, 8192, 128).startswith("wide_rows_kernel<bits=4,dense,row_tiles=4>")
    assert d("mtx", 4, 1, 64, 11008, 4096, 128).startswith("wide_rows_kernel<bits=4,dense,row_tiles=2> strips=16 row_blocks=2 ksplit=8")
    assert d("mtx", 4, 1, 40, 4096, 5120, 64, True).startswith("wide_rows_kernel<bits=4,16:32,row_tiles=3>")
    assert d("mtx", 4, 1, 40, 8192, 4096, 64, True).startswith("skinny_kernel<bits=4,16:32,columns_per_lane=2,row_tiles=4> strips=128 row_blocks=2")
    assert d("mtx", 4, 1, 257, K, S, 128).startswith("matmul_kernel_pipe<bits=4,dense,tile=128x256")


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
