"""Dry runs of the fused aggregation entry points on the CPU: which kernel a shape is sent to and
with what launch geometry (no device, no launch).  Every lane-group count a kernel's loops step
by must be at least one, for every shape the eligibility checks let through."""
import ctypes

import pytest

from f2cgt_amd import capi

A16 = ctypes.c_void_p(1 << 20)   # a 16-byte aligned stand-in for every buffer (never dereferenced)


def plan_log_sq(bits, feat_dim, rows=1000, fanout=10, n_cb=1, idx=capi.DT_I64):
    per = max(1, 8 // bits)
    src_dim = (feat_dim + per - 1) // per
    column_slice = (feat_dim + n_cb - 1) // n_cb
    dt = capi.DT_I16 if bits == 16 else (capi.DT_I8 if bits == 8 else capi.DT_U8)
    return capi.dry_run("f2cgt_sq_decompress_spmm_csr", A16, dt, A16, A16, A16, idx, A16, rows, rows * fanout,
                        5000, src_dim, feat_dim, n_cb, bits, column_slice, None)


def plan_affine(bits, feat_dim, rows=1000, fanout=10, idx=capi.DT_I64):
    per = 8 // bits
    src_dim = (feat_dim + per - 1) // per
    return capi.dry_run("f2cgt_sq_affine_decompress_spmm_csr", A16, A16, feat_dim, A16, A16, idx, A16, rows,
                        rows * fanout, 5000, src_dim, feat_dim, bits, None)


def check_geometry(plan):
    name = plan.kernel.decode()
    assert plan.grid >= 1 and plan.block in (64, 128, 256, 512, 1024), (name, plan.grid, plan.block)
    assert plan.lds_bytes <= 160 * 1024
    if name == "sq_block_kernel":
        assert plan.aux[0] >= 1 and plan.aux[1] >= 1 and plan.rows_per_block >= 1      # row slots, edge capacity
    elif name == "sq_rows_kernel":
        assert plan.aux[0] >= 1 and plan.aux[1] >= 1 and plan.aux[2] >= 8 and plan.rows_per_block >= 8
    elif name == "sq_affine_acc_kernel":
        assert plan.aux[0] >= 1 and plan.aux[1] >= 1 and plan.aux[2] >= 8 and plan.rows_per_block >= plan.aux[2]
    elif name == "hybrid_acc_kernel":
        assert plan.aux[0] >= 1 and plan.rows_per_block >= 8
    elif name == "agg_kernel":
        assert plan.aux[0] >= 1
    else:
        assert name in ("vq_wave_kernel", "vq_pipe_kernel", "vq_strip_kernel"), name
    return name


WIDE = [2040, 2044, 2048, 2052, 3000, 4080, 4088, 4092, 4096]


@pytest.mark.parametrize("bits", [1, 2, 4, 8])
def test_fused_sq_geometry_over_feature_widths(bits):
    per = 8 // bits
    dims = sorted(set([4, 8, 12, 16, 24, 36, 64, 100, 128, 256, 300, 512, 768, 1000, 1024, 2000] + WIDE +
                      [6, 10, 18, 30, 66, 102, 130, 602, 1022, 2042, 2046, 4090, 4094]))   # 4 k + 2 columns
    seen = set()
    for d in dims:
        for fanout in (1, 10, 60):
            if d % per == 0 or bits == 8:
                rc, plan = plan_log_sq(bits, d, fanout=fanout)
                assert rc == 0 and plan is not None, (bits, d, capi.lib().f2cgt_last_error())
                seen.add(check_geometry(plan))
            rc, plan = plan_affine(bits, d, fanout=fanout)
            assert rc == 0 and plan is not None, (bits, d, capi.lib().f2cgt_last_error())
            seen.add(check_geometry(plan))
    assert "sq_rows_kernel" in seen and (bits < 4 or "agg_kernel" in seen)


def test_even_widths_that_are_no_multiple_of_four_take_the_row_block_kernels():
    for d in (18, 66, 102, 602):
        for bits in (4, 8):
            assert plan_affine(bits, d)[1].kernel.decode() == "sq_affine_acc_kernel", (bits, d)
            assert plan_log_sq(bits, d)[1].kernel.decode() == "sq_rows_kernel", (bits, d)
    for bits in (1, 2):
        assert plan_log_sq(bits, 602)[1].kernel.decode() == "sq_rows_kernel"
        assert plan_affine(bits, 602)[1].kernel.decode() == "sq_rows_kernel"
    for d in (17, 101, 601):   # odd widths: one column per lane
        assert plan_affine(4, d)[1].kernel.decode() == "agg_kernel"
    vq = capi.dry_run("f2cgt_vq_decompress_spmm_csr", A16, capi.DT_U8, A16, A16, A16, capi.DT_I64, A16, 200_000,
                      2_000_000, 1_000_000, 602, 19, 256, 32, None)
    assert vq[0] == 0 and vq[1].kernel.decode() == "vq_wave_kernel" and vq[1].aux[0] == 1


def test_wide_rows_leave_the_row_block_kernels():
    # staged pitch above 2 KB: 8-bit codes from 2044 columns, 4-bit codes from 4088
    for bits, d in ((8, 2044), (8, 2048), (8, 4096), (4, 4088), (4, 4092), (4, 4096)):
        for planner in (plan_log_sq, plan_affine):
            rc, plan = planner(bits, d)
            assert rc == 0
            assert plan.kernel.decode() == "agg_kernel", (bits, d, plan.kernel)
    # just below the bound the staged-rows kernel still takes them
    assert plan_log_sq(8, 2040)[1].kernel.decode() == "sq_rows_kernel"
    assert plan_log_sq(4, 4080)[1].kernel.decode() == "sq_rows_kernel"


def test_headline_shapes_take_the_fast_kernels():
    rc, plan = plan_affine(4, 100, rows=250_000, fanout=2)
    assert rc == 0 and plan.kernel.decode() == "sq_affine_acc_kernel"
    rc, plan = plan_affine(8, 128, rows=10_000, fanout=10)
    assert rc == 0 and plan.kernel.decode() == "sq_affine_acc_kernel"
    rc, plan = plan_log_sq(4, 100, rows=250_000, fanout=2)
    assert rc == 0 and plan.kernel.decode() == "sq_rows_kernel"
    vq = lambda rows, fanout, d, n_cb, w: capi.dry_run(
        "f2cgt_vq_decompress_spmm_csr", A16, capi.DT_U8, A16, A16, A16, capi.DT_I64, A16, rows, rows * fanout,
        1_000_000, d, n_cb, 256, w, None)
    for rows, fanout, d, n_cb, w in ((500_000, 15, 128, 16, 8), (600_000, 10, 768, 24, 32), (4096, 15, 128, 16, 8)):
        rc, plan = vq(rows, fanout, d, n_cb, w)
        assert rc == 0 and plan.kernel.decode().startswith("vq_"), plan.kernel
        assert plan.lds_bytes <= 160 * 1024
    hyb = capi.dry_run("f2cgt_hybrid_decompress_spmm_csr", A16, A16, A16, 128, A16, A16, A16, A16, capi.DT_I64, A16,
                       1_000_000, 12_000_000, 100_000_000, 5_000_000, 95_000_000, 128, 8, 256, 16, None)
    assert hyb[0] == 0 and hyb[1].kernel.decode() == "hybrid_acc_kernel"
    # four columns: one chunk per row, outside the row-block form (its reciprocal does not fit 32 bits)
    hyb4 = capi.dry_run("f2cgt_hybrid_decompress_spmm_csr", A16, A16, A16, 4, A16, A16, A16, A16, capi.DT_I64, A16,
                        100, 1000, 1000, 500, 500, 4, 1, 256, 4, None)
    assert hyb4[0] == 0 and hyb4[1].kernel.decode() == "agg_kernel"


def test_unsigned_eight_bit_log_codes_are_refused():
    lib = capi.lib()
    rc = lib.f2cgt_sq_decompress(A16, capi.DT_U8, A16, A16, 4, 16, 16, 1, 8, 16, None)
    assert rc == -2 and b"int8" in lib.f2cgt_last_error()
    rc, _ = capi.dry_run("f2cgt_sq_decompress_spmm_csr", A16, capi.DT_U8, A16, A16, A16, capi.DT_I64, A16, 4, 8, 10,
                         16, 16, 1, 8, 16, None)
    assert rc == -2 and b"int8" in lib.f2cgt_last_error()
    rc, plan = capi.dry_run("f2cgt_sq_decompress_spmm_csr", A16, capi.DT_I8, A16, A16, A16, capi.DT_I64, A16, 4, 8,
                            10, 16, 16, 1, 8, 16, None)
    assert rc == 0 and plan is not None


def test_rows_per_block_follow_the_launch_size():
    # integer-accumulating kernel: the degree decides from 2.5e5 rows on, smaller launches get smaller
    # blocks (at least 8 rows) so that a CU still overlaps several of them
    want = {(250_000, 2): 64, (65_536, 2): 32, (16_384, 2): 8, (1024, 2): 8, (10_000, 10): 8}
    for (rows, fanout), rb in want.items():
        bits, d = (8, 128) if fanout == 10 else (4, 100)
        rc, plan = plan_affine(bits, d, rows=rows, fanout=fanout)
        assert rc == 0 and plan.kernel.decode() == "sq_affine_acc_kernel"
        assert plan.rows_per_block == rb, (rows, fanout, plan.rows_per_block)
        assert plan.rows_per_block % plan.aux[2] == 0 and plan.grid == -(-rows // rb)
    # staged-rows kernel: at least 16 rows, about a thousand workgroups
    for rows, rb in ((250_000, 64), (65_536, 64), (16_384, 16), (4096, 16), (20_000, 16)):
        rc, plan = plan_log_sq(4, 100, rows=rows, fanout=2)
        assert rc == 0 and plan.kernel.decode() == "sq_rows_kernel"
        assert plan.rows_per_block == rb, (rows, plan.rows_per_block)
    # long rows keep their small degree-based blocks
    rc, plan = plan_log_sq(4, 100, rows=4096, fanout=60)
    assert rc == 0 and plan.rows_per_block == 8


def test_fused_vq_store_form_by_shape():
    """aux[2] of a vq_wave_kernel plan is the store form: 1 = results turned round in LDS (up to 8 edges per row, and up
    to 16 for an output of 200 MB and more from a code table of 64 to 192 MB, or throughout in the streaming store mode),
    4 = halves exchanged inside lane quads (a cached table: up to 11 edges per row, or a large output), 0 = stored as they
    are; aux[3] is the binary logarithm of the number of lanes that own the columns of a code together (2 for
    codebooks of 32 columns from a cached table where neither of the other forms is taken)."""
    def form(rows, fanout, d, n_cb, w, n_src):
        rc, plan = capi.dry_run("f2cgt_vq_decompress_spmm_csr", A16, capi.DT_U8, A16, A16, A16, capi.DT_I64, A16, rows,
                                rows * fanout, n_src, d, n_cb, 256, w, None)
        assert rc == 0 and plan.kernel.decode() == "vq_wave_kernel"
        return plan.aux[2], plan.aux[3]
    assert form(300_000, 5, 128, 16, 8, 1_000_000) == (1, 0)
    assert form(300_000, 5, 128, 4, 32, 1_000_000) == (1, 0)
    assert form(300_000, 10, 128, 16, 8, 1_000_000) == (4, 0)
    assert form(150_000, 10, 256, 16, 16, 1_000_000) == (4, 0)
    assert form(300_000, 10, 256, 16, 16, 1_000_000) == (4, 0)      # 307 MB of output from 16 MB of codes
    assert form(300_000, 14, 256, 16, 16, 1_000_000) == (4, 0)
    assert form(300_000, 14, 256, 16, 16, 10_000_000) == (1, 0)     # from 160 MB of codes
    assert form(100_000, 14, 256, 16, 16, 1_000_000) == (0, 0)
    assert form(300_000, 10, 512, 16, 32, 1_000_000) == (4, 0)
    assert form(100_000, 14, 512, 16, 32, 1_000_000) == (0, 2)
    assert form(200_000, 10, 768, 24, 32, 1_000_000) == (0, 2)       # six column tiles
    assert form(500_000, 15, 128, 16, 8, 10_000_000) == (1, 0)      # 256 MB of output from a 160 MB table
    assert form(100_000, 15, 128, 16, 8, 10_000_000) == (0, 0)      # 51 MB of output: the halves meet in the cache
    assert form(600_000, 10, 768, 24, 32, 240_000_000) == (0, 0)    # a 5.8 GB table: the gather dominates
    assert form(200_000, 10, 768, 96, 8, 1_000_000) == (0, 0)       # six column tiles
    assert form(300_000, 10, 64, 8, 8, 1_000_000) == (0, 0)         # half the lanes of a row beyond the columns
    assert form(300_000, 20, 128, 16, 8, 1_000_000) == (0, 0)       # two-row mini-blocks
    assert form(300_000, 20, 128, 4, 32, 1_000_000) == (0, 0)
    assert form(300_000, 10, 600, 19, 32, 1_000_000) == (0, 0)      # 600 columns: the last tile ends inside a group of 32
    assert form(300_000, 10, 100, 13, 8, 1_000_000)[1] == 0         # four columns per lane: dense as they are
    was = capi.set_store_mode(capi.STORE_STREAM)
    try:
        assert form(600_000, 10, 768, 24, 32, 240_000_000) == (1, 0)
        assert form(300_000, 10, 128, 16, 8, 1_000_000) == (1, 0)
        assert form(300_000, 20, 128, 16, 8, 1_000_000) == (0, 0)
    finally:
        capi.set_store_mode(was)
    # aux[0]: float4 per lane and edge (2 = a lane owns eight columns); sparse rows that are no whole 128-byte lines
    # take one, code rows that are no multiple of a tile (24 x 8, 7 x 32) can take the turn through LDS
    lanes = lambda rows, fanout, d, n_cb, w: capi.dry_run(
        "f2cgt_vq_decompress_spmm_csr", A16, capi.DT_U8, A16, A16, A16, capi.DT_I64, A16, rows, rows * fanout,
        1_000_000, d, n_cb, 256, w, None)[1].aux[0]
    assert lanes(1_000_000, 3, 200, 25, 8) == 1 and lanes(300_000, 10, 200, 25, 8) == 2
    assert lanes(1_000_000, 3, 192, 24, 8) == 2 and form(1_000_000, 3, 192, 24, 8, 1_000_000) == (1, 0)
    assert lanes(1_000_000, 3, 224, 7, 32) == 2 and lanes(1_000_000, 3, 600, 19, 32) == 1
