"""Row fetch in front of the operators (the feature cache's `__getitem__`): the HIP kernel through
the C ABI against the oracle and torch indexing, bit for bit, for every row width class, with and
without a cache of hot rows, from device and from pinned host tables; then the `TensorCache`
class and the module function on top of it."""
import numpy as np
import pytest
import torch

import f2cgt_oracle as oc
from f2cgt_amd import capi

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


WIDTHS = [1, 2, 3, 4, 5, 7, 8, 9, 15, 16, 17, 24, 31, 32, 48, 50, 64, 100, 128, 400, 1000, 1024, 3072]


@pytest.mark.parametrize("idx", [np.int32, np.int64])
@pytest.mark.parametrize("row_bytes", WIDTHS)
def test_fetch_rows_every_width(row_bytes, idx):
    rng = np.random.default_rng(row_bytes)
    n = 4099
    table = rng.integers(0, 256, size=(n, row_bytes), dtype=np.uint8)
    index = rng.integers(0, n, size=3333).astype(idx)
    index[:5] = [0, n - 1, n - 1, 0, 1]
    got = host(capi.fetch_rows(dev(table), dev(index)))
    assert np.array_equal(got, oc.fetch_rows(table, index))
    assert np.array_equal(got, table[index])


@pytest.mark.parametrize("shift", [1, 2, 3, 4, 8, 12])
@pytest.mark.parametrize("row_bytes", [6, 16, 50, 64, 96])
def test_fetch_rows_from_misaligned_buffers(row_bytes, shift):
    rng = np.random.default_rng(100 * row_bytes + shift)
    n, m = 1500, 2000
    flat = dev(rng.integers(0, 256, size=n * row_bytes + 64, dtype=np.uint8))
    table = flat[shift:shift + n * row_bytes].view(n, row_bytes)
    out_flat = torch.zeros(m * row_bytes + 64, dtype=torch.uint8, device="cuda")
    out = out_flat[shift + 1:shift + 1 + m * row_bytes].view(m, row_bytes)
    index = rng.integers(0, n, size=m)
    capi.fetch_rows(table, dev(index), out=out)
    assert np.array_equal(host(out), host(table)[index])
    # nothing outside the output rows was written
    assert int(out_flat[:shift + 1].sum()) == 0 and int(out_flat[shift + 1 + m * row_bytes:].sum()) == 0


@pytest.mark.parametrize("row_bytes", [3, 16, 50, 128, 520])
def test_fetch_rows_through_a_cache_of_hot_rows(row_bytes):
    rng = np.random.default_rng(row_bytes + 7)
    n, n_hot = 6000, 700
    table = rng.integers(0, 256, size=(n, row_bytes), dtype=np.uint8)
    hot_ids = rng.permutation(n)[:n_hot]
    hot = ~table[hot_ids]                       # differs from the table, so the source of a row shows
    slot_map = np.full(n, -1, dtype=np.int32)
    slot_map[hot_ids] = np.arange(n_hot, dtype=np.int32)
    index = np.concatenate([rng.integers(0, n, size=5000), hot_ids[:300]])
    got = host(capi.fetch_rows(dev(table), dev(index), dev(hot), dev(slot_map)))
    want = oc.fetch_rows(table, index, hot, slot_map)
    assert np.array_equal(got, want)
    cached = slot_map[index] >= 0
    assert cached.any() and (~cached).any()
    assert np.array_equal(got[cached], ~table[index[cached]]) and np.array_equal(got[~cached], table[index[~cached]])


@pytest.mark.parametrize("dtype,cols", [(np.float32, 100), (np.int16, 24), (np.int8, 50), (np.float64, 3)])
def test_fetch_rows_from_pinned_host_memory(dtype, cols):
    rng = np.random.default_rng(cols)
    n = 20000
    table_np = (rng.standard_normal((n, cols)) * 100).astype(dtype)
    table = torch.empty((n, cols), dtype=torch.from_numpy(table_np).dtype, pin_memory=True)
    table.copy_(torch.from_numpy(table_np))
    index = rng.integers(0, n, size=7777)
    got = host(capi.fetch_rows(table, dev(index)))
    assert got.dtype == table_np.dtype and np.array_equal(got, table_np[index])
    # hot rows on the device, the rest from the host table
    hot_ids = np.arange(0, n, 3)
    slot_map = np.full(n, -1, dtype=np.int32)
    slot_map[hot_ids] = np.arange(hot_ids.size, dtype=np.int32)
    got = host(capi.fetch_rows(table, dev(index), dev(table_np[hot_ids]), dev(slot_map)))
    assert np.array_equal(got, table_np[index])


def test_fetch_rows_edge_cases():
    table = dev(np.arange(40, dtype=np.uint8).reshape(8, 5))
    empty = capi.fetch_rows(table, torch.empty(0, dtype=torch.int64, device="cuda"))
    assert tuple(empty.shape) == (0, 5)
    # ids outside the table are clamped, as everywhere in the library
    got = host(capi.fetch_rows(table, dev(np.array([-3, 100, 7], dtype=np.int64))))
    assert np.array_equal(got, host(table)[[0, 7, 7]])
    # a slot beyond the hot table falls back to the table row
    slot_map = dev(np.array([0, 5, -1, -1, -1, -1, -1, -1], dtype=np.int32))
    hot = dev(np.full((2, 5), 255, dtype=np.uint8))
    got = host(capi.fetch_rows(table, dev(np.array([0, 1, 2], dtype=np.int32)), hot, slot_map))
    assert np.array_equal(got, np.concatenate([np.full((1, 5), 255, dtype=np.uint8), host(table)[[1, 2]]]))
    with pytest.raises(capi.F2CGTError):
        capi.fetch_rows(torch.empty((0, 5), dtype=torch.uint8, device="cuda"), dev(np.array([0])))


def test_fetch_rows_large_gather():
    # more rows than one launch wave of workgroups, 64-bit byte offsets (table above 4 GiB would
    # be too slow to build here; 2^31 bytes is crossed by the output offsets instead)
    rng = np.random.default_rng(3)
    n, row_bytes, m = 1 << 20, 24, 3_000_000
    table = torch.randint(0, 256, (n, row_bytes), dtype=torch.uint8, device="cuda")
    index = torch.randint(0, n, (m,), device="cuda")
    got = capi.fetch_rows(table, index)
    assert torch.equal(got, table[index])
    wide = torch.randint(0, 256, (3000, 1 << 20), dtype=torch.uint8, device="cuda")        # 3 GB of rows
    index = torch.tensor([2999, 0, 2100, 2999, 1], device="cuda")
    assert torch.equal(capi.fetch_rows(wide, index), wide[index])


def test_tensor_cache_serves_hot_rows_from_the_device_copy():
    from f2cgt_amd import pipeline
    rng = np.random.default_rng(5)
    n, cols = 5000, 50
    table_np = rng.integers(-128, 128, size=(n, cols), dtype=np.int8)
    cache = pipeline.TensorCache(torch.from_numpy(table_np))
    assert cache.data.is_pinned() and not cache.has_cache
    index = dev(rng.integers(0, n, size=4000))
    assert np.array_equal(host(cache[index]), table_np[host(index)])
    hotness = torch.from_numpy(rng.random(n).astype(np.float32))
    full, item = cache.compute_weight_size(hotness)
    assert full == n * cols and item == pytest.approx(cols * float(hotness[hotness > 0].mean()))
    # room for 1000 rows beside the slot array
    cache.create_cache(4 * n + 1000 * cols, hotness)
    assert cache.has_cache and cache.gpu_data.shape == (1000, cols) and cache.data.is_pinned()
    top = torch.sort(hotness, descending=True)[1][:1000].numpy()
    assert np.array_equal(np.sort(np.nonzero(host(cache.slot_map) >= 0)[0]), np.sort(top))
    assert np.array_equal(host(cache[index]), table_np[host(index)])
    # overwrite the host table: cached ids keep the value they were cached with
    cache.data.fill_(7)
    got = host(cache[index])
    is_hot = np.isin(host(index), top)
    assert np.array_equal(got[is_hot], table_np[host(index)[is_hot]]) and np.all(got[~is_hot] == 7)
    cache.clear_cache()
    assert np.all(host(cache[index]) == 7)
    # a capacity that holds everything moves the table to the device
    cache.create_cache(n * cols, hotness)
    assert cache.data.is_cuda and not cache.has_cache
    assert np.all(host(cache[index.int()]) == 7)
    # a capacity the slot array alone exceeds leaves the cache off
    small = pipeline.TensorCache(torch.from_numpy(table_np))
    small.create_cache(4 * n, hotness)
    assert not small.has_cache


def test_manager_with_host_resident_tables_matches_device_resident():
    from f2cgt_amd import pipeline
    rng = np.random.default_rng(9)
    n, d = 3000, 64
    x = torch.from_numpy(rng.standard_normal((n, d)).astype(np.float32))
    torch.manual_seed(3)
    table, cbs = pipeline.vq_compress(x, 256, 8, sample_index=torch.arange(n))
    meta = {"methods": ["vq"], "feat_dim": d, "configs": [(8, 256)], "codebooks": [cbs],
            "compression_data": table.cpu()}
    keys = dev(rng.permutation(n)[:1200])
    on_device = pipeline.CompressionManager(meta, fusion=True)
    on_host = pipeline.CompressionManager(meta, fusion=True, device_resident=False)
    assert on_device.data.data.is_cuda and on_host.data.data.is_pinned()
    on_host.data.create_cache(4 * n + 500 * table.shape[1], torch.from_numpy(rng.random(n).astype(np.float32)))
    assert on_host.data.has_cache
    a, b = on_device.get_all_data(keys), on_host.get_all_data(keys)
    assert torch.equal(a, b) and torch.equal(a.cpu(), table.cpu()[keys.cpu()])


@pytest.mark.parametrize("method", ["sq", "vq"])
def test_aggregation_by_global_id_equals_fetch_then_fused(method):
    import f2cgt_amd
    from f2cgt_amd import pipeline
    lib = f2cgt_amd.load()
    rng = np.random.default_rng(13)
    n, d = 4000, 64
    x = torch.from_numpy(rng.standard_normal((n, d)).astype(np.float32))
    torch.manual_seed(4)
    if method == "sq":
        table, cbs = pipeline.sq_compress(x, 4, 32, sample_index=torch.arange(n))
        configs = [(32, 4)]
    else:
        table, cbs = pipeline.vq_compress(x, 256, 8, sample_index=torch.arange(n))
        configs = [(8, 256)]
    sm = pipeline.CompressionManager({"methods": [method], "feat_dim": d, "configs": configs, "codebooks": [cbs],
                                      "compression_data": table}, fusion=True)
    input_nodes = dev(rng.permutation(n)[:900])
    deg = rng.integers(0, 12, size=300)
    indptr = np.zeros(301, dtype=np.int64)
    indptr[1:] = np.cumsum(deg)
    indices = rng.integers(0, 900, size=int(indptr[-1]))
    ip, ix = dev(indptr), dev(indices)
    rows = sm.get_all_data(input_nodes)
    if method == "vq":
        two_step = lib.vq_decompress_spmm_csr(rows, sm.codebooks[0], ip, ix, d)
    else:
        two_step = lib.sq_decompress_spmm_csr(rows, sm.codebooks[0], ip, ix, 4, 32, d)
    assert torch.equal(sm.aggregate_global(ip, ix, input_nodes), two_step)


def test_module_fetch_rows():
    import f2cgt_amd
    lib = f2cgt_amd.load()
    rng = np.random.default_rng(2)
    table = dev(rng.standard_normal((1000, 33)).astype(np.float32))
    index = dev(rng.integers(0, 1000, size=500).astype(np.int32))
    assert torch.equal(lib.fetch_rows(table, index), table[index.long()])
    hot = table[:10] + 1
    slot_map = torch.full((1000,), -1, dtype=torch.int32, device="cuda")
    slot_map[:10] = torch.arange(10, dtype=torch.int32, device="cuda")
    got = lib.fetch_rows(table=table, index=index, hot=hot, slot_map=slot_map)
    want = torch.where((index < 10)[:, None], table[index.long()] + 1, table[index.long()])
    assert torch.equal(got, want)
    with pytest.raises(RuntimeError):
        lib.fetch_rows(table.cpu(), index)                      # pageable host memory
    with pytest.raises(RuntimeError):
        lib.fetch_rows(table, index, hot=hot)                   # cache without its slot array
