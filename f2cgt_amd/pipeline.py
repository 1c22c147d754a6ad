"""Callers of the operator library, mirrored from the reference's Python with plain tensors in
place of DGL blocks, ShmTensor and torch.distributed (one process, one GPU):

  * the offline encode pipeline: `sq_metadata`, `sq_compress`, `vq_metadata`, `vq_compress`
    (examples/process_compress.py:16-68, 71-144, 147-292), `run` that writes the artefact files
    (`:295-388`) and `load_compress_data` that reads them back (examples/load_dataset.py:63-85);
  * `TensorCache` (examples/tensor_cache.py:36-110): a table of rows on the device or in pinned
    host memory, with an optional device-resident copy of its hottest rows, indexed by global id;
  * `CompressionManager` (examples/compress.py:8-106): keeps the code tables and codebooks,
    serves seed rows (first level) and neighbour rows (second level);
  * `MySAGEConv` (examples/conv.py:9-76): GraphSAGE mean layer whose neighbour aggregation is the
    fused decompress + mean operator.

Everything numerical happens in `F2CGTLib` (f2cgt_amd.load()); this module only moves tensors.
"""
from __future__ import annotations

import math

import numpy as np
import torch
from torch import nn

import f2cgt_amd


def _capi():
    return f2cgt_amd.load()


# ---- encode pipeline -----------------------------------------------------------------------------
def normalize(data):
    """Every row rescaled to the mean row norm: directions kept, lengths equalised
    (examples/process_compress.py:16-18; same operation order, divide then multiply)."""
    lengths = torch.linalg.vector_norm(data, ord=2, dim=1, keepdim=True)
    return (data / lengths) * lengths.mean()


def sampling(sample_size, num_items, hotness=None, generator=None):
    """Row sample for the codebook statistics (examples/process_compress.py:21-34); with a
    hotness vector the sample follows it, otherwise it is uniform without replacement."""
    if hotness is None:
        return torch.randperm(num_items, generator=generator)[:sample_size]
    p = (hotness.double() / hotness.double().sum()).cpu().numpy()
    p[-1] = 1.0 - p[:-1].sum()
    size = min(sample_size, num_items)
    return torch.from_numpy(np.random.choice(num_items, size, replace=False, p=p))


def sq_metadata(sample):
    """(fmin, fmax, emin, emax, mean) of one column slice from a sample of its rows:
    float64 percentiles of |x| floored at 1e-5 / 2e-5, log2 in float64, mean lifted by 0.1 when
    below 0.1 (examples/process_compress.py:45-68)."""
    floor = 1e-5
    magnitude = sample.float().abs().cpu()
    # one percentile and one log2 at a time, as the reference does: numpy returns the sample's own
    # precision for a scalar quantile (float64 for a list of them), and torch's scalar and vector
    # log2 do not agree to the last bit
    lo, hi = np.percentile(magnitude.numpy(), 0.5), np.percentile(magnitude.numpy(), 99.5)
    fmin, fmax = torch.tensor(max(lo, floor)), torch.tensor(max(hi, 2 * floor))
    level = magnitude.mean()
    level = level + 0.1 if level < 0.1 else level
    return fmin, fmax, torch.log2(fmin), torch.log2(fmax) + floor, level


def sq_compress(features, target_bits, column_slice, hotness=None, sample_index=None, batch_rows=1_000_000):
    """-> (storage, codebooks).  storage: int8 [N, ceil(D * bits / 8)] holding the packed bit
    patterns (bits <= 8) or int16 [N, D]; codebooks fp32 [ceil(D / column_slice), 5] on the GPU
    (examples/process_compress.py:71-144, single process)."""
    capi = _capi()
    num_items, feat_dim = features.shape
    if sample_index is None:
        sample_index = sampling(250_000, num_items, hotness)
    num_codebooks = (feat_dim + column_slice - 1) // column_slice
    codebooks = torch.zeros((num_codebooks, 5), dtype=torch.float32)
    for i in range(num_codebooks):
        lo, hi = i * column_slice, min((i + 1) * column_slice, feat_dim)
        vals = sq_metadata(features[sample_index.to(features.device), lo:hi])
        for j, v in enumerate(vals):
            codebooks[i, j] = v
    codebooks = codebooks.cuda()
    if target_bits <= 8:
        dtype, tdim = torch.int8, int(math.ceil(feat_dim / 8 * target_bits))
    elif target_bits <= 16:
        dtype, tdim = torch.int16, feat_dim
    else:
        raise NotImplementedError
    out = torch.empty((num_items, tdim), dtype=dtype, device="cuda")
    for start in range(0, num_items, batch_rows):
        end = min(start + batch_rows, num_items)
        data = features[start:end].cuda().to(torch.float32)
        # one pass; the reference calls sq_compress, casts and packs (process_compress.py:128-139)
        out[start:end].copy_(capi.sq_encode(data, codebooks, target_bits, column_slice))
    return out, codebooks


class KMeansTrainer:
    """Codebook trainer of the offline compressor (examples/my_kmeans.py:73-113, 150-184), on the
    device from start to finish: assignment by `kmeans_predict`, centre update and stopping rule by
    `kmeans_update`.

    As in the reference: `cosine` starts from random unit-circle pairs (cos / sin of uniform angles,
    :9-24), `euclidean` from distinct random non-zero rows (:27-31); a centre is the plain mean of its
    members whatever the metric and keeps its value when it has none (:128-147); the fit ends when
    (sum_c |centre shift|)^2 < tol, with tol growing by a factor 1.2 per iteration (:100-111).
    The rule is evaluated by the update kernel, which freezes the centres when it holds; the host
    reads the flag every `check_every` iterations, so the loop runs without a read-back per step.
    """

    def __init__(self, num_clusters, metric="cosine", tol=1e-4, mode="fast", max_iter=1000, check_every=8,
                 generator=None):
        if metric not in ("cosine", "euclidean"):
            raise ValueError("metric must be 'cosine' or 'euclidean'")
        if mode not in ("fast", "normal"):
            raise ValueError("mode must be 'fast' or 'normal'")
        self.num_clusters, self.metric, self.tol, self.mode = num_clusters, metric, tol, mode
        self.max_iter, self.check_every, self.generator = max_iter, check_every, generator
        self.centers, self.n_iter = None, 0

    def _initial_centers(self, data):
        n, width = self.num_clusters, data.shape[1]
        if self.metric == "cosine":
            half = width // 2
            if width % 2 == 0:
                angles = torch.rand((n, half), generator=self.generator) * (2 * math.pi)
                start = torch.cat([torch.cos(angles), torch.sin(angles)], dim=1)
            else:
                radii = torch.rand((n, 1), generator=self.generator)
                angles = torch.rand((n, half + 1), generator=self.generator) * (2 * math.pi)
                start = radii * torch.cat([torch.cos(angles[:, :half]), torch.sin(angles)], dim=1)
            return start.float().cuda()
        alive = torch.nonzero(torch.count_nonzero(data, dim=1)).flatten()
        if alive.numel() < n:
            raise ValueError("fewer non-zero rows than clusters")
        pick = torch.randperm(alive.numel(), generator=self.generator)[:n].to(alive.device)
        return data[alive[pick]].float().cuda()

    def fit(self, data):
        capi = _capi()
        data = data.float().cuda().contiguous()
        centers = self._initial_centers(data).contiguous()
        metric = "cosine" if self.metric == "cosine" else "l2"
        stop = torch.zeros((1,), dtype=torch.int32, device="cuda")
        tol, self.n_iter = float(self.tol), 0
        for it in range(self.max_iter):
            labels = capi.kmeans_predict(data, centers, metric)
            capi.kmeans_update(data, labels, centers, stop, 2, tol)
            tol *= 1.2
            self.n_iter += 1
            if it % self.check_every == self.check_every - 1 and int(stop.item()):
                break
        if int(stop.item()) == 2:
            # the centre shift is not a number (NaN or infinite input): the reference's trainer gives
            # up on such a fit (examples/my_kmeans.py:108-109); so does this one, loudly
            import warnings
            warnings.warn("KMeansTrainer.fit: the centre shift became NaN; no centres were produced")
            self.centers = None
            return
        self.centers = centers

    def get_centers(self):
        return self.centers

    def predict(self, data, normalize_weights=False):
        metric = "cosine" if self.metric == "cosine" else "l2"
        return _capi().kmeans_predict(data.float().cuda().contiguous(), self.centers, metric)


def vq_metadata(features, n_clusters, column_slice, hotness=None, sample_index=None, max_iter=1000):
    """Codebooks fp32 [ceil(D / column_slice), n_clusters, column_slice]: per slice, rows of a
    sample inside the rim quantile are dropped, k-means (cosine, tol 5e-2) runs on the rest and the
    centres are rescaled to their mean norm (examples/process_compress.py:147-182)."""
    capi = _capi()
    num_items, feat_dim = features.shape
    if sample_index is None:
        sample_index = sampling(150_000, num_items, hotness)
    num_slice = (feat_dim + column_slice - 1) // column_slice
    codebooks = torch.zeros((num_slice, n_clusters, column_slice), device="cuda", dtype=torch.float32)
    for i in range(num_slice):
        lo, hi = i * column_slice, min((i + 1) * column_slice, feat_dim)
        data = features[sample_index.to(features.device), lo:hi].to(torch.float32).cuda()
        distance = data.norm(dim=1, p=2)
        rim = torch.quantile(distance, min(1.0, 0.00625 * (data.shape[1] / 8)))
        data = data[torch.ge(distance, rim)].contiguous()
        km = KMeansTrainer(n_clusters, metric="cosine", tol=5e-2, max_iter=max_iter)
        km.fit(data)
        centers = normalize(km.get_centers())
        codebooks[i, :, :hi - lo] = centers
    if torch.isnan(codebooks).any():
        raise ValueError("codebooks has nan")
    return codebooks


def vq_compress(features, n_clusters, column_slice, hotness=None, codebooks=None, sample_index=None,
                batch_rows=1_000_000):
    """-> (codes, codebooks).  codes: uint8 (K <= 256) or int16 [N, n_slices], one nearest
    (cosine) centre per column slice (examples/process_compress.py:185-292, single process)."""
    capi = _capi()
    num_items, feat_dim = features.shape
    if codebooks is None:
        codebooks = vq_metadata(features, n_clusters, column_slice, hotness, sample_index)
    num_slice = codebooks.shape[0]
    if n_clusters <= 256:
        dtype = torch.uint8
    elif n_clusters <= 32767:
        dtype = torch.int16
    else:
        raise NotImplementedError("more than 32767 centres do not fit the int16 code type")
    out = torch.empty((num_items, num_slice), dtype=dtype, device="cuda")
    predictors = [capi.KMeans(codebooks[i].contiguous(), "cosine") for i in range(num_slice)]
    for start in range(0, num_items, batch_rows):
        end = min(start + batch_rows, num_items)
        for i in range(num_slice):
            lo, hi = i * column_slice, min((i + 1) * column_slice, feat_dim)
            if hi <= lo:
                continue
            data = torch.zeros((end - start, column_slice), device="cuda", dtype=torch.float32)
            data[:, :hi - lo] = features[start:end, lo:hi].to(torch.float32)
            labels = predictors[i].predict(data, normalize_weights=False)
            out[start:end, i] = labels.to(dtype)
    return out, codebooks


def run(root, features, seeds=None, hotness=None, target_compression_ratio=32, n_clusters=256):
    """Compresses a feature table and writes the artefacts the training scripts load
    (examples/process_compress.py:295-388, single process, column slices as for one rank):

      * `compression_meta.pt`: dict with `methods` (['sq'] / ['vq'], preceded by 'sq' when seed
        rows get their own table), `codebooks` (CPU tensors, one per level), `configs`
        ((column_slice, target_bits) per level, target_bits -1 for VQ), `feat_dim`, `data`
        (name -> (dtype, shape) of each code table) and `seeds` (ids of the seed rows);
      * `compression_data.pt`: the code table of every row;
      * `seeds_compression_data.pt`: the code table of the seed rows (SQ at one eighth of the
        element width in bits, i.e. 4-bit codes for fp32 features).

    A ratio up to the element width in bits selects SQ with `width / ratio` bits per value; a
    larger one selects VQ with `ratio / element_size` columns per code byte (twice that for
    more than 256 centres).  Returns the meta dict."""
    import os
    feat_dim = features.shape[1]
    width_bits = features.element_size() * 8
    methods, configs, codebook_list, data, meta = [], [], [], {}, {}
    slice_of_row = (feat_dim + 7) // 8 * 8
    if seeds is not None:
        seed_bits = width_bits // 8
        seed_rows = features[seeds.to(features.device)]
        seed_codes, seed_cbs = sq_compress(seed_rows, seed_bits, slice_of_row, None)
        methods.append("sq")
        configs.append((slice_of_row, seed_bits))
        codebook_list.append(seed_cbs.cpu())
        data["seeds_compression_data"] = (seed_codes.dtype, seed_codes.shape)
        meta["seeds"] = seeds.cpu()
        torch.save(seed_codes.cpu(), os.path.join(root, "seeds_compression_data.pt"))
        del seed_codes
    if target_compression_ratio <= width_bits:
        target_bits = int(width_bits / target_compression_ratio)
        codes, cbs = sq_compress(features, target_bits, slice_of_row, hotness)
        methods.append("sq")
        configs.append((slice_of_row, target_bits))
    else:
        column_slice = target_compression_ratio // features.element_size()
        if n_clusters > 256:
            column_slice *= 2
        codes, cbs = vq_compress(features, n_clusters, column_slice, hotness)
        methods.append("vq")
        configs.append((column_slice, -1))
    codebook_list.append(cbs.cpu())
    data["compression_data"] = (codes.dtype, codes.shape)
    meta.update(methods=methods, codebooks=codebook_list, configs=configs, feat_dim=feat_dim, data=data)
    torch.save(meta, os.path.join(root, "compression_meta.pt"))
    torch.save(codes.cpu(), os.path.join(root, "compression_data.pt"))
    return meta


def load_compress_data(root):
    """The dict `CompressionManager` takes, read back from the files `run` wrote: the meta dict
    with every code table named in `data` added under its name
    (examples/load_dataset.py:63-85 without the shared-memory staging)."""
    import os
    meta = torch.load(os.path.join(root, "compression_meta.pt"), weights_only=True)
    for name, (dtype, shape) in meta["data"].items():
        table = torch.load(os.path.join(root, name + ".pt"), weights_only=True)
        if table.dtype != dtype or tuple(table.shape) != tuple(shape):
            raise ValueError("%s.pt does not match its entry in compression_meta.pt" % name)
        meta[name] = table
    return meta


# ---- runtime callers -------------------------------------------------------------------------------
class TensorCache:
    """examples/tensor_cache.py:36-110 without ShmTensor.

    `data` is a 2-D table of rows (code rows or plain features).  A host table is copied once
    into pinned memory that the device can address (the reference pins the shared-memory table in
    place; registering existing memory is not available here), and `cache[index]` reads its rows
    over the host link; `create_cache(capacity, hotness)` moves the whole table to the device
    when it fits in `capacity` bytes and otherwise keeps a device copy of the hottest rows plus a
    dense int32 array id -> cache slot (-1 = not cached) where the reference keeps a GPU hash
    map.  The array costs 4 bytes per table row and is charged to the capacity.
    `index` is a device tensor of int32/int64 ids; the result is a new device tensor."""

    def __init__(self, data):
        if data.dim() != 2:
            raise ValueError("TensorCache holds a 2-D table of rows")
        if data.device.type == "cpu":
            pinned = torch.empty(data.shape, dtype=data.dtype, pin_memory=True)
            pinned.copy_(data)
            data = pinned
        self.data = data.contiguous()
        self.gpu_data = None
        self.slot_map = None
        self.has_cache = False

    def __getitem__(self, index):
        capi = _capi()
        if index.dtype not in (torch.int32, torch.int64):
            index = index.long()
        if self.has_cache:
            return capi.fetch_rows(self.data, index, self.gpu_data, self.slot_map)
        return capi.fetch_rows(self.data, index)

    def create_cache(self, cache_capacity, hotness):
        if cache_capacity <= 0:
            return
        full_size = self.data.numel() * self.data.element_size()
        if full_size <= cache_capacity:
            self.data = self.data.cuda()
            return
        row_bytes = self.data.shape[1] * self.data.element_size()
        cache_num = int((cache_capacity - 4 * self.data.shape[0]) // row_bytes)
        if cache_num <= 0:
            return
        _, candidates = torch.sort(hotness, descending=True)
        candidates = candidates[:cache_num]
        self.gpu_data = self.data[candidates.to(self.data.device)].cuda()
        self.slot_map = torch.full((self.data.shape[0],), -1, dtype=torch.int32, device="cuda")
        self.slot_map[candidates.cuda().long()] = torch.arange(candidates.numel(), dtype=torch.int32, device="cuda")
        self.has_cache = True

    def clear_cache(self):
        self.has_cache = False
        self.gpu_data = None
        self.slot_map = None

    def compute_weight_size(self, hotness):
        """(bytes of the whole table, bytes of a row weighted by the mean hotness of the rows that are
        ever touched): the two inputs of the reference's cache-split cost model
        (examples/tensor_cache.py:102-106)."""
        row_bytes = self.data.shape[1] * self.data.element_size()
        touched = hotness[hotness > 0]
        return self.data.shape[0] * row_bytes, row_bytes * float(touched.float().mean())


class CompressionManager:
    """examples/compress.py:8-106 on plain tensors.

    `compress_data` keys (the layout of the reference's `compression_meta.pt` + data tensors):
    `methods` (list of 'sq' / 'vq', one entry, or two for seeds + everything), `feat_dim`,
    `configs` (per level (column_slice, target_bits)), `codebooks` (per level), `compression_data`
    (code table of the last level, [N, src_dim]), and for two levels `seeds_compression_data`
    (code table of the seed rows) with `seeds` (their global ids).

    The code tables sit behind `TensorCache`.  `device_resident=True` (the default: the largest
    table of the benchmark configurations is 5.76 GB against 288 GB of device memory) moves them
    to the device at construction, the reference's whole-table cache
    (examples/tensor_cache.py:66-70); `False` leaves host tables in pinned host memory until
    `manager.data.create_cache(capacity, hotness)` is called, as the reference does.
    """

    def __init__(self, compress_data, fusion=False, device_resident=True):
        self.meta = compress_data
        self.methods = compress_data["methods"]
        self.feat_dim = compress_data["feat_dim"]
        self.configs = compress_data["configs"]
        self.codebooks = [c.cuda() for c in compress_data["codebooks"]]
        place = (lambda t: t.cuda()) if device_resident else (lambda t: t)
        self.data = TensorCache(place(compress_data["compression_data"]))
        self.seeds_data = None
        self.is_two_level = len(self.methods) >= 2
        self.is_fusion = fusion
        # the seed rows are fetched and decoded on a stream of their own while the caller goes on to
        # sample and gather the block (examples/compress.py:36-53); default priority
        self.seeds_task_stream = torch.cuda.Stream()
        self.seeds_task_event = torch.cuda.Event()
        self.check_seed_keys = True   # a host round trip per call; the reference's hash map query has no such check
        if self.is_two_level:
            self.seeds_data = TensorCache(place(compress_data["seeds_compression_data"]))
            keys = compress_data["seeds"].long().cuda()
            # global id -> row of the seed table (the reference keeps a GPU hash map)
            self.seed_slot = torch.full((self.data.data.shape[0],), -1, dtype=torch.int32, device="cuda")
            self.seed_slot[keys] = torch.arange(keys.numel(), dtype=torch.int32, device="cuda")

    def _decompress(self, level, data):
        capi = _capi()
        if self.methods[level] == "vq":
            return capi.vq_decompress(data, self.codebooks[level], self.feat_dim)
        return capi.sq_decompress(data, self.codebooks[level], self.configs[level][1], self.configs[level][0],
                                  self.feat_dim)

    def get_seeds_data(self, seeds_key):
        """Decoded first-level rows of `seeds_key`, produced on `seeds_task_stream`; the result may be
        used on another stream only after `seeds_task_event` (reorganize_seeds_data waits for it)."""
        if not self.is_two_level:
            return None
        side = self.seeds_task_stream
        side.wait_stream(torch.cuda.current_stream())      # seeds_key may still be in the making
        with torch.cuda.stream(side):
            # the caller may drop seeds_key as soon as this returns: tie its memory to the side stream
            seeds_key.record_stream(side)
            slots = self.seed_slot[seeds_key.long()].long()
            if self.check_seed_keys and bool((slots < 0).any()):
                raise KeyError("a requested id is not a seed row")
            seeds_feature = self._decompress(0, self.seeds_data[slots])
            self.seeds_task_event.record(side)
        return seeds_feature

    def get_all_data(self, keys):
        data = self.data[keys]
        if self.is_fusion:
            return data
        return self._decompress(1 if self.is_two_level else 0, data)

    def aggregate_global(self, indptr, indices, input_nodes):
        """Mean aggregation of a sampled block straight from the device-resident code table:
        `indices` are positions in `input_nodes` (the block's source ids), which are composed
        into global ids so that the fused operator reads the table rows itself and the gathered
        copy of `get_all_data` is never written.  Same result as
        `fused_op(get_all_data(input_nodes), ..., indptr, indices)`."""
        if not self.data.data.is_cuda:
            raise RuntimeError("aggregate_global needs the code table on the device")
        capi = _capi()
        level = 1 if self.is_two_level else 0
        global_ids = input_nodes.to(indices.dtype)[indices.long()]
        if self.methods[level] == "vq":
            return capi.vq_decompress_spmm_csr(self.data.data, self.codebooks[level], indptr, global_ids,
                                               self.feat_dim)
        return capi.sq_decompress_spmm_csr(self.data.data, self.codebooks[level], indptr, global_ids,
                                           self.configs[level][1], self.configs[level][0], self.feat_dim)

    def reorganize_seeds_data(self, seeds_feature, all_feature, num_dst):
        if seeds_feature is not None:
            # the consumer joins the seed stream here (examples/compress.py:74-75)
            current = torch.cuda.current_stream()
            current.wait_event(self.seeds_task_event)
            seeds_feature.record_stream(current)
        if not self.is_fusion:
            if seeds_feature is None:
                return None
            num_seeds = seeds_feature.shape[0]
            return torch.cat([seeds_feature, all_feature[num_seeds:num_dst]], dim=0)
        if self.is_two_level:
            num_seeds = seeds_feature.shape[0]
            part = all_feature[num_seeds:num_dst]
        else:
            part = all_feature[:num_dst]
        part_feature = self._decompress(1 if self.is_two_level else 0, part.contiguous())
        if self.is_two_level:
            return torch.cat([seeds_feature, part_feature], dim=0)
        return part_feature


class MySAGEConv(nn.Module):
    """examples/conv.py:9-76.  `forward(csc, feat)`: `csc = (indptr, indices)` of the block
    (destination rows x source rows), `feat = (h_self, h_neigh)`; with a fusing manager `h_neigh`
    is the compressed code rows of the source nodes and the aggregation decodes them on the fly."""

    def __init__(self, in_feats, out_feats, aggregator_type, compression_manager, bias=True, norm=None,
                 activation=None):
        super().__init__()
        if aggregator_type != "mean":
            raise ValueError("the fused layer aggregates by mean only (got %r)" % (aggregator_type,))
        src_width, dst_width = (in_feats, in_feats) if isinstance(in_feats, int) else tuple(in_feats)
        self.sm = compression_manager
        self.activation, self.norm = activation, norm
        # the reference's attribute names (examples/conv.py:29-31): checkpoints of either load into the other
        self.fc_neigh = nn.Linear(src_width, out_feats, bias=False)
        self.fc_self = nn.Linear(dst_width, out_feats, bias=bias)
        self.reset_parameters()

    def reset_parameters(self):
        """Glorot-uniform weights scaled for a ReLU that follows (examples/conv.py:38-42)."""
        for layer in (self.fc_self, self.fc_neigh):
            nn.init.xavier_uniform_(layer.weight, gain=nn.init.calculate_gain("relu"))

    def forward(self, csc, feat):
        capi = _capi()
        indptr, indices = csc
        h_self, h_neigh = feat
        num_dst = indptr.numel() - 1
        if h_self is None:
            h_self = h_neigh[:num_dst]
        sm = self.sm
        if sm is None or not sm.is_fusion:
            h_neigh = capi.spmm_csr(h_neigh, indptr, indices)
        else:
            level = 1 if sm.is_two_level else 0
            if sm.methods[level] == "vq":
                h_neigh = capi.vq_decompress_spmm_csr(h_neigh, sm.codebooks[level], indptr, indices, sm.feat_dim)
            else:
                h_neigh = capi.sq_decompress_spmm_csr(h_neigh, sm.codebooks[level], indptr, indices,
                                                      sm.configs[level][1], sm.configs[level][0], sm.feat_dim)
        rst = self.fc_self(h_self) + self.fc_neigh(h_neigh)
        if self.activation is not None:
            rst = self.activation(rst)
        if self.norm is not None:
            rst = self.norm(rst)
        return rst
