"""ctypes binding of the C ABI in include/f2cgt.h (libf2cgt_hip.so).

This is the binding a non-pybind caller would write: raw device pointers, sizes and a
hipStream_t.  The helpers at the bottom accept torch tensors only to extract
`data_ptr()` and torch's current stream; they allocate the output with torch and call
the C entry point.  No computation happens on the Python side and there is no fallback.
"""
from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_int, c_int64, c_void_p

from . import capi_path

DT_U8, DT_I8, DT_I16, DT_I32, DT_I64, DT_F16, DT_F32, DT_F64 = range(8)
METRIC_L2, METRIC_COSINE = 0, 1

P, I, L = c_void_p, c_int, c_int64

SIGNATURES = {
    "f2cgt_version": ([], c_int),
    "f2cgt_last_error": ([], c_char_p),
    "f2cgt_num_cus": ([], c_int),
    "f2cgt_set_plan_only": ([I], c_int),
    "f2cgt_set_store_mode": ([I], c_int),
    "f2cgt_last_plan": ([P], c_int),
    "f2cgt_packbits": ([P, P, L, L, I, P], c_int),
    "f2cgt_unpackbits": ([P, P, L, L, L, I, P], c_int),
    "f2cgt_sq_compress": ([P, P, P, L, L, L, I, L, P], c_int),
    "f2cgt_sq_encode": ([P, P, P, L, L, L, I, L, P], c_int),
    "f2cgt_sq_decompress": ([P, I, P, P, L, L, L, L, I, L, P], c_int),
    "f2cgt_sq_affine_decompress": ([P, P, P, L, L, L, L, I, P], c_int),
    "f2cgt_vq_decompress": ([P, I, P, I, P, L, L, L, L, L, P], c_int),
    "f2cgt_spmm_csr": ([P, I, P, P, P, I, L, L, L, L, P], c_int),
    "f2cgt_vq_decompress_spmm_csr": ([P, I, P, P, P, I, P, L, L, L, L, L, L, L, P], c_int),
    "f2cgt_sq_decompress_spmm_csr": ([P, I, P, P, P, I, P, L, L, L, L, L, L, I, L, P], c_int),
    "f2cgt_sq_affine_decompress_spmm_csr": ([P, P, L, P, P, I, P, L, L, L, L, L, I, P], c_int),
    "f2cgt_hybrid_decompress_spmm_csr":
        ([P, P, P, L, P, P, P, P, I, P, L, L, L, L, L, L, L, L, L, P], c_int),
    "f2cgt_fetch_rows": ([P, P, P, P, I, P, L, L, L, L, P], c_int),
    "f2cgt_pairwise_distance": ([P, P, P, L, L, L, I, P], c_int),
    "f2cgt_kmeans_predict": ([P, P, P, P, L, L, L, I, P], c_int),
    "f2cgt_kmeans_update_workspace_bytes": ([L, L], c_int64),
    "f2cgt_kmeans_update": ([P, P, P, P, P, P, I, ctypes.c_float, P, L, L, L, L, P], c_int),
    "f2cgt_kmeans_update_static": ([P, P, P, P, P, P, I, ctypes.c_float, L, L, L, P], c_int),
}



class Plan(ctypes.Structure):
    """f2cgt_plan of include/f2cgt.h."""
    _fields_ = [("kernel", ctypes.c_char * 48), ("grid", c_int64), ("block", ctypes.c_int32),
                ("lds_bytes", c_int64), ("rows_per_block", ctypes.c_int32), ("aux", ctypes.c_int32 * 4)]


_lib = None


def lib():
    """The loaded libf2cgt_hip.so with argument types declared."""
    global _lib
    if _lib is None:
        import torch  # noqa: F401  (loads the HIP runtime the library links against)
        handle = ctypes.CDLL(capi_path())
        for name, (argtypes, restype) in SIGNATURES.items():
            fn = getattr(handle, name)  # AttributeError if the symbol is not exported
            fn.argtypes = argtypes
            fn.restype = restype
        _lib = handle
    return _lib


def dry_run(entry, *args):
    """Calls the fused entry point `entry` (a name in SIGNATURES) in plan-only mode: nothing is
    launched and no pointer is read.  Returns (return code, Plan or None)."""
    handle = lib()
    was = handle.f2cgt_set_plan_only(1)
    try:
        rc = getattr(handle, entry)(*args)
        plan = Plan()
        got = handle.f2cgt_last_plan(ctypes.byref(plan))
    finally:
        handle.f2cgt_set_plan_only(was)
    return rc, (plan if rc == 0 and got == 0 else None)


class F2CGTError(RuntimeError):
    pass


STORE_AUTO, STORE_STREAM, STORE_CACHED = 0, 1, 2


def set_store_mode(mode):
    """Output store policy of the row-block SQ aggregation kernels (f2cgt_set_store_mode): returns the
    previous mode."""
    was = lib().f2cgt_set_store_mode(int(mode))
    if was < 0:
        raise F2CGTError("set_store_mode failed (%d): %s" % (was, lib().f2cgt_last_error().decode()))
    return was


def _check(rc, name):
    if rc != 0:
        raise F2CGTError("%s failed (%d): %s" % (name, rc, lib().f2cgt_last_error().decode()))


def _tag(t):
    import torch
    return {torch.uint8: DT_U8, torch.int8: DT_I8, torch.int16: DT_I16, torch.int32: DT_I32,
            torch.int64: DT_I64, torch.float16: DT_F16, torch.float32: DT_F32,
            torch.float64: DT_F64}[t.dtype]


def _stream():
    import torch
    return torch.cuda.current_stream().cuda_stream


def _ptr(t):
    return None if t is None else t.data_ptr()


# ---- tensor-level helpers (tests, benchmark) ---------------------------------------------
def packbits(unpack, bits):
    import torch
    per = 8 // bits
    out = torch.empty((unpack.shape[0], (unpack.shape[1] + per - 1) // per), dtype=torch.uint8,
                      device=unpack.device)
    _check(lib().f2cgt_packbits(_ptr(unpack), _ptr(out), unpack.shape[0], unpack.shape[1], bits,
                                _stream()), "packbits")
    return out


def unpackbits(pack, bits, unpack_dim):
    import torch
    out = torch.empty((pack.shape[0], unpack_dim), dtype=torch.uint8, device=pack.device)
    _check(lib().f2cgt_unpackbits(_ptr(pack), _ptr(out), pack.shape[0], pack.shape[1], unpack_dim,
                                  bits, _stream()), "unpackbits")
    return out


def sq_compress(src, codebooks, bits, column_slice):
    import torch
    out = torch.empty_like(src)
    _check(lib().f2cgt_sq_compress(_ptr(src), _ptr(out), _ptr(codebooks), src.shape[0], src.shape[1],
                                   codebooks.shape[0], bits, column_slice, _stream()), "sq_compress")
    return out


def sq_encode(src, codebooks, bits, column_slice):
    import torch
    rows, d = src.shape
    if bits < 8:
        out = torch.empty((rows, (d * bits + 7) // 8), dtype=torch.uint8, device=src.device)
    else:
        out = torch.empty((rows, d), dtype=torch.int8 if bits == 8 else torch.int16, device=src.device)
    _check(lib().f2cgt_sq_encode(_ptr(src), _ptr(out), _ptr(codebooks), rows, d, codebooks.shape[0], bits,
                                 column_slice, _stream()), "sq_encode")
    return out


def sq_decompress(codes, codebooks, bits, column_slice, feat_dim):
    import torch
    out = torch.empty((codes.shape[0], feat_dim), dtype=torch.float32, device=codes.device)
    _check(lib().f2cgt_sq_decompress(_ptr(codes), _tag(codes), _ptr(out), _ptr(codebooks),
                                     codes.shape[0], codes.shape[1], feat_dim, codebooks.shape[0], bits,
                                     column_slice, _stream()), "sq_decompress")
    return out


def sq_affine_decompress(codes, params, bits, feat_dim):
    import torch
    out = torch.empty((codes.shape[0], feat_dim), dtype=torch.float32, device=codes.device)
    _check(lib().f2cgt_sq_affine_decompress(_ptr(codes), _ptr(out), _ptr(params), params.shape[1],
                                            codes.shape[0], codes.shape[1], feat_dim, bits, _stream()),
           "sq_affine_decompress")
    return out


def vq_decompress(codes, codebooks, feat_dim):
    import torch
    out = torch.empty((codes.shape[0], feat_dim), dtype=torch.float32, device=codes.device)
    _check(lib().f2cgt_vq_decompress(_ptr(codes), _tag(codes), _ptr(codebooks), _tag(codebooks),
                                     _ptr(out), codes.shape[0], feat_dim, codebooks.shape[0],
                                     codebooks.shape[1], codebooks.shape[2], _stream()), "vq_decompress")
    return out


def spmm_csr(feat, indptr, indices, out=None):
    import torch
    rows = indptr.numel() - 1
    if out is None:
        out = torch.empty((rows, feat.shape[1]), dtype=feat.dtype, device=feat.device)
    _check(lib().f2cgt_spmm_csr(_ptr(feat), _tag(feat), _ptr(out), _ptr(indptr), _ptr(indices),
                                _tag(indptr), rows, indices.numel(), feat.shape[0], feat.shape[1],
                                _stream()), "spmm_csr")
    return out


def vq_decompress_spmm_csr(codes, codebooks, indptr, indices, feat_dim, out=None):
    import torch
    rows = indptr.numel() - 1
    if out is None:
        out = torch.empty((rows, feat_dim), dtype=torch.float32, device=codes.device)
    _check(lib().f2cgt_vq_decompress_spmm_csr(
        _ptr(codes), _tag(codes), _ptr(codebooks), _ptr(indptr), _ptr(indices), _tag(indptr), _ptr(out),
        rows, indices.numel(), codes.shape[0], feat_dim, codebooks.shape[0], codebooks.shape[1],
        codebooks.shape[2], _stream()), "vq_decompress_spmm_csr")
    return out


def sq_decompress_spmm_csr(codes, codebooks, indptr, indices, bits, column_slice, feat_dim, out=None):
    import torch
    rows = indptr.numel() - 1
    if out is None:
        out = torch.empty((rows, feat_dim), dtype=torch.float32, device=codes.device)
    _check(lib().f2cgt_sq_decompress_spmm_csr(
        _ptr(codes), _tag(codes), _ptr(codebooks), _ptr(indptr), _ptr(indices), _tag(indptr), _ptr(out),
        rows, indices.numel(), codes.shape[0], codes.shape[1], feat_dim, codebooks.shape[0], bits,
        column_slice, _stream()), "sq_decompress_spmm_csr")
    return out


def sq_affine_decompress_spmm_csr(codes, params, indptr, indices, bits, feat_dim, out=None):
    import torch
    rows = indptr.numel() - 1
    if out is None:
        out = torch.empty((rows, feat_dim), dtype=torch.float32, device=codes.device)
    _check(lib().f2cgt_sq_affine_decompress_spmm_csr(
        _ptr(codes), _ptr(params), params.shape[1], _ptr(indptr), _ptr(indices), _tag(indptr), _ptr(out),
        rows, indices.numel(), codes.shape[0], codes.shape[1], feat_dim, bits, _stream()),
        "sq_affine_decompress_spmm_csr")
    return out


def hybrid_decompress_spmm_csr(row_map, sq_codes, sq_params, vq_codes, vq_codebooks, indptr, indices,
                               feat_dim, out=None):
    import torch
    rows = indptr.numel() - 1
    if out is None:
        out = torch.empty((rows, feat_dim), dtype=torch.float32, device=row_map.device)
    _check(lib().f2cgt_hybrid_decompress_spmm_csr(
        _ptr(row_map), _ptr(sq_codes), _ptr(sq_params), sq_params.shape[1], _ptr(vq_codes),
        _ptr(vq_codebooks), _ptr(indptr), _ptr(indices), _tag(indptr), _ptr(out), rows, indices.numel(),
        row_map.numel(), sq_codes.shape[0], vq_codes.shape[0], feat_dim, vq_codebooks.shape[0],
        vq_codebooks.shape[1], vq_codebooks.shape[2], _stream()), "hybrid_decompress_spmm_csr")
    return out


def fetch_rows(table, index, hot=None, slot_map=None, out=None):
    """out[i] = hot[slot_map[index[i]]] where that slot is >= 0, else table[index[i]].  `table` is
    any contiguous 2-D tensor on the device or in pinned host memory; rows are moved as bytes."""
    import torch
    row_bytes = table.shape[1] * table.element_size()
    if out is None:
        out = torch.empty((index.numel(), table.shape[1]), dtype=table.dtype, device=index.device)
    _check(lib().f2cgt_fetch_rows(_ptr(table), _ptr(hot), _ptr(slot_map), _ptr(index), _tag(index), _ptr(out),
                                  index.numel(), row_bytes, table.shape[0],
                                  0 if hot is None else hot.shape[0], _stream()), "fetch_rows")
    return out


def pairwise_distance(x, y, metric):
    import torch
    out = torch.empty((x.shape[0], y.shape[0]), dtype=torch.float32, device=x.device)
    _check(lib().f2cgt_pairwise_distance(_ptr(x), _ptr(y), _ptr(out), x.shape[0], y.shape[0], x.shape[1],
                                         METRIC_COSINE if metric == "cosine" else METRIC_L2, _stream()),
           "pairwise_distance")
    return out


def kmeans_predict(x, centers, metric, u8=False, out=None):
    import torch
    if out is None:
        out = torch.empty((x.shape[0],), dtype=torch.uint8 if u8 else torch.int64, device=x.device)
    _check(lib().f2cgt_kmeans_predict(_ptr(x), _ptr(centers), None if u8 else _ptr(out),
                                      _ptr(out) if u8 else None, x.shape[0], centers.shape[0], x.shape[1],
                                      METRIC_COSINE if metric == "cosine" else METRIC_L2, _stream()),
           "kmeans_predict")
    return out


def kmeans_update(x, labels, centers, stop=None, rule=0, tol=0.0, workspace=None, shift=None):
    """One centre update in place (f2cgt_kmeans_update); -> shift tensor [2] = (sum |dc|, sum |dc|^2)."""
    import torch
    n, k = centers.shape
    need = lib().f2cgt_kmeans_update_workspace_bytes(n, k)
    if workspace is None:
        workspace = torch.empty((need,), dtype=torch.uint8, device=x.device)
    if shift is None:
        shift = torch.empty((2,), dtype=torch.float32, device=x.device)
    u8 = labels.dtype == torch.uint8
    _check(lib().f2cgt_kmeans_update(_ptr(x), None if u8 else _ptr(labels), _ptr(labels) if u8 else None,
                                     _ptr(centers), _ptr(shift), _ptr(stop), rule, tol, _ptr(workspace),
                                     workspace.numel(), x.shape[0], n, k, _stream()), "kmeans_update")
    return shift
