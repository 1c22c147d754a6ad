"""The torch CPU flow used as the benchmark's cpu_baseline agrees with the numpy oracle."""
import numpy as np
import torch

import f2cgt_cpu_path as cp
import f2cgt_oracle as oc
from f2cgt_amd import synth


def _np(wl, key):
    return wl[key].numpy()


def test_cpu_path_matches_oracle_on_small_workloads():
    torch.set_num_threads(2)
    wl = synth.c2_sq4_affine(N=3000, R=500, chunk=1024)
    out, _, _ = cp.run(wl)
    want = oc.sq_affine_decompress_spmm_csr(_np(wl, "codes"), _np(wl, "params"), _np(wl, "indptr"),
                                            _np(wl, "indices"), 4, 100)
    assert np.allclose(out.numpy(), want, rtol=1e-5, atol=1e-5)
    wl = synth.c3_vq(N=4000, R=300)
    out, _, _ = cp.run(wl, rows=200)
    want = oc.vq_decompress_spmm_csr(_np(wl, "codes"), _np(wl, "codebooks"), _np(wl, "indptr")[:201],
                                     _np(wl, "indices")[:200 * 15], 128)
    assert np.allclose(out.numpy(), want, rtol=1e-5, atol=1e-5)
    wl = synth.c4_hybrid(N=4000, R=300)
    out, _, _ = cp.run(wl)
    want = oc.hybrid_decompress_spmm_csr(_np(wl, "row_map"), _np(wl, "sq_codes"), _np(wl, "sq_params"),
                                         _np(wl, "vq_codes"), _np(wl, "vq_codebooks"), _np(wl, "indptr"),
                                         _np(wl, "indices"), 128)
    assert np.allclose(out.numpy(), want, rtol=1e-5, atol=1e-5)
    wl = synth.c1_sq8_affine(N=2000, R=100)
    out, _, _ = cp.run(wl)
    want = oc.sq_affine_decompress_spmm_csr(_np(wl, "codes"), _np(wl, "params"), _np(wl, "indptr"),
                                            _np(wl, "indices"), 8, 128)
    assert np.allclose(out.numpy(), want, rtol=1e-5, atol=1e-5)
