"""Host-side pieces of f2cgt_amd/pipeline.py that need no GPU."""
import numpy as np
import torch

import f2cgt_oracle as oc
from f2cgt_amd import pipeline


def test_sq_metadata_is_the_reference_codebook_statement():
    rng = np.random.default_rng(0)
    for scale, shift in ((1.0, 0.0), (1e-4, 0.0), (3.0, 10.0)):
        x = (rng.standard_normal((5000, 7)) * scale + shift).astype(np.float32)
        got = np.array([float(v) for v in pipeline.sq_metadata(torch.from_numpy(x))], dtype=np.float32)
        want = oc.sq_codebook(x)
        assert np.array_equal(got[:4], want[:4])
        assert np.isclose(got[4], want[4], rtol=1e-6)


def test_normalize_rescales_rows_to_the_mean_norm():
    x = torch.tensor([[3.0, 4.0], [0.0, 1.0], [6.0, 8.0]])
    y = pipeline.normalize(x)
    mean_norm = (5.0 + 1.0 + 10.0) / 3.0
    assert torch.allclose(y.norm(dim=1), torch.full((3,), mean_norm))
    assert torch.allclose(y[0] / y[0].norm(), x[0] / x[0].norm())


def test_sampling_is_a_permutation_prefix_or_follows_hotness():
    g = torch.Generator().manual_seed(3)
    s = pipeline.sampling(10, 100, generator=g)
    assert s.numel() == 10 and s.unique().numel() == 10 and int(s.max()) < 100
    np.random.seed(0)
    hot = torch.zeros(50)
    hot[:5] = 1.0
    s = pipeline.sampling(5, 50, hotness=hot)
    assert sorted(s.tolist()) == [0, 1, 2, 3, 4]


def test_layer_rejects_other_aggregators():
    import pytest
    with pytest.raises(ValueError):
        pipeline.MySAGEConv(8, 4, "pool", None)
