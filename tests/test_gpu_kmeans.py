"""Codebook training on the GPU: the Lloyd update step against the oracle, the stopping rules that
the update kernel evaluates itself, and fit() checked as a fit (fixed point, inertia, recovered
clusters) through the module's KMeans class and the trainer of the encode pipeline."""
import warnings

import numpy as np
import pytest
import torch

import f2cgt_oracle as oc
import f2cgt_amd
from f2cgt_amd import capi, pipeline

pytestmark = pytest.mark.gpu
RTOL = 1e-5


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def blobs(rng, per, k, spread=8.0):
    dirs = rng.standard_normal((k, k)).astype(np.float32)
    dirs /= np.linalg.norm(dirs, axis=1, keepdims=True)
    pts = np.concatenate([rng.standard_normal((per, k)).astype(np.float32) * 0.3 + spread * d for d in dirs])
    return pts, np.repeat(np.arange(k), per), dirs * spread


@pytest.mark.parametrize("m,n,k,u8", [(5000, 11, 7, False), (150_000, 256, 32, True), (20_000, 256, 64, False),
                                      (3000, 300, 40, False), (1, 1, 1, False), (70_000, 1024, 96, False)])
def test_update_step_vs_oracle(m, n, k, u8):
    print("case kmeans_update m=%d n=%d k=%d u8=%s" % (m, n, k, u8), flush=True)
    rng = np.random.default_rng(m + n + k)
    x = rng.standard_normal((m, k)).astype(np.float32)
    centers = rng.standard_normal((n, k)).astype(np.float32)
    labels = rng.integers(0, max(1, n - 2), size=m)                     # the last two clusters stay empty
    want, s_abs, s_sq = oc.kmeans_update(x, labels, centers)
    c = dev(centers)
    lab = dev(labels.astype(np.uint8)) if u8 else dev(labels.astype(np.int64))
    shift = capi.kmeans_update(dev(x), lab, c)
    torch.cuda.synchronize()
    got = c.cpu().numpy()
    scale = np.abs(x).max()
    assert np.allclose(got, want, rtol=RTOL, atol=RTOL * scale)
    if n > 2:
        assert np.array_equal(got[n - 2:], centers[n - 2:])                 # untouched, bit for bit
    sh = shift.cpu().numpy()
    assert np.isclose(sh[0], s_abs, rtol=1e-4) and np.isclose(sh[1], s_sq, rtol=1e-4)


def test_update_step_stop_flag_and_rules():
    rng = np.random.default_rng(5)
    x = rng.standard_normal((4000, 8)).astype(np.float32)
    centers = rng.standard_normal((16, 8)).astype(np.float32)
    labels = rng.integers(0, 16, size=4000)
    _, s_abs, s_sq = oc.kmeans_update(x, labels, centers)
    for rule, value in ((1, s_sq), (2, s_abs * s_abs)):
        for tol, expect in ((value * 1.01, 1), (value * 0.99, 0)):
            c, stop = dev(centers), torch.zeros(1, dtype=torch.int32, device="cuda")
            capi.kmeans_update(dev(x), dev(labels), c, stop=stop, rule=rule, tol=float(tol))
            assert int(stop.item()) == expect == int(oc.kmeans_stop(s_abs, s_sq, float(np.float32(tol)), rule))
    # rule 0 never stops; a raised flag turns the call into a no-op
    c, stop = dev(centers), torch.zeros(1, dtype=torch.int32, device="cuda")
    capi.kmeans_update(dev(x), dev(labels), c, stop=stop, rule=0, tol=1e30)
    assert int(stop.item()) == 0 and not np.array_equal(c.cpu().numpy(), centers)
    c, stop = dev(centers), torch.ones(1, dtype=torch.int32, device="cuda")
    shift = torch.full((2,), 7.0, device="cuda")
    capi.kmeans_update(dev(x), dev(labels), c, stop=stop, rule=1, tol=0.0, shift=shift)
    assert np.array_equal(c.cpu().numpy(), centers) and shift.tolist() == [7.0, 7.0]


def test_lloyd_loop_lowers_the_inertia_and_recovers_blobs():
    rng = np.random.default_rng(11)
    pts, truth, means = blobs(rng, 2000, 6)
    x = dev(pts)
    centers = dev(pts[[int(np.flatnonzero(truth == c)[0]) for c in range(6)]].copy())   # one start per blob
    last = np.inf
    for _ in range(25):
        labels = capi.kmeans_predict(x, centers, "l2")
        inertia = float(((x.double() - centers[labels].double()) ** 2).sum())
        assert inertia <= last * (1 + 1e-6)
        last = inertia
        capi.kmeans_update(x, labels, centers)
    labels = capi.kmeans_predict(x, centers, "l2").cpu().numpy()
    assert np.array_equal(labels, truth)
    want = np.stack([pts[truth == c].astype(np.float64).mean(axis=0) for c in range(6)])
    assert np.allclose(centers.cpu().numpy(), want, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("metric", ["l2", "cosine"])
def test_kmeans_fit_reaches_a_fixed_point(metric):
    lib = f2cgt_amd.load()
    rng = np.random.default_rng(21)
    pts, _, _ = blobs(rng, 1500, 8)
    x = dev(pts)
    torch.manual_seed(3)
    km = lib.KMeans(12, 8, metric, max_iter=300, tol=1e-10)
    km.fit(x)
    centers = km.get_centers()
    assert centers.shape == (12, 8) and bool(torch.isfinite(centers).all())
    assert 1 <= km.n_iter <= 300
    # every centre with members is the mean of its members: one more update moves nothing
    labels = km.predict(x)
    assert labels.dtype == torch.int64 and int(labels.min()) >= 0 and int(labels.max()) < 12
    want, _, s_sq = oc.kmeans_update(pts, labels.cpu().numpy(), centers.cpu().numpy())
    assert s_sq < 1e-6 and np.allclose(centers.cpu().numpy(), want, atol=1e-4)
    # a loose tolerance stops earlier, in a multiple of the eight iterations between two looks at the flag
    torch.manual_seed(3)
    quick = lib.KMeans(12, 8, metric, max_iter=300, tol=1e-1)
    quick.fit(x)
    assert quick.n_iter <= km.n_iter and (quick.n_iter % 8 == 0 or quick.n_iter == 300)


def test_kmeans_warns_about_ignored_arguments():
    lib = f2cgt_amd.load()
    with warnings.catch_warnings(record=True) as seen:
        warnings.simplefilter("always")
        lib.KMeans(4, 8, "l2")
        assert not seen
        lib.KMeans(4, 8, "l2", n_init=3, batch_samples=1024, inertia_check=True)
        text = " ".join(str(w.message) for w in seen)
    assert "n_init" in text and "batch_samples" in text and "inertia_check" in text


@pytest.mark.parametrize("metric,width", [("cosine", 8), ("cosine", 7), ("euclidean", 16)])
def test_pipeline_trainer_follows_the_reference_rule(metric, width):
    rng = np.random.default_rng(31)
    pts, _, _ = blobs(rng, 1200, width, spread=5.0)
    x = dev(pts)
    runs = []
    for check_every in (1, 8):
        g = torch.Generator().manual_seed(9)
        km = pipeline.KMeansTrainer(10, metric=metric, tol=5e-2, check_every=check_every, generator=g)
        km.fit(x)
        assert km.get_centers().shape == (10, width) and bool(torch.isfinite(km.get_centers()).all())
        runs.append(km)
    # the kernel freezes the centres at the iteration the rule first holds: how often the host looks makes no difference
    assert runs[1].n_iter % 8 == 0 and runs[0].n_iter <= runs[1].n_iter
    assert torch.allclose(runs[0].get_centers(), runs[1].get_centers(), rtol=1e-4, atol=1e-5)
    # replay on the host with the oracle's update and rule, from the same start
    g = torch.Generator().manual_seed(9)
    centers = pipeline.KMeansTrainer(10, metric=metric, generator=g)._initial_centers(x).cpu().numpy()
    tol, it = 5e-2, 0
    oracle_metric = "cosine" if metric == "cosine" else "l2"
    while True:
        labels = oc.kmeans_predict(pts, centers, oracle_metric)[0]
        centers, s_abs, s_sq = oc.kmeans_update(pts, labels, centers)
        it += 1
        if oc.kmeans_stop(s_abs, s_sq, tol, 2) or it >= 1000:
            break
        tol *= 1.2
    assert it == runs[0].n_iter
    assert np.allclose(runs[0].get_centers().cpu().numpy(), centers, rtol=1e-3, atol=1e-3)
    labels = runs[0].predict(x)
    assert labels.shape == (len(pts),)


def test_nan_shift_raises_the_flag_and_ends_the_fit():
    """A centre shift that is not a number never satisfies `shift < tol`: the update kernel flags it
    (stop == 2), the trainer ends without centres like the reference's (examples/my_kmeans.py:108-109)
    and KMeans.fit raises."""
    rng = np.random.default_rng(77)
    x = rng.standard_normal((2000, 8)).astype(np.float32)
    x[17, 3] = np.nan
    centers = rng.standard_normal((8, 8)).astype(np.float32)
    labels = rng.integers(0, 8, size=2000)
    c, stop = dev(centers), torch.zeros(1, dtype=torch.int32, device="cuda")
    capi.kmeans_update(dev(x), dev(labels), c, stop=stop, rule=2, tol=1e-4)
    assert int(stop.item()) == 2
    frozen = c.clone()
    capi.kmeans_update(dev(x), dev(labels), c, stop=stop, rule=2, tol=1e-4)      # a no-op once the flag is up
    assert torch.equal(torch.nan_to_num(frozen), torch.nan_to_num(c)) and int(stop.item()) == 2
    km = pipeline.KMeansTrainer(8, metric="euclidean", tol=1e-4, generator=torch.Generator().manual_seed(1))
    with warnings.catch_warnings(record=True) as seen:
        warnings.simplefilter("always")
        km.fit(dev(x))
    assert km.get_centers() is None and km.n_iter <= 8 and any("NaN" in str(w.message) for w in seen)
    with pytest.raises(RuntimeError, match="NaN"):
        f2cgt_amd.load().KMeans(8, 8, "l2", max_iter=50).fit(dev(x))


def test_cosine_fit_with_a_zero_row():
    """A zero-norm row has no cosine distance (0 / 0): the reference's trainer sets such distances to 1
    before the arg-min (examples/my_kmeans.py:92-94), so the row goes to centre 0; here all its scores
    tie and the first centre wins as well, and nothing non-finite reaches the centres."""
    rng = np.random.default_rng(12)
    pts, _, _ = blobs(rng, 400, 8, spread=5.0)
    pts[5] = 0.0
    x = dev(pts)
    km = pipeline.KMeansTrainer(6, metric="cosine", tol=5e-2, generator=torch.Generator().manual_seed(4))
    km.fit(x)
    centers = km.get_centers()
    assert centers is not None and bool(torch.isfinite(centers).all())
    labels = km.predict(x)
    assert int(labels[5]) == 0
    want = oc.kmeans_predict(pts, centers.cpu().numpy(), "cosine")[0]
    assert int(want[5]) == 0
