"""The oracle's Lloyd update and stopping rules, pinned by independent statements: per-cluster means
by boolean masks, a hand-computed case, and what any Lloyd step must satisfy."""
import numpy as np

import f2cgt_oracle as oc


def test_update_equals_masked_means_and_keeps_empty_clusters():
    rng = np.random.default_rng(0)
    x = rng.standard_normal((5000, 7)).astype(np.float32)
    centers = rng.standard_normal((11, 7)).astype(np.float32)
    labels = rng.integers(0, 9, size=5000)            # clusters 9 and 10 stay empty
    new, s_abs, s_sq = oc.kmeans_update(x, labels, centers)
    for c in range(11):
        members = x[labels == c]
        want = members.astype(np.float64).mean(axis=0) if len(members) else centers[c]
        assert np.allclose(new[c], want, rtol=1e-6, atol=1e-7)
    assert np.array_equal(new[9:], centers[9:])
    d = new.astype(np.float64) - centers.astype(np.float64)
    assert np.isclose(s_abs, np.linalg.norm(d, axis=1).sum()) and np.isclose(s_sq, (d ** 2).sum())


def test_update_hand_computed():
    x = np.array([[0, 0], [2, 0], [10, 10], [10, 12], [10, 14]], dtype=np.float32)
    centers = np.array([[0, 1], [9, 9], [100, 100]], dtype=np.float32)
    labels = np.array([0, 0, 1, 1, 1])
    new, s_abs, s_sq = oc.kmeans_update(x, labels, centers)
    assert np.array_equal(new, np.array([[1, 0], [10, 12], [100, 100]], dtype=np.float32))
    # shifts: (1,-1) -> sqrt 2 ; (1,3) -> sqrt 10 ; 0
    assert np.isclose(s_abs, np.sqrt(2) + np.sqrt(10)) and np.isclose(s_sq, 12.0)
    assert oc.kmeans_stop(s_abs, s_sq, 12.5, 1) and not oc.kmeans_stop(s_abs, s_sq, 12.0, 1)
    assert oc.kmeans_stop(s_abs, s_sq, 21.0, 2) and not oc.kmeans_stop(s_abs, s_sq, 20.9, 2)   # (sqrt2+sqrt10)^2 = 20.94
    assert not oc.kmeans_stop(0.0, 0.0, 1.0, 0)


def test_lloyd_invariants():
    rng = np.random.default_rng(1)
    x = np.concatenate([rng.standard_normal((300, 4)) + 6 * e for e in np.eye(4)]).astype(np.float32)
    centers = x[rng.choice(len(x), 6, replace=False)].copy()
    last = np.inf
    for _ in range(40):
        labels = oc.kmeans_predict(x, centers, "l2")[0]
        inertia = float(((x.astype(np.float64) - centers[labels].astype(np.float64)) ** 2).sum())
        assert inertia <= last * (1 + 1e-6)           # assignment and mean both lower the inertia
        last = inertia
        centers, s_abs, s_sq = oc.kmeans_update(x, labels, centers)
        if s_sq == 0.0:
            break
    again, s_abs, s_sq = oc.kmeans_update(x, oc.kmeans_predict(x, centers, "l2")[0], centers)
    assert s_sq < 1e-10 and np.allclose(again, centers, atol=1e-6)   # a fixed point stays put
