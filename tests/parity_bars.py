"""The bars that a mean aggregation computed in another order than the reference's sequential fp32
sum has to meet (shared by the GPU parity tests)."""
import numpy as np

RTOL = 1e-5


def assert_mean_aggregate(got, want, exact, unit, deg=None):
    """`got`: the GPU result; `want`: the oracle's sequential fp32 evaluation (the reference's order);
    `exact`: the same mean in float64; `unit`: the largest decoded magnitude that enters a sum.

    * every element within 1e-5 of the row's largest magnitude of the reference result (the
      "1e-5 relative" of the contract, taken per destination row rather than over the whole output);
    * no further from the float64 mean than the reference's own fp32 evaluation is, up to four units
      in the last place of the largest summand;
    * a row with one neighbour is that neighbour's decoded row, bit for bit (when `deg` is given).
    """
    got = np.asarray(got)
    assert got.shape == want.shape
    row_scale = np.abs(want).max(axis=1, keepdims=True) if want.size else np.zeros((want.shape[0], 1))
    assert np.all(np.abs(got - want) <= RTOL * np.maximum(row_scale, 1e-30) + 1e-30), \
        float(np.max(np.abs(got - want) / np.maximum(row_scale, 1e-30)))
    if want.size:
        slack = 4 * float(np.spacing(np.float32(unit)))
        assert np.abs(got - exact).max() <= np.abs(want - exact).max() + slack
    if deg is not None:
        single = np.asarray(deg) <= 1
        assert np.array_equal(got[single], want[single])
