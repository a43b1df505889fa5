"""The fused layer publishes the routed ids before the softmax denominator is known: it accepts its candidates when
their exponentials e are separated by the margin below, and claims that the probabilities p = fl(e * inv) - one inv
per row, 1 / sum with 1 <= sum <= 1024, as in the reference (src/qwen38_moe.cuh:711-749) - are then strictly
ordered as well.  This checks the claim in float32 arithmetic on the tightest pairs the test lets through."""
import numpy as np

MARGIN = np.float32(1.000001)     # the constant of the device code
FLOOR = np.float32(2.0 ** -100)


def _tightest_pairs(rng, n):
    # e_b anywhere a softmax numerator can be (down to subnormals), e_a the smallest float the test accepts above it
    expo = rng.uniform(-149.0, 0.0, n)
    e_b = np.exp2(expo).astype(np.float32) * rng.uniform(1.0, 2.0, n).astype(np.float32)
    e_b = np.minimum(e_b, np.float32(1.0))
    below = (e_b * MARGIN).astype(np.float32)
    e_a = np.nextafter(np.maximum(below, np.nextafter(FLOOR, np.float32(0.0))), np.float32(np.inf))
    keep = e_a <= np.float32(1.0)
    return e_a[keep], e_b[keep]


def test_margin_on_exponentials_orders_the_probabilities():
    rng = np.random.default_rng(20261014)
    e_a, e_b = _tightest_pairs(rng, 2_000_000)
    assert np.all(e_a >= FLOOR) and np.all(e_a > (e_b * MARGIN).astype(np.float32))
    sums = np.concatenate([rng.uniform(1.0, 1024.0, e_a.size - 4), [1.0, 1024.0, 1.0 + 2.0 ** -40, 1023.999999]])
    inv = (1.0 / sums).astype(np.float32)   # static_cast<float>(1.0 / sum) of a double sum
    p_a = (e_a * inv).astype(np.float32)
    p_b = (e_b * inv).astype(np.float32)
    assert np.all(p_a > p_b)
    assert np.all(p_a >= np.float32(2.0 ** -111))   # far above the subnormal range, where products lose bits


def test_without_the_margin_the_order_can_collapse():
    # negative control: adjacent exponentials do round to the same probability for some denominators
    rng = np.random.default_rng(7)
    e_b = rng.uniform(0.5, 1.0, 200_000).astype(np.float32)
    e_a = np.nextafter(e_b, np.float32(np.inf))
    inv = (1.0 / rng.uniform(1.0, 1024.0, e_b.size)).astype(np.float32)
    assert np.any((e_a * inv).astype(np.float32) == (e_b * inv).astype(np.float32))
