"""The resize oracle against the library it restates (Pillow is installed: the oracle's output is compared with
PIL.Image.resize itself, bit for bit), smart_resize against its defining properties and hand-computed cases, and the
product's host-side coefficient tables / smart_resize against the oracle."""

import math

import numpy as np
import pytest

from oracle import resize_oracle as R

Image = pytest.importorskip("PIL.Image")
FILTERS = {R.BILINEAR: Image.Resampling.BILINEAR, R.BICUBIC: Image.Resampling.BICUBIC}


def _pil(img, oh, ow, name):
    return np.asarray(Image.fromarray(img).resize((ow, oh), FILTERS[name]))


@pytest.mark.parametrize("name", [R.BILINEAR, R.BICUBIC])
def test_oracle_equals_pillow_on_random_sizes(name):
    rng = np.random.default_rng(5)
    for _ in range(60):
        h, w = int(rng.integers(1, 90)), int(rng.integers(1, 90))
        oh, ow = int(rng.integers(1, 120)), int(rng.integers(1, 120))
        img = rng.integers(0, 256, (h, w, 3), dtype=np.uint8)
        assert np.array_equal(R.pil_resize(img, oh, ow, name), _pil(img, oh, ow, name)), (h, w, oh, ow)


@pytest.mark.parametrize("name", [R.BILINEAR, R.BICUBIC])
def test_oracle_equals_pillow_on_structured_images(name):
    """Saturated and high-contrast images exercise the clamp (bicubic overshoots) and the rounding."""
    rng = np.random.default_rng(6)
    checker = ((np.indices((56, 84)).sum(0) % 2) * 255).astype(np.uint8)[..., None].repeat(3, 2)
    ramp = np.linspace(0, 255, 84 * 56).reshape(56, 84).astype(np.uint8)[..., None].repeat(3, 2)
    flat = np.full((30, 40, 3), 255, np.uint8)
    sparse = (rng.random((70, 50, 3)) < 0.1).astype(np.uint8) * 255
    for img in (checker, ramp, flat, sparse):
        for oh, ow in ((28, 28), (56, 84), (112, 140), (img.shape[0], 28), (28, img.shape[1]), (196, 28)):
            assert np.array_equal(R.pil_resize(img, oh, ow, name), _pil(img, oh, ow, name)), (img.shape, oh, ow)


def test_oracle_equals_pillow_for_the_reference_fixed_size_resize():
    """python/data/preprocessing.py:126-131: img.resize((fixed, fixed), BILINEAR) with fixed = int(sqrt(max_pixels))."""
    rng = np.random.default_rng(7)
    fixed = int(math.sqrt(50176))  # 224
    img = rng.integers(0, 256, (317, 411, 3), dtype=np.uint8)
    assert np.array_equal(R.pil_resize(img, fixed, fixed, R.BILINEAR), _pil(img, fixed, fixed, R.BILINEAR))


def test_coefficients_are_a_partition_of_unity_and_identity_when_sizes_match():
    for name in (R.BILINEAR, R.BICUBIC):
        bounds, kk = R.resample_coefficients(40, 40, name)
        # same size: every window's weights sum to 2^22 and the centre tap carries (almost) all of it
        assert np.all(np.abs(kk.sum(1) - (1 << R.PRECISION_BITS)) <= 2)
        for a, b in ((97, 28), (28, 97), (300, 299)):
            bounds, kk = R.resample_coefficients(a, b, name)
            assert np.all(np.abs(kk.sum(1) - (1 << R.PRECISION_BITS)) <= kk.shape[1])  # rounding of each tap
            assert np.all(bounds[:, 0] >= 0) and np.all(bounds[:, 0] + bounds[:, 1] <= a) and np.all(bounds[:, 1] >= 1)


def test_smart_resize_properties_and_known_values():
    # hand-computed: 1000 x 700 -> round(35.71) * 28 = 1008, round(25) * 28 = 700; 1008 * 700 = 705,600 <= 1,003,520
    assert R.smart_resize(1000, 700) == (1008, 700)
    # too large: 4000 x 3000, beta = sqrt(12e6 / 1003520) = 3.458...; floor(4000 / beta / 28) = 41 -> 1148; floor(3000 / beta / 28) = 30 -> 840
    assert R.smart_resize(4000, 3000) == (1148, 840)
    # too small: 20 x 30 -> h_bar 28, w_bar 28 (784 < 3136): beta = sqrt(3136 / 600) = 2.286; ceil(20 * beta / 28) = 2 -> 56; ceil(30 * beta / 28) = 3 -> 84
    assert R.smart_resize(20, 30) == (56, 84)
    assert R.smart_resize(3584, 3584, max_pixels=3584 * 3584) == (3584, 3584)
    with pytest.raises(ValueError):
        R.smart_resize(10, 2001)
    rng = np.random.default_rng(8)
    for _ in range(2000):
        h, w = int(rng.integers(1, 5000)), int(rng.integers(1, 5000))
        if max(h, w) / min(h, w) > 200:
            continue
        th, tw = R.smart_resize(h, w)
        assert th % 28 == 0 and tw % 28 == 0 and th >= 28 and tw >= 28
        if th > 28 and tw > 28:
            assert th * tw <= 14 * 14 * 4 * 1280
        assert th * tw >= 56 * 56 or min(th, tw) == 28
    # round() is Python's round-half-to-even: 42 / 28 = 1.5 -> 2, 70 / 28 = 2.5 -> 2
    assert R.smart_resize(42 * 4, 70 * 4)[0] == 168 and R.smart_resize(70, 70 * 3) == (56, 224)


def test_product_host_logic_equals_the_oracle():
    """mi355_vit.pixels computes the coefficient tables with vectorised numpy and has its own smart_resize: both must
    be the oracle's, bit for bit."""
    import sys
    from pathlib import Path

    sys.path.insert(0, str(Path(__file__).resolve().parents[1] / "multimodal-training_amd"))
    from mi355_vit import pixels as P

    rng = np.random.default_rng(9)
    cases = [(int(rng.integers(1, 500)), int(rng.integers(1, 500))) for _ in range(150)]
    cases += [(3584, 1792), (1792, 3584), (5000, 3584), (3584, 3584), (1, 28), (28, 1), (4000, 28), (2, 3), (3, 2)]
    for a, b in cases:
        for name in (R.BILINEAR, R.BICUBIC):
            ob, ok = R.resample_coefficients(a, b, name)
            pb, pk = P.resample_coefficients(a, b, name)
            assert np.array_equal(ob, pb) and np.array_equal(ok, pk), (a, b, name)
    for h in range(1, 400, 7):
        for w in range(1, 400, 5):
            if max(h, w) / min(h, w) <= 200:
                assert P.smart_resize(h, w) == R.smart_resize(h, w)
    assert P.smart_resize(4000, 3000) == (1148, 840)
    with pytest.raises(ValueError):
        P.resample_coefficients(10, 10, "lanczos")
