"""Blockwise DCT-II on the matrix cores. The reference has no cosine transform (its "DCT"
emitter is the threshold codec), so there is no reference output to match: the transform is
pinned by the library definition scipy.fft.dct(type=2, norm="ortho") on blocks of 256, by the
orthonormality of the basis (Parseval) and by the round trip. Tolerance: 1e-5 relative to the
block's norm (a coefficient is a sum of 256 fp32 products; relative to a single coefficient no
bound exists, since coefficients pass through zero); test_fp32_accuracy_of_the_split_products
holds the kernels (fp32 products made of bf16 pieces) to what a plain fp32 product achieves."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dct2():
    from kraken_amd import api, dct2 as d
    api.lib()
    return d


def _ref(x, keep):
    fft = pytest.importorskip("scipy.fft")
    return fft.dct(x.reshape(-1, 256).astype(np.float64), type=2, norm="ortho", axis=1)[:, :keep]


@pytest.mark.parametrize("blocks", [1, 3, 128, 1000])
@pytest.mark.parametrize("keep", [64, 128, 256])
def test_forward_matches_scipy(dct2, blocks, keep):
    rng = np.random.default_rng(blocks + keep)
    x = rng.standard_normal(blocks * 256).astype(np.float32)
    got = dct2.forward(x, keep)
    want = _ref(x, keep)
    scale = np.linalg.norm(x.reshape(-1, 256), axis=1, keepdims=True)
    assert np.abs(got - want).max() <= 1e-5 * scale.max()
    assert (np.abs(got - want) <= 1e-5 * scale + 1e-7).all()


def test_known_vectors(dct2):
    """Closed forms: a constant block has only the k = 0 coefficient (= c * sqrt(256));
    a single cosine of the basis maps to a single coefficient."""
    x = np.full(256, 0.5, np.float32)
    y = dct2.forward(x, 256)[0]
    assert abs(y[0] - 0.5 * 16.0) < 1e-5 and np.abs(y[1:]).max() < 1e-5
    j = np.arange(256)
    k = 37
    x = (np.sqrt(2.0 / 256) * np.cos(np.pi * (2 * j + 1) * k / 512.0)).astype(np.float32)
    y = dct2.forward(x, 256)[0]
    assert abs(y[k] - 1.0) < 1e-5 and np.abs(np.delete(y, k)).max() < 1e-5


def test_round_trip_and_parseval(dct2):
    rng = np.random.default_rng(1)
    n = 4096 * 256
    x = rng.standard_normal(n).astype(np.float32)
    y = dct2.forward(x, 256)
    assert abs(np.sum(y.astype(np.float64) ** 2) / np.sum(x.astype(np.float64) ** 2) - 1.0) < 1e-5
    back = dct2.inverse(y, n, 256)
    assert np.abs(back - x).max() < 1e-5 * 16
    # truncated: inverse(keep) equals the inverse of the zero-padded coefficients
    y64 = dct2.forward(x, 64)
    assert np.array_equal(y64, y[:, :64])
    fft = pytest.importorskip("scipy.fft")
    pad = np.zeros((n // 256, 256))
    pad[:, :64] = y64
    want = fft.idct(pad, type=2, norm="ortho", axis=1).ravel()
    got = dct2.inverse(y64, n, 64)
    assert np.abs(got - want).max() < 1e-5 * 16


def test_fp32_accuracy_of_the_split_products(dct2):
    """The kernels multiply every fp32 operand as three bf16 pieces (six piece products out of
    nine, fp32 sums). What that must not cost: against float64 the coefficients stay within
    1e-6 of the block norm (a plain fp32 matrix product of the same data is at 2.3e-7 at worst,
    1.8e-8 rms; bf16 operands alone would be at 4e-3), also when the values of a block span
    e^-20 .. e^20, when they are exact small integers (every piece product exact: the result is
    the fp32 product's), and for powers of two near the ends of the fp32 range."""
    fft = pytest.importorskip("scipy.fft")
    rng = np.random.default_rng(77)
    blocks = 4096
    normal = rng.standard_normal(blocks * 256).astype(np.float32)
    wide = (normal * np.exp(rng.uniform(-20, 20, normal.size))).astype(np.float32)
    for x in (normal, wide, normal * np.float32(2.0 ** 100), normal * np.float32(2.0 ** -100)):
        want = fft.dct(x.reshape(-1, 256).astype(np.float64), type=2, norm="ortho", axis=1)
        nrm = np.linalg.norm(x.reshape(-1, 256).astype(np.float64), axis=1, keepdims=True)
        got = dct2.forward(x, 256)
        err = np.abs(got - want) / nrm
        assert err.max() <= 1e-6, err.max()
        assert np.sqrt(np.mean(err ** 2)) <= 3e-8
        back = dct2.inverse(got, x.size, 256).reshape(-1, 256)
        wb = fft.idct(got.astype(np.float64), type=2, norm="ortho", axis=1)
        errb = np.abs(back - wb) / np.linalg.norm(got.astype(np.float64), axis=1, keepdims=True)
        assert errb.max() <= 1e-6, errb.max()
    # a constant block of an integer: sums and differences exact, one nonzero coefficient
    x = np.full(256, 3.0, np.float32)
    y = dct2.forward(x, 256)[0]
    assert y[0] == np.float32(48.0) and np.abs(y[1:]).max() < 1e-5


def test_device_pointers_and_arguments(dct2):
    from kraken_amd import api
    rng = np.random.default_rng(2)
    x = rng.standard_normal(512 * 256).astype(np.float32)
    d = api.DeviceArray.from_host(x)
    y = dct2.forward(d, 64)
    assert np.array_equal(y.to_host(), dct2.forward(x, 64))
    with pytest.raises(api.KrakenHipError):
        dct2.forward(x[:100], 64)
    with pytest.raises(api.KrakenHipError):
        dct2.forward(x, 50)


@pytest.mark.parametrize("keep", [64, 128, 192, 256])
def test_several_tiles_per_workgroup_and_a_ragged_end(dct2, keep):
    """70 001 blocks: workgroups walk two or three row tiles each (a tile's results are stored
    while the next one is multiplied, the last one's after the loop) and the last tile holds 113
    rows. Every block against scipy, forward and back; keep 192 takes three column tiles."""
    fft = pytest.importorskip("scipy.fft")
    rng = np.random.default_rng(1000 + keep)
    blocks = 70_001
    x = rng.standard_normal(blocks * 256).astype(np.float32)
    got = dct2.forward(x, keep)
    want = _ref(x, keep)
    scale = np.linalg.norm(x.reshape(-1, 256).astype(np.float64), axis=1, keepdims=True)
    assert (np.abs(got - want) <= 1e-5 * scale + 1e-7).all()
    pad = np.zeros((blocks, 256))
    pad[:, :keep] = want
    back = dct2.inverse(got, blocks * 256, keep).reshape(-1, 256)
    assert (np.abs(back - fft.idct(pad, type=2, norm="ortho", axis=1)) <= 1e-5 * scale + 1e-7).all()


@pytest.mark.parametrize("keep", [64, 256])
def test_config_size_tensor(dct2, keep):
    """The configuration's own shape, fp32 [4096, 16384] of N(0, 1) = 262144 blocks: scipy on a
    random 1 % of the blocks at 1e-5 of the block norm, Parseval over the whole tensor (keep 256;
    for keep 64 the kept energy can only be smaller, and equals scipy's on the sample), and the
    round trip through the inverse."""
    fft = pytest.importorskip("scipy.fft")
    rng = np.random.default_rng(keep)
    n = 4096 * 16384
    x = rng.standard_normal(n, dtype=np.float32)
    y = dct2.forward(x, keep)
    assert y.shape == (n // 256, keep)
    blocks = rng.choice(n // 256, size=n // 256 // 100, replace=False)
    xb = x.reshape(-1, 256)[blocks]
    want = fft.dct(xb.astype(np.float64), type=2, norm="ortho", axis=1)[:, :keep]
    scale = np.linalg.norm(xb.astype(np.float64), axis=1, keepdims=True)
    err = np.abs(y[blocks] - want) / scale
    assert err.max() <= 1e-5, err.max()
    energy_x = float(np.sum(x.astype(np.float64) ** 2))
    energy_y = float(np.sum(y.astype(np.float64) ** 2))
    if keep == 256:
        assert abs(energy_y / energy_x - 1.0) < 1e-5
        back = dct2.inverse(y, n, keep)
        assert np.abs(back - x).max() <= 1e-5 * np.linalg.norm(xb, axis=1).max()
    else:
        assert energy_y < energy_x
        assert abs(np.sum(y[blocks].astype(np.float64) ** 2) / np.sum(want ** 2) - 1.0) < 1e-5
        pad = np.zeros((blocks.size, 256))
        pad[:, :keep] = want
        back = dct2.inverse(y, n, keep).reshape(-1, 256)[blocks]
        assert np.abs(back - fft.idct(pad, type=2, norm="ortho", axis=1)).max() <= 1e-5 * scale.max()
    print("keep %d: worst coefficient error %.2e of the block norm" % (keep, err.max()))
