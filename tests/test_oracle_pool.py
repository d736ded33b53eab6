"""Pins the pooling / concatenation oracles.

u8 pooling: bit for bit against the reference's own compiled pooling_uint8 (oracle/_ref) over max / mean,
padding on every side, strides, count_include_pad, ceil-mode windows that overhang the bottom / right edge,
global windows, and data on both sides of the zero point 128 (a negative mean saturates to 255 in the
reference, which the oracle must reproduce). Independently of the reference: the maximum against numpy, and
the mean against 128 + floor(sum / taps) on post-ReLU data with power-of-two windows, where the fixed-point
factor 65536 / taps is exact.

s8 concatenation: against the reference's concat_cpu (requantise to the smallest scale, then join) on
channel / height / batch axes in NCHWC16 and NCHW, and against numpy.concatenate for equal scales."""
import numpy as np
import pytest

from checkers_pool import orc_concat, orc_pooling, pool_desc, ref_concat, ref_pooling

POOL_CASES = [  # n, c, ih, iw, kh, kw, sh, sw, pt, pb, pl, pr, mean, count_include_pad, ceil
    (2, 32, 12, 12, 2, 2, 2, 2, 0, 0, 0, 0, 0, 0, 0),
    (2, 32, 12, 12, 2, 2, 2, 2, 0, 0, 0, 0, 1, 0, 0),
    (1, 16, 14, 14, 3, 3, 2, 2, 1, 1, 1, 1, 0, 0, 0),
    (1, 16, 14, 14, 3, 3, 2, 2, 1, 1, 1, 1, 1, 0, 0),
    (1, 16, 14, 14, 3, 3, 2, 2, 1, 1, 1, 1, 1, 1, 0),
    (1, 48, 13, 11, 3, 3, 2, 2, 0, 0, 0, 0, 0, 0, 1),   # ceil mode: windows overhang the bottom / right edge
    (1, 48, 13, 11, 3, 3, 2, 2, 0, 0, 0, 0, 1, 0, 1),
    (1, 16, 9, 17, 3, 5, 1, 3, 2, 2, 4, 4, 1, 0, 0),    # padding larger than the stride
    (1, 16, 9, 17, 3, 5, 1, 3, 2, 2, 4, 4, 0, 0, 0),
    (3, 64, 7, 7, 7, 7, 1, 1, 0, 0, 0, 0, 1, 0, 0),     # global average pooling
    (3, 64, 7, 7, 7, 7, 1, 1, 0, 0, 0, 0, 0, 0, 0),
    (1, 16, 23, 5, 1, 1, 1, 1, 0, 0, 0, 0, 1, 0, 0),    # 1 x 1: identity
    (1, 16, 8, 30, 2, 3, 2, 1, 1, 0, 2, 1, 1, 1, 0),
]


def pool_input(case, seed, relu):
    n, c, ih, iw = case[:4]
    rng = np.random.default_rng(seed)
    lo = 128 if relu else 0
    return rng.integers(lo, 256, size=n * c * ih * iw, dtype=np.uint8)


@pytest.mark.parametrize("relu", [True, False])
@pytest.mark.parametrize("case", POOL_CASES)
def test_pooling_oracle_vs_reference(oracle, ref, case, relu):
    d = pool_desc(case)
    x = pool_input(case, 11 + len(str(case)), relu)
    want, ws = ref_pooling(ref, d, x, 7.25)
    got, gs = orc_pooling(oracle, d, x, 7.25)
    assert np.array_equal(got, want)
    assert np.float32(gs).tobytes() == np.float32(ws).tobytes()


def windows(d, x):
    """[n][c16][oh][ow][taps...][16] gather of clipped windows, as lists per output pixel."""
    xs = x.reshape(d.n * (d.c // 16), d.ih, d.iw, 16)
    for p in range(xs.shape[0]):
        for h in range(d.oh):
            for w in range(d.ow):
                hs, ws = h * d.sh - d.pt, w * d.sw - d.pl
                he, we = min(hs + d.kh, d.ih), min(ws + d.kw, d.iw)
                yield p, h, w, xs[p, max(hs, 0):he, max(ws, 0):we, :].reshape(-1, 16)


@pytest.mark.parametrize("case", POOL_CASES)
def test_pooling_oracle_max_is_numpy_max(oracle, case):
    if case[12]:
        pytest.skip("mean case")
    d = pool_desc(case)
    x = pool_input(case, 5, False)
    got, gs = orc_pooling(oracle, d, x, 3.0)
    got = got.reshape(-1, d.oh, d.ow, 16)
    for p, h, w, win in windows(d, x):
        assert np.array_equal(got[p, h, w], win.max(axis=0))
    assert gs == np.float32(3.0)


@pytest.mark.parametrize("k", [(2, 2), (4, 4), (2, 8), (1, 1)])
def test_pooling_oracle_mean_is_floor_mean_for_power_of_two_windows(oracle, k):
    case = (2, 32, 16, 16, k[0], k[1], k[0], k[1], 0, 0, 0, 0, 1, 0, 0)
    d = pool_desc(case)
    x = pool_input(case, 9, True)
    got, gs = orc_pooling(oracle, d, x, 2.5)
    got = got.reshape(-1, d.oh, d.ow, 16)
    for p, h, w, win in windows(d, x):
        want = 128 + (win.astype(np.int64) - 128).sum(axis=0) // (k[0] * k[1])
        assert np.array_equal(got[p, h, w], want)
    assert gs == np.float32(2.5)   # 65536 / taps is exact, so the scale is unchanged


def test_pooling_oracle_mean_scale_for_odd_window(oracle):
    d = pool_desc((1, 16, 6, 6, 3, 3, 3, 3, 0, 0, 0, 0, 1, 0, 0))
    _, gs = orc_pooling(oracle, d, pool_input((1, 16, 6, 6), 1, True), 10.0)
    assert gs == np.float32(np.float32(np.float32(10.0) * np.float32(7281)) * np.float32(9)) / np.float32(65536)


CONCAT_CASES = [  # df, axis (from the outermost), per-input (n, c, h, w), scales
    (41, 1, [(2, 16, 5, 6), (2, 48, 5, 6), (2, 32, 5, 6)], [11.5, 3.25, 7.0]),
    (41, 1, [(1, 32, 3, 3), (1, 32, 3, 3)], [4.0, 4.0]),
    (0, 1, [(2, 3, 5, 7), (2, 5, 5, 7)], [20.0, 31.0]),
    (0, 2, [(2, 3, 4, 7), (2, 3, 9, 7)], [2.0, 1.5]),
    (0, 0, [(1, 3, 4, 5), (3, 3, 4, 5)], [9.0, 90.0]),
    (0, -1, [(2, 3, 4, 5), (2, 3, 4, 2), (2, 3, 4, 1)], [1.0, 3.0, 2.0]),
]


def concat_layout(case):
    """Bytes per row and rows of the interleave the case amounts to (concat.cpp:113-135)."""
    df, axis, dims, _ = case
    axis %= 4
    lens = [int(np.prod(d[axis:])) for d in dims]
    loops = int(np.prod(dims[0][:axis]))
    odims = list(dims[0])
    odims[axis] = sum(d[axis] for d in dims)
    return lens, loops, odims


def concat_inputs(case, seed):
    rng = np.random.default_rng(seed)
    return [rng.integers(-128, 128, size=int(np.prod(d)), dtype=np.int8) for d in case[2]]


@pytest.mark.parametrize("case", CONCAT_CASES)
def test_concat_oracle_vs_reference(oracle, ref, case):
    df, axis, dims, scales = case
    parts = concat_inputs(case, 3)
    lens, loops, odims = concat_layout(case)
    want, ws = ref_concat(ref, parts, dims, df, axis, scales, odims)
    got, gs = orc_concat(oracle, parts, lens, loops, scales)
    assert np.array_equal(got, want)
    assert np.float32(gs).tobytes() == np.float32(ws).tobytes()


def test_concat_oracle_equal_scales_is_numpy_concatenate(oracle):
    case = (0, 1, [(2, 3, 5, 7), (2, 5, 5, 7)], [6.0, 6.0])
    parts = concat_inputs(case, 4)
    lens, loops, odims = concat_layout(case)
    got, gs = orc_concat(oracle, parts, lens, loops, case[3])
    want = np.concatenate([p.reshape(d) for p, d in zip(parts, case[2])], axis=1)
    assert np.array_equal(got.reshape(odims), want) and gs == np.float32(6.0)
    got2, _ = orc_concat(oracle, parts, lens, loops, None)
    assert np.array_equal(got2, got)


def test_concat_oracle_rescale_truncates_toward_zero(oracle):
    parts = [np.arange(-128, 128, dtype=np.int8), np.arange(-128, 128, dtype=np.int8)]
    got, gs = orc_concat(oracle, parts, [256, 256], 1, [8.0, 2.0])
    r = np.float32(2.0) / np.float32(8.0)
    assert np.array_equal(got[:256], np.trunc(parts[0].astype(np.float32) * r).astype(np.int8))
    assert np.array_equal(got[256:], parts[1]) and gs == np.float32(2.0)
