"""The fused boost selection takes a channel's score - mean |k| over the page, rounded once to fp16 -
from an fp32 tree sum whenever both ends of an error interval around it round to the same fp16 number,
and adds exactly only otherwise (quant_pack.hip).  This restates that decision in numpy with the
kernel's order of additions and checks the claim it rests on: whenever the interval test says "no
doubt", the fp16 score equals the one from the exact sum.  Random pages at many scales, and sums
built to land on, next to, and far from the midpoints between fp16 numbers."""
import numpy as np

F = np.float32


def _tree8(x):
    """((x0 + x1) + (x2 + x3)) + ((x4 + x5) + (x6 + x7)) along the last axis, in fp32."""
    a = x[..., 0::2] + x[..., 1::2]
    b = a[..., 0::2] + a[..., 1::2]
    return b[..., 0] + b[..., 1]


def kernel_decision(page):
    """page: fp16 [channels, 128 tokens].  Returns (fp16 score bits where the kernel sees no doubt,
    doubt mask), following quant_k_page: a thread adds 8 tokens as a tree, a lane folds the partials
    of token groups g, g+2, ..., g+14 as a tree (g = 0 or 1), the two lanes of a pair add."""
    ax = np.abs(page.astype(F))                                   # [C, 128]
    part = _tree8(ax.reshape(-1, 16, 8))                          # [C, 16]: one per token group
    lane0, lane1 = _tree8(part[:, 0::2]), _tree8(part[:, 1::2])
    s = (lane0 + lane1).astype(F)
    mean = (s * F(1.0 / 128)).astype(F)
    lo = (mean * F(1.0 - 10 * 2.0 ** -24)).astype(F).astype(np.float16)
    hi = (mean * F(1.0 + 10 * 2.0 ** -24)).astype(F).astype(np.float16)
    doubt = (lo.view(np.uint16) != hi.view(np.uint16)) | ((mean < F(2.0 ** -13)) & (s != 0))
    return lo.view(np.uint16), doubt


def exact_score(page):
    """fp16(mean |k|) with one rounding: the sum of 128 fp16 magnitudes is exact in float64."""
    s = np.abs(page.astype(np.float64)).sum(axis=-1)
    return (s / 128.0).astype(np.float16).view(np.uint16)


def _check(page):
    got, doubt = kernel_decision(page)
    want = exact_score(page)
    bad = (~doubt) & (got != want)
    assert not bad.any(), (np.flatnonzero(bad)[:5], got[bad][:5], want[bad][:5])
    return doubt


def test_interval_test_never_accepts_a_wrong_score_on_random_pages():
    rng = np.random.default_rng(0)
    n_doubt = n = 0
    for scale in (1e-4, 1e-2, 0.3, 1.0, 7.0, 300.0, 2e4):
        for dist in ("normal", "student", "lognormal"):
            x = {"normal": rng.standard_normal((20000, 128)),
                 "student": rng.standard_t(3, (20000, 128)),
                 "lognormal": np.exp(3 * rng.standard_normal((20000, 128)))}[dist] * scale
            page = np.clip(x, -65504, 65504).astype(np.float16)
            d = _check(page)
            if scale >= 1e-2:                 # (below that the means are under 2^-13, where the exact path is the rule)
                n_doubt += int(d.sum())
                n += d.size
    assert 0 < n_doubt < n // 200         # the slow path is taken, and rarely (about one channel in 600)


def test_interval_test_on_sums_built_around_fp16_midpoints():
    """Pages whose exact mean is m, m - 2^-24 / 128 ... m + a few fp16 steps of one token, for
    midpoints m between fp16 numbers at several magnitudes: on the midpoint and within fp32's
    error of it the kernel must doubt; far from it must agree with the exact score either way."""
    rng = np.random.default_rng(1)
    pages = []
    for base in (1.0, 1000.0, 0.0123, 31.5, 4096.0):
        h = np.float16(base)
        step = float(np.nextafter(h, np.float16(np.inf))) - float(h)
        # 127 tokens at h, one token that moves the sum by k quarter-steps (exactly representable or not, the cast decides)
        for k in range(-8, 200):
            row = np.full(128, float(h))
            row[rng.integers(0, 128)] = float(h) + k * step * 0.25 * 128 / 4
            pages.append(row)
        # half a step spread over many tokens, plus the smallest subnormal in one of them
        for tiny in (0.0, 2.0 ** -24, 3 * 2.0 ** -24):
            row = np.full(128, float(h))
            row[:64] = float(h) + step
            row[127] = tiny if tiny else float(h)
            pages.append(row)
    page = np.array(pages).astype(np.float16)
    d = _check(page)
    assert d.any() and not d.all()


def test_zero_and_tiny_channels():
    page = np.zeros((4, 128), np.float16)
    page[1, 5] = 2.0 ** -24
    page[2, :] = 2.0 ** -24
    page[3, :] = 6.1e-5
    got, doubt = kernel_decision(page)
    assert not doubt[0] and got[0] == 0                  # an all-zero channel: score 0, no slow path
    assert doubt[1] and doubt[2] and doubt[3]            # means below 2^-13 always take the exact path
