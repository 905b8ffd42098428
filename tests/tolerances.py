"""How close the engine must be to the plain implementation. Fixed from the arithmetic, never
widened to pass.

float32: unit roundoff 2^-24 = 6e-8. A logit is the end of a chain of a few hundred sums per layer;
with every sum in float32 the error stays below about 1e-5 of the logits' scale. The bound allows
1e-4 of the largest absolute logit.

bfloat16: activations between kernels are rounded to 8 significant bits (half-ulp 2^-9 = 2e-3), about
ten roundings per layer on the path of a value, accumulating like a random walk; the residual sum
and all reductions stay in float32. The bound allows 5e-2 of the largest absolute logit at the worst
element and 1.2e-2 root-mean-square. A formula mistake (norm in the wrong place, wrong pairing,
a key too many) moves logits by the order of their scale.
"""

import numpy as np

F32_REL = 1e-4
BF16_REL_MAX = 5e-2
BF16_REL_RMS = 1.2e-2


def check_logits(got: np.ndarray, want: np.ndarray, dtype: str, what: str = "") -> None:
    assert got.shape == want.shape, f"{what}: shape {got.shape} != {want.shape}"
    assert np.isfinite(got).all(), f"{what}: non-finite logits"
    scale = float(np.abs(want).max())
    diff = np.abs(got.astype(np.float64) - want)
    worst = float(diff.max())
    if dtype == "float32":
        assert worst <= F32_REL * scale, f"{what}: float32 max |diff| {worst:.3e} > {F32_REL * scale:.3e} (scale {scale:.3f})"
    else:
        rms = float(np.sqrt((diff**2).mean()))
        assert worst <= BF16_REL_MAX * scale, f"{what}: bfloat16 max |diff| {worst:.3e} > {BF16_REL_MAX * scale:.3e}"
        assert rms <= BF16_REL_RMS * scale, f"{what}: bfloat16 rms diff {rms:.3e} > {BF16_REL_RMS * scale:.3e}"


BF16_FEW = 0.02       # the share of positions that may lie above BF16_REL_MAX
BF16_REL_CAP = 1.5e-1  # ... and what the worst of them may reach


def check_logits_by_position(got: np.ndarray, want: np.ndarray, dtype: str, what: str = "") -> None:
    """``check_logits`` for a design that divides every sublayer's output by that output's own root mean square. Where an
    output is the small remainder of large terms, its rounding error is divided by the small size too, so in bfloat16
    single positions carry several times the error of the rest (the same position in every schedule, with every kernel).
    The root mean square over all positions keeps its bound; the worst element keeps its bound at all but ``BF16_FEW`` of
    the positions (at least one), and stays below ``BF16_REL_CAP`` of the scale everywhere. A formula mistake moves the
    logits of most positions by the order of the scale. float32 is held to ``check_logits`` as it stands."""
    if dtype == "float32":
        return check_logits(got, want, dtype, what)
    assert got.shape == want.shape, f"{what}: shape {got.shape} != {want.shape}"
    assert np.isfinite(got).all(), f"{what}: non-finite logits"
    scale = float(np.abs(want).max())
    diff = np.abs(got.astype(np.float64) - want)
    rms = float(np.sqrt((diff**2).mean()))
    assert rms <= BF16_REL_RMS * scale, f"{what}: bfloat16 rms diff {rms:.3e} > {BF16_REL_RMS * scale:.3e}"
    worst = diff.reshape(len(diff), -1).max(axis=-1)
    over = int((worst > BF16_REL_MAX * scale).sum())
    assert over <= max(1, int(BF16_FEW * len(worst))), f"{what}: bfloat16 max |diff| above {BF16_REL_MAX * scale:.3e} at {over} of {len(worst)} positions"
    assert worst.max() <= BF16_REL_CAP * scale, f"{what}: bfloat16 max |diff| {worst.max():.3e} > {BF16_REL_CAP * scale:.3e}"


ROUNDING_TIMES = 3.0   # how many times the error that rounding alone causes a bfloat16 engine may be off at a position
ROUNDING_WORST = 1.5   # ... and how far beyond that the worst position may lie


def check_logits_against_rounding(got: np.ndarray, want: np.ndarray, rounded: np.ndarray, what: str = "") -> None:
    """A bfloat16 engine against the exact logits ``want``, measured by the error that rounding alone causes: ``rounded`` are
    the plain implementation's logits with every matrix product's input rounded to bfloat16 and nothing else changed.
    A position's error is the root mean square over the vocabulary of the difference (its mean taken off); it may be
    ``ROUNDING_TIMES`` the rounding sample's at that position (the sample is one draw: it is not taken below a third of
    its own median over the positions), at all positions but 2 % (at least one), and ``ROUNDING_WORST`` times that at
    the worst."""
    assert got.shape == want.shape == rounded.shape, f"{what}: shapes {got.shape}, {want.shape}, {rounded.shape}"
    assert np.isfinite(got).all(), f"{what}: non-finite logits"

    def per_position(a):
        d = a.astype(np.float64) - want
        d = d - d.mean(axis=-1, keepdims=True)
        return np.sqrt((d * d).mean(axis=-1))

    noise = per_position(rounded)
    limit = ROUNDING_TIMES * np.maximum(noise, np.median(noise) / 3.0)
    ratio = per_position(got) / limit
    over = int((ratio > 1.0).sum())
    assert over <= max(1, int(0.02 * len(ratio))), f"{what}: {over} of {len(ratio)} positions beyond {ROUNDING_TIMES} times the rounding error (worst {ratio.max():.2f})"
    assert ratio.max() <= ROUNDING_WORST, f"{what}: a position at {ratio.max():.2f} times its limit"
