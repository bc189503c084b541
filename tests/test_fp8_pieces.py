"""The arithmetic behind the fp8 x fp4 TQ1 GEMV, checked on the CPU: an activation is split into three OCP E4M3
pieces under a power-of-two prescale of its 128-wide group (deepseekternarized_amd/csrc/bp_tq1_gemv_fp4.hip). The
kernel's accuracy claim rests on two facts that do not need a GPU: E4M3 round-to-nearest-even as emulated here is
what the hardware conversion was observed to do (the known answers below were read back from v_cvt_pk_fp8_f32 /
v_cvt_f32_fp8 on gfx950), and the three pieces reconstruct a value to within 2^-20 of the group's largest
magnitude - exactly, for bf16 and int8 values that are not more than 2^9 below it."""

import numpy as np
import pytest

E4M3_VALUES = np.array(sorted({s * (m / 8.0 * 2.0 ** -6 if e == 0 else (1 + m / 8.0) * 2.0 ** (e - 7))
                               for s in (1.0, -1.0) for e in range(16) for m in range(8) if not (e == 15 and m == 7)}))


def e4m3_rne(x: np.ndarray) -> np.ndarray:
    """Nearest E4M3 value, ties to the even mantissa (|x| <= 448)."""
    x = np.asarray(x, np.float64)
    idx = np.clip(np.searchsorted(E4M3_VALUES, x), 1, len(E4M3_VALUES) - 1)
    lo, hi = E4M3_VALUES[idx - 1], E4M3_VALUES[idx]
    pick_hi = (x - lo) > (hi - x)
    tie = (x - lo) == (hi - x)

    def even(v):  # mantissa code of a grid value is even
        a = np.abs(v)
        e = np.floor(np.log2(np.maximum(a, 2.0 ** -9)))
        step = np.where(a < 2.0 ** -6, 2.0 ** -9, 2.0 ** (e - 3))
        return (np.round(a / step) % 2) == 0

    return np.where(pick_hi | (tie & even(hi) & ~even(lo)), hi, lo)


def split3(y: np.ndarray):
    p0 = e4m3_rne(y)
    p1 = e4m3_rne(y - p0)
    p2 = e4m3_rne((y - p0 - p1) * 256.0)
    return p0, p1, p2


def test_e4m3_known_answers_from_the_hardware():
    """Values and what v_cvt_pk_fp8_f32 followed by v_cvt_f32_fp8 returned for them on gfx950."""
    x = np.array([1.0, 448.0, 2.0 ** -9, 3.0, -1.5, 2.0 ** -10, 255.0, 17.0, 0.0, 1.0625, 1.1875, -0.0029296875, 240.0,
                  0.01171875, 0.013671875])
    want = np.array([1.0, 448.0, 2.0 ** -9, 3.0, -1.5, 0.0, 256.0, 16.0, 0.0, 1.0, 1.25, -0.00390625, 240.0, 0.01171875,
                     0.013671875])
    assert np.array_equal(e4m3_rne(x), want)
    assert len(E4M3_VALUES) == 253 and E4M3_VALUES.max() == 448.0  # +-0 once, no NaN codes


def _prescaled(x: np.ndarray) -> tuple[np.ndarray, float]:
    amax = np.abs(x).max()
    sh = 7 - int(np.floor(np.log2(amax)))  # brings the largest magnitude into [128, 256)
    return x.astype(np.float64) * 2.0 ** sh, 2.0 ** sh


@pytest.mark.parametrize("kind", ["bf16", "int8", "f16"])
def test_three_pieces_reconstruct_a_group(kind):
    rng = np.random.default_rng(1)
    for trial in range(50):
        x = rng.standard_normal(128) * np.exp(rng.uniform(-8, 3, 128))
        if kind == "bf16":
            x = (x.astype(np.float32).view(np.uint32) & 0xFFFF0000).view(np.float32).astype(np.float64)  # 8 significant bits
        elif kind == "f16":
            x = x.astype(np.float16).astype(np.float64)
        else:
            x = np.clip(np.rint(x * 20), -127, 127)
            if not x.any():
                x[0] = 1.0
        y, pre = _prescaled(x) if kind != "int8" else (x.copy(), 1.0)
        amax = np.abs(y).max()
        assert kind == "int8" or 128.0 <= amax < 256.0
        p0, p1, p2 = split3(y)
        err = np.abs(y - (p0 + p1 + p2 / 256.0))
        assert err.max() <= 2.0 ** -20 * max(amax, 128.0), (kind, trial, err.max())
        big = np.abs(y) >= 2.0 ** -9 * amax  # i.e. |y| >= 1/4: the remainder after the first piece is a multiple of 2^-9
        if kind in ("bf16", "int8"):  # 8 significant bits: two pieces suffice in that range
            assert np.array_equal((p0 + p1)[big], y[big])
        else:
            assert np.array_equal((p0 + p1 + p2 / 256.0)[big], y[big])


@pytest.mark.parametrize("kind", ["bf16", "int8"])
def test_two_pieces_for_small_batches(kind):
    """The small-batch variant keeps two pieces (bf16 / int8 activations only): exact down to 2^-9 of the group's largest
    magnitude, and what is dropped below that is at most 2^-17 of it."""
    rng = np.random.default_rng(5)
    for trial in range(200):
        x = rng.standard_normal(128) * np.exp(rng.uniform(-8, 8, 128))
        if kind == "bf16":
            x = (x.astype(np.float32).view(np.uint32) & 0xFFFF0000).view(np.float32).astype(np.float64)
            y, _ = _prescaled(x)
        else:
            y = np.clip(np.rint(x * 20), -127, 127)
        amax = max(np.abs(y).max(), 128.0)
        p0, p1, _ = split3(y)
        err = np.abs(y - (p0 + p1))
        assert err.max() <= 2.0 ** -17 * amax, (kind, trial, err.max())
        big = np.abs(y) >= 2.0 ** -9 * amax
        assert np.array_equal((p0 + p1)[big], y[big])


def test_pieces_stay_in_range():
    """No piece can overflow E4M3 (the conversion does not saturate: 500 became NaN on the hardware)."""
    y = np.concatenate([np.linspace(-255.99, 255.99, 100001), [255.9999, -255.9999, 2.0 ** -9, 2.0 ** -10]])
    p0, p1, p2 = split3(y)
    for p in (p0, p1, p2):
        assert np.abs(p).max() <= 448.0
    assert np.abs(y - p0).max() <= 8.0 and np.abs((y - p0 - p1) * 256.0).max() <= 256.0
