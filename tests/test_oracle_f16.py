"""Pins the oracle's fp32->fp16 rounding (the reference's __float2half in Padding,
src/OperationKernels.cu:846-860) against two independent implementations:
the CPU's F16C hardware converter (exhaustively, all 2^32 inputs) and numpy's
float16 cast, plus the named boundary cases."""
import struct

import numpy as np


def _bits(x: float) -> int:
    return struct.unpack("<I", struct.pack("<f", x))[0]


def test_narrowing_matches_f16c_hardware_exhaustively(oracle):
    bad, first = oracle.f16c_compare_range(0, 1 << 32, 1)
    assert bad == 0, f"{bad} mismatches, first at fp32 bits {first:#010x}"


def test_widening_matches_f16c_hardware_for_every_half(oracle):
    assert oracle.f16c_compare_widen() == 0


def test_named_boundaries(oracle):
    f = oracle.f32_to_f16_bits
    assert f(0.0) == 0x0000 and f(-0.0) == 0x8000
    assert f(1.0) == 0x3C00 and f(-2.0) == 0xC000
    assert f(65504.0) == 0x7BFF
    assert f(65519.99) == 0x7BFF            # below the tie to infinity
    assert f(65520.0) == 0x7C00             # tie rounds to even = inf
    assert f(1e9) == 0x7C00 and f(-1e9) == 0xFC00
    assert f(float("inf")) == 0x7C00
    assert (f(float("nan")) & 0x7C00) == 0x7C00 and (f(float("nan")) & 0x03FF) != 0
    assert f(2.0 ** -24) == 0x0001          # smallest subnormal half
    assert f(2.0 ** -25) == 0x0000          # exact tie -> even (zero)
    assert f(np.nextafter(np.float32(2.0 ** -25), np.float32(1.0))) == 0x0001
    assert f(2.0 ** -14) == 0x0400          # smallest normal half
    assert f(np.nextafter(np.float32(2.0 ** -14), np.float32(0.0))) == 0x0400  # rounds up into normal
    assert f(1.0 + 2.0 ** -11) == 0x3C00    # tie -> even (down)
    assert f(1.0 + 3 * 2.0 ** -11) == 0x3C02  # tie -> even (up)
    assert f(np.nextafter(np.float32(1.0 + 2.0 ** -11), np.float32(2.0))) == 0x3C01


def test_matches_numpy_float16_cast(oracle):
    rng = np.random.default_rng(7)
    bits = rng.integers(0, 1 << 32, size=2_000_000, dtype=np.uint64).astype(np.uint32)
    x = bits.view(np.float32)
    x = x[np.isfinite(x)]
    with np.errstate(over="ignore"):
        expect = x.astype(np.float16).astype(np.float32)
    got = oracle.round_f16(x)
    assert np.array_equal(expect.view(np.uint32), got.view(np.uint32))


def test_round_is_idempotent_and_monotone(oracle):
    x = np.sort(oracle.fill((200_000,), 5, "normal", 0.0, 100.0))
    r = oracle.round_f16(x)
    assert np.array_equal(r, oracle.round_f16(r))
    assert np.all(np.diff(r) >= 0)
    assert np.max(np.abs(r - x) / np.maximum(np.abs(x), 2.0 ** -14)) <= 2.0 ** -11
