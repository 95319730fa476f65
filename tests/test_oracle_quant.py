"""Pins the Q8_0 oracle (oracle/quant_oracle.c) without the GPU.

The reference holds no stored vectors for its quantisers: its test round-trips random rows through its own CPU
quantiser and compares the device dequantiser with the CPU one (reference: test/kernels.py:24-56).  Pins here:
the reference's quantiser source itself, compiled into oracle/_ref (byte equality; skipped where that library
has not been built), numpy's IEEE half conversions for the two conversions the oracle carries, hand-computed
blocks, and the bounds the format implies."""
import numpy as np
import pytest

import oracle


def _rows(seed, shape, scale=1.0):
    g = np.random.default_rng(seed)
    return (g.standard_normal(shape) * scale).astype(np.float32)


def test_half_conversions_match_numpy():
    lib = oracle.lib()
    # every fp16 bit pattern converts to the float numpy gives, and back to itself (NaNs keep their class)
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([lib.oracle_f16_to_f32(int(b)) for b in bits], dtype=np.float32)
    finite = np.isfinite(want)
    assert np.array_equal(got[finite], want[finite]) and np.array_equal(np.isnan(got), np.isnan(want))
    assert np.array_equal(np.isinf(got), np.isinf(want))
    back = np.array([lib.oracle_f32_to_f16(float(v)) for v in want[finite]], dtype=np.uint16)
    assert np.array_equal(back, bits[finite])
    # random floats over the whole half range, ties, overflow and underflow edges round as numpy rounds
    g = np.random.default_rng(0)
    vals = np.concatenate([
        (g.standard_normal(20000) * np.exp2(g.integers(-30, 18, 20000))).astype(np.float32),
        np.array([65504.0, 65519.99, 65520.0, 1e9, 2.0 ** -25, np.nextafter(np.float32(2.0 ** -25), np.float32(1)),
                  2.0 ** -24, 1.5 * 2.0 ** -24, 2.5 * 2.0 ** -24, 2049.0, 2051.0, 1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11,
                  0.0, -0.0, 6.1e-5, 6.0975e-5], dtype=np.float32)])
    with np.errstate(over="ignore"):
        want16 = vals.astype(np.float16).view(np.uint16)
    got16 = np.array([lib.oracle_f32_to_f16(float(v)) for v in vals], dtype=np.uint16)
    assert np.array_equal(got16, want16)


def test_hand_computed_blocks():
    # amax = 127 -> d = 1: quants are the values rounded, ties away from zero (roundf), not to even
    x = np.zeros((1, 32), np.float32)
    x[0, :8] = [127.0, -127.0, 0.5, -0.5, 1.5, 2.5, -2.5, 0.49]
    y = oracle.quant_q8_0(x)
    assert y.shape == (1, 34)
    assert y[0, :2].view(np.float16)[0] == np.float16(1.0)
    assert list(y[0, 2:10].view(np.int8)) == [127, -127, 1, -1, 2, 3, -3, 0]
    assert not y[0, 10:].any()
    # a zero block: d = 0, id = 0, all quants 0
    assert not oracle.quant_q8_0(np.zeros((2, 64), np.float32)).any()
    # two blocks per row, scales independent: second block amax = 63.5 -> d = 0.5 exactly
    x = np.zeros((1, 64), np.float32)
    x[0, 0], x[0, 32], x[0, 33] = -254.0, 63.5, 0.25
    y = oracle.quant_q8_0(x)
    assert y[0, 0:2].view(np.float16)[0] == np.float16(2.0) and y[0, 2:3].view(np.int8)[0] == -127
    assert y[0, 34:36].view(np.float16)[0] == np.float16(0.5)
    assert list(y[0, 36:38].view(np.int8)) == [127, 1]          # 0.25 / 0.5 = 0.5 rounds away from zero
    # dequantising multiplies by the stored (rounded) scale
    blk = np.zeros((1, 34), np.uint8)
    blk[0, :2] = np.array([0.1], np.float16).view(np.uint8)
    blk[0, 2:5] = np.array([100, -3, 127], np.int8).view(np.uint8)
    d = np.float32(np.float16(0.1))
    out = oracle.dequant_q8_0(blk)
    assert np.array_equal(out[0, :3], np.array([100, -3, 127], np.float32) * d)
    out16 = oracle.dequant_q8_0(blk, np.float16)
    assert np.array_equal(out16[0, :3], (np.array([100, -3, 127], np.float32) * d).astype(np.float16))


@pytest.mark.parametrize("scale", [1.0, 1e-3, 300.0])
def test_round_trip_bounds(scale):
    x = _rows(3, (64, 256), scale)
    y = oracle.quant_q8_0(x)
    d = y.reshape(64, 8, 34)[:, :, :2].copy().view(np.float16).astype(np.float32)            # [64, 8, 1]
    q = y.reshape(64, 8, 34)[:, :, 2:].view(np.int8)
    amax = np.abs(x.reshape(64, 8, 32)).max(-1, keepdims=True)
    # the largest element maps to +-127, nothing exceeds it, and the stored scale is amax/127 rounded to half
    assert np.abs(q).max(-1).min() == 127 and np.abs(q.astype(np.int32)).max() == 127
    assert np.array_equal(d, (amax / np.float32(127)).astype(np.float16).astype(np.float32))
    # |x - q * d_stored| <= d/2 from rounding q, plus 127 * |d - d_stored| from rounding d (2^-11 relative,
    # or half a subnormal step, 2^-25, for scales below the normal half range)
    dq = oracle.dequant_q8_0(y).reshape(64, 8, 32)
    bound = d * 0.5 + 127 * np.maximum(d * 2.0 ** -11, 2.0 ** -25)
    assert (np.abs(x.reshape(64, 8, 32) - dq) <= bound * 1.0001).all()
    # quantising the dequantised row again changes nothing
    assert np.array_equal(oracle.quant_q8_0(dq.reshape(64, 256)), y)
    # fp16 output is the fp32 output rounded once
    assert np.array_equal(oracle.dequant_q8_0(y, np.float16), oracle.dequant_q8_0(y).astype(np.float16))


def test_equals_reference_source_build():
    ref = oracle.ref_quants()
    if ref is None:
        pytest.skip("oracle/_ref/libref_quants.so not built (make -C oracle ref needs the reference tree)")
    quant, dequant32, dequant16 = ref
    for seed, scale in [(0, 1.0), (1, 1e-4), (2, 1e3), (3, 30.0)]:
        x = _rows(seed, (128, 512), scale)
        x[0, :32] = 0.0                                   # a zero block
        x[1, :8] = [0.5, -0.5, 1.5, -1.5, 2.5, 127.0, 63.5, -63.5]
        mine = oracle.quant_q8_0(x)
        theirs = quant(x)
        assert np.array_equal(mine, theirs)
        assert np.array_equal(oracle.dequant_q8_0(mine), dequant32(mine))
        assert np.array_equal(oracle.dequant_q8_0(mine, np.float16).view(np.uint16), dequant16(mine).view(np.uint16))
    # dequantisers agree on arbitrary bytes with finite scales as well
    g = np.random.default_rng(9)
    raw = g.integers(0, 256, (64, 4 * 34), dtype=np.uint8)
    sc = (g.standard_normal((64, 4)) * 0.05).astype(np.float16)
    raw.reshape(64, 4, 34)[:, :, :2] = sc.view(np.uint8).reshape(64, 4, 2)
    assert np.array_equal(oracle.dequant_q8_0(raw), dequant32(raw))
    assert np.array_equal(oracle.dequant_q8_0(raw, np.float16).view(np.uint16), dequant16(raw).view(np.uint16))


def test_decode_over_q8_caches_is_decode_over_dequantised_caches():
    g = np.random.default_rng(5)
    B, Hq, Hkv, Lmax, D = 2, 4, 2, 40, 64
    q = g.standard_normal((B, Hq, 1, D)).astype(np.float32)
    kq = oracle.quant_q8_0(g.standard_normal((B, Hkv, Lmax, D)).astype(np.float32))
    vq = oracle.quant_q8_0(g.standard_normal((B, Hkv, Lmax, D)).astype(np.float32))
    ctx = np.array([17, 40], np.int32)
    got = oracle.flash_attn_decode_q8_0(q, kq, vq, ctx)
    k16 = oracle.dequant_q8_0(kq).astype(np.float16)
    v16 = oracle.dequant_q8_0(vq).astype(np.float16)
    assert np.array_equal(got, oracle.flash_attn_decode(q, k16, v16, ctx))
