"""Pins oracle/quant.py: hand-computed rows that tell round-half-even from half-away, the clamps
of the scale and of the codes, the error bound of symmetric rounding, and bfloat16 rounding
against torch's own conversion."""
import numpy as np
import torch

from oracle import quant as Q


def test_known_rows():
    row = np.zeros(128, np.float32)
    row[:8] = [127, -127, 63.5, 62.5, -62.5, 0.4, -0.5, 1.5]           # max|x| = 127 -> scale exactly 1
    codes, scale = Q.quantize_rows(row[None])
    assert scale[0] == 1.0
    assert codes[0, :8].tolist() == [127, -127, 64, 62, -62, 0, 0, 2]   # ties go to the even code
    # all-zero row: scale clamps to 1e-5 and every code is 0
    codes, scale = Q.quantize_rows(np.zeros((1, 128), np.float32))
    assert scale[0] == np.float32(1e-5) and not codes.any()
    # huge row: scale clamps to 1e4, codes saturate at +127 / -128
    big = np.zeros((1, 128), np.float32); big[0, 0] = 3e6; big[0, 1] = -3e6; big[0, 2] = 5e3
    codes, scale = Q.quantize_rows(big)
    assert scale[0] == np.float32(1e4) and codes[0, :3].tolist() == [127, -128, 0]
    big[0, 2] = 1.5e4
    assert Q.quantize_rows(big)[0][0, 2] == 2                           # 1.5 -> 2 (even)


def test_error_bound_and_extremes():
    r = np.random.default_rng(0)
    x = (r.standard_normal((50, 4, 128)) * r.uniform(0.01, 30, (50, 4, 1))).astype(np.float32)
    codes, scale = Q.quantize_rows(x)
    assert codes.dtype == np.int8 and scale.dtype == np.float32 and scale.shape == (50, 4)
    err = np.abs(codes.astype(np.float64) * scale[..., None] - x)
    assert (err <= 0.5 * scale[..., None] * (1 + 1e-6)).all()           # nearest code
    assert (np.abs(codes).max(-1) == 127).all()                         # the largest entry maps to +-127
    np.testing.assert_array_equal(Q.quantize_rows(-x)[0], -codes)       # symmetric (no code hits -128 here)
    # scaling a row by a power of two scales the scale and leaves the codes alone
    c2, s2 = Q.quantize_rows(x * 4)
    np.testing.assert_array_equal(c2, codes); np.testing.assert_array_equal(s2, scale * 4)


def test_bf16_rounding_matches_torch():
    r = np.random.default_rng(1)
    x = (r.standard_normal(4096) * 10 ** r.uniform(-6, 6, 4096)).astype(np.float32)
    x[:4] = [1.00390625, 1.01171875, -1.00390625, 0.0]                  # ties: 1 + 2^-8 -> 1.0, 1 + 3*2^-8 -> 1.015625
    ref = torch.from_numpy(x).to(torch.bfloat16).float().numpy()
    np.testing.assert_array_equal(Q.round_to_bf16(x), ref)
    y = Q.quantize_sym(x[:128][None] , "bf16")
    assert np.array_equal(Q.round_to_bf16(y), y)                        # already bf16 values


def test_append_layout():
    r = np.random.default_rng(2)
    nb, bs, H, D = 4, 16, 4, 128
    kc = np.zeros((nb, bs, H, D), np.int8); vc = np.zeros_like(kc)
    ks = np.zeros((nb, H, bs), np.float32); vs = np.zeros_like(ks)
    k = r.standard_normal((3, H, D)).astype(np.float32); v = r.standard_normal((3, H, D)).astype(np.float32)
    Q.kv_append_int8(k, v, kc, vc, ks, vs, [17, -1, 63])
    c, s = Q.quantize_rows(k)
    np.testing.assert_array_equal(kc[1, 1], c[0]); np.testing.assert_array_equal(ks[1, :, 1], s[0])
    np.testing.assert_array_equal(kc[3, 15], c[2]); np.testing.assert_array_equal(ks[3, :, 15], s[2])
    assert np.count_nonzero(ks) == 2 * H and np.count_nonzero(vs) == 2 * H


def test_fp8_codes_known_values():
    """e4m3fn by hand: 1 sign, 4 exponent (bias 7), 3 mantissa bits; largest finite 448 = 0x7e; subnormal
    step 2^-9; ties to even; saturation instead of NaN beyond 464."""
    x = np.array([0.0, 1.0, -1.0, 448.0, 1000.0, -1e9, 2.0 ** -9, 2.0 ** -10, 1.5 * 2.0 ** -9, 1.0625, 1.1875, 17.0, 0.1],
                 np.float32)
    codes = Q.fp8_codes(x, 1.0)
    #                 0     1     -1    448   sat   -sat  min subnormal, tie->0, tie->2*2^-9, 1.0625->1.0, 1.1875->1.25, 17->16, 0.1
    assert codes.tolist() == [0x00, 0x38, 0xB8, 0x7E, 0x7E, 0xFE, 0x01, 0x00, 0x02, 0x38, 0x3A, 0x58, 0x1D]
    np.testing.assert_array_equal(Q.fp8_values(np.array([0x38, 0x7E, 0x01, 0x58], np.uint8), 2.0), [2.0, 896.0, 2.0 ** -8, 32.0])
    # scale: codes of x / scale; the round trip is idempotent
    y = Q.fp8_round(np.linspace(-30, 30, 64, dtype=np.float32), 0.25, "f32")
    np.testing.assert_array_equal(Q.fp8_round(y, 0.25, "f32"), y)
    assert np.isnan(Q.fp8_values(Q.fp8_codes(np.array([np.nan], np.float32), 1.0), 1.0)).all()
