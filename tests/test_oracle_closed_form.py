"""Pins the parts of the CPU oracle no reference-held vector covers.

Each check is chosen so a plausible slip (half-even instead of half-away, a
dropped zero point, multiply-vs-divide form, a transposed operand, a wrong
clamp range, NaN handling) fails it: hand-written tie/saturation vectors,
brute force in int64 / float64 with an independent formulation, invariants.
"""
import numpy as np
import pytest


def _round_half_away64(v):
    """Independent formulation in float64 (exact for f32 inputs)."""
    v = np.asarray(v, dtype=np.float64)
    return np.sign(v) * np.floor(np.abs(v) + 0.5)


def test_ties_round_half_away_by_default(oracle):
    x = np.array([0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 3.5, -3.5, 0.49999997, 126.5, 127.5, -127.5, -128.5], np.float32)
    want = np.array([1, 2, 3, -1, -2, -3, 4, -4, 0, 127, 127, -128, -128], np.float32)
    np.testing.assert_array_equal(oracle.quantize_per_tensor_affine(x, 1.0, 0), want)
    np.testing.assert_array_equal(oracle.quantize_per_tensor_affine_i8(x, 1.0, 0), want.astype(np.int8))
    big = np.tile(x, 10)  # len > 64 -> multiply-by-inverse branch
    np.testing.assert_array_equal(oracle.quantize_per_tensor_affine(big, 1.0, 0), np.tile(want, 10))


def test_half_even_mode_differs_only_on_ties(oracle):
    x = np.array([0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 0.75, -0.25], np.float32)
    oracle.set_round_mode(oracle.ROUND_HALF_EVEN)
    try:
        got = oracle.quantize_per_tensor_affine(x, 1.0, 0)
    finally:
        oracle.set_round_mode(oracle.ROUND_HALF_AWAY)
    np.testing.assert_array_equal(got, np.array([0, 2, 2, -0.0, -2, -2, 1, -0.0], np.float32))


def test_zero_point_added_after_rounding(oracle):
    # round(0.5)+3 = 4 (half away) whereas round(0.5+3)=4 too; use -0.5: round(-0.5)+3 = 2, round(2.5)=3
    assert oracle.quantize_per_tensor_affine(np.array([-0.5], np.float32), 1.0, 3)[0] == 2.0
    # torsh-core scalar types add the zero point BEFORE rounding
    assert oracle.qint8_quantize(-0.5, 1.0, 3) == 3


def test_clamp_is_i8_range_even_for_large_zero_point(oracle):
    x = np.array([100.0, -100.0, 0.0], np.float32)
    np.testing.assert_array_equal(oracle.quantize_per_tensor_affine(x, 1.0, 100), [127, 0, 100])
    np.testing.assert_array_equal(oracle.quantize_per_tensor_affine(x, 1.0, -100), [0, -128, -100])


def test_nan_and_inf(oracle):
    x = np.array([np.nan, np.inf, -np.inf, 1.0], np.float32)
    carrier = oracle.quantize_per_tensor_affine(x, 0.5, 0)
    assert np.isnan(carrier[0]) and carrier[1] == 127 and carrier[2] == -128 and carrier[3] == 2
    np.testing.assert_array_equal(oracle.quantize_per_tensor_affine_i8(x, 0.5, 0), [0, 127, -128, 2])
    # NaN-ignoring min/max (Rust f32::min/max)
    assert oracle.find_min_max(np.array([np.nan, 1.0, -2.0], np.float32)) == (-2.0, 1.0)
    with pytest.raises(oracle.OracleError):
        oracle.quantize_tensor_auto(np.array([1.0, np.inf], np.float32), 0, oracle.PER_TENSOR_SYMMETRIC)


def test_mul_inverse_vs_divide_forms_are_both_exactly_what_they_say(oracle):
    rng = np.random.default_rng(11)
    x = rng.standard_normal(4096).astype(np.float32) * 3
    for scale in (np.float32(0.0123), np.float32(0.1), np.float32(1 / 3)):
        inv = np.float32(1.0) / scale
        want_mul = np.clip(_round_half_away64(x * inv) + 7, -128, 127).astype(np.float32)
        want_div = np.clip(_round_half_away64(x / scale) + 7, -128, 127).astype(np.float32)
        np.testing.assert_array_equal(oracle.quantize_per_tensor_affine_simd(x, scale, 7), want_mul)
        np.testing.assert_array_equal(oracle.quantize_per_tensor_affine(x[:64], scale, 7), want_div[:64])
        np.testing.assert_array_equal(oracle.quantize_per_tensor_affine(x, scale, 7), want_mul)
        np.testing.assert_array_equal(oracle.quantize_per_tensor_affine_i8(x, scale, 7), want_div.astype(np.int8))


def test_symmetric_scale_is_absmax_over_qmax(oracle):
    s, z = oracle.calculate_symmetric_params(-3.0, 2.0, 0)
    assert s == np.float32(3.0) / np.float32(127.0) and z == 0
    s, _ = oracle.calculate_symmetric_params(-3.0, 2.0, 1)  # U8 -> qmax 255
    assert s == np.float32(3.0) / np.float32(255.0)
    # below f32::EPSILON -> (1.0, 0)
    assert oracle.calculate_symmetric_params(-1e-8, 1e-8, 0) == (1.0, 0)


def test_affine_params_closed_form(oracle):
    s, z = oracle.calculate_affine_params(-1.0, 3.0, 1)  # U8
    assert s == np.float32(4.0) / np.float32(255.0)
    assert z == int(_round_half_away64(np.float32(0.0) - np.float32(-1.0) / np.float32(s)))
    s, z = oracle.calculate_affine_params(0.0, 2.55, 1)
    assert z == 0
    # range is NOT widened to include zero: all-positive data maps min -> qmin
    s, z = oracle.calculate_affine_params(1.0, 2.0, 0)
    assert z == -128  # clamp(round(-128 - 1/(1/255))) = clamp(-383) = -128


def test_round_trip_config1_shape_properties(oracle):
    rng = np.random.default_rng(1)
    x = rng.standard_normal((256, 256)).astype(np.float32)
    q, s, z = oracle.quantize_tensor_auto(x, 0, oracle.PER_TENSOR_SYMMETRIC)
    assert z == 0 and s == np.abs(x).max() / np.float32(127.0)
    assert q.min() >= -127 and q.max() <= 127 and np.abs(q).max() == 127
    y = oracle.dequantize_per_tensor_affine(q, s, z)
    assert np.abs(y - x).max() <= 0.5 * s * (1 + 1e-6)
    np.testing.assert_array_equal(y, q * np.float32(s))


def test_per_channel_auto_matches_row_wise_formula(oracle):
    rng = np.random.default_rng(5)
    w = (rng.standard_normal((7, 33)) * 0.02).astype(np.float32)
    w[3] = 0  # degenerate channel -> scale 1.0
    q, scales, zps = oracle.quantize_per_channel_auto(w, 0, 0, oracle.PER_CHANNEL_SYMMETRIC)
    for r in range(7):
        am = np.abs(w[r]).max()
        s = np.float32(1.0) if am < np.finfo(np.float32).eps else am / np.float32(127.0)
        assert scales[r] == s and zps[r] == 0
        np.testing.assert_array_equal(q[r], np.clip(_round_half_away64(w[r] / s), -128, 127).astype(np.float32))


def test_per_channel_auto_other_axes(oracle):
    rng = np.random.default_rng(6)
    x = rng.standard_normal((3, 4, 5)).astype(np.float32)
    for axis in range(3):
        q, scales, zps = oracle.quantize_per_channel_auto(x, axis, 0, oracle.PER_CHANNEL_SYMMETRIC)
        xm = np.moveaxis(x, axis, 0).reshape(x.shape[axis], -1)
        qm = np.moveaxis(q, axis, 0).reshape(x.shape[axis], -1)
        for c in range(x.shape[axis]):
            s = np.abs(xm[c]).max() / np.float32(127.0)
            assert scales[c] == s
            np.testing.assert_array_equal(qm[c], np.clip(_round_half_away64(xm[c] / s), -128, 127))
    with pytest.raises(oracle.OracleError):
        oracle.quantize_per_channel_auto(x, 3, 0, oracle.PER_CHANNEL_SYMMETRIC)


def test_per_channel_explicit_params(oracle):
    rng = np.random.default_rng(7)
    x = rng.standard_normal((4, 6)).astype(np.float32)
    scales = np.array([0.01, 0.02, 0.05, 0.1], np.float32)
    zps = np.array([0, 3, -5, 10], np.int32)
    q = oracle.quantize_per_channel_affine(x, scales, zps, 0)
    want = np.clip(_round_half_away64(x / scales[:, None]) + zps[:, None], -128, 127)
    np.testing.assert_array_equal(q, want.astype(np.float32))
    y = oracle.dequantize_per_channel_affine(q, scales, zps, 0)
    np.testing.assert_array_equal(y, scales[:, None] * (q - zps[:, None].astype(np.float32)))
    q1 = oracle.quantize_per_channel_affine(x, scales[:1].repeat(6), np.zeros(6, np.int32), 1)
    np.testing.assert_array_equal(q1, np.clip(_round_half_away64(x / scales[0]), -128, 127))
    qs = oracle.quantize_per_channel_simd(x, scales, zps, 6)
    inv = np.float32(1.0) / scales
    np.testing.assert_array_equal(qs, np.clip(_round_half_away64(x * inv[:, None]) + zps[:, None], -128, 127))


def test_backend_flavour(oracle):
    # symmetric scale is 2*absmax/(qmax-qmin) = absmax/127.5, not absmax/127
    s, z = oracle.backend_params_symmetric(-2.0, 1.0, -128, 127)
    assert s == np.float32(4.0) / np.float32(255.0) and z == 0
    assert oracle.backend_params_symmetric(0.0, 0.0) == (1.0, 0)
    s, z = oracle.backend_params_asymmetric(0.0, 5.1, 0, 255)
    assert s == np.float32(5.1) / np.float32(255.0) and z == 0
    assert oracle.backend_params_asymmetric(2.0, 2.0, 0, 255) == (1.0, 0)
    with pytest.raises(oracle.OracleError):
        oracle.backend_params_asymmetric(2.0, 1.0, 0, 255)
    x = np.array([0.0, 0.5, 1.0, 300.0, -1.0, 2.5], np.float32)
    np.testing.assert_array_equal(oracle.backend_quantize_f32(x, 1.0, 0, 0, 255), [0, 1, 1, 255, 0, 3])
    # int8 stored as two's-complement bytes
    np.testing.assert_array_equal(oracle.backend_quantize_f32(x, 1.0, 0, -128, 127), [0, 1, 1, 127, 255, 3])
    np.testing.assert_array_equal(oracle.backend_dequantize_f32(np.array([255, 2], np.uint8), 0.5, 0, True), [-0.5, 1.0])
    np.testing.assert_array_equal(oracle.backend_dequantize_f32(np.array([255, 2], np.uint8), 0.5, 1, False), [127.0, 0.5])
    # ChannelWise = contiguous equal chunks
    q = oracle.backend_quantize_f32(np.array([1, 2, 3, 4], np.float32), [1.0, 0.5], [0, 1], 0, 255)
    np.testing.assert_array_equal(q, [1, 2, 7, 9])


def test_nn_flavour(oracle):
    assert oracle.nn_quantize_value_symmetric(2.5, 1.0) == 3
    assert oracle.nn_quantize_value_symmetric(-2.5, 1.0) == -3
    assert oracle.nn_quantize_value_symmetric(1e9, 1.0) == 127
    assert oracle.nn_quantize_value_asymmetric(-0.5, 1.0, 3, 0, 255) == 2
    assert oracle.nn_dequantize_value_asymmetric(5, 0.5, 3) == 1.0
    w = np.array([[1.0, -2.0, 0.5], [0.1, 0.2, -0.05]], np.float32)
    q, s = oracle.nn_per_channel_quantize_weights_sym_i8(w)
    assert s[0] == np.float32(2.0) / np.float32(127.0) and s[1] == np.float32(0.2) / np.float32(127.0)
    # negatives are carried as the two's-complement byte widened to f32
    np.testing.assert_array_equal(q[0], [64, 256 - 127, 32])
    # an all-zero channel: no zero guard, scale 0, 0/0 = NaN -> `as i32` 0
    q, s = oracle.nn_per_channel_quantize_weights_sym_i8(np.zeros((1, 4), np.float32))
    assert s[0] == 0.0 and (q == 0).all()
    # asymmetric uint8 arm by hand: channel [-1, 0, 1.55]: scale 2.55/255 = 0.01, zp = round(1/0.01) = 100,
    # codes round(v/0.01) + 100 = 0, 100, 255; channel [2, 4]: scale 2/255, zp = round(-2/scale) = -255 (not
    # clamped), codes clamp(255 - 255, 0, 255) = 0 and clamp(510 - 255) = 255
    q, s, z = oracle.nn_per_channel_quantize_weights_asym_u8(np.float32([[-1.0, 0.0, 1.55]]))
    assert s[0] == np.float32(2.55) / np.float32(255.0) and z[0] == 100
    np.testing.assert_array_equal(q[0], [0, 100, 255])
    q, s, z = oracle.nn_per_channel_quantize_weights_asym_u8(np.float32([[2.0, 4.0]]))
    assert z[0] == -255
    np.testing.assert_array_equal(q[0], [0, 255])
    # the scalar quantized types (zero point before rounding), unsigned: round(-2.5 + 5) = 3, not round(-2.5) + 5 = 2
    assert oracle.quint8_quantize(-2.5, 1.0, 5) == 3
    assert oracle.quint8_quantize(1000.0, 1.0, 5) == 255 and oracle.quint8_quantize(-1000.0, 1.0, 5) == 0


def test_int_gemm_vs_int64_bruteforce(oracle):
    rng = np.random.default_rng(3)
    for (m, k, n) in [(1, 1, 1), (3, 5, 7), (16, 64, 16), (33, 129, 65)]:
        a = rng.integers(-128, 128, size=(m, k), dtype=np.int8)
        b = rng.integers(-128, 128, size=(k, n), dtype=np.int8)  # reference layout [K,N]
        want = a.astype(np.int64) @ b.astype(np.int64)
        acc, clamped = oracle.backend_matmul_i32(a, b)
        np.testing.assert_array_equal(acc, want)
        np.testing.assert_array_equal(clamped.view(np.int8), np.clip(want, -128, 127).astype(np.int8))
        # [N,K] weight form used by the device kernels: same integers
        np.testing.assert_array_equal(oracle.gemm_i8_nk(a, np.ascontiguousarray(b.T)), want)
    # asymmetry check: A@B != B@A shape/values, catches a transposed operand
    a = np.array([[1, 2], [3, 4]], np.int8)
    b = np.array([[0, 1], [1, 0]], np.int8)
    np.testing.assert_array_equal(oracle.backend_matmul_i32(a, b)[0], [[2, 1], [4, 3]])
    # extreme values: K * 128 * 128 stays inside i32 for K = 4096
    a = np.full((2, 4096), -128, np.int8)
    np.testing.assert_array_equal(oracle.gemm_i8_nk(a, a), np.full((2, 2), 4096 * 16384, np.int64))


def _conv_bruteforce(x, zp, w, stride, pad):
    nb, c, h, wd = x.shape
    oc, _, kh, kw = w.shape
    xp = np.zeros((nb, c, h + 2 * pad[0], wd + 2 * pad[1]), np.int64)
    xp[:, :, pad[0]:pad[0] + h, pad[1]:pad[1] + wd] = x.astype(np.int64) - zp  # padding = real 0 = (zp - zp)
    ho = (h + 2 * pad[0] - kh) // stride[0] + 1
    wo = (wd + 2 * pad[1] - kw) // stride[1] + 1
    out = np.zeros((nb, oc, ho, wo), np.int64)
    for i in range(ho):
        for j in range(wo):
            patch = xp[:, :, i * stride[0]:i * stride[0] + kh, j * stride[1]:j * stride[1] + kw]
            out[:, :, i, j] = np.einsum("nchw,ochw->no", patch, w.astype(np.int64))
    return out


def test_int_conv_vs_bruteforce(oracle):
    rng = np.random.default_rng(4)
    for (nb, c, h, wd, oc, k, stride, pad, zp) in [
        (1, 1, 3, 3, 1, 3, (1, 1), (1, 1), 0),
        (2, 3, 5, 6, 4, 3, (1, 1), (1, 1), 7),
        (1, 2, 7, 7, 3, 3, (2, 2), (0, 0), 128),
        (2, 4, 6, 5, 2, 1, (1, 1), (0, 0), 3),
        (1, 2, 8, 8, 2, 5, (1, 2), (2, 1), 11),
    ]:
        x = rng.integers(0, 256, size=(nb, c, h, wd), dtype=np.uint8)
        w = rng.integers(-128, 128, size=(oc, c, k, k), dtype=np.int8)
        got = oracle.backend_conv2d_i32(x, zp, w, stride, pad)
        np.testing.assert_array_equal(got, _conv_bruteforce(x, zp, w, stride, pad))
    # 1x1 ones kernel on ones input (the shape of the reference's qconv smoke test)
    got = oracle.backend_conv2d_i32(np.ones((1, 1, 3, 3), np.uint8), 0, np.ones((1, 1, 1, 1), np.int8))
    np.testing.assert_array_equal(got, np.ones((1, 1, 3, 3)))


def test_linear_epilogue_closed_form(oracle):
    rng = np.random.default_rng(8)
    acc = rng.integers(-2_000_000, 2_000_000, size=(5, 9), dtype=np.int32)
    sw = rng.uniform(1e-4, 1e-2, 9).astype(np.float32)
    bias = rng.standard_normal(9).astype(np.float32) * 0.01
    for sa in (np.float32(0.031), rng.uniform(0.01, 0.05, 5).astype(np.float32)):
        got = oracle.linear_dequant_epilogue(acc, sa, sw, bias)
        sa_col = np.atleast_1d(sa).astype(np.float32).reshape(-1, 1)
        s = (sa_col * sw[None, :]).astype(np.float32)           # f32 product, rounded once
        want32 = (acc.astype(np.float32) * s).astype(np.float32) + bias[None, :]
        np.testing.assert_array_equal(got, want32.astype(np.float32))
        want64 = acc.astype(np.float64) * sa_col.astype(np.float64) * sw.astype(np.float64) + bias
        np.testing.assert_allclose(got, want64, rtol=1e-5, atol=1e-6)
    np.testing.assert_array_equal(oracle.linear_dequant_epilogue(acc, 0.5, sw, None),
                                  acc.astype(np.float32) * (np.float32(0.5) * sw)[None, :])


def test_requantize_epilogue_closed_form(oracle):
    rng = np.random.default_rng(9)
    acc = rng.integers(-50_000, 50_000, size=(6, 10), dtype=np.int32)
    sw = rng.uniform(1e-4, 1e-3, 10).astype(np.float32)
    bias = rng.standard_normal(10).astype(np.float32) * 0.01
    sa, s_out, zp_out = np.float32(0.02), np.float32(0.0071), -3
    got = oracle.requantize_epilogue(acc, sa, sw, bias, s_out, zp_out)
    v = (acc.astype(np.float32) * (sa * sw)[None, :]).astype(np.float32) + bias[None, :]
    want = np.clip(_round_half_away64((v / s_out).astype(np.float32)) + zp_out, -128, 127)
    np.testing.assert_array_equal(got, want.astype(np.int8))
    # channel on the row axis (NCHW conv output viewed [nb*c_out, ho*wo])
    sw_r = rng.uniform(1e-4, 1e-3, 3).astype(np.float32)
    b_r = rng.standard_normal(3).astype(np.float32) * 0.01
    got = oracle.requantize_epilogue(acc, sa, sw_r, b_r, s_out, zp_out, channel_axis_is_row=True, inner=3)
    ch = np.arange(6) % 3
    v = (acc.astype(np.float32) * (sa * sw_r)[ch][:, None]).astype(np.float32) + b_r[ch][:, None]
    want = np.clip(_round_half_away64((v / s_out).astype(np.float32)) + zp_out, -128, 127)
    np.testing.assert_array_equal(got, want.astype(np.int8))


def test_layer_norm_and_gelu(oracle):
    rng = np.random.default_rng(10)
    x = rng.standard_normal((4, 96)).astype(np.float32)
    y = oracle.layer_norm(x, None, None, 1e-5)
    np.testing.assert_allclose(y.mean(axis=1), 0, atol=1e-6)
    np.testing.assert_allclose(y.var(axis=1), 1, rtol=1e-4)
    g = oracle.gelu_tanh(np.array([0.0, 1.0, -1.0, 3.0], np.float32))
    np.testing.assert_allclose(g, [0.0, 0.841192, -0.158808, 2.996363], atol=1e-6)


def test_layer_norm_with_affine_parameters_and_large_eps(oracle):
    """crates/torsh-nn/src/layers/normalization/common.rs:389-404: (x - mean) / sqrt(var + eps) * weight + bias with
    the biased variance.  Random gamma and beta and an eps of the size of the variance, so that a dropped beta,
    gamma applied after beta, eps outside the square root or the unbiased variance would each miss by far more
    than the tolerance; a hand-computed row on top."""
    rng = np.random.default_rng(11)
    x = (rng.standard_normal((5, 48)) * rng.uniform(0.5, 3.0, (5, 1)) + rng.uniform(-2, 2, (5, 1))).astype(np.float32)
    gamma = rng.uniform(0.5, 2.0, 48).astype(np.float32)
    beta = rng.uniform(-1.0, 1.0, 48).astype(np.float32)
    for eps in (0.5, 1e-5):
        x64 = x.astype(np.float64)
        mean = x64.mean(axis=1, keepdims=True)
        var = ((x64 - mean) ** 2).mean(axis=1, keepdims=True)          # biased: divides by the row length
        want = (x64 - mean) / np.sqrt(var + eps) * gamma.astype(np.float64) + beta.astype(np.float64)
        np.testing.assert_allclose(oracle.layer_norm(x, gamma, beta, eps), want, rtol=2e-6, atol=2e-6)
        np.testing.assert_allclose(oracle.layer_norm(x, gamma, None, eps), want - beta, rtol=2e-6, atol=2e-6)
        np.testing.assert_allclose(oracle.layer_norm(x, None, beta, eps),
                                   (x64 - mean) / np.sqrt(var + eps) + beta, rtol=2e-6, atol=2e-6)
    # the wrong formulas really are far away at eps = 0.5 (the check above is not vacuous)
    x64 = x.astype(np.float64)
    mean = x64.mean(axis=1, keepdims=True)
    var = ((x64 - mean) ** 2).mean(axis=1, keepdims=True)
    good = (x64 - mean) / np.sqrt(var + 0.5) * gamma + beta
    for wrong in ((x64 - mean) / (np.sqrt(var) + 0.5) * gamma + beta,              # eps outside the square root
                  ((x64 - mean) / np.sqrt(var + 0.5) + beta) * gamma,              # gamma after beta
                  (x64 - mean) / np.sqrt(var * 48 / 47 + 0.5) * gamma + beta):     # unbiased variance
        assert np.abs(wrong - good).max() > 1e-2
    # by hand: row [1, 2, 3, 6]: mean 3, biased variance 3.5, eps 0.5 -> divide by 2
    y = oracle.layer_norm(np.float32([[1, 2, 3, 6]]), np.float32([1, 2, 3, 4]), np.float32([0.5, 0.5, -1, 0]), 0.5)
    np.testing.assert_allclose(y, [[-0.5, -0.5, -1.0, 6.0]], rtol=0, atol=1e-6)


def test_determinism(oracle):
    rng = np.random.default_rng(12)
    x = rng.standard_normal(100_000).astype(np.float32)
    a = oracle.quantize_tensor_auto(x, 0, oracle.PER_TENSOR_SYMMETRIC)
    b = oracle.quantize_tensor_auto(x, 0, oracle.PER_TENSOR_SYMMETRIC)
    np.testing.assert_array_equal(a[0], b[0])
    assert a[1:] == b[1:]


def test_backend_qadd_qrelu_closed_form(oracle):
    # bytes 10, 20, -30, 40 at scale 0.1 are 1, 2, -3, 4; bytes 1..4 at scale 0.5 are 0.5 .. 2.
    a, b = np.int8([10, 20, -30, 40]), np.int8([1, 2, 3, 4])
    out, s, z = oracle.backend_qadd(a, 0.1, 0, b, 0.5, 0)
    # sum = [1.5, 3, -1.5, 6]: scale = 7.5 / 255, zero point = round(-128 + 1.5 / scale) = round(-77) = -77
    assert s == np.float32(7.5) / np.float32(255.0) and z == -77
    np.testing.assert_array_equal(out, [-26, 25, -128, 127])
    # qrelu: [1, 2, 0, 4] with range (0, 4): scale 4 / 255, zero point -128
    out, s, z = oracle.backend_qrelu(a, 0.1, 0)
    assert s == np.float32(4.0) / np.float32(255.0) and z == -128
    np.testing.assert_array_equal(out, [-64, -1, -128, 127])       # round(63.75) - 128, round(127.5) - 128
    # symmetric scheme: scale = 2 * max|v| / 255, zero point 0
    out, s, z = oracle.backend_qadd(a, 0.1, 0, b, 0.5, 0, symmetric=True)
    assert s == np.float32(12.0) / np.float32(255.0) and z == 0
    # uint8 storage with a zero point, all-negative input to relu -> degenerate range (0, 0) -> (1.0, qmin)
    out, s, z = oracle.backend_qrelu(np.uint8([0, 50, 100]), 0.02, 128)
    assert (s, z) == (1.0, 0) and (out == 0).all()
