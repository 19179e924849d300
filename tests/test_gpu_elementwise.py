"""Parity of the HBM-streaming kernels (through the C-ABI) with the CPU oracle: bit-exact."""
import json
import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


def normal(seed, shape, std=1.0):
    return (np.random.default_rng(seed).standard_normal(shape) * std).astype(np.float32)


def test_golden_vectors_through_the_cabi(ctx, hipq, golden):
    for case in golden["quantize_per_tensor"] + golden["proptest_regressions"]:
        x = np.array(case["x"], np.float32)
        want = np.array(case["q"], np.int8)[: x.size]
        for mode in (hipq.FORM_MUL_INV, hipq.FORM_DIV):
            got = host(ctx.quantize_per_tensor_i8(dev(x), case["scale"], case["zp"], mode))
            np.testing.assert_array_equal(got, want, case["src"])
    for case in golden["dequantize_per_tensor"]:
        q = np.array(case["q"], np.float32)
        got = host(ctx.dequantize(dev(q), case["scale"], case["zp"]))
        np.testing.assert_allclose(got, np.array(case["y"], np.float32), atol=case["atol"], rtol=0)
    for case in golden["min_max"]:
        got = host(ctx.minmax(dev(np.array(case["x"], np.float32))))
        assert got[0] == np.float32(case["min"]) and got[1] == np.float32(case["max"])


def test_error_cases_match_the_reference(ctx, hipq):
    x = dev(np.array([1.0, 2.0], np.float32))
    for bad in (-1.0, 0.0):
        with pytest.raises(hipq.HipqError) as e:
            ctx.quantize_per_tensor_i8(x, bad, 0)
        assert e.value.code == hipq.INVALID_ARGUMENT and "Scale must be positive" in e.value.message
        with pytest.raises(hipq.HipqError):
            ctx.dequantize(x, bad, 0)
    with pytest.raises(hipq.HipqError) as e:
        ctx.minmax(torch.empty(0, dtype=torch.float32, device="cuda"))
    assert e.value.code == hipq.INVALID_ARGUMENT
    with pytest.raises(hipq.HipqError):
        ctx.quantize_dynamic_per_tensor(torch.empty(0, dtype=torch.float32, device="cuda"))
    with pytest.raises(hipq.HipqError):
        ctx.quantize_per_tensor_i8(x, 1.0, 0, mode=64)
    # empty input with a valid scale is a no-op, as the reference's loop over zero elements
    ctx.quantize_per_tensor_i8(torch.empty(0, dtype=torch.float32, device="cuda"), 1.0, 0)


@pytest.mark.parametrize("n", [1, 3, 63, 64, 65, 1000, 4096, 4097, 65536 + 5, 1 << 20])
def test_minmax_absmax(ctx, oracle, n):
    x = normal(n, n) * 3
    got = host(ctx.minmax(dev(x)))
    mn, mx = oracle.find_min_max(x)
    assert (got[0], got[1]) == (np.float32(mn), np.float32(mx))
    assert host(ctx.absmax(dev(x)))[0] == np.float32(max(abs(mn), abs(mx)))


def test_minmax_ignores_nan_and_handles_unaligned(ctx, oracle):
    x = normal(7, 5000)
    x[17] = np.nan
    x[4000] = np.nan
    t = dev(x)
    got = host(ctx.minmax(t))
    assert tuple(got) == tuple(np.float32(v) for v in oracle.find_min_max(x))
    got = host(ctx.minmax(t[1:]))  # base pointer no longer 16-byte aligned
    assert tuple(got) == tuple(np.float32(v) for v in oracle.find_min_max(x[1:]))


@pytest.mark.parametrize("n", [1, 5, 64, 65, 4095, 4096, 100_003, 1 << 20])
@pytest.mark.parametrize("mode_name", ["mul", "div", "mul_even", "div_even"])
def test_quantize_per_tensor_bit_exact(ctx, hipq, oracle, n, mode_name):
    x = normal(100 + n, n) * 2
    # plant exact ties and saturating values
    x[: min(n, 6)] = np.array([0.5, -0.5, 1.5, -2.5, 1000.0, -1000.0], np.float32)[: min(n, 6)]
    scale, zp = np.float32(0.03125 if n % 2 else 0.0173), 3
    x[: min(n, 4)] *= scale  # ties in units of the scale when scale is a power of two
    mode = (hipq.FORM_DIV if "div" in mode_name else 0) | (hipq.ROUND_HALF_EVEN if "even" in mode_name else 0)
    oracle.set_round_mode(1 if "even" in mode_name else 0)
    try:
        if "div" in mode_name:
            want = oracle.quantize_per_tensor_affine_i8(x, scale, zp)
        else:
            want = oracle.quantize_to_int8_simd(x, scale, zp)
        want_carrier = oracle.quantize_per_tensor_affine_simd(x, scale, zp) if "div" not in mode_name else None
    finally:
        oracle.set_round_mode(0)
    got = host(ctx.quantize_per_tensor_i8(dev(x), scale, zp, mode))
    np.testing.assert_array_equal(got, want)
    if want_carrier is not None:
        got_c = host(ctx.quantize_per_tensor_carrier(dev(x), scale, zp, mode))
        np.testing.assert_array_equal(got_c, want_carrier)


def test_quantize_ties_follow_the_rounding_mode(ctx, hipq):
    x = dev(np.array([0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 126.5, 127.5, -128.5], np.float32))
    away = host(ctx.quantize_per_tensor_i8(x, 1.0, 0, hipq.ROUND_HALF_AWAY))
    even = host(ctx.quantize_per_tensor_i8(x, 1.0, 0, hipq.ROUND_HALF_EVEN))
    np.testing.assert_array_equal(away, [1, 2, 3, -1, -2, -3, 127, 127, -128])
    np.testing.assert_array_equal(even, [0, 2, 2, 0, -2, -2, 126, 127, -128])


def test_quantize_nan_inf(ctx, oracle):
    x = np.array([np.nan, np.inf, -np.inf, 1.0, -3.0] * 30, np.float32)
    got = host(ctx.quantize_per_tensor_i8(dev(x), 0.5, 0))
    np.testing.assert_array_equal(got, oracle.quantize_to_int8_simd(x, 0.5, 0))
    car = host(ctx.quantize_per_tensor_carrier(dev(x), 0.5, 0))
    want = oracle.quantize_per_tensor_affine_simd(x, 0.5, 0)
    np.testing.assert_array_equal(np.isnan(car), np.isnan(want))
    np.testing.assert_array_equal(car[~np.isnan(car)], want[~np.isnan(want)])


def test_quantize_unaligned_views(ctx, oracle):
    x = normal(5, 10_007)
    t = dev(x)
    out = torch.empty(10_007 + 8, dtype=torch.int8, device="cuda")
    for off_in, off_out in [(1, 0), (0, 1), (3, 2), (2, 3)]:
        ctx.quantize_per_tensor_i8(t[off_in:], 0.02, -1, out=out[off_out: off_out + x.size - off_in])
        got = host(out[off_out: off_out + x.size - off_in])
        np.testing.assert_array_equal(got, oracle.quantize_to_int8_simd(x[off_in:], 0.02, -1))


@pytest.mark.parametrize("n", [2, 64, 65, 4096, 1 << 20, (1 << 20) + 7])
def test_u8_quantize_backend_flavour(ctx, hipq, oracle, n):
    x = np.maximum(normal(n, n), 0)
    mn, mx = oracle.find_min_max(x)
    scale, zp = oracle.backend_params_asymmetric(mn, mx, 0, 255)
    want = oracle.backend_quantize_f32(x, scale, zp, 0, 255)
    got = host(ctx.quantize_per_tensor_u8(dev(x), scale, zp, hipq.FORM_DIV))
    np.testing.assert_array_equal(got, want)
    # fully on-device: min/max -> asymmetric params -> quantize
    q, params = ctx.quantize_dynamic_per_tensor(dev(x), hipq.PARAMS_BACKEND_ASYMMETRIC, hipq.DTYPE_U8, hipq.FORM_DIV)
    p = ctx.read_qparams(params)
    assert p.status == 0 and p.scale == np.float32(scale) and p.zero_point == zp
    np.testing.assert_array_equal(host(q), want)
    deq = host(ctx.dequantize(q, scale, zp))
    np.testing.assert_array_equal(deq, oracle.backend_dequantize_f32(want, scale, zp, False))


@pytest.mark.parametrize("flavor_name", ["symmetric", "affine", "backend_symmetric", "backend_asymmetric"])
def test_qparams_from_minmax(ctx, hipq, oracle, flavor_name):
    cases = [(-1.0, 1.0), (0.0, 0.0), (1.0, 1.0), (-3.5, 0.25), (0.0, 6.0), (1.0, 2.0), (-1e-9, 1e-9), (2.0, 1.0),
             (float("nan"), 1.0), (0.0, float("inf"))]
    flavor = {"symmetric": hipq.PARAMS_SYMMETRIC, "affine": hipq.PARAMS_AFFINE,
              "backend_symmetric": hipq.PARAMS_BACKEND_SYMMETRIC,
              "backend_asymmetric": hipq.PARAMS_BACKEND_ASYMMETRIC}[flavor_name]
    for qmin, qmax, dt in ((-128, 127, 0), (0, 255, 1)):
        for mn, mx in cases:
            p = ctx.read_qparams(ctx.qparams_from_minmax(dev(np.array([mn, mx], np.float32)), flavor, qmin, qmax))
            try:
                if flavor_name == "symmetric":
                    want = oracle.calculate_symmetric_params(mn, mx, dt)
                elif flavor_name == "affine":
                    want = oracle.calculate_affine_params(mn, mx, dt)
                elif flavor_name == "backend_symmetric":
                    want = oracle.backend_params_symmetric(mn, mx, qmin, qmax)
                else:
                    want = oracle.backend_params_asymmetric(mn, mx, qmin, qmax)
            except oracle.OracleError:
                assert p.status == hipq.INVALID_ARGUMENT, (flavor_name, mn, mx)
                continue
            assert p.status == 0 and (p.scale, p.zero_point) == (np.float32(want[0]), want[1]), (flavor_name, mn, mx)


@pytest.mark.parametrize("shape", [(4, 4), (256, 256), (1000, 37), (1024, 1024)])
def test_config1_round_trip(ctx, hipq, oracle, shape):
    """Symmetric per-tensor int8 quantize -> dequantize of N(0,1) data (the round-trip configuration at small sizes)."""
    x = normal(1, shape)
    want_q, scale, zp = oracle.quantize_tensor_auto(x, 0, oracle.PER_TENSOR_SYMMETRIC)
    want_y = oracle.dequantize_per_tensor_affine(want_q, scale, zp)
    mode = hipq.FORM_MUL_INV if x.size > 64 else hipq.FORM_DIV  # the reference's len > 64 branch
    q, params = ctx.quantize_dynamic_per_tensor(dev(x), hipq.PARAMS_SYMMETRIC, hipq.DTYPE_I8, mode)
    p = ctx.read_qparams(params)
    assert p.status == 0 and p.scale == np.float32(scale) and p.zero_point == zp
    np.testing.assert_array_equal(host(q), want_q.astype(np.int8))
    y = host(ctx.dequantize_with_params(q, params))
    np.testing.assert_array_equal(y, want_y)  # (q - 0) * scale has one rounding: bit-exact
    np.testing.assert_allclose(y, want_y, rtol=1e-5, atol=0)
    assert np.abs(y - x).max() <= 0.5 * scale * (1 + 1e-4)


def test_config1_full_size_properties(ctx, hipq):
    """Full size [4096,4096]: size-independent properties instead of a CPU pass."""
    g = torch.Generator(device="cuda").manual_seed(1)
    x = torch.randn(4096, 4096, generator=g, device="cuda", dtype=torch.float32)
    q, params = ctx.quantize_dynamic_per_tensor(x, hipq.PARAMS_SYMMETRIC, hipq.DTYPE_I8, hipq.FORM_MUL_INV)
    p = ctx.read_qparams(params)
    absmax = x.abs().max().item()
    assert p.status == 0 and p.zero_point == 0
    assert p.scale == np.float32(absmax) / np.float32(127.0)
    assert (p.min_val, p.max_val) == (x.min().item(), x.max().item())
    assert int(q.abs().max().item()) == 127 and int(q.min().item()) >= -127
    y = ctx.dequantize_with_params(q, params)
    torch.cuda.synchronize()
    assert (y - x).abs().max().item() <= 0.5 * p.scale * (1 + 1e-4)
    # idempotence: quantizing the dequantized tensor with the same scale returns the same codes
    q2 = ctx.quantize_per_tensor_i8(y, p.scale, 0, hipq.FORM_MUL_INV)
    torch.cuda.synchronize()
    assert torch.equal(q2, q)
    # checksum against an independent torch formulation of the same f32 arithmetic
    inv = torch.tensor(1.0, device="cuda") / torch.tensor(p.scale, device="cuda")
    t = x * inv
    ref = torch.clamp(torch.sign(t) * torch.floor(t.abs().double() + 0.5).float(), -128, 127).to(torch.int8)
    assert torch.equal(q, ref)


def test_minmax_one_launch_and_its_bounded_wait(hipq):
    """hipq_minmax_f32 is one launch: every workgroup publishes its partial as tagged words of the context and
    workgroup 0 collects them.  Over a fresh context's first 40 calls (across the wrap of the meeting number,
    grids of different sizes) it equals the two-launch form (variant 6) and torch; with the spin limit forced to 0
    workgroup 0 looks once, too early for some of 512 partials: the outputs must then be NaN (never a range made of
    some of the partials) and the context reports HIPQ_DEVICE_ERROR once."""
    c = hipq.Context(0)
    try:
        g = torch.Generator(device="cuda").manual_seed(31)
        sizes = [1 << 22, 7, 4096, 1 << 24, 100003, 1 << 12]
        for it in range(40):
            x = torch.randn(sizes[it % len(sizes)], generator=g, device="cuda") * (it + 1)
            got = c.minmax(x)
            c.set_gemm_kernel_variant(6)
            want = c.minmax(x)
            c.set_gemm_kernel_variant(0)
            c.synchronize()
            assert torch.equal(got, want) and got[0].item() == x.min().item() and got[1].item() == x.max().item(), it
        x = torch.randn(1 << 24, generator=g, device="cuda")
        c.set_wait_spin_limit(0)
        got = c.minmax(x)
        with pytest.raises(hipq.HipqError) as e:
            c.synchronize()
        assert e.value.code == hipq.DEVICE_ERROR
        assert bool(torch.isnan(got).all())
        c.set_wait_spin_limit(-1)
        got = c.minmax(x)
        c.synchronize()
        assert got[0].item() == x.min().item() and got[1].item() == x.max().item()
    finally:
        c.close()


@pytest.mark.parametrize("n", [150, 152, 5 * (1 << 20)])
def test_non_finite_range_sets_status_and_skips(ctx, hipq, n):
    """150 elements take the two-launch path (not a multiple of 4), 152 the one-launch path with 4 float4 per
    lane, 5 Mi the one with 16: each must report the status and leave the output untouched."""
    x = torch.ones(n, device="cuda")
    x[n // 3] = float("inf")
    out = torch.full((n,), 77, dtype=torch.int8, device="cuda")
    _, params = ctx.quantize_dynamic_per_tensor(x, out=out)
    p = ctx.read_qparams(params)
    assert p.status == hipq.INVALID_ARGUMENT and p.scale == 1.0
    assert bool((out == 77).all())


@pytest.mark.parametrize("n", [1000, 6 * (1 << 20) + 4])
@pytest.mark.parametrize("dtype_name", ["i8", "u8"])
def test_dynamic_quantize_one_launch_matches_two_launches(hipq, n, dtype_name):
    """Every parameter flavour and both quantize forms and roundings through the one-launch dynamic quantizer (the
    tensor stays in registers between the range and the codes; 6 Mi + 4 elements: 16 float4 per lane and a ragged
    last workgroup) against the two-launch path (variant 6), whose kernels the oracle tests above pin."""
    c = hipq.Context(0)
    try:
        g = torch.Generator(device="cuda").manual_seed(n % 977)
        x = torch.randn(n, generator=g, device="cuda") * 3.0 + 0.5
        dtype = hipq.DTYPE_I8 if dtype_name == "i8" else hipq.DTYPE_U8
        for flavor in range(7):
            for mode in (0, hipq.FORM_DIV, hipq.ROUND_HALF_EVEN, hipq.FORM_DIV | hipq.ROUND_HALF_EVEN):
                q, params = c.quantize_dynamic_per_tensor(x, flavor, dtype, mode)
                c.set_gemm_kernel_variant(6)
                q2, params2 = c.quantize_dynamic_per_tensor(x, flavor, dtype, mode)
                c.set_gemm_kernel_variant(0)
                c.synchronize()
                a, b = c.read_qparams(params), c.read_qparams(params2)
                assert (a.scale, a.zero_point, a.min_val, a.max_val, a.status) == (b.scale, b.zero_point, b.min_val,
                                                                                b.max_val, b.status), (flavor, mode)
                assert torch.equal(q, q2), (flavor, mode)
    finally:
        c.close()


@pytest.mark.parametrize("lo,hi", [(2.0, 5.0), (-100.0, -99.0)])
@pytest.mark.parametrize("n", [4096, 4099, 1 << 20])
def test_dynamic_quantize_with_a_zero_point_outside_the_code_range(ctx, hipq, lo, hi, n):
    """The torsh-nn asymmetric rule does not clamp its zero point: an all-positive tensor in [2, 5] gives -170, an
    all-negative one in [-100, -99] gives 25500.  Such a zero point must not depend on which path a size and
    alignment select (sizes that qualify for the one-launch quantizer and one that does not): status SUCCESS, the
    parameters of the formula ((max - min) / 255, round(-min / scale)), and the codes
    clamp(round(x / scale) + zp, 0, 255), from numpy in float32."""
    rng = np.random.default_rng(n)
    x = (rng.random(n, dtype=np.float32) * np.float32(hi - lo) + np.float32(lo)).astype(np.float32)
    x[0], x[-1] = lo, hi
    q, params = ctx.quantize_dynamic_per_tensor(dev(x), hipq.PARAMS_NN_ASYMMETRIC, hipq.DTYPE_U8, hipq.FORM_DIV)
    ctx.synchronize()
    p = ctx.read_qparams(params)
    scale = np.float32(np.float32(hi) - np.float32(lo)) / np.float32(255.0)
    t = -np.float32(lo) / scale
    zp = int(np.trunc(t + np.copysign(np.float32(0.5), t)))  # f32::round of a value that is no tie
    assert p.status == hipq.SUCCESS and p.scale == scale and p.zero_point == zp
    assert zp == {2.0: -170, -100.0: 25500}[lo]
    v = x / scale
    r = np.trunc(v + np.copysign(np.float32(0.49999997), v))  # f32::round (tests/host/round_away_check.c)
    want = np.clip(r + np.float32(zp), 0, 255).astype(np.uint8)
    np.testing.assert_array_equal(host(q), want)


@pytest.mark.parametrize("shape", [(1, 8), (3, 33), (16, 4096), (5, 1024), (7, 1025), (4, 4100), (2, 20000), (64, 768)])
@pytest.mark.parametrize("flavor_name", ["symmetric", "affine"])
def test_per_row_quantize(ctx, hipq, oracle, shape, flavor_name):
    x = normal(shape[0] * 7 + shape[1], shape)
    if shape[0] > 2:
        x[2] = 0.0  # degenerate row -> (1.0, 0) / (1.0, -128)
    flavor = hipq.PARAMS_SYMMETRIC if flavor_name == "symmetric" else hipq.PARAMS_AFFINE
    scheme = oracle.PER_CHANNEL_SYMMETRIC if flavor_name == "symmetric" else oracle.PER_CHANNEL_AFFINE
    want_q, want_s, want_z = oracle.quantize_per_channel_auto(x, 0, 0, scheme)
    q, s, z, status = ctx.quantize_per_row(dev(x), flavor)
    assert host(status)[0] == 0
    np.testing.assert_array_equal(host(s), want_s)
    np.testing.assert_array_equal(host(z), want_z)
    np.testing.assert_array_equal(host(q), want_q.astype(np.int8))


def test_per_row_status_on_non_finite_row(ctx, hipq):
    x = normal(3, (4, 128))
    x[1, 5] = np.inf
    _, _, _, status = ctx.quantize_per_row(dev(x))
    assert host(status)[0] == hipq.INVALID_ARGUMENT


@pytest.mark.parametrize("axis", [0, 1, 2])
def test_per_channel_any_axis(ctx, hipq, oracle, axis):
    x = normal(21 + axis, (5, 6, 7))
    want_q, want_s, want_z = oracle.quantize_per_channel_auto(x, axis, 0, oracle.PER_CHANNEL_SYMMETRIC)
    q, s, z, status = ctx.quantize_per_channel_auto(dev(x), axis)
    assert host(status)[0] == 0
    np.testing.assert_array_equal(host(s), want_s)
    np.testing.assert_array_equal(host(q), want_q.astype(np.int8))
    # explicit parameters, both forms, and per-channel dequantize
    zps = np.arange(x.shape[axis], dtype=np.int32) - 2
    got = host(ctx.quantize_per_channel(dev(x), dev(want_s), dev(zps), axis, hipq.FORM_DIV))
    np.testing.assert_array_equal(got, oracle.quantize_per_channel_affine(x, want_s, zps, axis).astype(np.int8))
    deq = host(ctx.dequantize_per_channel(dev(got), dev(want_s), dev(zps), axis))
    np.testing.assert_array_equal(deq, oracle.dequantize_per_channel_affine(got.astype(np.float32), want_s, zps, axis))
    if axis == 0:
        got = host(ctx.quantize_per_channel(dev(x), dev(want_s), dev(zps), 0, hipq.FORM_MUL_INV))
        want = oracle.quantize_per_channel_simd(x.reshape(5, -1), want_s, zps, 42).reshape(x.shape)
        np.testing.assert_array_equal(got, want.astype(np.int8))


SPREAD_SHAPES = [((8, 64, 28, 28), 1, 1), ((300, 1000), 1, 1), ((64, 33, 130), 1, 4), ((5, 12, 4400), 1, 5),
                 ((20000, 16), 1, 1), ((9000, 8, 4), 1, 1), ((3, 700, 129), 2, 1), ((2, 3, 50000), 1, 1),
                 ((1025, 257), 1, 1), ((40, 2000, 4), 1, 3)]


@pytest.mark.parametrize("shape,axis,group", SPREAD_SHAPES)
def test_per_channel_auto_spread_over_columns(ctx, hipq, oracle, shape, axis, group):
    """Ranges, parameters and codes per channel / per group of channels over a channel axis that is not the leading one,
    at sizes where the work is spread over many workgroups by columns (few groups, or short runs per channel):
    vectors of four and single elements, column tiles narrower than a workgroup, a last group that is shorter."""
    x = normal(sum(shape) + axis, shape) * np.linspace(0.2, 3.0, shape[axis], dtype=np.float32).reshape(
        [-1 if i == axis else 1 for i in range(len(shape))])
    assert x.size >= 1 << 18
    outer = int(np.prod(shape[:axis], dtype=np.int64))
    inner = int(np.prod(shape[axis + 1:], dtype=np.int64))
    for qmin, qmax in ((-128, 127), (-8, 7)):
        q, s, z, status = ctx.quantize_per_group_auto(dev(x), outer, shape[axis], inner, group,
                                                      hipq.PARAMS_ZERO_INCLUDED, qmin, qmax, hipq.FORM_DIV)
        want, ws, wz, _, _ = oracle.quantize_group_wise(x, axis, group, qmin, qmax)
        assert int(host(status)[0]) == 0
        np.testing.assert_array_equal(host(s), ws)
        np.testing.assert_array_equal(host(z), wz)
        np.testing.assert_array_equal(host(q).astype(np.float32), want)
    if group == 1:
        for scheme, flavor in ((oracle.PER_CHANNEL_SYMMETRIC, hipq.PARAMS_SYMMETRIC),
                               (oracle.PER_CHANNEL_AFFINE, hipq.PARAMS_AFFINE)):
            want_q, want_s, want_z = oracle.quantize_per_channel_auto(x, axis, 0, scheme)
            q, s, z, status = ctx.quantize_per_channel_auto(dev(x), axis, flavor)
            assert host(status)[0] == 0
            np.testing.assert_array_equal(host(s), want_s)
            np.testing.assert_array_equal(host(z), want_z)
            np.testing.assert_array_equal(host(q), want_q.astype(np.int8))


def test_per_channel_auto_spread_half_even_and_bad_groups(ctx, hipq, oracle):
    """Round-half-even over columns equals the per-row kernel on the transposed matrix; a channel holding an infinity
    sets the status word and keeps its codes untouched while the other channels get theirs; NaNs are left out of a
    channel's range and become code 0."""
    x = np.round(normal(5, (600, 500)) * 8) / 16  # many exact .5 ties after the division
    xd = dev(x)
    q, s, z, status = ctx.quantize_per_channel_auto(xd, 1, hipq.PARAMS_AFFINE, hipq.ROUND_HALF_EVEN)
    qr, sr, zr, _ = ctx.quantize_per_row(xd.t().contiguous(), hipq.PARAMS_AFFINE, hipq.ROUND_HALF_EVEN)
    assert host(status)[0] == 0
    assert torch.equal(s, sr) and torch.equal(z, zr) and torch.equal(q, qr.t())
    q0, _, _, _ = ctx.quantize_per_channel_auto(xd, 1, hipq.PARAMS_AFFINE, 0)
    assert not torch.equal(q, q0)  # the ties do round differently
    bad = x.copy()
    bad[17, 3] = np.inf
    bad[5, 9] = np.nan
    out = torch.full((600, 500), 77, dtype=torch.int8, device="cuda")
    scales = torch.empty(500, dtype=torch.float32, device="cuda")
    zps = torch.empty(500, dtype=torch.int32, device="cuda")
    status = torch.empty(1, dtype=torch.int32, device="cuda")
    ctx.call("hipq_quantize_per_channel_auto_f32_i8", dev(bad).data_ptr(), 600, 500, 1, hipq.PARAMS_AFFINE, 0,
             out.data_ptr(), scales.data_ptr(), zps.data_ptr(), status.data_ptr())
    assert host(status)[0] == hipq.INVALID_ARGUMENT
    got = host(out)
    assert (got[:, 3] == 77).all()
    keep = np.ones(500, bool)
    keep[3] = False
    ref_in = bad.copy()
    ref_in[17, 3] = x[17, 3]
    want_q, want_s, want_z = oracle.quantize_per_channel_auto(ref_in, 1, 0, oracle.PER_CHANNEL_AFFINE)
    assert np.isnan(want_q[5, 9]) and got[5, 9] == 0  # the float carrier keeps the NaN; as an int8 code it is 0
    np.testing.assert_array_equal(got[:, keep], np.nan_to_num(want_q, nan=0.0).astype(np.int8)[:, keep])
    np.testing.assert_array_equal(host(scales)[keep], want_s[keep])
    np.testing.assert_array_equal(host(zps)[keep], want_z[keep])


@pytest.mark.parametrize("shape,axis", [((3, 8, 12), 0), ((3, 8, 12), 1), ((7, 5, 2048), 1), ((6, 1000), 0),
                                        ((300, 64, 36), 1), ((1, 1, 4), 2), ((257, 4100), 0), ((16, 4096), 1),
                                        ((8, 16384), 0), ((2, 64, 1024), 1)])
def test_per_channel_vector_forms(ctx, hipq, oracle, shape, axis):
    """Explicit-parameter per-channel quantize / dequantize where the run of one channel is a multiple of four
    elements (the kernels then work on vectors of four): power-of-two and other run lengths and channel counts,
    whole tiles and ragged tails, both rounding forms; and the same data one element off alignment, which takes
    the element-wise kernels and must give the same bytes."""
    x = normal(77 + axis, shape) * 3
    x.reshape(-1)[:4] = [np.nan, np.inf, -np.inf, 1e30]  # NaN -> the zero point's code; infinities saturate
    ch = shape[axis]
    rng = np.random.default_rng(9)
    scales = rng.uniform(0.01, 0.05, ch).astype(np.float32)
    zps = rng.integers(-7, 8, ch).astype(np.int32)
    want = oracle.quantize_per_channel_affine(x, scales, zps, axis).astype(np.int8)
    got = ctx.quantize_per_channel(dev(x), dev(scales), dev(zps), axis, hipq.FORM_DIV)
    np.testing.assert_array_equal(host(got), want)
    want_y = oracle.dequantize_per_channel_affine(want.astype(np.float32), scales, zps, axis)
    np.testing.assert_array_equal(host(ctx.dequantize_per_channel(got, dev(scales), dev(zps), axis)), want_y)
    for mode in (hipq.FORM_MUL_INV, hipq.FORM_DIV | hipq.ROUND_HALF_EVEN):
        # off alignment: the same elements at an address one element past a 16-byte boundary
        n = x.size
        pad = torch.empty(n + 4, dtype=torch.float32, device="cuda")
        pad[1:n + 1] = dev(x).reshape(-1)
        off = pad[1:n + 1].view(shape)
        assert off.data_ptr() % 16 == 4
        a = ctx.quantize_per_channel(dev(x), dev(scales), dev(zps), axis, mode)
        b = ctx.quantize_per_channel(off, dev(scales), dev(zps), axis, mode)
        assert torch.equal(a, b)
    if axis == 0 and len(shape) == 2:
        want = oracle.quantize_per_channel_simd(x, scales, zps, shape[1])
        got = ctx.quantize_per_channel(dev(x), dev(scales), dev(zps), 0, hipq.FORM_MUL_INV)
        # (the reference's f32 carrier keeps a NaN; as an int8 code it is 0, Rust's `NaN as i8`)
        np.testing.assert_array_equal(host(got), np.nan_to_num(want, nan=0.0).astype(np.int8))


@pytest.mark.parametrize("shape", [(1, 1), (5, 9), (64, 256), (100, 333)])
def test_requantize(ctx, hipq, oracle, shape):
    rng = np.random.default_rng(shape[1])
    acc = rng.integers(-3_000_000, 3_000_000, size=shape, dtype=np.int32)
    sw = rng.uniform(1e-4, 1e-3, shape[1]).astype(np.float32)
    bias = (rng.standard_normal(shape[1]) * 0.01).astype(np.float32)
    for sa in (np.array([0.02], np.float32), rng.uniform(0.01, 0.03, shape[0]).astype(np.float32)):
        want = oracle.requantize_epilogue(acc, sa, sw, bias, 0.31, -3)
        got = host(ctx.requantize(dev(acc), dev(sa), dev(sw), dev(bias), 0.31, -3))
        np.testing.assert_array_equal(got, want)
    want = oracle.requantize_epilogue(acc, sa, sw, None, 0.31, 0)
    got = host(ctx.requantize(dev(acc), dev(sa), dev(sw), None, 0.31, 0))
    np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("rows,cols", [(2304, 4096), (3000, 3072), (800, 11008), (4100, 2052), (16384, 768)])
def test_requantize_large_tensors_with_columns_fixed_per_thread(ctx, hipq, oracle, rows, cols):
    """Tensors of several tiles per workgroup take the form of the requantize kernel in which a thread meets the
    same column vectors in every tile and loads their weight scales and biases once (the grid is then a multiple of
    a period that depends on cols: 1, 3, 43, 513, 3 here).  One block of rows repeated, expected bytes from the
    oracle on the block; one activation scale and one per row, with and without bias, both roundings."""
    brows = 37
    reps = -(-rows // brows)
    rng = np.random.default_rng(rows + cols)
    acc0 = rng.integers(-3_000_000, 3_000_000, size=(brows, cols), dtype=np.int32)
    acc0[0, :8] = [2**31 - 1, -2**31, 0, 1, -1, 2_000_000_000, -2_000_000_000, 77]  # saturation either side
    sw = rng.uniform(1e-4, 1e-3, cols).astype(np.float32)
    bias = (rng.standard_normal(cols) * 0.01).astype(np.float32)
    acc = dev(acc0).repeat(reps, 1)[:rows].contiguous()
    for sa0 in (np.array([0.02], np.float32), rng.uniform(0.01, 0.03, brows).astype(np.float32)):
        sa = dev(sa0) if sa0.size == 1 else dev(sa0).repeat(reps)[:rows].contiguous()
        for b in (bias, None):
            for mode, rm in ((hipq.ROUND_HALF_AWAY, 0), (hipq.ROUND_HALF_EVEN, 1)):
                oracle.set_round_mode(rm)
                try:
                    want = oracle.requantize_epilogue(acc0, sa0, sw, b, 0.31, -3)
                finally:
                    oracle.set_round_mode(0)
                got = ctx.requantize(acc, sa, dev(sw), None if b is None else dev(b), 0.31, -3, mode)
                torch.cuda.synchronize()
                assert torch.equal(got, dev(want).repeat(reps, 1)[:rows]), (sa0.size, b is None, mode)


@pytest.mark.parametrize("n", [4, 1024, 8192, 8196, 1 << 20, 4096 * 4096, 4096 * 4096 + 8192])
@pytest.mark.parametrize("dtype_name", ["i8", "u8"])
def test_dynamic_quantize_equals_explicit_steps(ctx, hipq, n, dtype_name):
    """The dynamic entry point (range reduction, then quantize from the device-resident parameters) must agree
    bit for bit with min/max, parameter and quantize calls made one by one."""
    g = torch.Generator(device="cuda").manual_seed(n % 1000)
    x = torch.randn(n, generator=g, device="cuda")
    if dtype_name == "i8":
        flavor, dtype, qmin, qmax, mode = hipq.PARAMS_SYMMETRIC, hipq.DTYPE_I8, -128, 127, hipq.FORM_MUL_INV
    else:
        flavor, dtype, qmin, qmax, mode = hipq.PARAMS_BACKEND_ASYMMETRIC, hipq.DTYPE_U8, 0, 255, hipq.FORM_DIV
    q, params = ctx.quantize_dynamic_per_tensor(x, flavor, dtype, mode)
    p = ctx.read_qparams(params)
    mm = ctx.minmax(x)
    params2 = ctx.qparams_from_minmax(mm, flavor, qmin, qmax)
    q2 = torch.empty_like(q)
    name = "hipq_quantize_with_params_f32_i8" if dtype_name == "i8" else "hipq_quantize_with_params_f32_u8"
    ctx.call(name, x.data_ptr(), n, params2.data_ptr(), mode, q2.data_ptr())
    p2 = ctx.read_qparams(params2)
    ctx.synchronize()
    assert (p.scale, p.zero_point, p.min_val, p.max_val, p.status) == (p2.scale, p2.zero_point, p2.min_val, p2.max_val, 0)
    assert torch.equal(q, q2)


def test_dynamic_quantize_back_to_back(ctx, hipq):
    """Many calls in a row share the context's scratch (partials, parameters); stream order keeps them apart."""
    g = torch.Generator(device="cuda").manual_seed(3)
    xs = [torch.randn(512 * 4096, generator=g, device="cuda") * (i + 1) for i in range(6)]
    outs = [ctx.quantize_dynamic_per_tensor(x) for x in xs * 5]
    ctx.synchronize()
    for i, (q, params) in enumerate(outs):
        x = xs[i % len(xs)]
        p = ctx.read_qparams(params)
        assert p.status == 0 and p.scale == np.float32(x.abs().max().item()) / np.float32(127.0)
        assert int(q.abs().max().item()) == 127


def test_more_than_two_to_the_32_elements(ctx, hipq, oracle):
    """2^32 + 4099 elements (16 GiB of fp32) through range reduction, quantize, dequantize and the dynamic
    quantizer.  The input is one seeded block repeated; its length is odd, so an element index that wrapped
    at 32 bits would land in another phase of the block, and the extremes sit beyond element 2^32, where only
    64-bit indices reach them.  Expected values: the oracle's on the block, repeated the same way."""
    period = (1 << 20) + 7
    n = (1 << 32) + 4099
    reps = -(-n // period)
    base = normal(11, (period,))
    scale, lo_at, hi_at = np.float32(0.03), (1 << 32) + 5, n - 2
    x = dev(base).repeat(reps)[:n]
    x[lo_at], x[hi_at] = -11.25, 9.5
    mm = host(ctx.minmax(x))
    assert (mm[0], mm[1]) == (-11.25, 9.5)
    assert host(ctx.absmax(x))[0] == 11.25

    def repeated(block, lo_val, hi_val):
        t = dev(block).repeat(reps)[:n]
        t[lo_at], t[hi_at] = lo_val, hi_val
        return t

    q = ctx.quantize_per_tensor_i8(x, scale, 0, hipq.FORM_MUL_INV)
    want_q = repeated(oracle.quantize_to_int8_simd(base, scale, 0), -128, 127)
    torch.cuda.synchronize()
    assert torch.equal(q, want_q)
    y = ctx.dequantize(q, scale, 0)
    want_y_block = oracle.dequantize_per_tensor_affine(oracle.quantize_to_int8_simd(base, scale, 0).astype(np.float32),
                                                      scale, 0)
    want_y = repeated(want_y_block, float(np.float32(-128) * scale), float(np.float32(127) * scale))
    torch.cuda.synchronize()
    assert torch.equal(y, want_y)
    del y, want_y, want_q
    # dynamic: the planted minimum fixes the scale, 11.25 / 127
    qd, params = ctx.quantize_dynamic_per_tensor(x, hipq.PARAMS_SYMMETRIC, hipq.DTYPE_I8, hipq.FORM_MUL_INV, out=q)
    p = ctx.read_qparams(params)
    s_dyn = np.float32(11.25) / np.float32(127.0)
    assert p.status == 0 and p.scale == s_dyn and (p.min_val, p.max_val) == (-11.25, 9.5)
    want_qd = repeated(oracle.quantize_to_int8_simd(base, s_dyn, 0), -127,
                       int(oracle.quantize_to_int8_simd(np.full(65, 9.5, np.float32), s_dyn, 0)[0]))
    torch.cuda.synchronize()
    assert torch.equal(qd, want_qd)


def test_per_row_quantize_beyond_two_to_the_32_elements(ctx, hipq, oracle):
    """[2^20 + 3, 4100] rows (4.3 G elements): a block of 1021 rows repeated, expected codes and scales from the
    oracle on the block; row starts beyond byte 2^34 need 64-bit offsets."""
    rows, cols, brows = (1 << 20) + 3, 4100, 1021
    reps = -(-rows // brows)
    base = normal(12, (brows, cols))
    want_q, want_s, _ = oracle.quantize_per_channel_auto(base, 0, 0, oracle.PER_CHANNEL_SYMMETRIC)
    x = dev(base).repeat(reps, 1)[:rows]
    q, scales, zps, status = ctx.quantize_per_row(x, hipq.PARAMS_SYMMETRIC)
    torch.cuda.synchronize()
    assert int(status.item()) == 0 and not bool(zps.any())
    assert torch.equal(scales, dev(want_s.astype(np.float32)).repeat(reps)[:rows])
    assert torch.equal(q, dev(want_q.astype(np.int8)).repeat(reps, 1)[:rows])


def test_per_channel_and_requantize_beyond_two_to_the_32_elements(ctx, hipq, oracle):
    """Explicit-parameter per-channel quantize / dequantize over [4199, 1021, 1003] (channel axis in the middle,
    4.3 G elements) and requantize over [2^20 + 3, 4100] accumulators: one block repeated along the outer axis,
    expected bytes from the oracle on the block."""
    outer, ch, inner = 4199, 1021, 1003
    assert outer * ch * inner > 1 << 32
    rng = np.random.default_rng(5)
    base = normal(31, (1, ch, inner))
    scales = rng.uniform(0.01, 0.05, ch).astype(np.float32)
    zps = rng.integers(-5, 6, ch).astype(np.int32)
    want_q = oracle.quantize_per_channel_affine(base, scales, zps, 1).astype(np.int8)
    want_y = oracle.dequantize_per_channel_affine(want_q.astype(np.float32), scales, zps, 1)
    x = dev(base).repeat(outer, 1, 1)
    q = ctx.quantize_per_channel(x, dev(scales), dev(zps), 1, hipq.FORM_DIV)
    torch.cuda.synchronize()
    assert bool((q == dev(want_q)).all())  # broadcast over the outer axis
    y = ctx.dequantize_per_channel(q, dev(scales), dev(zps), 1)
    torch.cuda.synchronize()
    assert bool((y == dev(want_y)).all())
    del x, q, y
    rows, cols, brows = (1 << 20) + 3, 4100, 1021
    reps = -(-rows // brows)
    acc0 = rng.integers(-3_000_000, 3_000_000, size=(brows, cols), dtype=np.int32)
    sa0 = rng.uniform(0.01, 0.03, brows).astype(np.float32)
    sw = rng.uniform(1e-4, 1e-3, cols).astype(np.float32)
    bias = (rng.standard_normal(cols) * 0.01).astype(np.float32)
    want = oracle.requantize_epilogue(acc0, sa0, sw, bias, 0.31, -3)
    got = ctx.requantize(dev(acc0).repeat(reps, 1)[:rows], dev(sa0).repeat(reps)[:rows], dev(sw), dev(bias), 0.31, -3)
    torch.cuda.synchronize()
    assert torch.equal(got, dev(want).repeat(reps, 1)[:rows])


@pytest.mark.parametrize("n", [6, 256, 257, 4099, (1 << 20) + 3])
def test_mobile_quantizer_and_its_reduced_precision_rounding(ctx, hipq, oracle, n):
    """quantize_mobile_optimized: round(x * inv) up to 256 elements or without reduced precision, floor(x * inv + 0.5)
    beyond; ties, the 0.49999997 edge, saturation and NaN included."""
    x = normal(40 + n, (n,), 3.0)
    x[:6] = [1.25, -1.25, 0.24999999, -0.25, 1e9, np.nan]
    for reduced in (False, True):
        mode = hipq.FORM_MUL_INV | (hipq.ROUND_FLOOR_HALF_UP if (reduced and n > 256) else 0)
        got = host(ctx.quantize_per_tensor_i8(dev(x), 0.5, 3, mode))
        np.testing.assert_array_equal(got, oracle.quantize_mobile_optimized(x, 0.5, 3, reduced))
    # the other entry points do not know the mode, and two roundings at once are refused
    with pytest.raises(hipq.HipqError):
        ctx.quantize_per_tensor_u8(dev(x), 0.5, 3, hipq.ROUND_FLOOR_HALF_UP)
    with pytest.raises(hipq.HipqError):
        ctx.quantize_per_tensor_i8(dev(x), 0.5, 3, hipq.ROUND_FLOOR_HALF_UP | hipq.ROUND_HALF_EVEN)


def test_cache_aware_twins_share_the_carrier_kernel(ctx, hipq, oracle, golden):
    for case in golden["slice_variants"]["carrier"]:
        x = np.array(case["x"], np.float32)
        got = host(ctx.quantize_per_tensor_carrier(dev(x), case["scale"], case["zp"], hipq.FORM_MUL_INV))
        for idx, val in case["checks"]:
            assert got[idx] == np.float32(val), case["fn"]
    x = normal(77, (100_003,), 4.0)
    x[:3] = [np.nan, 1e9, -1e9]
    got = host(ctx.quantize_per_tensor_carrier(dev(x), 0.05, -3, hipq.FORM_MUL_INV))
    np.testing.assert_array_equal(got, oracle.quantize_cache_aware(x, 0.05, -3))


def test_scalar_qtypes_form_zero_point_before_rounding(ctx, hipq, oracle):
    """QInt8 / QUInt8::quantize (crates/torsh-core/src/dtype/quantized.rs:129-134, 285-290): round(v / scale + zp),
    clamped to the type.  Ties where the two orders differ (v / scale = -2.5, zp = 5: 3 against 2), saturation,
    NaN -> 0, and random data, element by element against the oracle's scalar functions."""
    rng = np.random.default_rng(21)
    special = np.float32([-2.5, 2.5, -0.5, 0.5, 0.0, 1e9, -1e9, np.nan, np.inf, -np.inf, 122.5, -133.5])
    for scale, zp in ((1.0, 5), (0.1, -7), (0.37, 100)):
        x = np.concatenate([special * np.float32(scale), rng.standard_normal(3000).astype(np.float32) * 40]).astype(np.float32)
        got = host(ctx.quantize_per_tensor_i8(dev(x), scale, zp, hipq.FORM_ZP_BEFORE_ROUND))
        want = np.array([oracle.qint8_quantize(float(v), scale, zp) for v in x], np.int8)
        np.testing.assert_array_equal(got, want)
        if zp >= 0:
            gotu = host(ctx.quantize_per_tensor_u8(dev(x), scale, zp, hipq.FORM_ZP_BEFORE_ROUND))
            wantu = np.array([oracle.quint8_quantize(float(v), scale, zp) for v in x], np.uint8)
            np.testing.assert_array_equal(gotu, wantu)
    # the order matters: the default form gives the other answer on the crafted tie
    x = dev(np.float32([-2.5]))
    assert int(host(ctx.quantize_per_tensor_i8(x, 1.0, 5, hipq.FORM_ZP_BEFORE_ROUND))[0]) == 3
    assert int(host(ctx.quantize_per_tensor_i8(x, 1.0, 5, hipq.FORM_DIV))[0]) == 2
    with pytest.raises(hipq.HipqError):  # two rounding rules at once
        ctx.quantize_per_tensor_i8(x, 1.0, 5, hipq.FORM_ZP_BEFORE_ROUND | hipq.ROUND_FLOOR_HALF_UP)


def test_torsh_nn_flavour(ctx, hipq, oracle):
    """torsh-nn's own quantizer (crates/torsh-nn/src/quantization/ops.rs:153-172, 296-373): values pass through
    `as i32` before the zero point is added (a NaN becomes the code zero_point, not a NaN carrier), per-channel
    weight scales have no zero guard, negative int8 codes are carried as 256 + q."""
    rng = np.random.default_rng(22)
    x = np.concatenate([np.float32([2.5, -2.5, 1e9, -1e9, np.nan, np.inf, -np.inf, 0.0]),
                        rng.standard_normal(2000).astype(np.float32) * 3]).astype(np.float32)
    for scale, zp, qmin, qmax in ((0.05, 0, -128, 127), (0.02, 77, 0, 255), (0.001, 0, -32768, 32767)):
        got = host(ctx.quantize_per_tensor_carrier(dev(x), scale, zp, hipq.FORM_INT_CAST, qmin, qmax))
        if zp == 0:
            want = [oracle.nn_quantize_value_symmetric(float(v), scale, qmin, qmax) for v in x]
        else:
            want = [oracle.nn_quantize_value_asymmetric(float(v), scale, zp, qmin, qmax) for v in x]
        np.testing.assert_array_equal(got, np.float32(want))
    # per-channel weights, symmetric int8: codes, unguarded scales (an all-zero and a tiny channel among them)
    w = (rng.standard_normal((9, 200)) * 0.02).astype(np.float32)
    w[3] = 0.0
    w[5] *= 1e-9
    want_carrier, want_s = oracle.nn_per_channel_quantize_weights_sym_i8(w)
    q, s, z, st = ctx.quantize_per_group_auto(dev(w), 1, 9, 200, 1, hipq.PARAMS_NN_SYMMETRIC, -128, 127, hipq.FORM_DIV)
    assert int(host(st)[0]) == 0
    np.testing.assert_array_equal(host(s), want_s)
    np.testing.assert_array_equal(host(q).view(np.uint8).astype(np.float32), want_carrier)  # 256 + q for negatives
    assert (host(z) == 0).all()
    # asymmetric uint8: unclamped zero point, bytes 0..255
    w2 = (rng.standard_normal((7, 130)) * 0.5 + 1.0).astype(np.float32)
    w2[2] = np.abs(w2[2]) + 2.0  # all positive: zero point far below 0
    want_carrier, want_s, want_z = oracle.nn_per_channel_quantize_weights_asym_u8(w2)
    q, s, z, st = ctx.quantize_per_group_auto(dev(w2), 1, 7, 130, 1, hipq.PARAMS_NN_ASYMMETRIC, 0, 255, hipq.FORM_DIV)
    np.testing.assert_array_equal(host(s), want_s)
    np.testing.assert_array_equal(host(z), want_z)
    np.testing.assert_array_equal(host(q).view(np.uint8).astype(np.float32), want_carrier)
    # a NaN weight becomes the code clamp(zero point) (`NaN as i32` is 0, then the zero point is added), in every
    # kernel form the entry point has: a channel per row, channels that are not the leading dimension (one workgroup
    # per channel), and the same spread over many workgroups
    w3 = (rng.standard_normal((7, 130)) * 0.5 + 0.3).astype(np.float32)
    w3[1, 5] = np.nan
    w3[4, 0] = np.nan
    w3[3] = 1.5   # constant channels: scale 0 (no guard), a zero point at the end of the i32 range
    w3[5] = -0.25
    want_carrier, want_s, want_z = oracle.nn_per_channel_quantize_weights_asym_u8(w3)
    q, s, z, st = ctx.quantize_per_group_auto(dev(w3), 1, 7, 130, 1, hipq.PARAMS_NN_ASYMMETRIC, 0, 255, hipq.FORM_DIV)
    np.testing.assert_array_equal(host(s), want_s)
    np.testing.assert_array_equal(host(z), want_z)
    np.testing.assert_array_equal(host(q).view(np.uint8).astype(np.float32), want_carrier)
    assert host(q).view(np.uint8)[1, 5] == np.clip(want_z[1], 0, 255) and host(q).view(np.uint8)[4, 0] == np.clip(want_z[4], 0, 255)
    for outer, inner in ((5, 26), (160, 832)):  # [outer, 7, inner]: 130 and 133120 values per channel
        wc = (rng.standard_normal((7, outer * inner)) * 0.5 + 0.3).astype(np.float32)
        wc[1, 5] = np.nan
        wc[6, outer * inner - 1] = np.nan
        want_carrier, want_s, want_z = oracle.nn_per_channel_quantize_weights_asym_u8(wc)
        x3 = np.ascontiguousarray(wc.reshape(7, outer, inner).transpose(1, 0, 2))
        q, s, z, st = ctx.quantize_per_group_auto(dev(x3), outer, 7, inner, 1, hipq.PARAMS_NN_ASYMMETRIC, 0, 255,
                                                  hipq.FORM_DIV)
        np.testing.assert_array_equal(host(s), want_s)
        np.testing.assert_array_equal(host(z), want_z)
        got = host(q).view(np.uint8).transpose(1, 0, 2).reshape(7, outer * inner).astype(np.float32)
        np.testing.assert_array_equal(got, want_carrier)
