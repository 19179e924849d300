"""qadd / qrelu of the backend trait (through the C-ABI) against the CPU oracle: bytes and parameters bit-exact."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


def rand_bytes(seed, n, dtype):
    rng = np.random.default_rng(seed)
    return rng.integers(-128, 128, n).astype(np.int8) if dtype == np.int8 else rng.integers(0, 256, n).astype(np.uint8)


@pytest.mark.parametrize("dtype", [np.int8, np.uint8])
@pytest.mark.parametrize("symmetric", [False, True])
@pytest.mark.parametrize("n", [1, 15, 16, 4097, 100003, 1 << 20])
def test_qadd_and_qrelu_are_bit_exact(ctx, hipq, oracle, dtype, symmetric, n):
    a, b = rand_bytes(n, n, dtype), rand_bytes(n + 1, n, dtype)
    sa, za, sb, zb = 0.0173, (-7 if dtype == np.int8 else 121), 0.0419, (12 if dtype == np.int8 else 99)
    flavor = hipq.PARAMS_BACKEND_SYMMETRIC if symmetric else hipq.PARAMS_BACKEND_ASYMMETRIC
    out, params = ctx.qadd(dev(a), sa, za, dev(b), sb, zb, flavor)
    want, s, z = oracle.backend_qadd(a, sa, za, b, sb, zb, symmetric)
    p = ctx.read_qparams(params)
    assert (p.scale, p.zero_point, p.status) == (s, z, 0)
    np.testing.assert_array_equal(host(out), want)
    out, params = ctx.qrelu(dev(a), sa, za, flavor)
    want, s, z = oracle.backend_qrelu(a, sa, za, symmetric)
    p = ctx.read_qparams(params)
    assert (p.scale, p.zero_point, p.min_val) == (s, z, 0.0)
    np.testing.assert_array_equal(host(out), want)


def test_mixed_operand_types_and_unaligned_views(ctx, hipq, oracle):
    n = 50021
    a, b = rand_bytes(1, n, np.uint8), rand_bytes(2, n, np.int8)
    out, params = ctx.qadd(dev(a), 0.02, 128, dev(b), 0.03, 0)
    want, s, z = oracle.backend_qadd(a, 0.02, 128, b, 0.03, 0)
    assert out.dtype == torch.uint8 and ctx.read_qparams(params).scale == s
    np.testing.assert_array_equal(host(out), want)
    da, db = dev(a), dev(a[::-1].copy())
    for off in (1, 3, 7):
        out, _ = ctx.qadd(da[off:], 0.02, 128, db[off:], 0.01, 100)
        want, _, _ = oracle.backend_qadd(a[off:], 0.02, 128, a[::-1][off:], 0.01, 100)
        np.testing.assert_array_equal(host(out), want)


def test_closed_forms_and_errors(ctx, hipq):
    # a = [1, 2, -3, 4] (scale 0.1 on bytes 10, 20, -30, 40), b = [0.5, 1, 1.5, 2]: sum range [-1.5, 6]
    a = dev(np.int8([10, 20, -30, 40]))
    b = dev(np.int8([1, 2, 3, 4]))
    out, params = ctx.qadd(a, 0.1, 0, b, 0.5, 0)
    p = ctx.read_qparams(params)
    assert p.scale == np.float32(7.5) / np.float32(255.0) and p.zero_point == -77
    assert (p.min_val, p.max_val) == (-1.5, 6.0)
    np.testing.assert_array_equal(host(out), np.int8([-26, 25, -128, 127]))
    # ReLU of all-negative data: range (0, 0) -> (scale 1, zero point qmin), every byte = qmin
    out, params = ctx.qrelu(dev(np.int8([-10, -20, -1])), 0.1, 0)
    p = ctx.read_qparams(params)
    assert (p.scale, p.zero_point) == (1.0, -128) and (host(out) == -128).all()
    # symmetric: zero point 0, scale 2 * max / 255
    out, params = ctx.qrelu(dev(np.int8([-10, 50, 100])), 0.1, 0, hipq.PARAMS_BACKEND_SYMMETRIC)
    p = ctx.read_qparams(params)
    assert p.zero_point == 0 and p.scale == np.float32(20.0) / np.float32(255.0)
    with pytest.raises(hipq.HipqError):
        ctx.qadd(a, 0.1, 0, b, 0.5, 0, flavor=hipq.PARAMS_SYMMETRIC)
    with pytest.raises(hipq.HipqError):
        ctx.qrelu(torch.empty(0, dtype=torch.int8, device="cuda"), 0.1, 0)


def test_full_size_properties(ctx, hipq):
    n = 4096 * 4096
    g = torch.Generator(device="cuda").manual_seed(5)
    a = torch.randint(-128, 128, (n,), generator=g, device="cuda", dtype=torch.int8)
    zero = torch.zeros(n, device="cuda", dtype=torch.int8)
    # a + 0 with the same scale re-quantizes a onto its own range: dequantized values agree to half a step
    out, params = ctx.qadd(a, 0.05, 0, zero, 0.05, 0)
    p = ctx.read_qparams(params)
    assert p.min_val == -6.4 or abs(p.min_val + 6.4) < 1e-6
    back = (out.to(torch.float32) - p.zero_point) * p.scale
    assert float((back - a.to(torch.float32) * 0.05).abs().max()) <= p.scale / 2 * (1 + 1e-5)
    # relu is idempotent on its own output
    r1, p1 = ctx.qrelu(a, 0.05, 0)
    q1 = ctx.read_qparams(p1)
    r2, p2 = ctx.qrelu(r1, q1.scale, q1.zero_point)
    q2 = ctx.read_qparams(p2)
    assert (q2.scale, q2.zero_point) == (q1.scale, q1.zero_point) or abs(q2.scale - q1.scale) < 1e-7
    assert int((r2.to(torch.int32) - r1.to(torch.int32)).abs().max()) <= 1
