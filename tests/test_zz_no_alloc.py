"""hipq_linear_dynamic_f32_noalloc (static device scratch, no allocation) against hipq_linear_dynamic_f32.

Both run the same kernels, so the fp32 outputs must be identical bit for bit (the 1e-5 relative bar of the
Linear forward is stated as well).  Two calls in a row, the second on a smaller input, so that whatever the
first call left in the shared static scratch cannot leak into the second.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

RTOL = 1e-5


def _case(ctx, hipq, seed, m, n, k, per_token):
    g = torch.Generator(device="cuda").manual_seed(seed)
    x = torch.randn(m, k, generator=g, device="cuda")
    wf = torch.randn(n, k, generator=g, device="cuda") * 0.02
    bias = torch.randn(n, generator=g, device="cuda") * 0.01
    wq, sw, _, _ = ctx.quantize_per_row(wf)
    want = ctx.linear_dynamic(x, wq, sw, bias, per_token=per_token, mode=hipq.FORM_MUL_INV)
    got = torch.full((m, n), float("nan"), device="cuda")
    ctx.linear_dynamic_noalloc(x, wq, sw, bias, per_token=per_token, mode=hipq.FORM_MUL_INV, out=got)
    torch.cuda.synchronize()
    w, g_ = want.cpu().numpy(), got.cpu().numpy()
    np.testing.assert_allclose(g_, w, rtol=RTOL, atol=0)
    np.testing.assert_array_equal(g_, w)


@pytest.mark.parametrize("per_token", [False, True])
def test_noalloc_matches_the_allocating_entry_point_twice(ctx, hipq, per_token):
    _case(ctx, hipq, 11, 512, 384, 1024, per_token)   # larger first ...
    _case(ctx, hipq, 12, 37, 200, 256, per_token)     # ... then smaller: stale scratch must not show
    _case(ctx, hipq, 13, 130, 72, 2048, per_token)


def test_noalloc_rejects_sizes_beyond_the_static_scratch(ctx, hipq):
    x = torch.zeros(8, 16, device="cuda")
    w = torch.zeros(8, 16, dtype=torch.int8, device="cuda")
    sw = torch.ones(8, device="cuda")
    out = torch.empty(8, 8, device="cuda")
    # the size check comes before any pointer is touched, so small buffers stand in for large shapes
    for m, k in ((16385, 16), (4096, 1025)):
        with pytest.raises(hipq.HipqError) as e:
            ctx.call("hipq_linear_dynamic_f32_noalloc", x.data_ptr(), 0, w.data_ptr(), sw.data_ptr(), 0, m, 8, k, 0,
                     out.data_ptr())
        assert e.value.code == hipq.SHAPE_ERROR
        assert "static scratch" in str(e.value)
