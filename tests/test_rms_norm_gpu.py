"""GPU parity of rms_norm / fused_add_rms_norm against the CPU oracle, and of
the six fused norm + quantise operators against the sequence the reference
defines them by (norm, then the separate quantiser: fusion.py:183-330) -- the
fused outputs must be bit-identical to that sequence."""
import numpy as np
import pytest
import torch

from oracle import norm as onorm

pytestmark = pytest.mark.gpu
RTOL = ATOL = 1e-2


@pytest.fixture(scope="module")
def ops():
    from vllm_gcu_amd.kernels import _custom_ops
    return _custom_ops


def rounder(dtype):
    return lambda a: torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(dtype).float().numpy()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("rows,K", [(1, 128), (7, 4096), (33, 7168), (3, 8), (5, 8192), (4, 8200), (3, 16384)])
def test_rms_norm_and_fused_add_vs_oracle(ops, dtype, rows, K):
    print(f"case rms_norm {dtype} rows={rows} K={K}", flush=True)
    rng = np.random.default_rng(rows * 131 + K)
    act = rounder(dtype)
    x = act(rng.standard_normal((rows, K)) * 2)
    r = act(rng.standard_normal((rows, K)))
    w = act(rng.uniform(0.5, 1.5, K))
    xd, rd, wd = (torch.from_numpy(a).to(dtype).cuda() for a in (x, r, w))
    out = torch.empty_like(xd)
    torch.ops._C.rms_norm(out, xd, wd, 1e-6)
    want = onorm.rms_norm(x, w, 1e-6, act)
    np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)
    # at most one unit in the last place of the activation type apart (rsqrt vs 1 / sqrt); a flip of the
    # first rounding (x * rs) times a weight up to 1.5 can land two units away, seen on rows of 8200
    ulp = 2.0 ** -10 if dtype == torch.float16 else 2.0 ** -7
    diff = np.abs(out.float().cpu().numpy() - want)
    assert np.all(diff <= 2 * ulp * np.maximum(np.abs(want), 2.0 ** -14) * 1.01)
    assert np.mean(diff > ulp * np.maximum(np.abs(want), 2.0 ** -14) * 1.01) < 1e-3
    xin, res = xd.clone(), rd.clone()
    torch.ops._C.fused_add_rms_norm(xin, res, wd, 1e-6)
    want_o, want_z = onorm.fused_add_rms_norm(x, r, w, 1e-6, act)
    assert np.array_equal(res.float().cpu().numpy(), want_z)          # the sum is exact arithmetic + one rounding
    np.testing.assert_allclose(xin.float().cpu().numpy(), want_o, rtol=RTOL, atol=ATOL)
    # in-place norm equals out-of-place norm of the summed residual
    out2 = torch.empty_like(xd)
    torch.ops._C.rms_norm(out2, res, wd, 1e-6)
    assert torch.equal(out2, xin)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("add", [False, True])
def test_fused_norm_quant_equals_norm_then_quant(ops, dtype, add):
    print(f"case rms_norm+quant {dtype} add={add}", flush=True)
    rng = np.random.default_rng(47 + int(add))
    rows, K, eps = 19, 2048, 1e-5
    x = torch.from_numpy(rng.standard_normal((rows, K)).astype(np.float32) * 3).to(dtype).cuda()
    r = torch.from_numpy(rng.standard_normal((rows, K)).astype(np.float32)).to(dtype).cuda()
    w = torch.from_numpy(rng.uniform(0.5, 1.5, K).astype(np.float32)).to(dtype).cuda()
    # the unfused first half
    if add:
        normed, res_ref = x.clone(), r.clone()
        torch.ops._C.fused_add_rms_norm(normed, res_ref, w, eps)
    else:
        normed = torch.empty_like(x)
        torch.ops._C.rms_norm(normed, x, w, eps)
    s8 = torch.tensor([0.043], dtype=torch.float32, device="cuda")
    sf = torch.tensor([0.0125], dtype=torch.float32, device="cuda")

    # static fp8
    want = torch.empty((rows, K), dtype=torch.float8_e4m3fn, device="cuda")
    torch.ops._C.static_scaled_fp8_quant(want, normed, sf)
    got, res = torch.empty_like(want), r.clone()
    if add:
        torch.ops._C.fused_add_rms_norm_static_fp8_quant(got, x, res, w, sf, eps)
        assert torch.equal(res, res_ref)
    else:
        torch.ops._C.rms_norm_static_fp8_quant(got, x, w, sf, eps)
    assert torch.equal(got.view(torch.uint8), want.view(torch.uint8))

    # static int8
    want = torch.empty((rows, K), dtype=torch.int8, device="cuda")
    torch.ops._C.static_scaled_int8_quant(want, normed, s8, None)
    got, res = torch.empty_like(want), r.clone()
    if add:
        torch.ops._C.fused_add_rms_norm_static_int8_quant(got, x, res, w, eps, s8)
        assert torch.equal(res, res_ref)
    else:
        torch.ops._C.rms_norm_static_int8_quant(got, x, w, s8, eps)
    assert torch.equal(got, want)

    # per-token-group fp8
    for g in (64, 128):
        want = torch.empty((rows, K), dtype=torch.float8_e4m3fn, device="cuda")
        want_s = torch.empty((rows, K // g), dtype=torch.float32, device="cuda")
        torch.ops._C.dynamic_per_token_group_fp8_quant(want, want_s, normed, g)
        got, got_s, res = torch.empty_like(want), torch.empty_like(want_s), r.clone()
        if add:
            torch.ops._C.fused_add_rms_norm_per_token_group_quant_fp8(got, res, got_s, x, w, eps, g)
            assert torch.equal(res, res_ref)
        else:
            torch.ops._C.rms_norm_per_token_group_quant_fp8(got, got_s, x, w, eps, g)
        assert torch.equal(got.view(torch.uint8), want.view(torch.uint8)) and torch.equal(got_s, want_s)


def test_rms_norm_argument_errors(ops):
    x = torch.zeros((2, 64), dtype=torch.float16, device="cuda")
    w = torch.ones(64, dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError):
        torch.ops._C.rms_norm(torch.empty((2, 32), dtype=torch.float16, device="cuda"), x, w, 1e-6)
    with pytest.raises(RuntimeError):
        torch.ops._C.rms_norm(torch.empty_like(x), x, torch.ones(32, dtype=torch.float16, device="cuda"), 1e-6)
    with pytest.raises(RuntimeError):
        torch.ops._C.rms_norm_static_int8_quant(torch.empty_like(x), x, w, torch.ones(1, device="cuda"), 1e-6)
    torch.ops._C.rms_norm(torch.empty((0, 64), dtype=torch.float16, device="cuda"), x[:0], w, 1e-6)   # empty: no-op
