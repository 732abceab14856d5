"""W4A16 GEMM at the four Llama-3-8B linear shapes (qkv, o, gate_up, down) and every row count the
benchmark sweep names, M in {1, 8, 16, 32, 128, 2048}, against the CPU oracle (``x.float() @ ((q -
z) * s)``, fp32) within rtol = atol = 1e-2.  One dequantisation per shape on the CPU; M = 2048 is
compared on sampled rows.  The down projection is the shape whose decode plan splits K across
workgroups; its result must also be identical run to run."""
import numpy as np
import pytest
import torch

from oracle import w4 as ow4

pytestmark = pytest.mark.gpu
RTOL = ATOL = 1e-2
SHAPES = {"qkv": (4096, 6144), "o": (4096, 4096), "gate_up": (4096, 28672), "down": (14336, 4096)}


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("layer", list(SHAPES))
def test_w4a16_llama3_8b_shape_all_row_counts(layer):
    from vllm_gcu_amd.kernels import _custom_ops as ops
    from vllm_gcu_amd.kernels.quantization import rearrange
    K, N = SHAPES[layer]
    g = 128
    rng = np.random.default_rng(sum(map(ord, layer)))
    # uniform random checkpoint words (= uniform nibbles); the oracle's unpack gives the logical matrix
    qweight = rng.integers(-2 ** 31, 2 ** 31, size=(K // 8, N), dtype=np.int64).astype(np.int32)
    q = ow4.gptq_unpack_weight(qweight)
    z = rng.integers(0, 16, size=(K // g, N), dtype=np.uint8)
    s = rng.uniform(0.001, 0.01, size=(K // g, N)).astype(np.float16)
    w, zp = rearrange.rearrange_uint4_int32_gptq(dev(qweight), dev(ow4.gptq_pack_zeros(z)))
    sd = dev(s)
    wf = ow4.dequantize(q, z, s.astype(np.float32), g)          # [K, N] fp32, once per shape
    del q, qweight
    for M in (1, 8, 16, 32, 128, 2048):
        print(f"case llama3-8b {layer} K={K} N={N} M={M}", flush=True)
        x = rng.standard_normal((M, K)).astype(np.float16)
        out = ops.gptq_gemm_gcu(dev(x), w, zp, sd, torch.empty(0, dtype=torch.int32, device="cuda"), 4, None, g)
        again = ops.gptq_gemm_gcu(dev(x), w, zp, sd, torch.empty(0, dtype=torch.int32, device="cuda"), 4, None, g)
        torch.cuda.synchronize()
        assert out.shape == (M, N) and torch.isfinite(out).all()
        assert torch.equal(out, again), "result depends on scheduling"
        got = out.float().cpu().numpy()
        rows = np.arange(M)
        if M > 128:
            rows = np.random.default_rng(M).choice(M, size=32, replace=False)
            rows[:3] = (0, 63, M - 1)
        want = x[rows].astype(np.float32) @ wf
        np.testing.assert_allclose(got[rows], want, rtol=RTOL, atol=ATOL)
