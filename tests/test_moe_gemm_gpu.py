"""GPU parity of the fused-MoE grouped GEMMs and of the whole fused-experts
sequence against the CPU oracle (naive per-(token, slot) loop over dense
dequantised experts).  fp16/bf16 outputs within rtol 1e-2 / atol 1e-2."""
import numpy as np
import pytest
import torch

from oracle import fp8 as of8
from oracle import moe as om
from oracle import w4 as ow4
from oracle import w8a8 as o8

pytestmark = pytest.mark.gpu


@pytest.fixture(params=[False, True], ids=["zeros-as-given", "zeros-recovered"])
def zero_reading(request, monkeypatch):
    """Pre-scaled zero-points either reach the kernels as given or, the default, are turned back into
    the packed integers once per tensor."""
    from vllm_gcu_amd.kernels import _custom_ops
    monkeypatch.setattr(_custom_ops, "_RECOVER_INTEGER_ZEROS", request.param)
    return request.param
RTOL = ATOL = 1e-2


@pytest.fixture(scope="module")
def ops():
    from vllm_gcu_amd.kernels import _custom_ops
    return _custom_ops


@pytest.fixture(scope="module")
def fmoe():
    from vllm_gcu_amd.kernels import fused_moe
    return fused_moe


@pytest.fixture(scope="module")
def rearrange():
    from vllm_gcu_amd.kernels.quantization import rearrange
    return rearrange


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def f16(a):
    return a.astype(np.float16).astype(np.float32)


def bf16(a):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(torch.bfloat16).float().numpy()


def make_int4_experts(rng, E, K, N, g=128):
    q = rng.integers(0, 16, size=(E, K, N), dtype=np.uint8)
    z = rng.integers(0, 16, size=(E, K // g, N), dtype=np.uint8)
    s = rng.uniform(0.001, 0.01, size=(E, K // g, N)).astype(np.float16)
    return q, z, s


def int4_to_device(rearrange, q, z):
    qw = np.stack([ow4.gptq_pack_weight(q[e]) for e in range(q.shape[0])])
    qz = np.stack([ow4.gptq_pack_zeros(z[e]) for e in range(z.shape[0])])
    return rearrange.rearrange_uint4_int32_gptq(dev(qw), dev(qz))


def run_grouped(fmoe, A, B, C, A_scale, B_scale, B_zp, tw, ids, E, block, mul, topk, **flags):
    s, e, n = fmoe.moe_align_block_size(ids, block, E)
    cfg = {"BLOCK_SIZE_M": block}
    kw = dict(use_fp8_w8a8=False, use_int8_w8a8=False, use_int8_w8a16=False, use_int4_w4a16=False)
    kw.update(flags)
    fmoe.invoke_fused_moe_kernel(A, B, C, A_scale, B_scale, B_zp, tw, ids, s, e, n, mul, topk, cfg, **kw)
    torch.cuda.synchronize()


@pytest.mark.parametrize("g", [128, 64, 32])
@pytest.mark.parametrize("block", [16, 32, 64, 128])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_grouped_w4a16_both_gemms(fmoe, rearrange, block, dtype, g):
    """Both expert GEMM forms on every align block size, with quantisation groups of 128, 64 and 32
    (groups of 128 on blocks of 16 / 32 slots: the grouped streaming kernel; everything else: the MFMA
    kernel, whose plain loop carries two or four groups per K block)."""
    print(f"case grouped w4a16 block={block} {dtype} g={g}", flush=True)
    rng = np.random.default_rng(block)
    M, E, T, K, N = 37, 4, 2, 256, 384
    q, z, s = make_int4_experts(rng, E, K, N, g)
    w, zp = int4_to_device(rearrange, q, z)
    x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(dtype)
    sd = torch.from_numpy(s).to(dtype)
    tw, ids, _ = om.topk_softmax(rng.standard_normal((M, E)).astype(np.float32), T, True)
    wf = lambda e: ow4.dequantize(q[e], z[e], sd[e].float().numpy(), g)
    # GEMM 1 form: A is [M, K], output row t reads A[t // topk], no routed weight
    C = torch.full((M, T, N), 7.0, dtype=dtype, device="cuda")
    run_grouped(fmoe, x.cuda(), w, C, None, sd.cuda(), zp, dev(tw), dev(ids), E, block, False, T,
                use_int4_w4a16=True, block_shape=[0, g])
    want = om.fused_moe_gemm(x.float().numpy(), wf, ids, T)
    np.testing.assert_allclose(C.view(-1, N).float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)
    # GEMM 2 form: A is [M * topk, K], topk = 1, routed weights applied
    x2 = torch.from_numpy(rng.standard_normal((M * T, K)).astype(np.float32)).to(dtype)
    C2 = torch.empty((M, T, N), dtype=dtype, device="cuda")
    run_grouped(fmoe, x2.cuda(), w, C2, None, sd.cuda(), zp, dev(tw), dev(ids), E, block, True, 1,
                use_int4_w4a16=True, block_shape=[0, g])
    want2 = om.fused_moe_gemm(x2.float().numpy(), wf, ids, 1, tw, True)
    np.testing.assert_allclose(C2.view(-1, N).float().cpu().numpy(), want2, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("K,N", [(512, 2048), (4096, 2048)])
def test_grouped_w4a16_bf16_rows_staged_as_fp16(fmoe, rearrange, K, N):
    """bf16 at prefill token counts (blocks of 64 slots, two million outputs or more): the activation rows
    are staged in the workspace as fp16 times a power of two each and take the pipelined fp16 loop; a
    slot's multiplier is that of the row it was gathered from.  Rows from 2^-40 to 2^40, both GEMM forms,
    every output compared at the magnitude of its row; K = 4096 also splits K two ways."""
    print(f"case grouped w4a16 bf16 staged K={K} N={N}", flush=True)
    rng = np.random.default_rng(K)
    M, E, T, g, block, dtype = 600, 4, 2, 128, 64, torch.bfloat16
    q, z, s = make_int4_experts(rng, E, K, N, g)
    w, zp = int4_to_device(rearrange, q, z)
    sd = torch.from_numpy(s).to(dtype)
    tw, ids, _ = om.topk_softmax(rng.standard_normal((M, E)).astype(np.float32), T, True)
    wf = lambda e: ow4.dequantize(q[e], z[e], sd[e].float().numpy(), g)
    mag = (2.0 ** rng.integers(-40, 41, size=M)).astype(np.float32)
    x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32) * mag[:, None]).to(dtype)
    C = torch.full((M, T, N), 7.0, dtype=dtype, device="cuda")
    run_grouped(fmoe, x.cuda(), w, C, None, sd.cuda(), zp, dev(tw), dev(ids), E, block, False, T,
                use_int4_w4a16=True, block_shape=[0, g])
    want = om.fused_moe_gemm(x.float().numpy(), wf, ids, T)
    norm = np.repeat(mag, T)[:, None]
    np.testing.assert_allclose(C.view(-1, N).float().cpu().numpy() / norm, want / norm, rtol=RTOL, atol=ATOL)
    mag2 = (2.0 ** rng.integers(-40, 41, size=M * T)).astype(np.float32)
    x2 = torch.from_numpy(rng.standard_normal((M * T, K)).astype(np.float32) * mag2[:, None]).to(dtype)
    C2 = torch.empty((M, T, N), dtype=dtype, device="cuda")
    run_grouped(fmoe, x2.cuda(), w, C2, None, sd.cuda(), zp, dev(tw), dev(ids), E, block, True, 1,
                use_int4_w4a16=True, block_shape=[0, g])
    want2 = om.fused_moe_gemm(x2.float().numpy(), wf, ids, 1, tw, True)
    np.testing.assert_allclose(C2.view(-1, N).float().cpu().numpy() / mag2[:, None], want2 / mag2[:, None], rtol=RTOL, atol=ATOL)
    C3 = torch.empty_like(C2)
    run_grouped(fmoe, x2.cuda(), w, C3, None, sd.cuda(), zp, dev(tw), dev(ids), E, block, True, 1,
                use_int4_w4a16=True, block_shape=[0, g])
    assert torch.equal(C2, C3)


@pytest.mark.parametrize("block", [16, 32, 64])
def test_grouped_w4a16_reference_layout_and_prescaled_zeros(fmoe, block, zero_reading):
    # what the reference's moe_wna16 loader leaves on the layer: uint8 [E, N, K/2]
    # half-group bytes (moe_wna16.py:464-466) and fp16 zeros = z * scales
    # (blocks of 16 / 32 slots run the weight-streaming kernel, 64 the MFMA tile kernel)
    print(f"case grouped w4a16 reference layout block={block}", flush=True)
    rng = np.random.default_rng(5)
    M, E, T, K, N = 20, 3, 2, 256, 256
    q, z, s = make_int4_experts(rng, E, K, N)
    rw = np.stack([np.ascontiguousarray(ow4.ref_halfgroup_pack(q[e]).T) for e in range(E)])
    zs = (z.astype(np.float32) * s.astype(np.float32)).astype(np.float16)
    x = rng.standard_normal((M, K)).astype(np.float16)
    tw, ids, _ = om.topk_softmax(rng.standard_normal((M, E)).astype(np.float32), T, True)
    C = torch.empty((M, T, N), dtype=torch.float16, device="cuda")
    run_grouped(fmoe, dev(x), dev(rw), C, None, dev(s), dev(zs), dev(tw), dev(ids), E, block, False, T,
                use_int4_w4a16=True, block_shape=[0, 128])
    want = om.fused_moe_gemm(x.astype(np.float32), lambda e: ow4.dequantize_prescaled_zeros(q[e], zs[e], s[e], 128), ids, T)
    np.testing.assert_allclose(C.view(-1, N).float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)
    # symmetric experts: no zero-point tensor, implicit zero 8
    C = torch.full((M, T, N), float("nan"), dtype=torch.float16, device="cuda")
    run_grouped(fmoe, dev(x), dev(rw), C, None, dev(s), None, dev(tw), dev(ids), E, block, False, T,
                use_int4_w4a16=True, block_shape=[0, 128])
    z8 = np.full_like(z, 8)
    want = om.fused_moe_gemm(x.astype(np.float32), lambda e: ow4.dequantize(q[e], z8[e], s[e].astype(np.float32), 128), ids, T)
    np.testing.assert_allclose(C.view(-1, N).float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("block", [16, 64, 128])
def test_grouped_fp8_block(fmoe, ops, block):
    print(f"case grouped fp8 block={block}", flush=True)
    rng = np.random.default_rng(7 + block)
    M, E, T, K, N = 50, 6, 3, 512, 384
    wf32 = (rng.standard_normal((E, N, K)) * 0.02).astype(np.float32)
    ws = rng.uniform(0.5, 2.0, size=(E, N // 128, K // 128)).astype(np.float32)
    wq = np.stack([of8.to_e4m3fn(np.clip(wf32[e] * 100, -448, 448)) for e in range(E)])      # codes
    x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(torch.bfloat16)
    xq, xs = ops.per_token_group_quant_fp8(x.cuda(), 128)
    tw, ids, _ = om.topk_softmax(rng.standard_normal((M, E)).astype(np.float32), T, True)
    C = torch.empty((M, T, N), dtype=torch.bfloat16, device="cuda")
    run_grouped(fmoe, xq, dev(wq).view(torch.float8_e4m3fn), C, xs, dev(ws), None, dev(tw), dev(ids), E, block,
                False, T, use_fp8_w8a8=True, block_shape=[128, 128])
    xq_c, xs_c = xq.view(torch.uint8).cpu().numpy(), xs.cpu().numpy()
    want = np.zeros((M * T, N), dtype=np.float32)
    flat = ids.reshape(-1)
    for t in range(M * T):
        e = flat[t]
        want[t] = of8.block_fp8_gemm(xq_c[t // T:t // T + 1], xs_c[t // T:t // T + 1], wq[e], ws[e])[0]
    got = C.view(-1, N).float().cpu().numpy()
    np.testing.assert_allclose(got, want, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("kslab", [False, True])
@pytest.mark.parametrize("M,E,T,K,N,blk", [(300, 6, 3, 512, 384, 256), (40, 4, 2, 384, 128, 256), (700, 3, 1, 1024, 256, 256),
                                           (300, 6, 3, 512, 384, 128), (700, 3, 1, 1024, 256, 128)])
def test_grouped_fp8_block_on_blocks_of_256_slots(fmoe, ops, rearrange, monkeypatch, M, E, T, K, N, blk, kslab):
    """Blocks of 256 slot ids (prefill token counts) run the MFMA tile kernel with its rows gathered through
    the ids.  Both GEMM forms (rows t // topk without routing weight; one row per slot with it), row-major
    and kslab weights, an expert that no token chose, one that expert_map sends elsewhere (its rows come
    back as zeros); against the oracle and against the weight-streaming kernel on blocks of 64."""
    print(f"case grouped fp8 tiles M={M} E={E} T={T} K={K} N={N} kslab={kslab}", flush=True)
    monkeypatch.setattr(ops, "_AUTO_KSLAB", False)       # (row-major weights stay row-major)
    rng = np.random.default_rng(M + K)
    wq = np.stack([of8.to_e4m3fn(np.clip(rng.standard_normal((N, K)) * 2, -448, 448).astype(np.float32)) for _ in range(E)])
    ws = rng.uniform(0.005, 0.02, size=(E, N // 128, K // 128)).astype(np.float32)
    wd = dev(wq).view(torch.float8_e4m3fn)
    if kslab:
        wd = rearrange.to_kslab(wd)
    logits = rng.standard_normal((M, E)).astype(np.float32)
    logits[:, E - 1] -= 50.0                                   # nobody routes to the last expert
    tw, ids, _ = om.topk_softmax(logits, T, True)
    flat = ids.reshape(-1)
    x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(torch.bfloat16)
    xq, xs = ops.per_token_group_quant_fp8(x.cuda(), 128)
    xq_c, xs_c = xq.view(torch.uint8).cpu().numpy(), xs.cpu().numpy()
    want = np.zeros((M * T, N), dtype=np.float32)
    for t in range(M * T):
        want[t] = of8.block_fp8_gemm(xq_c[t // T:t // T + 1], xs_c[t // T:t // T + 1], wq[flat[t]], ws[flat[t]])[0]
    C = torch.full((M, T, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    run_grouped(fmoe, xq, wd, C, xs, dev(ws), None, dev(tw), dev(ids), E, blk, False, T,
                use_fp8_w8a8=True, block_shape=[128, 128])
    got = C.view(-1, N).float().cpu().numpy()
    np.testing.assert_allclose(got, want, rtol=RTOL, atol=ATOL)
    C64 = torch.empty_like(C)
    run_grouped(fmoe, xq, wd, C64, xs, dev(ws), None, dev(tw), dev(ids), E, 64, False, T,
                use_fp8_w8a8=True, block_shape=[128, 128])
    assert (C.float() - C64.float()).abs().max().item() <= 2 ** -6 * max(1.0, float(np.abs(want).max()))
    # second form: one activation row per slot, routing weights applied; expert 0 mapped away
    x2 = torch.from_numpy(rng.standard_normal((M * T, K)).astype(np.float32)).to(torch.bfloat16)
    x2q, x2s = ops.per_token_group_quant_fp8(x2.cuda(), 128)
    emap = torch.arange(E, dtype=torch.int32)
    emap[0] = -1
    s_, e_, n_ = fmoe.moe_align_block_size(dev(ids), blk, E, emap.cuda())
    C2 = torch.full((M, T, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    fmoe.invoke_fused_moe_kernel(x2q, wd, C2, x2s, dev(ws), None, dev(tw), dev(ids), s_, e_, n_, True, 1,
                                 {"BLOCK_SIZE_M": blk}, use_fp8_w8a8=True, use_int8_w8a8=False, use_int8_w8a16=False,
                                 use_int4_w4a16=False, block_shape=[128, 128])
    torch.cuda.synchronize()
    x2q_c, x2s_c = x2q.view(torch.uint8).cpu().numpy(), x2s.cpu().numpy()
    want2 = np.zeros((M * T, N), dtype=np.float32)
    twf = tw.reshape(-1)
    for t in range(M * T):
        if flat[t] != 0:
            want2[t] = of8.block_fp8_gemm(x2q_c[t:t + 1], x2s_c[t:t + 1], wq[flat[t]], ws[flat[t]])[0] * twf[t]
    np.testing.assert_allclose(C2.view(-1, N).float().cpu().numpy(), want2, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("kslab", [False, True])
@pytest.mark.parametrize("M,E,T,K,N,blk", [(300, 6, 3, 512, 384, 256), (40, 4, 2, 384, 192, 256), (700, 3, 1, 1024, 256, 256),
                                           (300, 6, 3, 512, 384, 128), (700, 3, 1, 1024, 256, 128)])
def test_grouped_int8_on_blocks_of_256_slots(fmoe, ops, rearrange, monkeypatch, M, E, T, K, N, blk, kslab):
    """int8 experts (per-token x per-channel scales) on blocks of 256 slot ids: the int8 MFMA tile kernel
    with its rows gathered through the ids.  Both GEMM forms, row-major and kslab weights, an idle expert
    and one that expert_map sends elsewhere; the int32 sums are exact, so the outputs equal those of the
    weight-streaming kernel on blocks of 64 bit for bit."""
    print(f"case grouped int8 tiles M={M} E={E} T={T} K={K} N={N} kslab={kslab}", flush=True)
    monkeypatch.setattr(ops, "_AUTO_KSLAB", False)       # (row-major weights stay row-major)
    rng = np.random.default_rng(M + K + 1)
    wq = rng.integers(-127, 128, size=(E, N, K), dtype=np.int8)
    ws = rng.uniform(0.001, 0.02, size=(E, N, 1)).astype(np.float32)
    wd = dev(wq)
    if kslab:
        wd = rearrange.to_kslab(wd)
    logits = rng.standard_normal((M, E)).astype(np.float32)
    logits[:, E - 1] -= 50.0
    tw, ids, _ = om.topk_softmax(logits, T, True)
    flat = ids.reshape(-1)
    x = rng.standard_normal((M, K)).astype(np.float16)
    xq, xs = o8.dynamic_scaled_int8_quant(x)
    want = np.zeros((M * T, N), dtype=np.float32)
    for t in range(M * T):
        acc = o8.int8_gemm_i32(xq[t // T:t // T + 1], np.ascontiguousarray(wq[flat[t]].T))
        want[t] = o8.scaled_mm_epilogue(acc, xs[t // T], ws[flat[t], :, 0])[0]
    C = torch.full((M, T, N), float("nan"), dtype=torch.float16, device="cuda")
    run_grouped(fmoe, dev(xq), wd, C, dev(xs), dev(ws), None, dev(tw), dev(ids), E, blk, False, T, use_int8_w8a8=True)
    np.testing.assert_allclose(C.view(-1, N).float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)
    C64 = torch.empty_like(C)
    run_grouped(fmoe, dev(xq), wd, C64, dev(xs), dev(ws), None, dev(tw), dev(ids), E, 64, False, T, use_int8_w8a8=True)
    assert torch.equal(C, C64)
    # second form: one activation row per slot, routing weights applied; expert 0 mapped away
    x2 = rng.standard_normal((M * T, K)).astype(np.float16)
    x2q, x2s = o8.dynamic_scaled_int8_quant(x2)
    emap = torch.arange(E, dtype=torch.int32)
    emap[0] = -1
    s_, e_, n_ = fmoe.moe_align_block_size(dev(ids), blk, E, emap.cuda())
    C2 = torch.full((M, T, N), float("nan"), dtype=torch.float16, device="cuda")
    fmoe.invoke_fused_moe_kernel(dev(x2q), wd, C2, dev(x2s), dev(ws), None, dev(tw), dev(ids), s_, e_, n_, True, 1,
                                 {"BLOCK_SIZE_M": blk}, use_fp8_w8a8=False, use_int8_w8a8=True, use_int8_w8a16=False,
                                 use_int4_w4a16=False)
    torch.cuda.synchronize()
    want2 = np.zeros((M * T, N), dtype=np.float32)
    twf = tw.reshape(-1)
    for t in range(M * T):
        if flat[t] != 0:
            acc = o8.int8_gemm_i32(x2q[t:t + 1], np.ascontiguousarray(wq[flat[t]].T))
            want2[t] = o8.scaled_mm_epilogue(acc, x2s[t], ws[flat[t], :, 0])[0] * twf[t]
    np.testing.assert_allclose(C2.view(-1, N).float().cpu().numpy(), want2, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("kslab", [False, True])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M,E,T,K,N,blk", [(300, 6, 3, 512, 384, 256), (40, 4, 2, 384, 256, 256), (700, 3, 1, 1152, 256, 256),
                                           (300, 6, 3, 512, 384, 128), (700, 3, 1, 1152, 256, 128)])
def test_grouped_16bit_on_blocks_of_256_slots(fmoe, ops, rearrange, monkeypatch, M, E, T, K, N, blk, dtype, kslab):
    """Unquantised fp16 / bf16 experts on blocks of 256 or 128 slot ids: the MFMA tile kernel with its rows
    gathered through the ids, two 32-deep 16-bit MFMAs per 128-byte K tile.  Both GEMM forms, row-major and
    kslab weights, an odd and an even number of K tiles, an idle expert and one that expert_map sends
    elsewhere; against the fp32 oracle, and against the weight-streaming kernel on blocks of 64 (another
    order of the same fp32 additions)."""
    print(f"case grouped 16-bit tiles M={M} E={E} T={T} K={K} N={N} blk={blk} {dtype} kslab={kslab}", flush=True)
    monkeypatch.setattr(ops, "_AUTO_KSLAB", False)       # (row-major weights stay row-major)
    rng = np.random.default_rng(M + K + 2)
    w = torch.from_numpy((rng.standard_normal((E, N, K)) * 0.05).astype(np.float32)).to(dtype)
    wd = w.cuda()
    if kslab:
        wd = rearrange.to_kslab(wd)
    logits = rng.standard_normal((M, E)).astype(np.float32)
    logits[:, E - 1] -= 50.0
    tw, ids, _ = om.topk_softmax(logits, T, True)
    flat = ids.reshape(-1)
    x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(dtype)
    wf, xf = w.float().numpy(), x.float().numpy()
    want = np.zeros((M * T, N), dtype=np.float32)
    for e in range(E):
        rows = np.nonzero(flat == e)[0]
        if rows.size:
            want[rows] = xf[rows // T] @ wf[e].T
    C = torch.full((M, T, N), float("nan"), dtype=dtype, device="cuda")
    run_grouped(fmoe, x.cuda(), wd, C, None, None, None, dev(tw), dev(ids), E, blk, False, T)
    np.testing.assert_allclose(C.view(-1, N).float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)
    C64 = torch.empty_like(C)
    run_grouped(fmoe, x.cuda(), wd, C64, None, None, None, dev(tw), dev(ids), E, 64, False, T)
    np.testing.assert_allclose(C.float().cpu().numpy(), C64.float().cpu().numpy(), rtol=RTOL, atol=ATOL)
    # second form: one activation row per slot, routing weights applied; expert 0 mapped away
    x2 = torch.from_numpy(rng.standard_normal((M * T, K)).astype(np.float32)).to(dtype)
    emap = torch.arange(E, dtype=torch.int32)
    emap[0] = -1
    s_, e_, n_ = fmoe.moe_align_block_size(dev(ids), blk, E, emap.cuda())
    C2 = torch.full((M, T, N), float("nan"), dtype=dtype, device="cuda")
    fmoe.invoke_fused_moe_kernel(x2.cuda(), wd, C2, None, None, None, dev(tw), dev(ids), s_, e_, n_, True, 1,
                                 {"BLOCK_SIZE_M": blk}, use_fp8_w8a8=False, use_int8_w8a8=False, use_int8_w8a16=False,
                                 use_int4_w4a16=False)
    torch.cuda.synchronize()
    x2f, twf = x2.float().numpy(), tw.reshape(-1)
    want2 = np.zeros((M * T, N), dtype=np.float32)
    for e in range(1, E):
        rows = np.nonzero(flat == e)[0]
        if rows.size:
            want2[rows] = (x2f[rows] @ wf[e].T) * twf[rows, None]
    np.testing.assert_allclose(C2.view(-1, N).float().cpu().numpy(), want2, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("N", [260, 264, 200])
def test_grouped_int8_and_fp16_and_w8a16(fmoe, ops, N):
    # widths that end inside a 64-column group: 260 takes the 8-byte output stores (not a multiple of 8),
    # 264 and 200 the 16-byte ones with a last piece of 8 columns
    print(f"case grouped int8 / fp16 / w8a16 N={N}", flush=True)
    rng = np.random.default_rng(11)
    M, E, T, K = 33, 4, 2, 256
    ids_w, ids, _ = om.topk_softmax(rng.standard_normal((M, E)).astype(np.float32), T, True)
    # int8 per-token x per-channel
    x = rng.standard_normal((M, K)).astype(np.float16)
    xq, xs = o8.dynamic_scaled_int8_quant(x)
    wq = rng.integers(-127, 128, size=(E, N, K), dtype=np.int8)
    ws = rng.uniform(0.001, 0.02, size=(E, N, 1)).astype(np.float32)
    C = torch.empty((M, T, N), dtype=torch.float16, device="cuda")
    run_grouped(fmoe, dev(xq), dev(wq), C, dev(xs), dev(ws), None, dev(ids_w), dev(ids), E, 32, False, T,
                use_int8_w8a8=True)
    want = np.zeros((M * T, N), dtype=np.float32)
    flat = ids.reshape(-1)
    for t in range(M * T):
        e = flat[t]
        acc = o8.int8_gemm_i32(xq[t // T:t // T + 1], np.ascontiguousarray(wq[e].T))
        want[t] = o8.scaled_mm_epilogue(acc, xs[t // T], ws[e, :, 0])[0]
    np.testing.assert_allclose(C.view(-1, N).float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)
    # unquantised fp16 experts (fused_moe_kernel), routed weight applied
    wf = (rng.standard_normal((E, N, K)) * 0.05).astype(np.float16)
    C = torch.empty((M, T, N), dtype=torch.float16, device="cuda")
    run_grouped(fmoe, dev(x), dev(wf), C, None, None, None, dev(ids_w), dev(ids), E, 16, True, T)
    want = om.fused_moe_gemm(x.astype(np.float32), lambda e: wf[e].astype(np.float32).T, ids, T, ids_w, True)
    np.testing.assert_allclose(C.view(-1, N).float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)
    # W8A16 per channel
    s16 = rng.uniform(0.001, 0.01, size=(E, N)).astype(np.float16)
    C = torch.empty((M, T, N), dtype=torch.float16, device="cuda")
    run_grouped(fmoe, dev(x), dev(wq), C, None, dev(s16), None, dev(ids_w), dev(ids), E, 64, False, T,
                use_int8_w8a16=True, block_shape=[0, -1])
    want = om.fused_moe_gemm(x.astype(np.float32),
                             lambda e: (wq[e].astype(np.float32) * s16[e].astype(np.float32)[:, None]).T, ids, T)
    np.testing.assert_allclose(C.view(-1, N).float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)


def test_dense_block_fp8_and_w8a16(ops):
    rng = np.random.default_rng(13)
    M, K, N = 70, 512, 384
    x = torch.from_numpy(rng.standard_normal((3, M, K)).astype(np.float32)).to(torch.bfloat16)
    xq, xs = ops.per_token_group_quant_fp8(x.cuda(), 128)
    wq = of8.to_e4m3fn(np.clip(rng.standard_normal((N, K)) * 2, -448, 448).astype(np.float32))
    ws = rng.uniform(0.005, 0.02, size=(N // 128, K // 128)).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    out = ops.w8a8_block_fp8_matmul(xq, dev(wq).view(torch.float8_e4m3fn), xs, dev(ws), [128, 128], torch.bfloat16,
                                    torch.from_numpy(bias).to(torch.bfloat16).cuda())
    assert out.shape == (3, M, N) and out.dtype == torch.bfloat16
    want = of8.block_fp8_gemm(xq.view(torch.uint8).cpu().numpy().reshape(-1, K), xs.cpu().numpy().reshape(-1, K // 128),
                              wq, ws, bias=bf16(bias))
    np.testing.assert_allclose(out.float().cpu().numpy().reshape(-1, N), want, rtol=RTOL, atol=ATOL)
    # GPTQ-8bit path: gptq_gemm_gcu(bit=8) -> weight_only_quant (_custom_ops.py:269-275)
    w8 = rng.integers(-128, 128, size=(N, K), dtype=np.int8)
    s16 = rng.uniform(0.001, 0.01, N).astype(np.float16)
    xh = rng.standard_normal((M, K)).astype(np.float16)
    out = ops.gptq_gemm_gcu(dev(xh), dev(w8), torch.empty(0, device="cuda"), dev(s16), torch.empty(0, device="cuda"), 8, None, -1)
    want = o8.weight_only_int8(xh, w8, s16, -1)
    np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("M", [1, 5, 17, 33])
def test_dense_w8a16_ragged_width_splits_k_inside_the_workgroup(ops, M):
    # few rows and a width that is no multiple of 64 (row-major weights): the launch splits K over
    # the wavefronts of a workgroup, the last column group is partly outside the matrix
    rng = np.random.default_rng(50 + M)
    K, N = 640, 100
    print(f"case dense w8a16 ragged M={M} K={K} N={N}", flush=True)
    w8 = rng.integers(-128, 128, size=(N, K), dtype=np.int8)
    s16 = rng.uniform(0.001, 0.01, N).astype(np.float16)
    xh = rng.standard_normal((M, K)).astype(np.float16)
    out = ops.gptq_gemm_gcu(dev(xh), dev(w8), torch.empty(0, device="cuda"), dev(s16), torch.empty(0, device="cuda"), 8, None, -1)
    want = o8.weight_only_int8(xh, w8, s16, -1)
    np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("dtype,shape", [(np.uint8, (3, 128, 256)), (np.uint16, (2, 64, 384)), (np.uint8, (192, 128))])
def test_kslab_repack_bit_exact(rearrange, dtype, shape):
    print(f"case kslab repack {dtype.__name__} {shape}", flush=True)
    rng = np.random.default_rng(17)
    w = rng.integers(0, np.iinfo(dtype).max, size=shape, dtype=dtype)
    tdt = torch.int8 if dtype == np.uint8 else torch.float16
    got = rearrange.to_kslab(dev(w).view(tdt))
    assert rearrange.is_kslab(got) and got.shape == tuple(shape) and got.dtype == tdt
    want = o8.kslab_pack(w)
    assert np.array_equal(got.view(torch.uint8).cpu().numpy().reshape(-1), want.view(np.uint8).reshape(-1))
    assert rearrange.to_kslab(got) is got
    with pytest.raises(RuntimeError):
        rearrange.to_kslab(torch.zeros((100, 128), dtype=torch.int8, device="cuda"))


def test_kslab_and_row_major_weights_give_identical_results(fmoe, ops, rearrange, monkeypatch):
    """Same kernel arithmetic in either weight order: outputs must be bit-identical,
    for weights converted by the caller, converted implicitly, and left row-major."""
    rng = np.random.default_rng(19)
    M, E, T, K, N = 45, 5, 2, 384, 320
    wq = np.stack([of8.to_e4m3fn(np.clip(rng.standard_normal((N, K)) * 3, -448, 448).astype(np.float32))
                   for _ in range(E)])
    ws = rng.uniform(0.5, 2.0, size=(E, (N + 127) // 128, K // 128)).astype(np.float32)
    x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(torch.bfloat16)
    xq, xs = ops.per_token_group_quant_fp8(x.cuda(), 128)
    tw, ids, _ = om.topk_softmax(rng.standard_normal((M, E)).astype(np.float32), T, True)
    outs = []
    for how in ("row-major", "implicit", "explicit"):
        print(f"case kslab equivalence grouped fp8 {how}", flush=True)
        monkeypatch.setattr(ops, "_AUTO_KSLAB", how != "row-major")
        w = dev(wq).view(torch.float8_e4m3fn)
        if how == "explicit":
            w = rearrange.to_kslab(w)
        C = torch.empty((M, T, N), dtype=torch.bfloat16, device="cuda")
        run_grouped(fmoe, xq, w, C, xs, dev(ws), None, dev(tw), dev(ids), E, 16, False, T, use_fp8_w8a8=True,
                    block_shape=[128, 128])
        outs.append(C.view(torch.int16).cpu().numpy())
    assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[0], outs[2])
    # dense W8A16 (2-byte activations, 1-byte weights) and dense 16-bit weights through linear_quant's kernel
    w8 = rng.integers(-128, 128, size=(N, K), dtype=np.int8)
    s16 = rng.uniform(0.001, 0.01, N).astype(np.float16)
    xh = dev(rng.standard_normal((M, K)).astype(np.float16))
    outs = []
    for auto in (False, True):
        print(f"case kslab equivalence dense w8a16 auto={auto}", flush=True)
        monkeypatch.setattr(ops, "_AUTO_KSLAB", auto)
        o = ops.gptq_gemm_gcu(xh, dev(w8), torch.empty(0, device="cuda"), dev(s16), torch.empty(0, device="cuda"),
                              8, None, -1)
        outs.append(o.view(torch.int16).cpu().numpy())
    assert np.array_equal(outs[0], outs[1])
    want = o8.weight_only_int8(xh.cpu().numpy(), w8, s16, -1)
    np.testing.assert_allclose(o.float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("g", [64, 128])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_w8a16_group_scales_dense_and_grouped(fmoe, ops, g, dtype):
    """weight_only_quant / w8a16 experts with scales [K/g, N] (weight_only_quant.cpp:28-101,
    fused_moe.py:163-169)."""
    print(f"case w8a16 group={g} {dtype}", flush=True)
    rng = np.random.default_rng(37 + g)
    M, E, T, K, N = 35, 3, 2, 384, 320
    rnd = bf16 if dtype == torch.bfloat16 else f16
    xh = rnd(rng.standard_normal((M, K)).astype(np.float32))
    w8 = rng.integers(-128, 128, size=(E, N, K), dtype=np.int8)
    sg = rnd(rng.uniform(0.001, 0.01, size=(E, K // g, N)).astype(np.float32))
    xd = torch.from_numpy(xh).to(dtype).cuda()
    # dense, through the 8-bit GPTQ entry (the group scales are what it forwards)
    out = ops.gptq_gemm_gcu(xd, dev(w8[0]), torch.empty(0, device="cuda"), torch.from_numpy(sg[0]).to(dtype).cuda(),
                            torch.empty(0, device="cuda"), 8, None, g)
    want = o8.weight_only_int8(xh, w8[0], sg[0], g)
    np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)
    # grouped
    tw, ids, _ = om.topk_softmax(rng.standard_normal((M, E)).astype(np.float32), T, True)
    C = torch.empty((M, T, N), dtype=dtype, device="cuda")
    run_grouped(fmoe, xd, dev(w8), C, None, torch.from_numpy(sg).to(dtype).cuda(), None, dev(tw), dev(ids), E, 32,
                True, T, use_int8_w8a16=True, block_shape=[0, g])

    def wf(e):
        return (w8[e].astype(np.float32).reshape(N, K // g, g) * sg[e].T.reshape(N, K // g, 1)).reshape(N, K).T

    want = om.fused_moe_gemm(xh, wf, ids, T, tw, True)
    np.testing.assert_allclose(C.view(-1, N).float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)


def make_w4a8_experts(rng, E, K, N):
    """Logical unsigned weights, their reference-layout int8 tensor [E, N, K/2]
    (memory [E, K/2, N], w4a8.py:199-220) and the AWQ checkpoint tensor."""
    wl = rng.integers(0, 16, size=(E, K, N), dtype=np.uint8)
    s = rng.uniform(0.002, 0.02, size=(E, K // 128, N)).astype(np.float32)
    awq = np.stack([ow4.awq_pack(wl[e]) for e in range(E)])
    ref = np.stack([ow4.rearrange_awq(awq[e], None, s[e], rearrange_group=64, zeros_in_int8=True, use_w4a8=True)[0]
                    for e in range(E)])                      # int8 [E, K/2, N]
    return wl, s, awq, ref


def test_w4a8_reference_layout_and_checkpoint_repack_bit_exact(rearrange):
    print("case w4a8 repack", flush=True)
    rng = np.random.default_rng(23)
    E, K, N = 3, 256, 384
    wl, s, awq, ref = make_w4a8_experts(rng, E, K, N)
    want = np.stack([ow4.native_pack(wl[e]) for e in range(E)])
    got_ref = rearrange.from_reference_w4a8(dev(ref).view(E, N, K // 2))
    got_awq, _ = rearrange.rearrange_uint4_int32_awq(dev(awq), None)
    assert np.array_equal(got_ref.cpu().numpy(), want)
    assert np.array_equal(got_awq.cpu().numpy(), want)


@pytest.mark.parametrize("dtype,block,mul", [(torch.bfloat16, 16, False), (torch.float16, 64, True),
                                            (torch.bfloat16, 128, True)])
def test_fused_moe_quant_kernel_ex_w4a8(fmoe, rearrange, dtype, block, mul):
    """fp8 activations x symmetric int4 experts with fp32 group scales, divided by the
    reciprocal input scale: out[t] = (deq(A)[t / T] @ ((w - 8) s)[e]) / A_scale_rec."""
    print(f"case w4a8 grouped {dtype} block={block} mul={mul}", flush=True)
    rng = np.random.default_rng(29 + block)
    M, E, T, K, N = 41, 4, 2, 256, 384
    wl, s, awq, ref = make_w4a8_experts(rng, E, K, N)
    a_scale = np.float32(0.037)
    x = rng.standard_normal((M, K)).astype(np.float32)
    xq = of8.to_e4m3fn(np.clip(x / a_scale, -448, 448))                    # codes
    tw, ids, _ = om.topk_softmax(rng.standard_normal((M, E)).astype(np.float32), T, True)
    rec = torch.tensor([1.0 / a_scale], dtype=torch.float32, device="cuda")
    sort, eids, npp = fmoe.moe_align_block_size(dev(ids), block, E)
    a_deq = of8.from_e4m3fn(xq)
    want = om.fused_moe_gemm(a_deq, lambda e: (wl[e].astype(np.float32) - 8.0) * np.repeat(s[e], 128, 0), ids, T,
                             tw if mul else None, mul) * a_scale
    for how in ("reference layout", "slab"):
        B = dev(ref).view(E, N, K // 2) if how == "reference layout" else rearrange.rearrange_uint4_int32_awq(dev(awq), None)[0]
        C = torch.full((M, T, N), float("nan"), dtype=dtype, device="cuda")
        torch.ops._C.fused_moe_quant_kernel_ex(C, dev(xq).view(torch.float8_e4m3fn), B, rec, dev(s), None, None,
                                               dev(tw), dev(ids), sort, eids, npp, None, mul, T, block, 128, -1)
        torch.cuda.synchronize()
        got = C.view(-1, N).float().cpu().numpy()
        np.testing.assert_allclose(got, want, rtol=RTOL, atol=ATOL, err_msg=how)


# ---------------------------------------------------- whole sequence ----
def build_moe(mode):
    from vllm_gcu_amd.kernels.modular_experts import TritonExpertsPad
    from vllm_gcu_amd.kernels.modular_kernel import FusedMoEModularKernel
    from vllm_gcu_amd.kernels.prepare_finalize import MoEPrepareAndFinalizeNoEP
    if mode == "w4a16":
        fe = TritonExpertsPad(use_int4_w4a16=True, block_shape=[0, 128])
    else:
        fe = TritonExpertsPad(use_fp8_w8a8=True, block_shape=[128, 128])
    return FusedMoEModularKernel(MoEPrepareAndFinalizeNoEP(), fe)


@pytest.mark.parametrize("M,E,T,H,I", [(64, 8, 2, 512, 768), (5, 4, 2, 256, 256), (300, 8, 2, 512, 1024)])
def test_fused_experts_w4a16_sequence(ops, rearrange, M, E, T, H, I):
    print(f"case fused w4a16 M={M} E={E}", flush=True)
    rng = np.random.default_rng(M)
    q13, z13, s13 = make_int4_experts(rng, E, H, 2 * I)
    q2, z2, s2 = make_int4_experts(rng, E, I, H)
    w13, zp13 = int4_to_device(rearrange, q13, z13)
    w2, zp2 = int4_to_device(rearrange, q2, z2)
    x = rng.standard_normal((M, H)).astype(np.float16)
    logits = rng.standard_normal((M, E)).astype(np.float32)
    tw, ids = ops.fused_topk(None, dev(logits), T, True)
    out = build_moe("w4a16")(dev(x), w13, w2, tw, ids, w1_scale=dev(s13), w2_scale=dev(s2), w1_zp=zp13, w2_zp=zp2)
    two, ido, _ = om.topk_softmax(logits, T, True)
    assert np.array_equal(ids.cpu().numpy(), ido)
    want = om.fused_experts(x.astype(np.float32), lambda e: ow4.dequantize(q13[e], z13[e], s13[e], 128),
                            lambda e: ow4.dequantize(q2[e], z2[e], s2[e], 128), two, ido, f16)
    np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("M,E,T,H,I", [(48, 16, 4, 512, 256), (400, 8, 2, 512, 256)])
def test_fused_experts_fp8_block_sequence(ops, fmoe, M, E, T, H, I):
    """The whole fused-experts sequence on fp8 block-scaled experts; the second case has 100 rows per expert
    on average, where the configuration takes align blocks of 128 slots and both GEMMs run the MFMA tile
    kernel with gathered rows (the upper half of every row tile only copies)."""
    print(f"case fused fp8 M={M} E={E}", flush=True)
    assert fmoe.get_default_config(M, E, 2 * I, H, T, None, False, [128, 128])["BLOCK_SIZE_M"] == (128 if M == 400 else 16)
    assert fmoe.get_default_config(4 * M, E, 2 * I, H, T, None, False, [128, 128])["BLOCK_SIZE_M"] == (256 if M == 400 else 128)
    assert fmoe.get_default_config(3 * M, E, 2 * I, H, T, None, False, [0, 128])["BLOCK_SIZE_M"] == 64      # (W4A16 experts: 64)
    rng = np.random.default_rng(3)
    w13 = of8.to_e4m3fn(np.clip(rng.standard_normal((E, 2 * I, H)) * 0.5, -448, 448).astype(np.float32))
    w2 = of8.to_e4m3fn(np.clip(rng.standard_normal((E, H, I)) * 0.5, -448, 448).astype(np.float32))
    s13 = rng.uniform(0.02, 0.1, size=(E, 2 * I // 128, H // 128)).astype(np.float32)
    s2 = rng.uniform(0.02, 0.1, size=(E, H // 128, I // 128)).astype(np.float32)
    x = torch.from_numpy(rng.standard_normal((M, H)).astype(np.float32)).to(torch.bfloat16)
    logits = rng.standard_normal((M, E)).astype(np.float32)
    groups = 4 if E >= 16 else 2
    tw, ids = fmoe.grouped_topk(x.cuda(), dev(logits), T, True, groups, 2, "sigmoid", None)
    out = build_moe("fp8")(x.cuda(), dev(w13).view(torch.float8_e4m3fn), dev(w2).view(torch.float8_e4m3fn), tw, ids,
                           w1_scale=dev(s13), w2_scale=dev(s2))
    two, ido = om.grouped_topk(logits, T, True, groups, 2, "sigmoid", None)
    assert np.array_equal(ids.cpu().numpy(), ido)

    def deq(codes, sc):
        return (of8.from_e4m3fn(codes) * np.repeat(np.repeat(sc, 128, 0), 128, 1)).T   # [K, N]

    def qdq(a):                     # per-token-group fp8 round trip of an activation
        qa, sa = of8.per_token_group_quant_fp8(a, 128)
        return of8.from_e4m3fn(qa) * np.repeat(sa, 128, -1)

    want = om.fused_experts(qdq(x.float().numpy()), lambda e: deq(w13[e], s13[e]), lambda e: deq(w2[e], s2[e]),
                            two, ido, bf16, quant_a2=qdq)
    got = out.float().cpu().numpy()
    np.testing.assert_allclose(got, want, rtol=RTOL, atol=ATOL)


def test_config3_full_size_properties_and_sample(ops, rearrange):
    # benchmark configuration 3: 512 tokens, hidden 4096, 8 experts, intermediate 14336, top-2, int4 g=128
    print("case config3", flush=True)
    M, E, T, H, I = 512, 8, 2, 4096, 14336
    g = torch.Generator().manual_seed(0)
    w13 = torch.randint(-2**31, 2**31 - 1, (E, H // 8, 2 * I), dtype=torch.int32, generator=g)   # GPTQ words
    w2 = torch.randint(-2**31, 2**31 - 1, (E, I // 8, H), dtype=torch.int32, generator=g)
    z13 = torch.randint(-2**31, 2**31 - 1, (E, H // 128, 2 * I // 8), dtype=torch.int32, generator=g)
    z2 = torch.randint(-2**31, 2**31 - 1, (E, I // 128, H // 8), dtype=torch.int32, generator=g)
    s13 = (torch.rand(E, H // 128, 2 * I, generator=g) * 0.009 + 0.001).to(torch.float16)
    s2 = (torch.rand(E, I // 128, H, generator=g) * 0.009 + 0.001).to(torch.float16)
    x = torch.randn(M, H, generator=g).to(torch.float16)
    logits = torch.randn(M, E, generator=g)
    w13d, zp13 = rearrange.rearrange_uint4_int32_gptq(w13.cuda(), z13.cuda())
    w2d, zp2 = rearrange.rearrange_uint4_int32_gptq(w2.cuda(), z2.cuda())
    moe = build_moe("w4a16")
    tw, ids = ops.fused_topk(None, logits.cuda(), T, True)
    kw = dict(w1_scale=s13.cuda(), w2_scale=s2.cuda(), w1_zp=zp13, w2_zp=zp2)
    out = moe(x.cuda(), w13d, w2d, tw, ids, **kw)
    # permuting the tokens permutes the outputs bit for bit (rows are independent)
    perm = torch.randperm(M, generator=g)
    out_p = moe(x[perm].cuda(), w13d, w2d, tw[perm.cuda()], ids[perm.cuda()], **kw)
    assert torch.equal(out_p, out[perm.cuda()])
    # up to sixteen tokens against the oracle: for every expert and slot position the first token routed
    # there (each expert is dequantised once per GEMM on the CPU)
    two, ido, _ = om.topk_softmax(logits.numpy(), T, True)
    assert np.array_equal(ids.cpu().numpy(), ido)
    toks = []
    for e in range(E):
        for slot in range(T):
            toks += [int(t) for t in np.nonzero(ido[:, slot] == e)[0][:1]]
    toks = sorted(set(toks))
    assert len(toks) >= 8 and set(np.unique(ido[toks])) == set(range(E))

    buf = np.empty(H * 2 * I, np.float32)      # one dense expert matrix, reused: sixteen of them are dequantised

    def expert(wq, zq, sc, e, rows=512):
        K, N = wq.shape[1] * 8, wq.shape[2]
        dense = buf[:K * N].reshape(K, N)
        wn, zn, sn = wq[e].numpy(), zq[e].numpy(), sc[e].numpy()
        for k0 in range(0, K, rows):
            dense[k0:k0 + rows] = ow4.dequantize(ow4.gptq_unpack_weight(wn[k0 // 8:(k0 + rows) // 8]),
                                                 ow4.gptq_unpack_zeros(zn[k0 // 128:(k0 + rows) // 128]),
                                                 sn[k0 // 128:(k0 + rows) // 128], 128)
        return dense

    want, slots = om.fused_experts(x[toks].float().numpy(), lambda e: expert(w13, z13, s13, e),
                                   lambda e: expert(w2, z2, s2, e), two[toks], ido[toks], f16, return_slots=True)
    got = out[toks].float().cpu().numpy()
    # The layer stores each slot's term in fp16 before the sum (modular_experts.py:257-288).  Terms reach
    # 8..32 here, where fp16 steps are 2^-7..2^-6, and outputs are differences of such terms: a term whose
    # fp32 value rounds the other way moves the sum by one step of that term however small the sum is.  So
    # the bound per output is rtol * |want| + atol plus one fp16 step of each of its terms.
    step = np.where(slots != 0, 2.0 ** (np.floor(np.log2(np.maximum(np.abs(slots), 2.0 ** -14))) - 10), 0.0).sum(axis=1)
    err = np.abs(got - want)
    bound = ATOL + RTOL * np.abs(want) + step
    assert (err <= bound).all(), f"max excess {(err - bound).max()} at {np.unravel_index((err - bound).argmax(), err.shape)}"
    # and without that allowance all but a handful of the outputs are inside the plain tolerance
    assert (err > ATOL + RTOL * np.abs(want)).mean() < 1e-3


@pytest.mark.parametrize("block", [16, 32, 64])
def test_expert_map_with_non_local_experts_zeroes_their_rows(fmoe, ops, rearrange, block):
    """Under an expert map the reference maps non-local experts to -1 (fused_moe.py:70-71, 106-107).
    Blocks of such experts must read no weights and leave zeros in their slot rows; local experts are
    renumbered.  Checked through both align paths and the three grouped kernels (int4 streaming /
    MFMA tile by block size, K-contiguous fp16)."""
    print(f"case expert_map -1 block={block}", flush=True)
    rng = np.random.default_rng(40 + block)
    M, E, T, K, N = 45, 6, 2, 256, 384
    emap = np.array([-1, 0, -1, 1, 2, -1], dtype=np.int32)      # 3 local experts
    L = 3
    q, z, s = make_int4_experts(rng, L, K, N)
    w, zp = int4_to_device(rearrange, q, z)
    x = rng.standard_normal((M, K)).astype(np.float16)
    tw, ids, _ = om.topk_softmax(rng.standard_normal((M, E)).astype(np.float32), T, True)
    flat = ids.reshape(-1)
    assert (emap[flat] < 0).any() and (emap[flat] >= 0).any()
    wf = lambda e: ow4.dequantize(q[e], z[e], s[e].astype(np.float32), 128)
    want = np.zeros((M * T, N), dtype=np.float32)
    for t in range(M * T):
        le = emap[flat[t]]
        if le >= 0:
            want[t] = x[t // T].astype(np.float32) @ wf(le)
    cfg = {"BLOCK_SIZE_M": block}
    count = torch.full((1,), M, dtype=torch.int32, device="cuda")
    for topk_ids_size in (None, count):      # plain align + host-side map; exts align with the map inside
        so, eo, no = fmoe.moe_align_block_size(dev(ids), block, E, dev(emap), topk_ids_size)
        assert (eo[: int(no.item()) // block].cpu().numpy() < L).all()
        C = torch.full((M, T, N), float("nan"), dtype=torch.float16, device="cuda")
        fmoe.invoke_fused_moe_kernel(dev(x), w, C, None, dev(s), zp, dev(tw), dev(ids), so, eo, no, False, T, cfg,
                                     use_fp8_w8a8=False, use_int8_w8a8=False, use_int8_w8a16=False,
                                     use_int4_w4a16=True, block_shape=[0, 128])
        torch.cuda.synchronize()
        got = C.view(-1, N).float().cpu().numpy()
        assert np.isfinite(got).all()
        assert (got[emap[flat] < 0] == 0).all()
        np.testing.assert_allclose(got, want, rtol=RTOL, atol=ATOL)
    # the K-contiguous kernel (unquantised fp16 experts)
    wf16 = (rng.standard_normal((L, N, K)) * 0.05).astype(np.float16)
    so, eo, no = fmoe.moe_align_block_size(dev(ids), block, E, dev(emap), None)
    C = torch.full((M, T, N), float("nan"), dtype=torch.float16, device="cuda")
    fmoe.invoke_fused_moe_kernel(dev(x), dev(wf16), C, None, None, None, dev(tw), dev(ids), so, eo, no, False, T, cfg,
                                 use_fp8_w8a8=False, use_int8_w8a8=False, use_int8_w8a16=False, use_int4_w4a16=False)
    torch.cuda.synchronize()
    got = C.view(-1, N).float().cpu().numpy()
    want = np.zeros((M * T, N), dtype=np.float32)
    for t in range(M * T):
        le = emap[flat[t]]
        if le >= 0:
            want[t] = x[t // T].astype(np.float32) @ wf16[le].astype(np.float32).T
    assert (got[emap[flat] < 0] == 0).all()
    np.testing.assert_allclose(got, want, rtol=RTOL, atol=ATOL)


def test_config4_full_size_properties_and_samples(ops, fmoe, rearrange, monkeypatch):
    """Benchmark configuration 4 at full size: 256 tokens, hidden 7168, 256 routed experts, intermediate
    2048, top-8 with grouped routing (8 groups, top-4), fp8-e4m3 weights ~ N(0, 0.02) with 128 x 128
    block scales in the kslab order, per-token-per-128 fp8 activations, bf16 output.  Size-independent
    property: permuting the tokens permutes the outputs bit for bit; three tokens are compared with
    the CPU oracle (only their experts are dequantised there) within rtol = atol = 1e-2."""
    print("case config4", flush=True)
    M, E, T, H, I = 256, 256, 8, 7168, 2048
    torch.manual_seed(4)
    w13 = torch.empty((E, 2 * I, H), dtype=torch.float8_e4m3fn, device="cuda")
    w2 = torch.empty((E, H, I), dtype=torch.float8_e4m3fn, device="cuda")
    for e in range(E):                                  # N(0, 0.02) rounded to e4m3fn, drawn on the device
        w13[e] = (torch.randn(2 * I, H, device="cuda") * 0.02).to(torch.float8_e4m3fn)
        w2[e] = (torch.randn(H, I, device="cuda") * 0.02).to(torch.float8_e4m3fn)
    s13 = torch.rand(E, 2 * I // 128, H // 128, device="cuda") + 0.5
    s2 = torch.rand(E, H // 128, I // 128, device="cuda") + 0.5
    g = torch.Generator().manual_seed(4)
    x = torch.randn(M, H, generator=g).to(torch.bfloat16)
    logits = torch.randn(M, E, generator=g)
    tw, ids = fmoe.grouped_topk(x.cuda(), logits.cuda(), T, True, 8, 4, "softmax", None)
    two, ido = om.grouped_topk(logits.numpy(), T, True, 8, 4, "softmax", None)
    assert np.array_equal(ids.cpu().numpy(), ido)
    w13k, w2k = rearrange.to_kslab(w13), rearrange.to_kslab(w2)
    moe = build_moe("fp8")
    kw = dict(w1_scale=s13, w2_scale=s2)
    out = moe(x.cuda(), w13k, w2k, tw, ids, **kw)
    torch.cuda.synchronize()
    assert out.shape == (M, H) and out.dtype == torch.bfloat16 and torch.isfinite(out).all()
    perm = torch.randperm(M, generator=g)
    out_p = moe(x[perm].cuda(), w13k, w2k, tw[perm.cuda()], ids[perm.cuda()], **kw)
    assert torch.equal(out_p, out[perm.cuda()])
    # row-major weights (the checkpoint's order) give the same bits
    monkeypatch.setattr(ops, "_AUTO_KSLAB", False)
    out_r = moe(x.cuda(), w13, w2, tw, ids, **kw)
    assert torch.equal(out_r, out)

    def deq(w, sc, e):
        codes = w[e].view(torch.uint8).cpu().numpy()
        return (of8.from_e4m3fn(codes) * np.repeat(np.repeat(sc[e].cpu().numpy(), 128, 0), 128, 1)).T   # [K, N]

    def qdq(a):
        qa, sa = of8.per_token_group_quant_fp8(a, 128)
        return of8.from_e4m3fn(qa) * np.repeat(sa, 128, -1)

    xf = x.float().numpy()
    for tok in (0, 101, 255):
        want = om.fused_experts(qdq(xf[tok:tok + 1]), lambda e: deq(w13, s13, e), lambda e: deq(w2, s2, e),
                                two[tok:tok + 1], ido[tok:tok + 1], bf16, quant_a2=qdq)
        got = out[tok:tok + 1].float().cpu().numpy()
        assert np.abs(want).max() > 0.05                    # the comparison is not vacuous
        np.testing.assert_allclose(got, want, rtol=RTOL, atol=ATOL, err_msg=f"token {tok}")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_grouped_w4a16_split_k_long_k_narrow_n(fmoe, ops, rearrange, dtype):
    """Second-GEMM shape (long K, few column tiles, blocks of 64): the launch splits K into fp32 partial
    tiles and a second kernel adds them, applies the routing weight and zeroes the rows of non-local
    experts.  Checked against the oracle and against the unsplit launch (no workspace)."""
    from vllm_gcu_amd import _lib
    print(f"case grouped split-K {dtype}", flush=True)
    rng = np.random.default_rng(77)
    M, E, K, N = 300, 5, 4096, 256                        # M slots, topk = 1 as in the second GEMM
    emap = np.array([0, 1, -1, 2, 3], dtype=np.int32)
    L = 4
    blocks = M // 64 + E
    assert _lib.load().mi355q_moe_gemm_workspace_bytes(_lib.Q_W4A16, M, 64, M + E * 63, L, K, N) > 0
    qw = rng.integers(-2**31, 2**31 - 1, size=(L, K // 8, N), dtype=np.int64).astype(np.int32)
    q = np.stack([ow4.gptq_unpack_weight(qw[e]) for e in range(L)])
    z = rng.integers(0, 16, size=(L, K // 128, N), dtype=np.uint8)
    s = rng.uniform(0.001, 0.01, size=(L, K // 128, N)).astype(np.float16)
    qz = np.stack([ow4.gptq_pack_zeros(z[e]) for e in range(L)])
    w, zp = rearrange.rearrange_uint4_int32_gptq(dev(qw), dev(qz))
    x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(dtype)
    sd = torch.from_numpy(s).to(dtype)
    ids = rng.integers(0, E, size=(M, 1)).astype(np.int32)
    tw = rng.uniform(0.1, 1.0, size=(M, 1)).astype(np.float32)
    so, eo, no = fmoe.moe_align_block_size(dev(ids), 64, E, dev(emap), None)
    assert blocks >= int(no.item()) // 64
    cfg = {"BLOCK_SIZE_M": 64}
    kw = dict(use_fp8_w8a8=False, use_int8_w8a8=False, use_int8_w8a16=False, use_int4_w4a16=True, block_shape=[0, 128])
    C = torch.full((M, 1, N), float("nan"), dtype=dtype, device="cuda")
    fmoe.invoke_fused_moe_kernel(x.cuda(), w, C, None, sd.cuda(), zp, dev(tw), dev(ids), so, eo, no, True, 1, cfg, **kw)
    torch.cuda.synchronize()
    got = C.view(M, N).float().cpu().numpy()
    want = np.zeros((M, N), dtype=np.float32)
    for t in range(M):
        le = emap[ids[t, 0]]
        if le >= 0:
            want[t] = (x[t].float().numpy() @ ow4.dequantize(q[le], z[le], sd[le].float().numpy(), 128)) * tw[t, 0]
    assert np.isfinite(got).all() and (got[emap[ids[:, 0]] < 0] == 0).all()
    np.testing.assert_allclose(got, want, rtol=RTOL, atol=ATOL)


def test_grouped_split_k_leaves_rows_of_dropped_ids_alone(fmoe, ops, rearrange):
    """Ids the alignment drops -- experts outside [0, E) and rows past the valid count of the `_pad`
    operators -- sit in no block, so no split writes their partial tiles.  The split-K reduction must
    not read those (stale, possibly NaN) partial rows: their output rows keep what they held, as with
    the unsplit launch."""
    from vllm_gcu_amd import _lib
    from vllm_gcu_amd.kernels import _runtime as rt
    print("case grouped split-K with dropped ids", flush=True)
    rng = np.random.default_rng(78)
    M, E, K, N = 300, 4, 4096, 256
    valid = 260                                            # rows past this count are padding
    assert _lib.load().mi355q_moe_gemm_workspace_bytes(_lib.Q_W4A16, M, 64, (M + E * 63) // 64, E, K, N) > 0
    q, z, s = make_int4_experts(rng, E, K, N)
    w, zp = int4_to_device(rearrange, q, z)
    x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).half()
    ids = rng.integers(0, E, size=(M, 1)).astype(np.int32)
    ids[rng.choice(valid, 40, replace=False), 0] = E + 3   # out of range: dropped
    tw = rng.uniform(0.1, 1.0, size=(M, 1)).astype(np.float32)
    so, eo, no = fmoe.moe_align_block_size(dev(ids), 64, E, None, torch.tensor([valid], dtype=torch.int32).cuda())
    # poison the workspace the launch will use, so a read of an unwritten partial row shows
    ws = rt.workspace(torch.device("cuda", torch.cuda.current_device()), 1)
    ws[1 << 20:(1 << 20) + 4 * 4 * M * N].view(torch.float32).fill_(float("nan"))
    cfg = {"BLOCK_SIZE_M": 64}
    kw = dict(use_fp8_w8a8=False, use_int8_w8a8=False, use_int8_w8a16=False, use_int4_w4a16=True, block_shape=[0, 128])
    C = torch.full((M, 1, N), 123.0, dtype=torch.float16, device="cuda")
    fmoe.invoke_fused_moe_kernel(x.cuda(), w, C, None, dev(s), zp, dev(tw), dev(ids), so, eo, no, True, 1, cfg, **kw)
    torch.cuda.synchronize()
    got = C.view(M, N).float().cpu().numpy()
    live = (np.arange(M) < valid) & (ids[:, 0] < E)
    assert (got[~live] == 123.0).all(), "rows of dropped ids were written"
    for t in np.nonzero(live)[0][::7]:
        e = ids[t, 0]
        want = (x[t].float().numpy() @ ow4.dequantize(q[e], z[e], s[e].astype(np.float32), 128)) * tw[t, 0]
        np.testing.assert_allclose(got[t], want, rtol=RTOL, atol=ATOL)
    assert np.isfinite(got).all()
