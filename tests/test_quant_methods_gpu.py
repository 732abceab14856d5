"""The quantization method classes (create_weights -> load checkpoint tensors ->
process_weights_after_loading -> apply) against the CPU oracle, the way a
model layer drives them (gptq.py:105-296, awq.py:69-134, w8a8.py:88-171,
fp8.py:49-205, moe_wna16.py:160-643 of the reference)."""
import numpy as np
import pytest
import torch

from oracle import fp8 as of8
from oracle import moe as om
from oracle import w4 as ow4
from oracle import w8a8 as o8

pytestmark = pytest.mark.gpu
RTOL = ATOL = 1e-2


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def load(layer, name, value):
    p = getattr(layer, name)
    assert tuple(p.shape) == tuple(value.shape), (name, p.shape, value.shape)
    p.data = value.to(p.dtype) if value.dtype != p.dtype else value


def int4_case(rng, K, N, g):
    q = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    z = rng.integers(0, 16, size=(K // g, N), dtype=np.uint8)
    s = rng.uniform(0.001, 0.01, size=(K // g, N)).astype(np.float16)
    return q, z, s


@pytest.mark.parametrize("M", [1, 16, 300])
def test_gptq_linear_method(M):
    from vllm_gcu_amd.kernels.quantization.gptq import GPTQGCUConfig
    print(f"case gptq method M={M}", flush=True)
    K, N, g = 1024, 768, 128
    rng = np.random.default_rng(M)
    q, z, s = int4_case(rng, K, N, g)
    method = GPTQGCUConfig.from_config({"bits": 4, "group_size": g}).get_quant_method()
    layer = torch.nn.Module()
    method.create_weights(layer, K, [512, 256], K, N, torch.float16)
    layer.cuda()
    load(layer, "qweight", dev(ow4.gptq_pack_weight(q)))
    load(layer, "qzeros", dev(ow4.gptq_pack_zeros(z)))
    load(layer, "scales", dev(s))
    method.process_weights_after_loading(layer)
    x = rng.standard_normal((2, M, K)).astype(np.float16) if M == 16 else rng.standard_normal((M, K)).astype(np.float16)
    bias = rng.standard_normal(N).astype(np.float16)
    out = method.apply(layer, dev(x), dev(bias))
    want = ow4.w4a16_gemm(x.reshape(-1, K).astype(np.float32), q, z, s.astype(np.float32), g, bias.astype(np.float32))
    assert out.shape == x.shape[:-1] + (N,)
    np.testing.assert_allclose(out.float().cpu().numpy().reshape(-1, N), want, rtol=RTOL, atol=ATOL)
    assert method.apply(layer, dev(x[:0])).shape[0] == 0


def test_gptq_rejects_act_order_and_bad_group():
    from vllm_gcu_amd.kernels.quantization.gptq import GPTQGCUConfig
    method = GPTQGCUConfig(4, 128).get_quant_method()
    layer = torch.nn.Module()
    with pytest.raises(ValueError):
        method.create_weights(layer, 192, [128], 192, 128, torch.float16)
    method.create_weights(layer, 256, [128], 256, 128, torch.float16)
    layer.cuda()
    layer.g_idx.data = layer.g_idx.data.flip(0).contiguous()
    with pytest.raises(ValueError):
        method.process_weights_after_loading(layer)


def test_gptq_8bit_symmetric():
    from vllm_gcu_amd.kernels.quantization.gptq import GPTQGCUConfig
    K, N = 512, 256
    rng = np.random.default_rng(8)
    w = rng.integers(0, 256, size=(K, N), dtype=np.uint8)                 # stored value, true weight = w - 128
    s = rng.uniform(0.001, 0.01, size=(1, N)).astype(np.float16)
    method = GPTQGCUConfig(8, -1).get_quant_method()
    layer = torch.nn.Module()
    method.create_weights(layer, K, [N], K, N, torch.float16)
    layer.cuda()
    packed = w.reshape(K // 4, 4, N).astype(np.uint32)
    packed = (packed[:, 0] | (packed[:, 1] << 8) | (packed[:, 2] << 16) | (packed[:, 3] << 24)).view(np.int32)
    load(layer, "qweight", dev(packed))
    load(layer, "qzeros", dev(np.full((1, N // 4), 0x7f7f7f7f, dtype=np.int32)))
    load(layer, "scales", dev(s))
    method.process_weights_after_loading(layer)
    x = rng.standard_normal((7, K)).astype(np.float16)
    out = method.apply(layer, dev(x))
    want = x.astype(np.float32) @ ((w.astype(np.float32) - 128) * s.astype(np.float32))
    np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)
    layer.qzeros = None
    layer2 = torch.nn.Module()
    method.create_weights(layer2, K, [N], K, N, torch.float16)
    layer2.cuda()
    layer2.qzeros.data.zero_()
    with pytest.raises(ValueError):
        method.process_weights_after_loading(layer2)


@pytest.mark.parametrize("M,dtype", [(4, torch.float16), (200, torch.bfloat16)])
def test_awq_linear_method(M, dtype):
    from vllm_gcu_amd.kernels.quantization.awq import AWQGCUConfig
    print(f"case awq method M={M}", flush=True)
    K, N, g = 512, 1024, 128
    rng = np.random.default_rng(M)
    q, z, s = int4_case(rng, K, N, g)
    method = AWQGCUConfig.from_config({"w_bit": 4, "q_group_size": g, "zero_point": True}).get_quant_method()
    layer = torch.nn.Module()
    method.create_weights(layer, K, [N], K, N, dtype)
    layer.cuda()
    load(layer, "qweight", dev(ow4.awq_pack(q)))
    load(layer, "qzeros", dev(ow4.awq_pack(z)))
    sd = torch.from_numpy(s).to(dtype)
    load(layer, "scales", sd.cuda())
    method.process_weights_after_loading(layer)
    x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(dtype)
    out = method.apply(layer, x.cuda())
    want = ow4.w4a16_gemm(x.float().numpy(), q, z, sd.float().numpy(), g)
    np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)


def test_w8a8_linear_method_static_input_scales():
    from vllm_gcu_amd.kernels.quantization.w8a8 import W8A8Config
    print("case w8a8 method", flush=True)
    M, K, N = 37, 512, 384
    rng = np.random.default_rng(5)
    w = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
    in_scales = rng.uniform(0.01, 0.05, size=K).astype(np.float16)
    out_scales = rng.uniform(1e-4, 1e-3, size=N).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float16)
    x = rng.standard_normal((M, K)).astype(np.float16)
    method = W8A8Config().get_quant_method()
    layer = torch.nn.Module()
    method.create_weights(layer, K, [N], K, N, torch.float16)
    layer.cuda()
    load(layer, "weight", dev(w))
    load(layer, "in_scales", dev(in_scales))
    load(layer, "out_scales", dev(out_scales))
    method.process_weights_after_loading(layer)
    out = method.apply(layer, dev(x), dev(bias))
    xq = o8.static_scaled_int8_quant(x, in_scales)
    acc = o8.int8_gemm_i32(xq, np.ascontiguousarray(w.T))
    want = o8.scaled_mm_epilogue(acc, 1.0, out_scales, bias.astype(np.float32))
    assert out.dtype == torch.float16 and out.shape == (M, N)
    np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)


def test_compressed_tensors_int8_kernel_dynamic():
    from vllm_gcu_amd.kernels.quantization.w8a8 import CompressedTensorMMLinearKernel
    M, K, N = 20, 256, 512
    rng = np.random.default_rng(6)
    w = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
    ws = rng.uniform(1e-3, 1e-2, size=(N, 1)).astype(np.float32)
    x = rng.standard_normal((2, M, K)).astype(np.float16)
    layer = torch.nn.Module()
    layer.weight = torch.nn.Parameter(dev(w), requires_grad=False)
    layer.weight_scale = torch.nn.Parameter(dev(ws), requires_grad=False)
    k = CompressedTensorMMLinearKernel()
    k.process_weights_after_loading(layer)
    out = k.apply_weights(layer, dev(x))
    xq, xs = o8.dynamic_scaled_int8_quant(x.reshape(-1, K))
    want = o8.scaled_mm_epilogue(o8.int8_gemm_i32(xq, np.ascontiguousarray(w.T)), xs, ws.reshape(-1))
    assert out.shape == (2, M, N)
    np.testing.assert_allclose(out.float().cpu().numpy().reshape(-1, N), want, rtol=RTOL, atol=ATOL)


def test_fp8_linear_method_block_scaled():
    from vllm_gcu_amd.kernels.quantization.fp8 import Fp8GCUConfig
    print("case fp8 method", flush=True)
    M, K, N = 33, 512, 768
    rng = np.random.default_rng(7)
    w = of8.to_e4m3fn(np.clip(rng.standard_normal((N, K)) * 0.5, -448, 448).astype(np.float32))
    ws = rng.uniform(0.02, 0.1, size=(N // 128, K // 128)).astype(np.float32)
    x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(torch.bfloat16)
    bias = torch.from_numpy(rng.standard_normal(N).astype(np.float32)).to(torch.bfloat16)
    layer = torch.nn.Module()
    layer.weight = torch.nn.Parameter(dev(w).view(torch.float8_e4m3fn), requires_grad=False)
    layer.weight_scale_inv = torch.nn.Parameter(dev(ws), requires_grad=False)
    method = Fp8GCUConfig.from_config({"weight_block_size": [128, 128]}).get_quant_method()
    before = method.apply(layer, x.cuda(), bias.cuda())
    method.process_weights_after_loading(layer)
    assert getattr(layer.weight, "_mi355q_kslab", False)          # re-ordered in place at load time
    out = method.apply(layer, x.cuda(), bias.cuda())
    assert torch.equal(before, out)
    xq, xs = of8.per_token_group_quant_fp8(x.float().numpy(), 128)
    want = of8.block_fp8_gemm(xq, xs, w, ws) + bias.float().numpy()
    assert out.dtype == torch.bfloat16 and out.shape == (M, N)
    np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("fmt", ["gptq", "awq"])
def test_moe_wna16_method(fmt):
    from vllm_gcu_amd.kernels.quantization.moe_wna16 import MoeWNA16GCUConfig
    print(f"case moe_wna16 method {fmt}", flush=True)
    M, E, T, H, I, g = 40, 8, 2, 512, 384, 128
    rng = np.random.default_rng(9)
    q13 = rng.integers(0, 16, size=(E, H, 2 * I), dtype=np.uint8)
    q2 = rng.integers(0, 16, size=(E, I, H), dtype=np.uint8)
    z13 = rng.integers(0, 16, size=(E, H // g, 2 * I), dtype=np.uint8)
    z2 = rng.integers(0, 16, size=(E, I // g, H), dtype=np.uint8)
    s13 = rng.uniform(0.001, 0.01, size=(E, H // g, 2 * I)).astype(np.float16)
    s2 = rng.uniform(0.001, 0.01, size=(E, I // g, H)).astype(np.float16)
    pw = ow4.gptq_pack_weight if fmt == "gptq" else ow4.awq_pack
    pz = ow4.gptq_pack_zeros if fmt == "gptq" else ow4.awq_pack
    layer = torch.nn.Module()
    for name, qq, zz, ss in (("w13", q13, z13, s13), ("w2", q2, z2, s2)):
        setattr(layer, f"{name}_qweight", torch.nn.Parameter(dev(np.stack([pw(a) for a in qq])), requires_grad=False))
        setattr(layer, f"{name}_qzeros", torch.nn.Parameter(dev(np.stack([pz(a) for a in zz])), requires_grad=False))
        setattr(layer, f"{name}_scales", torch.nn.Parameter(dev(ss), requires_grad=False))
    method = MoeWNA16GCUConfig(fmt, 4, g, True).get_quant_method()
    method.process_weights_after_loading(layer)
    x = rng.standard_normal((M, H)).astype(np.float16)
    logits = rng.standard_normal((M, E)).astype(np.float32)
    out = method.apply(layer, dev(x).clone(), dev(logits), top_k=T, renormalize=True)
    two, ido, _ = om.topk_softmax(logits, T, True)
    f16 = lambda a: a.astype(np.float16).astype(np.float32)   # noqa: E731
    want = om.fused_experts(x.astype(np.float32), lambda e: ow4.dequantize(q13[e], z13[e], s13[e].astype(np.float32), g),
                            lambda e: ow4.dequantize(q2[e], z2[e], s2[e].astype(np.float32), g), two, ido, f16)
    np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)


def test_fp8_and_int8_moe_methods_grouped_routing():
    from vllm_gcu_amd.kernels.quantization.fp8 import Fp8GCUConfig
    from vllm_gcu_amd.kernels.quantization.w8a8 import W8A8Config
    print("case fp8/int8 moe methods", flush=True)
    M, E, T, H, I = 24, 16, 4, 256, 256
    rng = np.random.default_rng(10)
    x = torch.from_numpy(rng.standard_normal((M, H)).astype(np.float32)).to(torch.bfloat16)
    logits = rng.standard_normal((M, E)).astype(np.float32)
    two, ido = om.grouped_topk(logits, T, True, 4, 2, "sigmoid", None)
    bf16 = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(torch.bfloat16).float().numpy()   # noqa: E731
    route = dict(top_k=T, renormalize=True, use_grouped_topk=True, topk_group=2, num_expert_group=4,
                 scoring_func="sigmoid")
    # fp8 block-scaled experts
    w13 = of8.to_e4m3fn(np.clip(rng.standard_normal((E, 2 * I, H)) * 0.5, -448, 448).astype(np.float32))
    w2 = of8.to_e4m3fn(np.clip(rng.standard_normal((E, H, I)) * 0.5, -448, 448).astype(np.float32))
    s13 = rng.uniform(0.02, 0.1, size=(E, 2 * I // 128, H // 128)).astype(np.float32)
    s2 = rng.uniform(0.02, 0.1, size=(E, H // 128, I // 128)).astype(np.float32)
    layer = torch.nn.Module()
    layer.w13_weight = dev(w13).view(torch.float8_e4m3fn)
    layer.w2_weight = dev(w2).view(torch.float8_e4m3fn)
    layer.w13_weight_scale_inv, layer.w2_weight_scale_inv = dev(s13), dev(s2)
    method = Fp8GCUConfig().get_quant_method(moe=True)
    method.process_weights_after_loading(layer)
    assert layer.w13_weight._mi355q_kslab and layer.w2_weight._mi355q_kslab
    out = method.apply(layer, x.cuda().clone(), dev(logits), **route)

    def deq(codes, sc):
        return (of8.from_e4m3fn(codes) * np.repeat(np.repeat(sc, 128, 0), 128, 1)).T

    def qdq(a):
        qa, sa = of8.per_token_group_quant_fp8(a, 128)
        return of8.from_e4m3fn(qa) * np.repeat(sa, 128, -1)

    want = om.fused_experts(qdq(x.float().numpy()), lambda e: deq(w13[e], s13[e]), lambda e: deq(w2[e], s2[e]),
                            two, ido, bf16, quant_a2=qdq)
    np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)

    # int8 per-channel experts, per-token dynamic activations
    w13i = rng.integers(-127, 128, size=(E, 2 * I, H), dtype=np.int8)
    w2i = rng.integers(-127, 128, size=(E, H, I), dtype=np.int8)
    c13 = rng.uniform(1e-3, 4e-3, size=(E, 2 * I)).astype(np.float32)
    c2 = rng.uniform(1e-3, 4e-3, size=(E, H)).astype(np.float32)
    m8 = W8A8Config().get_quant_method(moe=True)
    layer8 = torch.nn.Module()
    m8.create_weights(layer8, E, H, I, torch.bfloat16)
    layer8.cuda()
    load(layer8, "w13_weight", dev(w13i)); load(layer8, "w2_weight", dev(w2i))
    load(layer8, "w13_out_scales", dev(c13)); load(layer8, "w2_out_scales", dev(c2))
    m8.process_weights_after_loading(layer8)
    assert layer8.w13_weight._mi355q_kslab and layer8.w2_weight._mi355q_kslab
    out8 = m8.apply(layer8, x.cuda().clone(), dev(logits), **route)

    def qdq8(a):
        qa, sa = o8.dynamic_scaled_int8_quant(a)
        return qa.astype(np.float32) * sa

    want8 = om.fused_experts(qdq8(x.float().numpy()), lambda e: (w13i[e].astype(np.float32) * c13[e][:, None]).T,
                             lambda e: (w2i[e].astype(np.float32) * c2[e][:, None]).T, two, ido, bf16, quant_a2=qdq8)
    np.testing.assert_allclose(out8.float().cpu().numpy(), want8, rtol=RTOL,
                               atol=ATOL)

    # the same experts under the compressed-tensors parameter names
    from vllm_gcu_amd.kernels.quantization.w8a8 import GCUCompressedTensorsW8A8Int8MoEMethod
    mc = GCUCompressedTensorsW8A8Int8MoEMethod()
    layerc = torch.nn.Module()
    mc.create_weights(layerc, E, H, I, torch.bfloat16)
    layerc.cuda()
    load(layerc, "w13_weight", dev(w13i)); load(layerc, "w2_weight", dev(w2i))
    load(layerc, "w13_weight_scale", dev(c13[:, :, None])); load(layerc, "w2_weight_scale", dev(c2[:, :, None]))
    mc.process_weights_after_loading(layerc)
    outc = mc.apply(layerc, x.cuda().clone(), dev(logits), **route)
    assert torch.equal(outc, out8)


@pytest.mark.parametrize("rearranged", [False, True])
def test_moe_w4a8_method(rearranged):
    """W4A8Config -> MoeW4A8Method: create_weights / load / process / apply against the float
    layer evaluated on the same quantised operands (fp8 activations with the static scales,
    symmetric int4 experts with fp32 group scales)."""
    from vllm_gcu_amd.kernels.quantization import QUANTIZATION_METHODS
    print(f"case w4a8 moe method rearranged={rearranged}", flush=True)
    M, E, T, H, I = 37, 8, 2, 256, 384
    rng = np.random.default_rng(31)
    cfg = QUANTIZATION_METHODS["w4a8_gcu"].from_config(
        {"quant_method": "w4a8", "bits": 4, "group_size": 128, "zero_point": False, "rearranged": rearranged})
    method = cfg.get_quant_method(moe=True)
    w13 = rng.integers(0, 16, size=(E, H, 2 * I), dtype=np.uint8)
    w2 = rng.integers(0, 16, size=(E, I, H), dtype=np.uint8)
    s13 = rng.uniform(0.002, 0.01, size=(E, H // 128, 2 * I)).astype(np.float32)
    s2 = rng.uniform(0.002, 0.01, size=(E, I // 128, H)).astype(np.float32)
    a1, a2 = np.float32(0.02), np.float32(0.05)            # activation scales; the checkpoint holds 1 / scale

    def ckpt(w, s):
        if not rearranged:
            return np.stack([ow4.awq_pack(w[e]) for e in range(E)])
        return np.stack([ow4.rearrange_awq(ow4.awq_pack(w[e]), None, s[e], rearrange_group=64, zeros_in_int8=True,
                                           use_w4a8=True)[0] for e in range(E)])

    layer = torch.nn.Module()
    method.create_weights(layer, E, H, I, torch.bfloat16)
    layer.cuda()
    load(layer, "w13_qweight", dev(ckpt(w13, s13))); load(layer, "w2_qweight", dev(ckpt(w2, s2)))
    load(layer, "w13_scales", dev(s13)); load(layer, "w2_scales", dev(s2))
    method.load_input_scale(layer.w13_input_scale, torch.tensor([1.0 / a1], device="cuda"))
    method.load_input_scale(layer.w2_input_scale, torch.tensor([1.0 / a2], device="cuda"))
    method.process_weights_after_loading(layer)
    assert layer.w13_qweight.dtype == torch.int32 and tuple(layer.w13_qweight.shape) == (E, H // 8, 2 * I)
    x = torch.from_numpy(rng.standard_normal((M, H)).astype(np.float32)).to(torch.bfloat16)
    logits = rng.standard_normal((M, E)).astype(np.float32)
    out = method.apply(layer, x.cuda(), dev(logits), top_k=T, renormalize=True)
    assert out.dtype == torch.bfloat16 and out.shape == (M, H)

    def fake_quant(v, sc):
        return of8.from_e4m3fn(of8.to_e4m3fn(np.clip(v / sc, -448, 448).astype(np.float32))) * sc

    bf16 = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(torch.bfloat16).float().numpy()   # noqa: E731
    two, ido, _ = om.topk_softmax(logits, T, True)
    want = om.fused_experts(fake_quant(x.float().numpy(), a1),
                            lambda e: (w13[e].astype(np.float32) - 8) * np.repeat(s13[e], 128, 0),
                            lambda e: (w2[e].astype(np.float32) - 8) * np.repeat(s2[e], 128, 0),
                            two, ido, bf16, quant_a2=lambda v: fake_quant(v, a2))
    np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)


def test_fused_qkv_ops_equal_the_unfused_gemm_split_by_columns():
    """``fused_qkv_proj`` / ``fused_qkv_gemm_quant`` (torch_bindings.cpp:1204-1217): the reference
    holds no caller, test or description of them (parity unpinned); what is checked is the
    definition this build gives them -- the merged GEMM, columns split into q and kv -- against the
    oracle of that GEMM."""
    from oracle import w4 as ow4
    from vllm_gcu_amd.kernels.quantization import rearrange
    print("case fused qkv ops", flush=True)
    rng = np.random.default_rng(21)
    M, K, NQ, NKV = 19, 512, 384, 128
    N = NQ + NKV
    # fp8 block-scaled
    w = of8.to_e4m3fn(np.clip(rng.standard_normal((N, K)) * 0.5, -448, 448).astype(np.float32))
    ws = rng.uniform(0.02, 0.1, size=(N // 128, K // 128)).astype(np.float32)
    xq, xs = of8.per_token_group_quant_fp8(rng.standard_normal((M, K)).astype(np.float32), 128)
    q = torch.full((M, NQ), float("nan"), dtype=torch.bfloat16, device="cuda")
    kv = torch.full((M, NKV), float("nan"), dtype=torch.bfloat16, device="cuda")
    torch.ops._C.fused_qkv_proj(q, kv, dev(xq).view(torch.float8_e4m3fn), dev(w).view(torch.float8_e4m3fn),
                                dev(xs), dev(ws), 128)
    want = of8.block_fp8_gemm(xq, xs, w, ws)
    got = torch.cat([q, kv], dim=1).float().cpu().numpy()
    np.testing.assert_allclose(got, want, rtol=RTOL, atol=ATOL)
    # W4A16, GPTQ checkpoint tensors
    g = 128
    qw = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    z = rng.integers(0, 16, size=(K // g, N), dtype=np.uint8)
    s = rng.uniform(0.001, 0.01, size=(K // g, N)).astype(np.float32)
    x = rng.standard_normal((M, K)).astype(np.float32)
    wq, zz = rearrange.rearrange_uint4_int32_gptq(dev(ow4.gptq_pack_weight(qw)), dev(ow4.gptq_pack_zeros(z)))
    q = torch.full((M, NQ), float("nan"), dtype=torch.float16, device="cuda")
    kv = torch.full((M, NKV), float("nan"), dtype=torch.float16, device="cuda")
    xh = torch.from_numpy(x).to(torch.float16)
    torch.ops._C.fused_qkv_gemm_quant(q, kv, xh.cuda(), wq, torch.from_numpy(s).to(torch.float16).cuda(), zz, g)
    sh = torch.from_numpy(s).to(torch.float16).float().numpy()
    want = ow4.w4a16_gemm(xh.float().numpy(), qw, z, sh, g)
    got = torch.cat([q, kv], dim=1).float().cpu().numpy()
    np.testing.assert_allclose(got, want, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("M,K,N", [(65, 384, 256), (129, 128, 128), (300, 512, 384), (513, 1024, 256), (2050, 256, 1152),
                                   (2305, 128, 1024), (4200, 128, 2048)])     # > 8 row tiles, XCD-aware order
@pytest.mark.parametrize("kslab", [False, True])
def test_fp8_block_gemm_tile_kernel(M, K, N, kslab, monkeypatch):
    """linear_quant above 64 rows (and enough output tiles) runs the MFMA tile kernel; checked against the oracle of the
    block-scaled GEMM and, bit for bit, between the two weight orders."""
    from vllm_gcu_amd.kernels import _custom_ops
    from vllm_gcu_amd.kernels.quantization import rearrange
    print(f"case fp8 tile M={M} K={K} N={N} kslab={kslab}", flush=True)
    monkeypatch.setattr(_custom_ops, "_FP8_TILE_MIN_TILES", 1)      # small shapes: take the tile kernel anyway
    rng = np.random.default_rng(M + K + N)
    w = of8.to_e4m3fn(np.clip(rng.standard_normal((N, K)) * 0.5, -448, 448).astype(np.float32))
    ws = rng.uniform(0.02, 0.1, size=(N // 128, K // 128)).astype(np.float32)
    xq, xs = of8.per_token_group_quant_fp8(rng.standard_normal((M, K)).astype(np.float32), 128)
    bias = torch.from_numpy(rng.standard_normal(N).astype(np.float32)).to(torch.bfloat16)
    wd = dev(w).view(torch.float8_e4m3fn)
    if kslab:
        wd = rearrange.to_kslab(wd)
    out = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    torch.ops._C.linear_quant(out, dev(xq).view(torch.float8_e4m3fn), wd, bias.cuda(), dev(xs), dev(ws))
    want = of8.block_fp8_gemm(xq, xs, w, ws) + bias.float().numpy()
    np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)
    if kslab:
        ref = torch.empty_like(out)
        torch.ops._C.linear_quant(ref, dev(xq).view(torch.float8_e4m3fn), dev(w).view(torch.float8_e4m3fn),
                                  bias.cuda(), dev(xs), dev(ws))
        assert torch.equal(out, ref)


def test_fp8_full_size_layer_tile_kernel_against_streaming_kernel(monkeypatch):
    """K = 8192, N = 28672, 300 rows: the MFMA tile kernel and the weight-streaming kernel are
    independent implementations of the same block-scaled sum; they must agree to fp32
    accumulation-order accuracy, and sampled entries must match the oracle."""
    from vllm_gcu_amd.kernels import _custom_ops
    from vllm_gcu_amd.kernels.quantization import rearrange
    print("case fp8 full size tile vs streamer", flush=True)
    M, K, N = 300, 8192, 28672
    g = torch.Generator(device="cuda").manual_seed(5)
    w = (torch.randn(N, K, device="cuda", generator=g) * 0.5).to(torch.float8_e4m3fn)
    ws = torch.rand(N // 128, K // 128, device="cuda", generator=g) * 0.05 + 0.02
    x = torch.randn(M, K, device="cuda", generator=g).to(torch.bfloat16)
    xq, xs = _custom_ops.per_token_group_quant_fp8(x, 128)
    wk = rearrange.to_kslab(w)
    tile = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    torch.ops._C.linear_quant(tile, xq, wk, None, xs, ws)
    monkeypatch.setattr(_custom_ops, "_FP8_TILE_MIN_M", 1 << 30)
    stream = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    torch.ops._C.linear_quant(stream, xq, wk, None, xs, ws)
    d = (tile.float() - stream.float()).abs()
    scale = stream.float().abs().max().item()
    assert d.max().item() <= 2 ** -7 * scale + 1e-3          # one bf16 ulp of the largest output
    rows = np.array([0, 150, 299])
    cols = np.random.default_rng(1).integers(0, N, size=48)
    want = of8.block_fp8_gemm(xq.view(torch.uint8)[rows].cpu().numpy(), xs[rows].cpu().numpy(),
                              w.view(torch.uint8).cpu().numpy()[np.concatenate([np.arange(c // 128 * 128, c // 128 * 128 + 128) for c in cols])],
                              np.repeat(ws.cpu().numpy()[cols // 128], 1, axis=0))
    want = want.reshape(3, len(cols), 128)[:, np.arange(len(cols)), cols % 128]
    got = tile[rows][:, cols].float().cpu().numpy()
    np.testing.assert_allclose(got, want, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("M", [65, 100, 128])
def test_fp8_dense_65_to_128_rows_single_block(M):
    """65..128 rows of the fp8 block-scaled linear run as one 128-row block of the weight-streaming
    kernel with K split over the workgroup's wavefronts."""
    print(f"case fp8 dense 128-row block M={M}", flush=True)
    rng = np.random.default_rng(M)
    K, N = 1024, 384
    w = of8.to_e4m3fn(np.clip(rng.standard_normal((N, K)) * 0.5, -448, 448).astype(np.float32))
    ws = rng.uniform(0.02, 0.1, size=(N // 128, K // 128)).astype(np.float32)
    xq, xs = of8.per_token_group_quant_fp8(rng.standard_normal((M, K)).astype(np.float32), 128)
    out = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    torch.ops._C.linear_quant(out, dev(xq).view(torch.float8_e4m3fn), dev(w).view(torch.float8_e4m3fn), None,
                              dev(xs), dev(ws))
    want = of8.block_fp8_gemm(xq, xs, w, ws)
    np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)


def test_moe_wna16_create_weights_then_load_8bit_gptq_experts():
    """8-bit GPTQ experts (moe_wna16.py:364-401): ``create_weights`` registers int32 ``[E, K/4, N]`` words,
    symmetric zero-points stored as 127, scales ``[E, K/g, N]``; after loading they become int8
    ``[E, N, K]`` = byte - 128 and take the W8A16 grouped GEMM with group scales."""
    from vllm_gcu_amd.kernels.quantization.moe_wna16 import MoeWNA16GCUConfig
    print("case moe_wna16 8-bit", flush=True)
    M, E, T, H, I, g = 36, 4, 2, 256, 384, 128
    rng = np.random.default_rng(21)
    cfg = MoeWNA16GCUConfig.from_config({"quant_method": "gptq", "bits": 8, "group_size": g, "sym": True})
    assert cfg.weight_bits == 8 and not cfg.has_zp and int(cfg.pack_factor) == 4
    method = cfg.get_quant_method()
    layer = torch.nn.Module()
    method.create_weights(layer, E, H, I, torch.float16, weight_loader=None)
    assert tuple(layer.w13_qweight.shape) == (E, H // 4, 2 * I) and tuple(layer.w2_qweight.shape) == (E, I // 4, H)
    assert tuple(layer.w13_scales.shape) == (E, H // g, 2 * I) and tuple(layer.w13_qzeros.shape) == (E, H // g, 2 * I // 4)
    assert layer.w13_qweight.is_transposed and layer.w13_qweight.quant_method == "group"
    layer.cuda()
    u13 = rng.integers(0, 256, size=(E, H, 2 * I), dtype=np.uint8)       # stored bytes: w + 128
    u2 = rng.integers(0, 256, size=(E, I, H), dtype=np.uint8)
    s13 = rng.uniform(0.001, 0.004, size=(E, H // g, 2 * I)).astype(np.float16)
    s2 = rng.uniform(0.001, 0.004, size=(E, I // g, H)).astype(np.float16)

    def pack8(u):                         # [E, K, N] bytes -> int32 [E, K/4, N], byte i of a word = k 4r + i
        Ex, K, N = u.shape
        v = u.reshape(Ex, K // 4, 4, N).astype(np.uint32)
        return (v[:, :, 0] | (v[:, :, 1] << 8) | (v[:, :, 2] << 16) | (v[:, :, 3] << 24)).view(np.int32)
    load(layer, "w13_qweight", dev(pack8(u13))); load(layer, "w2_qweight", dev(pack8(u2)))
    load(layer, "w13_scales", dev(s13)); load(layer, "w2_scales", dev(s2))
    layer.w13_qzeros.data.fill_(0x7f7f7f7f); layer.w2_qzeros.data.fill_(0x7f7f7f7f)
    method.process_weights_after_loading(layer)
    assert layer.w13_qweight.dtype == torch.int8 and tuple(layer.w13_qweight.shape) == (E, 2 * I, H)
    x = rng.standard_normal((M, H)).astype(np.float16)
    logits = rng.standard_normal((M, E)).astype(np.float32)
    out = method.apply(layer, dev(x).clone(), dev(logits), top_k=T, renormalize=True)
    two, ido, _ = om.topk_softmax(logits, T, True)
    f16 = lambda a: a.astype(np.float16).astype(np.float32)   # noqa: E731

    def wf(u, s, e):
        return (u[e].astype(np.float32) - 128.0) * np.repeat(s[e].astype(np.float32), g, 0)
    want = om.fused_experts(x.astype(np.float32), lambda e: wf(u13, s13, e), lambda e: wf(u2, s2, e), two, ido, f16)
    np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)
    # a zero-point that is not the symmetric one is refused, as in the reference
    bad = torch.nn.Module()
    method.create_weights(bad, E, H, I, torch.float16)
    bad.cuda()
    bad.w13_qzeros.data.fill_(0x7f7f7f7e); bad.w2_qzeros.data.fill_(0x7f7f7f7f)
    with pytest.raises(AssertionError):
        method.process_weights_after_loading(bad)


def test_moe_wna16_create_weights_4bit_and_act_order_refused():
    from vllm_gcu_amd.kernels.quantization.moe_wna16 import MoeWNA16GCUConfig
    E, H, I, g = 2, 256, 256, 128
    for fmt, shapes in (("gptq", ((E, H // 8, 2 * I), (E, I // 8, H))), ("awq", ((E, H, 2 * I // 8), (E, I, H // 8)))):
        conf = {"quant_method": fmt, "bits": 4, "group_size": g, "sym": True, "zero_point": True}
        method = MoeWNA16GCUConfig.from_config(conf).get_quant_method()
        layer = torch.nn.Module()
        method.create_weights(layer, E, H, I, torch.bfloat16)
        assert tuple(layer.w13_qweight.shape) == shapes[0] and tuple(layer.w2_qweight.shape) == shapes[1]
        assert tuple(layer.w13_qzeros.shape) == (E, H // g, 2 * I // 8) and layer.w2_scales.dtype == torch.bfloat16
        assert hasattr(layer, "w13_g_idx") == (fmt == "gptq")
    # GPTQ: a g_idx that is not made of consecutive runs (act-order) is refused at load time
    method = MoeWNA16GCUConfig.from_config({"quant_method": "gptq", "bits": 4, "group_size": g, "sym": False}).get_quant_method()
    layer = torch.nn.Module()
    method.create_weights(layer, E, H, I, torch.float16)
    layer.cuda()
    layer.w13_g_idx.data.copy_((torch.arange(H, device="cuda") // g).expand(E, H))
    layer.w2_g_idx.data.copy_((torch.arange(I, device="cuda") // g).flip(0).expand(E, I))
    for n in ("w13_qweight", "w2_qweight", "w13_qzeros", "w2_qzeros"):
        getattr(layer, n).data.zero_()
    with pytest.raises(AssertionError):
        method.process_weights_after_loading(layer)


def test_fp8_create_weights_shapes():
    from vllm_gcu_amd.kernels.quantization.fp8 import Fp8GCUConfig
    moe = Fp8GCUConfig().get_quant_method(moe=True)
    layer = torch.nn.Module()
    moe.create_weights(layer, 4, 512, 384, torch.bfloat16)
    assert tuple(layer.w13_weight.shape) == (4, 768, 512) and layer.w13_weight.dtype == torch.float8_e4m3fn
    assert tuple(layer.w13_weight_scale_inv.shape) == (4, 6, 4) and tuple(layer.w2_weight_scale_inv.shape) == (4, 4, 3)
    lin = Fp8GCUConfig().get_quant_method()
    l2 = torch.nn.Module()
    lin.create_weights(l2, 512, [256, 128], 512, 384, torch.bfloat16)
    assert tuple(l2.weight.shape) == (384, 512) and tuple(l2.weight_scale_inv.shape) == (3, 4)


def test_modular_kernel_chunks_tokens(monkeypatch):
    """``VLLM_FUSED_MOE_CHUNK_SIZE`` (modular_kernel.py:167-286): with workspaces sized for one chunk the
    layer gives what one pass gives, for a token count that is no multiple of the chunk, in place and
    out of place.  (Not bit for bit: a chunk of 64 tokens picks smaller align blocks than 150 tokens
    do, hence another kernel and another fp32 summation order; both are held to the oracle.)"""
    from vllm_gcu_amd.kernels import _custom_ops as ops
    from vllm_gcu_amd.kernels.modular_experts import TritonExpertsPad
    from vllm_gcu_amd.kernels.modular_kernel import FusedMoEModularKernel
    from vllm_gcu_amd.kernels.prepare_finalize import MoEPrepareAndFinalizeNoEP
    from vllm_gcu_amd.kernels.quantization import rearrange
    print("case modular kernel chunking", flush=True)
    M, E, T, H, I, g = 150, 8, 2, 256, 384, 128
    rng = np.random.default_rng(33)
    q13 = rng.integers(0, 16, size=(E, H, 2 * I), dtype=np.uint8)
    q2 = rng.integers(0, 16, size=(E, I, H), dtype=np.uint8)
    z13 = rng.integers(0, 16, size=(E, H // g, 2 * I), dtype=np.uint8)
    z2 = rng.integers(0, 16, size=(E, I // g, H), dtype=np.uint8)
    s13 = dev(rng.uniform(0.001, 0.01, size=(E, H // g, 2 * I)).astype(np.float16))
    s2 = dev(rng.uniform(0.001, 0.01, size=(E, I // g, H)).astype(np.float16))
    w13, zp13 = rearrange.rearrange_uint4_int32_gptq(dev(np.stack([ow4.gptq_pack_weight(a) for a in q13])),
                                                     dev(np.stack([ow4.gptq_pack_zeros(a) for a in z13])))
    w2, zp2 = rearrange.rearrange_uint4_int32_gptq(dev(np.stack([ow4.gptq_pack_weight(a) for a in q2])),
                                                   dev(np.stack([ow4.gptq_pack_zeros(a) for a in z2])))
    x = dev(rng.standard_normal((M, H)).astype(np.float16))
    tw, ids = ops.fused_topk(x, dev(rng.standard_normal((M, E)).astype(np.float32)), T, True)
    moe = FusedMoEModularKernel(MoEPrepareAndFinalizeNoEP(), TritonExpertsPad(use_int4_w4a16=True, block_shape=[0, g]))
    kw = dict(w1_scale=s13, w2_scale=s2, w1_zp=zp13, w2_zp=zp2)
    whole = moe(x, w13, w2, tw, ids, **kw)
    monkeypatch.setenv("VLLM_FUSED_MOE_CHUNK_SIZE", "64")
    chunked = moe(x, w13, w2, tw, ids, **kw)
    two, ido = tw.cpu().numpy(), ids.cpu().numpy()
    f16 = lambda a: a.astype(np.float16).astype(np.float32)   # noqa: E731
    sn13, sn2 = s13.cpu().numpy().astype(np.float32), s2.cpu().numpy().astype(np.float32)
    want = om.fused_experts(x.float().cpu().numpy(), lambda e: ow4.dequantize(q13[e], z13[e], sn13[e], g),
                            lambda e: ow4.dequantize(q2[e], z2[e], sn2[e], g), two, ido, f16)
    np.testing.assert_allclose(whole.float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(chunked.float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)
    xin = x.clone()
    inplace = moe(xin, w13, w2, tw, ids, inplace=True, **kw)
    assert inplace.data_ptr() == xin.data_ptr() and torch.equal(inplace, chunked)


def test_vllm_wiring_pieces_without_vllm():
    """init_prepare_finalize / shared-experts hook (patch_0_9_2/moe_layer.py:21-79), the x_scale
    pass-through forward (kernels/linear.py:117-129) and the int8 hook (patch_0_9_2/utils.py:13-15),
    on stand-ins for the vLLM objects they read."""
    import types
    from vllm_gcu_amd.kernels import linear, moe_layer
    from vllm_gcu_amd.kernels.modular_kernel import FusedMoEModularKernel
    from vllm_gcu_amd.kernels.prepare_finalize import MoEPrepareAndFinalizeNoEP
    from vllm_gcu_amd.kernels.quantization.fp8 import Fp8GCUConfig
    from vllm_gcu_amd.kernels import _custom_ops as ops
    moe_cfg = types.SimpleNamespace(use_pplx_kernels=False, use_deepep_ht_kernels=False, use_deepep_ll_kernels=False,
                                    moe_parallel_config=types.SimpleNamespace(ep_size=1, dp_size=1))
    method = Fp8GCUConfig().get_quant_method(moe=True)
    method.fused_experts = None
    moe_layer.init_prepare_finalize(method, moe_cfg, None)
    assert isinstance(method.fused_experts, FusedMoEModularKernel)
    assert isinstance(method.fused_experts.prepare_finalize, MoEPrepareAndFinalizeNoEP)
    assert method.topk_indices_dtype is None
    moe_cfg.moe_parallel_config.ep_size = 2
    with pytest.raises(NotImplementedError):
        moe_layer.init_prepare_finalize(method, moe_cfg, None)
    shared = lambda a: a          # noqa: E731
    layer = types.SimpleNamespace(quant_method=method, shared_experts=shared, routed_scaling_factor=2.5)
    moe_layer.set_shared_experts(layer)
    assert method.fused_experts.prepare_finalize.shared_experts is shared
    assert method.fused_experts.prepare_finalize.routed_scaling_factor == 2.5
    with pytest.raises(ImportError):
        moe_layer.install()
    x = torch.randn(5, 256, device="cuda", dtype=torch.float16)
    q, s = moe_layer.per_token_quant_int8_gcu(x)
    q2, s2, _ = ops.scaled_int8_quant(x)
    assert torch.equal(q, q2) and torch.equal(s, s2)

    # x_scale pass-through: pre-quantised fp8 activations + their group scales give what the method
    # gives when it quantises the bf16 activations itself
    rng = np.random.default_rng(5)
    N, K = 256, 512
    lin_method = Fp8GCUConfig().get_quant_method()

    class Lin(linear.MergedReplicatedLinearMixin, torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.bias, self.skip_bias_add, self.return_bias, self.quant_method = None, False, False, lin_method
    lin = Lin()
    lin_method.create_weights(lin, K, [N], K, N, torch.bfloat16)
    lin.cuda()
    lin.weight.data = (torch.randn(N, K, device="cuda") * 0.5).to(torch.float8_e4m3fn)
    lin.weight_scale_inv.data = torch.rand(N // 128, K // 128, device="cuda") * 0.05 + 0.02
    lin_method.process_weights_after_loading(lin)
    xb = torch.from_numpy(rng.standard_normal((7, K)).astype(np.float32)).to(torch.bfloat16).cuda()
    plain = lin(xb)
    xq, xs = ops.per_token_group_quant_fp8(xb, 128)
    passed = lin(xq, xs)
    assert passed.dtype == torch.bfloat16 and torch.equal(plain, passed)


def test_w8a8_moe_static_per_expert_input_scales():
    """FusedW8A8MoEMethod as the reference runs it (w8a8.py:174-342): ``w13_in_scales [E, H]`` /
    ``w2_in_scales [E, I]`` hold reciprocal scales, 16-bit activations are quantised per (token, slot)
    with the expert's vector, int8 GEMM, per-channel output scales.  int8 codes and int32 sums are exact,
    so the result is held to the oracle of the same definition (the vendor kernel itself is unpinned)."""
    from vllm_gcu_amd.kernels.quantization.w8a8 import W8A8Config
    print("case w8a8 moe static in-scales", flush=True)
    M, E, T, H, I = 30, 4, 2, 256, 384
    rng = np.random.default_rng(44)
    m8 = W8A8Config().get_quant_method(moe=True)
    layer = torch.nn.Module()
    m8.create_weights(layer, E, H, I, torch.float16, static_in_scales=True)
    assert tuple(layer.w13_in_scales.shape) == (E, H) and layer.w2_in_scales.dtype == torch.float16
    layer.cuda()
    w13 = rng.integers(-127, 128, size=(E, 2 * I, H), dtype=np.int8)
    w2 = rng.integers(-127, 128, size=(E, H, I), dtype=np.int8)
    c13 = rng.uniform(1e-4, 4e-4, size=(E, 2 * I)).astype(np.float32)
    c2 = rng.uniform(1e-4, 4e-4, size=(E, H)).astype(np.float32)
    in13 = rng.uniform(0.02, 0.05, size=(E, H)).astype(np.float32)      # checkpoint scales
    in2 = rng.uniform(0.02, 0.06, size=(E, I)).astype(np.float32)
    load(layer, "w13_weight", dev(w13)); load(layer, "w2_weight", dev(w2))
    load(layer, "w13_out_scales", dev(c13)); load(layer, "w2_out_scales", dev(c2))
    for e in range(E):
        m8.load_in_scales(layer.w13_in_scales, e, dev(in13[e]))
        m8.load_in_scales(layer.w2_in_scales, e, dev(in2[e]))
    m8.process_weights_after_loading(layer)
    x = rng.standard_normal((M, H)).astype(np.float16)
    logits = rng.standard_normal((M, E)).astype(np.float32)
    out = m8.apply(layer, dev(x).clone(), dev(logits), top_k=T, renormalize=True)
    tw, ids, _ = om.topk_softmax(logits, T, True)
    rec13 = layer.w13_in_scales.float().cpu().numpy()
    rec2 = layer.w2_in_scales.float().cpu().numpy()
    f16 = lambda a: a.astype(np.float16).astype(np.float32)   # noqa: E731
    flat = ids.reshape(-1)
    q1 = o8.moe_expert_int8_quant(x, rec13, ids)                                  # [M*T, H]
    c1 = np.zeros((M * T, 2 * I), dtype=np.float32)
    for t in range(M * T):
        e = flat[t]
        c1[t] = o8.int8_gemm_i32(q1[t:t + 1], np.ascontiguousarray(w13[e].T))[0].astype(np.float32) * c13[e]
    a2 = f16(om.silu_and_mul(f16(c1))).astype(np.float16)
    q2 = o8.moe_expert_int8_quant(a2, rec2, flat.reshape(-1, 1))                  # one row per slot
    c3 = np.zeros((M * T, H), dtype=np.float32)
    for t in range(M * T):
        e = flat[t]
        c3[t] = o8.int8_gemm_i32(q2[t:t + 1], np.ascontiguousarray(w2[e].T))[0].astype(np.float32) * c2[e]
    c3 = f16(c3 * tw.reshape(-1, 1))
    want = f16(c3.reshape(M, T, H).sum(1))
    assert np.abs(want).max() > 0.05
    np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)
