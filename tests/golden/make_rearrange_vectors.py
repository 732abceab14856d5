"""Writes ``rearrange_vectors.npz``: input / output vectors of the reference's
own int4 weight re-packing functions.

Runs in the build container only.  It loads
``vllm_gcu/kernels/quantization/rearrange.py`` of the reference checkout BY
FILE PATH (that file imports nothing but ``torch``; the package around it is
not importable) and records what its two functions return for small seeded
inputs.  Only the resulting ``.npz`` (inputs and expected outputs, under 100 KB:
the shapes are the smallest the device layout accepts, K and N multiples of 128) is
committed and travels to the GPU box; the reference file never does.

    python tests/golden/make_rearrange_vectors.py [/root/reference]

Cases (all weights 4 bit, pack factor 8):
  gptq_g128        rearrange_uint4_int32_uint8_gptq, group 128, fp16 scales
  (qzeros None and zeros_in_int8 return the same weight bytes as the cases
   beside them; the script asserts that and stores them once)
  awq_fzeros       rearrange_uint4_int32_uint8_awq, zeros * scales (fp16)
  awq_i8zeros      same, zeros_in_int8=True
  awq_w4a8_g64     same, use_w4a8=True, rearrange_group 64, zeros_in_int8=True
"""
import importlib.util
import os
import sys
import types

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def load_reference(ref_root):
    path = os.path.join(ref_root, "vllm_gcu", "kernels", "quantization", "rearrange.py")
    spec = importlib.util.spec_from_file_location("_reference_rearrange", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def method_stub(group_size):
    cfg = types.SimpleNamespace(weight_bits=4, group_size=group_size, pack_factor=8)
    return types.SimpleNamespace(quant_config=cfg)


def rand_i32(rng, shape):
    return rng.integers(0, 2 ** 32, size=shape, dtype=np.uint64).astype(np.uint32).view(np.int32)


def main():
    ref_root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    ref = load_reference(ref_root)
    rng = np.random.default_rng(20240607)
    out = {}

    # GPTQ: qweight int32 [K/8, N], qzeros int32 [K/g, N/8], scales fp16 [K/g, N]
    K, N, g = 256, 128, 128
    qw = rand_i32(rng, (K // 8, N))
    qz = rand_i32(rng, (K // g, N // 8))
    qz[0, 0] = -1                      # every nibble 15: the "+1" wraps to 0
    sc = rng.uniform(0.001, 0.01, size=(K // g, N)).astype(np.float16)
    rw, zf = ref.rearrange_uint4_int32_uint8_gptq(
        method_stub(g), torch.from_numpy(qw), torch.from_numpy(qz), torch.from_numpy(sc))
    out.update(gptq_g128_qweight=qw, gptq_g128_qzeros=qz, gptq_g128_scales=sc,
               gptq_g128_rweight=rw.numpy(), gptq_g128_zeros=zf.numpy())
    assert rw.dtype == torch.uint8 and zf.dtype == torch.float16

    rw, zf = ref.rearrange_uint4_int32_uint8_gptq(
        method_stub(g), torch.from_numpy(qw), None, torch.from_numpy(sc))
    assert zf is None and np.array_equal(rw.numpy(), out["gptq_g128_rweight"])   # same bytes: not stored twice

    # AWQ: qweight int32 [K, N/8], qzeros int32 [K/g, N/8]
    K, N, g = 256, 128, 128
    qw = rand_i32(rng, (K, N // 8))
    qz = rand_i32(rng, (K // g, N // 8))
    sc = rng.uniform(0.001, 0.01, size=(K // g, N)).astype(np.float16)
    rw, zf = ref.rearrange_uint4_int32_uint8_awq(
        method_stub(g), torch.from_numpy(qw), torch.from_numpy(qz), torch.from_numpy(sc))
    out.update(awq_qweight=qw, awq_qzeros=qz, awq_scales=sc,
               awq_fzeros_rweight=rw.numpy(), awq_fzeros_zeros=zf.numpy())
    assert rw.dtype == torch.uint8 and zf.dtype == torch.float16

    rw, zi = ref.rearrange_uint4_int32_uint8_awq(
        method_stub(g), torch.from_numpy(qw), torch.from_numpy(qz), torch.from_numpy(sc),
        zeros_in_int8=True)
    assert rw.dtype == torch.int8 and zi.dtype == torch.int8
    assert np.array_equal(rw.numpy().view(np.uint8), out["awq_fzeros_rweight"])           # same bytes as int8
    out.update(awq_i8zeros_zeros=zi.numpy())

    rw, zn = ref.rearrange_uint4_int32_uint8_awq(
        method_stub(64), torch.from_numpy(qw), torch.from_numpy(qz), torch.from_numpy(sc),
        rearrange_group=64, zeros_in_int8=True, use_w4a8=True)
    assert zn is None and rw.dtype == torch.int8
    out.update(awq_w4a8_g64_rweight=rw.numpy())

    dst = os.path.join(HERE, "rearrange_vectors.npz")
    np.savez_compressed(dst, **out)
    print("wrote", dst, os.path.getsize(dst), "bytes;", sorted(out))


if __name__ == "__main__":
    main()
