"""GPU parity of the int4 format kernels and the W4A16 GEMM against the CPU
oracle.  Integer unpack is bit-exact; fp16/bf16 GEMM outputs are within
rtol 1e-2 / atol 1e-2 of ``x.float() @ ((q - z) * s)`` (fp32 accumulation),
and bit-exact in the special cases where every partial sum is representable."""
import numpy as np
import pytest
import torch

from oracle import w4 as ow4

pytestmark = pytest.mark.gpu

RTOL = ATOL = 1e-2


@pytest.fixture(scope="module")
def ops():
    from vllm_gcu_amd.kernels import _custom_ops
    return _custom_ops


@pytest.fixture(scope="module")
def rearrange():
    from vllm_gcu_amd.kernels.quantization import rearrange
    return rearrange


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.fixture(params=[False, True], ids=["zeros-as-given", "zeros-recovered"])
def zero_reading(request, monkeypatch):
    """Pre-scaled zero-points (z * s in the activation type) either reach the kernels as given
    (w = q * s - zeros: the kernels' pre-scaled variants) or, the default, are turned back into the packed
    integers once per tensor (w = (q - z) * s: the integer variants)."""
    from vllm_gcu_amd.kernels import _custom_ops
    monkeypatch.setattr(_custom_ops, "_RECOVER_INTEGER_ZEROS", request.param)
    return request.param


def make_case(seed, M, K, N, g, dtype=np.float16, exact=False):
    rng = np.random.default_rng(seed)
    G = K // (K if g == -1 else g)
    q = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    z = rng.integers(0, 16, size=(G, N), dtype=np.uint8)
    if exact:
        s = (2.0 ** -rng.integers(4, 8, size=(G, N))).astype(np.float32)
        x = rng.integers(-4, 5, size=(M, K)).astype(np.float32)
    else:
        s = rng.uniform(0.001, 0.01, size=(G, N)).astype(np.float32)
        x = rng.standard_normal((M, K)).astype(np.float32)
    return q, z, s, x


def to_act(a, dtype):
    return torch.from_numpy(a).to(dtype)


# ------------------------------------------------------------ formats ----
@pytest.mark.parametrize("K,N", [(128, 128), (512, 384), (4096, 4096)])
def test_repack_all_sources_bit_exact(rearrange, K, N):
    print(f"case repack K={K} N={N}", flush=True)
    rng = np.random.default_rng(K + N)
    q = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    want = ow4.native_pack(q)
    w_gptq, _ = rearrange.rearrange_uint4_int32_gptq(dev(ow4.gptq_pack_weight(q)), None)
    w_awq, _ = rearrange.rearrange_uint4_int32_awq(dev(ow4.awq_pack(q)), None)
    w_kn = rearrange.from_reference_layout(dev(ow4.ref_halfgroup_pack(q)))
    nk = np.ascontiguousarray(ow4.ref_halfgroup_pack(q).T)
    w_nk = rearrange.from_reference_layout(dev(nk), transposed=True)
    for name, got in [("gptq", w_gptq), ("awq", w_awq), ("ref_kn", w_kn), ("ref_nk", w_nk)]:
        assert got.shape == (K // 8, N) and got.dtype == torch.int32
        assert np.array_equal(got.cpu().numpy(), want), name
    assert np.array_equal(rearrange.unpack_slab(w_gptq).cpu().numpy(), q)


def test_repack_batched_experts_and_zeros(rearrange):
    rng = np.random.default_rng(11)
    E, K, N, G = 3, 256, 128, 2
    q = rng.integers(0, 16, size=(E, K, N), dtype=np.uint8)
    z = rng.integers(0, 16, size=(E, G, N), dtype=np.uint8)
    z[0, 0, :16] = np.arange(16)
    qw = np.stack([ow4.gptq_pack_weight(q[e]) for e in range(E)])
    qz = np.stack([ow4.gptq_pack_zeros(z[e]) for e in range(E)])
    w, zp = rearrange.rearrange_uint4_int32_gptq(dev(qw), dev(qz))
    assert np.array_equal(rearrange.unpack_slab(w).cpu().numpy(), q)
    want_z = np.stack([ow4.native_pack_zeros(z[e]) for e in range(E)])
    assert np.array_equal(zp.cpu().numpy(), want_z)
    az = np.stack([ow4.awq_pack(z[e]) for e in range(E)])
    _, zp2 = rearrange.rearrange_uint4_int32_awq(dev(np.stack([ow4.awq_pack(q[e]) for e in range(E)])), dev(az))
    assert np.array_equal(zp2.cpu().numpy(), want_z)
    assert np.array_equal(rearrange.pack_int8_zeros(dev(z.astype(np.int8))).cpu().numpy(), want_z)


def test_repack_against_reference_written_vectors(rearrange):
    """tests/golden/rearrange_vectors.npz holds what the reference's own rearrange.py
    (rearrange.py:6-133) returned for these checkpoint words.  The device repack of the same
    checkpoint words, and the device repack of the reference's returned bytes, must describe
    the same int4 matrix, nibble for nibble."""
    import os
    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "rearrange_vectors.npz"),
                allow_pickle=False)
    # GPTQ: checkpoint words -> slab -> one value per byte, against the reference's uint8 [K/2, N]
    w, zp = rearrange.rearrange_uint4_int32_gptq(dev(g["gptq_g128_qweight"]), dev(g["gptq_g128_qzeros"]))
    q_dev = rearrange.unpack_slab(w).cpu().numpy()
    rw = g["gptq_g128_rweight"]
    K, N = 2 * rw.shape[0], rw.shape[1]
    q_ref = np.empty((K, N), np.uint8)
    for G in range(K // 128):                      # rearrange.py:46-54: low nibble = first half of the group
        q_ref[128 * G:128 * G + 64] = rw[64 * G:64 * G + 64] & 15
        q_ref[128 * G + 64:128 * G + 128] = rw[64 * G:64 * G + 64] >> 4
    assert np.array_equal(q_dev, q_ref)
    w_from_ref = rearrange.from_reference_layout(dev(rw))
    assert torch.equal(w_from_ref, w)
    # zero-points: device keeps packed true z; the reference returned fp16 z * s
    zw = zp.cpu().numpy().view(np.uint32)
    z_dev = np.stack([(zw >> np.uint32(4 * j)) & 15 for j in range(8)], axis=-1).reshape(zw.shape[0], -1)
    zs = (z_dev.astype(np.float16) * g["gptq_g128_scales"]).astype(np.float16)
    assert np.array_equal(zs.view(np.uint16), g["gptq_g128_zeros"].view(np.uint16))
    # AWQ
    w, zp = rearrange.rearrange_uint4_int32_awq(dev(g["awq_qweight"]), dev(g["awq_qzeros"]))
    q_dev = rearrange.unpack_slab(w).cpu().numpy()
    rw = g["awq_fzeros_rweight"]
    for G in range(K // 128):
        q_ref[128 * G:128 * G + 64] = rw[64 * G:64 * G + 64] & 15
        q_ref[128 * G + 64:128 * G + 128] = rw[64 * G:64 * G + 64] >> 4
    assert np.array_equal(q_dev, q_ref)
    assert torch.equal(rearrange.from_reference_layout(dev(rw.view(np.int8))), w)
    zw = zp.cpu().numpy().view(np.uint32)
    z_dev = np.stack([(zw >> np.uint32(4 * j)) & 15 for j in range(8)], axis=-1).reshape(zw.shape[0], -1)
    assert np.array_equal(z_dev.astype(np.int8), g["awq_i8zeros_zeros"])
    assert torch.equal(rearrange.pack_int8_zeros(dev(g["awq_i8zeros_zeros"])), zp)
    # w4a8: signed nibbles w - 8 in half-groups of 32 rows; expert tensor [E, N, K/2] over [E, K/2, N] memory
    r8 = g["awq_w4a8_g64_rweight"]
    t = dev(r8).view(1, K // 2, N).view(1, N, K // 2)
    assert torch.equal(rearrange.from_reference_w4a8(t)[0], w)


# --------------------------------------------------------------- GEMM ----
def run_gemm(ops, rearrange, q, z, s, x, g, dtype, bias=None, split_k=0, family=0):
    w, zp = rearrange.rearrange_uint4_int32_gptq(dev(ow4.gptq_pack_weight(q)), dev(ow4.gptq_pack_zeros(z)))
    # the output starts full of NaN: a tile that no workgroup stores cannot pass as a stale value
    out = torch.full((x.shape[0], q.shape[1]), float("nan"), dtype=dtype, device="cuda")
    out = ops.w4a16_gemm(to_act(x, dtype).cuda(), w, to_act(s, dtype).cuda(), zp,
                         None if bias is None else to_act(bias, dtype).cuda(), g, split_k=split_k, family=family,
                         out=out)
    torch.cuda.synchronize()
    return out


def oracle(q, z, s, x, g, dtype, bias=None):
    xs = to_act(x, dtype).float().numpy()
    ss = to_act(s, dtype).float().numpy()
    b = None if bias is None else to_act(bias, dtype).float().numpy()
    return ow4.w4a16_gemm(xs, q, z, ss, g, bias=b)


@pytest.mark.parametrize("M", [1, 3, 8, 16, 17, 32, 33, 64])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_stream_gemm_parity(ops, rearrange, M, dtype):
    K, N, g = 1024, 384, 128
    print(f"case stream M={M} K={K} N={N} {dtype}", flush=True)
    q, z, s, x = make_case(M, M, K, N, g)
    got = run_gemm(ops, rearrange, q, z, s, x, g, dtype).float().cpu().numpy()
    want = oracle(q, z, s, x, g, dtype)
    np.testing.assert_allclose(got, want, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("M", [33, 48, 64])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("family", [1, 2])
def test_33_to_64_rows_either_kernel_family(ops, rearrange, M, dtype, family):
    """The dispatcher picks the family by dtype in this range; both must hold the tolerance for both."""
    K, N, g = 2048, 512, 128
    print(f"case family={family} M={M} {dtype}", flush=True)
    q, z, s, x = make_case(100 + M, M, K, N, g)
    bias = np.random.default_rng(M).standard_normal(N).astype(np.float32)
    got = run_gemm(ops, rearrange, q, z, s, x, g, dtype, bias=bias, family=family).float().cpu().numpy()
    want = oracle(q, z, s, x, g, dtype, bias=bias)
    np.testing.assert_allclose(got, want, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("split_k", [1, 2, 3, 8])
def test_stream_gemm_exact_and_split_invariant(ops, rearrange, split_k):
    # power-of-two scales + small integer activations: every product and every
    # partial sum is exact in fp32, so any split / summation order must give
    # the same bits as the oracle
    M, K, N, g = 16, 2048, 256, 128
    print(f"case exact split_k={split_k}", flush=True)
    q, z, s, x = make_case(7, M, K, N, g, exact=True)
    got = run_gemm(ops, rearrange, q, z, s, x, g, torch.float16, split_k=split_k)
    want = torch.from_numpy(oracle(q, z, s, x, g, torch.float16)).to(torch.float16)
    assert torch.equal(got.cpu(), want)


def test_split_k_layers_of_different_width_share_a_workspace(ops, rearrange):
    # one workspace serves every layer: a narrow layer's split-K partial tiles must not land on
    # the arrival counters a wider layer uses afterwards.  run_gemm hands over an output full of NaN,
    # so a launch that never stores (a corrupted counter) cannot pass on stale memory.
    g = 128
    cases = [(4, 1024, 256, 4 | (2 << 8)), (4, 1024, 2048, 2 | (1 << 8)), (4, 1024, 256, 2 | (1 << 8))]
    for i, (M, K, N, split_k) in enumerate(cases):
        print(f"case shared workspace M={M} K={K} N={N} split_k={split_k:#x}", flush=True)
        q, z, s, x = make_case(40 + i, M, K, N, g, exact=True)
        want = torch.from_numpy(oracle(q, z, s, x, g, torch.float16)).to(torch.float16)
        got = run_gemm(ops, rearrange, q, z, s, x, g, torch.float16, split_k=split_k)
        assert torch.equal(got.cpu(), want)


@pytest.mark.parametrize("g", [32, 64, 128, 256, -1])
def test_stream_gemm_group_sizes_and_bias(ops, rearrange, g):
    M, K, N = 5, 512, 128
    print(f"case group g={g}", flush=True)
    q, z, s, x = make_case(100 + g, M, K, N, g)
    bias = np.random.default_rng(5).standard_normal(N).astype(np.float32)
    got = run_gemm(ops, rearrange, q, z, s, x, g, torch.float16, bias=bias).float().cpu().numpy()
    want = oracle(q, z, s, x, g, torch.float16, bias=bias)
    np.testing.assert_allclose(got, want, rtol=RTOL, atol=ATOL)


def test_config0_full_size_and_determinism(ops, rearrange):
    # benchmark configuration 0: x f16 [16, 4096], int4 [4096, 4096], g = 128
    M, K, N, g = 16, 4096, 4096, 128
    print("case config0", flush=True)
    q, z, s, x = make_case(0, M, K, N, g)
    a = run_gemm(ops, rearrange, q, z, s, x, g, torch.float16)
    b = run_gemm(ops, rearrange, q, z, s, x, g, torch.float16)
    assert torch.equal(a, b), "split-K result depends on scheduling"
    want = oracle(q, z, s, x, g, torch.float16)
    np.testing.assert_allclose(a.float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)


def test_symmetric_default_zero_point(ops, rearrange):
    M, K, N, g = 4, 256, 128, 128
    q, z, s, x = make_case(21, M, K, N, g)
    w, _ = rearrange.rearrange_uint4_int32_gptq(dev(ow4.gptq_pack_weight(q)), None)
    out = ops.gptq_gemm_gcu(to_act(x, torch.float16).cuda(), w, torch.empty(0, dtype=torch.int32, device="cuda"),
                            to_act(s, torch.float16).cuda(), torch.empty(0, dtype=torch.int32, device="cuda"),
                            4, None, g)
    want = oracle(q, None, s, x, g, torch.float16)
    np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("M", [2, 48])
def test_reference_layout_drop_in(ops, M, zero_reading):
    # exactly what the reference's GPTQ loader leaves on the layer
    # (gptq.py:229-261): uint8 half-group weights, fp16 zeros = z * scales
    K, N, g = 512, 256, 128
    print(f"case reference-layout M={M}", flush=True)
    q, z, s, x = make_case(31 + M, M, K, N, g)
    s16 = s.astype(np.float16)
    rweight, zeros_f = ow4.rearrange_gptq(ow4.gptq_pack_weight(q), ow4.gptq_pack_zeros(z), s16)
    out = ops.gptq_gemm_gcu(to_act(x, torch.float16).cuda().reshape(1, M, K), dev(rweight), dev(zeros_f),
                            dev(s16), torch.arange(K, dtype=torch.int32, device="cuda") // g, 4, None, g)
    assert out.shape == (1, M, N)
    xs = to_act(x, torch.float16).float().numpy()
    want = xs @ ow4.dequantize_prescaled_zeros(q, zeros_f, s16, g)
    np.testing.assert_allclose(out.float().cpu().numpy()[0], want, rtol=RTOL, atol=ATOL)
    # AWQ form: int8 zero-points kept as integers (awq.py:80-106)
    rw8, z8 = ow4.rearrange_awq(ow4.awq_pack(q), ow4.awq_pack(z), s16, zeros_in_int8=True)
    out2 = ops.awq_gemm_gcu(to_act(x, torch.float16).cuda(), dev(rw8), dev(s16), dev(z8), 8, None, g)
    want2 = oracle(q, z, s, x, g, torch.float16)
    np.testing.assert_allclose(out2.float().cpu().numpy(), want2, rtol=RTOL, atol=ATOL)


def test_empty_input_returns_empty(ops, rearrange):
    q, z, s, x = make_case(1, 1, 128, 128, 128)
    w, zp = rearrange.rearrange_uint4_int32_gptq(dev(ow4.gptq_pack_weight(q)), dev(ow4.gptq_pack_zeros(z)))
    out = ops.w4a16_gemm(torch.empty(0, 128, dtype=torch.float16, device="cuda"), w,
                         to_act(s, torch.float16).cuda(), zp, None, 128)
    assert out.shape == (0, 128)


# ------------------------------------------------------- MFMA tile kernel ----
@pytest.mark.parametrize("M,K,N", [(65, 256, 256), (128, 512, 384), (200, 1024, 512), (2048, 4096, 4096)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_tile_gemm_parity(ops, rearrange, M, K, N, dtype):
    g = 128
    print(f"case tile M={M} K={K} N={N} {dtype}", flush=True)
    q, z, s, x = make_case(M + K, M, K, N, g)
    bias = np.random.default_rng(9).standard_normal(N).astype(np.float32)
    got = run_gemm(ops, rearrange, q, z, s, x, g, dtype, bias=bias).float().cpu().numpy()
    want = oracle(q, z, s, x, g, dtype, bias=bias)
    np.testing.assert_allclose(got, want, rtol=RTOL, atol=ATOL)


def test_tile_gemm_exact_and_agrees_with_stream(ops, rearrange):
    # exact case: both kernel families must reproduce the oracle bit for bit
    M, K, N, g = 64, 512, 256, 128
    q, z, s, x = make_case(3, M, K, N, g, exact=True)
    want = torch.from_numpy(oracle(q, z, s, x, g, torch.float16)).to(torch.float16)
    a = run_gemm(ops, rearrange, q, z, s, x, g, torch.float16, family=1)
    b = run_gemm(ops, rearrange, q, z, s, x, g, torch.float16, family=2)
    assert torch.equal(a.cpu(), want) and torch.equal(b.cpu(), want)


@pytest.mark.parametrize("M,K,N", [(128, 4096, 512), (96, 2048, 256), (130, 1536, 384)])
def test_tile_gemm_split_k_small_grid(ops, rearrange, M, K, N):
    # few output tiles and a long K: the MFMA kernel splits K over workgroups
    # and a second kernel adds the fp32 partial tiles (and the bias) in order
    print(f"case tile split-K M={M} K={K} N={N}", flush=True)
    g = 128
    q, z, s, x = make_case(M + N, M, K, N, g)
    bias = np.random.default_rng(2).standard_normal(N).astype(np.float32)
    a = run_gemm(ops, rearrange, q, z, s, x, g, torch.float16, bias=bias, family=2)
    b = run_gemm(ops, rearrange, q, z, s, x, g, torch.float16, bias=bias, family=2)
    assert torch.equal(a, b)                               # run-to-run identical
    want = oracle(q, z, s, x, g, torch.float16, bias=bias)
    np.testing.assert_allclose(a.float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)
    # exact inputs: any split must reproduce the oracle bit for bit
    q, z, s, x = make_case(5, M, K, N, g, exact=True)
    got = run_gemm(ops, rearrange, q, z, s, x, g, torch.float16, family=2)
    assert torch.equal(got.cpu(), torch.from_numpy(oracle(q, z, s, x, g, torch.float16)).to(torch.float16))


def test_tile_gemm_three_way_split_between_half_and_full_round(ops, rearrange):
    # 288 output tiles over a long K (more than half of the 512 resident workgroups, fewer than 0.7
    # of them): K is split three ways; sampled rows against the oracle, exact inputs bit for bit
    M, K, N, g = 1152, 8192, 4096, 128
    print(f"case tile 3-way split M={M} K={K} N={N}", flush=True)
    q, z, s, x = make_case(77, M, K, N, g)
    got = run_gemm(ops, rearrange, q, z, s, x, g, torch.float16).float().cpu().numpy()
    rows = np.random.default_rng(3).choice(M, size=48, replace=False)
    rows[:3] = (0, 63, M - 1)
    want = oracle(q, z, s, x[rows], g, torch.float16)
    np.testing.assert_allclose(got[rows], want, rtol=RTOL, atol=ATOL)
    assert np.isfinite(got).all()
    q, z, s, x = make_case(78, M, K, N, g, exact=True)
    got = run_gemm(ops, rearrange, q, z, s, x, g, torch.float16).cpu()
    want = torch.from_numpy(oracle(q, z, s, x[rows], g, torch.float16)).to(torch.float16)
    assert torch.equal(got[torch.from_numpy(rows)], want)


def test_tile_gemm_zero_kinds_and_group_256(ops, rearrange, zero_reading):
    M, K, N, g = 130, 512, 256, 256
    q, z, s, x = make_case(77, M, K, N, g)
    got = run_gemm(ops, rearrange, q, z, s, x, g, torch.float16).float().cpu().numpy()
    np.testing.assert_allclose(got, oracle(q, z, s, x, g, torch.float16), rtol=RTOL, atol=ATOL)
    # symmetric default (no zero-points) and the reference's pre-scaled fp16 zeros
    w, _ = rearrange.rearrange_uint4_int32_gptq(dev(ow4.gptq_pack_weight(q)), None)
    xs = to_act(x, torch.float16).cuda()
    out = ops.w4a16_gemm(xs, w, to_act(s, torch.float16).cuda(), None, None, g)
    np.testing.assert_allclose(out.float().cpu().numpy(), oracle(q, None, s, x, g, torch.float16), rtol=RTOL, atol=ATOL)
    s16 = s.astype(np.float16)
    zs = (z.astype(np.float32) * s16.astype(np.float32)).astype(np.float16)
    out = ops.w4a16_gemm(xs, w, dev(s16), dev(zs), None, g)
    want = to_act(x, torch.float16).float().numpy() @ ow4.dequantize_prescaled_zeros(q, zs, s16, g)
    np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("M", [33, 64, 100, 128])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_narrow_tiles_mid_rows(ops, rearrange, M, dtype):
    """33..128 rows on layers up to 8192 wide run 32-row x 64-column workgroups (one tile per wavefront,
    two K blocks in flight), with K split up to four ways on a narrow layer: packed, absent and float
    zero-points, group 128 and 256, bias, ragged last row block, exact inputs bit for bit."""
    print(f"case narrow tiles M={M} {dtype}", flush=True)
    for K, N, g in ((4096, 512, 128), (1024, 1152, 256)):
        q, z, s, x = make_case(M + K + N, M, K, N, g)
        bias = np.random.default_rng(4).standard_normal(N).astype(np.float32)
        got = run_gemm(ops, rearrange, q, z, s, x, g, dtype, bias=bias, family=2)
        assert torch.equal(got, run_gemm(ops, rearrange, q, z, s, x, g, dtype, bias=bias, family=2))
        np.testing.assert_allclose(got.float().cpu().numpy(), oracle(q, z, s, x, g, dtype, bias=bias), rtol=RTOL, atol=ATOL)
        w, _ = rearrange.rearrange_uint4_int32_gptq(dev(ow4.gptq_pack_weight(q)), None)
        xs, sd = to_act(x, dtype).cuda(), to_act(s, dtype).cuda()
        out = ops.w4a16_gemm(xs, w, sd, None, None, g, family=2)
        np.testing.assert_allclose(out.float().cpu().numpy(), oracle(q, None, s, x, g, dtype), rtol=RTOL, atol=ATOL)
        sf = to_act(s, dtype).float().numpy()
        zs = to_act(z.astype(np.float32) * sf, dtype)
        out = ops.w4a16_gemm(xs, w, sd, zs.cuda(), None, g, family=2)
        # the kernels recover the integer zero-point from z * s (rounded to the activation type), so the
        # result is that of the integer form; q * s - round(z * s) differs from it by the rounding of z * s
        np.testing.assert_allclose(out.float().cpu().numpy(), oracle(q, z, s, x, g, dtype), rtol=RTOL, atol=ATOL)
    q, z, s, x = make_case(6, M, 4096, 256, 128, exact=True)
    got = run_gemm(ops, rearrange, q, z, s, x, 128, torch.float16, family=2)
    assert torch.equal(got.cpu(), torch.from_numpy(oracle(q, z, s, x, 128, torch.float16)).to(torch.float16))


# ------------------------------------------------ 128-row ring kernel (family 3) ----
@pytest.mark.parametrize("M,K,N,g,split", [(128, 512, 256, 128, 1), (100, 1024, 384, 128, 1), (17, 512, 128, 128, 1),
                                           (64, 2048, 512, 256, 0), (128, 4096, 512, 128, 0), (128, 1536, 256, 128, 3),
                                           (48, 4096, 256, 128, 4), (130, 1024, 256, 128, 1), (300, 1024, 640, 128, 0),
                                           (2048, 2048, 384, 128, 0)])
@pytest.mark.parametrize("tw", [2, 1, 4])
def test_ring_gemm_parity(ops, rearrange, M, K, N, g, split, tw):
    """The kernel that owns up to 128 rows per workgroup and streams K through a ring of LDS stages
    (fp16; B operands are (q - z) * s rounded to fp16), with two 16-column tiles per wavefront
    (workgroups of 256 columns), with one (128 columns) and with four (512 columns, always 128 rows
    per workgroup): ragged M, a half-empty last column tile and workgroups with whole slabs past N,
    several row blocks, K split with the separate reduction, groups of 256, bias; run-to-run
    identical; exact inputs bit for bit (every scale a power of two, so the fp16 weights are exact)."""
    print(f"case ring M={M} K={K} N={N} g={g} split={split} tiles per wavefront={tw}", flush=True)
    split |= tw << 8
    q, z, s, x = make_case(M + K, M, K, N, g)
    bias = np.random.default_rng(9).standard_normal(N).astype(np.float32)
    got = run_gemm(ops, rearrange, q, z, s, x, g, torch.float16, bias=bias, family=3, split_k=split)
    assert torch.equal(got, run_gemm(ops, rearrange, q, z, s, x, g, torch.float16, bias=bias, family=3, split_k=split))
    np.testing.assert_allclose(got.float().cpu().numpy(), oracle(q, z, s, x, g, torch.float16, bias=bias), rtol=RTOL, atol=ATOL)
    q, z, s, x = make_case(5, M, K, N, g, exact=True)
    got = run_gemm(ops, rearrange, q, z, s, x, g, torch.float16, family=3, split_k=split)
    assert torch.equal(got.cpu(), torch.from_numpy(oracle(q, z, s, x, g, torch.float16)).to(torch.float16))


@pytest.mark.parametrize("tw", [2, 1, 4])
@pytest.mark.parametrize("M", [32, 64, 128, 200])
def test_ring_gemm_zero_kinds(ops, rearrange, M, tw, zero_reading):
    """No zero-points (z = 8) and the reference's pre-scaled fp16 zero-points, where the kernel forms
    q * s - zs in one fused multiply-add: the oracle of that form is dequantize_prescaled_zeros."""
    K, N, g = 1024, 384, 128
    print(f"case ring zero kinds M={M}", flush=True)
    q, z, s, x = make_case(M + 1, M, K, N, g)
    w, _ = rearrange.rearrange_uint4_int32_gptq(dev(ow4.gptq_pack_weight(q)), None)
    xs = to_act(x, torch.float16).cuda()
    out = ops.w4a16_gemm(xs, w, to_act(s, torch.float16).cuda(), None, None, g, family=3, split_k=tw << 8)
    np.testing.assert_allclose(out.float().cpu().numpy(), oracle(q, None, s, x, g, torch.float16), rtol=RTOL, atol=ATOL)
    s16 = s.astype(np.float16)
    zs = (z.astype(np.float32) * s16.astype(np.float32)).astype(np.float16)
    out = ops.w4a16_gemm(xs, w, dev(s16), dev(zs), None, g, family=3, split_k=tw << 8)
    want = to_act(x, torch.float16).float().numpy() @ ow4.dequantize_prescaled_zeros(q, zs, s16, g)
    np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)


def test_mid_rows_take_the_ring_kernel_where_k_is_long(ops, rearrange):
    """33..128 rows on a layer whose workgroups walk ten K blocks or more: the dispatcher takes the ring
    kernel with 128-column workgroups and splits K four ways here (64 column tiles on 256 CUs).  Sampled
    columns against the oracle, the forced 64-row tile kernel beside it, run-to-run identical."""
    M, K, N, g = 96, 5120, 8192, 128
    print(f"case ring auto M={M} K={K} N={N}", flush=True)
    q, z, s, x = make_case(21, M, K, N, g)
    bias = np.random.default_rng(3).standard_normal(N).astype(np.float32)
    got = run_gemm(ops, rearrange, q, z, s, x, g, torch.float16, bias=bias)
    assert torch.equal(got, run_gemm(ops, rearrange, q, z, s, x, g, torch.float16, bias=bias))
    want = oracle(q, z, s, x, g, torch.float16, bias=bias)
    np.testing.assert_allclose(got.float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)
    tile = run_gemm(ops, rearrange, q, z, s, x, g, torch.float16, bias=bias, family=2)
    np.testing.assert_allclose(tile.float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)


def test_even_rounds_take_the_512_column_ring_workgroups(ops, rearrange):
    """1024 rows x 16384 columns is exactly one round of 128 x 512 workgroups on 256 CUs and two rounds of
    either other kernel: the dispatcher takes the 512-column ring workgroups, so its result is bit for
    bit that of the forced launch; against the oracle, and the 64-row tiles beside it."""
    M, K, N, g = 1024, 512, 16384, 128
    print(f"case ring 512 columns auto M={M} K={K} N={N}", flush=True)
    q, z, s, x = make_case(33, M, K, N, g)
    got = run_gemm(ops, rearrange, q, z, s, x, g, torch.float16)
    forced = run_gemm(ops, rearrange, q, z, s, x, g, torch.float16, family=3, split_k=4 << 8)
    assert torch.equal(got, forced)
    want = oracle(q, z, s, x, g, torch.float16)
    np.testing.assert_allclose(got.float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)
    tile = run_gemm(ops, rearrange, q, z, s, x, g, torch.float16, family=2)
    np.testing.assert_allclose(tile.float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)


def test_ring_gemm_is_fp16_only_and_tile_family_still_forced(ops, rearrange):
    M, K, N, g = 160, 512, 256, 128
    q, z, s, x = make_case(8, M, K, N, g)
    # (bf16 reaches the ring kernels as staged fp16 rows, above 64 rows only)
    with pytest.raises(RuntimeError, match="fp16"):
        run_gemm(ops, rearrange, q, z, s, x[:48], g, torch.bfloat16, family=3)
    # family 2 keeps meaning the 64-row tile kernel; both agree with the oracle
    a = run_gemm(ops, rearrange, q, z, s, x, g, torch.float16, family=2).float().cpu().numpy()
    b = run_gemm(ops, rearrange, q, z, s, x, g, torch.float16, family=3).float().cpu().numpy()
    want = oracle(q, z, s, x, g, torch.float16)
    np.testing.assert_allclose(a, want, rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(b, want, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("M,K,N,zeros", [(65, 256, 28672, True), (129, 512, 16384, True), (300, 4096, 7168, True), (640, 1024, 3328, False),
                                         (2400, 14336, 1024, True), (256, 16512, 8192, True)])
def test_bf16_rows_staged_as_fp16_for_the_pipelined_loop(ops, rearrange, M, K, N, zeros):
    """bf16 from 129 rows on, the library's own choice with the operator's workspace: each row times a
    power of two of its own becomes fp16 in the workspace (exact), the fp16 loop multiplies it with the
    exact integers q - z, the epilogue undoes the power of two.  Rows of magnitudes from 2^-100 to 2^100,
    a row of zeros and a row that holds an infinity; each row is compared at its own magnitude.  The
    fourth case is taller than the staging area (2400 x 14336 x 2 bytes > 64 MiB): two row chunks; the
    last has rows too long to stay in registers between the two passes of the conversion."""
    from vllm_gcu_amd import _lib
    g = 128
    print(f"case bf16 staged M={M} K={K} N={N} zeros={zeros}", flush=True)
    assert _lib.load().mi355q_w4a16_workspace_bytes(M, K, N) > (65 << 20)     # room for the staging area is asked for
    q, z, s, x = make_case(M * 3 + K, M, K, N, g)
    if not zeros:
        z[:] = 8
    rng = np.random.default_rng(M)
    mag = (2.0 ** rng.integers(-100, 101, size=M)).astype(np.float32)
    mag[:4] = [1.0, 2.0 ** 100, 2.0 ** -100, 2.0 ** 15]
    x = x * mag[:, None]
    x[5] = 0.0
    x[7, K // 2] = np.inf
    bias = rng.standard_normal(N).astype(np.float32) * 0.0 if M != 300 else rng.standard_normal(N).astype(np.float32)
    got = run_gemm(ops, rearrange, q, z, s, x, g, torch.bfloat16, bias=bias).float().cpu().numpy()
    plain = run_gemm(ops, rearrange, q, z, s, x, g, torch.bfloat16, bias=bias, family=2).float().cpu().numpy()
    with np.errstate(invalid="ignore", over="ignore"):
        want = oracle(q, z, s, x, g, torch.bfloat16, bias=bias)
    assert not np.isfinite(got[7]).any() and not np.isfinite(plain[7]).any()
    rows = np.array([m for m in range(M) if m != 7])
    assert np.isfinite(got[rows]).all()
    if M == 300:                      # (with a bias the rows cannot be rescaled: unit magnitudes there)
        rows = rows[(mag[rows] >= 0.5) & (mag[rows] <= 2.0)]
        mag = np.ones_like(mag)
    np.testing.assert_allclose(got[rows] / mag[rows, None], want[rows] / mag[rows, None], rtol=RTOL, atol=ATOL)
    # and against the bf16 loop (same products, fp32 sums in another order, one bf16 rounding each)
    np.testing.assert_allclose(got[rows] / mag[rows, None], plain[rows] / mag[rows, None], rtol=2 ** -7, atol=1e-3)
    np.testing.assert_array_equal(got[5], np.float32(torch.from_numpy(bias).to(torch.bfloat16).float().numpy()))
    # every partial sum representable: bit for bit the oracle
    q, z, s, x = make_case(11, M, K, N, g, exact=True)
    want = torch.from_numpy(oracle(q, z, s, x, g, torch.bfloat16)).to(torch.bfloat16)
    assert torch.equal(run_gemm(ops, rearrange, q, z, s, x, g, torch.bfloat16).cpu(), want)


def test_bf16_staging_area_at_the_front_of_the_workspace_for_tall_inputs(ops, rearrange):
    """4800 x 14336 bf16 is 138 MB as fp16 rows: no launch of that height splits K, so the staging area takes
    the place of the partial tiles at the front of the workspace and the rows go in two chunks of 2400.
    Sampled rows against the oracle, everything against the bf16 loop."""
    M, K, N, g = 4800, 14336, 2048, 128
    print(f"case bf16 staged tall M={M} K={K} N={N}", flush=True)
    q, z, s, x = make_case(77, M, K, N, g)
    got = run_gemm(ops, rearrange, q, z, s, x, g, torch.bfloat16)
    assert torch.equal(got, run_gemm(ops, rearrange, q, z, s, x, g, torch.bfloat16))
    plain = run_gemm(ops, rearrange, q, z, s, x, g, torch.bfloat16, family=2)
    np.testing.assert_allclose(got.float().cpu().numpy(), plain.float().cpu().numpy(), rtol=2 ** -6, atol=2e-2)
    rows = np.array([0, 1, 63, 64, 2399, 2400, 2401, 3000, 4736, 4799])
    want = oracle(q, z, s, x[rows], g, torch.bfloat16)
    np.testing.assert_allclose(got[torch.from_numpy(rows).cuda()].float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("tw", [2, 4])
@pytest.mark.parametrize("M,K,N,zeros", [(65, 256, 512, True), (300, 1024, 1024, True), (1000, 2048, 640, False)])
def test_bf16_rows_staged_as_fp16_on_the_ring_kernels(ops, rearrange, M, K, N, zeros, tw):
    """The ring kernels (forced: family 3) on bf16 rows staged as fp16: the bf16 scales become fp16 times
    one power of two for the whole array, taken from the largest of them; row and scale powers of two
    are undone exactly in the epilogue.  Rows from 2^-60 to 2^60, columns whose scales lie up to 2^-12
    below the largest; every output is compared at the magnitude of its row and column."""
    g = 128
    print(f"case bf16 staged ring M={M} K={K} N={N} zeros={zeros} tw={tw}", flush=True)
    q, z, s, x = make_case(M + K + tw, M, K, N, g)
    if not zeros:
        z[:] = 8
    rng = np.random.default_rng(M + tw)
    rmag = (2.0 ** rng.integers(-60, 61, size=M)).astype(np.float32)
    cmag = (2.0 ** -rng.integers(0, 13, size=N).astype(np.float32)).astype(np.float32)
    cmag[0] = 1.0
    x = x * rmag[:, None]
    s = s * cmag[None, :] * np.float32(2.0 ** 9)
    x[3] = 0.0
    got = run_gemm(ops, rearrange, q, z, s, x, g, torch.bfloat16, family=3, split_k=tw << 8).float().cpu().numpy()
    want = oracle(q, z, s, x, g, torch.bfloat16)
    assert np.isfinite(got).all() and (got[3] == 0).all()
    norm = rmag[:, None] * cmag[None, :] * np.float32(2.0 ** 9)
    np.testing.assert_allclose(got / norm, want / norm, rtol=RTOL, atol=ATOL)
    # a bias, at unit magnitudes
    q, z, s, x = make_case(M + 1, M, K, N, g)
    bias = rng.standard_normal(N).astype(np.float32)
    got = run_gemm(ops, rearrange, q, z, s, x, g, torch.bfloat16, bias=bias, family=3, split_k=tw << 8)
    np.testing.assert_allclose(got.float().cpu().numpy(), oracle(q, z, s, x, g, torch.bfloat16, bias=bias), rtol=RTOL, atol=ATOL)
    # every product and partial sum representable: bit for bit the oracle
    q, z, s, x = make_case(13, M, K, N, g, exact=True)
    want = torch.from_numpy(oracle(q, z, s, x, g, torch.bfloat16)).to(torch.bfloat16)
    assert torch.equal(run_gemm(ops, rearrange, q, z, s, x, g, torch.bfloat16, family=3, split_k=tw << 8).cpu(), want)


def test_bf16_even_rounds_take_the_512_column_ring_workgroups(ops, rearrange):
    """The shape that the fp16 path gives to the 512-column ring workgroups (one round of 128 x 512 on 256
    CUs) takes them for bf16 too: the library's own choice is bit for bit the forced launch."""
    M, K, N, g = 1024, 512, 16384, 128
    print(f"case bf16 ring 512 columns auto M={M} K={K} N={N}", flush=True)
    q, z, s, x = make_case(34, M, K, N, g)
    got = run_gemm(ops, rearrange, q, z, s, x, g, torch.bfloat16)
    forced = run_gemm(ops, rearrange, q, z, s, x, g, torch.bfloat16, family=3, split_k=4 << 8)
    assert torch.equal(got, forced)
    np.testing.assert_allclose(got.float().cpu().numpy(), oracle(q, z, s, x, g, torch.bfloat16), rtol=RTOL, atol=ATOL)


def test_large_m_small_group_goes_through_stream_chunks(ops, rearrange):
    """Groups of 64 on the streaming kernel when it is forced (32 rows per launch) and through the
    library's own choice (the MFMA kernel from 65 rows on)."""
    M, K, N, g = 150, 256, 128, 64
    q, z, s, x = make_case(5, M, K, N, g)
    want = oracle(q, z, s, x, g, torch.float16)
    got = run_gemm(ops, rearrange, q, z, s, x, g, torch.float16, family=1).float().cpu().numpy()
    np.testing.assert_allclose(got, want, rtol=RTOL, atol=ATOL)
    got = run_gemm(ops, rearrange, q, z, s, x, g, torch.float16).float().cpu().numpy()
    np.testing.assert_allclose(got, want, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("g", [64, 32])
@pytest.mark.parametrize("M,K,N", [(65, 512, 256, ), (100, 1024, 384), (300, 2048, 640), (1100, 8192, 256), (2048, 1024, 1024)])
def test_tile_gemm_groups_of_64_and_32(ops, rearrange, M, K, N, g, dtype):
    """Group sizes below a K block on the MFMA kernel (two or four groups per K block of 128, each with a
    partial tile, scale and zero-point of its own): ragged M, a half-empty last column tile, a shape
    that splits K (1100 x 8192 x 256), bias; the streaming kernel on the same data beside it; run-to-run
    identical; exact inputs bit for bit."""
    print(f"case small groups M={M} K={K} N={N} g={g} {dtype}", flush=True)
    q, z, s, x = make_case(M + g, M, K, N, g)
    bias = np.random.default_rng(4).standard_normal(N).astype(np.float32)
    got = run_gemm(ops, rearrange, q, z, s, x, g, dtype, bias=bias)
    assert torch.equal(got, run_gemm(ops, rearrange, q, z, s, x, g, dtype, bias=bias))
    want = oracle(q, z, s, x, g, dtype, bias=bias)
    np.testing.assert_allclose(got.float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)
    forced = run_gemm(ops, rearrange, q, z, s, x, g, dtype, bias=bias, family=2)
    assert torch.equal(got, forced)
    if M <= 300:
        stream = run_gemm(ops, rearrange, q, z, s, x, g, dtype, bias=bias, family=1)
        np.testing.assert_allclose(stream.float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)
    q, z, s, x = make_case(5, M, K, N, g, exact=True)
    got = run_gemm(ops, rearrange, q, z, s, x, g, dtype, family=2)
    assert torch.equal(got.cpu(), torch.from_numpy(oracle(q, z, s, x, g, dtype)).to(dtype))


@pytest.mark.parametrize("g", [64, 32])
def test_tile_gemm_small_groups_zero_kinds(ops, rearrange, g, zero_reading):
    """No zero-points and pre-scaled 16-bit zero-points with groups of 64 and 32 on the MFMA kernel."""
    M, K, N = 200, 1024, 384
    print(f"case small groups zero kinds g={g}", flush=True)
    q, z, s, x = make_case(M + 1, M, K, N, g)
    w, _ = rearrange.rearrange_uint4_int32_gptq(dev(ow4.gptq_pack_weight(q)), None)
    for dtype in (torch.float16, torch.bfloat16):
        xs, sd = to_act(x, dtype).cuda(), to_act(s, dtype).cuda()
        out = ops.w4a16_gemm(xs, w, sd, None, None, g)
        np.testing.assert_allclose(out.float().cpu().numpy(), oracle(q, None, s, x, g, dtype), rtol=RTOL, atol=ATOL)
        sf = to_act(s, dtype).float().numpy()
        zs = to_act(z.astype(np.float32) * sf, dtype)
        out = ops.w4a16_gemm(xs, w, sd, zs.cuda(), None, g)
        np.testing.assert_allclose(out.float().cpu().numpy(), oracle(q, z, s, x, g, dtype), rtol=RTOL, atol=ATOL)


def _random_cases():
    rng = np.random.default_rng(2024)
    cases = []
    for i in range(28):
        g = int(rng.choice([128, 128, 128, 64, 32, 256, -1]))
        K = 128 * int(rng.integers(1, 33))
        if g == 256:
            K = 256 * max(1, K // 256)
        N = 128 * int(rng.integers(1, 25))
        M = int(rng.choice([rng.integers(1, 33), rng.integers(33, 129), rng.integers(129, 700), rng.integers(700, 2600)]))
        cases.append((i, M, K, N, g, ["f16", "bf16"][int(rng.integers(0, 2))], int(rng.integers(0, 3)), bool(rng.integers(0, 2))))
    # wide enough for the 512-column ring workgroups and for several rounds of every kernel
    cases += [(100, 2048, 1024, 8192, 128, "f16", 1, True), (101, 1536, 512, 12288, 128, "f16", 0, False),
              (102, 1300, 2048, 4096, 128, "bf16", 1, True), (103, 640, 1024, 16384, 64, "f16", 1, False),
              # bf16 rows staged as fp16: the 512-column ring workgroups, 64-row tiles with and without zero-points
              (104, 1024, 1024, 16384, 128, "bf16", 2, True), (105, 200, 512, 12288, 128, "bf16", 0, False),
              (106, 90, 768, 28672, 256, "bf16", 1, True)]
    return cases


@pytest.mark.parametrize("seed,M,K,N,g,dt,zk,with_bias", _random_cases())
def test_random_shapes_through_the_library_s_own_choice(ops, rearrange, seed, M, K, N, g, dt, zk, with_bias, zero_reading):
    """Seeded random shapes, group sizes, types, zero-point kinds and bias through mi355q_w4a16_gemm as a
    caller uses it (no family forced): whichever kernel and split the dispatcher takes, the result is the
    oracle's within the tolerance and run-to-run identical."""
    dtype = torch.float16 if dt == "f16" else torch.bfloat16
    print(f"case random {seed}: M={M} K={K} N={N} g={g} {dt} zeros kind {zk} bias {with_bias}", flush=True)
    q, z, s, x = make_case(1000 + seed, M, K, N, g)
    bias = np.random.default_rng(seed).standard_normal(N).astype(np.float32) if with_bias else None
    gg = K if g == -1 else g
    w, zp = rearrange.rearrange_uint4_int32_gptq(dev(ow4.gptq_pack_weight(q)), dev(ow4.gptq_pack_zeros(z)))
    xs, sd = to_act(x, dtype).cuda(), to_act(s, dtype).cuda()
    bd = None if bias is None else to_act(bias, dtype).cuda()
    if zk == 0:                                      # symmetric: no zero-points, z = 8
        zeros, want = None, oracle(q, None, s, x, gg, dtype, bias=bias)
    elif zk == 1:                                    # packed integer zero-points
        zeros, want = zp, oracle(q, z, s, x, gg, dtype, bias=bias)
    else:                                            # z * s rounded to the activation type
        sf = to_act(s, dtype).float().numpy()
        zs = to_act(z.astype(np.float32) * sf, dtype)
        zeros, want = zs.cuda(), oracle(q, z, s, x, gg, dtype, bias=bias)
    got = ops.w4a16_gemm(xs, w, sd, zeros, bd, g)
    again = ops.w4a16_gemm(xs, w, sd, zeros, bd, g)
    assert torch.equal(got, again)
    got = got.float().cpu().numpy()
    if zk == 2 and not np.allclose(got, want, rtol=RTOL, atol=ATOL):
        # the streaming and ring kernels take the pre-scaled value as it is, q * s - zs, where the tile kernel
        # recovers the integer zero-point: the two readings differ by the rounding of z * s times the sum of
        # a group's activations, which a group of many hundred rows in bf16 makes visible
        want = to_act(x, dtype).float().numpy() @ ow4.dequantize_prescaled_zeros(q, zs.float().numpy(), sf, gg)
        if bias is not None:
            want = want + to_act(bias, dtype).float().numpy()[None, :]
    np.testing.assert_allclose(got, want, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_integer_zero_points_are_recovered_only_when_exact(ops, rearrange, dtype):
    """zeros == z.to(dtype) * scales bit for bit with z in 0..15 (what the reference's loaders store) comes
    back as the packed integers; one element one step off, a zero-point of 16, or a non-integer multiple
    keeps the tensor as given.  A scale of 0 with a zero of 0 is an integer zero-point (any: 0 is taken)."""
    rng = np.random.default_rng(17)
    G, N = 6, 256
    z = rng.integers(0, 16, size=(G, N), dtype=np.uint8)
    s = to_act(rng.uniform(0.001, 0.01, size=(G, N)).astype(np.float32), dtype).cuda()
    s[2, 5] = 0.0
    zt = torch.from_numpy(z).cuda()
    zs = zt.to(dtype) * s
    packed = ops._integer_zeros(zs, s)
    assert packed is not None and packed.dtype == torch.int32 and packed.shape == (G, N // 8)
    z_expect = z.copy()
    z_expect[2, 5] = 0
    assert torch.equal(packed, rearrange.pack_int8_zeros(torch.from_numpy(z_expect).cuda()))
    assert ops._integer_zeros(zs, s) is packed                       # cached on the tensor
    z_kind = ops._zero_points(zs, dtype, s)
    assert z_kind[1] == ops._lib.ZP_PACKED and z_kind[0] is packed
    off = zs.clone()
    off[1, 7] = (off[1, 7].view(torch.int16) + 1).view(dtype)           # one step of the type
    assert ops._integer_zeros(off, s) is None and ops._zero_points(off, dtype, s)[1] == ops._lib.ZP_PRESCALED
    assert ops._integer_zeros((zt.to(dtype) + 16) * s, s) is None       # out of the int4 range
    assert ops._integer_zeros(zs * 0.5 + s * 0.25, s) is None           # not integers
    assert ops._zero_points(zs, dtype, s.float())[1] == ops._lib.ZP_PRESCALED   # scales the caller holds in another type


def test_operand_shapes_are_checked_on_the_host(ops, rearrange):
    """The kernels index scales, zero-points and bias by (group row, column) without bounds checks, so
    the wrapper refuses operands whose sizes do not fit K / group_size x N before anything is launched."""
    print("case w4a16 operand shape checks", flush=True)
    q, z, s, x = make_case(5, 4, 256, 256, 128)
    qw, qz = rearrange.rearrange_uint4_int32_gptq(dev(ow4.gptq_pack_weight(q)), dev(ow4.gptq_pack_zeros(z)))
    xs, sc = to_act(x, torch.float16).cuda(), to_act(s, torch.float16).cuda()
    good = ops.w4a16_gemm(xs, qw, sc, qz, None, 128)
    assert good.shape == (4, 256)
    with pytest.raises(RuntimeError, match="zero-points"):
        ops.w4a16_gemm(xs, qw, sc, qz.to(torch.float16), None, 128)       # [K/g, N/8] values, not [K/g, N]
    with pytest.raises(RuntimeError, match="scales"):
        ops.w4a16_gemm(xs, qw, sc[:1], qz, None, 128)
    with pytest.raises(RuntimeError, match="bias"):
        ops.w4a16_gemm(xs, qw, sc, qz, torch.zeros(8, dtype=torch.float16, device="cuda"), 128)
