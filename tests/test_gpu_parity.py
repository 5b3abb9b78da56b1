"""GPU parity of the HIP kernels, called through the C ABI, against the CPU oracle.

Bars: packing / unpacking / gather / routing indices are bit-exact.  Matmul outputs obey the
tolerance quoted for this path against an fp32 (here float64-summed) dequantize-then-matmul:
    max|y - ref| <= 1e-2 * max|x| * sqrt(K) / 64   and   ||y - ref||_2 / ||ref||_2 <= 2e-3.
"""

import os
import zlib

import numpy as np
import pytest
import torch

import mlc_llm_amd as gq
from mlc_llm_amd import ops
from oracle import gq_oracle as o

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
SCHEMES = {"q4f16_1": o.SCHEMES["q4f16_1"], "q3f16_1": o.SCHEMES["q3f16_1"]}
REL_L2 = 2e-3


def seed_of(*parts) -> int:
    return zlib.crc32(repr(parts).encode())


def dev(a: np.ndarray) -> torch.Tensor:
    if a.dtype == np.uint32:
        a = a.view(np.int32)
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def host_u32(t: torch.Tensor) -> np.ndarray:
    return t.cpu().numpy().view(np.uint32)


def host_f16_bits(t: torch.Tensor) -> np.ndarray:
    return t.cpu().numpy().view(np.uint16)


def assert_linear_ok(y: torch.Tensor, ref64: np.ndarray, x: np.ndarray, k: int, what=""):
    err, bound, rel = o.check_linear(y.float().cpu().numpy(), ref64, x, k)
    assert err <= bound, f"{what}: max abs err {err:.3e} > bound {bound:.3e}"
    assert rel <= REL_L2, f"{what}: rel-L2 {rel:.3e} > {REL_L2}"


def test_device_is_gfx950():
    gq._lib.call("mi355gq_check_device")


# ------------------------------------------------------------------ packing: bit-exact


@pytest.mark.parametrize("name", ["q4f16_1", "q3f16_1"])
@pytest.mark.parametrize("shape", [(2, 13), (16, 120), (16, 128), (5, 200), (3, 1), (64, 4096), (7, 11008)])
@pytest.mark.parametrize("mode", [0, 1])
def test_quantize_bit_exact(name, shape, mode):
    s = SCHEMES[name]
    rng = np.random.default_rng(seed_of(name, shape, mode))
    w = (rng.standard_normal(shape) * 0.02).astype(np.float16)
    w[0, : min(s.group_size, shape[1])] = 0  # all-zero group
    if shape[0] > 1:
        w[1, ::3] = np.float16(0.01)
    qw_ref, qs_ref = o.quantize(w, s, ["half_away", "half_even"][mode])
    qw, qs = ops.quantize(dev(w), s.bits, s.group_size, mode)
    assert (host_u32(qw) == qw_ref).all()
    assert (host_f16_bits(qs) == qs_ref.view(np.uint16)).all()


def test_quantize_golden(golden):
    for name in ("q4f16_1", "q3f16_1"):
        s = SCHEMES[name]
        for shp in ("2x13", "16x128" if name == "q4f16_1" else "16x120", "5x200"):
            for kind in ("uniform", "normal"):
                z = golden(f"quant_{name}_{shp}_{kind}")
                for mode, mname in ((0, "half_away"), (1, "half_even")):
                    qw, qs = ops.quantize(dev(z["w"]), s.bits, s.group_size, mode)
                    assert (host_u32(qw) == z[f"q_weight_{mname}"]).all(), (name, shp, kind, mname)
                    assert (host_f16_bits(qs) == z[f"q_scale_{mname}"].view(np.uint16)).all()


def test_quantize_extreme_values():
    # subnormal maxima (scale rounds to 0 -> +-inf codes), huge values, signed zeros
    s = SCHEMES["q4f16_1"]
    w = np.zeros((4, 64), np.float16)
    w[0, :4] = np.array([6e-8, -6e-8, 0.0, 1.2e-7], np.float16)
    w[1, :3] = np.array([65504.0, -65504.0, 1.0], np.float16)
    w[2, :] = np.float16(-0.0)
    w[3, 32:40] = np.array([1e-4, -1e-4, 5e-5, 2.5e-5, -7.5e-5, 0, 1e-5, -1e-5], np.float16)
    qw_ref, qs_ref = o.quantize(w, s)
    qw, qs = ops.quantize(dev(w), 4, 32)
    assert (host_u32(qw) == qw_ref).all() and (host_f16_bits(qs) == qs_ref.view(np.uint16)).all()


@pytest.mark.parametrize("name", ["q4f16_1", "q3f16_1"])
@pytest.mark.parametrize("mode", [0, 1])
def test_quantize_bit_exact_16m_values_all_magnitudes(name, mode):
    # 16.7 M values whose group maxima sweep the whole fp16 exponent range (denormal scales
    # included): the kernel's divide is a reciprocal plus one Newton step, and must still land on
    # the half the plain fp16 divide gives, every time.  Checked against the C restatement.
    from oracle import c_oracle

    s = SCHEMES[name]
    rng = np.random.default_rng(1234 + mode)
    rows, k = 4096, 4096 if s.bits == 4 else 4080
    mag = np.exp2(rng.uniform(-24, 15, size=(rows, k // s.group_size, 1))).astype(np.float32)
    w = (rng.standard_normal((rows, k // s.group_size, s.group_size)).astype(np.float32) * mag)
    w = np.clip(w, -65504, 65504).astype(np.float16).reshape(rows, k)
    w[::97, ::5] = 0
    qw_ref, qs_ref = c_oracle.quantize(w, s.bits, s.group_size, mode)
    qw, qs = ops.quantize(dev(w), s.bits, s.group_size, mode)
    assert np.array_equal(host_f16_bits(qs), qs_ref.view(np.uint16))
    bad = np.nonzero(host_u32(qw) != qw_ref)
    assert bad[0].size == 0, f"{bad[0].size} words differ, first at {bad[0][0]}, {bad[1][0]}"


@pytest.mark.parametrize("name", ["q4f16_1", "q3f16_1"])
def test_quantize_full_size_roundtrip_properties(name):
    # full decode shape: codes in range, re-quantizing the dequantized matrix is idempotent on
    # the codes' dequantized values, and a row sample agrees with the oracle bit for bit
    s = SCHEMES[name]
    n, k = (4096, 14336) if name == "q4f16_1" else (4096, 11008)
    g = torch.Generator(device=DEV).manual_seed(0)
    w = (torch.randn((n, k), generator=g, device=DEV) * 0.02).half()
    qw, qs = ops.quantize(w, s.bits, s.group_size)
    d = ops.dequantize(qw, qs, k, s.bits, s.group_size)
    step = qs.float().repeat_interleave(s.group_size, dim=1)[:, :k]
    assert bool(((d.float() - w.float()).abs() <= 0.5 * step * 1.04 + 1e-6).all())
    qw2, qs2 = ops.quantize(d, s.bits, s.group_size)
    d2 = ops.dequantize(qw2, qs2, k, s.bits, s.group_size)
    # dequantized values lie on the grid of their own group, so a second pass reproduces them
    # wherever the group maximum is still attained (always true when an extreme code is used)
    same = (d2 == d).float().mean().item()
    assert same > 0.999, same
    rows = [0, 1, n // 2, n - 1]
    qw_ref, qs_ref = o.quantize(w[rows].cpu().numpy(), s)
    assert (host_u32(qw[rows]) == qw_ref).all() and (host_f16_bits(qs[rows]) == qs_ref.view(np.uint16)).all()
    assert (host_f16_bits(d[rows]) == o.dequantize(qw_ref, qs_ref, s, k).view(np.uint16)).all()


@pytest.mark.parametrize("name", ["q4f16_1", "q3f16_1"])
@pytest.mark.parametrize("shape", [(2, 13), (16, 120), (16, 128), (5, 200), (33, 4096)])
def test_dequantize_bit_exact(name, shape):
    # random full-range storage words and scales, like the reference's test_dequantize_weight
    s = SCHEMES[name]
    rng = np.random.default_rng(seed_of(name, shape))
    n, k = shape
    qw = rng.integers(0, 2**32, (n, s.num_storage(k)), dtype=np.uint64).astype(np.uint32)
    qs = rng.random((n, s.num_group(k))).astype(np.float16)
    qs[0, 0] = np.float16(6e-8)  # subnormal scale
    d = ops.dequantize(dev(qw), dev(qs), k, s.bits, s.group_size)
    assert (host_f16_bits(d) == o.dequantize(qw, qs, s, k).view(np.uint16)).all()


def test_dequantize_golden(golden):
    for name in ("q4f16_1", "q3f16_1"):
        s = SCHEMES[name]
        for shp in ("2x13", "16x128" if name == "q4f16_1" else "16x120", "5x200"):
            z = golden(f"dequant_{name}_{shp}")
            k = z["dequant"].shape[1]
            d = ops.dequantize(dev(z["q_weight"]), dev(z["q_scale"]), k, s.bits, s.group_size)
            assert (host_f16_bits(d) == z["dequant"].view(np.uint16)).all()


@pytest.mark.parametrize("name", ["q4f16_1", "q3f16_1"])
def test_dequantize_via_identity_matmul(name):
    # the reference test's own trick: identity activations through the linear layer return W^T
    s = SCHEMES[name]
    rng = np.random.default_rng(5)
    n, k = 16, 120 if s.bits == 3 else 128
    qw = rng.integers(0, 2**32, (n, s.num_storage(k)), dtype=np.uint64).astype(np.uint32)
    qs = rng.random((n, s.num_group(k))).astype(np.float16)
    eye = np.eye(k, dtype=np.float16)
    y = ops.linear(dev(eye), dev(qw), dev(qs), s.bits, s.group_size)  # M = k > 8: GEMM path
    ref = o.dequantize(qw, qs, s, k).T
    np.testing.assert_allclose(y.cpu().numpy().astype(np.float32), ref.astype(np.float32), rtol=1e-3, atol=1e-3)
    for r0 in range(0, k, 8):  # and through the GEMV path, 8 rows at a time
        y8 = ops.linear(dev(eye[r0:r0 + 8]), dev(qw), dev(qs), s.bits, s.group_size)
        np.testing.assert_allclose(y8.cpu().numpy().astype(np.float32), ref[r0:r0 + 8].astype(np.float32),
                                   rtol=1e-3, atol=1e-3)


@pytest.mark.parametrize("name", ["q4f16_1", "q3f16_1"])
def test_embedding_take_bit_exact(name):
    s = SCHEMES[name]
    rng = np.random.default_rng(9)
    num, k = 1000, 4096 if s.bits == 4 else 200
    w = (rng.standard_normal((num, k)) * 0.02).astype(np.float16)
    qw, qs = o.quantize(w, s)
    ids = rng.integers(0, num, (3, 17)).astype(np.int32)
    ids[0, 0], ids[0, 1] = 0, num - 1
    emb = gq.GroupQuantizeEmbedding(num, k, gq.QUANTIZATION[name], device=DEV)
    emb.q_weight.data = dev(qw)
    emb.q_scale.data = dev(qs)
    out = emb(dev(ids))
    assert tuple(out.shape) == (3, 17, k)
    ref = o.embedding_take(ids.reshape(-1), qw, qs, s, k).reshape(3, 17, k)
    assert (host_f16_bits(out) == ref.view(np.uint16)).all()
    assert emb(dev(ids[:0])).shape == (0, 17, k)  # empty batch


# ------------------------------------------------------------------ GEMV / GEMM: tolerance


def _linear_case(s, m, n, k, seed, bias=False, scale=0.02):
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal((n, k)) * scale).astype(np.float16)
    qw, qs = o.quantize(w, s)
    x = rng.standard_normal((m, k)).astype(np.float16)
    b = rng.standard_normal(n).astype(np.float16) if bias else None
    return x, qw, qs, b


@pytest.mark.parametrize("name", ["q4f16_1", "q3f16_1"])
@pytest.mark.parametrize("m,n,k", [(1, 64, 20480), (2, 64, 20480), (1, 36, 28672), (2, 128, 9000), (1, 62, 20481),
                                   (2, 62, 20004), (1, 130, 18944), (1, 64, 24576), (1, 64, 24584)])
def test_one_and_two_rows_of_a_long_k(name, m, n, k):
    # K past what the register GEMV holds per lane (12 groups for one row, 4 for two): the quad-row kernel takes
    # over (two rows: from K > 8192; one row: from K > 24576), the LDS GEMV where that one declines the shape
    # (N % 4, K % 8)
    s = SCHEMES[name]
    x, qw, qs, b = _linear_case(s, m, n, k, 7 * m + n + k, bias=True)
    y = ops.linear(dev(x), dev(qw), dev(qs), s.bits, s.group_size, dev(b))
    ref = o.linear_fp32(x, qw, qs, s, b)
    assert_linear_ok(y, ref, x, k, f"long K {name} {m}x{n}x{k}")
    y32 = ops.linear(dev(x), dev(qw), dev(qs), s.bits, s.group_size, dev(b), out_dtype=torch.float32)
    assert_linear_ok(y32, ref, x, k, f"long K {name} {m}x{n}x{k} fp32 out")
    if n % 2 == 0:
        fused = ops.linear_silu_mul(dev(x), dev(qw), dev(qs), s.bits, s.group_size)
        assert torch.equal(fused, ops.silu_mul(ops.linear(dev(x), dev(qw), dev(qs), s.bits, s.group_size)))


@pytest.mark.parametrize("name", ["q4f16_1", "q3f16_1"])
@pytest.mark.parametrize("ksplit", [0, 1])
@pytest.mark.parametrize("n,k", [(130, 8200), (1000, 11008), (4100, 14336), (66, 18944), (64, 24576), (40, 10240),
                                 (9000, 8192)])
def test_gemv_long_k_shared_between_two_waves(name, ksplit, n, k):
    """One row, 5 to 12 groups per lane: two neighbouring waves take half of K each and their row sums meet in LDS after
    the walk (odd group counts per lane, a last group that is partly filled, more row sets than waves, float32 output,
    expert ids with their own rows of x); against the oracle, and forced off for the whole-K form next to it."""
    s = SCHEMES[name]
    x, qw, qs, _ = _linear_case(s, 1, n, k, n + k + ksplit, bias=False)
    gq._lib.set_option("gemv_ksplit", ksplit)
    try:
        y = ops.linear(dev(x), dev(qw), dev(qs), s.bits, s.group_size, None)
        kern = gq._lib.last_kernel()
        y32 = ops.linear(dev(x), dev(qw), dev(qs), s.bits, s.group_size, None, torch.float32)
        # two expert slots reading rows 0 and 1 of x (the same matrix as both experts' weights, stacked)
        x2 = np.concatenate([x, x[:, ::-1]], axis=0).copy()
        qw2, qs2 = np.stack([qw, qw]), np.stack([qs, qs])
        ids = np.array([[1, 0]], np.int32)
        ym = ops.moe_gemv(dev(x2), dev(qw2), dev(qs2), dev(ids), s.bits, s.group_size)
    finally:
        gq._lib.set_option("gemv_ksplit", -1)
    groups_per_lane = -(-(-(-k // s.group_size)) // 64)
    # (forced on, the pair form takes any K of two groups per lane or more; by itself it runs from five on, and on
    #  K of exactly two for mid-sized matrices: test_gemv_short_k_pairs)
    assert kern.startswith("gq::gemv_reg_kernel") and kern.endswith(",2>") == (ksplit == 1 and groups_per_lane >= 2), kern
    ref = o.linear_fp32(x, qw, qs, s)
    assert_linear_ok(y, ref, x, k, f"gemv long K {name} ksplit={ksplit} {n}x{k}")
    assert_linear_ok(y32, ref, x, k, f"gemv long K ksplit={ksplit} fp32 out")
    assert_linear_ok(ym, o.moe_dequantize_gemv_fp32(x2, qw2, qs2, ids, s), x2, k, f"moe gemv long K ksplit={ksplit}")


@pytest.mark.parametrize("name", ["q4f16_1", "q3f16_1"])
@pytest.mark.parametrize("n", [6144, 6150, 28672])
def test_gemv_short_k_pairs(name, n):
    """K of two groups per lane on a mid-sized matrix: by default two neighbouring waves take one group per lane each
    (one row per set, the halves meet in LDS after the walk); against the oracle, float32 output too."""
    s = SCHEMES[name]
    k = 4096
    x, qw, qs, _ = _linear_case(s, 1, n, k, n + 5, bias=False)
    y = ops.linear(dev(x), dev(qw), dev(qs), s.bits, s.group_size, None)
    kern = gq._lib.last_kernel()
    assert kern.startswith("gq::gemv_reg_kernel") and kern.endswith(",2>"), kern
    y32 = ops.linear(dev(x), dev(qw), dev(qs), s.bits, s.group_size, None, torch.float32)
    ref = o.linear_fp32(x, qw, qs, s)
    assert_linear_ok(y, ref, x, k, f"gemv short K pairs {name} n={n}")
    assert_linear_ok(y32, ref, x, k, f"gemv short K pairs {name} n={n} fp32")


@pytest.mark.parametrize("name", ["q4f16_1", "q3f16_1"])
@pytest.mark.parametrize("m", [1, 2, 3, 4, 5, 6, 7, 8])
def test_gemv_all_batches(name, m):
    s = SCHEMES[name]
    n, k = 384, 1024 if s.bits == 4 else 1000
    x, qw, qs, b = _linear_case(s, m, n, k, 100 + m, bias=(m % 2 == 0))
    y = ops.linear(dev(x), dev(qw), dev(qs), s.bits, s.group_size, dev(b) if b is not None else None)
    assert y.dtype == torch.float16 and tuple(y.shape) == (m, n)
    assert_linear_ok(y, o.linear_fp32(x, qw, qs, s, b), x, k, f"gemv {name} m={m}")


@pytest.mark.parametrize("name,n,k", [
    ("q4f16_1", 4096, 4096),     # config 1 / o_proj
    ("q4f16_1", 6144, 4096),     # fused qkv
    ("q4f16_1", 4096, 14336),    # down
    ("q3f16_1", 4096, 4096),     # o (K is not a multiple of 40: padded last group)
    ("q3f16_1", 4096, 11008),    # down (padded K)
    ("q4f16_1", 1000, 72),       # ragged: N not a multiple of the row block, K of 8 only
    ("q4f16_1", 7, 13),          # the reference test's odd shape
    ("q3f16_1", 7, 13),
    ("q4f16_1", 33, 20000),      # long K: several LDS chunks
])
@pytest.mark.parametrize("m", [1, 4, 8])
def test_gemv_shapes(name, n, k, m):
    s = SCHEMES[name]
    x, qw, qs, _ = _linear_case(s, m, n, k, n + k + m)
    y = ops.linear(dev(x), dev(qw), dev(qs), s.bits, s.group_size)
    assert_linear_ok(y, o.linear_fp32(x, qw, qs, s), x, k, f"gemv {name} {n}x{k} m={m}")


@pytest.mark.parametrize("rows_per_wave", [1, 2, 4])
def test_gemv_rows_per_wave_variants(rows_per_wave):
    s = SCHEMES["q4f16_1"]
    x, qw, qs, _ = _linear_case(s, 2, 1030, 2048, 77)
    gq._lib.set_option("gemv_rows_per_wave", rows_per_wave)
    try:
        y = ops.linear(dev(x), dev(qw), dev(qs), 4, 32)
    finally:
        gq._lib.set_option("gemv_rows_per_wave", -1)
    assert_linear_ok(y, o.linear_fp32(x, qw, qs, s), x, 2048, f"R={rows_per_wave}")


@pytest.mark.parametrize("name", ["q4f16_1", "q3f16_1"])
@pytest.mark.parametrize("m", [1, 2, 5])
def test_gemv_lds_kernel_forced(name, m):
    # the LDS-staged fallback kernel must agree too (it normally only sees odd shapes)
    s = SCHEMES[name]
    n, k = 777, 2048 if s.bits == 4 else 2000
    x, qw, qs, b = _linear_case(s, m, n, k, 900 + m, bias=True)
    gq._lib.set_option("gemv_variant", 0)
    gq._lib.set_option("gemm_variant", 2)  # keep 3..8 rows on the GEMV path for q4 as well
    try:
        y = ops.linear(dev(x), dev(qw), dev(qs), s.bits, s.group_size, dev(b))
    finally:
        gq._lib.set_option("gemv_variant", -1)
        gq._lib.set_option("gemm_variant", -1)
    assert_linear_ok(y, o.linear_fp32(x, qw, qs, s, b), x, k, f"lds gemv {name} m={m}")


@pytest.mark.parametrize("mode", [2, 3, 4])  # unpipelined, chunk-pipelined, persistent
@pytest.mark.parametrize("m", [3, 4, 8, 9, 16])
@pytest.mark.parametrize("n,k", [(520, 1024), (100, 4096), (2100, 72), (64, 6176)])
def test_skinny_kernel_forms(mode, m, n, k):
    s = SCHEMES["q4f16_1"]
    x, qw, qs, b = _linear_case(s, m, n, k, 31 * m + n + k, bias=True)
    gq._lib.set_option("gemv_variant", mode)
    try:
        y = ops.linear(dev(x), dev(qw), dev(qs), 4, 32, dev(b))
        y32 = ops.linear(dev(x), dev(qw), dev(qs), 4, 32, None, torch.float32)
    finally:
        gq._lib.set_option("gemv_variant", -1)
    ref = o.linear_fp32(x, qw, qs, s, b)
    assert_linear_ok(y, ref, x, k, f"skinny mode {mode} {m}x{n}x{k}")
    assert_linear_ok(y32, ref - b.astype(np.float64), x, k, f"skinny mode {mode} fp32 out")


@pytest.mark.parametrize("form", [-1, 2, 4])  # ring of two tiles with the offsets kept, four without, three with
@pytest.mark.parametrize("m", [1, 9, 16, 17, 40])  # one pass, a full one, and rows that take two and three passes
@pytest.mark.parametrize("n,k", [(96, 256), (1000, 1024), (520, 4096), (72, 8192), (256, 14336), (16, 512)])
def test_midrow_kernel(form, m, n, k):
    """The kernel that feeds the matrix instruction unscaled weight operands and scales its result, forced (it runs by
    default on large matrices at 9..16 rows): K of one to sixteen wave shares and of several phases, a last tile of
    fewer than 16 weight rows, bias, residual and float32 output."""
    s = SCHEMES["q4f16_1"]
    x, qw, qs, b = _linear_case(s, m, n, k, 13 * m + n + k + form, bias=True)
    res = np.random.default_rng(m + n).standard_normal((m, n)).astype(np.float16)
    gq._lib.set_option("gemv_variant", 10)
    gq._lib.set_option("gemv_rows_per_wave", form)
    try:
        y = ops.linear(dev(x), dev(qw), dev(qs), 4, 32, dev(b))
        kern = gq._lib.last_kernel()
        y32 = ops.linear(dev(x), dev(qw), dev(qs), 4, 32, None, torch.float32)
        yr = ops.linear(dev(x), dev(qw), dev(qs), 4, 32, dev(b), residual=dev(res))
    finally:
        gq._lib.set_option("gemv_variant", -1)
        gq._lib.set_option("gemv_rows_per_wave", -1)
    if k > 4096 and form == 2:  # (several phases exist for the default instance only: K slices where the call's scratch
        #                          holds their partial sums, else the shape falls through)
        assert not kern.startswith("gq::midrow_kernel") or " phases=1 " in kern, kern
    else:
        assert kern.startswith("gq::midrow_kernel<"), kern
    ref = o.linear_fp32(x, qw, qs, s, b)
    assert_linear_ok(y, ref, x, k, f"mid-row form {form} {m}x{n}x{k} [{kern}]")
    assert_linear_ok(y32, ref - b.astype(np.float64), x, k, f"mid-row form {form} fp32 out")
    assert_linear_ok(yr, ref + res.astype(np.float64), x, k, f"mid-row form {form} residual")


def test_midrow_kernel_random_shapes():
    """Forty random shapes through the forced kernel against the oracle: rows 1..48 (one to three passes of one or two batch
    tiles), N from 16 up (whole and ragged last tiles), K of 1 to 40 wave shares (1, 2, 4, 8, 16 waves per tile, one to three
    phases), with and without bias."""
    s = SCHEMES["q4f16_1"]
    rng = np.random.default_rng(20250)
    for case in range(40):
        m = int(rng.integers(1, 49))
        n = int(rng.choice([16, 31, 48, 100, 257, 512, 1000, 1552, 3000]))
        k = 256 * int(rng.choice([1, 2, 3, 4, 5, 8, 13, 16, 17, 24, 40]))
        x, qw, qs, b = _linear_case(s, m, n, k, 1000 + case, bias=bool(case & 1))
        gq._lib.set_option("gemv_variant", 10)
        try:
            y = ops.linear(dev(x), dev(qw), dev(qs), 4, 32, None if b is None else dev(b))
            kern = gq._lib.last_kernel()
        finally:
            gq._lib.set_option("gemv_variant", -1)
        assert kern.startswith("gq::midrow_kernel<"), (m, n, k, kern)
        assert_linear_ok(y, o.linear_fp32(x, qw, qs, s, b), x, k, f"mid-row random case {case}: {m}x{n}x{k} [{kern}]")


@pytest.mark.parametrize("m", [9, 12, 16, 17, 32])
@pytest.mark.parametrize("n,k", [(6144, 4096), (28672, 4096), (8192, 8192)])
def test_midrow_kernel_is_the_default_on_large_matrices(m, n, k):
    """9..16 rows of q4 on matrices of 24 M weights or more with K up to 4096 (48 M with K up to 8192, two phases), 17..32 rows
    from 48 M weights on with K up to 4096: the default dispatch, against the oracle on a sample of the columns; the fused gate/up form takes the same kernel and equals
    linear + silu_mul bit for bit."""
    s = SCHEMES["q4f16_1"]
    rng = np.random.default_rng(seed_of("midrow", m, n, k))
    qw = rng.integers(0, 2**32, (n, k // 8), dtype=np.uint32)
    qs = (rng.random((n, k // 32)) * 0.02 + 0.001).astype(np.float16)
    x = rng.standard_normal((m, k)).astype(np.float16)
    cols = np.unique(np.concatenate([[0, 1, n // 2, n - 1], rng.integers(0, n, 300)]))
    # (17..32 rows: two batch tiles, from 48 M weights on and with K of one phase only)
    want = m <= 16 or (n * k >= 48 << 20 and k <= 4096)
    y = ops.linear(dev(x), dev(qw), dev(qs), 4, 32)
    assert gq._lib.last_kernel().startswith(f"gq::midrow_kernel<{1 if m <= 16 else 2},") == want, gq._lib.last_kernel()
    assert_linear_ok(y[:, torch.from_numpy(cols).to(DEV)], o.linear_fp32(x, qw[cols], qs[cols], s), x, k, f"mid-row {m}x{n}x{k}")
    fused = ops.linear_silu_mul(dev(x), dev(qw), dev(qs), 4, 32)
    assert gq._lib.last_kernel().startswith("gq::midrow_kernel<") == want, gq._lib.last_kernel()
    assert torch.equal(fused, ops.silu_mul(y))


@pytest.mark.parametrize("m,n,k", [(9, 4096, 14336), (16, 4096, 14336), (32, 4096, 14336), (12, 5120, 13824), (16, 8192, 28672),
                                   (9, 10240, 8192), (24, 32768, 8192), (32, 2048, 8192), (5, 5120, 13824), (8, 8192, 28672),
                                   (7, 4096, 14336)])
def test_midrow_kernel_k_slices(m, n, k):
    """A K of several phases on a plain linear whose caller brings the scratch: one workgroup row per phase's worth of K,
    fp32 partial sums, a reduction that adds bias and residual and casts.  The default at 9..16 rows from 24 M weights on, at
    17..32 rows from 256 M and at 5..8 rows of a K beyond 8192 from 64 M; forced elsewhere.  Against the oracle on a sample of the columns, with bias, residual and
    float32 output; the fused gate/up form equals linear + silu_mul bit for bit; without the scratch the call still answers
    (phases inside the workgroup, or the GEMM's tiles)."""
    s = SCHEMES["q4f16_1"]
    rng = np.random.default_rng(seed_of("midrow-slices", m, n, k))
    qw = rng.integers(0, 2**32, (n, k // 8), dtype=np.uint32)
    qs = (rng.random((n, k // 32)) * 0.02 + 0.001).astype(np.float16)
    x = rng.standard_normal((m, k)).astype(np.float16)
    bias = rng.standard_normal(n).astype(np.float16)
    res = rng.standard_normal((m, n)).astype(np.float16)
    cols = np.unique(np.concatenate([[0, 1, n // 2, n - 1], rng.integers(0, n, 200)]))
    pick = torch.from_numpy(cols).to(DEV)
    default = (8 < m <= 16 and n * k >= 24 << 20) or (m > 16 and n * k >= 256 << 20) or (m <= 8 and k > 8192 and n * k >= 64 << 20)
    phases = -(-(k // 32) // 128)
    if not default:
        gq._lib.set_option("gemv_variant", 10)
    try:
        y = ops.linear(dev(x), dev(qw), dev(qs), 4, 32)
        kern = gq._lib.last_kernel()
        yb = ops.linear(dev(x), dev(qw), dev(qs), 4, 32, bias=dev(bias), residual=dev(res), out_dtype=torch.float32)
        fused = ops.linear_silu_mul(dev(x), dev(qw), dev(qs), 4, 32)
        kern_fused = gq._lib.last_kernel()
    finally:
        gq._lib.set_option("gemv_variant", -1)
    assert kern.startswith(f"gq::midrow_kernel<{1 if m <= 16 else 2},") and f"slices={phases} " in kern, kern
    assert kern_fused.startswith("gq::midrow_kernel<") and f"slices={phases} " in kern_fused, kern_fused
    ref = o.linear_fp32(x, qw[cols], qs[cols], s)
    assert_linear_ok(y[:, pick], ref, x, k, f"mid-row slices {m}x{n}x{k}")
    assert_linear_ok(yb[:, pick], ref + bias[cols].astype(np.float32) + res[:, cols].astype(np.float32), x, k,
                     f"mid-row slices, bias + residual, f32 {m}x{n}x{k}")
    assert torch.equal(fused, ops.silu_mul(y))
    # no scratch: the same call answers without the slices
    out = torch.empty((m, n), dtype=torch.float16, device=DEV)
    dx, dqw, dqs = dev(x), dev(qw), dev(qs)
    gq._lib.call("mi355gq_linear", dx.data_ptr(), dqw.data_ptr(), dqs.data_ptr(), None, m, n, k, 4, 32, gq._lib.F16,
                 out.data_ptr(), None, 0, ops._stream())
    torch.cuda.synchronize()
    assert "slices=" not in gq._lib.last_kernel() or "slices=1 " in gq._lib.last_kernel(), gq._lib.last_kernel()
    assert_linear_ok(out[:, pick], ref, x, k, f"no scratch {m}x{n}x{k}")


@pytest.mark.parametrize("k", [1024, 4096, 14336])
@pytest.mark.parametrize("paired", [False, True])
@pytest.mark.parametrize("tiles", [1, 2])  # batch tiles of 16 rows per pass
def test_midrow_kernel_grouped(k, paired, tiles):
    """Expert segments: an empty expert, one of a single row, one of 16 rows (a full pass of one batch tile), one of 19 (two
    passes of one tile, one of two) and one of 40 (three passes / two), the gather of the activation rows folded in, int32 and
    int64 indptr; the fused gate/up form against linear + silu_mul of the same kernel, bit for bit."""
    s = SCHEMES["q4f16_1"]
    rng = np.random.default_rng(63 + k)
    ne, n = 5, 224
    w = (rng.standard_normal((ne, n, k)) * 0.02).astype(np.float16)
    qw, qs = o.quantize(w, s)
    ip = np.array([0, 1, 1, 17, 36, 76], np.int32)
    xs = rng.standard_normal((25, k)).astype(np.float16)
    rows = rng.integers(0, 25, 76).astype(np.int32)
    x = xs[rows]
    gq._lib.set_option("gemv_variant", 9 + tiles)
    try:
        out = ops.moe_experts(dev(xs), dev(rows), dev(qw), dev(qs), dev(ip), 4, 32, silu_mul_halves=paired)
        kern = gq._lib.last_kernel()
        out64 = ops.moe_experts(dev(x), None, dev(qw), dev(qs), dev(ip.astype(np.int64)), 4, 32, silu_mul_halves=paired)
        plain = ops.moe_experts(dev(x), None, dev(qw), dev(qs), dev(ip), 4, 32)
    finally:
        gq._lib.set_option("gemv_variant", -1)
    assert kern.startswith(f"gq::midrow_kernel<{tiles},"), kern
    assert torch.equal(out, out64)
    assert_linear_ok(plain, o.dequantize_group_gemm_fp32(x, qw, qs, ip, s), x, k, f"grouped mid-row k={k}")
    if paired:
        assert torch.equal(out, ops.silu_mul(plain))
    else:
        assert torch.equal(out, plain)


def test_midrow_kernel_is_the_default_between_few_rows_and_tiles():
    """Four to eight rows per expert on average (up to 16 experts, q4) with one batch tile per pass, up to 24 with two where
    K is one phase: the default dispatch of the grouped matmul."""
    s = SCHEMES["q4f16_1"]
    rng = np.random.default_rng(64)
    ne, n, k = 8, 96, 512
    w = (rng.standard_normal((ne, n, k)) * 0.02).astype(np.float16)
    qw, qs = o.quantize(w, s)
    ip = np.array([0, 4, 10, 15, 28, 37, 42, 55, 63], np.int32)
    for scale_rows, rows, want in ((1, 32, ""), (1, 33, "gq::midrow_kernel<1,"), (1, 63, "gq::midrow_kernel<1,"),
                                   (3, 65, "gq::midrow_kernel<2,"), (3, 189, "gq::midrow_kernel<2,"), (4, 200, "")):
        ipr = np.minimum(ip * scale_rows, rows).astype(np.int32)
        ipr[-1] = rows
        x = rng.standard_normal((rows, k)).astype(np.float16)
        out = ops.moe_group_gemm(dev(x), dev(qw), dev(qs), dev(ipr), 4, 32)
        kern = gq._lib.last_kernel()
        assert (kern.startswith(want) if want else not kern.startswith("gq::midrow_kernel")), (rows, kern)
        assert_linear_ok(out, o.dequantize_group_gemm_fp32(x, qw, qs, ipr, s), x, k, f"grouped, {rows} rows over {ne} experts")
    # many experts (their longest segment is further above the average): 2 to 6 rows per expert with one batch tile, up to 16 with two
    ne = 40
    w = (rng.standard_normal((ne, 32, k)) * 0.02).astype(np.float16)
    qw, qs = o.quantize(w, s)
    for rows, want in ((80, ""), (90, "gq::midrow_kernel<1,"), (240, "gq::midrow_kernel<1,"), (250, "gq::midrow_kernel<2,"),
                       (640, "gq::midrow_kernel<2,"), (650, "")):
        cuts = np.sort(rng.integers(0, rows + 1, ne - 1))
        ipr = np.concatenate([[0], cuts, [rows]]).astype(np.int32)
        x = rng.standard_normal((rows, k)).astype(np.float16)
        out = ops.moe_group_gemm(dev(x), dev(qw), dev(qs), dev(ipr), 4, 32)
        kern = gq._lib.last_kernel()
        assert (kern.startswith(want) if want else not kern.startswith("gq::midrow_kernel")), (rows, kern)
        assert_linear_ok(out, o.dequantize_group_gemm_fp32(x, qw, qs, ipr, s), x, k, f"grouped, {rows} rows over {ne} experts")


@pytest.mark.parametrize("mode", [2, 3, 4])
def test_skinny_kernel_forms_grouped(mode):
    s = SCHEMES["q4f16_1"]
    rng = np.random.default_rng(61)
    ne, n, k = 5, 200, 1024
    w = (rng.standard_normal((ne, n, k)) * 0.02).astype(np.float16)
    qw, qs = o.quantize(w, s)
    ip = np.array([0, 2, 2, 21, 22, 40], np.int32)  # an empty expert and one with 19 rows (2 m-tiles)
    x = rng.standard_normal((40, k)).astype(np.float16)
    gq._lib.set_option("gemv_variant", mode)
    try:
        out = ops.moe_group_gemm(dev(x), dev(qw), dev(qs), dev(ip), 4, 32)
    finally:
        gq._lib.set_option("gemv_variant", -1)
    assert_linear_ok(out, o.dequantize_group_gemm_fp32(x, qw, qs, ip, s), x, k, f"grouped skinny mode {mode}")


@pytest.mark.parametrize("name", ["q4f16_1", "q3f16_1"])
@pytest.mark.parametrize("u", [-1, 2, 8])  # iterations per item: heuristic, smallest, largest
@pytest.mark.parametrize("qp", [1, 2])  # quads per item (two: each read of x meets the weights of two quads)
@pytest.mark.parametrize("m", [3, 4, 5, 8])
@pytest.mark.parametrize("n,k", [(520, 1024), (100, 4096), (2100, 72), (64, 6176), (4, 256)])
def test_quadrow_kernel(name, u, qp, m, n, k):
    # the 4x4x4-MFMA kernel, forced; it is also what 3 <= M <= 8 takes by default
    s = SCHEMES[name]
    if s.bits == 3:
        k = {1024: 1000, 4096: 4000, 72: 80, 6176: 6200, 256: 240}[k]  # whole, partial and odd group counts of 40
    x, qw, qs, b = _linear_case(s, m, n, k, 77 * m + n + k, bias=True)
    gq._lib.set_option("gemv_variant", 6)
    gq._lib.set_option("gemv_rows_per_wave", u)
    gq._lib.set_option("quad_pairs", qp)
    try:
        y = ops.linear(dev(x), dev(qw), dev(qs), s.bits, s.group_size, dev(b))
        assert gq._lib.last_kernel().endswith(f",{qp}>"), gq._lib.last_kernel()
        y32 = ops.linear(dev(x), dev(qw), dev(qs), s.bits, s.group_size, None, torch.float32)
    finally:
        gq._lib.set_option("gemv_variant", -1)
        gq._lib.set_option("gemv_rows_per_wave", -1)
        gq._lib.set_option("quad_pairs", -1)
    ref = o.linear_fp32(x, qw, qs, s, b)
    assert_linear_ok(y, ref, x, k, f"quad-row {name} u={u} qp={qp} {m}x{n}x{k}")
    assert_linear_ok(y32, ref - b.astype(np.float64), x, k, f"quad-row u={u} qp={qp} fp32 out")


@pytest.mark.parametrize("name", ["q4f16_1", "q3f16_1"])
@pytest.mark.parametrize("ksplit", [-1, 0, 1, 2, 3])  # log2 of the waves that share a quad's K range
@pytest.mark.parametrize("waves", [-1, 16])  # 16 waves in all: every walker goes through many quads
@pytest.mark.parametrize("m", [3, 4, 5, 8])
@pytest.mark.parametrize("n,k", [(520, 1024), (100, 4096), (2100, 72), (64, 6176), (4, 256), (36, 14336), (1024, 4096)])
def test_quadreg_kernel(name, ksplit, waves, m, n, k):
    """The few-row kernel that keeps its slice of x in registers, forced: every split of K among 1..8 waves that the
    shape admits (iterations per wave 1..4; the others must be declined), one quad per walker and many, bias + residual,
    float32 output, and the folded activation bit for bit against the two steps."""
    s = SCHEMES[name]
    if s.bits == 3:
        k = {1024: 1000, 4096: 4000, 72: 80, 6176: 6200, 256: 240, 14336: 11008}[k]
    x, qw, qs, b = _linear_case(s, m, n, k, 13 * m + n + k + ksplit, bias=True)
    res = np.random.default_rng(n + k).standard_normal((m, n)).astype(np.float16)
    niter = -(-s.num_group(k) // 16)
    umax = 2 if m > 4 else 4
    gq._lib.set_option("gemv_variant", 9)
    gq._lib.set_option("quad_ksplit", ksplit)
    gq._lib.set_option("gemv_waves", waves)
    try:
        y = ops.linear(dev(x), dev(qw), dev(qs), s.bits, s.group_size, dev(b), residual=dev(res))
        kern = gq._lib.last_kernel()
        if ksplit >= 0 and waves < 0:  # (with 16 waves the partial sums of a long walk may not fit LDS: declined too)
            u = -(-niter // (1 << ksplit))
            fits = u <= umax and niter <= 16
            assert kern.startswith("gq::quadreg_kernel") == fits, (kern, niter, ksplit)
        y32 = ops.linear(dev(x), dev(qw), dev(qs), s.bits, s.group_size, None, torch.float32)
        y16 = ops.linear(dev(x), dev(qw), dev(qs), s.bits, s.group_size, None)
        kern16 = gq._lib.last_kernel()
        if n % 8 == 0:
            fused = ops.linear_silu_mul(dev(x), dev(qw), dev(qs), s.bits, s.group_size)
            # (a declined shape falls back to different kernels for the two forms: equal bits only within a family)
            if kern16.startswith("gq::quadreg_kernel") and gq._lib.last_kernel().startswith("gq::quadreg_kernel"):
                assert torch.equal(fused, ops.silu_mul(y16))
    finally:
        for opt in ("gemv_variant", "quad_ksplit", "gemv_waves"):
            gq._lib.set_option(opt, -1)
    ref = o.linear_fp32(x, qw, qs, s)
    what = f"quadreg {name} ksplit={ksplit} waves={waves} {m}x{n}x{k} [{kern}]"
    assert_linear_ok(y, ref + b.astype(np.float64) + res.astype(np.float64), x, k, what)
    assert_linear_ok(y32, ref, x, k, what + " fp32 out")
    assert_linear_ok(y16, ref, x, k, what + " plain")


@pytest.mark.parametrize("name", ["q4f16_1", "q3f16_1"])
@pytest.mark.parametrize("m", [1, 3, 4, 8, 16, 40])
@pytest.mark.parametrize("log2_scale", [-6, -10, -13])
def test_linear_small_activations(name, m, log2_scale):
    """Activations far below 1 (N(0, 1) * 2^-6, 2^-10, 2^-13; the last are float16 subnormals in part): the bound
    scales with max|x|, so a kernel that loses bits of small activations fails it.  The few-row kernel divides the
    activations of its scaled operand classes by 16 (q3: 8, 64) in float16, which is exact down to |x| = 2^-10 (2^-8);
    below that a product moves by at most 2^-25 * 16 (64) * (q - m) * scale: at 2^-13 the relative L2 error may reach
    4e-3 there (q3), which the test allows for that kernel and that scale only."""
    s = SCHEMES[name]
    n, k = 520, 4096 if s.bits == 4 else 4000
    rng = np.random.default_rng(seed_of("small", name, m, log2_scale))
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float16)
    qw, qs = o.quantize(w, s)
    x = (rng.standard_normal((m, k)) * 2.0**log2_scale).astype(np.float16)
    y = ops.linear(dev(x), dev(qw), dev(qs), s.bits, s.group_size, None, torch.float32)
    kern = gq._lib.last_kernel()
    ref = o.linear_fp32(x, qw, qs, s)
    err, bound, rel = o.check_linear(y.cpu().numpy(), ref, x, k)
    loose = log2_scale == -13 and kern.startswith(("gq::quad_kernel", "gq::quadreg_kernel"))
    assert err <= bound, (kern, err, bound)
    assert rel <= (6e-3 if loose else REL_L2), (kern, rel)


@pytest.mark.parametrize("name", ["q4f16_1", "q3f16_1"])
@pytest.mark.parametrize("u", [-1, 2, 4, 8])
@pytest.mark.parametrize("qp", [1, 2])
@pytest.mark.parametrize("m", [3, 4, 7])
@pytest.mark.parametrize("n,k", [(520, 1024), (2100, 200), (72, 6176)])
def test_quadrow_kernel_many_quads_per_wave(name, u, qp, m, n, k):
    """Sixteen waves in all, so that every wave walks many quad sets and items of different quads follow each other in its
    register ring (with the default launch shape a wave has one quad set): every item size and quads-per-item form, with
    bias + residual, plain with float32 output, and the folded activation, against the oracle."""
    s = SCHEMES[name]
    if s.bits == 3:
        k = {1024: 1000, 200: 200, 6176: 6200}[k]
    x, qw, qs, b = _linear_case(s, m, n, k, 11 * m + n + k + u, bias=True)
    res = np.random.default_rng(n + k).standard_normal((m, n)).astype(np.float16)
    gq._lib.set_option("gemv_variant", 6)
    gq._lib.set_option("gemv_rows_per_wave", u)
    gq._lib.set_option("quad_pairs", qp)
    gq._lib.set_option("gemv_waves", 16)
    try:
        y = ops.linear(dev(x), dev(qw), dev(qs), s.bits, s.group_size, dev(b), residual=dev(res))
        assert gq._lib.last_kernel().startswith("gq::quad_kernel") and gq._lib.last_kernel().endswith(f",{qp}>")
        y32 = ops.linear(dev(x), dev(qw), dev(qs), s.bits, s.group_size, None, torch.float32)
        y16 = ops.linear(dev(x), dev(qw), dev(qs), s.bits, s.group_size, None)
        if n % 8 == 0:
            assert torch.equal(ops.linear_silu_mul(dev(x), dev(qw), dev(qs), s.bits, s.group_size), ops.silu_mul(y16))
            assert gq._lib.last_kernel().startswith("gq::quad_kernel")
    finally:
        for opt in ("gemv_variant", "gemv_rows_per_wave", "quad_pairs", "gemv_waves"):
            gq._lib.set_option(opt, -1)
    ref = o.linear_fp32(x, qw, qs, s)
    assert_linear_ok(y, ref + b.astype(np.float64) + res.astype(np.float64), x, k, f"quad-row walk {name} u={u} qp={qp} {m}x{n}x{k}")
    assert_linear_ok(y32, ref, x, k, f"quad-row walk u={u} qp={qp} fp32 out")
    assert_linear_ok(y16, ref, x, k, f"quad-row walk u={u} qp={qp}")


@pytest.mark.parametrize("name", ["q4f16_1", "q3f16_1"])
@pytest.mark.parametrize("ksplit", [0, 1, 2])  # 1, 2, 4 neighbouring waves share the K range of a quad set
@pytest.mark.parametrize("qp", [1, 2])
@pytest.mark.parametrize("m", [3, 4, 8])
@pytest.mark.parametrize("n,k", [(520, 1024), (100, 4096), (1024, 4096), (64, 6176), (4, 256), (36, 2080)])
def test_quadrow_kernel_k_shared_between_waves(name, ksplit, qp, m, n, k):
    """Matrices with few quads: the waves of a workgroup split the K range of a quad set and the first of them adds the
    shares up after the walk (step counts that do not divide, shares that come out empty, an odd number of quads with two
    quads per item); plain, float32 and folded-activation outputs against the oracle."""
    s = SCHEMES[name]
    if s.bits == 3:
        k = {1024: 1000, 4096: 4000, 6176: 6200, 256: 240, 2080: 2080}[k]
    x, qw, qs, _ = _linear_case(s, m, n, k, 3 * m + n + k + ksplit, bias=False)
    gq._lib.set_option("gemv_variant", 6)
    gq._lib.set_option("quad_pairs", qp)
    gq._lib.set_option("quad_ksplit", ksplit)
    try:
        y = ops.linear(dev(x), dev(qw), dev(qs), s.bits, s.group_size, None)
        assert gq._lib.last_kernel().startswith("gq::quad_kernel"), gq._lib.last_kernel()
        y32 = ops.linear(dev(x), dev(qw), dev(qs), s.bits, s.group_size, None, torch.float32)
        if n % 8 == 0:  # the folded activation shares the K range the same way: same bits as the two steps
            assert torch.equal(ops.linear_silu_mul(dev(x), dev(qw), dev(qs), s.bits, s.group_size), ops.silu_mul(y))
    finally:
        gq._lib.set_option("gemv_variant", -1)
        gq._lib.set_option("quad_pairs", -1)
        gq._lib.set_option("quad_ksplit", -1)
    ref = o.linear_fp32(x, qw, qs, s)
    assert_linear_ok(y, ref, x, k, f"quad-row k shared {name} ksplit={ksplit} qp={qp} {m}x{n}x{k}")
    assert_linear_ok(y32, ref, x, k, f"quad-row k shared ksplit={ksplit} qp={qp} fp32 out")


@pytest.mark.parametrize("name", ["q4f16_1", "q3f16_1"])
@pytest.mark.parametrize("waves", [-1, 8])  # 8 waves in all: every wave walks many quads
@pytest.mark.parametrize("qp", [1, 2])
@pytest.mark.parametrize("m,n,k", [(8, 64, 14336), (5, 520, 20520), (3, 132, 20480), (8, 520, 8200), (8, 36, 14336)])
def test_quadrow_kernel_k_phases(name, waves, qp, m, n, k):
    # x does not fit LDS whole: K is walked in 2-3 phases with partial sums parked in LDS (N = 36: an odd number of
    # quads, so the last item of the two-quad form holds one quad only)
    s = SCHEMES[name]
    x, qw, qs, b = _linear_case(s, m, n, k, 5 * m + n + k, bias=True)
    gq._lib.set_option("gemv_variant", 7)
    gq._lib.set_option("gemv_waves", waves)
    gq._lib.set_option("quad_pairs", qp)
    try:
        y = ops.linear(dev(x), dev(qw), dev(qs), s.bits, s.group_size, dev(b))
    finally:
        gq._lib.set_option("gemv_variant", -1)
        gq._lib.set_option("gemv_waves", -1)
        gq._lib.set_option("quad_pairs", -1)
    assert_linear_ok(y, o.linear_fp32(x, qw, qs, s, b), x, k, f"quad-row phases {name} {m}x{n}x{k} waves={waves} qp={qp}")


@pytest.mark.parametrize("m", [9, 12, 16])
@pytest.mark.parametrize("n,k", [(520, 4000), (64, 14320), (132, 80)])
def test_q3_nine_to_sixteen_rows_as_concurrent_passes(m, n, k):
    # q3f16_1 has no 16x16x32 kernel: 9..16 rows run as two 8-row passes (four 4-row passes when
    # 8 rows of x do not fit LDS) of the quad-row kernel, on the default path
    s = SCHEMES["q3f16_1"]
    x, qw, qs, b = _linear_case(s, m, n, k, 7 * m + n + k, bias=True)
    res = np.random.default_rng(m + n).standard_normal((m, n)).astype(np.float16)
    y = ops.linear(dev(x), dev(qw), dev(qs), 3, 40, dev(b), residual=dev(res))
    assert_linear_ok(y, o.linear_fp32(x, qw, qs, s, b) + res.astype(np.float64), x, k, f"q3 {m}x{n}x{k}")


@pytest.mark.parametrize("m,n,k", [(8, 64, 14336), (7, 520, 1024)])
def test_quadrow_kernel_two_passes(m, n, k):
    # 5..8 rows as two concurrent 4-row passes (the default when 8 rows of x do not fit LDS)
    s = SCHEMES["q4f16_1"]
    x, qw, qs, b = _linear_case(s, m, n, k, 3 * m + n + k, bias=True)
    gq._lib.set_option("gemv_variant", 8)
    try:
        y = ops.linear(dev(x), dev(qw), dev(qs), 4, 32, dev(b))
    finally:
        gq._lib.set_option("gemv_variant", -1)
    assert_linear_ok(y, o.linear_fp32(x, qw, qs, s, b), x, k, f"quad-row two passes {m}x{n}x{k}")


def test_quadrow_kernel_declines_odd_shapes():
    # N not a multiple of 4: the forced kernel declines and the 16x16x32 kernel answers
    s = SCHEMES["q4f16_1"]
    x, qw, qs, b = _linear_case(s, 5, 2101, 256, 9, bias=True)
    gq._lib.set_option("gemv_variant", 6)
    try:
        y = ops.linear(dev(x), dev(qw), dev(qs), 4, 32, dev(b))
    finally:
        gq._lib.set_option("gemv_variant", -1)
    assert_linear_ok(y, o.linear_fp32(x, qw, qs, s, b), x, 256, "quad-row declined")


@pytest.mark.parametrize("n,k", [(512, 4096), (1000, 1024), (260, 8192)])
def test_two_rows_of_q4_take_the_register_fewrow_kernel(n, k):
    """Two activation rows of a q4f16_1 linear run on the few-row kernel with x in registers (it is ahead of the two-row
    GEMV on every decode shape); a long K, which that kernel declines, and q3f16_1 keep their kernels.  Plain, with bias and
    residual, float32 output, and the fused gate/up form against the two steps."""
    s = SCHEMES["q4f16_1"]
    x, qw, qs, b = _linear_case(s, 2, n, k, 5 * n + k, bias=True)
    res = np.random.default_rng(n).standard_normal((2, n)).astype(np.float16)
    y = ops.linear(dev(x), dev(qw), dev(qs), 4, 32)
    assert gq._lib.last_kernel().startswith("gq::quadreg_kernel<4,1,"), gq._lib.last_kernel()
    yb = ops.linear(dev(x), dev(qw), dev(qs), 4, 32, dev(b), residual=dev(res))
    assert gq._lib.last_kernel().startswith("gq::quadreg_kernel<4,1,"), gq._lib.last_kernel()
    y32 = ops.linear(dev(x), dev(qw), dev(qs), 4, 32, None, torch.float32)
    ref = o.linear_fp32(x, qw, qs, s)
    assert_linear_ok(y, ref, x, k, f"two rows {n}x{k}")
    assert_linear_ok(y32, ref, x, k, f"two rows f32 {n}x{k}")
    assert_linear_ok(yb, o.linear_fp32(x, qw, qs, s, b) + res.astype(np.float64), x, k, f"two rows bias+residual {n}x{k}")
    fused = ops.linear_silu_mul(dev(x), dev(qw), dev(qs), 4, 32)
    assert gq._lib.last_kernel().startswith("gq::quadreg_kernel<4,1,"), gq._lib.last_kernel()
    assert torch.equal(fused, ops.silu_mul(y))
    s3 = SCHEMES["q3f16_1"]
    k3 = k // 40 * 40
    x3, qw3, qs3, _ = _linear_case(s3, 2, n, k3, n + k3, bias=False)
    y3 = ops.linear(dev(x3), dev(qw3), dev(qs3), 3, 40)
    assert "quadreg" not in gq._lib.last_kernel(), gq._lib.last_kernel()
    assert_linear_ok(y3, o.linear_fp32(x3, qw3, qs3, s3), x3, k3, f"two rows q3 {n}x{k3}")


@pytest.mark.parametrize("name", ["q4f16_1", "q3f16_1"])
def test_grouped_many_experts_more_than_128_rows(name):
    """Many experts with a few rows each: the few-row kernel serves up to seven rows per expert whatever the total (200 rows
    over 40 experts here: segments of 0 to 19 rows, i.e. up to three passes), where a cap of 128 rows once sent such calls to
    the GEMM's mostly empty tiles.  Against the oracle, int32 and int64 indptr."""
    s = SCHEMES[name]
    rng = np.random.default_rng(91)
    ne, n, k = 40, 132, 640 if s.bits == 4 else 640
    w = (rng.standard_normal((ne, n, k)) * 0.02).astype(np.float16)
    qw, qs = o.quantize(w, s)
    sizes = rng.integers(0, 9, ne)
    sizes[7] = 19
    sizes[-1] += 200 - sizes.sum()
    assert sizes.min() >= 0 and sizes.sum() == 200
    ip = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int32)
    x = rng.standard_normal((200, k)).astype(np.float16)
    out = ops.moe_group_gemm(dev(x), dev(qw), dev(qs), dev(ip), s.bits, s.group_size)
    assert gq._lib.last_kernel().startswith("gq::quad_kernel<"), gq._lib.last_kernel()
    out64 = ops.moe_group_gemm(dev(x), dev(qw), dev(qs), dev(ip.astype(np.int64)), s.bits, s.group_size)
    ref = o.dequantize_group_gemm_fp32(x, qw, qs, ip, s)
    assert_linear_ok(out, ref, x, k, f"grouped, 40 experts, 200 rows {name}")
    assert torch.equal(out, out64)


@pytest.mark.parametrize("name", ["q4f16_1", "q3f16_1"])
@pytest.mark.parametrize("qp", [1, 2])
@pytest.mark.parametrize("k", [1024, 14336])
def test_quadrow_kernel_grouped(name, qp, k):
    s = SCHEMES[name]
    if s.bits == 3:
        k = k // 40 * 40
    rng = np.random.default_rng(62)
    ne, n = 5, 200
    w = (rng.standard_normal((ne, n, k)) * 0.02).astype(np.float16)
    qw, qs = o.quantize(w, s)
    ip = np.array([0, 2, 2, 21, 22, 40], np.int32)  # an empty expert and one with 19 rows (3 passes)
    x = rng.standard_normal((40, k)).astype(np.float16)
    gq._lib.set_option("gemv_variant", 6)
    gq._lib.set_option("quad_pairs", qp)
    try:
        out = ops.moe_group_gemm(dev(x), dev(qw), dev(qs), dev(ip), s.bits, s.group_size)
        out64 = ops.moe_group_gemm(dev(x), dev(qw), dev(qs), dev(ip.astype(np.int64)), s.bits, s.group_size)
    finally:
        gq._lib.set_option("gemv_variant", -1)
        gq._lib.set_option("quad_pairs", -1)
    ref = o.dequantize_group_gemm_fp32(x, qw, qs, ip, s)
    assert_linear_ok(out, ref, x, k, f"grouped quad-row {name} qp={qp} k={k}")
    assert_linear_ok(out64, ref, x, k, f"grouped quad-row k={k} int64 indptr")


@pytest.mark.parametrize("variant", [3, 4, 6, 7, 9])  # plain 128/256 tiles, pipelined 128/256 tiles, pipelined 128x256
@pytest.mark.parametrize("fast_loop", [-1, 0])  # the K loop without zero-selects where K allows it / the general loop always
@pytest.mark.parametrize("m,n,k", [(300, 512, 1024), (17, 260, 4096), (513, 300, 192), (130, 100, 128), (257, 129, 64)])
def test_gemm_kernel_variants(variant, fast_loop, m, n, k):
    # ragged rows and columns on every tile, K of whole K tiles (both loops apply) and the general loop forced
    s = SCHEMES["q4f16_1"]
    x, qw, qs, b = _linear_case(s, m, n, k, variant * 1000 + m + n + k, bias=True)
    gq._lib.set_option("gemm_variant", variant)
    gq._lib.set_option("gemm_fast_loop", fast_loop)
    try:
        y = ops.linear(dev(x), dev(qw), dev(qs), 4, 32, dev(b))
    finally:
        gq._lib.set_option("gemm_variant", -1)
        gq._lib.set_option("gemm_fast_loop", -1)
    assert_linear_ok(y, o.linear_fp32(x, qw, qs, s, b), x, k, f"gemm variant {variant} fast_loop {fast_loop} {m}x{n}x{k}")


@pytest.mark.parametrize("name", ["q4f16_1", "q3f16_1"])
@pytest.mark.parametrize("m", [17, 64, 100, 300, 1100])
def test_gemm_fast_and_general_loop_agree_bit_for_bit(name, m):
    """The K loop without zero-selects (K of whole K tiles) against the general loop on the same launch shape: identical
    bits, on ragged rows and columns, with bias + residual, float32 output, the folded activation and split K."""
    s = SCHEMES[name]
    n, k = 1060, 16 * s.group_size
    x, qw, qs, b = _linear_case(s, m, n, k, 31 * m + n, bias=True)
    res = np.random.default_rng(m).standard_normal((m, n)).astype(np.float16)
    outs = []
    for fast_loop in (-1, 0):
        gq._lib.set_option("gemm_fast_loop", fast_loop)
        try:
            outs.append((ops.linear(dev(x), dev(qw), dev(qs), s.bits, s.group_size, dev(b), residual=dev(res)),
                         ops.linear(dev(x), dev(qw), dev(qs), s.bits, s.group_size, None, torch.float32),
                         ops.linear_silu_mul(dev(x), dev(qw), dev(qs), s.bits, s.group_size)))
        finally:
            gq._lib.set_option("gemm_fast_loop", -1)
    for a, c in zip(*outs):
        assert torch.equal(a, c)
    assert_linear_ok(outs[0][1], o.linear_fp32(x, qw, qs, s), x, k, f"fast loop {name} m={m}")


@pytest.mark.parametrize("m", [17, 100, 300, 1100])
@pytest.mark.parametrize("k", [256, 768, 1280, 11008])
def test_gemm_q4_scale_blocks_odd_and_even_trip_counts(m, k):
    """q4f16_1, K loop without zero-selects: scales are read 16 bytes (four K tiles) at a time into two register blocks that
    swap roles from trip to trip, two trips per loop round and a peeled last one.  K of one block (the peeled trip alone),
    three, five and 43 blocks (odd counts), against the general loop bit for bit and against the oracle; the same launch
    with a scale tensor that is not 16-byte aligned must take the per-tile scale loads and give the same bits."""
    s = SCHEMES["q4f16_1"]
    n = 520 if k <= 1280 else 300
    x, qw, qs, b = _linear_case(s, m, n, k, 13 * m + k, bias=True)
    outs = []
    for fast_loop in (-1, 0):
        gq._lib.set_option("gemm_fast_loop", fast_loop)
        try:
            outs.append((ops.linear(dev(x), dev(qw), dev(qs), 4, 32, dev(b)),
                         ops.linear(dev(x), dev(qw), dev(qs), 4, 32, None, torch.float32),
                         ops.linear_silu_mul(dev(x), dev(qw), dev(qs), 4, 32)))
            if fast_loop == -1 and m > 16:
                assert gq._lib.last_kernel().startswith("gq::gemm_pipe_kernel<4,") and \
                    gq._lib.last_kernel().endswith("true>"), gq._lib.last_kernel()
        finally:
            gq._lib.set_option("gemm_fast_loop", -1)
    for a, c in zip(*outs):
        assert torch.equal(a, c)
    assert_linear_ok(outs[0][1], o.linear_fp32(x, qw, qs, s), x, k, f"q4 scale blocks m={m} k={k}")
    # scales at an address that is 2 bytes past a 16-byte boundary
    flat = torch.zeros(qs.size + 8, dtype=torch.float16, device="cuda")
    flat[1:1 + qs.size] = dev(qs).reshape(-1)
    qs_odd = flat[1:1 + qs.size].view(qs.shape)
    assert qs_odd.data_ptr() % 16 == 2
    y_odd = ops.linear(dev(x), dev(qw), qs_odd, 4, 32, None, torch.float32)
    assert gq._lib.last_kernel().endswith("false>"), gq._lib.last_kernel()
    assert torch.equal(y_odd, outs[0][1])


def test_grouped_gemm_q4_scale_blocks_on_ragged_segments():
    """The grouped tiles with skipped row blocks and the deeper weight ring (four K tiles per trip), K of three scale blocks
    (a loop round and the peeled trip): against the general loop bit for bit, and the oracle."""
    s = SCHEMES["q4f16_1"]
    rng = np.random.default_rng(77)
    ne, n, k = 4, 300, 768
    w = (rng.standard_normal((ne, n, k)) * 0.02).astype(np.float16)
    qw, qs = o.quantize(w, s)
    ip = np.array([0, 130, 131, 400, 520], np.int32)  # 130, 1, 269 and 120 rows
    x = rng.standard_normal((520, k)).astype(np.float16)
    outs = []
    for fast_loop in (-1, 0):
        gq._lib.set_option("gemm_fast_loop", fast_loop)
        try:
            outs.append(ops.moe_group_gemm(dev(x), dev(qw), dev(qs), dev(ip), 4, 32))
            name = gq._lib.last_kernel()
            assert name.startswith("gq::gemm_pipe_kernel<4,256,") and name.endswith("true>" if fast_loop else "false>"), name
        finally:
            gq._lib.set_option("gemm_fast_loop", -1)
    assert torch.equal(outs[0], outs[1])
    assert_linear_ok(outs[0], o.dequantize_group_gemm_fp32(x, qw, qs, ip, s), x, k, "grouped scale blocks")


@pytest.mark.parametrize("m", [17, 100, 300, 1100, 2048])
@pytest.mark.parametrize("k", [4096, 1000, 11008, 200, 88])
def test_gemm_q3_fast_loop_with_a_k_tail(m, k):
    """q3f16_1: K is rarely whole 80-wide K tiles (4096 = 51.2 of them), so its K loop without zero-selects masks the
    activation chunks at k >= K and zeroes the scale of a group past the last.  Against the general loop: identical bits,
    also when the values a masked chunk reads (the head of the next row of x) are NaN; against the oracle on the rest."""
    s = SCHEMES["q3f16_1"]
    n = 1060 if k <= 4096 else 300
    x, qw, qs, b = _linear_case(s, m, n, k, 7 * m + k, bias=True)
    x = x.copy()
    bad = min(5, m - 1)
    x[bad, : min(64, k)] = np.nan  # what the last K tile of row bad - 1 reads past its end
    outs = []
    for fast_loop in (-1, 0):
        gq._lib.set_option("gemm_fast_loop", fast_loop)
        try:
            outs.append((ops.linear(dev(x), dev(qw), dev(qs), s.bits, s.group_size, dev(b)),
                         ops.linear(dev(x), dev(qw), dev(qs), s.bits, s.group_size, None, torch.float32),
                         ops.linear_silu_mul(dev(x), dev(qw), dev(qs), s.bits, s.group_size)))
            if fast_loop == -1 and m == 2048 and k == 4096:  # (the shape of the benchmark's q3f16_1 prefill)
                assert gq._lib.last_kernel().startswith("gq::gemm_pipe_kernel<3,") and \
                    gq._lib.last_kernel().endswith("true>"), gq._lib.last_kernel()
        finally:
            gq._lib.set_option("gemm_fast_loop", -1)
    keep = np.arange(m) != bad
    for a, c in zip(*outs):
        a, c = a.cpu().numpy(), c.cpu().numpy()
        assert np.isnan(a[bad]).all() and np.isnan(c[bad]).all()
        assert np.array_equal(a[keep], c[keep])
    y32 = outs[0][1].cpu().numpy()[keep]
    assert np.isfinite(y32).all()
    assert_linear_ok(torch.from_numpy(y32), o.linear_fp32(x[keep], qw, qs, s), x[keep], k, f"q3 fast loop k tail m={m} k={k}")


@pytest.mark.parametrize("name", ["q4f16_1", "q3f16_1"])
@pytest.mark.parametrize("m", [17, 32, 33, 64, 100, 129, 256, 300, 700, 1024])
@pytest.mark.parametrize("n,k", [(520, 4096), (130, 14336), (384, 1000)])
def test_few_row_gemm_split_k(name, m, n, k):
    # 17..1024 rows: tile height follows the rows and K is cut across workgroups (as far as the partial
    # sums stay cheaper than the weights), partial sums go through the workspace and a reduction
    # kernel (bias and the output type are applied there)
    s = SCHEMES[name]
    x, qw, qs, b = _linear_case(s, m, n, k, 13 * m + n + k, bias=True)
    ws = gq._lib.lib().mi355gq_linear_workspace_bytes(m, n, k, s.bits, s.group_size)
    y = ops.linear(dev(x), dev(qw), dev(qs), s.bits, s.group_size, dev(b))
    y32 = ops.linear(dev(x), dev(qw), dev(qs), s.bits, s.group_size, None, torch.float32)
    ref = o.linear_fp32(x, qw, qs, s, b)
    assert_linear_ok(y, ref, x, k, f"few-row gemm {name} {m}x{n}x{k} (workspace {ws} B)")
    assert_linear_ok(y32, ref - b.astype(np.float64), x, k, f"few-row gemm {name} fp32 out")
    if k >= 4096 and k // (7 * m) >= 2:
        assert ws > 0 and ws % (m * n * 4) == 0  # these shapes do split


@pytest.mark.parametrize("m", [17, 32, 33, 64, 65, 96, 128])
@pytest.mark.parametrize("n,k", [(520, 4096), (130, 14336), (384, 1000), (257, 4104)])
def test_few_row_gemm_q4_with_residual(m, n, k):
    s = SCHEMES["q4f16_1"]
    x, qw, qs, b = _linear_case(s, m, n, k, 17 * m + n + k, bias=True)
    res = np.random.default_rng(m + k).standard_normal((m, n)).astype(np.float16)
    y = ops.linear(dev(x), dev(qw), dev(qs), 4, 32, dev(b), residual=dev(res))
    y32 = ops.linear(dev(x), dev(qw), dev(qs), 4, 32, None, torch.float32)
    ref = o.linear_fp32(x, qw, qs, s, b)
    assert_linear_ok(y, ref + res.astype(np.float64), x, k, f"few-row gemm {m}x{n}x{k}")
    assert_linear_ok(y32, ref - b.astype(np.float64), x, k, f"few-row gemm fp32 out {m}x{n}x{k}")


@pytest.mark.parametrize("want", [64, 4096])  # few / as many splits as K allows
def test_few_row_gemm_split_counts_and_missing_workspace(want):
    s = SCHEMES["q4f16_1"]
    m, n, k = 40, 260, 8192
    x, qw, qs, b = _linear_case(s, m, n, k, 99, bias=True)
    ref = o.linear_fp32(x, qw, qs, s, b)
    gq._lib.set_option("gemm_split_k", want)
    try:
        y = ops.linear(dev(x), dev(qw), dev(qs), 4, 32, dev(b))
        ws = gq._lib.lib().mi355gq_linear_workspace_bytes(m, n, k, 4, 32)
    finally:
        gq._lib.set_option("gemm_split_k", -1)
    assert ws > 0
    assert_linear_ok(y, ref, x, k, f"few-row gemm, {want} workgroups wanted")
    # no workspace handed over: same tiles, no split, same answer
    xd, qwd, qsd, bd = dev(x), dev(qw), dev(qs), dev(b)
    out = torch.empty((m, n), dtype=torch.float16, device=xd.device)
    gq._lib.call("mi355gq_linear", xd.data_ptr(), qwd.data_ptr(), qsd.data_ptr(), bd.data_ptr(), m, n, k, 4, 32,
                 gq._lib.F16, out.data_ptr(), None, 0, torch.cuda.current_stream().cuda_stream)
    assert_linear_ok(out, ref, x, k, "few-row gemm without workspace")


@pytest.mark.parametrize("m,n,k", [(300, 512, 1000), (129, 260, 4000), (513, 300, 200)])
def test_gemm_q3_wide_tile(m, n, k):
    # q3f16_1 on the 128 x 256 tile (a round of its activation loads covers only part of the threads)
    s = SCHEMES["q3f16_1"]
    x, qw, qs, b = _linear_case(s, m, n, k, 9000 + m + n + k, bias=True)
    gq._lib.set_option("gemm_variant", 9)
    try:
        y = ops.linear(dev(x), dev(qw), dev(qs), 3, 40, dev(b))
    finally:
        gq._lib.set_option("gemm_variant", -1)
    assert_linear_ok(y, o.linear_fp32(x, qw, qs, s, b), x, k, f"q3 128x256 tile {m}x{n}x{k}")


def test_gemm_k_not_multiple_of_8_takes_fallback():
    # K = 100: rows of x are not 16-byte aligned, the pipelined kernel declines and the plain one runs
    for name in ("q4f16_1", "q3f16_1"):
        s = SCHEMES[name]
        x, qw, qs, _ = _linear_case(s, 40, 96, 100, 5)
        y = ops.linear(dev(x), dev(qw), dev(qs), s.bits, s.group_size)
        assert_linear_ok(y, o.linear_fp32(x, qw, qs, s), x, 100, f"gemm K=100 {name}")


def test_gemv_config1_golden_shape_fp32_out_and_lm_head():
    # config 1: N = K = 4096, weights N(0, 0.02) seed 0, activation N(0, 1); also the fp32-output
    # path used by GroupQuantizeEmbedding.lm_head_forward
    s = SCHEMES["q4f16_1"]
    rng = np.random.default_rng(0)
    w = (rng.standard_normal((4096, 4096)) * 0.02).astype(np.float16)
    x = np.random.default_rng(1).standard_normal((1, 4096)).astype(np.float16)
    qw_d, qs_d = ops.quantize(dev(w), 4, 32)
    qw, qs = host_u32(qw_d), qs_d.cpu().numpy()
    ref = o.linear_fp32(x, qw, qs, s)
    y = ops.linear(dev(x), qw_d, qs_d, 4, 32)
    assert_linear_ok(y, ref, x, 4096, "config 1")
    emb = gq.GroupQuantizeEmbedding(4096, 4096, gq.QUANTIZATION["q4f16_1"], device=DEV)
    emb.q_weight.data, emb.q_scale.data = qw_d, qs_d
    logits = emb.lm_head_forward(dev(x))
    assert logits.dtype == torch.float32
    err = np.abs(logits.cpu().numpy().astype(np.float64) - ref).max()
    assert err <= 2e-3, err  # fp32 output: only the accumulation order differs


def test_gemv_linearity_and_zero_input():
    # y(a*x1 + x2) = a*y(x1) + y(x2) up to fp16 rounding; zero activations give exactly bias
    s = SCHEMES["q4f16_1"]
    x, qw, qs, b = _linear_case(s, 2, 512, 1024, 31, bias=True)
    qw_d, qs_d, b_d = dev(qw), dev(qs), dev(b)
    y0 = ops.linear(torch.zeros((1, 1024), dtype=torch.float16, device=DEV), qw_d, qs_d, 4, 32, b_d)
    assert (host_f16_bits(y0[0]) == b.view(np.uint16)).all() or bool((y0[0].cpu() == torch.from_numpy(b)).all())
    x3 = (2.0 * x[0].astype(np.float32) + x[1].astype(np.float32)).astype(np.float16)[None]
    y = ops.linear(dev(np.concatenate([x, x3])), qw_d, qs_d, 4, 32, None, torch.float32).cpu().numpy()
    lin = 2.0 * y[0] + y[1]
    # x3 was rounded to fp16: bound the difference by that rounding through |W| row sums
    wabs = np.abs(o.dequantize(qw, qs, s, 1024).astype(np.float64)).sum(1)
    assert (np.abs(y[2] - lin) <= 2.0**-10 * np.abs(x3).max() * wabs + 1e-3).all()


@pytest.mark.parametrize("name", ["q4f16_1", "q3f16_1"])
@pytest.mark.parametrize("m,n,k", [(9, 64, 128), (128, 256, 512), (200, 130, 1000), (257, 384, 4096), (16, 100, 72)])
def test_gemm_shapes(name, m, n, k):
    s = SCHEMES[name]
    x, qw, qs, b = _linear_case(s, m, n, k, m + n + k, bias=True)
    y = ops.linear(dev(x), dev(qw), dev(qs), s.bits, s.group_size, dev(b))
    assert_linear_ok(y, o.linear_fp32(x, qw, qs, s, b), x, k, f"gemm {name} {m}x{n}x{k}")


def test_gemm_prefill_shape_and_gemv_agreement():
    # M = 256 on the o_proj shape; the first 8 rows must agree with the GEMV path on the same data
    s = SCHEMES["q4f16_1"]
    x, qw, qs, _ = _linear_case(s, 256, 4096, 4096, 2024)
    qw_d, qs_d, x_d = dev(qw), dev(qs), dev(x)
    y = ops.linear(x_d, qw_d, qs_d, 4, 32)
    assert_linear_ok(y, o.linear_fp32(x, qw, qs, s), x, 4096, "gemm 256x4096x4096")
    y8 = ops.linear(x_d[:8].contiguous(), qw_d, qs_d, 4, 32)
    assert float((y[:8].float() - y8.float()).abs().max()) <= 2 * o.linear_tolerance(x[:8], 4096)
    y32 = ops.linear(x_d, qw_d, qs_d, 4, 32, None, torch.float32)
    assert y32.dtype == torch.float32
    assert_linear_ok(y32, o.linear_fp32(x, qw, qs, s), x, 4096, "gemm fp32 out")


# (float16 models at full size, every row regime against the oracle: tests/test_gpu_baseline_configs.py)


@pytest.mark.parametrize("n,k", [(28672, 4096), (4096, 14336)])
def test_every_row_regime_agrees_at_full_size_bfloat16(n, k):
    """The same for a q4bf16_1 model (register GEMV, quad-row kernel, few-row and large GEMM tiles in bf16).
    Tolerance: the matmul one plus the rounding of the output to bfloat16 (2^-9 per element)."""
    g = torch.Generator(device=DEV).manual_seed(n + k + 1)
    w = (torch.randn((n, k), generator=g, device=DEV) * 0.02).bfloat16()
    qw, qs = ops.quantize(w, 4, 32)
    del w
    wd = ops.dequantize(qw, qs, k, 4, 32).double()
    x = torch.randn((2048, k), generator=g, device=DEV).bfloat16()
    ref = x[:3].double() @ wd.t()
    del wd
    tol = 1e-2 * float(x[:3].float().abs().max()) * np.sqrt(k) / 64 + 2.0 ** -8 * float(ref.abs().max())
    for m in (1, 2, 3, 4, 8, 9, 16, 32, 64, 128, 256, 300, 1024, 2048):
        y = ops.linear(x[:m].contiguous(), qw, qs, 4, 32)
        assert y.dtype == torch.bfloat16
        rows = min(m, 3)
        err = (y[:rows].double() - ref[:rows]).abs().max().item()
        rel = ((y[:rows].double() - ref[:rows]).norm() / ref[:rows].norm()).item()
        assert err <= tol and rel <= 3e-3, f"bf16 {n}x{k} M={m}: max err {err:.3e} (tol {tol:.3e}), rel-L2 {rel:.2e}"


def test_linear_module_matches_reference_interface():
    cfg = gq.QUANTIZATION["q4f16_1"]
    lin = gq.GroupQuantizeLinear(256, 96, cfg, bias=True, device=DEV)
    rng = np.random.default_rng(3)
    w = (rng.standard_normal((96, 256)) * 0.05).astype(np.float16)
    qw, qs = cfg.quantize_weight(dev(w))
    lin.q_weight.data, lin.q_scale.data = qw, qs
    b = rng.standard_normal(96).astype(np.float16)
    lin.bias.data = dev(b)
    x = rng.standard_normal((2, 3, 256)).astype(np.float16)
    y = lin(dev(x))
    assert tuple(y.shape) == (2, 3, 96)
    ref = o.linear_fp32(x.reshape(6, 256), host_u32(qw), qs.cpu().numpy(), SCHEMES["q4f16_1"], b)
    assert_linear_ok(y.reshape(6, 96), ref, x, 256, "module")
    assert (host_f16_bits(cfg.dequantize_weight(qw, qs, 256)) ==
            o.dequantize(host_u32(qw), qs.cpu().numpy(), SCHEMES["q4f16_1"], 256).view(np.uint16)).all()


@pytest.mark.parametrize("kn_name,nk_name", [("q4f16_0", "q4f16_1"), ("q3f16_0", "q3f16_1")])
def test_kn_layout_is_the_transposed_nk_tensors(kn_name, nk_name):
    # q4f16_0 / q3f16_0 (reference quantization.py:47-79, transpose at group_quantization.py:299-305)
    kn, nk = gq.QUANTIZATION[kn_name], gq.QUANTIZATION[nk_name]
    s = SCHEMES[nk_name]
    k = 8 * s.group_size
    rng = np.random.default_rng(21)
    w = (rng.standard_normal((96, k)) * 0.05).astype(np.float16)
    qw_ref, qs_ref = o.quantize(w, s)
    qw, qs = kn.quantize_weight(dev(w), output_transpose=True)
    assert tuple(qw.shape) == (qw_ref.shape[1], 96) and tuple(qs.shape) == (qs_ref.shape[1], 96)
    assert np.array_equal(host_u32(qw), qw_ref.T) and np.array_equal(host_f16_bits(qs), qs_ref.view(np.uint16).T)
    lin_kn = gq.GroupQuantizeLinear(k, 96, kn, bias=False, device=DEV)
    lin_nk = gq.GroupQuantizeLinear(k, 96, nk, bias=False, device=DEV)
    lin_kn.q_weight.data, lin_kn.q_scale.data = qw, qs
    lin_nk.q_weight.data, lin_nk.q_scale.data = dev(qw_ref), dev(qs_ref)
    for m in (1, 5, 40):
        xh = rng.standard_normal((m, k)).astype(np.float16)
        if m > 8:  # an NK copy and the NK kernels: the same bits
            assert torch.equal(lin_kn(dev(xh)), lin_nk(dev(xh)))
        else:  # decode batches stream the KN tensors as stored (another order of summation)
            assert_linear_ok(lin_kn(dev(xh)), o.linear_fp32(xh, qw_ref, qs_ref, s), xh, k, f"KN module M={m}")
    # new parameters are picked up (the transposed copy is remade)
    w2 = (rng.standard_normal((96, k)) * 0.05).astype(np.float16)
    qw2, qs2 = kn.quantize_weight(dev(w2), output_transpose=True)
    lin_kn.load_state_dict({"q_weight": qw2, "q_scale": qs2})
    x = rng.standard_normal((3, k)).astype(np.float16)
    q2w, q2s = o.quantize(w2, s)
    assert_linear_ok(lin_kn(dev(x)), o.linear_fp32(x, q2w, q2s, s), x, k, "KN after update")


@pytest.mark.parametrize("name", ["q4f16_1", "q3f16_1"])
@pytest.mark.parametrize("n,k", [(96, 256), (4096, 4096), (130, 1000), (28672, 4096), (7, 72)])
def test_kn_entry_points(name, n, k):
    """The C ABI on KN-layout tensors (q_weight [nw, N], q_scale [ng, N], as quantize_weight(output_transpose=True)
    stores them, group_quantization.py:299-305): both transposes bit for bit, the dequantisation along axis 0 bit for
    bit (the oracle's NK dequantisation, transposed), and the linear against the oracle at decode batches (the GEMV that
    streams the stored tensors, N % 4 == 0) and beyond (an NK copy in the workspace), with bias and float32 output."""
    s = SCHEMES[name]
    if s.bits == 3:
        k = {256: 240, 4096: 4096, 1000: 1000, 72: 80}[k]
    rng = np.random.default_rng(seed_of("kn", name, n, k))
    rows = min(n, 520)  # (the oracle's float64 matmul on a sample of the output columns of the large shapes)
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float16)
    qw, qs = o.quantize(w, s)
    qw_kn, qs_kn = dev(np.ascontiguousarray(qw.T)), dev(np.ascontiguousarray(qs.T))
    nk_w, nk_s = ops.kn_to_nk(qw_kn, qs_kn, k, s.bits, s.group_size)
    assert np.array_equal(host_u32(nk_w), qw) and np.array_equal(host_f16_bits(nk_s), qs.view(np.uint16))
    back_w, back_s = ops.nk_to_kn(nk_w, nk_s, k, s.bits, s.group_size)
    assert torch.equal(back_w, qw_kn) and torch.equal(back_s, qs_kn)
    cols = np.unique(np.concatenate([[0, 1, n // 2, n - 1], rng.integers(0, n, rows)]))
    d = ops.dequantize_kn(qw_kn, qs_kn, k, s.bits, s.group_size)
    assert tuple(d.shape) == (k, n)
    want = o.dequantize(qw[cols], qs[cols], s, k)
    assert np.array_equal(host_f16_bits(d[:, torch.from_numpy(cols).to(DEV)]), want.T.view(np.uint16))
    b = rng.standard_normal(n).astype(np.float16)
    for m in (1, 2, 4, 8, 19):
        x = rng.standard_normal((m, k)).astype(np.float16)
        ref = o.linear_fp32(x, qw[cols], qs[cols], s)
        y = ops.linear_kn(dev(x), qw_kn, qs_kn, s.bits, s.group_size)
        kern = gq._lib.last_kernel()
        # 16-byte rows of x: the 4x4x4 matrix-instruction form; else the GEMV (and for one row of q3 over a large matrix)
        quad = m <= 8 and n % 4 == 0 and k % 8 == 0 and not (s.bits == 3 and m == 1 and n * k >= 40 << 20)
        assert kern.startswith("gq::kn_quad_kernel") == quad, (kern, m, n)
        assert kern.startswith("gq::gemv_kn_kernel") == (m <= 8 and n % 4 == 0 and not quad), (kern, m, n)
        if quad:  # ... against the GEMV on the same tensors (forced), and also for a single row (forced)
            gq._lib.set_option("gemv_variant", 0)
            try:
                y_gemv = ops.linear_kn(dev(x), qw_kn, qs_kn, s.bits, s.group_size)
                assert gq._lib.last_kernel().startswith("gq::gemv_kn_kernel")
            finally:
                gq._lib.set_option("gemv_variant", -1)
            assert (y.float() - y_gemv.float()).abs().max().item() <= 2e-2 * max(1.0, y_gemv.float().abs().max().item())
        assert_linear_ok(y[:, torch.from_numpy(cols).to(DEV)], ref, x, k, f"linear_kn {name} {m}x{n}x{k} [{kern}]")
        y32 = ops.linear_kn(dev(x), qw_kn, qs_kn, s.bits, s.group_size, dev(b), torch.float32)
        assert_linear_ok(y32[:, torch.from_numpy(cols).to(DEV)], ref + b[cols].astype(np.float64), x, k,
                         f"linear_kn bias fp32 {name} {m}x{n}x{k}")


def test_linear_kn_workspace_contract():
    """Without a workspace the decode GEMV runs unsplit (same tolerance); the other shapes need room for the NK copy
    and say so (MI355GQ_ERR_WORKSPACE) before anything is launched."""
    lib = gq._lib
    s = SCHEMES["q4f16_1"]
    rng = np.random.default_rng(77)
    n, k = 512, 2048
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float16)
    qw, qs = o.quantize(w, s)
    qw_kn, qs_kn = dev(np.ascontiguousarray(qw.T)), dev(np.ascontiguousarray(qs.T))
    x = rng.standard_normal((3, k)).astype(np.float16)
    xd = dev(x)
    y = torch.empty((3, n), dtype=torch.float16, device=DEV)
    assert lib.lib().mi355gq_linear_kn_workspace_bytes(3, n, k, 4, 32) > 0  # (few column blocks: K is split)
    lib.call("mi355gq_linear_kn", xd.data_ptr(), qw_kn.data_ptr(), qs_kn.data_ptr(), None, 3, n, k, 4, 32, lib.F16,
             y.data_ptr(), None, 0, torch.cuda.current_stream().cuda_stream)
    assert gq._lib.last_kernel().endswith("slices=1")
    assert_linear_ok(y, o.linear_fp32(x, qw, qs, s), x, k, "linear_kn without a workspace")
    x40 = dev(rng.standard_normal((40, k)).astype(np.float16))
    y40 = torch.empty((40, n), dtype=torch.float16, device=DEV)
    with pytest.raises(lib.Mi355gqError) as ei:
        lib.call("mi355gq_linear_kn", x40.data_ptr(), qw_kn.data_ptr(), qs_kn.data_ptr(), None, 40, n, k, 4, 32, lib.F16,
                 y40.data_ptr(), None, 0, torch.cuda.current_stream().cuda_stream)
    assert ei.value.code == lib.ERR_WORKSPACE


# ------------------------------------------------------------------ MoE


def test_routing_golden_bit_exact(golden):
    for name in ("routing_t7_e8_k2", "routing_t33_e6_k3", "routing_t1_e8_k2"):
        z = golden(name)
        t, ne = z["logits"].shape
        k = z["ids"].shape[1]
        w, ids = ops.gating_softmax_topk(dev(z["logits"]), k)
        assert (ids.cpu().numpy() == z["ids"]).all(), name
        # softmax weights: exp differs by an ulp between libms; one fp16 ulp allowed
        dw = np.abs(w.cpu().numpy().astype(np.float32) - z["weights"].astype(np.float32))
        assert (dw <= 2.0**-11).all(), dw.max()
        cs = ops.moe_cumsum(ids, ne)
        assert (cs.cpu().numpy() == z["cumsum"]).all()
        rev, tok = ops.get_indices(cs, ids)
        assert (rev.cpu().numpy() == z["reverse_indices"]).all() and (tok.cpu().numpy() == z["token_indices"]).all()
        assert (ops.get_indptr(cs, ne, t, False).cpu().numpy() == z["indptr"]).all()
        inc = ops.get_indptr(cs, ne, t, True, torch.int64)
        assert inc.dtype == torch.int64 and (inc.cpu().numpy() == z["indptr_inclusive"]).all()


def test_moe_cumsum_docstring_example_on_gpu():
    ids = torch.tensor([[0, 1], [1, 2], [3, 4], [2, 5]], dtype=torch.int32, device=DEV)
    want = [[1, 1, 1, 1], [2, 3, 3, 3], [3, 4, 4, 5], [5, 5, 6, 6], [6, 6, 7, 7], [7, 7, 7, 8]]
    assert ops.moe_cumsum(ids, 6).reshape(6, 4).cpu().tolist() == want


@pytest.mark.parametrize("t", [1, 2, 513, 3000])
def test_routing_large_against_oracle(t):
    rng = np.random.default_rng(t)
    ne, k = 8, 2
    logits = rng.standard_normal((t, ne)).astype(np.float16)
    w_ref, ids_ref = o.gating_softmax_topk(logits, k)
    w, ids = ops.gating_softmax_topk(dev(logits), k)
    assert (ids.cpu().numpy() == ids_ref).all()
    cs_ref = o.moe_cumsum(ids_ref, ne)
    cs = ops.moe_cumsum(ids, ne)
    assert (cs.cpu().numpy() == cs_ref).all()
    rev, tok = ops.get_indices(cs, ids)
    rev_ref, tok_ref = o.get_indices(cs_ref, ids_ref)
    assert (rev.cpu().numpy() == rev_ref).all() and (tok.cpu().numpy() == tok_ref).all()
    x = rng.standard_normal((t * k, 64)).astype(np.float16)
    xs = ops.take_rows(dev(x), rev)  # gather by a permutation, then scatter back
    assert (host_f16_bits(ops.scatter_output(xs, rev)) == x.view(np.uint16)).all()


@pytest.mark.parametrize("name", ["q4f16_1", "q3f16_1"])
@pytest.mark.parametrize("x_rows", [1, 2])
def test_moe_gemv(name, x_rows):
    s = SCHEMES[name]
    rng = np.random.default_rng(41)
    ne, n, k = 8, 520, 1024 if s.bits == 4 else 1000
    w = (rng.standard_normal((ne, n, k)) * 0.02).astype(np.float16)
    qw, qs = o.quantize(w, s)
    x = rng.standard_normal((x_rows, k)).astype(np.float16)
    ids = np.array([[5, 2]], np.int32)
    out = ops.moe_gemv(dev(x), dev(qw), dev(qs), dev(ids), s.bits, s.group_size)
    ref = o.moe_dequantize_gemv_fp32(x, qw, qs, ids, s)
    assert_linear_ok(out, ref, x, k, f"moe_gemv {name}")


@pytest.mark.parametrize("name", ["q4f16_1", "q3f16_1"])
@pytest.mark.parametrize("k", [1004, 1001, 37])
@pytest.mark.parametrize("variant", [-1, 0])
def test_moe_gemv_unaligned_rows_of_x(name, k, variant):
    """x with top_k rows and K not a multiple of 8 (op/moe_matmul.py:147-176 has no such restriction): the second
    slot's row of x then starts off a 16-byte boundary; both GEMV kernels (register, LDS-staged) against the oracle."""
    s = SCHEMES[name]
    rng = np.random.default_rng(43)
    ne, n = 4, 72
    w = (rng.standard_normal((ne, n, k)) * 0.02).astype(np.float16)
    qw, qs = o.quantize(w, s)
    x = rng.standard_normal((2, k)).astype(np.float16)
    ids = np.array([[3, 1]], np.int32)
    gq._lib.set_option("gemv_variant", variant)
    try:
        out = ops.moe_gemv(dev(x), dev(qw), dev(qs), dev(ids), s.bits, s.group_size)
    finally:
        gq._lib.set_option("gemv_variant", -1)
    ref = o.moe_dequantize_gemv_fp32(x, qw, qs, ids, s)
    assert_linear_ok(out, ref, x, k, f"moe_gemv {name} K={k}")


@pytest.mark.parametrize("name", ["q4f16_1", "q3f16_1"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("ne,top_k", [(8, 2), (8, 1), (64, 2), (3, 2)])
def test_moe_gemv_routed_silu_mul(name, dtype, ne, top_k):
    """One token routing itself inside the e1_e3 expert matmul: ids and weights bit for bit those of the routing
    operator (ties included: two equal logits, the lower expert first), the output bit for bit that of the
    operator pair it replaces, and the oracle's values."""
    s = SCHEMES[name]
    rng = np.random.default_rng(47 + ne + top_k)
    n, k = 520, 1024 if s.bits == 4 else 1000
    w = (rng.standard_normal((ne, n, k)) * 0.02).astype(np.float16)
    qw, qs = o.quantize(w, s)
    x = dev(rng.standard_normal((1, k)).astype(np.float16)).to(dtype)
    logits = rng.standard_normal((1, ne)).astype(np.float16)
    logits[0, ne - 1] = logits[0, 1] = logits.max() + 0.5  # a tie for the first place
    gate = dev(logits).to(dtype)
    qs_d = dev(qs).to(dtype)
    out, weights, ids = ops.moe_gemv_routed_silu_mul(x, gate, top_k, dev(qw), qs_d, s.bits, s.group_size)
    assert gq._lib.last_kernel().startswith("gq::gemv_reg_kernel"), gq._lib.last_kernel()
    w_ref, ids_ref = ops.gating_softmax_topk(gate, top_k)
    assert torch.equal(ids, ids_ref) and torch.equal(weights, w_ref)
    assert ids[0, 0].item() == 1 and (top_k == 1 or ids[0, 1].item() == ne - 1)
    pair = ops.moe_gemv(x, dev(qw), qs_d, ids_ref, s.bits, s.group_size, silu_mul_halves=True)
    assert torch.equal(out, pair)
    if dtype == torch.float16:
        full = o.moe_dequantize_gemv_fp32(x.cpu().numpy(), qw, qs, ids.cpu().numpy(), s)
        ref = o.silu_mul_f16(full.astype(np.float16)).astype(np.float64)
        got = out.float().cpu().numpy()
        assert np.abs(got - ref).max() <= 2e-2 * max(1.0, np.abs(ref).max()), np.abs(got - ref).max()


@pytest.mark.parametrize("name", ["q4f16_1", "q3f16_1"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("n,k", [(520, 14336), (4100, 14336), (100, 8200), (64, 5200), (36, 15360), (1000, 11008)])
def test_moe_gemv_combine(name, dtype, n, k):
    """One token's e2 expert matmul and the weighted sum over its two experts in one launch, against the operator pair it
    replaces (bit for bit wherever the pair's matmul splits K the same way, i.e. from 5 groups per lane on; a last place
    of the model dtype otherwise, where the pair adds a row's K in one run) and against the oracle's values."""
    s = SCHEMES[name]
    rng = np.random.default_rng(n + k)
    ne = 4
    w = (rng.standard_normal((ne, n, k)) * 0.02).astype(np.float16)
    qw, qs = o.quantize(w, s)
    x = dev(rng.standard_normal((2, k)).astype(np.float16)).to(dtype)
    ids = dev(np.array([[3, 1]], np.int32))
    weights = dev(np.array([[0.625, 0.375]], np.float16)).to(dtype)
    qs_d = dev(qs).to(dtype)
    out = ops.moe_gemv_combine(x, dev(qw), qs_d, ids, weights, s.bits, s.group_size)
    assert gq._lib.last_kernel().startswith("gq::gemv_reg_kernel") and ",4," in gq._lib.last_kernel(), gq._lib.last_kernel()
    y = ops.moe_gemv(x, dev(qw), qs_d, ids, s.bits, s.group_size)
    pair = ops.moe_combine(y.reshape(1, 2, n), weights)
    assert out.shape == pair.shape == (1, n)
    groups_per_lane = -(-(-(-k // s.group_size)) // 64)
    if groups_per_lane >= 5:
        assert torch.equal(out, pair)
    else:
        err = (out.float() - pair.float()).abs().max().item()
        assert err <= (2 ** -7 if dtype == torch.bfloat16 else 2 ** -10) * max(1.0, pair.float().abs().max().item()), err
    if dtype == torch.float16:
        full = o.moe_dequantize_gemv_fp32(x.cpu().numpy(), qw, qs, ids.cpu().numpy(), s)  # [2, n] float64
        ref = 0.625 * full[0] + 0.375 * full[1]
        got = out.float().cpu().numpy()[0]
        assert np.abs(got - ref).max() <= 1e-2 * max(1.0, np.abs(ref).max()), np.abs(got - ref).max()


def test_moe_gemv_combine_declines():
    s = SCHEMES["q4f16_1"]
    rng = np.random.default_rng(6)
    ne, n = 4, 64
    for k, top_k, f32 in [(14336, 3, False), (14336, 2, True), (1024, 2, False)]:  # three slots; float32; a short K
        qw, qs = o.quantize((rng.standard_normal((ne, n, k)) * 0.02).astype(np.float16), s)
        x = dev(rng.standard_normal((top_k, k)).astype(np.float16))
        ids = dev(np.arange(top_k, dtype=np.int32).reshape(1, top_k))
        wts = dev(np.full((1, top_k), 0.25, np.float16))
        qs_d = dev(qs)
        if f32:
            x, wts, qs_d = x.float(), wts.float(), qs_d.float()
        with pytest.raises(gq._lib.Mi355gqError) as err:
            ops.moe_gemv_combine(x, dev(qw), qs_d, ids, wts, 4, 32)
        assert err.value.code == gq._lib.ERR_UNSUPPORTED


def test_moe_gemv_routed_silu_mul_declines():
    s = SCHEMES["q4f16_1"]
    rng = np.random.default_rng(5)
    ne, n, k = 8, 64, 256
    qw, qs = o.quantize((rng.standard_normal((ne, n, k)) * 0.02).astype(np.float16), s)
    x = dev(rng.standard_normal((1, k)).astype(np.float16))
    gate = dev(rng.standard_normal((1, ne)).astype(np.float16))
    with pytest.raises(gq._lib.Mi355gqError) as err:  # three slots: the operator pair serves those
        ops.moe_gemv_routed_silu_mul(x, gate, 3, dev(qw), dev(qs), 4, 32)
    assert err.value.code == gq._lib.ERR_UNSUPPORTED
    with pytest.raises(gq._lib.Mi355gqError) as err:  # float32 models
        ops.moe_gemv_routed_silu_mul(x.float(), gate.float(), 2, dev(qw), dev(qs).float(), 4, 32)
    assert err.value.code == gq._lib.ERR_UNSUPPORTED


@pytest.mark.parametrize("name", ["q4f16_1", "q3f16_1"])
@pytest.mark.parametrize("indptr", [[0, 3, 3, 40, 41], [0, 0, 0, 0, 130], [0, 1, 2, 3, 4], [0, 0, 0, 0, 0],
                                    [0, 33, 34, 60, 64], [0, 70, 70, 71, 200]])
def test_moe_group_gemm(name, indptr):
    s = SCHEMES[name]
    rng = np.random.default_rng(43)
    ne, n, k = 4, 200, 512 if s.bits == 4 else 520
    rows = max(indptr[-1], 1)
    w = (rng.standard_normal((ne, n, k)) * 0.02).astype(np.float16)
    qw, qs = o.quantize(w, s)
    x = rng.standard_normal((rows, k)).astype(np.float16)
    ip = np.array(indptr, np.int32)
    out = ops.moe_group_gemm(dev(x), dev(qw), dev(qs), dev(ip), s.bits, s.group_size)
    ref = o.dequantize_group_gemm_fp32(x, qw, qs, ip, s)
    assert_linear_ok(out, ref, x, k, f"group_gemm {name} {indptr}")
    out64 = ops.moe_group_gemm(dev(x), dev(qw), dev(qs), dev(ip.astype(np.int64)), s.bits, s.group_size)
    assert bool((out64 == out).all())


@pytest.mark.parametrize("name", ["q4f16_1", "q3f16_1"])
@pytest.mark.parametrize("model_dtype", ["float16", "bfloat16"])
def test_moe_group_gemm_about_one_row_per_expert(name, model_dtype):
    """Up to num_experts rows: one grid row of the GEMV per activation row, its expert found from indptr.
    Empty experts, experts with several rows, rows outside every segment, int64 indptr, the gather index
    and the fused SiLU form."""
    s = SCHEMES[name]
    rng = np.random.default_rng(53)
    ne, n = 70, 264  # more experts than one wave's lanes
    k = 1024 if s.bits == 4 else 1000
    tdt = torch.float16 if model_dtype == "float16" else torch.bfloat16
    w = (rng.standard_normal((ne, n, k)) * 0.02).astype(np.float16)
    qw, qs16 = o.quantize(w, s)
    qs = torch.from_numpy(qs16.astype(np.float32)).to(DEV).to(tdt)
    qs_ref = qs.float().cpu().numpy()
    qwd = dev(qw)
    for rows, cuts in ((1, {69: 1}), (9, {0: 2, 3: 1, 64: 3, 69: 3}), (70, {5: 30, 6: 1, 68: 39}), (33, {1: 7, 40: 20})):
        counts = np.zeros(ne, np.int64)
        for e, c in cuts.items():
            counts[e] = c
        ip = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)  # the last case covers 27 of 33 rows
        x = torch.from_numpy(rng.standard_normal((rows, k)).astype(np.float32)).to(DEV).to(tdt)
        x_ref = x.float().cpu().numpy()
        out = torch.full((rows, n), 7.0, dtype=tdt, device=DEV)
        if model_dtype == "float16":
            gq._lib.call("mi355gq_moe_group_gemm", x.data_ptr(), rows, qwd.data_ptr(), qs.data_ptr(), dev(ip).data_ptr(),
                         gq._lib.I32, ne, n, k, s.bits, s.group_size, out.data_ptr(), 0)
        else:
            gq._lib.call("mi355gq_moe_group_gemm_dt", x.data_ptr(), rows, qwd.data_ptr(), qs.data_ptr(),
                         dev(ip).data_ptr(), gq._lib.I32, ne, n, k, s.bits, s.group_size, gq._lib.BF16, out.data_ptr(), 0)
        torch.cuda.synchronize()
        covered = int(ip[-1])
        ref = o.dequantize_group_gemm_dt_fp64(x_ref, qw, qs_ref, ip, s, model_dtype)[:covered]
        got = out.float().cpu().numpy()
        assert (got[covered:] == 7.0).all()  # rows that no segment covers are left alone
        err = np.abs(got[:covered] - ref)
        scale = np.abs(ref).max() + 1e-6
        assert err.max() <= (2e-3 if model_dtype == "float16" else 1.2e-2) * scale, (rows, err.max(), scale)
        if covered == rows:
            out2 = ops.moe_group_gemm(x, qwd, qs, dev(ip.astype(np.int64)), s.bits, s.group_size)
            assert torch.equal(out2, out)
            src = torch.from_numpy(rng.standard_normal((rows + 5, k)).astype(np.float32)).to(DEV).to(tdt)
            idx = torch.from_numpy(rng.integers(0, rows + 5, rows).astype(np.int32)).to(DEV)
            for silu in (False, True):
                want = ops.moe_group_gemm(ops.take_rows(src, idx), qwd, qs, dev(ip), s.bits, s.group_size, silu)
                assert torch.equal(ops.moe_experts(src, idx, qwd, qs, dev(ip), s.bits, s.group_size, silu), want)
                if silu:
                    plain = ops.moe_group_gemm(ops.take_rows(src, idx), qwd, qs, dev(ip), s.bits, s.group_size)
                    assert torch.equal(want, ops.silu_mul(plain))


@pytest.mark.parametrize("name", ["q4f16_1", "q3f16_1"])
def test_moe_group_gemm_wide_tile(name):
    """Enough rows per expert and enough column tiles for the 128 x 256 grouped tile; ragged segments."""
    s = SCHEMES[name]
    rng = np.random.default_rng(45)
    ne, n, k = 2, 49152, 256 if s.bits == 4 else 240
    ip = np.array([0, 131, 262], np.int32)
    w = (rng.standard_normal((ne, n, k)) * 0.02).astype(np.float16)
    qw, qs = o.quantize(w, s)
    x = rng.standard_normal((262, k)).astype(np.float16)
    out = ops.moe_group_gemm(dev(x), dev(qw), dev(qs), dev(ip), s.bits, s.group_size)
    ref = o.dequantize_group_gemm_fp32(x, qw, qs, ip, s)
    assert_linear_ok(out, ref, x, k, f"group_gemm wide {name}")
    fused = ops.moe_experts(dev(x), None, dev(qw), dev(qs), dev(ip), s.bits, s.group_size, silu_mul_halves=True)
    assert bool((fused == ops.silu_mul(out)).all())


@pytest.mark.parametrize("name", ["q4f16_1", "q3f16_1"])
@pytest.mark.parametrize("variant", [-1, 1, 10, 11])  # heuristic, 128-row tiles, 256 x 256 / 256 x 128 tiles that skip empty row blocks
def test_moe_group_gemm_tall_tiles_on_ragged_segments(name, variant):
    """Grouped matmul from about 64 rows per expert on: 256-row tiles whose waves skip the 32-row blocks past the
    end of a segment.  Segments of 1, 31..33, 127..129 and 300 rows (two tiles), an empty expert, the gather index,
    the folded activation and both indptr dtypes; every tile choice must give the same bits."""
    s = SCHEMES[name]
    if variant == 10 and s.bits == 3:
        pytest.skip("q3 has no 256 x 256 tile (its K tile does not fit LDS)")
    rng = np.random.default_rng(61)
    counts = [300, 0, 129, 33, 1, 127, 32, 31]
    ne, n, k = len(counts), 520, 512 if s.bits == 4 else 480
    ip = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    rows = int(ip[-1])
    w = (rng.standard_normal((ne, n, k)) * 0.02).astype(np.float16)
    qw, qs = o.quantize(w, s)
    x = rng.standard_normal((rows, k)).astype(np.float16)
    ref = o.dequantize_group_gemm_fp32(x, qw, qs, ip, s)
    base = ops.moe_group_gemm(dev(x), dev(qw), dev(qs), dev(ip), s.bits, s.group_size)
    src = rng.standard_normal((rows + 7, k)).astype(np.float16)
    idx = rng.integers(0, rows + 7, rows).astype(np.int32)
    gq._lib.set_option("gemm_variant", variant)
    try:
        out = ops.moe_group_gemm(dev(x), dev(qw), dev(qs), dev(ip), s.bits, s.group_size)
        out64 = ops.moe_group_gemm(dev(x), dev(qw), dev(qs), dev(ip.astype(np.int64)), s.bits, s.group_size)
        fused = ops.moe_experts(dev(x), None, dev(qw), dev(qs), dev(ip), s.bits, s.group_size, silu_mul_halves=True)
        gathered = ops.moe_experts(dev(src), dev(idx), dev(qw), dev(qs), dev(ip), s.bits, s.group_size)
        gq._lib.set_option("gemm_fast_loop", 0)  # the general K loop (this K is whole K tiles: the other one ran above)
        general = ops.moe_group_gemm(dev(x), dev(qw), dev(qs), dev(ip), s.bits, s.group_size)
    finally:
        gq._lib.set_option("gemm_variant", -1)
        gq._lib.set_option("gemm_fast_loop", -1)
    assert_linear_ok(out, ref, x, k, f"grouped tall tiles {name} variant {variant}")
    assert torch.equal(out, base) and torch.equal(out64, out) and torch.equal(general, out)
    assert torch.equal(fused, ops.silu_mul(out))
    assert_linear_ok(gathered, o.dequantize_group_gemm_fp32(src[idx], qw, qs, ip, s), src[idx], k, "gathered")


def test_moe_group_gemm_last_round_on_the_narrow_tile():
    """A grouped matmul wide enough for more than one round of 256 x 256 workgroups leaves the columns of a last round
    that is at most about half full to a second launch on the 256 x 128 tile (8 experts x 36 column tiles = 288
    workgroups: 32 full column tiles, then 4 x 2 narrow ones).  Same bits as the single launch, plain and with the
    folded activation (whose column order interleaves gate and up blocks)."""
    s = SCHEMES["q4f16_1"]
    rng = np.random.default_rng(67)
    counts = [70, 64, 100, 65, 90, 128, 66, 77]
    ne, n, k = len(counts), 9216, 64
    ip = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    rows = int(ip[-1])
    qw = rng.integers(0, 2**32, (ne, n, k // 8), dtype=np.uint64).astype(np.uint32)
    qs = (rng.random((ne, n, k // 32)) * 0.01 + 0.001).astype(np.float16)
    x = rng.standard_normal((rows, k)).astype(np.float16)
    out = ops.moe_group_gemm(dev(x), dev(qw), dev(qs), dev(ip), 4, 32)
    assert gq._lib.last_kernel().startswith("gq::gemm_pipe_kernel<4,256,128,"), gq._lib.last_kernel()  # the second launch
    fused = ops.moe_experts(dev(x), None, dev(qw), dev(qs), dev(ip), 4, 32, silu_mul_halves=True)
    gq._lib.set_option("gemm_variant", 10)
    try:
        one = ops.moe_group_gemm(dev(x), dev(qw), dev(qs), dev(ip), 4, 32)
        assert gq._lib.last_kernel().startswith("gq::gemm_pipe_kernel<4,256,256,"), gq._lib.last_kernel()
        fused_one = ops.moe_experts(dev(x), None, dev(qw), dev(qs), dev(ip), 4, 32, silu_mul_halves=True)
    finally:
        gq._lib.set_option("gemm_variant", -1)
    assert torch.equal(out, one) and torch.equal(fused, fused_one)
    sel = rng.choice(n, 96, replace=False)
    sel[:4] = [0, 8191, 8192, n - 1]  # both sides of the seam
    ref = o.dequantize_group_gemm_fp32(x, qw[:, sel], qs[:, sel], ip, s)
    assert_linear_ok(out[:, torch.from_numpy(sel).to(out.device)], ref, x, k, "grouped, last round on the narrow tile")


def test_silu_mul_and_combine():
    rng = np.random.default_rng(47)
    x = (rng.standard_normal((5, 192)) * 3).astype(np.float16)
    got = ops.silu_mul(dev(x)).cpu().numpy()
    ref = o.silu_mul_f16(x)
    ulp = np.abs(got.view(np.int16).astype(np.int32) - ref.view(np.int16).astype(np.int32))
    assert ulp.max() <= 2, ulp.max()
    y = rng.standard_normal((6, 2, 64)).astype(np.float16)
    w = rng.random((6, 2)).astype(np.float16)
    out = ops.moe_combine(dev(y), dev(w)).cpu().numpy()
    p = (y * w[:, :, None]).astype(np.float16)
    assert (out.view(np.uint16) == (p[:, 0] + p[:, 1]).astype(np.float16).view(np.uint16)).all()


@pytest.mark.parametrize("case", ["moe_t1", "moe_t9"])
def test_mixtral_moe_layer_golden(golden, case):
    from mlc_llm_amd.nn import MixtralMoE

    z = golden(case)
    t, h = z["x"].shape
    ne, two_i, _ = z["q13"].shape
    moe = MixtralMoE(h, two_i // 2, ne, 2, gq.QUANTIZATION["q4f16_1"], device=DEV)
    moe.e1_e3.q_weight.data, moe.e1_e3.q_scale.data = dev(z["q13"]), dev(z["s13"])
    moe.e2.q_weight.data, moe.e2.q_scale.data = dev(z["q2"]), dev(z["s2"])
    y = moe(dev(z["x"]).reshape(1, t, h), dev(z["logits"])).reshape(t, h).cpu().numpy()
    ref = z["y"].astype(np.float64)
    err = np.abs(y.astype(np.float64) - ref).max()
    rel = np.linalg.norm(y.astype(np.float64) - ref) / np.linalg.norm(ref)
    assert rel <= 4e-3 and err <= 0.05, (err, rel)  # two chained matmuls + fp16 glue


# ------------------------------------------------------------------ fused residual addition

@pytest.mark.parametrize("name", ["q4f16_1", "q3f16_1"])
@pytest.mark.parametrize("m", [1, 2, 3, 4, 7, 8, 12, 16, 40, 100, 300])  # every regime of the dispatcher
def test_linear_residual_every_regime(name, m):
    s = SCHEMES[name]
    n, k = 264, 4096 if s.bits == 4 else 4000
    x, qw, qs, b = _linear_case(s, m, n, k, 400 + m, bias=True)
    res = np.random.default_rng(m).standard_normal((m, n)).astype(np.float16)
    ref = o.linear_fp32(x, qw, qs, s, b) + res.astype(np.float64)
    y = ops.linear(dev(x), dev(qw), dev(qs), s.bits, s.group_size, dev(b), residual=dev(res))
    y32 = ops.linear(dev(x), dev(qw), dev(qs), s.bits, s.group_size, None, torch.float32, residual=dev(res))
    assert_linear_ok(y, ref, x, k, f"linear+residual {name} M={m}")
    assert_linear_ok(y32, ref - b.astype(np.float64), x, k, f"linear+residual {name} M={m} fp32 out")
    # in place: hidden += proj(x)
    hidden = dev(res)
    out = ops.linear(dev(x), dev(qw), dev(qs), s.bits, s.group_size, dev(b), out=hidden, residual=hidden)
    assert out.data_ptr() == hidden.data_ptr()
    assert torch.equal(out, y), f"in-place residual differs from out-of-place, {name} M={m}"


@pytest.mark.parametrize("variant", [0, 2, 3, 4, 7, 8])  # LDS GEMV, the skinny forms, quad-row phases / 4-row passes
def test_linear_residual_forced_kernels(variant):
    s = SCHEMES["q4f16_1"]
    m, n, k = (5, 520, 14336) if variant in (7, 8) else ((2, 520, 1024) if variant == 0 else (9, 520, 1024))
    x, qw, qs, b = _linear_case(s, m, n, k, 500 + variant, bias=True)
    res = np.random.default_rng(variant).standard_normal((m, n)).astype(np.float16)
    gq._lib.set_option("gemv_variant", variant)
    try:
        y = ops.linear(dev(x), dev(qw), dev(qs), 4, 32, dev(b), residual=dev(res))
    finally:
        gq._lib.set_option("gemv_variant", -1)
    assert_linear_ok(y, o.linear_fp32(x, qw, qs, s, b) + res.astype(np.float64), x, k, f"residual, variant {variant}")


def test_linear_residual_argument_checks():
    s = SCHEMES["q4f16_1"]
    x, qw, qs, _ = _linear_case(s, 2, 64, 128, 1)
    xd, qwd, qsd = dev(x), dev(qw), dev(qs)
    out32 = torch.empty((2, 64), dtype=torch.float32, device=xd.device)
    rc = gq._lib.lib().mi355gq_linear_residual(xd.data_ptr(), qwd.data_ptr(), qsd.data_ptr(), None, None, 2, 64, 128,
                                                4, 32, gq._lib.F16, out32.data_ptr(), None, 0, None)
    assert rc == -1 and "residual is null" in gq._lib.lib().mi355gq_last_error().decode()
    rc = gq._lib.lib().mi355gq_linear_residual(xd.data_ptr(), qwd.data_ptr(), qsd.data_ptr(), None, out32.data_ptr(),
                                                2, 64, 128, 4, 32, gq._lib.F32, out32.data_ptr(), None, 0, None)
    assert rc == -1 and "in-place" in gq._lib.lib().mi355gq_last_error().decode()


def test_stream_read_probe_runs_and_validates():
    a = torch.arange(4096 + 8, dtype=torch.int32, device="cuda:0")  # sizes that exercise the tail loop
    b = torch.ones(64, dtype=torch.int32, device="cuda:0")
    sink = torch.zeros(1, dtype=torch.int32, device="cuda:0")
    gq._lib.call("mi355gq_testing_stream_read", a.data_ptr(), a.numel() * 4, b.data_ptr(), b.numel() * 4,
                 sink.data_ptr(), torch.cuda.current_stream().cuda_stream)
    gq._lib.call("mi355gq_testing_stream_read", a.data_ptr(), a.numel() * 4, None, 0, None,
                 torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert gq._lib.lib().mi355gq_testing_stream_read(a.data_ptr(), 24, None, 0, None, None) == -1  # not a multiple of 16


@pytest.mark.parametrize("name", ["q4f16_1", "q3f16_1"])
def test_quantize_dequantize_every_row_length(name):
    # the kernels find (row, word) of a thread by a multiply-high with a constant per row length:
    # walk many lengths (odd, powers of two, just under / over a group) and rows that are not a multiple
    # of anything
    s = SCHEMES[name]
    rng = np.random.default_rng(123)
    ks = sorted(set(list(range(1, 330, 7)) + [32, 40, 64, 80, 128, 256, 512, 1024, 1000, 2047, 2048, 4100, 9999]))
    for k in ks:
        rows = 37 if k < 3000 else 5
        w = (rng.standard_normal((rows, k)) * 0.1).astype(np.float16)
        qw_ref, qs_ref = o.quantize(w, s)
        qw, qs = ops.quantize(dev(w), s.bits, s.group_size)
        assert np.array_equal(host_u32(qw), qw_ref), k
        assert np.array_equal(host_f16_bits(qs), qs_ref.view(np.uint16)), k
        d = ops.dequantize(qw, qs, k, s.bits, s.group_size)
        assert np.array_equal(host_f16_bits(d), o.dequantize(qw_ref, qs_ref, s, k).view(np.uint16)), k


# ------------------------------------------------------------------ other model dtypes (q4f32_1, q4bf16_*)

_TORCH_OF = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def _carrier(t: torch.Tensor) -> np.ndarray:
    return t.float().cpu().numpy()


@pytest.mark.parametrize("model_dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("bits_name", ["q4f16_1", "q3f16_1"])
@pytest.mark.parametrize("mode", [0, 1])
def test_packing_other_model_dtypes_bit_exact(model_dtype, bits_name, mode):
    s = SCHEMES[bits_name]
    dt = _TORCH_OF[model_dtype]
    rng = np.random.default_rng(77)
    for rows, k in ((5, 13), (16, 120), (16, 128), (33, 4096), (7, 1000)):
        w32 = o.round_to((rng.standard_normal((rows, k)) * 0.07).astype(np.float32), model_dtype)
        w32[0, : min(k, s.group_size)] = 0          # an all-zero group: 0 / 0
        w32[1, 0] = float(o.round_to(np.array([3.0e4], dtype=np.float32), model_dtype)[0])  # one large value in a group of small ones
        w = torch.from_numpy(w32).to(dt).to(DEV)
        assert np.array_equal(_carrier(w), w32)
        qw_ref, qs_ref = o.quantize_dt(w32, s, model_dtype, ["half_away", "half_even"][mode])
        qw, qs = ops.quantize(w, s.bits, s.group_size, mode)
        assert qs.dtype == dt
        assert np.array_equal(_carrier(qs), qs_ref), (rows, k)
        assert np.array_equal(host_u32(qw), qw_ref), (rows, k)
        d = ops.dequantize(qw, qs, k, s.bits, s.group_size)
        assert d.dtype == dt
        d_ref = o.dequantize_dt(qw_ref, qs_ref, s, k, model_dtype)
        assert np.array_equal(_carrier(d), d_ref), (rows, k)
        ids = torch.tensor([rows - 1, 0, 2, 2, 99, -1], dtype=torch.int32, device=DEV)
        emb = ops.embedding_take(ids, qw, qs, k, s.bits, s.group_size)
        assert np.array_equal(_carrier(emb), d_ref[[rows - 1, 0, 2, 2, rows - 1, 0]])


@pytest.mark.parametrize("model_dtype", ["float32", "bfloat16"])
def test_other_model_dtypes_golden(golden, model_dtype):
    dt = _TORCH_OF[model_dtype]
    for shp in ("2x13", "16x128", "5x200"):
        z = golden(f"dtype_{model_dtype}_{shp}")
        k = z["w"].shape[1]
        w = torch.from_numpy(z["w"]).to(dt).to(DEV)
        for mode, key in ((0, "half_away"), (1, "half_even")):
            qw, qs = ops.quantize(w, 4, 32, mode)
            assert np.array_equal(host_u32(qw), z[f"q_weight_{key}"]) and np.array_equal(_carrier(qs), z[f"q_scale_{key}"])
        qw, qs = dev(z["q_weight_half_away"]), torch.from_numpy(z["q_scale_half_away"]).to(dt).to(DEV)
        assert np.array_equal(_carrier(ops.dequantize(qw, qs, k, 4, 32)), z["dequant"])
        y = ops.linear(torch.from_numpy(z["x"]).to(dt).to(DEV), qw, qs, 4, 32, out_dtype=torch.float32)
        err = np.linalg.norm(y.double().cpu().numpy() - z["y"]) / np.linalg.norm(z["y"])
        # (bfloat16, few rows: the kernels that scale group sums skip _dequantize's per-weight rounding, which
        #  the fixture's product includes: the matmul tolerance applies, not the fp32-accumulation one)
        assert err <= (2e-3 if model_dtype == "bfloat16" else 2e-6), err


def test_other_model_dtypes_modules():
    # registry entries: quantize_weight / dequantize_weight / embedding work; the matmul says what is missing
    for name in ("q4bf16_1", "q4f32_1", "q4bf16_0"):
        cfg = gq.QUANTIZATION[name]
        dt = _TORCH_OF[cfg.model_dtype]
        w = (torch.randn(48, 96, device=DEV) * 0.05)
        qw, qs = cfg.quantize_weight(w, output_transpose=cfg.linear_weight_layout == "KN")
        assert qs.dtype == dt
        if cfg.linear_weight_layout == "KN":
            assert tuple(qw.shape) == (12, 48) and tuple(qs.shape) == (3, 48)
            qw, qs = qw.t().contiguous(), qs.t().contiguous()
        back = cfg.dequantize_weight(qw, qs, 96)
        # half a step, plus the bf16 roundings of the quotient and of the product
        assert back.dtype == dt and (back.float() - w.to(dt).float()).abs().max() <= qs.float().abs().max() * (0.51 if dt == torch.float32 else 0.6)
        emb = gq.GroupQuantizeEmbedding(48, 96, cfg, device=DEV)
        if cfg.linear_weight_layout == "NK":
            emb.q_weight.data.copy_(qw)
            emb.q_scale.data.copy_(qs)
            out = emb(torch.tensor([[3, 47]], device=DEV))
            assert torch.equal(out[0], back[[3, 47]])
        if cfg.linear_weight_layout == "NK":  # (the reference has no KN expert stack either)
            experts = gq.GroupQuantizeMixtralExperts(2, 96, 48, cfg, device=DEV)
            experts.q_weight.data.copy_(torch.stack([qw, qw.flip(0)]))
            experts.q_scale.data.copy_(torch.stack([qs, qs.flip(0)]))
            x = torch.randn(3, 96, device=DEV).to(dt)
            # single token: the selected experts' rows are the one-row linear over the same weights
            picked = experts(x[:1], torch.tensor([[1, 0]], dtype=torch.int32, device=DEV))
            assert picked.dtype == dt and tuple(picked.shape) == (2, 48)
            assert torch.equal(picked[1], ops.linear(x[:1], qw, qs, cfg.bits, cfg.group_size)[0])
            assert torch.equal(picked[0], ops.linear(x[:1], qw.flip(0), qs.flip(0), cfg.bits, cfg.group_size)[0])
            grouped = experts(x, torch.tensor([0, 1, 3], dtype=torch.int32, device=DEV))
            want = x.double() @ back.double().t()
            assert (grouped[0].double() - want[0]).norm() / want[0].norm() <= (3e-3 if dt == torch.bfloat16 else 1e-6)
            assert (grouped[1:].double() - want[1:].flip(1)).norm() / want[1:].norm() <= (3e-3 if dt == torch.bfloat16 else 1e-6)


@pytest.mark.parametrize("model_dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("bits_name,m,n,k", [
    ("q4f16_1", 1, 512, 4096), ("q4f16_1", 2, 100, 1000), ("q4f16_1", 4, 257, 2048), ("q4f16_1", 8, 128, 8192),
    ("q4f16_1", 3, 64, 13), ("q4f16_1", 1, 40, 40000),                     # ragged K; K past the GEMV's LDS
    ("q4f16_1", 1, 130, 14336), ("q4f16_1", 2, 96, 8192), ("q4f16_1", 2, 33, 1001), ("q3f16_1", 2, 64, 2000),
    ("q4f16_1", 2, 64, 14336), ("q4f16_1", 3, 1024, 4096), ("q4f16_1", 5, 64, 14336), ("q4f16_1", 7, 132, 1000),
    ("q3f16_1", 4, 96, 4096), ("q3f16_1", 8, 64, 10000),
    ("q4f16_1", 9, 256, 512), ("q4f16_1", 130, 200, 1024), ("q4f16_1", 300, 384, 360), ("q4f16_1", 64, 130, 100),
    ("q3f16_1", 1, 256, 4096), ("q3f16_1", 5, 96, 1000), ("q3f16_1", 200, 136, 2000),
])
def test_linear_other_model_dtypes(model_dtype, bits_name, m, n, k):
    s = SCHEMES[bits_name]
    dt = _TORCH_OF[model_dtype]
    rng = np.random.default_rng(m * 1000 + n)
    w32 = o.round_to((rng.standard_normal((n, k)) * 0.05).astype(np.float32), model_dtype)
    x32 = o.round_to(rng.standard_normal((m, k)).astype(np.float32), model_dtype)
    b32 = o.round_to(rng.standard_normal(n).astype(np.float32), model_dtype)
    qw_ref, qs_ref = o.quantize_dt(w32, s, model_dtype)
    qw, qs = dev(qw_ref), torch.from_numpy(qs_ref).to(dt).to(DEV)
    x, b = torch.from_numpy(x32).to(dt).to(DEV), torch.from_numpy(b32).to(dt).to(DEV)
    ref = o.linear_dt_fp64(x32, qw_ref, qs_ref, s, model_dtype, b32)
    den = np.linalg.norm(ref)
    # float32 result: only the fp32 accumulation separates it from the exact product of the same operands
    y32 = ops.linear(x, qw, qs, s.bits, s.group_size, b, out_dtype=torch.float32)
    assert y32.dtype == torch.float32 and tuple(y32.shape) == (m, n)
    err = y32.double().cpu().numpy() - ref
    ng = -(-k // s.group_size)
    # one row up to 8 groups per lane, two rows up to 4: the register GEMV; 2..8 rows the quad-row kernel
    unrounded = (m == 1 and ng <= 512) or (m == 2 and ng <= 256) or (2 <= m <= 8 and k % 8 == 0 and n % 4 == 0)
    if model_dtype == "bfloat16" and unrounded:
        # these kernels scale each group's integer dot product, so their operands are the weights before
        # _dequantize's rounding to bfloat16: exact against those, and within the matmul tolerance (2^-9 per
        # weight, random in sign) of the product with the rounded ones
        exact = y32.double().cpu().numpy() - o.linear_dt_fp64(x32, qw_ref, qs_ref, s, model_dtype, b32, unrounded_weights=True)
        # (its fp32 sums run over x * (128 + q), some 40 times the size of x * (q - m): that much more rounding)
        assert np.linalg.norm(exact) / den <= 5e-6 + 1e-7 * np.sqrt(k), np.linalg.norm(exact) / den
        assert np.linalg.norm(err) / den <= 2e-3, np.linalg.norm(err) / den
    else:
        # (relative error of a float32 sum of k terms grows like sqrt(k) * 2^-24)
        assert np.linalg.norm(err) / den <= 1e-6 + 4e-8 * np.sqrt(k), np.linalg.norm(err) / den
    assert np.abs(err).max() <= 1e-2 * np.abs(x32).max() * np.sqrt(k) / 64
    # output in the model dtype: the same numbers rounded once
    y = ops.linear(x, qw, qs, s.bits, s.group_size, b)
    assert y.dtype == dt
    assert np.array_equal(_carrier(y), o.round_to(y32.cpu().numpy(), model_dtype))


@pytest.mark.parametrize("m", [3, 4, 8])
@pytest.mark.parametrize("n,k", [(512, 4096), (132, 1000), (260, 8192)])
def test_bfloat16_few_rows_take_the_register_fewrow_kernel(m, n, k):
    """q4bf16_1 at 3..8 rows: the few-row kernel with x in registers on the bf16 4x4x4 matrix instruction (K up to 8192).
    Float32 output exact against the unrounded-weight product (the kernel scales each group's integer dot product), the
    bfloat16 output the same numbers rounded once; bias and residual; the fused gate/up form against the two steps."""
    s = SCHEMES["q4f16_1"]
    rng = np.random.default_rng(m * 100 + n)
    w32 = o.round_to((rng.standard_normal((n, k)) * 0.05).astype(np.float32), "bfloat16")
    x32 = o.round_to(rng.standard_normal((m, k)).astype(np.float32), "bfloat16")
    b32 = o.round_to(rng.standard_normal(n).astype(np.float32), "bfloat16")
    r32 = o.round_to(rng.standard_normal((m, n)).astype(np.float32), "bfloat16")
    qw_ref, qs_ref = o.quantize_dt(w32, s, "bfloat16")
    qw, qs = dev(qw_ref), torch.from_numpy(qs_ref).to(torch.bfloat16).to(DEV)
    x, b, r = (torch.from_numpy(a).to(torch.bfloat16).to(DEV) for a in (x32, b32, r32))
    y32 = ops.linear(x, qw, qs, 4, 32, None, out_dtype=torch.float32)
    kern = gq._lib.last_kernel()
    assert kern.startswith("gq::quadreg_kernel<4,") and kern.endswith(",true>"), kern
    exact = o.linear_dt_fp64(x32, qw_ref, qs_ref, s, "bfloat16", None, unrounded_weights=True)
    den = np.linalg.norm(exact)
    assert np.linalg.norm(y32.double().cpu().numpy() - exact) / den <= 5e-6 + 1e-7 * np.sqrt(k)
    y = ops.linear(x, qw, qs, 4, 32)
    assert y.dtype == torch.bfloat16 and np.array_equal(_carrier(y), o.round_to(y32.cpu().numpy(), "bfloat16"))
    yb = ops.linear(x, qw, qs, 4, 32, b, out_dtype=torch.float32, residual=r)
    assert gq._lib.last_kernel().startswith("gq::quadreg_kernel<4,") and gq._lib.last_kernel().endswith("1,true>")
    want = exact + b32.astype(np.float64) + r32.astype(np.float64)
    assert np.linalg.norm(yb.double().cpu().numpy() - want) / np.linalg.norm(want) <= 5e-6 + 1e-7 * np.sqrt(k)
    fused = ops.linear_silu_mul(x, qw, qs, 4, 32)
    assert gq._lib.last_kernel().endswith("2,true>"), gq._lib.last_kernel()
    assert torch.equal(fused, ops.silu_mul(y))


@pytest.mark.parametrize("m", [9, 16, 23])  # one batch tile, a full one, two (forced)
@pytest.mark.parametrize("n,k", [(512, 4096), (96, 1024), (160, 8192), (224, 14336)])  # (the last two: K slices at 9 and 16 rows)
def test_bfloat16_midrow_kernel(m, n, k):
    """q4bf16_1 on the kernel that scales the matrix instruction's result (its bfloat16 instance: every field shifted to
    the low bits, offset 128 + 7, x as it is), forced on small shapes: float32 output exact against the unrounded-weight
    product, the bfloat16 output the same numbers rounded once; bias and residual; the fused gate/up form against the two steps."""
    s = SCHEMES["q4f16_1"]
    rng = np.random.default_rng(m * 100 + n)
    w32 = o.round_to((rng.standard_normal((n, k)) * 0.05).astype(np.float32), "bfloat16")
    x32 = o.round_to(rng.standard_normal((m, k)).astype(np.float32), "bfloat16")
    b32 = o.round_to(rng.standard_normal(n).astype(np.float32), "bfloat16")
    r32 = o.round_to(rng.standard_normal((m, n)).astype(np.float32), "bfloat16")
    qw_ref, qs_ref = o.quantize_dt(w32, s, "bfloat16")
    qw, qs = dev(qw_ref), torch.from_numpy(qs_ref).to(torch.bfloat16).to(DEV)
    x, b, r = (torch.from_numpy(a).to(torch.bfloat16).to(DEV) for a in (x32, b32, r32))
    gq._lib.set_option("gemv_variant", 10)
    try:
        y32 = ops.linear(x, qw, qs, 4, 32, None, out_dtype=torch.float32)
        kern = gq._lib.last_kernel()
        y = ops.linear(x, qw, qs, 4, 32)
        yb = ops.linear(x, qw, qs, 4, 32, b, out_dtype=torch.float32, residual=r)
        fused = ops.linear_silu_mul(x, qw, qs, 4, 32)
        kern_fused = gq._lib.last_kernel()
    finally:
        gq._lib.set_option("gemv_variant", -1)
    assert kern.startswith(f"gq::midrow_kernel<{1 if m <= 16 else 2},") and ",true>" in kern, kern
    assert kern_fused.startswith("gq::midrow_kernel<") and ",true>" in kern_fused, kern_fused
    exact = o.linear_dt_fp64(x32, qw_ref, qs_ref, s, "bfloat16", None, unrounded_weights=True)
    assert np.linalg.norm(y32.double().cpu().numpy() - exact) / np.linalg.norm(exact) <= 5e-6 + 1e-7 * np.sqrt(k)
    assert y.dtype == torch.bfloat16 and np.array_equal(_carrier(y), o.round_to(y32.cpu().numpy(), "bfloat16"))
    want = exact + b32.astype(np.float64) + r32.astype(np.float64)
    assert np.linalg.norm(yb.double().cpu().numpy() - want) / np.linalg.norm(want) <= 5e-6 + 1e-7 * np.sqrt(k)
    assert torch.equal(fused, ops.silu_mul(y))


@pytest.mark.parametrize("m", [6, 12])
def test_bfloat16_midrow_kernel_k_slices_default(m):
    """q4bf16_1, 5120 x 13824 (a K of four phases, 68 M weights): five rows and more take the K slices of the kernel on unscaled
    weight operands by default; a sample of the columns against the exact product, the fused gate/up form against the two steps."""
    s = SCHEMES["q4f16_1"]
    n, k = 5120, 13824
    rng = np.random.default_rng(90 + m)
    qw_ref = rng.integers(0, 2**32, (n, k // 8), dtype=np.uint32)
    qs_ref = o.round_to((rng.random((n, k // 32)) * 0.02 + 0.001).astype(np.float32), "bfloat16")
    x32 = o.round_to(rng.standard_normal((m, k)).astype(np.float32), "bfloat16")
    qw, qs = dev(qw_ref), torch.from_numpy(qs_ref).to(torch.bfloat16).to(DEV)
    x = torch.from_numpy(x32).to(torch.bfloat16).to(DEV)
    cols = np.unique(np.concatenate([[0, 1, n // 2, n - 1], rng.integers(0, n, 200)]))
    y32 = ops.linear(x, qw, qs, 4, 32, None, out_dtype=torch.float32)
    kern = gq._lib.last_kernel()
    assert kern.startswith("gq::midrow_kernel<1,") and ",true>" in kern and "slices=4 " in kern, kern
    y = ops.linear(x, qw, qs, 4, 32)
    fused = ops.linear_silu_mul(x, qw, qs, 4, 32)
    assert gq._lib.last_kernel().startswith("gq::midrow_kernel<1,"), gq._lib.last_kernel()
    exact = o.linear_dt_fp64(x32, qw_ref[cols], qs_ref[cols], s, "bfloat16", None, unrounded_weights=True)
    got = y32[:, torch.from_numpy(cols).to(DEV)].double().cpu().numpy()
    assert np.linalg.norm(got - exact) / np.linalg.norm(exact) <= 5e-6 + 1e-7 * np.sqrt(k)
    assert np.array_equal(_carrier(y), o.round_to(y32.cpu().numpy(), "bfloat16"))
    assert torch.equal(fused, ops.silu_mul(y))


def test_bfloat16_midrow_kernel_grouped_default():
    """q4bf16_1 expert segments at six and at sixteen rows per expert on average: the default dispatch takes the bfloat16
    instance (one and two batch tiles per pass); against the exact product, and the fused gate/up form bit for bit."""
    s = SCHEMES["q4f16_1"]
    rng = np.random.default_rng(71)
    ne, n, k = 4, 96, 1024
    w32 = o.round_to((rng.standard_normal((ne, n, k)) * 0.05).astype(np.float32), "bfloat16")
    qw_ref, qs_ref = o.quantize_dt(w32, s, "bfloat16")
    qw, qs = dev(qw_ref), torch.from_numpy(qs_ref).to(torch.bfloat16).to(DEV)
    for ip, tiles in ((np.array([0, 3, 3, 20, 24], np.int32), 1), (np.array([0, 30, 31, 45, 64], np.int32), 2)):
        rows = int(ip[-1])
        x32 = o.round_to(rng.standard_normal((rows, k)).astype(np.float32), "bfloat16")
        x = torch.from_numpy(x32).to(torch.bfloat16).to(DEV)
        out = ops.moe_experts(x, None, qw, qs, dev(ip), 4, 32)
        kern = gq._lib.last_kernel()
        assert kern.startswith(f"gq::midrow_kernel<{tiles},") and ",true>" in kern, kern
        ref = o.dequantize_group_gemm_dt_fp64(x32, qw_ref, qs_ref, ip, s, "bfloat16")
        _assert_dt_matmul_ok(out, ref, x32, k, "bfloat16", f"grouped bf16 mid-row, {tiles} tile(s)")
        fused = ops.moe_experts(x, None, qw, qs, dev(ip), 4, 32, silu_mul_halves=True)
        assert torch.equal(fused, ops.silu_mul(out))


def _assert_dt_matmul_ok(y: torch.Tensor, ref: np.ndarray, x32: np.ndarray, k: int, model_dtype: str, what=""):
    """Output in the model dtype against the exact product of the same operands: the fp32 accumulation
    (relative error of a sum of k terms grows like sqrt(k) * 2^-24) plus, for bfloat16, the one rounding of
    the output (2^-9 per element)."""
    err = y.double().cpu().numpy() - ref
    den = max(np.linalg.norm(ref), 1e-30)
    rel = 1e-6 + 4e-8 * np.sqrt(k) + (2.5e-3 if model_dtype == "bfloat16" else 0.0)
    assert np.linalg.norm(err) / den <= rel, f"{what}: rel-L2 {np.linalg.norm(err) / den:.3e}"
    slack = 2.0 ** -8 * np.abs(ref).max() if model_dtype == "bfloat16" else 0.0
    assert np.abs(err).max() <= 1e-2 * np.abs(x32).max() * np.sqrt(k) / 64 + slack, what


@pytest.mark.parametrize("model_dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("bits_name,k", [("q4f16_1", 512), ("q4f16_1", 1000), ("q3f16_1", 520), ("q3f16_1", 75)])
def test_moe_matmuls_other_model_dtypes(model_dtype, bits_name, k):
    """GroupQuantizeMixtralExperts.forward's two matmuls with x, q_scale and the result in the model dtype."""
    s = SCHEMES[bits_name]
    dt = _TORCH_OF[model_dtype]
    rng = np.random.default_rng(k)
    ne, n = 4, 200
    w32 = o.round_to((rng.standard_normal((ne, n, k)) * 0.05).astype(np.float32), model_dtype)
    qw_ref, qs_ref = o.quantize_dt(w32, s, model_dtype)
    qw, qs = dev(qw_ref), torch.from_numpy(qs_ref).to(dt).to(DEV)
    ids = np.array([[3, 1]], np.int32)
    for x_rows in (1, 2):
        x32 = o.round_to(rng.standard_normal((x_rows, k)).astype(np.float32), model_dtype)
        y = ops.moe_gemv(torch.from_numpy(x32).to(dt).to(DEV), qw, qs, dev(ids), s.bits, s.group_size)
        assert y.dtype == dt and tuple(y.shape) == (2, n)
        ref = o.moe_dequantize_gemv_dt_fp64(x32, qw_ref, qs_ref, ids, s, model_dtype)
        _assert_dt_matmul_ok(y, ref, x32, k, model_dtype, f"moe_gemv x_rows={x_rows}")
    for indptr in ([0, 3, 3, 40, 41], [0, 1, 2, 3, 4], [0, 0, 0, 0, 9], [0, 0, 0, 0, 130], [0, 140, 140, 150, 300],
                   [0, 0, 0, 0, 0]):
        rows = max(indptr[-1], 1)
        x32 = o.round_to(rng.standard_normal((rows, k)).astype(np.float32), model_dtype)
        ip = np.array(indptr, np.int32)
        x = torch.from_numpy(x32).to(dt).to(DEV)
        y = ops.moe_group_gemm(x, qw, qs, dev(ip), s.bits, s.group_size)
        assert y.dtype == dt and tuple(y.shape) == (rows, n)
        ref = o.dequantize_group_gemm_dt_fp64(x32, qw_ref, qs_ref, ip, s, model_dtype)
        _assert_dt_matmul_ok(y, ref, x32, k, model_dtype, f"group_gemm {indptr}")
        y64 = ops.moe_group_gemm(x, qw, qs, dev(ip.astype(np.int64)), s.bits, s.group_size)
        assert torch.equal(y64, y)


@pytest.mark.parametrize("model_dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("m,n,k", [(1, 256, 4096), (2, 64, 14336), (4, 132, 2048), (8, 64, 1000), (3, 64, 13),
                                   (16, 128, 8192), (40, 200, 4096), (130, 264, 1024), (600, 384, 512)])
def test_linear_residual_other_model_dtypes(model_dtype, m, n, k):
    """The residual operand in every kernel family of the float32 / bfloat16 linear: the result equals the plain
    linear's float32 output plus the residual, rounded once (same operations in the same order)."""
    s = SCHEMES["q4f16_1"]
    dt = _TORCH_OF[model_dtype]
    rng = np.random.default_rng(m + n + k)
    w32 = o.round_to((rng.standard_normal((n, k)) * 0.05).astype(np.float32), model_dtype)
    qw_ref, qs_ref = o.quantize_dt(w32, s, model_dtype)
    qw, qs = dev(qw_ref), torch.from_numpy(qs_ref).to(dt).to(DEV)
    x = torch.from_numpy(o.round_to(rng.standard_normal((m, k)).astype(np.float32), model_dtype)).to(dt).to(DEV)
    b = torch.from_numpy(o.round_to(rng.standard_normal(n).astype(np.float32), model_dtype)).to(dt).to(DEV)
    res = torch.from_numpy(o.round_to(rng.standard_normal((m, n)).astype(np.float32), model_dtype)).to(dt).to(DEV)
    y32 = ops.linear(x, qw, qs, 4, 32, b, out_dtype=torch.float32)
    y = ops.linear(x, qw, qs, 4, 32, b, residual=res)
    assert y.dtype == dt
    assert torch.equal(y, (y32 + res.float()).to(dt))
    y_f32 = ops.linear(x, qw, qs, 4, 32, b, out_dtype=torch.float32, residual=res)
    assert torch.equal(y_f32, y32 + res.float())
    # in place: the residual buffer is the output
    acc = res.clone()
    ops.linear(x, qw, qs, 4, 32, b, out=acc, residual=acc)
    assert torch.equal(acc, y)


@pytest.mark.parametrize("model_dtype", ["float32", "bfloat16"])
def test_routing_glue_other_model_dtypes(model_dtype):
    """gating_softmax_topk, moe_route, take_rows / scatter_output, silu_mul and the combine with logits,
    weights and activations in the model dtype."""
    dt = _TORCH_OF[model_dtype]
    rng = np.random.default_rng(5)
    for t, ne, k in ((1, 8, 2), (7, 8, 2), (33, 6, 3), (300, 8, 2)):
        lg32 = o.round_to((rng.standard_normal((t, ne)) * 2).astype(np.float32), model_dtype)
        lg = torch.from_numpy(lg32).to(dt).to(DEV)
        w, ids = ops.gating_softmax_topk(lg, k)
        w_ref, ids_ref = o.gating_softmax_topk_dt(lg32, k, model_dtype)
        assert w.dtype == dt and np.array_equal(ids.cpu().numpy(), ids_ref)
        # the softmax runs in fp32 on both sides with different exp implementations: one ulp of the dtype
        assert np.abs(_carrier(w) - w_ref).max() <= (2.0 ** -8 if model_dtype == "bfloat16" else 1e-6)
        w2, ids2, tok, rev, pos, indptr = ops.moe_route(lg, k)
        assert torch.equal(w2, w) and torch.equal(ids2, ids)
        cs = o.moe_cumsum(ids_ref, ne)
        rev_ref, tok_ref = o.get_indices(cs, ids_ref)
        assert np.array_equal(tok.cpu().numpy(), tok_ref) and np.array_equal(rev.cpu().numpy(), rev_ref)
        assert np.array_equal(indptr.cpu().numpy(), o.get_indptr(cs, ne, t, inclusive=False))
        x32 = o.round_to(rng.standard_normal((t, 40)).astype(np.float32), model_dtype)
        x = torch.from_numpy(x32).to(dt).to(DEV)
        g = ops.take_rows(x, tok)
        assert g.dtype == dt and np.array_equal(_carrier(g), x32[tok_ref])
        sc = ops.scatter_output(g, rev)
        assert np.array_equal(_carrier(sc), o.scatter_output(x32[tok_ref], rev_ref))
        # combine: slot order and expert-sorted order
        y32 = o.round_to(rng.standard_normal((t * k, 24)).astype(np.float32), model_dtype)
        y = torch.from_numpy(y32).to(dt).to(DEV)
        prod = o.round_to(y32.reshape(t, k, 24) * _carrier(w).reshape(t, k, 1), model_dtype)
        want = prod[:, 0]
        for j in range(1, k):
            want = o.round_to(want + prod[:, j], model_dtype)
        assert np.array_equal(_carrier(ops.moe_combine(y.reshape(t, k, 24), w)), want)
        y_sorted = torch.from_numpy(y32[rev_ref]).to(dt).to(DEV)  # row p of the sorted order is slot rev[p]
        assert np.array_equal(_carrier(ops.moe_combine_sorted(y_sorted, pos, w)), want)
    a32 = o.round_to((rng.standard_normal((5, 192)) * 3).astype(np.float32), model_dtype)
    got = _carrier(ops.silu_mul(torch.from_numpy(a32).to(dt).to(DEV)))
    ref = o.silu_mul_dt(a32, model_dtype)
    assert np.abs(got - ref).max() <= np.abs(ref).max() * (2.0 ** -7 if model_dtype == "bfloat16" else 1e-6)


@pytest.mark.parametrize("model_dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("t", [1, 9, 70])
def test_mixtral_moe_layer_other_model_dtypes(model_dtype, t):
    from mlc_llm_amd.nn import MixtralMoE

    cfg = gq.QUANTIZATION["q4f32_1" if model_dtype == "float32" else "q4bf16_1"]
    dt = _TORCH_OF[model_dtype]
    s = SCHEMES["q4f16_1"]
    rng = np.random.default_rng(60 + t)
    h, inter, ne = 128, 192, 4
    w13 = o.round_to((rng.standard_normal((ne, 2 * inter, h)) * 0.08).astype(np.float32), model_dtype)
    w2 = o.round_to((rng.standard_normal((ne, h, inter)) * 0.08).astype(np.float32), model_dtype)
    q13, s13 = o.quantize_dt(w13, s, model_dtype)
    q2, s2 = o.quantize_dt(w2, s, model_dtype)
    x32 = o.round_to(rng.standard_normal((t, h)).astype(np.float32), model_dtype)
    lg32 = o.round_to(rng.standard_normal((t, ne)).astype(np.float32), model_dtype)
    moe = MixtralMoE(h, inter, ne, 2, cfg, device=DEV)
    moe.e1_e3.q_weight.data, moe.e1_e3.q_scale.data = dev(q13), torch.from_numpy(s13).to(dt).to(DEV)
    moe.e2.q_weight.data, moe.e2.q_scale.data = dev(q2), torch.from_numpy(s2).to(dt).to(DEV)
    y = moe(torch.from_numpy(x32).to(dt).to(DEV).reshape(1, t, h), torch.from_numpy(lg32).to(dt).to(DEV))
    assert y.dtype == dt
    y = y.reshape(t, h).double().cpu().numpy()
    ref = o.mixtral_moe_dt(x32, lg32, q13, s13, q2, s2, s, model_dtype).astype(np.float64)
    rel = np.linalg.norm(y - ref) / np.linalg.norm(ref)
    # two chained matmuls and the glue's roundings in the model dtype
    assert rel <= (1.5e-2 if model_dtype == "bfloat16" else 1e-5), rel


@pytest.mark.parametrize("bits_name", ["q4f16_1", "q3f16_1"])
@pytest.mark.parametrize("m,n,k", [(1, 256, 4096), (1, 128, 8192), (1, 64, 14336), (2, 256, 4096), (2, 128, 8192),
                                   (4, 132, 2048), (8, 64, 1000), (3, 64, 13), (16, 128, 8192), (40, 192, 4096),
                                   (100, 200, 1024), (130, 256, 1024), (600, 384, 512)])
def test_linear_silu_mul_bfloat16_equals_the_two_steps(bits_name, m, n, k):
    """The folded gate/up activation of a bfloat16 model in every kernel family; shapes without a fused kernel
    run the two steps, so the equality holds for all of them."""
    s = SCHEMES[bits_name]
    rng = np.random.default_rng(m + n + k)
    w32 = o.round_to((rng.standard_normal((n, k)) * 0.05).astype(np.float32), "bfloat16")
    qw_ref, qs_ref = o.quantize_dt(w32, s, "bfloat16")
    qw, qs = dev(qw_ref), torch.from_numpy(qs_ref).bfloat16().to(DEV)
    x = torch.from_numpy(rng.standard_normal((m, k)).astype(np.float32)).bfloat16().to(DEV)
    fused = ops.linear_silu_mul(x, qw, qs, s.bits, s.group_size)
    assert fused.dtype == torch.bfloat16 and tuple(fused.shape) == (m, n // 2)
    plain = ops.linear(x, qw, qs, s.bits, s.group_size)
    two = ops.silu_mul(plain)
    # a fused GEMM whose plain counterpart splits K sums in another order (N % 64 != 0 keeps the fused one unsplit)
    split_differs = m > 8 and n % 64 != 0 and gq._lib.lib().mi355gq_linear_dt_workspace_bytes(m, n, k, s.bits, s.group_size, 2) > 0
    if split_differs:
        assert (fused.float() - two.float()).abs().max() <= 2.0 ** -6 * two.float().abs().max()
    else:
        assert torch.equal(fused, two), f"{(fused != two).sum().item()} of {fused.numel()} differ"
    # and the value: silu(g) * u of the oracle's product, at the matmul tolerance carried through the two factors
    ref = o.linear_dt_fp64(_carrier(x), qw_ref, qs_ref, s, "bfloat16")
    g, u = ref[:, : n // 2], ref[:, n // 2:]
    want = g / (1.0 + np.exp(-g)) * u
    err = np.abs(fused.double().cpu().numpy() - want)
    tol = 1e-2 * float(x.float().abs().max()) * np.sqrt(k) / 64
    bound = tol * (1.1 * np.abs(u) + np.abs(g / (1.0 + np.exp(-g)))) + 3 * 2.0 ** -8 * np.abs(want) + 2.0 ** -14
    assert (err <= bound).all(), (err - bound).max()


def test_moe_silu_mul_bfloat16_equals_the_two_steps():
    s = SCHEMES["q4f16_1"]
    rng = np.random.default_rng(92)
    ne, n, k = 4, 512, 1280
    w32 = o.round_to((rng.standard_normal((ne, n, k)) * 0.05).astype(np.float32), "bfloat16")
    qw_ref, qs_ref = o.quantize_dt(w32, s, "bfloat16")
    qw, qs = dev(qw_ref), torch.from_numpy(qs_ref).bfloat16().to(DEV)
    x1 = torch.from_numpy(rng.standard_normal((1, k)).astype(np.float32)).bfloat16().to(DEV)
    ids = torch.tensor([[3, 1]], dtype=torch.int32, device=DEV)
    y = ops.moe_gemv(x1, qw, qs, ids, 4, 32, silu_mul_halves=True)
    assert y.dtype == torch.bfloat16 and tuple(y.shape) == (2, n // 2)
    assert torch.equal(y, ops.silu_mul(ops.moe_gemv(x1, qw, qs, ids, 4, 32)))
    for rows, indptr in ((20, [0, 7, 7, 15, 20]), (50, [0, 20, 21, 21, 50]), (100, [0, 40, 41, 41, 100]),
                         (700, [0, 300, 380, 700, 700])):
        x = torch.from_numpy(rng.standard_normal((rows, k)).astype(np.float32)).bfloat16().to(DEV)
        ip = torch.tensor(indptr, dtype=torch.int32, device=DEV)
        y = ops.moe_group_gemm(x, qw, qs, ip, 4, 32, silu_mul_halves=True)
        assert tuple(y.shape) == (rows, n // 2)
        two = ops.silu_mul(ops.moe_group_gemm(x, qw, qs, ip, 4, 32))
        assert torch.equal(y, two), f"rows={rows}: {(y != two).sum().item()} differ"


def test_moe_experts_gather_bfloat16():
    """The gather folded into the expert matmul for a bfloat16 model equals take_rows + moe_group_gemm bit for
    bit (quad-row kernel and GEMM tiles; with and without the folded activation)."""
    s = SCHEMES["q4f16_1"]
    rng = np.random.default_rng(93)
    ne, n, k, t = 4, 256, 1024, 90
    w32 = o.round_to((rng.standard_normal((ne, n, k)) * 0.05).astype(np.float32), "bfloat16")
    qw_ref, qs_ref = o.quantize_dt(w32, s, "bfloat16")
    qw, qs = dev(qw_ref), torch.from_numpy(qs_ref).bfloat16().to(DEV)
    x = torch.from_numpy(rng.standard_normal((t, k)).astype(np.float32)).bfloat16().to(DEV)
    for rows, indptr in ((12, [0, 3, 3, 8, 12]), (60, [0, 20, 21, 21, 60]), (180, [0, 40, 90, 91, 180])):
        idx = torch.from_numpy(rng.integers(0, t, rows).astype(np.int32)).to(DEV)
        ip = torch.tensor(indptr, dtype=torch.int32, device=DEV)
        for fold in (False, True):
            got = ops.moe_experts(x, idx, qw, qs, ip, 4, 32, silu_mul_halves=fold)
            want = ops.moe_group_gemm(ops.take_rows(x, idx), qw, qs, ip, 4, 32, silu_mul_halves=fold)
            assert got.dtype == torch.bfloat16 and torch.equal(got, want), (rows, fold)
    # float32 models have no such kernel: the call still answers, through the two steps
    x32 = x.float()
    qs32 = qs.float()
    idx = torch.arange(12, dtype=torch.int32, device=DEV)
    ip = torch.tensor([0, 3, 3, 8, 12], dtype=torch.int32, device=DEV)
    got = ops.moe_experts(x32, idx, qw, qs32, ip, 4, 32)
    assert got.dtype == torch.float32 and torch.equal(got, ops.moe_group_gemm(x32[:12].contiguous(), qw, qs32, ip, 4, 32))


def test_linear_other_model_dtypes_through_the_modules():
    for name in ("q4f32_1", "q4bf16_1", "q4bf16_0"):
        cfg = gq.QUANTIZATION[name]
        dt = _TORCH_OF[cfg.model_dtype]
        torch.manual_seed(4)
        src = torch.nn.Linear(256, 72, bias=True, device=DEV)
        lin = gq.GroupQuantizeLinear.from_linear(src, cfg)
        qw, qs = cfg.quantize_weight(src.weight.data, output_transpose=cfg.linear_weight_layout == "KN")
        lin.q_weight.data.copy_(qw)
        lin.q_scale.data.copy_(qs)
        lin.bias.data.copy_(src.bias.data.to(dt))
        x = torch.randn(3, 5, 256, device=DEV).to(dt)
        y = lin(x)
        assert y.dtype == dt and tuple(y.shape) == (3, 5, 72)
        nk_w, nk_s = (qw.t().contiguous(), qs.t().contiguous()) if cfg.linear_weight_layout == "KN" else (qw, qs)
        w_deq = cfg.dequantize_weight(nk_w, nk_s, 256)
        want = x.double() @ w_deq.double().t() + lin.bias.double()
        assert (y.double() - want).norm() / want.norm() <= (3e-3 if dt == torch.bfloat16 else 1e-6)
        emb = gq.GroupQuantizeEmbedding(72, 256, cfg, device=DEV)
        emb.q_weight.data.copy_(nk_w)
        emb.q_scale.data.copy_(nk_s)
        logits = emb.lm_head_forward(x)
        assert logits.dtype == torch.float32
        assert (logits.double() - x.double() @ w_deq.double().t()).norm() / want.norm() <= 1e-5


# ------------------------------------------------------------------ gate_up with the activation folded in

def assert_silu_mul_ok(y: torch.Tensor, ref64: np.ndarray, x: np.ndarray, k: int, what=""):
    """y = silu(g) * u against the float64 product of the oracle's matmul: the matmul tolerance,
    carried through d(silu(g) u) <= |u| 1.1 dg + |silu(g)| du, plus the three fp16 roundings."""
    half = ref64.shape[-1] // 2
    g, u = ref64[..., :half], ref64[..., half:]
    silu = g / (1.0 + np.exp(-g))
    tol = o.linear_tolerance(x, k)
    bound = tol * (1.1 * np.abs(u) + np.abs(silu)) + 3 * 2.0 ** -10 * np.abs(silu * u) + 2.0 ** -20
    err = np.abs(y.double().cpu().numpy() - silu * u)
    assert (err <= bound).all(), f"{what}: worst excess {(err - bound).max():.3e}"


@pytest.mark.parametrize("name,m,n,k", [
    ("q4f16_1", 1, 512, 4096), ("q4f16_1", 2, 264, 1024), ("q4f16_1", 1, 2048, 8192),   # register GEMV
    ("q4f16_1", 1, 256, 14336), ("q4f16_1", 2, 128, 8192),                                # long K: declined, GEMM
    ("q4f16_1", 3, 512, 4096), ("q4f16_1", 8, 1032, 2048), ("q4f16_1", 5, 520, 20520),    # quad-row (+ K phases)
    ("q4f16_1", 6, 130, 512), ("q4f16_1", 3, 64, 100), ("q4f16_1", 11, 64, 100),                                                            # N % 4 != 0: GEMM
    ("q4f16_1", 12, 256, 2048), ("q4f16_1", 16, 1032, 4096), ("q4f16_1", 20, 28672, 512), ("q4f16_1", 32, 200, 1024), ("q4f16_1", 32, 192, 1024),
    ("q4f16_1", 24, 512, 8192), ("q4f16_1", 40, 512, 4096), ("q4f16_1", 100, 1024, 1024), # few-row GEMM, split K
    ("q4f16_1", 64, 144, 256), ("q4f16_1", 300, 328, 512), ("q4f16_1", 130, 2, 64),       # gate half not whole blocks
    ("q3f16_1", 1, 512, 4096), ("q3f16_1", 2, 256, 2560), ("q3f16_1", 5, 512, 4080),
    ("q3f16_1", 12, 264, 2000), ("q3f16_1", 40, 512, 4096), ("q3f16_1", 200, 192, 1040),
])
def test_linear_silu_mul_equals_the_two_steps(name, m, n, k):
    s = SCHEMES[name]
    x, qw, qs, _ = _linear_case(s, m, n, k, 1000 + m + n, scale=0.05)
    xd, qwd, qsd = dev(x), dev(qw), dev(qs)
    y = ops.linear_silu_mul(xd, qwd, qsd, s.bits, s.group_size)
    assert tuple(y.shape) == (m, n // 2) and y.dtype == torch.float16
    assert_silu_mul_ok(y, o.linear_fp32(x, qw, qs, s), x, k, f"{name} {m}x{n}x{k}")
    # The fused call walks the same regimes as the plain linear (register GEMV, quad-row, skinny, GEMM)
    # with the same kernels, so the two-step result is reproduced bit for bit.  The one exception: K
    # too long for the register GEMV, where the plain linear has another GEMV and the fused call none;
    # and 17..256 rows with a gate half that is not whole 32-row blocks, where only the plain linear may
    # split K (another summation order).
    ng = -(-k // s.group_size)
    if (m <= 2 and ng > (256 if m == 1 else 128)) or (16 < m <= 256 and n % 64 != 0):
        return
    two = ops.silu_mul(ops.linear(xd, qwd, qsd, s.bits, s.group_size))
    assert torch.equal(y, two), f"{name} {m}x{n}x{k}: {(y != two).sum().item()} of {y.numel()} differ"


@pytest.mark.parametrize("variant,m,n,k", [(6, 200, 384, 512), (7, 300, 640, 384), (9, 200, 768, 256)])
def test_linear_silu_mul_every_gemm_tile(variant, m, n, k):
    s = SCHEMES["q4f16_1"]
    x, qw, qs, _ = _linear_case(s, m, n, k, 77 + variant, scale=0.05)
    xd, qwd, qsd = dev(x), dev(qw), dev(qs)
    gq._lib.set_option("gemm_variant", variant)
    try:
        y = ops.linear_silu_mul(xd, qwd, qsd, 4, 32)
        two = ops.silu_mul(ops.linear(xd, qwd, qsd, 4, 32))
        torch.cuda.synchronize()
    finally:
        gq._lib.set_option("gemm_variant", -1)
    assert_silu_mul_ok(y, o.linear_fp32(x, qw, qs, s), x, k, f"variant {variant}")
    assert torch.equal(y, two)


def test_linear_silu_mul_without_a_fused_kernel_runs_the_two_calls():
    # q3 with K % 8 != 0: the quad-row kernel and the pipelined GEMM both need 16-byte aligned rows of x
    s = SCHEMES["q3f16_1"]
    x, qw, qs, _ = _linear_case(s, 3, 64, 100, 5, scale=0.05)
    xd, qwd, qsd = dev(x), dev(qw), dev(qs)
    out = torch.empty((3, 32), dtype=torch.float16, device=DEV)
    with pytest.raises(gq._lib.Mi355gqError) as e:
        gq._lib.call("mi355gq_linear_silu_mul", xd.data_ptr(), qwd.data_ptr(), qsd.data_ptr(), 3, 64, 100, 3, 40,
                     out.data_ptr(), None, 0, None)
    assert e.value.code == gq._lib.ERR_UNSUPPORTED
    with pytest.raises(gq._lib.Mi355gqError) as e:  # odd N is an argument error, not a missing kernel
        gq._lib.call("mi355gq_linear_silu_mul", xd.data_ptr(), qwd.data_ptr(), qsd.data_ptr(), 3, 63, 80, 3, 40,
                     out.data_ptr(), None, 0, None)
    assert e.value.code == gq._lib.ERR_ARG
    y = ops.linear_silu_mul(xd, qwd, qsd, 3, 40)
    assert torch.equal(y, ops.silu_mul(ops.linear(xd, qwd, qsd, 3, 40)))
    assert_silu_mul_ok(y, o.linear_fp32(x, qw, qs, s), x, 100, "q3 K=100")


@pytest.mark.parametrize("name", ["q4f16_1", "q3f16_1"])
def test_moe_experts_silu_mul_equals_the_two_steps(name):
    s = SCHEMES[name]
    rng = np.random.default_rng(91)
    ne, n, k = 4, 512, 1280
    w = (rng.standard_normal((ne, n, k)) * 0.05).astype(np.float16)
    qw, qs = o.quantize(w, s)
    qwd, qsd = dev(qw), dev(qs)
    # single token: the selected experts' GEMV
    x1 = rng.standard_normal((1, k)).astype(np.float16)
    ids = torch.tensor([[3, 1]], dtype=torch.int32, device=DEV)
    y = ops.moe_gemv(dev(x1), qwd, qsd, ids, s.bits, s.group_size, silu_mul_halves=True)
    assert tuple(y.shape) == (2, n // 2)
    assert torch.equal(y, ops.silu_mul(ops.moe_gemv(dev(x1), qwd, qsd, ids, s.bits, s.group_size)))
    for e_slot, e in enumerate((3, 1)):
        assert_silu_mul_ok(y[e_slot:e_slot + 1], o.linear_fp32(x1, qw[e], qs[e], s), x1, k, f"moe_gemv {name}")
    # grouped: few rows (quad-row kernel), more rows (GEMM)
    # (50 and 100 rows: the GEMM's 32- and 64-row grouped tiles)
    for rows, indptr, gemm_only in ((20, [0, 7, 7, 15, 20], False), (50, [0, 20, 21, 21, 50], False),
                                    (100, [0, 40, 41, 41, 100], False),
                                    (150, [0, 40, 41, 41, 150], False), (700, [0, 300, 380, 700, 700], False)):
        x = rng.standard_normal((rows, k)).astype(np.float16)
        ip = torch.tensor(indptr, dtype=torch.int32, device=DEV)
        y = ops.moe_group_gemm(dev(x), qwd, qsd, ip, s.bits, s.group_size, silu_mul_halves=True)
        assert tuple(y.shape) == (rows, n // 2)
        if gemm_only:
            gq._lib.set_option("gemm_variant", 1)
        try:
            two = ops.silu_mul(ops.moe_group_gemm(dev(x), qwd, qsd, ip, s.bits, s.group_size))
            torch.cuda.synchronize()
        finally:
            gq._lib.set_option("gemm_variant", -1)
        assert torch.equal(y, two), f"{name} rows={rows}: {(y != two).sum().item()} differ"
        ref = o.dequantize_group_gemm_fp32(x, qw, qs, np.asarray(indptr, dtype=np.int32), s)
        assert_silu_mul_ok(y, ref, x, k, f"group gemm {name} rows={rows}")


def _op_by_op_layer(moe, x, gate):
    """MixtralMoE.forward as the reference writes it (mixtral_model.py:77-117), one call per op."""
    from mlc_llm_amd.op import moe_misc
    t = x.shape[0] * x.shape[1]
    h = x.shape[2]
    xx = x.reshape(t, h).contiguous()
    w, ids = moe_misc.gating_softmax_topk(gate, moe.num_experts_per_tok)
    if t == 1:
        y = moe.e2(ops.silu_mul(moe.e1_e3(xx, ids)), ids)
    else:
        cumsum = moe_misc.moe_cumsum(ids, moe.num_local_experts)
        rev, tok = moe_misc.get_indices(cumsum, ids)
        indptr = moe_misc.get_indptr(cumsum, moe.num_local_experts, t, inclusive=False, out_dtype="int32")
        y = moe.e2(ops.silu_mul(moe.e1_e3(ops.take_rows(xx, tok), indptr)), indptr)
        y = moe_misc.scatter_output(y, rev)
    return ops.moe_combine(y.reshape(t, moe.num_experts_per_tok, h), w).reshape(x.shape)


def test_mixtral_moe_layer_fused_forms_change_no_bit():
    # folded activation, fused routing, gather in the matmul, scatter in the combine: same output as the
    # op-by-op sequence, for a single token, few tokens (quad-row), more (skinny) and many (GEMM)
    from mlc_llm_amd.nn.mixtral_moe import MixtralMoE
    s = gq.QUANTIZATION["q4f16_1"]
    torch.manual_seed(3)
    moe = MixtralMoE(256, 384, 4, 2, s, device=DEV)
    for p_ in (moe.e1_e3, moe.e2):
        w = (torch.randn(p_.num_local_experts, p_.out_features, p_.in_features, device=DEV) * 0.05).half()
        qw, qs = ops.quantize(w, 4, 32)
        p_.q_weight.data.copy_(qw)
        p_.q_scale.data.copy_(qs)
    for t in (1, 2, 9, 40, 300, 1500):
        x = torch.randn(1, t, 256, device=DEV).half()
        gate = torch.randn(t, 4, device=DEV).half()
        assert torch.equal(moe(x, gate), _op_by_op_layer(moe, x, gate)), t


@pytest.mark.parametrize("t,ne,k", [(2, 8, 2), (9, 8, 2), (100, 4, 1), (1000, 8, 2), (1500, 8, 4), (5000, 6, 2),
                                    (64, 64, 8), (3, 3, 3)])
def test_moe_route_equals_the_four_calls(t, ne, k):
    torch.manual_seed(t + ne + k)
    logits = torch.randn(t, ne, device=DEV).half()
    w, ids, tok, rev, pos, indptr = ops.moe_route(logits, k)
    w0, ids0 = ops.gating_softmax_topk(logits, k)
    cumsum = ops.moe_cumsum(ids0, ne)
    rev0, tok0 = ops.get_indices(cumsum, ids0)
    indptr0 = ops.get_indptr(cumsum, ne, t, inclusive=False)
    assert torch.equal(w, w0) and torch.equal(ids, ids0)
    assert torch.equal(tok, tok0) and torch.equal(rev, rev0) and torch.equal(indptr, indptr0)
    assert torch.equal(rev[pos.long()], torch.arange(t * k, dtype=torch.int32, device=DEV))  # the inverse permutation
    assert torch.equal(ops.moe_route(logits, k, torch.int64)[5], indptr0.long())


@pytest.mark.parametrize("t,ne,k", [(1, 64, 8), (2, 64, 8), (16, 64, 8), (17, 60, 4), (200, 64, 6), (1024, 64, 8),
                                    (40, 160, 6), (3, 256, 8), (5, 200, 8), (1100, 33, 7), (7, 65, 1),
                                    (2, 128, 8), (512, 128, 8), (100, 256, 2)])
def test_many_expert_routing_against_oracle(t, ne, k):
    """Many experts or many slots: the top-k runs one wave per token and the route step by slot.  Logits
    drawn from a few values so that ties abound, plus rows that cannot fill their k slots."""
    rng = np.random.default_rng(t * 1000 + ne + k)
    logits = rng.standard_normal((t, ne)).astype(np.float16)
    logits[::3] = rng.integers(-3, 4, logits[::3].shape).astype(np.float16)  # ties: the lower index first
    logits[-1, :] = np.float16(-65504.0)  # nothing exceeds min_value: every slot stays (min_value, expert 0)
    if t > 2:
        logits[1, :] = -np.inf
        logits[1, ne // 2] = 1.0  # one placeable logit
    w_ref, ids_ref = o.gating_softmax_topk(logits, k)
    w, ids = ops.gating_softmax_topk(dev(logits), k)
    assert (ids.cpu().numpy() == ids_ref).all()
    dw = np.abs(w.cpu().numpy().astype(np.float32) - w_ref.astype(np.float32))
    assert (dw <= 2.0**-11).all(), dw.max()  # one fp16 ulp between libms, as for the golden vectors
    if ne * ((t * k + 63) // 64) <= 8192:  # the one-launch route step covers the shape
        w2, ids2, tok, rev, pos, indptr = ops.moe_route(dev(logits), k)
        assert torch.equal(w2, w) and torch.equal(ids2, ids)
        cs_ref = o.moe_cumsum(ids_ref, ne)
        rev_ref, tok_ref = o.get_indices(cs_ref, ids_ref)
        n_pairs = int(cs_ref.reshape(-1)[-1])  # rows with repeated ids leave the tail of the order unwritten
        indptr_ref = o.get_indptr(cs_ref, ne, t, inclusive=False)
        assert (indptr.cpu().numpy() == indptr_ref).all()
        tok_h, rev_h = tok.cpu().numpy()[:n_pairs], rev.cpu().numpy()[:n_pairs]
        assert (tok_h == tok_ref[:n_pairs]).all() and (rev_h // k == tok_h).all()
        distinct = np.array([len(set(row)) == k for row in ids_ref.tolist()])[tok_h]  # a repeated id counts once,
        assert (rev_h[distinct] == rev_ref[:n_pairs][distinct]).all()  # under its first slot here
        assert (ids_ref.reshape(-1)[rev_h] == np.repeat(np.arange(ne), np.diff(indptr_ref))).all()
        assert torch.equal(pos[rev[:n_pairs].long()], torch.arange(n_pairs, dtype=torch.int32, device=DEV))


def test_moe_route_past_one_workgroup_is_unsupported():
    for t, ne in ((9000, 8), (5000, 128), (4097, 32)):
        with pytest.raises(gq._lib.Mi355gqError) as e:
            ops.moe_route(torch.zeros(t, ne, device=DEV).half(), 2)
        assert e.value.code == gq._lib.ERR_UNSUPPORTED


@pytest.mark.parametrize("name", ["q4f16_1", "q3f16_1"])
def test_moe_experts_with_the_gather_folded_in(name):
    s = SCHEMES[name]
    rng = np.random.default_rng(17)
    ne, n, k, t = 4, 256, 640, 37
    w = (rng.standard_normal((ne, n, k)) * 0.05).astype(np.float16)
    qw, qs = o.quantize(w, s)
    qwd, qsd = dev(qw), dev(qs)
    x = dev(rng.standard_normal((t, k)).astype(np.float16))
    for rows, indptr in ((20, [0, 7, 7, 15, 20]), (100, [0, 40, 41, 41, 100]), (700, [0, 300, 380, 700, 700])):
        idx = torch.from_numpy(rng.integers(0, t, rows).astype(np.int32)).to(DEV)
        ip = torch.tensor(indptr, dtype=torch.int32, device=DEV)
        gathered = ops.take_rows(x, idx)
        for silu in (False, True):
            got = ops.moe_experts(x, idx, qwd, qsd, ip, s.bits, s.group_size, silu)
            want = ops.moe_group_gemm(gathered, qwd, qsd, ip, s.bits, s.group_size, silu)
            assert torch.equal(got, want), (name, rows, silu)
            assert torch.equal(ops.moe_experts(gathered, None, qwd, qsd, ip, s.bits, s.group_size, silu), want)
    # an index outside x is clamped, never followed
    bad = torch.tensor([0, -5, 36, 99, 2**30], dtype=torch.int32, device=DEV)
    ip = torch.tensor([0, 5, 5, 5, 5], dtype=torch.int32, device=DEV)
    got = ops.moe_experts(x, bad, qwd, qsd, ip, s.bits, s.group_size)
    ok = torch.tensor([0, 0, 36, 36, 36], dtype=torch.int32, device=DEV)
    assert torch.equal(got, ops.moe_group_gemm(ops.take_rows(x, ok), qwd, qsd, ip, s.bits, s.group_size))


def test_moe_combine_sorted_equals_scatter_then_combine():
    torch.manual_seed(5)
    t, k, h = 33, 2, 192
    logits = torch.randn(t, 8, device=DEV).half()
    w, ids, tok, rev, pos, indptr = ops.moe_route(logits, k)
    y = torch.randn(t * k, h, device=DEV).half()
    want = ops.moe_combine(ops.scatter_output(y, rev).reshape(t, k, h), w)
    assert torch.equal(ops.moe_combine_sorted(y, pos, w), want)


# ------------------------------------------------------------------ degenerate and hostile inputs

def test_degenerate_sizes_every_entry_point():
    s = SCHEMES["q4f16_1"]
    x, qw, qs, _ = _linear_case(s, 3, 8, 64, 5)
    xd, qwd, qsd = dev(x), dev(qw), dev(qs)
    # no rows / no columns: nothing is launched, shapes come back right
    assert tuple(ops.linear(xd[:0], qwd, qsd, 4, 32).shape) == (0, 8)
    assert tuple(ops.linear(xd, qwd[:0], qsd[:0], 4, 32).shape) == (3, 0)
    q0, s0 = ops.quantize(torch.empty((0, 64), dtype=torch.float16, device=DEV), 4, 32)
    assert tuple(q0.shape) == (0, 8) and tuple(s0.shape) == (0, 2)
    assert tuple(ops.dequantize(qwd[:0], qsd[:0], 64, 4, 32).shape) == (0, 64)
    # K = 0: the product is the bias
    b = dev(np.arange(8, dtype=np.float16))
    y = ops.linear(torch.empty((3, 0), dtype=torch.float16, device=DEV), qwd[:, :0].contiguous(),
                   qsd[:, :0].contiguous(), 4, 32, b)
    assert torch.equal(y, b.expand(3, 8))
    res = dev(np.random.default_rng(1).standard_normal((3, 8)).astype(np.float16))
    xe = torch.empty((3, 0), dtype=torch.float16, device=DEV)
    for m in (1, 3, 12, 40):  # one per kernel regime: each hands K = 0 to the same fill
        yr = ops.linear(xe[:1].expand(m, 0).contiguous(), qwd[:, :0].contiguous(), qsd[:, :0].contiguous(), 4, 32, b,
                        out_dtype=torch.float32, residual=res[:1].expand(m, 8).contiguous())
        assert torch.equal(yr, (b.float() + res[:1].float()).expand(m, 8))
    ew, es = torch.zeros((4, 8, 0), dtype=torch.int32, device=DEV), torch.zeros((4, 8, 0), dtype=torch.float16, device=DEV)
    eids = torch.tensor([[0, 3]], dtype=torch.int32, device=DEV)
    assert torch.equal(ops.moe_gemv(xe[:1], ew, es, eids, 4, 32), torch.zeros((2, 8), dtype=torch.float16, device=DEV))
    ip = torch.tensor([0, 1, 1, 2, 3], dtype=torch.int32, device=DEV)
    assert torch.equal(ops.moe_group_gemm(xe, ew, es, ip, 4, 32), torch.zeros((3, 8), dtype=torch.float16, device=DEV))
    # routing with no tokens
    w, ids = ops.gating_softmax_topk(torch.empty((0, 8), dtype=torch.float16, device=DEV), 2)
    assert tuple(w.shape) == (0, 2) and tuple(ids.shape) == (0, 2)
    # grouped matmul where every expert is empty
    eqw = torch.zeros((4, 8, 8), dtype=torch.int32, device=DEV)
    eqs = torch.zeros((4, 8, 2), dtype=torch.float16, device=DEV)
    out = ops.moe_group_gemm(torch.empty((0, 64), dtype=torch.float16, device=DEV), eqw, eqs,
                             torch.zeros(5, dtype=torch.int32, device=DEV), 4, 32)
    assert tuple(out.shape) == (0, 8)


def test_hostile_indices_stay_inside_the_tensors():
    # ids outside the table, expert ids outside the experts and a scrambled indptr are clamped:
    # results for the valid entries are right and nothing outside the buffers is touched
    s = SCHEMES["q4f16_1"]
    rng = np.random.default_rng(8)
    w = (rng.standard_normal((3, 16, 64)) * 0.05).astype(np.float16)
    qw, qs = o.quantize(w, s)
    table_w, table_s = dev(qw[0]), dev(qs[0])
    ids = torch.tensor([0, 15, -7, 16, 2**30], dtype=torch.int32, device=DEV)
    emb = ops.embedding_take(ids, table_w, table_s, 64, 4, 32)
    ref = o.dequantize(qw[0], qs[0], s, 64)
    assert np.array_equal(host_f16_bits(emb[:2]), ref[[0, 15]].view(np.uint16))
    assert np.array_equal(host_f16_bits(emb[2:]), ref[[0, 15, 15]].view(np.uint16))  # clamped into the table
    x = rng.standard_normal((1, 64)).astype(np.float16)
    eids = torch.tensor([[1, 9]], dtype=torch.int32, device=DEV)  # 9 is past the 3 experts: clamped to 2
    y = ops.moe_gemv(dev(x), dev(qw), dev(qs), eids, 4, 32)
    assert_linear_ok(y[0:1], o.linear_fp32(x, qw[1], qs[1], s), x, 64, "expert 1")
    assert_linear_ok(y[1:2], o.linear_fp32(x, qw[2], qs[2], s), x, 64, "expert id clamped")
    xs = rng.standard_normal((6, 64)).astype(np.float16)
    # decreasing, then past the rows: read as [0,4) [4,4) [2,6), so rows 2..3 belong to two experts
    # (either may win) and the others to exactly one
    bad_ip = torch.tensor([0, 4, 2, 99], dtype=torch.int32, device=DEV)
    out = ops.moe_group_gemm(dev(xs), dev(qw), dev(qs), bad_ip, 4, 32)
    torch.cuda.synchronize()
    assert tuple(out.shape) == (6, 16) and torch.isfinite(out.float()).all()
    assert_linear_ok(out[:2], o.linear_fp32(xs[:2], qw[0], qs[0], s), xs[:2], 64, "rows of the first segment only")
    assert_linear_ok(out[4:], o.linear_fp32(xs[4:], qw[2], qs[2], s), xs[4:], 64, "rows of the clamped last segment")


@pytest.mark.parametrize("model_dtype", ["float32", "bfloat16"])
def test_hostile_indices_other_model_dtypes(model_dtype):
    # the same clamping in the expert matmuls of the float32 / bfloat16 models
    s = SCHEMES["q4f16_1"]
    dt = _TORCH_OF[model_dtype]
    rng = np.random.default_rng(9)
    w32 = o.round_to((rng.standard_normal((3, 16, 64)) * 0.05).astype(np.float32), model_dtype)
    qw_ref, qs_ref = o.quantize_dt(w32, s, model_dtype)
    qw, qs = dev(qw_ref), torch.from_numpy(qs_ref).to(dt).to(DEV)
    x32 = o.round_to(rng.standard_normal((1, 64)).astype(np.float32), model_dtype)
    eids = torch.tensor([[-4, 9]], dtype=torch.int32, device=DEV)  # clamped to experts 0 and 2
    y = ops.moe_gemv(torch.from_numpy(x32).to(dt).to(DEV), qw, qs, eids, 4, 32)
    ref = o.moe_dequantize_gemv_dt_fp64(x32, qw_ref, qs_ref, np.array([[0, 2]], np.int32), s, model_dtype)
    _assert_dt_matmul_ok(y, ref, x32, 64, model_dtype, "expert ids clamped")
    for rows in (6, 70):  # the dot-product kernel's segments and the tiled kernels' row tiles
        xs32 = o.round_to(rng.standard_normal((rows, 64)).astype(np.float32), model_dtype)
        bad_ip = torch.tensor([0, 4, 2, 9999], dtype=torch.int32, device=DEV)  # read as [0,4) [4,4) [2,rows)
        out = ops.moe_group_gemm(torch.from_numpy(xs32).to(dt).to(DEV), qw, qs, bad_ip, 4, 32)
        torch.cuda.synchronize()
        assert tuple(out.shape) == (rows, 16) and torch.isfinite(out.float()).all()
        full = o.dequantize_group_gemm_dt_fp64(xs32, qw_ref, qs_ref, np.array([0, 2, 2, rows], np.int32), s, model_dtype)
        _assert_dt_matmul_ok(out[:2], full[:2], xs32[:2], 64, model_dtype, "rows of the first segment only")
        _assert_dt_matmul_ok(out[4:], full[4:], xs32[4:], 64, model_dtype, "rows of the clamped last segment")


# ------------------------------------------------------------------ HIP graph capture

def test_linear_and_moe_replay_in_hip_graph():
    # every regime of the dispatcher recorded into one graph; each replay (with new activations
    # written in place, and eager work between replays) must equal the eager result bit for bit
    s = SCHEMES["q4f16_1"]
    rng = np.random.default_rng(77)
    n, k = 264, 4096
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float16)
    qw, qs = o.quantize(w, s)
    qw_d, qs_d = dev(qw), dev(qs)
    ms = [1, 2, 4, 8, 16, 40, 300]  # GEMV, GEMV, quad-row x2, skinny, few-row split-K GEMM, GEMM
    xs = [torch.zeros((m, k), dtype=torch.float16, device="cuda:0") for m in ms]
    outs = [torch.empty((m, n), dtype=torch.float16, device="cuda:0") for m in ms]
    wss = [torch.empty(max(16, gq._lib.lib().mi355gq_linear_workspace_bytes(m, n, k, 4, 32)), dtype=torch.uint8,
                       device="cuda:0") for m in ms]

    def run_all():
        for m, x, out, ws in zip(ms, xs, outs, wss):
            gq._lib.call("mi355gq_linear", x.data_ptr(), qw_d.data_ptr(), qs_d.data_ptr(), None, m, n, k, 4, 32,
                         gq._lib.F16, out.data_ptr(), ws.data_ptr(), ws.numel(),
                         torch.cuda.current_stream().cuda_stream)

    run_all()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        run_all()
    for rep in range(3):
        for x in xs:
            x.copy_(torch.from_numpy(rng.standard_normal(tuple(x.shape)).astype(np.float16)))
        graph.replay()
        torch.cuda.synchronize()
        replayed = [out.clone() for out in outs]
        for out in outs:
            out.zero_()
        run_all()  # eager, same inputs
        torch.cuda.synchronize()
        for m, a, b in zip(ms, replayed, outs):
            assert torch.equal(a, b), f"graph replay {rep} differs from eager at M={m}"
        ref = o.linear_fp32(xs[-2].cpu().numpy(), qw, qs, s)
        assert_linear_ok(replayed[-2], ref, xs[-2].cpu().numpy(), k, f"replay {rep}, M=40")


# ------------------------------------------------------------------ the C ABI from plain C

def test_c_abi_from_plain_c():
    # tests/c_abi/c_abi_check.c: no Python, no torch; quantize + linear in three regimes against the C oracle
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.abspath(__file__)), "c_abi", "c_abi_check")
    assert os.path.exists(exe), f"{exe} is missing: run __graft_entry__.build() (or make -C tests/c_abi)"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=100)
    assert r.returncode == 0, f"exit {r.returncode}\n{r.stdout}\n{r.stderr}"
    assert "c_abi_check ok" in r.stdout


# ------------------------------------------------------------------ tiny K, gating_topk, norm_topk_prob=False

@pytest.mark.parametrize("name", ["q4f16_1", "q3f16_1"])
@pytest.mark.parametrize("k", [1, 3, 7, 8, 9])
@pytest.mark.parametrize("m", [1, 2, 5])
def test_linear_tiny_k(name, k, m):
    # fewer than 8 halves per activation row: the register GEMV (whole 16-byte loads of x) must decline
    s = SCHEMES[name]
    # (no bias: the bound scales with sqrt(K) and would sit below the fp16 rounding of an O(1) output)
    x, qw, qs, _ = _linear_case(s, m, 24, k, 31 * k + m)
    xd = torch.empty(m * k + 64, dtype=torch.float16, device=DEV)[: m * k].view(m, k)
    xd.copy_(dev(x))
    y = ops.linear(xd, dev(qw), dev(qs), s.bits, s.group_size)
    assert_linear_ok(y, o.linear_fp32(x, qw, qs, s), x, k, f"tiny K {name} k={k} m={m}")


def _ulp16(a, b):
    def line(v):
        u = np.asarray(v, np.float16).view(np.uint16).astype(np.int64)
        return np.where(u & 0x8000, -(u & 0x7FFF), u)
    return np.abs(line(a) - line(b))


@pytest.mark.parametrize("t,ne,k", [(1, 8, 2), (16, 8, 2), (512, 8, 2), (70, 64, 6), (33, 6, 3), (5, 200, 8)])
def test_gating_topk_bit_exact(t, ne, k):
    # moe_misc.py:63-132: scores pass through, ties keep the lower index
    rng = np.random.default_rng(seed_of("topk", t, ne, k))
    sc = rng.random((t, ne)).astype(np.float16)
    sc[0, :] = 0.5
    if t > 2:
        sc[2, ne // 2:] = sc[2, : ne - ne // 2]
    v_ref, i_ref = o.gating_topk(sc, k)
    v, i = ops.gating_topk(dev(sc), k)
    assert np.array_equal(i.cpu().numpy(), i_ref)
    assert np.array_equal(host_f16_bits(v), v_ref.view(np.uint16))


@pytest.mark.parametrize("t,ne,k", [(1, 8, 2), (16, 8, 2), (512, 8, 2), (70, 64, 6), (257, 60, 4)])
def test_gating_softmax_topk_without_renormalisation(t, ne, k):
    """norm_topk_prob=False (moe_misc.py:234-235): softmax over all experts in fp32, cast, top-k of the rounded
    scores.  The device's exp differs from numpy's in the last place of fp32, which can move a score across an
    fp16 rounding boundary (one unit) and with it a near tie; so: weights within one unit of the oracle's score of
    the chosen expert, the choice a valid top-k of scores within one unit, and, on rows whose k + 1 best scores
    lie more than three units apart, exactly the oracle's experts in the oracle's order."""
    rng = np.random.default_rng(seed_of("full", t, ne, k))
    logits = rng.standard_normal((t, ne)).astype(np.float16)
    logits[0, :] = 1.0          # exact ties are exact on both sides: 1 / ne each, experts 0 .. k-1
    w_ref, i_ref = o.gating_softmax_topk_full(logits, k)
    w, i = ops.gating_softmax_topk(dev(logits), k, norm_topk_prob=False)
    w, i = w.cpu().numpy(), i.cpu().numpy()
    assert i[0].tolist() == list(range(k)) and np.array_equal(w[0], w_ref[0])
    p16 = o.softmax_fp32(logits.astype(np.float32)).astype(np.float16)
    line = lambda v: int(np.float16(v).view(np.uint16))  # positive scores: the bit pattern is monotone
    exact_rows = 0
    for r in range(t):
        chosen = i[r]
        assert len(set(chosen.tolist())) == k
        assert _ulp16(w[r], p16[r, chosen]).max() <= 1
        rest = np.setdiff1d(np.arange(ne), chosen)
        # nothing left out beats the last one chosen by more than the one-unit slack on either side
        if rest.size:
            assert max(line(p16[r, e]) for e in rest) <= line(w[r, -1]) + 2
        assert all(line(w[r, j]) >= line(w[r, j + 1]) for j in range(k - 1))
        top = np.sort(p16[r].astype(np.float64))[::-1][: k + 1]
        bits = np.array([line(v) for v in top])
        if (bits[:-1] - bits[1:] > 3).all():
            exact_rows += 1
            assert chosen.tolist() == i_ref[r].tolist(), r
    assert exact_rows >= t // 2 or ne > 32
    # the float32 / bfloat16 forms run the same kernel with their own rounding
    for tdt, md in ((torch.float32, "float32"), (torch.bfloat16, "bfloat16")):
        lg = torch.from_numpy(logits.astype(np.float32)).to(DEV).to(tdt)
        w2, i2 = ops.gating_softmax_topk(lg, k, norm_topk_prob=False)
        w2_ref, i2_ref = o.gating_softmax_topk_full(lg.float().cpu().numpy(), k, md)
        same = (i2.cpu().numpy() == i2_ref).all(axis=1)
        assert same.mean() >= (0.97 if md == "float32" else 0.8)
        np.testing.assert_allclose(w2.float().cpu().numpy()[same], w2_ref[same], rtol=2.0 ** -7 if md == "bfloat16" else 1e-5)
