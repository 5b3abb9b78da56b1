"""The benchmark definition's configurations at their full sizes, through the C ABI, against the CPU oracle.

The oracle cannot multiply a 128256 x 4096 matrix by 8192 rows in seconds, but weight rows (output columns) and
activation rows are independent of each other in every operator here, so the oracle is run on a sample of both:
first and last rows, the rows either side of every tile boundary the kernels use, and random ones.  Packed words
and scales of the sampled rows are copied from the device tensor the kernel read, so the check does not depend on
the quantizer (whose bits other tests compare with the oracle).  Bars as everywhere: integer results bit-exact,
matmul outputs within max|err| <= 1e-2 * max|x| * sqrt(K) / 64 and rel-L2 <= 2e-3 of the float64-summed
dequantize-then-matmul.
"""

import numpy as np
import pytest
import torch

import mlc_llm_amd as gq
from mlc_llm_amd import ops
from oracle import c_oracle
from oracle import gq_oracle as o

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
Q4, Q3 = o.SCHEMES["q4f16_1"], o.SCHEMES["q3f16_1"]
LLAMA3 = {"qkv": (6144, 4096), "o_proj": (4096, 4096), "gate_up": (28672, 4096), "down": (4096, 14336),
          "lm_head": (128256, 4096)}
LLAMA2_Q3 = {"qkv": (12288, 4096), "o_proj": (4096, 4096), "gate_up": (22016, 4096), "down": (4096, 11008)}

_cache = {}


def _weights(scheme, n, k, seed):
    """(q_weight, q_scale) on the device, N(0, 0.02) fp16 weights quantised by the library; kept for the module."""
    key = (scheme.name, n, k, seed)
    if key not in _cache:
        if len(_cache) >= 3:  # a handful of GiB at most
            _cache.pop(next(iter(_cache)))
        g = torch.Generator(device=DEV).manual_seed(seed)
        w = (torch.randn((n, k), generator=g, device=DEV) * 0.02).half()
        _cache[key] = ops.quantize(w, scheme.bits, scheme.group_size)
        del w
    return _cache[key]


def _sample(count, total, rng, edges=(16, 32, 64, 128, 256)):
    """Indices in [0, total): both ends, both sides of every multiple of the tile sizes near the ends and a few
    in the middle, and random ones up to `count`."""
    pick = {0, total - 1}
    for e in edges:
        for base in (e, 2 * e, (total // 2) // e * e, (total - 1) // e * e):
            for d in (-1, 0, 1):
                if 0 <= base + d < total:
                    pick.add(base + d)
    pick = sorted(pick)
    if len(pick) > count:
        keep = rng.choice(len(pick), count, replace=False)
        pick = sorted({pick[i] for i in keep} | {0, total - 1})
    extra = count - len(pick)
    if extra > 0 and total > len(pick):
        pick = sorted(set(pick) | set(rng.choice(total, min(extra, total), replace=False).tolist()))
    return np.array(pick, np.int64)


def _check_sampled(y, x, qw, qs, scheme, rng, what, n_cols=512, n_rows=24, bias=None):
    """y [M, N] on the device against the oracle on sampled activation rows x sampled weight rows."""
    m, k = x.shape
    n = qw.shape[0]
    cols = _sample(min(n_cols, n), n, rng)
    rows = np.arange(m) if m <= n_rows else _sample(n_rows, m, rng)
    ct, rt = torch.from_numpy(cols).to(DEV), torch.from_numpy(rows).to(DEV)
    qw_h = qw[ct].cpu().numpy().view(np.uint32)
    qs_h = qs[ct].cpu().numpy()
    x_h = x[rt].cpu().numpy()
    got = y[rt][:, ct].float().cpu().numpy()
    b_h = bias[ct].cpu().numpy() if bias is not None else None
    ref = o.linear_fp32(x_h, qw_h, qs_h, scheme, b_h)
    err, bound, rel = o.check_linear(got, ref, x_h, k)
    assert err <= bound, f"{what}: max abs err {err:.3e} > bound {bound:.3e}"
    assert rel <= 2e-3, f"{what}: rel-L2 {rel:.3e}"


# ------------------------------------------------------------------ configs[1]: q4f16_1 decode linears, B in {1, 4, 8}

@pytest.mark.parametrize("b", [1, 4, 8])
@pytest.mark.parametrize("name", list(LLAMA3))
def test_llama3_decode_linears(name, b):
    n, k = LLAMA3[name]
    qw, qs = _weights(Q4, n, k, 11)
    rng = np.random.default_rng(n + k + b)
    x = torch.randn((b, k), generator=torch.Generator(device=DEV).manual_seed(b), device=DEV).half()
    y = ops.linear(x, qw, qs, 4, 32)
    _check_sampled(y, x, qw, qs, Q4, rng, f"{name} {n}x{k} B={b}", n_cols=768)
    if name == "lm_head":  # GroupQuantizeEmbedding.lm_head_forward: float32 logits
        y32 = ops.linear(x, qw, qs, 4, 32, None, torch.float32)
        assert y32.dtype == torch.float32
        _check_sampled(y32, x, qw, qs, Q4, rng, f"lm_head fp32 logits B={b}", n_cols=768)


# ------------------------------------------------------------------ configs[2]: q4f16_1 prefill GEMM, M in {256, 2048, 8192}

@pytest.mark.parametrize("m", [256, 2048, 8192])
@pytest.mark.parametrize("name", list(LLAMA3))
def test_llama3_prefill_gemm(name, m):
    n, k = LLAMA3[name]
    qw, qs = _weights(Q4, n, k, 11)
    rng = np.random.default_rng(n + k + m)
    x = torch.randn((m, k), generator=torch.Generator(device=DEV).manual_seed(m), device=DEV).half()
    y = ops.linear(x, qw, qs, 4, 32)
    _check_sampled(y, x, qw, qs, Q4, rng, f"{name} {n}x{k} M={m}", n_cols=512, n_rows=40)
    del y


# ------------------------------------------------------------------ configs[3]: q3f16_1 decode GEMV, Llama-2-7B shapes

@pytest.mark.parametrize("b", [1, 4, 8])
@pytest.mark.parametrize("name", list(LLAMA2_Q3))
def test_llama2_q3_decode_linears(name, b):
    n, k = LLAMA2_Q3[name]
    qw, qs = _weights(Q3, n, k, 13)
    assert tuple(qw.shape) == (n, Q3.num_storage(k)) and tuple(qs.shape) == (n, Q3.num_group(k))
    rng = np.random.default_rng(n + k + b)
    x = torch.randn((b, k), generator=torch.Generator(device=DEV).manual_seed(b + 50), device=DEV).half()
    y = ops.linear(x, qw, qs, 3, 40)
    _check_sampled(y, x, qw, qs, Q3, rng, f"q3 {name} {n}x{k} B={b}", n_cols=768)


@pytest.mark.parametrize("name", ["qkv", "gate_up"])
def test_llama2_q3_prefill_gemm(name):
    n, k = LLAMA2_Q3[name]
    qw, qs = _weights(Q3, n, k, 13)
    rng = np.random.default_rng(n + k)
    x = torch.randn((2048, k), generator=torch.Generator(device=DEV).manual_seed(77), device=DEV).half()
    y = ops.linear(x, qw, qs, 3, 40)
    _check_sampled(y, x, qw, qs, Q3, rng, f"q3 {name} M=2048", n_cols=384, n_rows=32)


# ------------------------------------------------------------------ every row regime at full size, against the oracle

@pytest.mark.parametrize("scheme,n,k", [(Q4, 28672, 4096), (Q4, 4096, 14336), (Q3, 22016, 4096), (Q3, 4096, 11008)],
                         ids=["q4-gate_up", "q4-down", "q3-gate_up", "q3-down"])
def test_every_row_regime_at_full_size_against_the_oracle(scheme, n, k):
    """gate_up and down_proj at their real sizes through every regime of the dispatcher (1 .. 2048 rows): sampled
    rows spread over the batch (first, last, either side of the tile boundaries) x sampled weight rows."""
    qw, qs = _weights(scheme, n, k, 17)
    rng = np.random.default_rng(n * 3 + k)
    xall = torch.randn((2048, k), generator=torch.Generator(device=DEV).manual_seed(5), device=DEV).half()
    for m in (1, 2, 3, 4, 8, 9, 16, 17, 32, 33, 64, 128, 129, 256, 300, 1024, 2048):
        x = xall[:m].contiguous()
        y = ops.linear(x, qw, qs, scheme.bits, scheme.group_size)
        _check_sampled(y, x, qw, qs, scheme, rng, f"{scheme.name} {n}x{k} M={m}", n_cols=256, n_rows=20)


# ------------------------------------------------------------------ configs[4]: Mixtral-8x7B MoE layer, T in {1, 16, 512}

NE, TOPK, H, INTER = 8, 2, 4096, 14336


@pytest.fixture(scope="module")
def mixtral():
    from mlc_llm_amd.nn import MixtralMoE

    _cache.clear()
    moe = MixtralMoE(H, INTER, NE, TOPK, gq.QUANTIZATION["q4f16_1"], device=DEV)
    for e in range(NE):
        g = torch.Generator(device=DEV).manual_seed(7000 + e)
        w13 = (torch.randn((2 * INTER, H), generator=g, device=DEV) * 0.02).half()
        moe.e1_e3.q_weight.data[e], moe.e1_e3.q_scale.data[e] = ops.quantize(w13, 4, 32)
        w2 = (torch.randn((H, INTER), generator=g, device=DEV) * 0.02).half()
        moe.e2.q_weight.data[e], moe.e2.q_scale.data[e] = ops.quantize(w2, 4, 32)
        del w13, w2
    yield moe
    del moe
    torch.cuda.empty_cache()


def _moe_inputs(t):
    rng = np.random.default_rng(900 + t)
    x = rng.standard_normal((t, H)).astype(np.float16)
    logits = rng.standard_normal((t, NE)).astype(np.float16)
    if t >= 16:
        logits[3] = logits[2]      # two tokens with the same experts
        logits[5, :] = 0.25        # a full tie: experts 0 and 1, in that order
    return x, logits


def _expert_stage_check(out, xs_h, qw, qs, indptr, rng, what, n_cols=256):
    """Grouped matmul output [rows, N] against the oracle: per expert, a sample of >= n_cols output columns and of
    the expert's rows."""
    k = xs_h.shape[1]
    n = qw.shape[1]
    for e in range(NE):
        lo, hi = int(indptr[e]), int(indptr[e + 1])
        if hi == lo:
            continue
        cols = _sample(n_cols, n, rng)
        rows = lo + (np.arange(hi - lo) if hi - lo <= 12 else _sample(12, hi - lo, rng))
        ct = torch.from_numpy(cols).to(DEV)
        qw_h = qw[e][ct].cpu().numpy().view(np.uint32)
        qs_h = qs[e][ct].cpu().numpy()
        ref = o.linear_fp32(xs_h[rows], qw_h, qs_h, Q4)
        got = out[torch.from_numpy(rows).to(DEV)][:, ct].float().cpu().numpy()
        err, bound, rel = o.check_linear(got, ref, xs_h[rows], k)
        assert err <= bound and rel <= 2e-3, f"{what} expert {e}: err {err:.3e} bound {bound:.3e} rel {rel:.3e}"


@pytest.mark.parametrize("t", [1, 16, 512])
def test_mixtral_routing_bit_exact(t):
    _, logits = _moe_inputs(t)
    w_ref, ids_ref = o.gating_softmax_topk(logits, TOPK)
    w, ids = ops.gating_softmax_topk(torch.from_numpy(logits).to(DEV), TOPK)
    assert np.array_equal(ids.cpu().numpy(), ids_ref)
    ulp = np.abs(w.cpu().numpy().view(np.int16).astype(np.int32) - w_ref.view(np.int16).astype(np.int32))
    assert ulp.max() <= 1
    cs_ref = o.moe_cumsum(ids_ref, NE)
    rev_ref, tok_ref = o.get_indices(cs_ref, ids_ref)
    ip_ref = o.get_indptr(cs_ref, NE, t, False)
    cs = ops.moe_cumsum(ids, NE)
    rev, tok = ops.get_indices(cs, ids)
    assert np.array_equal(cs.cpu().numpy(), cs_ref)
    assert np.array_equal(rev.cpu().numpy(), rev_ref) and np.array_equal(tok.cpu().numpy(), tok_ref)
    assert np.array_equal(ops.get_indptr(cs, NE, t, False, torch.int32).cpu().numpy(), ip_ref)
    # the one-launch route step gives the same plan
    r = ops.moe_route(torch.from_numpy(logits).to(DEV), TOPK)
    w2, ids2, tok2, rev2, pos2, ip2 = r
    assert np.array_equal(ids2.cpu().numpy(), ids_ref) and torch.equal(w2, w)
    assert np.array_equal(tok2.cpu().numpy(), tok_ref) and np.array_equal(rev2.cpu().numpy(), rev_ref)
    assert np.array_equal(ip2.cpu().numpy(), ip_ref)
    inv = np.empty_like(rev_ref)
    inv[rev_ref] = np.arange(rev_ref.size)
    assert np.array_equal(pos2.cpu().numpy(), inv)


@pytest.mark.parametrize("t", [16, 512])
def test_mixtral_expert_stages_sampled(mixtral, t):
    """dequantize_group_gemm at the two expert shapes ([8, 28672, 4096], [8, 4096, 14336]), stage inputs from the
    oracle side (the routing plan, the gathered rows, a seeded activation for the second stage): nothing a stage
    reads was produced by the kernel before it."""
    rng = np.random.default_rng(t)
    x, logits = _moe_inputs(t)
    _, ids = o.gating_softmax_topk(logits, TOPK)
    cs = o.moe_cumsum(ids, NE)
    rev, tok = o.get_indices(cs, ids)
    indptr = o.get_indptr(cs, NE, t, False)
    xs = x[tok]
    ip_d = torch.from_numpy(indptr).to(DEV)
    q13, s13 = mixtral.e1_e3.q_weight.data, mixtral.e1_e3.q_scale.data
    q2, s2 = mixtral.e2.q_weight.data, mixtral.e2.q_scale.data
    y13 = ops.moe_group_gemm(torch.from_numpy(xs).to(DEV), q13, s13, ip_d, 4, 32)
    _expert_stage_check(y13, xs, q13, s13, indptr, rng, f"e1_e3 T={t}")
    # the gather folded into the matmul, and the activation folded in, give the same bits as the separate steps
    y13g = ops.moe_experts(torch.from_numpy(x).to(DEV), torch.from_numpy(tok).to(DEV), q13, s13, ip_d, 4, 32, False)
    assert torch.equal(y13g, y13)
    act = ops.silu_mul(y13)
    fused = ops.moe_experts(torch.from_numpy(x).to(DEV), torch.from_numpy(tok).to(DEV), q13, s13, ip_d, 4, 32, True)
    assert torch.equal(fused, act)
    # silu * mul on a sample of rows of the kernel's own first-stage output (elementwise: two units at most)
    rows = _sample(8, 2 * t, rng)
    a_ref = o.silu_mul_f16(y13[torch.from_numpy(rows).to(DEV)].cpu().numpy())
    a_got = act[torch.from_numpy(rows).to(DEV)].cpu().numpy()
    ulp = np.abs(a_got.view(np.int16).astype(np.int32) - a_ref.view(np.int16).astype(np.int32))
    assert ulp.max() <= 2
    # second stage on a seeded activation of the intermediate shape
    a = (rng.standard_normal((2 * t, INTER)) * 0.3).astype(np.float16)
    y2 = ops.moe_group_gemm(torch.from_numpy(a).to(DEV), q2, s2, ip_d, 4, 32)
    _expert_stage_check(y2, a, q2, s2, indptr, rng, f"e2 T={t}")
    # int64 indptr (the reference's other variant) gives the same bits
    y2b = ops.moe_group_gemm(torch.from_numpy(a).to(DEV), q2, s2, torch.from_numpy(indptr.astype(np.int64)).to(DEV), 4, 32)
    assert torch.equal(y2b, y2)


def test_mixtral_single_token_gemv_sampled(mixtral):
    """dequantize_gemv (T = 1) at both expert shapes against the oracle on sampled output columns."""
    rng = np.random.default_rng(1)
    x, logits = _moe_inputs(1)
    _, ids = o.gating_softmax_topk(logits, TOPK)
    ids_d = torch.from_numpy(ids).to(DEV)
    for qw, qs, xin in ((mixtral.e1_e3.q_weight.data, mixtral.e1_e3.q_scale.data, x),
                        (mixtral.e2.q_weight.data, mixtral.e2.q_scale.data,
                         (rng.standard_normal((TOPK, INTER)) * 0.3).astype(np.float16))):
        out = ops.moe_gemv(torch.from_numpy(xin).to(DEV), qw, qs, ids_d, 4, 32)
        n = qw.shape[1]
        cols = _sample(512, n, rng)
        ct = torch.from_numpy(cols).to(DEV)
        for j in range(TOPK):
            e = int(ids[0, j])
            xr = xin[0 if xin.shape[0] == 1 else j][None, :]
            ref = o.linear_fp32(xr, qw[e][ct].cpu().numpy().view(np.uint32), qs[e][ct].cpu().numpy(), Q4)
            err, bound, rel = o.check_linear(out[j][ct].float().cpu().numpy()[None, :], ref, xr, xr.shape[1])
            assert err <= bound and rel <= 2e-3, (j, err, bound, rel)


@pytest.mark.parametrize("t", [1, 16, 512])
def test_mixtral_layer_end_to_end(mixtral, t):
    """MixtralMoE.forward at the full shapes against the composed oracle.  A token's output depends on its own
    activation and logits only, so for T = 512 the oracle runs on a sample of the tokens (first, last, the two
    tokens with equal experts, the full tie); its matmuls are the C restatement (fp32 accumulation), its
    composition the numpy one."""
    x, logits = _moe_inputs(t)
    y = mixtral(torch.from_numpy(x).to(DEV).reshape(1, t, H), torch.from_numpy(logits).to(DEV)).reshape(t, H)
    y = y.float().cpu().numpy()
    toks = np.arange(t) if t <= 16 else np.array([0, 2, 3, 5, 100, 255, 256, 511])
    q13 = mixtral.e1_e3.q_weight.data.cpu().numpy().view(np.uint32)
    s13 = mixtral.e1_e3.q_scale.data.cpu().numpy()
    q2 = mixtral.e2.q_weight.data.cpu().numpy().view(np.uint32)
    s2 = mixtral.e2.q_scale.data.cpu().numpy()

    def c_gemv(xx, qw, qs, ids, scheme):
        return np.stack([c_oracle.linear(np.ascontiguousarray(xx[0 if xx.shape[0] == 1 else j][None, :]),
                                         qw[int(ids[0, j])], qs[int(ids[0, j])], 4, 32)[0]
                         for j in range(ids.shape[1])])

    def c_group(xx, qw, qs, indptr, scheme):
        return c_oracle.group_gemm(np.ascontiguousarray(xx), qw, qs, indptr.astype(np.int32), 4, 32)

    if t == 1:
        ref = o.mixtral_moe(x, logits, q13, s13, q2, s2, Q4, TOPK, gemv=c_gemv, group_gemm=c_group)
    else:
        ref = o.mixtral_moe(x[toks], logits[toks], q13, s13, q2, s2, Q4, TOPK, gemv=c_gemv, group_gemm=c_group)
    ref = ref.astype(np.float64)
    got = y[toks].astype(np.float64)
    err = np.abs(got - ref).max()
    rel = np.linalg.norm(got - ref) / np.linalg.norm(ref)
    # two chained matmuls with an fp16 rounding and the activation between them, then the fp16 combine
    assert rel <= 4e-3 and err <= 1e-2 * np.abs(ref).max(), (t, err, rel)
