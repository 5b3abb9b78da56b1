"""mi355gq_linear_static_scratch: the linear for callers that cannot allocate (split-K partial sums in a device
array of the library's own).  Through the C ABI, against mi355gq_linear with a caller's workspace: same kernels,
same split plan, so the same bits; and against the oracle.  Two calls in a row, the second on a smaller input,
because every call on a GPU shares the one array."""

import numpy as np
import pytest
import torch

import mlc_llm_amd as gq
from oracle import gq_oracle as o

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _case(m, n, k, seed):
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float16)
    qw, qs = o.quantize(w, o.SCHEMES["q4f16_1"])
    x = rng.standard_normal((m, k)).astype(np.float16)
    b = rng.standard_normal(n).astype(np.float16)
    return x, qw, qs, b


def _run_both(x, qw, qs, b, out_dtype, check_memory):
    lib = gq._lib
    m, k = x.shape
    n = qw.shape[0]
    xd, bd = torch.from_numpy(x).to(DEV), torch.from_numpy(b).to(DEV)
    qwd, qsd = torch.from_numpy(qw.view(np.int32)).to(DEV), torch.from_numpy(qs).to(DEV)
    tdt = torch.float16 if out_dtype == lib.F16 else torch.float32
    want = torch.empty((m, n), dtype=tdt, device=DEV)
    got = torch.full((m, n), 3.0, dtype=tdt, device=DEV)
    need = lib.lib().mi355gq_linear_workspace_bytes(m, n, k, 4, 32)
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=DEV)
    stream = torch.cuda.current_stream().cuda_stream
    lib.call("mi355gq_linear", xd.data_ptr(), qwd.data_ptr(), qsd.data_ptr(), bd.data_ptr(), m, n, k, 4, 32, out_dtype,
             want.data_ptr(), ws.data_ptr(), need, stream)
    torch.cuda.synchronize()
    free0 = torch.cuda.mem_get_info()[0]
    lib.call("mi355gq_linear_static_scratch", xd.data_ptr(), qwd.data_ptr(), qsd.data_ptr(), bd.data_ptr(), m, n, k, 4,
             32, out_dtype, got.data_ptr(), stream)
    torch.cuda.synchronize()
    if check_memory:
        assert torch.cuda.mem_get_info()[0] >= free0  # no device memory was taken by the call
    return want, got, need


def test_static_scratch_linear_two_calls_in_a_row():
    lib = gq._lib
    assert lib.lib().mi355gq_linear_static_scratch_max_bytes() == 32 << 20
    s = o.SCHEMES["q4f16_1"]
    # first call: 64 rows of a long K (the few-row GEMM splits K: megabytes of partial sums); second call: a smaller
    # matmul that splits into fewer, smaller partial tiles and finds the first call's sums still in the array;
    # then one-row and large-M calls that need no scratch at all
    cases = [(64, 1024, 8192, lib.F16), (24, 520, 4096, lib.F16), (40, 260, 8192, lib.F32), (1, 384, 1024, lib.F16),
             (300, 256, 512, lib.F16), (12, 2048, 14336, lib.F16)]  # (the last: K slices of the 9..16-row kernel)
    needs = []
    lib.call("mi355gq_linear_static_scratch_init")  # the per-device set-up (address look-up), outside any call that must not allocate
    for i, (m, n, k, od) in enumerate(cases):
        x, qw, qs, b = _case(m, n, k, 100 + i)
        want, got, need = _run_both(x, qw, qs, b, od, check_memory=True)
        needs.append(need)
        assert torch.equal(got, want), (m, n, k)
        err, bound, rel = o.check_linear(got.float().cpu().numpy(), o.linear_fp32(x, qw, qs, s, b), x, k)
        assert err <= bound and rel <= 2e-3, (m, n, k, err, bound, rel)
    assert needs[0] > needs[1] > 0 and needs[3] == 0 and needs[5] == 4 * 12 * 2048 * 4  # the cases do what the comments say


def test_static_scratch_linear_rejects_what_does_not_fit():
    """The default split plan stays under 30 MiB of partial sums (at most 456 tiles of 128 x 128 floats), so the
    limit is met only when a tuning run asks for more workgroups through the test hook: that is how it is reached
    here.  The size check comes first: nothing is launched and no pointer is dereferenced."""
    lib = gq._lib
    cap = lib.lib().mi355gq_linear_static_scratch_max_bytes()
    m, n, k = 128, 8192, 65536
    assert lib.lib().mi355gq_linear_workspace_bytes(m, n, k, 4, 32) <= cap
    t = torch.zeros(64, dtype=torch.uint8, device=DEV)
    lib.set_option("gemm_split_k", 4096)
    try:
        assert lib.lib().mi355gq_linear_workspace_bytes(m, n, k, 4, 32) > cap
        with pytest.raises(lib.Mi355gqError) as ei:
            lib.call("mi355gq_linear_static_scratch", t.data_ptr(), t.data_ptr(), t.data_ptr(), None, m, n, k, 4, 32,
                     lib.F16, t.data_ptr(), torch.cuda.current_stream().cuda_stream)
    finally:
        lib.set_option("gemm_split_k", -1)
    assert ei.value.code == lib.ERR_WORKSPACE and "partial sums" in str(ei.value)


def test_static_scratch_linear_runs_without_the_k_slices_where_they_do_not_fit():
    """32 rows of 16416 x 65536: the K slices of the 17..32-row kernel would keep 16 x 32 x 16416 floats, just over the array;
    they are an option of the dispatch, so the call answers on the GEMM's tiles (whose own split fits) instead of
    rejecting the shape.  A sample of the columns against the oracle."""
    lib = gq._lib
    s = o.SCHEMES["q4f16_1"]
    m, n, k = 32, 16416, 65536
    cap = lib.lib().mi355gq_linear_static_scratch_max_bytes()
    assert lib.lib().mi355gq_linear_workspace_bytes(m, n, k, 4, 32) > cap
    rng = np.random.default_rng(7)
    qw = rng.integers(0, 2**32, (n, k // 8), dtype=np.uint32)
    qs = (rng.random((n, k // 32)) * 0.02 + 0.001).astype(np.float16)
    x = rng.standard_normal((m, k)).astype(np.float16)
    xd = torch.from_numpy(x).to(DEV)
    qwd, qsd = torch.from_numpy(qw.view(np.int32)).to(DEV), torch.from_numpy(qs).to(DEV)
    got = torch.full((m, n), 3.0, dtype=torch.float16, device=DEV)
    lib.call("mi355gq_linear_static_scratch", xd.data_ptr(), qwd.data_ptr(), qsd.data_ptr(), None, m, n, k, 4, 32, lib.F16,
             got.data_ptr(), torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert not lib.last_kernel().startswith("gq::midrow_kernel"), lib.last_kernel()
    cols = np.unique(np.concatenate([[0, 1, n - 1], rng.integers(0, n, 60)]))
    ref = o.linear_fp32(x, qw[cols], qs[cols], s)
    err, bound, rel = o.check_linear(got[:, torch.from_numpy(cols).to(DEV)].float().cpu().numpy(), ref, x, k)
    assert err <= bound and rel <= 2e-3, (err, bound, rel)
