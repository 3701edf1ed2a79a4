"""The output projection behind the attention (single-rank row_parallel_linear,
src/ppl/kernel/llm/cuda/pmx/row_parallel_linear.cu:25-110): output = input * weight^T + bias, half tensors, float32
accumulation.  CPU: the oracle against numpy in binary64, exact cases and invariants.  GPU: the HIP kernel against
the oracle through the C ABI.

Tolerance of the GPU result against the oracle: both accumulate in float32 and round once to half, in different
orders, so they differ by at most one half ulp of the result plus the float32 accumulation noise:
|got - ref| <= 2^-10 |ref| + 2e-6 * sum_k |a_k w_k|."""
import numpy as np
import pytest


def draw(rng, m, n, k, outliers=True):
    a = rng.standard_normal((m, k), dtype=np.float32)
    if outliers:
        a[:, rng.choice(k, size=max(1, k // 50), replace=False)] *= 10.0
    w = (rng.standard_normal((n, k), dtype=np.float32) / np.sqrt(k)).astype(np.float16)
    b = rng.standard_normal(n, dtype=np.float32).astype(np.float16)
    return a.astype(np.float16), w, b


def assert_close(got, a, w, b, what):
    ref = a.astype(np.float64) @ w.astype(np.float64).T + (0 if b is None else b.astype(np.float64))
    mag = np.abs(a.astype(np.float64)) @ np.abs(w.astype(np.float64)).T
    err = np.abs(got.astype(np.float64) - ref)
    tol = 2.0 ** -10 * np.abs(ref) + 2e-6 * mag + 1e-7
    assert (err <= tol).all(), "%s: %d of %d outside tolerance, worst %g over %g" % (
        what, int((err > tol).sum()), err.size, float((err - tol).max()), float(tol.flat[np.argmax(err - tol)]))


def test_oracle_matches_numpy_float64(oracle):
    rng = np.random.default_rng(11)
    for m, n, k in ((5, 16, 32), (33, 48, 96), (128, 64, 512)):
        a, w, b = draw(rng, m, n, k)
        assert_close(oracle.row_parallel_linear(a, w, b), a, w, b, "oracle %s" % ((m, n, k),))
        assert_close(oracle.row_parallel_linear(a, w, None), a, w, None, "oracle, no bias")


def test_oracle_exact_cases(oracle):
    rng = np.random.default_rng(12)
    # small integers: every product and sum is exact in float32 and in half
    a = rng.integers(-3, 4, (7, 64)).astype(np.float16)
    w = rng.integers(-2, 3, (32, 64)).astype(np.float16)
    b = rng.integers(-5, 6, 32).astype(np.float16)
    want = a.astype(np.int64) @ w.astype(np.int64).T + b.astype(np.int64)
    assert np.array_equal(oracle.row_parallel_linear(a, w, b).astype(np.int64), want)
    # identity weight copies the input; a zero input leaves the bias
    x = rng.standard_normal((9, 32)).astype(np.float16)
    eye = np.eye(32, dtype=np.float16)
    assert np.array_equal(oracle.row_parallel_linear(x, eye), x)
    assert np.array_equal(oracle.row_parallel_linear(np.zeros_like(x), eye, b), np.tile(b, (9, 1)))
    # a transposed operand or swapped indices would fail this one: weight rows select single input channels
    sel = np.zeros((16, 32), dtype=np.float16)
    cols = rng.choice(32, size=16, replace=False)
    sel[np.arange(16), cols] = 1
    assert np.array_equal(oracle.row_parallel_linear(x, sel), x[:, cols])
    # linear in the input (exactly, for power-of-two factors)
    a2, w2, _ = draw(rng, 6, 16, 64)
    assert np.array_equal(oracle.row_parallel_linear(a2 * np.float16(2), w2), oracle.row_parallel_linear(a2, w2) * np.float16(2))


def test_c_entry_point_rejects_bad_arguments_without_launching(pkg, hip_lib):
    f = hip_lib.pmxhip_row_parallel_linear
    assert f(None, 16, 16, None, 0, 32, 16, 32, 32, 16, 0, None, 16) == 0            # no rows: nothing to do
    assert f(None, 16, 16, None, 4, 32, 24, 32, 32, 24, 0, None, 16) == 2            # out_features % 16
    assert f(None, 16, 16, None, 4, 40, 16, 40, 40, 16, 0, None, 16) == 2            # in_features % 32
    assert f(None, None, 16, None, 4, 32, 16, 32, 32, 16, 0, None, 16) == 4          # null input
    assert f(None, 16, 16, None, 4, 32, 16, 16, 32, 16, 0, None, 16) == 4            # input stride shorter than a row
    assert f(None, 24, 16, None, 4, 32, 16, 32, 32, 16, 0, None, 16) == 2            # input not 16-byte aligned
    assert f(None, 16, 16, None, -1, 32, 16, 32, 32, 16, 0, None, 16) == 4


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(1, 16, 32), (7, 48, 96), (128, 4096, 4096), (64, 1024, 8192), (200, 256, 512),
                                   (128, 14336 // 8, 4096), (3, 4096, 32), (129, 32, 4064), (17, 64, 64), (128, 128, 3136),
                                   (300, 8192, 1024), (5, 64, 2240), (1, 64, 512), (16, 128, 1024), (17, 64, 1536), (33, 192, 2048),
                                   (65, 64, 512), (130, 192, 2048), (240, 4096, 4096),
                                   # many rows (a prefill chunk's): this library's kernels, 128 rows at a time
                                   (384, 256, 512), (1000, 512, 1024), (2500, 1024, 2048), (640, 4096, 4096)])
def test_hip_linear_matches_oracle(pkg, oracle, shape, vendor_gemm=False):
    import torch
    m, n, k = shape
    rng = np.random.default_rng(100 + m + n)
    a, w, b = draw(rng, m, n, k)
    da, dw, db = (torch.from_numpy(x).cuda() for x in (a, w, b))
    ws_bytes = pkg.ops.row_parallel_linear_workspace_size(m, k, n, vendor_gemm=vendor_gemm)
    for bias, with_ws in ((db, True), (None, True), (db, False)):  # with the k-split's workspace and without
        out = torch.full((m, n), float("nan"), dtype=torch.float16, device="cuda")
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda") if with_ws and ws_bytes else None
        pkg.ops.row_parallel_linear(da, dw, bias, out, workspace=ws, vendor_gemm=vendor_gemm)
        torch.cuda.synchronize()
        got = out.cpu().numpy()
        assert_close(got, a, w, b if bias is not None else None, "hip %s" % (shape,))
        if m * n * k <= 1 << 26:  # the oracle's triple loop, where it finishes in seconds
            # against the oracle's own half result: one rounding to half on either side plus two float32
            # accumulations in different orders (where sums cancel, an ulp of the small result is far below that noise)
            ref = oracle.row_parallel_linear(a, w, b if bias is not None else None).astype(np.float64)
            mag = np.abs(a.astype(np.float64)) @ np.abs(w.astype(np.float64)).T
            assert (np.abs(got.astype(np.float64) - ref) <= 2.0 ** -10 * np.abs(ref) + 4e-6 * mag + 1e-7).all()
    if vendor_gemm:
        return
    # twice the same call: the partial tiles are added in a fixed order
    out2 = torch.empty_like(out)
    pkg.ops.row_parallel_linear(da, dw, db, out2)
    torch.cuda.synchronize()
    assert torch.equal(out.view(torch.int16), out2.view(torch.int16))


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(384, 256, 512), (1000, 512, 1024), (2500, 1024, 2048), (200, 256, 512)])
def test_hip_linear_vendor_gemm_on_request(pkg, oracle, shape):
    """PMXHIP_LINEAR_VENDOR_GEMM: from 384 rows on the GEMM goes to hipBLASLt where that loads (below, and where it
    does not, the flag changes nothing); same tolerance against the oracle."""
    if not pkg.ops.vendor_gemm_available():
        pytest.skip("hipBLASLt cannot be loaded on this box")
    test_hip_linear_matches_oracle(pkg, oracle, shape, vendor_gemm=True)


@pytest.mark.gpu
@pytest.mark.parametrize("m", [37, 700])
def test_hip_linear_strided_rows_and_attention_hand_off(pkg, oracle, m):
    """Rows with padding between them (the strides of the C ABI), and the attention output (B, Hq, D) used in place
    as the (B, Hq * D) input; a decode-sized and a prefill-sized row count."""
    import torch
    rng = np.random.default_rng(7)
    hq, d, n = 8, 64, 128
    k = hq * d
    a, w, b = draw(rng, m, n, k)
    buf_in = torch.zeros((m, k + 64), dtype=torch.float16, device="cuda")
    buf_in[:, :k] = torch.from_numpy(a).cuda()
    buf_out = torch.full((m, n + 32), float("nan"), dtype=torch.float16, device="cuda")
    pkg.ops.row_parallel_linear(buf_in[:, :k], torch.from_numpy(w).cuda(), torch.from_numpy(b).cuda(), buf_out[:, :n])
    torch.cuda.synchronize()
    assert_close(buf_out[:, :n].cpu().numpy(), a, w, b, "strided")
    assert torch.isnan(buf_out[:, n:]).all()
    attn = torch.from_numpy(a).cuda().view(m, hq, d)  # the decode output as the operator writes it
    out = torch.empty((m, n), dtype=torch.float16, device="cuda")
    pkg.ops.row_parallel_linear(attn, torch.from_numpy(w).cuda(), None, out)
    torch.cuda.synchronize()
    assert_close(out.cpu().numpy(), a, w, None, "attention output in place")
