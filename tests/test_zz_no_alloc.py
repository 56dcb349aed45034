"""sa_gemm_f32_static (the entry point that allocates nothing: its problem table lives in a file-scope device array)
against sa_gemm_f32 through the C ABI: same kernels, so the results must be bit-identical.  Two calls in a row, the
second with a smaller input, so that the table's left-over contents from the first call are exercised."""

import pytest
import torch

pytestmark = pytest.mark.gpu


def _call(fn, name, A, B, M, N, K, al, bl, batch):
    from optimizers_amd import native

    C = torch.full((batch, M, N), float("nan"), device=A.device, dtype=torch.float32)
    lda, ldb = A.shape[-1], B.shape[-1]
    sa = A.shape[-2] * A.shape[-1] if batch > 1 else 0
    sb = B.shape[-2] * B.shape[-1] if batch > 1 else 0
    st = native.current_stream_ptr(A.device)
    native.check(fn(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, lda, ldb, N, al, bl, batch, sa, sb, M * N, st), name)
    torch.cuda.synchronize()
    return C


def _operands(M, N, K, al, bl, batch, seed):
    g = torch.Generator().manual_seed(seed)
    A = torch.randn((batch, M, K) if al == 0 else (batch, K, M), generator=g).cuda()
    B = torch.randn((batch, K, N) if bl == 0 else (batch, N, K), generator=g).cuda()
    return A, B


@pytest.mark.parametrize("layouts", [(0, 0), (1, 0), (0, 1), (1, 1)])
def test_static_gemm_equals_gemm_on_two_calls_in_a_row(layouts):
    from optimizers_amd import native

    lib = native.load()
    al, bl = layouts
    # first call: 6 aligned problems (unguarded loader); second call: 2 ragged ones (guarded loader) of fewer tiles
    for k, (M, N, K, batch) in enumerate([(256, 384, 512, 6), (81, 200, 37, 2)]):
        print(f"case layouts={layouts} call={k} shape={(M, N, K)} batch={batch}", flush=True)
        A, B = _operands(M, N, K, al, bl, batch, seed=11 * k + al * 2 + bl)
        want = _call(lib.sa_gemm_f32, "sa_gemm_f32", A, B, M, N, K, al, bl, batch)
        got = _call(lib.sa_gemm_f32_static, "sa_gemm_f32_static", A, B, M, N, K, al, bl, batch)
        assert torch.isfinite(got).all()
        assert torch.equal(got, want)
        ref = torch.bmm((A if al == 0 else A.transpose(1, 2)).double(), (B if bl == 0 else B.transpose(1, 2)).double())
        assert ((got.double() - ref).norm() / ref.norm()).item() < 2e-6


def test_static_gemm_leaves_the_free_device_memory_unchanged():
    """The property the entry point exists for: after one warm-up call (code object, symbol address) a call takes no
    device memory - hipMemGetInfo reads the same free byte count before and after, with the output allocated beforehand."""
    from optimizers_amd import native

    lib = native.load()
    M, N, K, batch = 256, 256, 128, 4
    A, B = _operands(M, N, K, 0, 0, batch, seed=3)
    C = torch.empty((batch, M, N), device=A.device, dtype=torch.float32)
    st = native.current_stream_ptr(A.device)
    args = (A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, K, N, N, 0, 0, batch, M * K, K * N, M * N, st)
    native.check(lib.sa_gemm_f32_static(*args), "sa_gemm_f32_static")  # warm-up
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    for _ in range(3):
        native.check(lib.sa_gemm_f32_static(*args), "sa_gemm_f32_static")
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before, (free_before, free_after)
    ref = torch.bmm(A.double(), B.double())
    assert ((C.double() - ref).norm() / ref.norm()).item() < 2e-6


def test_static_gemm_rejects_a_batch_beyond_its_table():
    from optimizers_amd import native

    lib = native.load()
    A = torch.zeros(1, device="cuda")
    st = native.current_stream_ptr(A.device)
    rc = lib.sa_gemm_f32_static(A.data_ptr(), A.data_ptr(), A.data_ptr(), 1, 1, 1, 1, 1, 1, 0, 0, 1025, 0, 0, 0, st)
    assert rc == 1
    assert b"exceeds the static problem table" in lib.sa_last_error()
