"""Grouped fp32 MFMA GEMM (sa_gemm_f32 through the C ABI) against a float64 product."""

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _run(lib, A, B, M, N, K, al, bl, batch=1):
    from optimizers_amd import native

    C = torch.full((batch, M, N), float("nan"), device=A.device, dtype=torch.float32)
    lda = A.shape[-1]
    ldb = B.shape[-1]
    sa = A.shape[-2] * A.shape[-1] if batch > 1 else 0
    sb = B.shape[-2] * B.shape[-1] if batch > 1 else 0
    st = native.current_stream_ptr(A.device)
    native.check(
        lib.sa_gemm_f32(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, lda, ldb, N, al, bl, batch, sa, sb, M * N, st),
        "sa_gemm_f32",
    )
    torch.cuda.synchronize()
    return C


@pytest.mark.parametrize("al", [0, 1])
@pytest.mark.parametrize("bl", [0, 1])
@pytest.mark.parametrize("shape", [(128, 128, 16), (256, 384, 512), (81, 200, 37), (1, 5, 3), (130, 1, 129), (300, 260, 1)])
def test_gemm_layouts_and_ragged_shapes(al, bl, shape):
    from optimizers_amd import native

    lib = native.load()
    M, N, K = shape
    print(f"case al={al} bl={bl} shape={shape}", flush=True)
    g = torch.Generator().manual_seed(M * 7 + N * 3 + K)
    A = torch.randn((M, K) if al == 0 else (K, M), generator=g)
    B = torch.randn((K, N) if bl == 0 else (N, K), generator=g)
    want = (A if al == 0 else A.T).double() @ (B if bl == 0 else B.T).double()
    got = _run(lib, A.cuda(), B.cuda(), M, N, K, al, bl)[0].cpu().double()
    assert torch.isfinite(got).all()
    err = (got - want).norm() / want.norm()
    assert err < 2e-6, err


def test_gemm_batched_2048_matches_fp64_sample():
    from optimizers_amd import native

    lib = native.load()
    g = torch.Generator().manual_seed(5)
    A = torch.randn(3, 1024, 1024, generator=g).cuda()
    B = torch.randn(3, 1024, 1024, generator=g).cuda()
    got = _run(lib, A, B, 1024, 1024, 1024, 0, 0, batch=3)
    want = torch.bmm(A.double(), B.double())
    err = ((got.double() - want).norm() / want.norm()).item()
    assert err < 2e-6, err


@pytest.mark.parametrize("al", [0, 1])
@pytest.mark.parametrize("bl", [0, 1])
@pytest.mark.parametrize(
    "shape",
    [(256, 128, 32), (128, 256, 64), (256, 256, 96), (128, 128, 48), (256, 128, 80), (32, 96, 1024), (81, 200, 64), (4, 8, 32), (300, 132, 160)],
)
def test_gemm_on_views_that_end_with_their_allocation(al, bl, shape):
    """Shapes with K a multiple of 32 take the unguarded main loop (two slabs per trip; its loads go through buffer
    resources that end with the operand and fetch two slabs ahead without asking whether there are any), ragged M and N
    included: what such a tile fetches past M or N lands in rows and columns the guarded epilogue drops (the parents are
    filled with NaN outside the operands here, so a dropped guard would show).  Other K (48, 80) take the guarded loop.
    The operands are column slices of wider parents whose last row ends the allocation, so an extent computed too
    short would read zeros for the last rows and one computed from the parent's pitch would reach past the
    allocation."""
    from optimizers_amd import native

    lib = native.load()
    M, N, K = shape
    print(f"case al={al} bl={bl} shape={shape}", flush=True)
    g = torch.Generator().manual_seed(M + 3 * N + 7 * K + al + 2 * bl)
    ra, ca = (M, K) if al == 0 else (K, M)
    rb, cb = (K, N) if bl == 0 else (N, K)
    pa = torch.full((ra, ca + 64), float("nan"))
    pb = torch.full((rb, cb + 192), float("nan"))
    pa[:, 64:] = torch.randn(ra, ca, generator=g)
    pb[:, 192:] = torch.randn(rb, cb, generator=g)
    pa, pb = pa.cuda(), pb.cuda()
    A, B = pa[:, 64:], pb[:, 192:]
    want = (A if al == 0 else A.T).double() @ (B if bl == 0 else B.T).double()
    C = torch.full((M, N), float("nan"), device="cuda", dtype=torch.float32)
    st = native.current_stream_ptr(C.device)
    native.check(
        lib.sa_gemm_f32(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, ca + 64, cb + 192, N, al, bl, 1, 0, 0, 0, st),
        "sa_gemm_f32",
    )
    torch.cuda.synchronize()
    assert torch.isfinite(C).all()
    err = ((C.double() - want).norm() / want.norm()).item()
    assert err < 2e-6, err
