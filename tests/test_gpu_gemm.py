"""fp32 MFMA GEMM vs fp64 NumPy matmul, through the C-ABI (haste_hip_gemm_f32)."""
import numpy as np
import pytest

from util import dev, host, relerr

pytestmark = pytest.mark.gpu

SHAPES = [
    # (trans_a, M, N, K)
    (False, 128, 128, 16), (False, 256, 384, 64), (False, 100, 200, 50), (False, 1, 1, 1),
    (False, 37, 53, 29), (True, 128, 128, 32), (True, 70, 130, 45), (True, 5, 20, 33),
    (False, 6400, 2048, 512),   # x*W of the metric config
    (False, 512, 2048, 6400),   # dW: split along K
    (True, 512, 2048, 6400),    # dR: split along K, A = h^T
    (False, 6400, 512, 2048),   # dx
    (False, 96, 96, 5000),      # split-K with ragged tiles
    # M <= 64 with a long enough K: the kernel that streams B into the MFMA operands
    (False, 64, 1024, 4096), (False, 47, 6144, 1536), (False, 33, 772, 3000), (False, 128, 1024, 4096),
    (False, 100, 768, 3072),
    (False, 1, 2048, 512), (False, 16, 6144, 1536), (False, 5, 1300, 5200), (False, 32, 768, 3072),
    (False, 17, 4100, 332), (False, 3, 64, 1024), (False, 32, 16384, 1000),
    # whole tiles beside edge tiles, K pieces that are and are not multiples of 16: the unmasked
    # and the masked loop in one launch
    (False, 300, 260, 250), (True, 384, 1000, 1600), (False, 640, 192, 2048), (True, 800, 512, 1000),
    (False, 1024, 1024, 17),
]


@pytest.mark.parametrize("trans_a,M,N,K", SHAPES)
@pytest.mark.parametrize("accumulate", [False, True])
def test_gemm_matches_numpy(trans_a, M, N, K, accumulate):
    from haste_amd import ops
    import torch
    r = np.random.default_rng(M * 7 + N * 3 + K)
    a = r.standard_normal((K, M) if trans_a else (M, K)).astype(np.float32)
    b = r.standard_normal((K, N)).astype(np.float32)
    c0 = r.standard_normal((M, N)).astype(np.float32)
    print("gemm", trans_a, M, N, K, accumulate, flush=True)
    out = dev(c0)
    ops.gemm(dev(a), dev(b), out=out, trans_a=trans_a, accumulate=accumulate)
    torch.cuda.synchronize()
    a64 = a.astype(np.float64)
    ref = (a64.T if trans_a else a64) @ b.astype(np.float64)
    if accumulate:
        ref = ref + c0
    assert relerr(host(out), ref) < 1e-5  # fp32 accumulation over K up to 6400


@pytest.mark.parametrize("trans_a,M,N,K,pad_a,pad_b", [(False, 256, 256, 128, 4, 4), (True, 384, 128, 96, 3, 1),
                                                        (False, 130, 100, 64, 3, 4), (True, 128, 256, 2048, 4, 0)])
def test_gemm_padded_leading_dimensions(trans_a, M, N, K, pad_a, pad_b):
    """Operands that are column ranges of wider arrays (lda > K, ldb > N), aligned and not."""
    import torch
    from haste_amd import lib as hlib
    g = torch.Generator().manual_seed(M + N + K)
    a_full = torch.randn((K, M + pad_a) if trans_a else (M, K + pad_a), generator=g).cuda()
    b_full = torch.randn(K, N + pad_b, generator=g).cuda()
    a = a_full[:, :M] if trans_a else a_full[:, :K]
    out = torch.zeros(M, N, device="cuda")
    print("gemm padded", trans_a, M, N, K, pad_a, pad_b, flush=True)
    hlib.call("haste_hip_gemm_f32", int(trans_a), M, N, K, a_full, a_full.stride(0), b_full, b_full.stride(0),
              out, out.stride(0), 0)
    torch.cuda.synchronize()
    ref = (a.double().t() if trans_a else a.double()) @ b_full[:, :N].double()
    assert relerr(host(out), host(ref)) < 1e-5


def test_gemm_split_k_is_run_to_run_identical():
    from haste_amd import ops
    import torch
    r = np.random.default_rng(5)
    a = dev(r.standard_normal((512, 6400)))
    b = dev(r.standard_normal((6400, 2048)))
    o1 = ops.gemm(a, b)
    o2 = ops.gemm(a, b)
    torch.cuda.synchronize()
    assert torch.equal(o1, o2)


@pytest.mark.parametrize("shape", [(1, 1), (3, 5), (64, 64), (65, 63), (100, 7, 33), (6400, 512), (512, 2048)])
def test_transpose(shape):
    import torch
    from haste_amd import ops
    a = torch.randn(*shape, device="cuda")
    out = ops.transpose(a)
    ref = a.reshape(-1, shape[-1]).t().contiguous().reshape((shape[-1],) + tuple(shape[:-1]))
    assert out.shape == ref.shape and torch.equal(out, ref)


@pytest.mark.parametrize("shapes", [((1, 1), (3, 5), (65, 63)), ((100, 7, 33), (64, 64), (2, 130)),
                                    ((6400, 512), (512, 2048), (512, 2048))])
def test_three_transposes_in_one_launch(shapes):
    import torch
    from haste_amd import ops
    ms = [torch.randn(*s, device="cuda") for s in shapes]
    outs = ops.transpose3(*ms)
    for m, out in zip(ms, outs):
        assert torch.equal(out, ops.transpose(m))


@pytest.mark.parametrize("trans_a", [True, False])
def test_gemm_operand_of_more_than_2_gib(trans_a):
    """B[K, N] of 2.1 GB (the dv of a backward pass with T*N*H = 2^27 and beyond: dW = x^T dv
    contracts over T*N): the contraction is cut into runs whose panels the kernel can address.
    Against the float64 product of the same float32 operands, on the GPU (NumPy would take
    minutes)."""
    import torch
    from haste_amd import ops
    M, N, K = 256, 2048, (1 << 18) + 48
    g = torch.Generator(device="cuda").manual_seed(5)
    a = torch.randn((K, M) if trans_a else (M, K), generator=g, device="cuda")
    b = torch.randn(K, N, generator=g, device="cuda")
    assert b.numel() * 4 > 1 << 31
    print("gemm over 2 GiB, trans_a =", trans_a, flush=True)
    c0 = torch.randn(M, N, generator=g, device="cuda")
    out = c0.clone()
    ops.gemm(a, b, out=out, trans_a=trans_a, accumulate=True)
    torch.cuda.synchronize()
    ref = c0.double()
    step = 1 << 15   # float64 copies of the operands, a slab of K at a time
    for k0 in range(0, K, step):
        a_slab = (a[k0:k0 + step].double().t() if trans_a else a[:, k0:k0 + step].double())
        ref += a_slab @ b[k0:k0 + step].double()
    err = float((out.double() - ref).abs().max() / ref.abs().max())
    assert err < 1e-5, err
