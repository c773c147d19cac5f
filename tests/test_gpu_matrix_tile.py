"""The matrix-core tile on its own (the diagnostics entries of the C ABI): every combination of
operand orientations against a plain fp32 product of the same 16-bit operands, a product continued
over several calls against one call, and repeats bit for bit. The products of 16-bit numbers are
exact in fp32, so what differs from the reference is the order of the fp32 additions only."""
import pytest
import torch

from openrlhf_amd import _lib
from openrlhf_amd._lib import call, ptr, stream_of

pytestmark = pytest.mark.gpu


def _product(cuda, a, b, code, a_mn, b_mn, m, n, k, into=None, k_from=0, k_len=None):
    """c = (or +=) A[:, k_from : k_from + k_len] * B[:, same]^T with the operands as they lie."""
    k_len = k - k_from if k_len is None else k_len
    esz = a.element_size()
    c = torch.full((m, n), float("nan"), device=cuda) if into is None else into
    pa = ptr(a) + (k_from * a.stride(0) if a_mn else k_from) * esz
    pb = ptr(b) + (k_from * b.stride(0) if b_mn else k_from) * esz
    call("orlhf_matrix_tile_product", pa, pb, code, m, n, k_len, a.stride(0), b.stride(0), int(a_mn), int(b_mn),
         0 if into is None else 1, ptr(c), c.stride(0), stream_of(cuda))
    return c


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("m,n,k", [(256, 256, 64), (256, 256, 192), (300, 516, 204), (1000, 258, 4102), (64, 700, 130),
                                   (2, 2, 2), (512, 768, 4096)])
def test_every_operand_orientation(cuda, dtype, m, n, k):
    g = torch.Generator().manual_seed(m + n + k)
    A = torch.randn(m, k, generator=g).to(dtype).to(cuda)
    B = torch.randn(n, k, generator=g).to(dtype).to(cuda)
    ref = A.double() @ B.double().T
    scale = (A.double().abs() @ B.double().abs().T)
    code = _lib.dtype_code(A)
    results = []
    for a_mn in (False, True):
        for b_mn in (False, True):
            # padded leading dimensions, NaN in the padding: it must never reach a stored element
            a = torch.full((k, m + 6) if a_mn else (m, k + 10), float("nan"), dtype=dtype, device=cuda)
            b = torch.full((k, n + 2) if b_mn else (n, k + 4), float("nan"), dtype=dtype, device=cuda)
            if a_mn:
                a[:, :m] = A.t()
            else:
                a[:, :k] = A
            if b_mn:
                b[:, :n] = B.t()
            else:
                b[:, :k] = B
            av = a[:, :m] if a_mn else a[:, :k]
            bv = b[:, :n] if b_mn else b[:, :k]
            # (an MN-major operand's rows past its extent reach only outputs nobody stores; k past the
            # depth reads as zero because these operands end where their matrices end)
            c = _product(cuda, av, bv, code, a_mn, b_mn, m, n, k)
            assert torch.isfinite(c).all(), (a_mn, b_mn)
            assert ((c.double() - ref).abs() <= 1e-6 * scale + 1e-30).all(), (a_mn, b_mn, (c.double() - ref).abs().max().item())
            results.append(c)
    for c in results[1:]:  # the same additions in the same order whatever the orientation
        assert torch.equal(c, results[0])


@pytest.mark.parametrize("a_mn,b_mn", [(False, False), (False, True), (True, True)])
def test_continued_product_is_the_whole_product(cuda, a_mn, b_mn):
    """A product cut into stretches of k and continued inside the accumulators gives the bits of the
    product over the whole depth, wherever the cuts are (multiples of the 64-wide slab)."""
    m, n, k = 700, 520, 1536
    g = torch.Generator().manual_seed(9)
    A = torch.randn(m, k, generator=g).to(torch.bfloat16).to(cuda)
    B = torch.randn(n, k, generator=g).to(torch.bfloat16).to(cuda)
    a = A.t().contiguous() if a_mn else A
    b = B.t().contiguous() if b_mn else B
    whole = _product(cuda, a, b, _lib.BF16, a_mn, b_mn, m, n, k)
    for cuts in ((512, 1024), (64, 128, 1472), (768,)):
        c, lo = None, 0
        for hi in cuts + (k,):
            pa = ptr(a) + (lo * a.stride(0) if a_mn else lo) * 2
            pb = ptr(b) + (lo * b.stride(0) if b_mn else lo) * 2
            out = torch.full((m, n), float("nan"), device=cuda) if c is None else c
            call("orlhf_matrix_tile_product", pa, pb, _lib.BF16, m, n, hi - lo, a.stride(0), b.stride(0), int(a_mn), int(b_mn),
                 0 if c is None else 1, ptr(out), out.stride(0), stream_of(cuda))
            c, lo = out, hi
        assert torch.equal(c, whole), cuts


@pytest.mark.parametrize("a_mn,b_mn,m,n,k", [(False, False, 8192, 8192, 8192), (False, True, 4096, 4096, 32768),
                                             (True, True, 8192, 4096, 4096), (True, False, 4096, 8192, 4100)])
def test_products_repeat_bit_for_bit(cuda, a_mn, b_mn, m, n, k):
    """Every orientation at a size that keeps every CU busy for thousands of slabs (and one whose
    last slab goes through registers): three runs, the same bits. A slab published before its loads
    had landed, or read while it is being overwritten, would show up as a run that differs."""
    g = torch.Generator(device=cuda).manual_seed(m + k)
    a = torch.randn((k, m) if a_mn else (m, k), generator=g, device=cuda).to(torch.bfloat16)
    b = torch.randn((k, n) if b_mn else (n, k), generator=g, device=cuda).to(torch.bfloat16)
    runs = [_product(cuda, a, b, _lib.BF16, a_mn, b_mn, m, n, k) for _ in range(3)]
    assert torch.equal(runs[0], runs[1]) and torch.equal(runs[0], runs[2])
    rows = torch.arange(0, m, 997, device=cuda)
    A = (a.t() if a_mn else a)[rows].float()
    Bf = (b.t() if b_mn else b).float()
    ref = A @ Bf.T
    assert ((runs[0][rows] - ref).abs() <= 1e-5 * (A.abs() @ Bf.abs().T)).all()


@pytest.mark.parametrize("m,n,k", [(256, 256, 64), (300, 515, 204), (1000, 259, 4102), (64, 700, 130)])
def test_matrix_tile_probe_sums(cuda, m, n, k):
    """The timing entry computes the product it times: the 256 thread sums of every tile add up to
    the sum of that 256 x 256 block of a @ b.T (fp32 reference on the same bf16 operands)."""
    g = torch.Generator().manual_seed(m + n + k)
    a = torch.randn(m, k, generator=g).to(torch.bfloat16).to(cuda)
    b = torch.randn(n, k, generator=g).to(torch.bfloat16).to(cuda)
    tm, tn = (m + 255) // 256, (n + 255) // 256
    sums = torch.full((tm * tn * 256,), float("nan"), device=cuda)
    call("orlhf_matrix_tile_probe", ptr(a), ptr(b), _lib.BF16, m, n, k, k, k, 0, ptr(sums), stream_of(cuda))
    c = a.float() @ b.float().T
    scale = c.abs().sum().item() / (tm * tn)
    for i in range(tm):
        for j in range(tn):
            want = c[i * 256:(i + 1) * 256, j * 256:(j + 1) * 256].double().sum().item()
            got = sums[(i * tn + j) * 256:(i * tn + j + 1) * 256].double().sum().item()
            assert abs(got - want) <= 1e-5 * scale + 1e-3, (i, j, got, want)
    with pytest.raises(_lib.KernelError):
        call("orlhf_matrix_tile_probe", ptr(a), ptr(b), _lib.F32, m, n, k, k, k, 0, ptr(sums), stream_of(cuda))
