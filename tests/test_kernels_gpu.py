"""Each HIP kernel alone against the plain formulas of tests/plain_lfm2.py, at
sizes other than the engine's (odd widths, tails in every dimension, head sizes
from 16 to 256, any group size).

Tolerances, set from the arithmetic and confirmed by measurement: a kernel computing in 32-bit must agree with the
float64 formula to 2e-5 of the result's largest magnitude (accumulation order);
a kernel that stores bfloat16 adds one rounding of the stored value, 2^-8
relative, so 6e-3 of the largest magnitude.
"""

import math

import pytest
import torch

import plain_lfm2 as plain

pytestmark = pytest.mark.gpu

F32_TOL = 2e-5
BF16_TOL = 6e-3


def dev():
    return torch.device("cuda", 0)


def ops():
    from zig_ai_amd.kernels import ops as _ops
    return _ops


def rel_err(actual: torch.Tensor, expected: torch.Tensor) -> float:
    a = actual.detach().double().cpu()
    e = expected.detach().double().cpu()
    assert a.shape == e.shape, (a.shape, e.shape)
    assert torch.isfinite(a).all()
    return float((a - e).abs().max() / e.abs().max().clamp_min(1e-30))


def tol_of(dtype):
    return F32_TOL if dtype == torch.float32 else BF16_TOL


def rand(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


# ----------------------------------------------------------------------- norm
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,width", [(1, 64), (7, 96), (33, 100), (5, 2048), (3, 4099)])
def test_add_rmsnorm(dtype, rows, width):
    x = rand((rows, width), torch.float32, 1, 3.0)
    delta = rand((rows, width), dtype, 2)
    w = rand((width,), torch.float32, 3) + 1.0
    eps = 1e-5
    res = x.clone().to(dev())
    out = ops().add_rmsnorm(res, delta.to(dev()), w.to(dev()), eps, dtype)
    h = x.double() + delta.double()
    expect = plain.rms_norm(h, w.double(), eps)
    assert rel_err(res, h) < F32_TOL                      # the stream took the sum, in 32-bit
    assert rel_err(out, expect) < tol_of(dtype)
    # norm of the stream alone leaves it untouched
    res2 = x.clone().to(dev())
    out2 = ops().add_rmsnorm(res2, None, w.to(dev()), eps, dtype)
    assert torch.equal(res2.cpu(), x)
    assert rel_err(out2, plain.rms_norm(x.double(), w.double(), eps)) < tol_of(dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_add_rmsnorm_selected_rows(dtype):
    x = rand((20, 72), torch.float32, 4)
    delta = rand((20, 72), dtype, 5)
    w = rand((72,), torch.float32, 6)
    rows = torch.tensor([19, 0, 7], dtype=torch.int32)
    res = x.clone().to(dev())
    out = ops().add_rmsnorm(res, delta.to(dev()), w.to(dev()), 1e-6, dtype, rows=rows.to(dev()))
    assert torch.equal(res.cpu(), x)                      # nothing stored back
    expect = plain.rms_norm((x.double() + delta.double())[rows.long()], w.double(), 1e-6)
    assert rel_err(out, expect) < tol_of(dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [64, 100, 2048, 3000, 4096, 5000])
def test_add_rmsnorm_partial_sums(dtype, width):
    """A stack of partial sums as delta is added up while it is read."""
    x = rand((5, width), torch.float32, 1)
    parts = rand((3, 5, width), torch.float32, 2)
    w = rand((width,), torch.float32, 3)
    res = x.clone().to(dev())
    out = ops().add_rmsnorm(res, parts.to(dev()), w.to(dev()), 1e-5, dtype)
    h = x.double() + parts.double().sum(0)
    assert rel_err(res, h) < F32_TOL
    assert rel_err(out, plain.rms_norm(h, w.double(), 1e-5)) < tol_of(dtype)


def test_rmsnorm_reference_vectors():
    """The inputs of /root/reference/src/transformer/norm.zig:83-103 ([1,2,3,4] and
    [1,1,1,1], weight 1): the values follow from the formula; ones stay ones."""
    x = torch.tensor([[1.0, 2.0, 3.0, 4.0], [1.0, 1.0, 1.0, 1.0]])
    out = ops().add_rmsnorm(x.to(dev()), None, torch.ones(4, device=dev()), 0.0, torch.float32,
                            write_residual=False).cpu()
    assert torch.allclose(out[0], x[0] / math.sqrt(7.5), atol=1e-6)
    assert torch.allclose(out[1], torch.ones(4), atol=1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embed_gather(dtype):
    table = rand((37, 50), dtype, 7)
    tokens = torch.tensor([0, 5, 10, 20, 30, 36, 5], dtype=torch.int32)
    out = ops().embed_gather(tokens.to(dev()), table.to(dev())).cpu()
    assert out.dtype == torch.float32
    assert torch.equal(out, table.float()[tokens.long()])


# ----------------------------------------------------------------------- gemm
@pytest.mark.parametrize("M,N,K", [(1, 7, 5), (33, 65, 17), (130, 200, 96), (64, 64, 64), (2, 301, 80)])
def test_gemm_f32(M, N, K):
    x, w, b = rand((M, K), torch.float32, 8), rand((N, K), torch.float32, 9), rand((N,), torch.float32, 10)
    out = ops().linear(x.to(dev()), w.to(dev()), b.to(dev()))
    expect = x.double() @ w.double().T + b.double()
    assert out.dtype == torch.float32
    assert rel_err(out, expect) < F32_TOL
    out_nb = ops().linear(x.to(dev()), w.to(dev()))
    assert rel_err(out_nb, x.double() @ w.double().T) < F32_TOL


def test_gemm_f32_weight_with_bf16_activations():
    """A weight stored in 32-bit stays 32-bit in a bfloat16 run."""
    x, w = rand((9, 40), torch.bfloat16, 11), rand((23, 40), torch.float32, 12)
    out = ops().linear(x.to(dev()), w.to(dev()))
    assert out.dtype == torch.bfloat16
    assert rel_err(out, x.double() @ w.double().T) < BF16_TOL


@pytest.mark.parametrize("M", [1, 3, 8, 16, 17, 33, 64, 65, 130, 300])
@pytest.mark.parametrize("N,K", [(50, 96), (130, 264), (16, 8), (257, 1024)])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_gemm_bf16(M, N, K, out_dtype):
    x, w, b = rand((M, K), torch.bfloat16, 13), rand((N, K), torch.bfloat16, 14), rand((N,), torch.float32, 15)
    out = ops().linear(x.to(dev()), w.to(dev()), b.to(dev()), out_dtype=out_dtype)
    expect = x.double() @ w.double().T + b.double()
    assert out.dtype == out_dtype
    assert rel_err(out, expect) < tol_of(out_dtype)


@pytest.mark.parametrize("M", [1, 16, 40, 64])
def test_gemm_bf16_skinny_and_tiled_agree(M):
    """The bfloat16 kernels may differ in rounding only (a bias keeps the product
    in this package's kernels at every M)."""
    x, w, b = rand((M, 512), torch.bfloat16, 16), rand((96, 512), torch.bfloat16, 17), rand((96,), torch.float32, 15)
    a = ops().linear(x.to(dev()), w.to(dev()), b.to(dev()), out_dtype=torch.float32)
    c = ops().linear(x.to(dev()), w.to(dev()), b.to(dev()), out_dtype=torch.float32, force_tiled=True)
    assert rel_err(a, c.double()) < F32_TOL


@pytest.mark.parametrize("partial_ok", [False, True])
def test_gemm_bf16_without_an_algorithm_of_the_library(monkeypatch, partial_ok):
    """Where the library names no algorithm for a shape (made so here), the product
    runs on this package's kernels, and the library's own answer agrees with theirs."""
    x, w = rand((40, 4096), torch.bfloat16, 42), rand((200, 4096), torch.bfloat16, 43)
    want = x.double() @ w.double().T

    def total(out):
        return out.sum(0) if out.dim() == 3 else out

    with_library = ops().linear(x.to(dev()), w.to(dev()), out_dtype=torch.float32, partial_ok=partial_ok)
    assert with_library.dim() == (3 if partial_ok else 2)
    monkeypatch.setattr(ops(), "_library_matmul", lambda *a: None)
    without = ops().linear(x.to(dev()), w.to(dev()), out_dtype=torch.float32, partial_ok=partial_ok)
    assert without.shape == (40, 200)
    assert rel_err(total(with_library), want) < F32_TOL and rel_err(without, want) < F32_TOL


@pytest.mark.parametrize("M", [17, 40, 64, 65, 300])
@pytest.mark.parametrize("N,K", [(50, 96), (257, 1024), (2048, 2048), (1000, 4096)])
def test_gemm_bf16_library_keeps_32_bits(M, N, K):
    """More rows than a decode batch, no bias: the library's product.  Asked for a
    32-bit result it must give the 32-bit sums, not a bfloat16 result widened: the
    error against 64-bit is that of 32-bit summation."""
    x, w = rand((M, K), torch.bfloat16, 40), rand((N, K), torch.bfloat16, 41)
    out = ops().linear(x.to(dev()), w.to(dev()), out_dtype=torch.float32)
    assert out.dtype == torch.float32 and out.shape == (M, N)
    assert rel_err(out, x.double() @ w.double().T) < F32_TOL
    low = ops().linear(x.to(dev()), w.to(dev()))
    assert low.dtype == torch.bfloat16
    assert rel_err(low, x.double() @ w.double().T) < BF16_TOL


@pytest.mark.parametrize("M,N,K", [(256, 2048, 2048), (700, 1000, 4096), (512, 520, 1024),
                                   (64, 3072, 2048), (20, 1000, 4096)])
def test_gemm_bf16_library_candidates_timed_at_first_use(M, N, K, monkeypatch):
    """The library's candidates for a shape are timed at its first call (below 256 rows
    with the weights out of the caches) and the fastest is kept: the result is a product like any other, a second call runs
    the same kernel (the same bits), a neighbouring row count takes the same choice, and
    with the timing switched off the first candidate gives the same product to rounding."""
    x, w = rand((M, K), torch.bfloat16, 140), rand((N, K), torch.bfloat16, 141)
    exact = x.double() @ w.double().T
    xd, wd = x.to(dev()), w.to(dev())
    monkeypatch.setattr(ops(), "library_tuning", True)
    first = ops().linear(xd, wd, out_dtype=torch.float32)
    assert rel_err(first, exact) < F32_TOL
    assert torch.equal(ops().linear(xd, wd, out_dtype=torch.float32), first)
    near = ops().linear(xd[:M - 3].contiguous(), wd, out_dtype=torch.float32)
    assert rel_err(near, exact[:M - 3]) < F32_TOL
    low = ops().linear(xd, wd)
    assert low.dtype == torch.bfloat16 and rel_err(low, exact) < BF16_TOL
    monkeypatch.setattr(ops(), "library_tuning", False)
    plain = ops().linear(xd, wd, out_dtype=torch.float32)
    assert rel_err(plain, exact) < F32_TOL
    assert torch.equal(ops().linear(xd, wd, out_dtype=torch.float32), plain)


def test_gemm_rows_do_not_depend_on_batch():
    """A token's projection is the same whatever else is in the step: bitwise
    within one of this package's kernels (each sums over k in an order fixed by K
    alone), within rounding between kernels and in the library."""
    x, w = rand((64, 256), torch.bfloat16, 18), rand((80, 256), torch.bfloat16, 19)
    bias = rand((80,), torch.float32, 20).to(dev())

    def run(m, **kw):
        return ops().linear(x[:m].contiguous().to(dev()), w.to(dev()), out_dtype=torch.float32, **kw).cpu()

    full = run(16)
    for m in (1, 5):
        assert torch.equal(run(m), full[:m])
    full = run(64, bias=bias)                            # with a bias: the kernel for 17..64 rows
    for m in (17, 33):
        assert torch.equal(run(m, bias=bias), full[:m])
    tiled = run(64, force_tiled=True)
    for m in (3, 40):
        assert torch.equal(run(m, force_tiled=True), tiled[:m])
    assert rel_err(run(16), tiled[:16].double()) < F32_TOL
    for m in (17, 33, 64):                               # the library
        assert rel_err(run(m), tiled[:m].double()) < F32_TOL
    x32, w32 = x.float(), w.float()
    full32 = ops().linear(x32.to(dev()), w32.to(dev())).cpu()
    part32 = ops().linear(x32[:3].contiguous().to(dev()), w32.to(dev())).cpu()
    assert torch.equal(part32, full32[:3])


@pytest.mark.parametrize("K", [8, 72, 512, 520, 2048, 2056, 4096, 8192, 8200])
@pytest.mark.parametrize("M,N", [(1, 48), (8, 50), (16, 33)])
def test_gemm_bf16_decode_rows_all_k_ranges(M, N, K):
    """The decode kernel picks its shape by K; every range, with tails."""
    x, w, b = rand((M, K), torch.bfloat16, 27), rand((N, K), torch.bfloat16, 28), rand((N,), torch.float32, 29)
    out = ops().linear(x.to(dev()), w.to(dev()), b.to(dev()), out_dtype=torch.float32)
    assert rel_err(out, x.double() @ w.double().T + b.double()) < F32_TOL


@pytest.mark.parametrize("M,N,K", [(1, 64, 4096), (8, 2048, 8192), (16, 2048, 8192), (8, 100, 4160),
                                   (3, 4096, 4096)])
def test_gemm_bf16_partial_sums(M, N, K):
    """K split over workgroups: the stack of partial results sums to the product."""
    x, w, b = rand((M, K), torch.bfloat16, 30), rand((N, K), torch.bfloat16, 31), rand((N,), torch.float32, 32)
    stack = ops().linear(x.to(dev()), w.to(dev()), b.to(dev()), partial_ok=True)
    assert stack.dim() == 3 and stack.dtype == torch.float32 and stack.shape[0] in (2, 4)
    assert rel_err(stack.sum(0), x.double() @ w.double().T + b.double()) < F32_TOL
    many = ops().linear(rand((1100, K), torch.bfloat16, 33).to(dev()), w.to(dev()), partial_ok=True)
    assert many.dim() == 2                                  # beyond 1,024 rows nothing is split


def test_library_product_again_on_the_same_operands():
    """The library is called through a prepared instance once a shape's operands have
    been seen before (the allocator hands the same addresses back): every call gives
    the bits of the first, with and without ranges of K, and other contents at the same
    addresses give their own result."""
    o = ops()
    x, w = rand((40, 1024), torch.bfloat16, 44).to(dev()), rand((96, 1024), torch.bfloat16, 45).to(dev())
    for kw in ({}, {"partial_ok": True}, {"out_dtype": torch.float32}):
        first = o.linear(x, w, **kw).clone()
        for _ in range(8):
            y = o.linear(x, w, **kw)
            assert torch.equal(y, first)
            del y
    expect = x.double().cpu() @ w.double().cpu().T
    assert rel_err(o.linear(x, w, out_dtype=torch.float32), expect) < F32_TOL
    x.mul_(-2)                                            # same address, other contents
    for _ in range(3):
        assert rel_err(o.linear(x, w, out_dtype=torch.float32), -2 * expect) < F32_TOL


def test_library_products_when_the_table_of_instances_is_full():
    """With room for four prepared instances and twelve shapes called in turn, the table
    is emptied again and again (after the device has finished): every result is right."""
    import os
    import subprocess
    import sys
    code = (
        "import torch\n"
        "from zig_ai_amd.kernels import ops\n"
        "dev = torch.device('cuda', 0)\n"
        "g = torch.Generator().manual_seed(3)\n"
        "w = torch.randn(64, 256, generator=g).to(torch.bfloat16)\n"
        "xs = [torch.randn(17 + i, 256, generator=g).to(torch.bfloat16) for i in range(12)]\n"
        "wd, xd = w.to(dev), [x.to(dev) for x in xs]\n"
        "worst = 0.0\n"
        "for turn in range(6):\n"
        "    for x, xg in zip(xs, xd):\n"
        "        y = ops.linear(xg, wd, out_dtype=torch.float32).double().cpu()\n"
        "        e = x.double() @ w.double().T\n"
        "        worst = max(worst, float((y - e).abs().max() / e.abs().max()))\n"
        "print('worst', worst)\n")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    for limit in ("4", "0"):
        env = dict(os.environ, ZIG_AI_GEMM_INSTANCES=limit, PYTHONPATH=root)
        out = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True,
                             timeout=300)
        assert out.returncode == 0, out.stderr[-2000:]
        assert float(out.stdout.split()[-1]) < F32_TOL, out.stdout


def _normed_operands(x: torch.Tensor, weight: torch.Tensor, eps: float):
    """What the decode kernels make of a norm handed to them: the operands
    bf16(x * weight) and the row's scale, which multiplies the 32-bit sums."""
    xd = x.double()
    scale = 1.0 / torch.sqrt((xd * xd).mean(-1, keepdim=True) + eps)
    return (x * weight).to(torch.bfloat16).double(), scale


@pytest.mark.parametrize("K", [8, 512, 520, 1024, 1536, 2048, 2560, 3584, 4096, 4608])
@pytest.mark.parametrize("M,N", [(1, 48), (8, 50), (16, 33), (16, 16400), (11, 16385), (9, 200), (13, 96)])
def test_gemm_bf16_decode_rows_normalised_by_the_kernel(M, N, K):
    """A norm that has not run yet as the product's input: every K the fused form takes
    (multiples of 512 up to 4096, also those that leave waves idle; up to 16 rows, nine
    and more in two turns through LDS) and some it does not, with a bias, and rows picked
    out of a longer stream.  The
    row's scale is applied to the 32-bit sums, so against the same operands the error
    is that of 32-bit summation; against the norm as a kernel of its own (which rounds
    after scaling) it is one bfloat16 rounding."""
    eps = 1e-5
    stream = rand((M + 3, K), torch.float32, 50) * 3.0
    nw = 1.0 + rand((K,), torch.float32, 51)
    w, b = rand((N, K), torch.bfloat16, 52), rand((N,), torch.float32, 53)
    rows = torch.tensor([(5 * i + 2) % (M + 3) for i in range(M)], dtype=torch.int32)
    o = ops()
    for pick in (None, rows):
        x = stream[:M] if pick is None else stream[pick.long()]
        src = stream[:M].contiguous() if pick is None else stream
        normed = o.NormedRows(src.to(dev()), nw.to(dev()), eps, torch.bfloat16,
                              None if pick is None else pick.to(dev()))
        assert normed.shape == (M, K)
        out = o.linear(normed, w.to(dev()), b.to(dev()), out_dtype=torch.float32)
        if o.normed_rows_pay(M, N, K):
            a, scale = _normed_operands(x, nw, eps)
            assert rel_err(out, scale * (a @ w.double().T) + b.double()) < F32_TOL
        separate = o.linear(normed.materialise(), w.to(dev()), b.to(dev()), out_dtype=torch.float32)
        assert rel_err(out, separate.double()) < BF16_TOL
        # both at once: the norm on the way in, the sum added to a stream on the way out
        base = rand((M, N), torch.float32, 49)
        stream_out = base.clone().to(dev())
        assert o.linear(normed, w.to(dev()), b.to(dev()), accumulate=stream_out) is None
        assert rel_err(stream_out, base.double() + out.double().cpu()) < F32_TOL
        exact = plain.rms_norm(x.double(), nw.double(), eps) @ w.double().T + b.double()
        assert rel_err(out, exact) < BF16_TOL


def test_a_product_that_reads_and_adds_to_the_same_stream():
    """``linear(NormedRows(stream), W[H, H], accumulate=stream)``: workgroups would read rows
    of the stream while others add to them; the norm is run first instead, and the result is
    stream + norm(stream as it was) W^T."""
    o = ops()
    H = 2048
    x0 = rand((8, H), torch.float32, 90)
    nw = rand((H,), torch.float32, 91, 0.2) + 1
    w = rand((H, H), torch.bfloat16, 92, 0.05)
    stream = x0.to(dev())
    normed = o.NormedRows(stream, nw.to(dev()), 1e-5, torch.bfloat16)
    assert o.linear(normed, w.to(dev()), accumulate=stream) is None
    a = plain.rms_norm(x0.double(), nw.double(), 1e-5).to(torch.bfloat16).double()
    assert rel_err(stream, x0.double() + a @ w.double().T) < 1e-4
    # with another tensor to add to, the kernel runs the norm itself
    other = torch.zeros((8, H), dtype=torch.float32, device=dev())
    o.form_log = []
    try:
        o.linear(o.NormedRows(x0.to(dev()), nw.to(dev()), 1e-5, torch.bfloat16), w.to(dev()), accumulate=other)
        assert o.form_log[-1]["norm_in_product"] and o.form_log[-1]["added_to_stream"]
    finally:
        o.form_log = None
    assert rel_err(other, a @ w.double().T) < BF16_TOL


def test_normed_rows_beyond_the_fused_kernel_run_the_norm_kernel():
    """More than 16 rows, a K no workgroup covers, 32-bit weights: the norm runs as a
    kernel of its own and the product is the usual one."""
    o = ops()
    eps = 1e-6
    for M, K, wdtype in ((17, 512, torch.bfloat16), (4, 4608, torch.bfloat16), (4, 520, torch.bfloat16),
                         (4, 512, torch.float32)):
        x = rand((M, K), torch.float32, 54)
        nw = 1.0 + rand((K,), torch.float32, 55)
        w = rand((24, K), wdtype, 56)
        dtype = torch.bfloat16 if wdtype == torch.bfloat16 else torch.float32
        normed = o.NormedRows(x.to(dev()), nw.to(dev()), eps, dtype)
        out = o.linear(normed, w.to(dev()), out_dtype=torch.float32)
        same = o.linear(normed.materialise(), w.to(dev()), out_dtype=torch.float32)
        assert torch.equal(out, same)
        exact = plain.rms_norm(x.double(), nw.double(), eps) @ w.double().T
        assert rel_err(out, exact) < (BF16_TOL if dtype == torch.bfloat16 else F32_TOL)


@pytest.mark.parametrize("M,I,K", [(1, 40, 512), (8, 100, 1536), (16, 256, 2048), (5, 72, 4096)])
def test_linear_swiglu_normalised_by_the_kernel(M, I, K):
    eps = 1e-5
    x = rand((M, K), torch.float32, 57) * 2.0
    nw = 1.0 + rand((K,), torch.float32, 58)
    w = rand((2 * I, K), torch.bfloat16, 59)
    o = ops()
    normed = o.NormedRows(x.to(dev()), nw.to(dev()), eps, torch.bfloat16)
    out = o.linear_swiglu(normed, w.to(dev()))
    a, scale = _normed_operands(x, nw, eps)
    gu = scale * (a @ w.double().T)
    g, u = gu[:, :I], gu[:, I:]
    assert out.dtype == torch.bfloat16
    assert rel_err(out, g / (1 + torch.exp(-g)) * u) < BF16_TOL


@pytest.mark.parametrize("M,N,K", [(1, 64, 4096), (8, 2048, 8192), (16, 2048, 2048), (8, 100, 4160),
                                   (3, 4096, 512), (8, 2048, 16384), (2, 40, 72),
                                   (8, 6144, 12288), (3, 8192, 28672), (16, 5136, 9216),
                                   (2, 48, 8200)])
def test_gemm_bf16_decode_rows_added_to_the_stream(M, N, K):
    """A decode batch's product added to the 32-bit stream by the kernel itself, K in
    as many ranges as fill the chip; twice, since the stream keeps what it holds.  Wide
    models (many outputs AND a long K) get more ranges than the chip wants rather than a
    range longer than a workgroup covers; a K that no cut fits (8200) comes back as a
    product instead."""
    x, w, b = rand((M, K), torch.bfloat16, 60), rand((N, K), torch.bfloat16, 61), rand((N,), torch.float32, 62)
    stream0 = rand((M, N), torch.float32, 63)
    stream = stream0.to(dev())
    o = ops()
    product = x.double() @ w.double().T + b.double()
    if o.accumulate_plan(M, N, K, False) == 0:
        back = o.linear(x.to(dev()), w.to(dev()), b.to(dev()), accumulate=stream)
        assert back is not None and torch.equal(stream.cpu(), stream0)
        assert rel_err(back, product) < BF16_TOL
        return
    assert o.linear(x.to(dev()), w.to(dev()), b.to(dev()), partial_ok=True, accumulate=stream) is None
    assert rel_err(stream, stream0.double() + product) < F32_TOL
    assert o.linear(x.to(dev()), w.to(dev()), b.to(dev()), accumulate=stream) is None
    assert rel_err(stream, stream0.double() + 2 * product) < F32_TOL
    # more rows than any kernel that adds takes, or 32-bit weights: the product comes back instead
    many = rand((70, K), torch.bfloat16, 64).to(dev())
    kept = torch.zeros((70, N), dtype=torch.float32, device=dev())
    back = o.linear(many, w.to(dev()), accumulate=kept)
    assert back is not None and not kept.any()
    kept = torch.zeros((M, N), dtype=torch.float32, device=dev())
    back = o.linear(x.float().to(dev()), w.float().to(dev()), accumulate=kept)
    assert back is not None and not kept.any()


@pytest.mark.parametrize("src_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("dst_dtype", [torch.float32, torch.bfloat16])
def test_copy_columns(src_dtype, dst_dtype):
    """Columns of a matrix's rows into a new tensor or into columns of another: exact when
    the types agree or widen, one rounding when they narrow; everything else untouched."""
    o = ops()
    src = rand((37, 100), src_dtype, 120)
    part = o.copy_columns(src.to(dev()), 13, 50, dtype=dst_dtype)
    assert part.shape == (37, 50) and part.dtype == dst_dtype
    assert torch.equal(part.cpu(), src[:, 13:63].to(dst_dtype))
    out = rand((37, 77), dst_dtype, 121)
    on_device = out.clone().to(dev())
    assert o.copy_columns(src.to(dev()), 90, 10, on_device, 60) is on_device
    want = out.clone()
    want[:, 60:70] = src[:, 90:100].to(dst_dtype)
    assert torch.equal(on_device.cpu(), want)
    with pytest.raises(o.KernelError):
        o.copy_columns(src.to(dev()), 95, 10)
    with pytest.raises(o.KernelError):
        o.copy_columns(src.to(dev()), 0, 10, on_device, 70)


# ------------------------------------------------- products of 17 to 64 rows, fused forms
@pytest.mark.parametrize("M", [1, 5, 17, 20, 32, 33, 47, 64])
@pytest.mark.parametrize("N,K", [(50, 1024), (200, 1536), (6144, 2048), (130, 4096), (64, 2560)])
def test_rows64_products(M, N, K):
    """The kernel for steps of 17 to 64 rows, alone: every number of row blocks (and fewer
    rows than a block), tiles with tails in N, two to eight spans of K, odd numbers of
    spans; stored, with the norm run by the kernel (rows picked out of a longer stream),
    through the SwiGLU gate, and added to a stream with K in ranges."""
    o = ops()
    eps = 1e-5
    w = rand((N, K), torch.bfloat16, 80)
    x = rand((M, K), torch.bfloat16, 81)
    exact = x.double() @ w.double().T
    got = o.linear_rows64(x.to(dev()), w.to(dev()))
    assert got.dtype == torch.bfloat16 and rel_err(got, exact) < BF16_TOL
    # the norm on the way in
    stream = rand((M + 3, K), torch.float32, 82) * 3.0
    nw = 1.0 + rand((K,), torch.float32, 83)
    rows = torch.tensor([(5 * i + 2) % (M + 3) for i in range(M)], dtype=torch.int32)
    for pick in (None, rows):
        xs = stream[:M] if pick is None else stream[pick.long()]
        src = stream[:M].contiguous() if pick is None else stream
        normed = o.NormedRows(src.to(dev()), nw.to(dev()), eps, torch.bfloat16,
                              None if pick is None else pick.to(dev()))
        a, scale = _normed_operands(xs, nw, eps)
        want = scale * (a @ w.double().T)
        assert rel_err(o.linear_rows64(normed, w.to(dev())), want) < BF16_TOL
        if N % 2 == 0:
            I = N // 2
            g, u = want[:, :I], want[:, I:]
            gated = o.linear_rows64(normed, w.to(dev()), mode=o.ROWS64_SWIGLU)
            assert gated.shape == (M, I) and rel_err(gated, g / (1 + torch.exp(-g)) * u) < BF16_TOL
    # added to a stream, K in every number of ranges the kernel takes
    for ks in (1, 2, 3, 4):
        if not o.rows64_takes(M, K, ks):
            continue
        base = rand((M, N), torch.float32, 84)
        on_device = base.clone().to(dev())
        assert o.linear_rows64(x.to(dev()), w.to(dev()), mode=o.ROWS64_ADD, accumulate=on_device,
                               ksplit=ks) is None
        assert rel_err(on_device, base.double() + exact) < F32_TOL
        o.linear_rows64(x.to(dev()), w.to(dev()), mode=o.ROWS64_ADD, accumulate=on_device, ksplit=ks)
        assert rel_err(on_device, base.double() + 2 * exact) < F32_TOL


def test_rows64_rows_do_not_depend_on_the_batch():
    """A row's result is a function of that row: the same bits whichever rows stand beside
    it and wherever it stands (the sums over K run in one order for every row)."""
    o = ops()
    N, K = 300, 2048
    w = rand((N, K), torch.bfloat16, 85).to(dev())
    x = rand((64, K), torch.bfloat16, 86)
    whole = o.linear_rows64(x.to(dev()), w).cpu()
    some = o.linear_rows64(x[10:30].contiguous().to(dev()), w).cpu()
    assert torch.equal(some, whole[10:30])
    one = o.linear_rows64(x[63:64].contiguous().to(dev()), w).cpu()
    assert torch.equal(one, whole[63:64])


def test_rows64_refuses_what_it_does_not_take():
    o = ops()
    w = rand((64, 1024), torch.bfloat16, 87).to(dev())
    with pytest.raises(o.KernelError, match="64 rows"):
        o.linear_rows64(rand((65, 1024), torch.bfloat16, 88).to(dev()), w)
    for K in (512, 1000, 1280):                         # one span only; no multiple of 512
        wk = rand((64, K), torch.bfloat16, 89).to(dev())
        with pytest.raises(o.KernelError):
            o.linear_rows64(rand((20, K), torch.bfloat16, 90).to(dev()), wk)
    with pytest.raises(o.KernelError):                  # ranges of K only when adding
        o.linear_rows64(rand((20, 2048), torch.bfloat16, 91).to(dev()),
                        rand((64, 2048), torch.bfloat16, 92).to(dev()), ksplit=2)
    # the norm's weight lies in LDS: K up to 4096
    wide = o.NormedRows(rand((20, 8192), torch.float32, 93).to(dev()),
                        rand((8192,), torch.float32, 94).to(dev()), 1e-5, torch.bfloat16)
    with pytest.raises(o.KernelError, match="does not support"):
        o.linear_rows64(wide, rand((64, 8192), torch.bfloat16, 95).to(dev()))
    assert not o.rows64_swiglu_fusable(20, 8192) and not o.rows64_swiglu_fusable(16, 2048)
    assert o.rows64_swiglu_fusable(17, 2048) and o.rows64_swiglu_fusable(32, 1024)
    assert o.rows64_swiglu_fusable(48, 2048) and not o.rows64_swiglu_fusable(49, 2048)
    assert o.rows64_swiglu_fusable(64, 1024) and not o.rows64_swiglu_fusable(65, 1024)


@pytest.mark.parametrize("M", [17, 24, 32])
def test_steps_of_17_to_32_rows_through_linear(M):
    """What the parts call: ``linear(..., accumulate=stream)`` of such a step adds to the
    stream itself (and says so): through the library where a fused feed-forward can follow
    on a stream of that width, else on this package's kernel; ``linear_swiglu`` takes rows
    that await their norm; with a long K the product comes back."""
    o = ops()
    K = 2048
    x = rand((M, K), torch.bfloat16, 97)
    for N, kernel in ((3072, "library"), (3080, "rows64")):
        w = rand((N, K), torch.bfloat16, 96)
        base = rand((M, N), torch.float32, 98)
        on_device = base.clone().to(dev())
        o.form_log = []
        try:
            for _ in range(2):               # (a first call times the library's candidates)
                assert o.linear(x.to(dev()), w.to(dev()), partial_ok=True, accumulate=on_device) is None
            log = o.form_log
        finally:
            o.form_log = None
        assert log[-1]["added_to_stream"] and log[-1].get("kernel") == kernel
        assert rel_err(on_device, base.double() + 2.0 * (x.double() @ w.double().T)) < F32_TOL
    N = 3072
    w = rand((N, K), torch.bfloat16, 96)
    long_k = rand((256, 8192), torch.bfloat16, 99).to(dev())
    kept = torch.zeros((M, 256), dtype=torch.float32, device=dev())
    back = o.linear(rand((M, 8192), torch.bfloat16, 100).to(dev()), long_k, partial_ok=True, accumulate=kept)
    assert back is not None and not kept.any()
    stream = rand((M, K), torch.float32, 101) * 2.0
    nw = 1.0 + rand((K,), torch.float32, 102)
    normed = o.NormedRows(stream.to(dev()), nw.to(dev()), 1e-5, torch.bfloat16)
    out = o.linear_swiglu(normed, w.to(dev()))
    a, scale = _normed_operands(stream, nw, 1e-5)
    gu = scale * (a @ w.double().T)
    g, u = gu[:, :N // 2], gu[:, N // 2:]
    assert rel_err(out, g / (1 + torch.exp(-g)) * u) < BF16_TOL
    with pytest.raises(o.KernelError):                  # plain rows of such a step: not this call
        o.linear_swiglu(x.to(dev()), w.to(dev()))


@pytest.mark.parametrize("M,N,K", [(1100, 520, 4096), (2048, 2048, 8192), (1025, 136, 4104)])
def test_library_product_added_to_the_stream(M, N, K):
    """Beyond 1,024 rows a product with K >= 4096 that is asked to add itself to the stream
    does so in the GEMM library (twice in a row: the second is added to the first; timing
    the library's candidates at the first call leaves the stream alone); a shorter K, or
    fewer rows, comes back or goes the ways tested above."""
    o = ops()
    assert o.library_adds(M, N, K) and not o.library_adds(M, N, 2048) and not o.library_adds(1024, N, K)
    w = rand((N, K), torch.bfloat16, 140)
    x = rand((M, K), torch.bfloat16, 141)
    base = rand((M, N), torch.float32, 142) * 3.0
    stream = base.clone().to(dev())
    o.form_log = []
    try:
        for _ in range(2):
            assert o.linear(x.to(dev()), w.to(dev()), partial_ok=True, accumulate=stream) is None
        log = o.form_log
    finally:
        o.form_log = None
    assert all(r["added_to_stream"] and r.get("kernel") == "library" for r in log[-2:])
    assert rel_err(stream, base.double() + 2.0 * (x.double() @ w.double().T)) < F32_TOL
    short = torch.zeros((M, N), dtype=torch.float32, device=dev())
    back = o.linear(x[:, :2048].contiguous().to(dev()), w[:, :2048].contiguous().to(dev()),
                    partial_ok=True, accumulate=short)
    assert back is not None and not short.any()


def library_ranges(M, N, K):
    """The documented choice: with few outputs, K >= 4096 goes in 8 ranges up to 256 rows
    and in 4 up to 1,024, K >= 2048 in 4 ranges up to 128 rows; a range is a multiple of
    128 elements."""
    choices = ()
    if N <= 4096 and K >= 4096 and M <= 1024:
        choices = (8, 4, 2) if M <= 256 else (4, 2)
    elif N <= 4096 and K >= 2048 and M <= 128:
        choices = (4, 2)
    return next((p for p in choices if K % (p * 128) == 0), 1)


@pytest.mark.parametrize("M", [17, 40, 64, 128, 200, 300, 700, 1100])
@pytest.mark.parametrize("N,K", [(2048, 8192), (2048, 2048), (300, 4096), (1024, 4608), (2048, 4160),
                                 (6144, 2048), (64, 1024)])
def test_gemm_bf16_library_partial_sums(M, N, K):
    """Beyond a decode batch the library is given K in ranges when N is small: the
    stack of 32-bit partial results sums to the product."""
    x, w = rand((M, K), torch.bfloat16, 42), rand((N, K), torch.bfloat16, 43)
    out = ops().linear(x.to(dev()), w.to(dev()), partial_ok=True)
    expect = x.double() @ w.double().T
    split = library_ranges(M, N, K)
    if split > 1:
        assert out.dim() == 3 and out.dtype == torch.float32 and out.shape == (split, M, N)
        assert out.is_contiguous()
        assert rel_err(out.sum(0), expect) < F32_TOL
        part = x[:, :K // split].double() @ w[:, :K // split].double().T
        assert rel_err(out[0], part) < F32_TOL
    else:
        assert out.shape == (M, N) and out.dtype == torch.bfloat16
        assert rel_err(out, expect) < BF16_TOL


@pytest.mark.parametrize("M,N,K,split", [(8, 2048, 2048, 2), (16, 1024, 3072, 2), (1, 2048, 2080, 1),
                                         (8, 6144, 2048, 1), (4, 64, 1024, 1)])
def test_gemm_bf16_decode_rows_split_short_k(M, N, K, split):
    x, w = rand((M, K), torch.bfloat16, 44), rand((N, K), torch.bfloat16, 45)
    out = ops().linear(x.to(dev()), w.to(dev()), partial_ok=True)
    expect = x.double() @ w.double().T
    if split > 1:
        assert out.shape == (split, M, N) and out.dtype == torch.float32
        assert rel_err(out.sum(0), expect) < F32_TOL
    else:
        assert out.shape == (M, N) and out.dtype == torch.bfloat16
        assert rel_err(out, expect) < BF16_TOL


@pytest.mark.parametrize("M,I,K", [(1, 48, 64), (8, 8192, 2048), (16, 100, 520), (5, 176, 96),
                                   (3, 40, 8192), (8, 33000, 64)])
def test_linear_swiglu(M, I, K):
    """The gate applied to the projection's accumulators equals projection, then gate."""
    x, w = rand((M, K), torch.bfloat16, 34), rand((2 * I, K), torch.bfloat16, 35, 0.1)
    out = ops().linear_swiglu(x.to(dev()), w.to(dev()))
    gu = x.double() @ w.double().T
    assert out.shape == (M, I) and out.dtype == torch.bfloat16
    assert rel_err(out, torch.nn.functional.silu(gu[:, :I]) * gu[:, I:]) < BF16_TOL


def test_gemm_bf16_refuses_odd_k():
    from zig_ai_amd.kernels import KernelError
    x, w = rand((4, 12), torch.bfloat16, 20), rand((8, 12), torch.bfloat16, 21)
    with pytest.raises(KernelError, match="multiple of 8"):
        ops().linear(x.to(dev()), w.to(dev()))


# ---------------------------------------------------------------- rope + cache
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh,nkv,d,rot,pairing", [
    (4, 2, 16, 16, "half"), (3, 1, 32, 32, "half"), (5, 5, 48, 48, "adjacent"),
    (8, 2, 64, 32, "half"), (2, 2, 256, 256, "half"), (6, 3, 128, 64, "adjacent"),
    (4, 2, 64, 24, "half"), (8, 2, 64, 64, "adjacent"), (7, 7, 32, 16, "half"), (32, 8, 64, 64, "half")])
def test_qk_norm_rope_kv_write(dtype, nh, nkv, d, rot, pairing):
    T, page_size, pages = 11, 4, 9
    theta, eps = 10000.0, 1e-5
    qkv = rand((T, (nh + 2 * nkv) * d), dtype, 22)
    qw, kw = rand((d,), torch.float32, 23) + 1.0, rand((d,), torch.float32, 24) + 1.0
    positions = torch.tensor([0, 1, 2, 3, 100, 101, 7, 8, 9, 10, 11], dtype=torch.int32)
    perm = torch.randperm(pages * page_size, generator=torch.Generator().manual_seed(25))[:T]
    slots = perm.to(torch.int32)
    inv = (1.0 / torch.pow(torch.tensor(theta, dtype=torch.float64),
                           2.0 * torch.arange(0, rot // 2, dtype=torch.float64) / rot)).float()
    cache = torch.zeros((pages, 2, nkv, page_size, d), dtype=dtype, device=dev())
    q = ops().qk_norm_rope_kv_write(qkv.to(dev()), positions.to(dev()), slots.to(dev()),
                                    qw.to(dev()), kw.to(dev()), inv.to(dev()), cache, nh, nkv, d,
                                    rot, pairing == "adjacent", eps)
    heads = qkv.double().view(T, nh + 2 * nkv, d)
    qe = plain.apply_rope(plain.rms_norm(heads[:, :nh], qw.double(), eps), positions, theta, rot, pairing)
    ke = plain.apply_rope(plain.rms_norm(heads[:, nh:nh + nkv], kw.double(), eps), positions, theta,
                          rot, pairing)
    ve = heads[:, nh + nkv:]
    # angles are computed in 32-bit: position 101 * 2^-24 relative error in the angle
    tol = tol_of(dtype) + 101 * 1.2e-7
    assert rel_err(q, qe) < tol
    c = cache.cpu()
    got_k = torch.stack([c[s // page_size, 0, :, s % page_size, :] for s in slots.tolist()])
    cv = c[:, 1].reshape(pages, nkv, d, page_size)        # values: [kv_head][head_dim][offset]
    got_v = torch.stack([cv[s // page_size, :, :, s % page_size] for s in slots.tolist()])
    assert rel_err(got_k, ke) < tol
    assert torch.equal(got_v.double(), ve)                 # values are stored as they are
    written = torch.zeros(pages * page_size, dtype=torch.bool)
    written[slots.long()] = True
    untouched_k = c[:, 0].permute(0, 2, 1, 3).reshape(pages * page_size, -1)[~written]
    untouched_v = cv.permute(0, 3, 1, 2).reshape(pages * page_size, -1)[~written]
    assert (untouched_k == 0).all() and (untouched_v == 0).all()   # nothing else was touched


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh,nkv,d,rot,pairing,page_size", [
    (32, 8, 64, 64, "half", 16), (3, 1, 128, 128, "half", 8), (4, 2, 32, 16, "adjacent", 16),
    (8, 2, 64, 64, "half", 4), (2, 2, 16, 16, "adjacent", 32)])
def test_qk_norm_rope_kv_write_many_tokens(dtype, nh, nkv, d, rot, pairing, page_size):
    """A step with prompt portions: blocks take eight tokens each and store the
    values of eight neighbouring offsets side by side.  Stretches that start at a
    multiple of eight, one that starts at offset 5, single decoded tokens between
    them, a tail that is no multiple of eight: bit for bit what the same tokens give
    in calls small enough to go one token per block, and right."""
    theta, eps = 10000.0, 1e-5
    stretches = [(0, 0, 64), (1, 5, 70), (2, 300, 1), (3, 17, 1), (4, 32, 40), (5, 999, 1),
                 (6, 8, 27)]                          # (request, first position, tokens)
    per_req = (1024 + page_size - 1) // page_size + 1
    pages = per_req * len(stretches)
    order = torch.randperm(pages, generator=torch.Generator().manual_seed(31)).tolist()
    positions, slots = [], []
    for r, first, n in stretches:
        for p in range(first, first + n):
            positions.append(p)
            slots.append(order[r * per_req + p // page_size] * page_size + p % page_size)
    T = len(positions)
    assert T >= 128 and T % 8 != 0
    positions = torch.tensor(positions, dtype=torch.int32)
    slots = torch.tensor(slots, dtype=torch.int32)
    qkv = rand((T, (nh + 2 * nkv) * d), dtype, 32)
    qw, kw = rand((d,), torch.float32, 33) + 1.0, rand((d,), torch.float32, 34) + 1.0
    inv = (1.0 / torch.pow(torch.tensor(theta, dtype=torch.float64),
                           2.0 * torch.arange(0, rot // 2, dtype=torch.float64) / rot)).float()

    def run(cuts):
        cache = torch.zeros((pages, 2, nkv, page_size, d), dtype=dtype, device=dev())
        qs = []
        for a, b in zip(cuts[:-1], cuts[1:]):
            qs.append(ops().qk_norm_rope_kv_write(
                qkv[a:b].contiguous().to(dev()), positions[a:b].to(dev()), slots[a:b].to(dev()),
                qw.to(dev()), kw.to(dev()), inv.to(dev()), cache, nh, nkv, d, rot,
                pairing == "adjacent", eps))
        return torch.cat(qs).cpu(), cache.cpu()

    q_all, cache_all = run([0, T])
    q_few, cache_few = run(list(range(0, T, 50)) + [T])
    assert torch.equal(q_all, q_few) and torch.equal(cache_all, cache_few)
    heads = qkv.double().view(T, nh + 2 * nkv, d)
    qe = plain.apply_rope(plain.rms_norm(heads[:, :nh], qw.double(), eps), positions, theta, rot, pairing)
    ke = plain.apply_rope(plain.rms_norm(heads[:, nh:nh + nkv], kw.double(), eps), positions, theta,
                          rot, pairing)
    tol = tol_of(dtype) + 1100 * 1.2e-7
    assert rel_err(q_all, qe) < tol
    got_k = torch.stack([cache_all[s // page_size, 0, :, s % page_size, :] for s in slots.tolist()])
    cv = cache_all[:, 1].reshape(pages, nkv, d, page_size)
    got_v = torch.stack([cv[s // page_size, :, :, s % page_size] for s in slots.tolist()])
    assert rel_err(got_k, ke) < tol
    assert torch.equal(got_v.double(), heads[:, nh + nkv:])
    written = torch.zeros(pages * page_size, dtype=torch.bool)
    written[slots.long()] = True
    untouched_v = cv.permute(0, 3, 1, 2).reshape(pages * page_size, -1)[~written]
    assert (untouched_v == 0).all()


def test_rope_position_zero_is_identity_and_norm_is_kept():
    """rope.zig:226-253 holds the rotation to preserving the norm; position 0 rotates
    by nothing."""
    nh, nkv, d = 2, 1, 64
    T = 6
    qkv = rand((T, (nh + 2 * nkv) * d), torch.float32, 26)
    positions = torch.tensor([0, 1, 5, 50, 500, 4000], dtype=torch.int32)
    inv = (1.0 / torch.pow(torch.tensor(10000.0, dtype=torch.float64),
                           2.0 * torch.arange(0, d // 2, dtype=torch.float64) / d)).float()
    q = ops().qk_norm_rope_kv_write(qkv.to(dev()), positions.to(dev()), None, None, None,
                                    inv.to(dev()), None, nh, nkv, d, d, False, 0.0,
                                    write_kv=False).cpu()
    src = qkv.view(T, nh + 2 * nkv, d)[:, :nh]
    assert torch.equal(q[0], src[0])
    assert torch.allclose(q.norm(dim=-1), src.norm(dim=-1), rtol=1e-5)


# ------------------------------------------------------------------ attention
def paged_from_dense(k, v, page_size, dtype, extra_pages=3, seed=0):
    """Scatter dense per-request K/V ``[len, nkv, d]`` into a shuffled paged cache
    (per page: keys [kv_head][offset][head_dim], then values [kv_head][head_dim][offset]).
    Returns cache, block table [S, max_pages]."""
    nkv, d = k[0].shape[1], k[0].shape[2]
    need = [(x.shape[0] + page_size - 1) // page_size for x in k]
    total = sum(need) + extra_pages
    order = torch.randperm(total, generator=torch.Generator().manual_seed(seed)).tolist()
    cache = torch.zeros((total, 2, nkv, page_size, d), dtype=dtype)
    # poison pages nobody owns so that a stray read shows
    table = torch.full((len(k), max(need)), -1, dtype=torch.int32)
    nxt = 0
    for s, (ks, vs) in enumerate(zip(k, v)):
        for p in range(need[s]):
            page = order[nxt]
            nxt += 1
            table[s, p] = page
            lo, hi = p * page_size, min((p + 1) * page_size, ks.shape[0])
            cache[page, 0, :, : hi - lo] = ks[lo:hi].transpose(0, 1).to(dtype)
            # values are stored turned round: [kv_head][head_dim][offset]
            cache[page, 1].view(nkv, d, page_size)[:, :, : hi - lo] = vs[lo:hi].permute(1, 2, 0).to(dtype)
    for page in order[nxt:]:
        cache[page] = 1e4
    return cache, table


def items_for(seq_lens, rows_per_item):
    """The kernels' work items, laid out here and not by the engine's own code: runs of
    at most ``rows_per_item`` consecutive query rows of one request."""
    seq, row0, cnt = [], [], []
    first = 0
    for s, n in enumerate(seq_lens):
        for lo in range(0, n, rows_per_item):
            seq.append(s)
            row0.append(first + lo)
            cnt.append(min(rows_per_item, n - lo))
        first += n
    mk = lambda x: torch.tensor(x, dtype=torch.int32, device=dev())
    return mk(seq), mk(row0), mk(cnt), len(seq)


def run_attention(dtype, nh, nkv, d, page_size, ctx, new, window=0, keys_per_split=0, nsplit=1,
                  seed=30, sharpen=False, mfma=False, mfma_decode=False, tile_keys=64):
    """ctx[s] cached tokens and new[s] query tokens per request."""
    G = nh // nkv
    ks, vs, qs, pos = [], [], [], []
    for s, (c, n) in enumerate(zip(ctx, new)):
        k = rand((c + n, nkv, d), dtype, seed + 3 * s)
        v = rand((c + n, nkv, d), dtype, seed + 3 * s + 1)
        q = rand((n, nh, d), dtype, seed + 3 * s + 2)
        if sharpen and c > 3:
            # one far key matches the last query strongly: its value must dominate
            k[1] = 0
            k[1, :, 0] = 8.0
            q[-1] = 0
            q[-1, :, 0] = 8.0
        ks.append(k); vs.append(v); qs.append(q)
        pos += list(range(c, c + n))
    cache, table = paged_from_dense(ks, vs, page_size, dtype, seed=seed)
    q_all = torch.cat(qs).to(dev())
    positions = torch.tensor(pos, dtype=torch.int32, device=dev())
    if mfma_decode:
        out = ops().paged_attention_decode_mfma(q_all, cache.to(dev()), table.to(dev()), positions,
                                                *items_for(new, max(1, 16 // G)),
                                                1.0 / math.sqrt(d), window, keys_per_split, nsplit)
    elif mfma:
        out = ops().paged_attention_mfma(q_all, cache.to(dev()), table.to(dev()), positions,
                                         *items_for(new, max(1, 128 // G)), 1.0 / math.sqrt(d),
                                         window, keys_per_split, nsplit, tile_keys=tile_keys)
    else:
        out = ops().paged_attention(q_all, cache.to(dev()), table.to(dev()), positions,
                                    *items_for(new, max(1, 32 // G)), 1.0 / math.sqrt(d), window,
                                    keys_per_split, nsplit)
    expect = []
    for s, (c, n) in enumerate(zip(ctx, new)):
        full_q = torch.zeros((c + n, nh, d), dtype=torch.float64)
        full_q[c:] = qs[s].double()
        o = plain.causal_attention(full_q, ks[s].double(), vs[s].double(), window=window)
        expect.append(o[c:])
    return out, torch.cat(expect)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh,nkv,d,page_size", [
    (4, 2, 16, 4), (3, 1, 32, 8), (5, 5, 48, 16), (32, 8, 64, 16), (8, 1, 128, 16),
    (2, 2, 256, 8), (16, 1, 64, 32)])
def test_paged_attention_mixed_batch(dtype, nh, nkv, d, page_size):
    """Portions of prompts beside single decoded tokens, in one launch."""
    ctx = [0, 37, 129, 5, 64]
    new = [33, 1, 1, 70, 2]
    out, expect = run_attention(dtype, nh, nkv, d, page_size, ctx, new)
    assert rel_err(out, expect) < tol_of(dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_paged_attention_reference_shapes(dtype):
    """The shapes of the reference's own attention tests
    (/root/reference/tests/test_paged_attention_gpu.zig:40-131, 284-327): 9 decoded
    tokens at block size 4 with 8 query / 2 key heads of size 8; a 6-token prompt;
    40 tokens at block size 16 with head size 128.  Their tolerance is 5e-3 to 1e-2."""
    for nh, nkv, d, ps, ctx, new in [(8, 2, 8, 4, [8], [1]), (8, 2, 8, 4, [0], [6]),
                                     (32, 8, 128, 16, [39], [1])]:
        out, expect = run_attention(dtype, nh, nkv, d, ps, ctx, new)
        assert rel_err(out, expect) < tol_of(dtype)


@pytest.mark.parametrize("nh,nkv,d,page_size", [
    (32, 8, 64, 16), (4, 4, 64, 4), (8, 4, 128, 16), (16, 2, 64, 8), (16, 1, 128, 32), (2, 1, 64, 16),
    (6, 2, 64, 12), (5, 1, 128, 20), (7, 7, 64, 64)])
@pytest.mark.parametrize("window", [0, 70])
@pytest.mark.parametrize("tile_keys", [64, 128])
def test_paged_attention_matrix_cores(nh, nkv, d, page_size, window, tile_keys):
    """The matrix-core kernel on mixed steps: long portions, portions that do not fill
    a work item, single tokens with long contexts; with tiles of 64 and of 128 keys."""
    ctx = [0, 37, 129, 5, 300]
    new = [150, 1, 17, 70, 2]
    out, expect = run_attention(torch.bfloat16, nh, nkv, d, page_size, ctx, new, window=window,
                                mfma=True, tile_keys=tile_keys)
    assert rel_err(out, expect) < BF16_TOL
    out, expect = run_attention(torch.bfloat16, nh, nkv, d, page_size, [700, 300], [1, 40],
                                sharpen=True, mfma=True, tile_keys=tile_keys)
    assert rel_err(out, expect) < BF16_TOL
    assert float(expect.abs().max()) > 0.5


@pytest.mark.parametrize("keys,nsplit", [(64, 12), (256, 3), (1024, 1)])
@pytest.mark.parametrize("window", [0, 70])
@pytest.mark.parametrize("tile_keys", [64, 128])
def test_paged_attention_matrix_cores_cut_contexts(keys, nsplit, window, tile_keys):
    """Prompt portions with their contexts cut into ranges: ranges that a row cannot
    see at all, ranges that end inside a tile's worth of rows, empty ranges."""
    ctx = [700, 0, 255, 64, 300]
    new = [40, 150, 3, 70, 1]
    for nh, nkv, d, ps in [(32, 8, 64, 16), (6, 2, 128, 8)]:
        out, expect = run_attention(torch.bfloat16, nh, nkv, d, ps, ctx, new, window=window,
                                    keys_per_split=keys, nsplit=nsplit, sharpen=True, mfma=True,
                                    tile_keys=tile_keys)
        assert rel_err(out, expect) < BF16_TOL


def test_paged_attention_matrix_cores_paired_items():
    """So many work items that a workgroup takes two of them, a late and an early
    one, with an odd number of items so that the middle one stays alone."""
    out, expect = run_attention(torch.bfloat16, 64, 64, 64, 16, [0, 90], [1000, 37], mfma=True)
    assert rel_err(out, expect) < BF16_TOL
    out, expect = run_attention(torch.bfloat16, 64, 64, 64, 16, [0, 90, 3], [1000, 37, 130],
                                window=200, mfma=True)
    assert rel_err(out, expect) < BF16_TOL


@pytest.mark.parametrize("nh,nkv,d,page_size", [
    (32, 8, 64, 16), (4, 4, 64, 4), (8, 4, 128, 16), (16, 1, 64, 8), (2, 1, 128, 32),
    (6, 2, 64, 12), (5, 1, 128, 20)])
@pytest.mark.parametrize("keys,nsplit", [(0, 1), (64, 12), (256, 3)])
@pytest.mark.parametrize("window", [0, 70])
def test_paged_attention_decode_matrix_cores(nh, nkv, d, page_size, keys, nsplit, window):
    """The decode kernel: single tokens (and pairs) with contexts from nothing to
    several hundred keys, whole and cut."""
    ctx = [700, 0, 255, 64, 1, 300]
    new = [1, 1, 1, 1, 2, 3]
    out, expect = run_attention(torch.bfloat16, nh, nkv, d, page_size, ctx, new, window=window,
                                keys_per_split=keys, nsplit=nsplit, sharpen=True,
                                mfma_decode=True)
    assert rel_err(out, expect) < BF16_TOL


def light_attention(q, k, v, positions, window=0):
    """Causal attention for a few query rows against a long context: q [n, nh, d] at
    ``positions``, k and v [T, nkv, d]; float64, one score row per query."""
    n, nh, d = q.shape
    nkv = k.shape[1]
    out = torch.zeros((n, nh, d), dtype=torch.float64)
    keys = torch.arange(k.shape[0])
    for h in range(nh):
        g = h // (nh // nkv)
        s = (q[:, h].double() @ k[:, g].double().T) / math.sqrt(d)
        mask = keys[None, :] > positions[:, None]
        if window > 0:
            mask = mask | (keys[None, :] <= positions[:, None] - window)
        p = torch.softmax(s.masked_fill(mask, float("-inf")), dim=-1)
        out[:, h] = p @ v[:, g].double()
    return out


@pytest.mark.parametrize("window", [0, 3000])
def test_attention_over_long_contexts(window):
    """Tens of thousands of keys: a portion of a prompt far into its request, and
    single tokens whose context is cut into many ranges; one key far back is made to
    dominate the last query."""
    nh, nkv, d, ps = 8, 2, 64, 16
    ctx, n = 20000, 150
    k = rand((ctx + n, nkv, d), torch.bfloat16, 91)
    v = rand((ctx + n, nkv, d), torch.bfloat16, 92)
    q = rand((n, nh, d), torch.bfloat16, 93)
    far = ctx + n - 2500                    # inside the window when there is one
    k[far] = 0
    k[far, :, 3] = 16.0
    q[-1] = 0
    q[-1, :, 3] = 16.0                      # score 32 against N(0, 4) for the other keys
    cache, table = paged_from_dense([k], [v], ps, torch.bfloat16, seed=9)
    positions = torch.arange(ctx, ctx + n, dtype=torch.int32)
    expect = light_attention(q, k, v, positions.long(), window)
    assert float((expect[-1] - v[far].double().repeat_interleave(nh // nkv, 0)).abs().max()) < 0.05
    args = (cache.to(dev()), table.to(dev()), positions.to(dev()))
    for keys, nsplit in [(0, 1), (4096, 5), (1024, 20)]:
        out = ops().paged_attention_mfma(q.to(dev()), *args, *items_for([n], 128 // (nh // nkv)),
                                         1.0 / math.sqrt(d), window, keys, nsplit)
        assert rel_err(out, expect) < BF16_TOL, (keys, nsplit)
    # the last 16 tokens one by one, as a decode step of 16 requests would bring them:
    # 16 requests that share the pages but stand at different positions
    m = 16
    tables = table.repeat(m, 1).to(dev())
    pos_m = positions[-m:].to(dev())
    for keys, nsplit in [(0, 1), (1024, (ctx + n + 1023) // 1024), (256, (ctx + n + 255) // 256)]:
        out = ops().paged_attention_decode_mfma(q[-m:].to(dev()), cache.to(dev()), tables, pos_m,
                                                None, None, None, m, 1.0 / math.sqrt(d), window,
                                                keys, nsplit)
        assert rel_err(out, expect[-m:]) < BF16_TOL, (keys, nsplit)
        out = ops().paged_attention(q[-m:].to(dev()), cache.to(dev()), tables, pos_m,
                                    *items_for([1] * m, 1), 1.0 / math.sqrt(d), window, keys, nsplit)
        assert rel_err(out, expect[-m:]) < BF16_TOL, (keys, nsplit)


@pytest.mark.parametrize("nh,nkv,d,requests", [(16, 8, 64, 49), (4, 2, 128, 6), (8, 8, 128, 50)])
def test_decode_attention_beyond_4096_keys_uncut(nh, nkv, d, requests):
    """The decode kernel fetches the block-table entries of sixteen tiles a wave at once and
    fetches again when they are used up: with four waves a workgroup (the form taken when
    requests x key/value heads fill the chip, here 392 and 400 workgroups) that is after
    4,096 keys of an uncut context, with eight after 8,192.  Contexts of 4,900 to 9,000 keys,
    uncut; one key before and one behind the place of the second fetch are made to
    dominate a query each, so that a tile read through a stale or misplaced entry shows."""
    ps = 16
    ctx = 9000 if requests < 10 else 4900
    total = ctx + requests
    k = rand((total, nkv, d), torch.bfloat16, 110)
    v = rand((total, nkv, d), torch.bfloat16, 111)
    q = rand((requests, nh, d), torch.bfloat16, 112)
    near, far = 100, ctx - 300                 # (far lies behind every fetch but the last)
    for key, row, elem in ((near, 0, 3), (far, 1, 5)):
        k[key] = 0
        k[key, :, elem] = 16.0
        q[row] = 0
        q[row, :, elem] = 16.0                 # score 32 / sqrt(d) x 8 against N(0, 4)
    cache, table = paged_from_dense([k], [v], ps, torch.bfloat16, seed=12)
    positions = torch.arange(ctx, ctx + requests, dtype=torch.int32)
    expect = light_attention(q, k, v, positions.long(), 0)
    group = nh // nkv
    assert float((expect[0] - v[near].double().repeat_interleave(group, 0)).abs().max()) < 0.05
    assert float((expect[1] - v[far].double().repeat_interleave(group, 0)).abs().max()) < 0.05
    tables = table.repeat(requests, 1).to(dev())
    out = ops().paged_attention_decode_mfma(q.to(dev()), cache.to(dev()), tables, positions.to(dev()),
                                            None, None, None, requests, 1.0 / math.sqrt(d), 0, 0, 1)
    assert rel_err(out, expect) < BF16_TOL


@pytest.mark.parametrize("keys_per_split,nsplit", [(0, 1), (1024, 12), (512, 24)])
def test_rope_attention_decode_beyond_8192_keys(keys_per_split, nsplit):
    """The attention that prepares its own token, far into long contexts (the second fetch of
    table entries, the token's own place in a late tile): the bits of the two kernels it
    replaces, in the result and in the cache, uncut and in ranges."""
    o = ops()
    nh, nkv, d, page_size = 8, 2, 64, 16
    positions = [8191, 8192, 8300, 9001, 12000]
    qkv, cache, table, pos, slots = decode_step_case(nh, nkv, d, page_size, positions, 1200)
    T = len(positions)
    qw = (rand((d,), torch.float32, 1201) * 0.3 + 1.0).to(dev())
    kw = (rand((d,), torch.float32, 1202) * 0.3 + 1.0).to(dev())
    inv = (1.0 / torch.pow(torch.tensor(1e6, dtype=torch.float64),
                           2.0 * torch.arange(0, d // 2, dtype=torch.float64) / d)).float().to(dev())
    eps, scale = 1e-5, 1.0 / math.sqrt(d)
    two = cache.clone()
    q = o.qk_norm_rope_kv_write(qkv, pos, slots, qw, kw, inv, two, nh, nkv, d, d, False, eps)
    want = o.paged_attention_decode_mfma(q, two, table, pos, None, None, None, T, scale, 0,
                                         keys_per_split, nsplit)
    one = cache.clone()
    got = o.rope_attention_decode(qkv, pos, slots, qw, kw, inv, one, table, nh, eps, scale, 0,
                                  keys_per_split, nsplit)
    assert torch.equal(one, two) and not torch.equal(one, cache)
    assert torch.equal(got, want)


def test_single_token_attention_returns_value():
    """One key: the softmax is 1 and the output is V (derived, but only checked for
    finiteness, in /root/reference/src/transformer/hybrid_attn.zig:1207-1212)."""
    nh, nkv, d = 4, 2, 16
    k, v, q = rand((1, nkv, d), torch.float32, 40), rand((1, nkv, d), torch.float32, 41), rand((1, nh, d), torch.float32, 42)
    cache, table = paged_from_dense([k], [v], 4, torch.float32)
    out = ops().paged_attention(q.to(dev()), cache.to(dev()), table.to(dev()),
                                torch.zeros(1, dtype=torch.int32, device=dev()),
                                *items_for([1], 16), 0.25).cpu()
    for h in range(nh):
        assert torch.allclose(out[0, h], v[0, h // 2], atol=1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_paged_attention_far_key_dominates(dtype):
    """One early key among hundreds carries the weight: a kernel that loses far
    keys (a page's edge, a tile's edge) cannot pass."""
    out, expect = run_attention(dtype, 8, 2, 64, 16, [700, 300], [1, 5], sharpen=True)
    assert rel_err(out, expect) < tol_of(dtype)
    assert float(expect.abs().max()) > 0.5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("keys,nsplit", [(64, 12), (256, 3), (128, 8)])
def test_paged_attention_split_context(dtype, keys, nsplit):
    ctx, new = [700, 1, 255, 64], [1, 1, 1, 1]
    whole, expect = run_attention(dtype, 8, 2, 64, 16, ctx, new, sharpen=True)
    cut, _ = run_attention(dtype, 8, 2, 64, 16, ctx, new, keys_per_split=keys, nsplit=nsplit,
                           sharpen=True)
    assert rel_err(cut, expect) < tol_of(dtype)
    assert rel_err(cut, whole.double()) < tol_of(dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window", [1, 5, 16, 100])
def test_paged_attention_window(dtype, window):
    out, expect = run_attention(dtype, 6, 2, 32, 8, [0, 90, 41], [50, 1, 9], window=window)
    assert rel_err(out, expect) < tol_of(dtype)


def test_paged_attention_window_skips_freed_pages():
    """Pages behind the window may be gone from the table (-1): never read."""
    nh, nkv, d, ps, window = 4, 2, 16, 4, 6
    c, n = 40, 3
    k, v, q = rand((c + n, nkv, d), torch.float32, 50), rand((c + n, nkv, d), torch.float32, 51), rand((n, nh, d), torch.float32, 52)
    cache, table = paged_from_dense([k], [v], ps, torch.float32)
    first_needed = c - window + 1
    for p in range(first_needed // ps):
        cache[table[0, p]] = float("nan")
        table[0, p] = -1
    pos = torch.arange(c, c + n, dtype=torch.int32, device=dev())
    out = ops().paged_attention(q.to(dev()), cache.to(dev()), table.to(dev()), pos,
                                *items_for([n], 16), 0.25, window)
    full_q = torch.zeros((c + n, nh, d), dtype=torch.float64)
    full_q[c:] = q.double()
    expect = plain.causal_attention(full_q, k.double(), v.double(), window=window)[c:]
    assert rel_err(out, expect) < F32_TOL


def decode_step_case(nh, nkv, d, page_size, positions, seed):
    """A decode step: request i holds positions[i] cached tokens and brings one more.
    Returns qkv [T, (nh + 2 nkv) d], the cache with random contents in the requests' pages
    (the new tokens' places included: what was there before must not count), block table,
    positions and the new tokens' places, all on the device."""
    T = len(positions)
    ks = [rand((p + 1, nkv, d), torch.bfloat16, seed + 2 * i) for i, p in enumerate(positions)]
    vs = [rand((p + 1, nkv, d), torch.bfloat16, seed + 2 * i + 1) for i, p in enumerate(positions)]
    cache, table = paged_from_dense(ks, vs, page_size, torch.bfloat16, seed=seed)
    slots = torch.tensor([int(table[i, p // page_size]) * page_size + p % page_size
                          for i, p in enumerate(positions)], dtype=torch.int32)
    qkv = rand((T, (nh + 2 * nkv) * d), torch.bfloat16, seed + 100)
    pos = torch.tensor(positions, dtype=torch.int32)
    return qkv.to(dev()), cache.to(dev()), table.to(dev()), pos.to(dev()), slots.to(dev())


@pytest.mark.parametrize("nh,nkv,d,page_size", [(8, 2, 64, 16), (3, 3, 64, 4), (16, 1, 64, 32),
                                                (5, 1, 64, 12), (32, 8, 64, 16), (4, 2, 128, 16),
                                                (6, 1, 128, 8), (2, 2, 128, 20)])
@pytest.mark.parametrize("keys_per_split,nsplit,window", [(0, 1, 0), (256, 5, 0), (0, 1, 100),
                                                          (128, 9, 70)])
@pytest.mark.parametrize("norms", [True, False])
def test_rope_attention_decode_is_the_two_kernels_in_one(nh, nkv, d, page_size, keys_per_split,
                                                         nsplit, window, norms):
    """A decode step's norm, rotation and cache write inside its attention kernel: the bits
    of qk_norm_rope_kv_write followed by paged_attention_decode_mfma, in the result and in
    the cache; positions at the edges of tiles (64 keys), of pages and of the ranges."""
    o = ops()
    positions = [0, 1, 3, 62, 63, 64, 65, 127, 128, 255, 256, 257, 700, 1023, 1100]
    qkv, cache, table, pos, slots = decode_step_case(nh, nkv, d, page_size, positions, 900 + nh + d)
    T = len(positions)
    qw = (rand((d,), torch.float32, 901) * 0.3 + 1.0).to(dev()) if norms else None
    kw = (rand((d,), torch.float32, 902) * 0.3 + 1.0).to(dev()) if norms else None
    inv = (1.0 / torch.pow(torch.tensor(1e6, dtype=torch.float64),
                           2.0 * torch.arange(0, d // 2, dtype=torch.float64) / d)).float().to(dev())
    eps, scale = 1e-5, 1.0 / math.sqrt(d)
    two = cache.clone()
    q = o.qk_norm_rope_kv_write(qkv, pos, slots, qw, kw, inv, two, nh, nkv, d, d, False, eps)
    want = o.paged_attention_decode_mfma(q, two, table, pos, None, None, None, T, scale, window,
                                         keys_per_split, nsplit)
    one = cache.clone()
    got = o.rope_attention_decode(qkv, pos, slots, qw, kw, inv, one, table, nh, eps, scale, window,
                                  keys_per_split, nsplit)
    assert torch.equal(one, two)
    assert torch.equal(got, want)
    assert not torch.equal(one, cache)            # something was stored


def test_rope_attention_decode_stores_the_token_whatever_the_ranges():
    """Ranges that end before a token's position (a caller's mistake) must not leave its key
    and value out of the cache: the last range takes the keys that are left."""
    o = ops()
    nh, nkv, d, page_size = 8, 2, 64, 16
    positions = [5, 300, 700]
    qkv, cache, table, pos, slots = decode_step_case(nh, nkv, d, page_size, positions, 970)
    inv = (1.0 / torch.pow(torch.tensor(1e4, dtype=torch.float64),
                           2.0 * torch.arange(0, d // 2, dtype=torch.float64) / d)).float().to(dev())
    two = cache.clone()
    q = o.qk_norm_rope_kv_write(qkv, pos, slots, None, None, inv, two, nh, nkv, d, d, False, 1e-5)
    want = o.paged_attention_decode_mfma(q, two, table, pos, None, None, None, 3, 0.125)
    one = cache.clone()
    got = o.rope_attention_decode(qkv, pos, slots, None, None, inv, one, table, nh, 1e-5, 0.125,
                                  0, 128, 2)                   # two ranges of 128 keys: 256 < 700
    assert torch.equal(one, two)
    assert rel_err(got, want.double().cpu()) < 2e-2


@pytest.mark.parametrize("nh,nkv,d,H", [(32, 8, 64, 2048), (16, 8, 64, 1024), (8, 2, 128, 512), (24, 8, 64, 1536)])
@pytest.mark.parametrize("T,keys_per_split,nsplit", [(1, 256, 8), (3, 256, 5), (4, 128, 8), (8, 1024, 2), (7, 512, 3),
                                                     (1, 128, 12), (2, 128, 16), (3, 128, 11)])
def test_output_projection_merges_the_context_ranges_itself(nh, nkv, d, H, T, keys_per_split, nsplit):
    """The decode attention may leave its ranges' partial results unmerged (MergedRows) and
    the output projection merge them on its way in: the merge has the combine kernel's bits,
    the product stored has the bits of the product of the merged rows, and added to a stream
    it agrees to rounding (the additions of the ranges of K arrive in any order)."""
    o = ops()
    positions = [1100, 3, 700, 64, 1023, 255, 256, 900][:T]
    qkv, cache, table, pos, slots = decode_step_case(nh, nkv, d, 16, positions, 980 + T)
    inv = (1.0 / torch.pow(torch.tensor(1e6, dtype=torch.float64),
                           2.0 * torch.arange(0, d // 2, dtype=torch.float64) / d)).float().to(dev())
    scale = 1.0 / math.sqrt(d)
    want = o.rope_attention_decode(qkv, pos, slots, None, None, inv, cache.clone(), table, nh, 1e-5,
                                   scale, 0, keys_per_split, nsplit)
    parts = o.rope_attention_decode(qkv, pos, slots, None, None, inv, cache.clone(), table, nh, 1e-5,
                                    scale, 0, keys_per_split, nsplit, combine=False)
    assert isinstance(parts, o.MergedRows) and parts.shape == (T, nh * d) and parts.ranges == nsplit
    assert torch.equal(parts.materialise().view(T, nh, d), want)
    w = rand((H, nh * d), torch.bfloat16, 985).to(dev())
    stored = o.linear(want.view(T, nh * d), w, out_dtype=torch.float32)
    direct = torch.empty((T, H), dtype=torch.float32, device=dev())
    rc = o._fn("gemm", "za_gemm_bf16_rows16_merged")(
        o._ptr(parts.acc), o._ptr(parts.ml), nsplit, d, o._ptr(w), o._ptr(direct), T, H, nh * d, 1, 0,
        o._stream())
    assert rc == 0
    assert torch.equal(direct, stored)
    base = rand((T, H), torch.float32, 986).to(dev())
    a, b = base.clone(), base.clone()
    o.form_log = []
    try:
        assert o.linear(parts, w, partial_ok=True, accumulate=a) is None
        took_the_merge = any(r.get("merged_ranges") for r in o.form_log if r["op"] == "linear")
    finally:
        o.form_log = None
    assert o.linear(want.view(T, nh * d), w, partial_ok=True, accumulate=b) is None
    assert rel_err(a, b.double().cpu()) < 1e-5
    assert took_the_merge == o.merged_rows_pay(T, nsplit)     # (every width here is a multiple of 512)


def test_merged_rows_fall_back_to_the_combine_kernel():
    """What the merging product does not take (a bias, a product that is stored, many rows)
    goes through the combine kernel and the ordinary product."""
    o = ops()
    T, nh, d, nsplit = 12, 4, 64, 3
    acc = rand((T, nh, nsplit, d), torch.float32, 990).to(dev())
    ml = torch.stack([torch.randint(-3, 4, (T, nh, nsplit)).float(), torch.rand(T, nh, nsplit) + 0.5],
                     dim=-1).contiguous().to(dev())
    ml[0, 0, 1, 0] = float("-inf")                  # a range without keys
    ml[0, 0, 1, 1] = 0.0
    parts = o.MergedRows(acc, ml)
    rows = parts.materialise()
    m, l = ml[..., 0].double().cpu(), ml[..., 1].double().cpu()
    wgt = torch.exp2(m - m.max(dim=-1, keepdim=True).values)
    expect = ((acc.double().cpu() * wgt[..., None]).sum(2) / (l * wgt).sum(-1, keepdim=True)).reshape(T, nh * d)
    assert rel_err(rows, expect) < 1e-2
    w = rand((96, nh * d), torch.bfloat16, 991).to(dev())
    bias = rand((96,), torch.float32, 992).to(dev())
    assert torch.equal(o.linear(parts, w, bias), o.linear(rows, w, bias))
    stream = torch.zeros((T, 96), device=dev())
    assert not o.merged_rows_pay(T, nsplit)
    got = o.linear(parts, w, partial_ok=True, accumulate=stream)       # twelve rows: not merged on the way in
    expect_y = rows.double().cpu() @ w.double().cpu().T
    y = stream if got is None else (got.sum(0) if got.dim() == 3 else got)
    assert rel_err(y, expect_y) < 1e-2


def test_rope_attention_decode_refuses_what_it_cannot_take():
    o = ops()
    qkv, cache, table, pos, slots = decode_step_case(4, 2, 64, 16, [5, 9], 950)
    inv = torch.ones(32, device=dev())
    assert not o.decode_rope_fusable(qkv, 4, 2, 64, 32, False, 16, 0.125)     # a partial rotation
    assert not o.decode_rope_fusable(qkv, 4, 2, 64, 64, True, 16, 0.125)      # adjacent pairs
    assert not o.decode_rope_fusable(qkv.float(), 4, 2, 64, 64, False, 16, 0.125)
    assert not o.decode_rope_fusable(qkv, 4, 2, 64, 64, False, 6, 0.125)      # the page size
    assert o.decode_rope_fusable(qkv, 4, 2, 64, 64, False, 16, 0.125)
    with pytest.raises(ops().KernelError):
        o.rope_attention_decode(qkv[:, :-64], pos, slots, None, None, inv, cache, table, 4, 1e-5, 0.125)
    with pytest.raises(ops().KernelError):
        o.rope_attention_decode(qkv, pos, slots[:1], None, None, inv, cache, table, 4, 1e-5, 0.125)


# ------------------------------------------------------------------ short conv
def conv_reference(z, w, b, H):
    B, C, x = z[:, :H], z[:, H:2 * H], z[:, 2 * H:]
    return C * plain.causal_depthwise_conv(B * x, w, b)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,L,bias", [(64, 3, False), (96, 4, True), (80, 2, True), (300, 1, False),
                                      (2048, 3, False), (40, 8, True)])
def test_short_conv_whole_and_in_portions(dtype, H, L, bias):
    """Three requests packed in one launch; then the same tokens in portions of
    changing size (down to one token) with the carried state: same result."""
    lens = [23, 1, 9]
    zs = [rand((n, 3 * H), dtype, 60 + i) for i, n in enumerate(lens)]
    w = rand((H, L), torch.float32, 70)
    b = rand((H,), torch.float32, 71) if bias else None
    expect = [conv_reference(z.double(), w.double(), b.double() if bias else None, H) for z in zs]

    def launch(parts, state, slot_ids):
        z = torch.cat(parts).to(dev())
        n = [p.shape[0] for p in parts]
        token_seq = torch.cat([torch.full((m,), i, dtype=torch.int32) for i, m in enumerate(n)])
        seq_start = torch.tensor([0] + list(torch.tensor(n).cumsum(0)), dtype=torch.int32)
        return ops().short_conv(z, w.t().contiguous().to(dev()), b.to(dev()) if bias else None, state,
                                token_seq.to(dev()), seq_start.to(dev()),
                                torch.tensor(slot_ids, dtype=torch.int32, device=dev()))

    # slots live in a wider row, as the cache manager lays them out
    memory = torch.zeros((5, H * L + 7), dtype=torch.float32, device=dev())
    state = memory[:, 3:3 + H * L].unflatten(1, (H, L))
    y = launch(zs, state, [4, 0, 2])
    assert rel_err(y, torch.cat(expect)) < tol_of(dtype)
    # the state holds the last L gated inputs, oldest first, zeros before the start
    for z, slot in zip(zs, [4, 0, 2]):
        u = (z.double()[:, :H] * z.double()[:, 2 * H:])
        padded = torch.cat([torch.zeros(L, H, dtype=torch.float64), u])[-L:]
        assert rel_err(state[slot].cpu().T, padded) < F32_TOL if padded.abs().max() > 0 else True
    assert (memory[[1, 3]] == 0).all() and (memory[:, :3] == 0).all() and (memory[:, 3 + H * L:] == 0).all()

    memory.zero_()
    cuts = [[5, 1, 2, 7, 1, 1, 6], [1], [2, 2, 1, 4]]
    cursor = [0, 0, 0]
    got = [[] for _ in lens]
    for step in range(max(len(c) for c in cuts)):
        parts, slots, who = [], [], []
        for i in range(3):
            if step < len(cuts[i]):
                n = cuts[i][step]
                parts.append(zs[i][cursor[i]:cursor[i] + n])
                cursor[i] += n
                slots.append([4, 0, 2][i])
                who.append(i)
        y = launch(parts, state, slots).cpu()
        row = 0
        for i, p in zip(who, parts):
            got[i].append(y[row:row + p.shape[0]])
            row += p.shape[0]
    for i in range(3):
        assert rel_err(torch.cat(got[i]), expect[i]) < tol_of(dtype)


@pytest.mark.parametrize("M,H,L,bias", [(1, 512, 3, False), (8, 2048, 3, False), (5, 1024, 4, True),
                                        (8, 2560, 3, True), (3, 1536, 1, False), (7, 4096, 8, True),
                                        (2, 3584, 2, False), (9, 1024, 3, True), (16, 2048, 3, False),
                                        (13, 2560, 8, True)])
def test_in_proj_gated_conv_is_the_three_kernels_in_one(M, H, L, bias):
    """A decode batch of the ShortConv mixer, one token a request: norm + in_proj +
    convolution in one kernel give the bits (outputs AND new state) that the norm inside
    in_proj followed by the convolution's own kernel give, over three steps of the same
    requests (so the carried state matters), at widths other than the engine's, with
    slots out of order in a wider row; and both agree with the plain formulas."""
    K = H
    w_in = rand((3 * H, K), torch.bfloat16, 300, 0.03).to(dev())
    taps = rand((H, L), torch.float32, 301)
    b = rand((H,), torch.float32, 302) if bias else None
    norm_w = (1.0 + 0.3 * rand((K,), torch.float32, 303)).to(dev())
    slots = [5, 0, 7, 2, 6, 1, 3, 4, 15, 9, 12, 8, 14, 10, 13, 11][:M]
    slot_id = torch.tensor(slots, dtype=torch.int32, device=dev())
    token_seq = torch.arange(M, dtype=torch.int32, device=dev())
    seq_start = torch.arange(M + 1, dtype=torch.int32, device=dev())
    taps_t, bd = taps.t().contiguous().to(dev()), b.to(dev()) if bias else None

    def memory():
        mem = torch.zeros((16, H * L + 5), dtype=torch.float32, device=dev())
        return mem, mem[:, 2:2 + H * L].unflatten(1, (H, L))

    (mem_a, state_a), (mem_b, state_b) = memory(), memory()
    hist = torch.zeros((M, L, H), dtype=torch.float64)
    for step in range(3):
        stream = rand((M, K), torch.float32, 310 + step, 2.0).to(dev())
        x = ops().NormedRows(stream, norm_w, 1e-5, torch.bfloat16)
        assert ops().gated_conv_fusable(x, w_in, taps_t)
        mem_before = mem_a.clone()
        fused = ops().in_proj_gated_conv(x, w_in, taps_t, bd, state_a, slot_id)
        z = ops().linear(x, w_in)
        apart = ops().short_conv(z, taps_t, bd, state_b, token_seq, seq_start, slot_id)
        assert torch.equal(fused, apart), (step, rel_err(fused, apart))
        assert torch.equal(mem_a, mem_b)
        for channels in (4, 8, 16):             # however many channels a workgroup takes
            mem_c = mem_before.clone()
            state_c = mem_c[:, 2:2 + H * L].unflatten(1, (H, L))
            again = ops().in_proj_gated_conv(x, w_in, taps_t, bd, state_c, slot_id, channels=channels)
            assert torch.equal(again, apart) and torch.equal(mem_c, mem_b), channels
        # the plain formulas, on the projection's own (rounded) output
        zd = z.double().cpu()
        u = zd[:, :H] * zd[:, 2 * H:]
        hist = torch.cat([hist[:, 1:], u[:, None, :]], dim=1)
        c = (hist * taps.double().T[None]).sum(dim=1) + (b.double() if bias else 0.0)
        assert rel_err(fused, zd[:, H:2 * H] * c) < BF16_TOL
    for m, slot in enumerate(slots):
        assert rel_err(state_a[slot].cpu().T, hist[m]) < F32_TOL
    untouched = [s for s in range(16) if s not in slots]
    assert (mem_a[untouched] == 0).all() and (mem_a[:, :2] == 0).all() and (mem_a[:, 2 + H * L:] == 0).all()


def test_in_proj_gated_conv_refuses_what_it_cannot_take():
    w = rand((3 * 96, 512), torch.bfloat16, 320).to(dev())          # width 96: fine; K 512
    taps = rand((3, 96), torch.float32, 321).to(dev())
    nw = torch.ones(512, device=dev())
    many = ops().NormedRows(torch.zeros((17, 512), device=dev()), nw, 1e-5, torch.bfloat16)
    assert not ops().gated_conv_fusable(many, w, taps)                 # seventeen rows
    odd = ops().NormedRows(torch.zeros((2, 520), device=dev()), torch.ones(520, device=dev()), 1e-5,
                           torch.bfloat16)
    assert not ops().gated_conv_fusable(odd, rand((3 * 96, 520), torch.bfloat16, 322).to(dev()), taps)
    assert not ops().gated_conv_fusable(torch.zeros((2, 512), dtype=torch.bfloat16, device=dev()), w, taps)
    narrow = rand((3, 104), torch.float32, 323).to(dev())             # width no multiple of 16
    few = ops().NormedRows(torch.zeros((2, 512), device=dev()), nw, 1e-5, torch.bfloat16)
    assert not ops().gated_conv_fusable(few, rand((312, 512), torch.bfloat16, 324).to(dev()), narrow)
    with pytest.raises(ops().KernelError):
        ops().in_proj_gated_conv(many, w, taps, None, torch.zeros((1, 96, 3), device=dev()),
                                 torch.zeros(17, dtype=torch.int32, device=dev()))


def test_short_conv_identity_filter():
    """Filter e_{L-1} with B = C = 1 passes x through."""
    H, L, T = 32, 3, 10
    x = rand((T, H), torch.float32, 80)
    z = torch.cat([torch.ones(T, H), torch.ones(T, H), x], dim=1)
    w = torch.zeros(H, L)
    w[:, L - 1] = 1.0
    state = torch.zeros((1, H, L), device=dev())
    y = ops().short_conv(z.to(dev()), w.t().contiguous().to(dev()), None, state,
                         torch.zeros(T, dtype=torch.int32, device=dev()),
                         torch.tensor([0, T], dtype=torch.int32, device=dev()),
                         torch.zeros(1, dtype=torch.int32, device=dev())).cpu()
    assert torch.equal(y, x)


# ------------------------------------------------------------------ activation
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,I", [(1, 8), (5, 176), (3, 13), (4, 128), (2, 8192)])
def test_swiglu(dtype, T, I):
    gu = rand((T, 2 * I), dtype, 90, 2.0)
    out = ops().swiglu(gu.to(dev()))
    g, u = gu.double()[:, :I], gu.double()[:, I:]
    assert out.shape == (T, I)
    assert rel_err(out, torch.nn.functional.silu(g) * u) < tol_of(dtype)


def test_cast_round_trip():
    x = rand((1000,), torch.float32, 91)
    b = ops().cast(x.to(dev()), torch.bfloat16)
    assert torch.equal(b.cpu(), x.to(torch.bfloat16))       # round to nearest even, as torch
    assert torch.equal(ops().cast(b, torch.float32).cpu(), x.to(torch.bfloat16).float())


# -------------------------------------------------------------------- sampling
def test_argmax_first_occurrence():
    logits = rand((6, 1000), torch.float32, 100)
    logits[0, 17] = logits[0, 900] = 50.0       # a tie: the first index wins
    logits[1, 999] = 60.0
    logits[2, 0] = 60.0
    logits[3] = 0.0                             # all equal
    out = ops().argmax(logits.to(dev())).cpu().tolist()
    assert out == [plain.argmax_first(r) for r in logits]
    assert out[0] == 17 and out[1] == 999 and out[2] == 0 and out[3] == 0


@pytest.mark.parametrize("rows,vocab", [(1, 65536), (8, 65536), (3, 10000), (70, 65536), (2, 301)])
def test_argmax_long_rows(rows, vocab):
    """Few rows of a long vocabulary are cut into chunks; ties across chunks still
    go to the first index."""
    logits = rand((rows, vocab), torch.float32, 102)
    logits[0, vocab - 1] = logits[0, 7] = 99.0
    if rows > 1:
        logits[1, vocab // 2] = logits[1, vocab // 2 + 4097 if vocab > 9000 else vocab - 2] = 99.0
    out = ops().argmax(logits.to(dev())).cpu().tolist()
    assert out == logits.argmax(dim=1).tolist() or out == [plain.argmax_first(r) for r in logits]
    assert out[0] == 7


@pytest.mark.parametrize("vocab", [50, 1000, 1003, 65536])
def test_sample_matches_plain(vocab):
    R = 12
    logits = rand((R, vocab), torch.float32, 101, 3.0)
    temps = torch.tensor([0.0, 0.7, 1.0, 1.5, 0.7, 0.7, 1.0, 0.2, 1.0, 1.0, 0.7, 0.0])
    top_k = torch.tensor([0, 0, 0, 0, 5, 0, 40, 0, 1, 0, 10, 3], dtype=torch.int32)
    top_p = torch.tensor([1.0, 1.0, 1.0, 1.0, 1.0, 0.9, 0.5, 1.0, 1.0, 0.01, 0.8, 0.9])
    u = torch.tensor([0.3, 0.0, 0.999999, 0.5, 0.25, 0.75, 0.6, 0.1, 0.9, 0.4, 0.33, 0.5])
    out = ops().sample(logits.to(dev()), temps.to(dev()), top_k.to(dev()), top_p.to(dev()),
                       u.to(dev())).cpu().tolist()
    for r in range(R):
        want = plain.sample_token(logits[r].double(), float(temps[r]), float(u[r]),
                                  int(top_k[r]), float(top_p[r]))
        if out[r] != want:
            # the draw may fall within rounding of a boundary between two tokens:
            # accept the neighbour only if u sits on that boundary
            v = logits[r].double() / float(temps[r])
            keep = plain.kept_after_top_k_top_p(v, int(top_k[r]), float(top_p[r]))
            assert bool(keep[out[r]]), (r, out[r], want)
            e = torch.where(keep, torch.exp(v - v[keep].max()), torch.zeros_like(v))
            cdf = torch.cumsum(e, 0) / e.sum()
            lo = float(cdf[out[r] - 1]) if out[r] > 0 else 0.0
            assert lo - 1e-5 <= float(u[r]) <= float(cdf[out[r]]) + 1e-5, (r, out[r], want)


def sample_settings(R, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    temps = torch.tensor([0.3, 0.7, 1.0, 1.7])[torch.randint(0, 4, (R,), generator=g)]
    ks = torch.tensor([0, 1, 2, 7, 50, 1000, vocab - 1, vocab + 5])[torch.randint(0, 8, (R,), generator=g)]
    ps = torch.tensor([1.0, 0.999, 0.95, 0.9, 0.5, 0.1, 1e-6, 0.0])[torch.randint(0, 8, (R,), generator=g)]
    u = torch.rand(R, generator=g)
    return temps, ks.clamp(max=2 ** 31 - 1).to(torch.int32), ps, u


@pytest.mark.parametrize("vocab", [640, 4099, 65536, 200003])
@pytest.mark.parametrize("ties", [False, True])
def test_sample_thresholds_two_ways_agree(vocab, ties):
    """The thresholds of top-k and top-p are searched in one bin's values or, for a
    bin too full, over the whole row; probability mass is summed in integers, so
    both find the same key: the same tokens, exactly.  With logits rounded to
    halves, bins hold thousands of equal values and the first way gives up."""
    R = 32
    logits = rand((R, vocab), torch.float32, 110, 3.0)
    if ties:
        logits = torch.round(logits * 2) / 2
    logits[3, ::2] = float("-inf")
    temps, ks, ps, u = sample_settings(R, vocab, 111)
    args = [t.to(dev()) for t in (logits, temps, ks, ps, u)]
    fast = ops().sample(*args).cpu()
    slow = ops().sample(*args, whole_row_only=True).cpu()
    assert torch.equal(fast, slow)
    for r in range(R):                                  # and the token is one the plain rule keeps
        v = logits[r].double() / float(temps[r])
        keep = plain.kept_after_top_k_top_p(v, int(ks[r]), float(ps[r]))
        tok = int(fast[r])
        if not bool(keep[tok]):
            # only a value within rounding of the threshold may differ
            edge = v[keep].min()
            assert abs(float(v[tok] - edge)) <= 1e-5 * max(1.0, abs(float(edge))), (r, tok)


def test_sample_flat_and_tied_rows():
    """All values equal: top-k keeps them all (ties with the k-th are kept), and the
    draw walks the row in index order.  Five values tied for third place: all five
    stay candidates."""
    vocab = 65536
    logits = torch.zeros((4, vocab))
    u = torch.tensor([0.0, 0.25, 0.5, 0.999])
    out = ops().sample(logits.to(dev()), torch.ones(4, device=dev()),
                       torch.full((4,), 10, dtype=torch.int32, device=dev()),
                       torch.ones(4, device=dev()), u.to(dev())).cpu().tolist()
    for r in range(4):
        want = max(0, int(math.ceil(float(u[r]) * vocab)) - 1)
        assert abs(out[r] - want) <= 1, (r, out[r], want)
    n = 512
    row = torch.full((vocab,), -5.0)
    row[[11, 70000 % vocab]] = 4.0
    tied = [5, 1000, 30000, 50000, 65535]
    row[tied] = 3.0
    us = (torch.arange(n, dtype=torch.float32) + 0.5) / n
    out = ops().sample(row.repeat(n, 1).to(dev()), torch.ones(n, device=dev()),
                       torch.full((n,), 3, dtype=torch.int32, device=dev()),
                       torch.ones(n, device=dev()), us.to(dev())).cpu().tolist()
    assert set(out) == set(tied) | {11, 70000 % vocab}


def test_sample_distribution():
    """Frequencies over many uniforms follow softmax(logits / T)."""
    vocab, n = 8, 4000
    row = torch.tensor([2.0, 1.0, 0.5, 0.0, -1.0, 3.0, 1.5, -2.0])
    logits = row.repeat(n, 1)
    u = (torch.arange(n, dtype=torch.float32) + 0.5) / n
    out = ops().sample(logits.to(dev()), torch.full((n,), 0.7, device=dev()),
                       torch.zeros(n, dtype=torch.int32, device=dev()),
                       torch.ones(n, device=dev()), u.to(dev())).cpu()
    freq = torch.bincount(out.long(), minlength=vocab).double() / n
    assert (freq - torch.softmax(row.double() / 0.7, 0)).abs().max() < 2.0 / n + 1e-3


def test_repetition_penalty():
    logits = torch.tensor([[2.0, -2.0, 0.0, 4.0], [1.0, 1.0, -1.0, -1.0]])
    rows = torch.tensor([0, 0, 1, 1], dtype=torch.int32)
    toks = torch.tensor([0, 1, 3, 0], dtype=torch.int32)
    fac = torch.tensor([2.0, 2.0, 4.0, 1.5])
    work = logits.clone().to(dev())
    ops().repetition_penalty_(work, rows.to(dev()), toks.to(dev()), fac.to(dev()))
    assert torch.allclose(work.cpu(), torch.tensor([[1.0, -4.0, 0.0, 4.0], [1.0 / 1.5, 1.0, -1.0, -4.0]]))
