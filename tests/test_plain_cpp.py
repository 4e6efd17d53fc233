"""The plain C++ statements of the kernels (csrc/plain.cpp) from both sides: against
the plain Python formulas of tests/plain_lfm2.py (on the CPU), and each HIP kernel
against its C++ twin on the same operands, the paged cache and the packed step
included (on the GPU).

Tolerances as in test_kernels_gpu.py: 2e-5 of the largest magnitude for 32-bit
kernels, 6e-3 where bfloat16 is stored.
"""

import math

import pytest
import torch

import plain_lfm2 as plain
from zig_ai_amd.kernels import plain as twin

F32_TOL = 2e-5
BF16_TOL = 6e-3
DTYPES = [torch.float32, torch.bfloat16]


def rand(shape, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(shape, generator=g) * scale


def rel_err(actual, expected):
    a, e = actual.detach().double().cpu(), expected.detach().double().cpu()
    assert a.shape == e.shape, (a.shape, e.shape)
    assert torch.isfinite(a).all()
    return float((a - e).abs().max() / e.abs().max().clamp_min(1e-30))


def i32(x):
    return torch.tensor(x, dtype=torch.int32)


# ------------------------------------------------- the twins against the formulas
def test_twin_add_rmsnorm():
    res, delta, w = rand((5, 100), 1), rand((3, 5, 100), 2), rand((100,), 3)
    total, out = twin.add_rmsnorm(res, delta, w, 1e-5)
    want = res.double() + delta.double().sum(0)
    assert rel_err(total, want) < 1e-6
    assert rel_err(out, plain.rms_norm(want, w.double(), 1e-5)) < 1e-6
    total, out = twin.add_rmsnorm(None, delta[0].contiguous(), w, 1e-6)
    assert torch.equal(total, delta[0])
    assert rel_err(out, plain.rms_norm(delta[0].double(), w.double(), 1e-6)) < 1e-6
    # the reference's own vector: [1, 2, 3, 4] with unit weights (norm.zig:83-103)
    _, out = twin.add_rmsnorm(torch.tensor([[1.0, 2.0, 3.0, 4.0]]), None, torch.ones(4), 1e-5)
    assert rel_err(out, torch.tensor([[1.0, 2.0, 3.0, 4.0]]) / math.sqrt(7.5 + 1e-5)) < 1e-6


def test_twin_embed_linear_swiglu():
    table = rand((20, 12), 4)
    assert torch.equal(twin.embed(i32([0, 19, 7, 7]), table), plain.embedding([0, 19, 7, 7], table.double()).float())
    with pytest.raises(twin.PlainError):
        twin.embed(i32([20]), table)
    x, w, b = rand((7, 33), 5), rand((19, 33), 6), rand((19,), 7)
    assert rel_err(twin.linear(x, w, b), x.double() @ w.double().T + b.double()) < 1e-6
    gu = rand((6, 26), 8, 3.0)
    want = torch.nn.functional.silu(gu[:, :13].double()) * gu[:, 13:].double()
    assert rel_err(twin.swiglu(gu), want) < 1e-6


@pytest.mark.parametrize("nh,nkv,d,rot,adjacent,page_size,window", [
    (4, 2, 16, 16, False, 4, 0), (3, 1, 32, 32, False, 8, 0), (6, 3, 24, 12, True, 5, 7),
    (2, 2, 8, 0, False, 3, 0)])
def test_twin_attention_path(nh, nkv, d, rot, adjacent, page_size, window):
    """Two requests written into shuffled pages in two portions each, then read:
    the same as norm, rotation and causal attention over the whole sequences."""
    lens = [13, 22]
    theta, eps = 10000.0, 1e-5
    qw, kw = rand((d,), 10).abs() + 0.5, rand((d,), 11).abs() + 0.5
    inv_freq = plain.rope_inv_freq(rot, theta).float() if rot else None
    n_pages = sum((n + page_size - 1) // page_size for n in lens) + 2
    order = torch.randperm(n_pages, generator=torch.Generator().manual_seed(3)).tolist()
    cache = torch.full((n_pages, 2, nkv, page_size, d), 1e4)
    table = torch.full((2, max((n + page_size - 1) // page_size for n in lens)), -1, dtype=torch.int32)
    for s, n in enumerate(lens):
        for p in range((n + page_size - 1) // page_size):
            table[s, p] = order.pop()
    qkvs = [rand((n, (nh + 2 * nkv) * d), 20 + s) for s, n in enumerate(lens)]
    outs = [[], []]
    for lo_frac, hi_frac in ((0.0, 0.4), (0.4, 1.0)):
        rows, pos, seq, slots = [], [], [], []
        for s, n in enumerate(lens):
            lo, hi = int(n * lo_frac), int(n * hi_frac)
            rows.append(qkvs[s][lo:hi])
            pos += list(range(lo, hi))
            seq += [s] * (hi - lo)
            slots += [int(table[s, p // page_size]) * page_size + p % page_size for p in range(lo, hi)]
        q = twin.qk_norm_rope_kv_write(torch.cat(rows), i32(pos), i32(slots), qw, kw, inv_freq, cache,
                                       nh, nkv, d, rot, adjacent, eps)
        o = twin.paged_attention(q, cache, table, i32(pos), i32(seq), 1.0 / math.sqrt(d), window)
        row = 0
        for s, n in enumerate(lens):
            m = int(n * hi_frac) - int(n * lo_frac)
            outs[s].append(o[row:row + m])
            row += m
    for s, n in enumerate(lens):
        x = qkvs[s].double().view(n, nh + 2 * nkv, d)
        q, k, v = x[:, :nh], x[:, nh:nh + nkv], x[:, nh + nkv:]
        positions = torch.arange(n)
        q = plain.rms_norm(q, qw.double(), eps)
        k = plain.rms_norm(k, kw.double(), eps)
        if rot:
            pairing = "adjacent" if adjacent else "half"
            q = plain.apply_rope(q, positions, theta, rot, pairing)
            k = plain.apply_rope(k, positions, theta, rot, pairing)
        want = plain.causal_attention(q, k, v, window=window)
        assert rel_err(torch.cat(outs[s]), want) < 2e-6


@pytest.mark.parametrize("H,L,bias", [(10, 3, False), (7, 4, True), (5, 1, True)])
def test_twin_short_conv_in_portions(H, L, bias):
    lens, slots = [11, 1, 6], [2, 0, 3]
    zs = [rand((n, 3 * H), 30 + i) for i, n in enumerate(lens)]
    w = rand((H, L), 33)
    b = rand((H,), 34) if bias else None
    state = torch.zeros((4, H, L))
    cuts = [[4, 1, 6], [1], [2, 4]]
    got = [[] for _ in lens]
    cursor = [0, 0, 0]
    for step in range(3):
        parts, who = [], []
        for i in range(3):
            if step < len(cuts[i]):
                parts.append(zs[i][cursor[i]:cursor[i] + cuts[i][step]])
                cursor[i] += cuts[i][step]
                who.append(i)
        starts = [0]
        for p in parts:
            starts.append(starts[-1] + p.shape[0])
        y = twin.short_conv(torch.cat(parts), w, b, state, i32(starts), i32([slots[i] for i in who]))
        for k, i in enumerate(who):
            got[i].append(y[starts[k]:starts[k + 1]])
    for i, z in enumerate(zs):
        zd = z.double()
        want = zd[:, H:2 * H] * plain.causal_depthwise_conv(zd[:, :H] * zd[:, 2 * H:], w.double(),
                                                            b.double() if bias else None)
        assert rel_err(torch.cat(got[i]), want) < 1e-6
        u = torch.cat([torch.zeros(L, H, dtype=torch.float64), zd[:, :H] * zd[:, 2 * H:]])[-L:]
        assert torch.allclose(state[slots[i]].double().T, u, atol=1e-6)
    assert (state[1] == 0).all()


def test_twin_sampler():
    vocab, R = 301, 64
    logits = rand((R, vocab), 40, 3.0)
    logits[5, ::3] = float("-inf")
    g = torch.Generator().manual_seed(41)
    temps = torch.tensor([0.0, 0.3, 0.7, 1.0, 1.7])[torch.randint(0, 5, (R,), generator=g)]
    ks = torch.tensor([0, 1, 2, 7, 50, 300, 400])[torch.randint(0, 7, (R,), generator=g)].to(torch.int32)
    ps = torch.tensor([1.0, 0.95, 0.5, 0.1, 0.0])[torch.randint(0, 5, (R,), generator=g)]
    u = torch.rand(R, generator=g)
    out = twin.sample(logits, temps, ks, ps, u).tolist()
    for r in range(R):
        assert out[r] == plain.sample_token(logits[r], float(temps[r]), float(u[r]), int(ks[r]), float(ps[r])), r
        if temps[r] > 0:
            _, keep = twin.sample_weights(logits[r], float(temps[r]), int(ks[r]), float(ps[r]))
            want = plain.kept_after_top_k_top_p(logits[r].double() / float(temps[r]), int(ks[r]), float(ps[r]))
            assert torch.equal(keep, want), r
    tie = torch.zeros((2, 9))
    tie[0, [3, 7]] = 5.0
    assert twin.argmax(tie).tolist() == [3, 0]
    work = torch.tensor([[2.0, -2.0, 0.0, 4.0], [1.0, 1.0, -1.0, -1.0]])
    twin.repetition_penalty_(work, i32([0, 0, 1, 1]), i32([0, 1, 3, 0]), torch.tensor([2.0, 2.0, 4.0, 1.5]))
    assert torch.allclose(work, torch.tensor([[1.0, -4.0, 0.0, 4.0], [1.0 / 1.5, 1.0, -1.0, -4.0]]))
    for row in work:
        hist = [0, 1]
        assert torch.allclose(plain.apply_repetition_penalty(torch.tensor([2.0, -2.0, 0.0, 4.0]), hist, 2.0),
                              torch.tensor([1.0, -4.0, 0.0, 4.0]))


# ------------------------------------------------- the kernels against their twins
def dev():
    return torch.device("cuda", 0)


def ops():
    from zig_ai_amd.kernels import ops as _ops
    return _ops


def tol_of(dtype):
    return F32_TOL if dtype == torch.float32 else BF16_TOL


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,width,partials", [(3, 100, 0), (9, 2048, 4), (17, 136, 2), (1, 4099, 8)])
def test_kernel_add_rmsnorm_against_twin(dtype, rows, width, partials):
    res = rand((rows, width), 50)
    delta = rand((partials, rows, width), 51) if partials else rand((rows, width), 51).to(dtype).float()
    w = rand((width,), 52)
    want_res, want = twin.add_rmsnorm(res, delta, w, 1e-5)
    r = res.clone().to(dev())
    d = delta.to(dev()) if partials else delta.to(dtype).to(dev())
    out = ops().add_rmsnorm(r, d, w.to(dev()), 1e-5, dtype)
    assert rel_err(r, want_res) < F32_TOL
    assert rel_err(out, want) < tol_of(dtype)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,N,K,bias", [(1, 50, 96, False), (8, 130, 264, True), (40, 70, 520, False),
                                        (16, 33, 2048, False), (200, 96, 136, True)])
def test_kernel_linear_against_twin(dtype, M, N, K, bias):
    x, w = rand((M, K), 53).to(dtype), rand((N, K), 54, 0.05).to(dtype)
    b = rand((N,), 55) if bias else None
    want = twin.linear(x.float(), w.float(), b)
    got = ops().linear(x.to(dev()), w.to(dev()), b.to(dev()) if bias else None, out_dtype=torch.float32)
    assert rel_err(got, want) < F32_TOL
    gu = rand((M, 2 * N), 56, 2.0).to(dtype)
    assert rel_err(ops().swiglu(gu.to(dev())), twin.swiglu(gu.float())) < tol_of(dtype)


@pytest.mark.gpu
@pytest.mark.parametrize("M,N,K,bias", [(1, 50, 512, False), (8, 130, 1536, True), (5, 70, 2048, False),
                                        (16, 16400, 1024, False)])
def test_kernel_decode_forms_against_twins(M, N, K, bias):
    """A decode batch in bfloat16: the projection that runs the norm before it against
    the norm's twin followed by the product's twin (the twin rounds nothing, the kernel
    rounds the operands once), also into the SwiGLU gate; and the projection that adds
    to the stream against the product's twin plus the stream."""
    o = ops()
    res, nw = rand((M, K), 70, 2.0), 1.0 + rand((K,), 71, 0.3)
    w = rand((N, K), 72, 0.05).to(torch.bfloat16)
    b = rand((N,), 73) if bias else None
    _, normed = twin.add_rmsnorm(res, None, nw, 1e-5)
    want = twin.linear(normed, w.float(), b)
    x = o.NormedRows(res.to(dev()), nw.to(dev()), 1e-5, torch.bfloat16)
    assert o.normed_rows_pay(M, N, K)
    got = o.linear(x, w.to(dev()), b.to(dev()) if bias else None, out_dtype=torch.float32)
    assert rel_err(got, want) < BF16_TOL
    if N % 2 == 0 and not bias:
        assert rel_err(o.linear_swiglu(x, w.to(dev())), twin.swiglu(want)) < BF16_TOL
    a = rand((M, K), 74).to(torch.bfloat16)
    stream = rand((M, N), 75)
    on_device = stream.clone().to(dev())
    assert o.linear(a.to(dev()), w.to(dev()), b.to(dev()) if bias else None, accumulate=on_device) is None
    assert rel_err(on_device, stream + twin.linear(a.float(), w.float(), b)) < F32_TOL


@pytest.mark.gpu
@pytest.mark.parametrize("M,N,K", [(20, 96, 1024), (32, 200, 2048), (64, 130, 1536), (17, 64, 4096)])
def test_kernel_for_17_to_64_rows_against_the_twins(M, N, K):
    """csrc/gemm_rows64.hip against the plain C++ functions: the norm twin followed by the
    product's twin (the kernel rounds the operands once, as the norm kernel does, and scales
    the sums), into the SwiGLU twin, and the product's twin plus the stream."""
    o = ops()
    res, nw = rand((M, K), 76, 2.0), 1.0 + rand((K,), 77, 0.3)
    w = rand((N, K), 78, 0.05).to(torch.bfloat16)
    _, normed = twin.add_rmsnorm(res, None, nw, 1e-5)
    want = twin.linear(normed, w.float(), None)
    x = o.NormedRows(res.to(dev()), nw.to(dev()), 1e-5, torch.bfloat16)
    assert rel_err(o.linear_rows64(x, w.to(dev())), want) < BF16_TOL
    assert rel_err(o.linear_rows64(x, w.to(dev()), mode=o.ROWS64_SWIGLU), twin.swiglu(want)) < BF16_TOL
    a = rand((M, K), 79).to(torch.bfloat16)
    stream = rand((M, N), 80)
    on_device = stream.clone().to(dev())
    o.linear_rows64(a.to(dev()), w.to(dev()), mode=o.ROWS64_ADD, accumulate=on_device,
                    ksplit=2 if K >= 2048 else 1)
    assert rel_err(on_device, stream + twin.linear(a.float(), w.float(), None)) < F32_TOL



@pytest.mark.gpu
@pytest.mark.parametrize("dtype", DTYPES)
def test_kernel_embed_against_twin(dtype):
    table = rand((300, 72), 57).to(dtype)
    tokens = i32([0, 299, 17, 17, 150])
    got = ops().embed_gather(tokens.to(dev()), table.to(dev()))
    assert torch.equal(got.float().cpu(), twin.embed(tokens, table.float()))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,d,rot,adjacent,page_size,window", [
    (4, 2, 16, 16, False, 4, 0), (3, 1, 32, 32, False, 8, 0), (6, 3, 48, 24, True, 12, 20),
    (32, 8, 64, 64, False, 16, 0), (8, 2, 128, 128, False, 16, 0), (16, 4, 64, 64, False, 32, 50)])
def test_kernel_attention_path_against_twin(dtype, nh, nkv, d, rot, adjacent, page_size, window):
    """Three steps of a small batch through the two kernels of an attention layer and
    through their twins, both on caches of their own with the same block table:
    portions of prompts, then further portions beside a decoded token, then decoded
    tokens only.  Queries, every element of both caches, and the outputs agree."""
    def work_items(counts, rows_per_item):
        seq, row0, cnt, first = [], [], [], 0
        for s, n in enumerate(counts):
            for lo in range(0, n, rows_per_item):
                seq.append(s); row0.append(first + lo); cnt.append(min(rows_per_item, n - lo))
            first += n
        return seq, row0, cnt

    steps = [[(0, 0, 37), (1, 0, 70)], [(0, 37, 1), (1, 70, 45), (2, 0, 9)], [(0, 38, 1), (1, 115, 1), (2, 9, 1)]]
    ends = [39, 116, 10]
    eps = 1e-5
    qw, kw = rand((d,), 60).abs() + 0.5, rand((d,), 61).abs() + 0.5
    inv_freq = plain.rope_inv_freq(rot, 1e6).float()
    pages_of = [(n + page_size - 1) // page_size for n in ends]
    n_pages = sum(pages_of) + 2
    order = torch.randperm(n_pages, generator=torch.Generator().manual_seed(5)).tolist()
    table = torch.full((3, max(pages_of)), 0, dtype=torch.int32)
    for s in range(3):
        for p in range(pages_of[s]):
            table[s, p] = order.pop()
    host_cache = torch.zeros((n_pages, 2, nkv, page_size, d))
    gpu_cache = torch.zeros((n_pages, 2, nkv, page_size, d), dtype=dtype, device=dev())
    G = nh // nkv
    mfma = ops().attention_mfma_supported(dtype, nh, nkv, d, page_size, 1.0)
    fused_steps = []
    for step_no, step in enumerate(steps):
        pos, seq, slots, counts = [], [], [], []
        for s, lo, n in step:
            pos += list(range(lo, lo + n))
            seq += [s] * n
            slots += [int(table[s, p // page_size]) * page_size + p % page_size for p in range(lo, lo + n)]
            counts.append(n)
        T = len(pos)
        qkv = rand((T, (nh + 2 * nkv) * d), 70 + step_no).to(dtype)
        before = gpu_cache.clone()
        want_q = twin.qk_norm_rope_kv_write(qkv.float(), i32(pos), i32(slots), qw, kw, inv_freq, host_cache,
                                            nh, nkv, d, rot, adjacent, eps)
        got_q = ops().qk_norm_rope_kv_write(qkv.to(dev()), i32(pos).to(dev()), i32(slots).to(dev()),
                                            qw.to(dev()), kw.to(dev()), inv_freq.to(dev()), gpu_cache,
                                            nh, nkv, d, rot, adjacent, eps)
        assert rel_err(got_q, want_q) < tol_of(dtype)
        assert rel_err(gpu_cache, host_cache) < tol_of(dtype)
        # both sides go on from the same stored values, so that only the attention differs
        host_cache.copy_(gpu_cache.float().cpu())
        q = got_q.float().cpu()
        want = twin.paged_attention(q, host_cache, table, i32(pos), i32(seq), 1.0 / math.sqrt(d), window)
        step_table = table[[s for s, _, _ in step]].contiguous().to(dev())
        local_seq = [i for i, n in enumerate(counts) for _ in range(n)]
        assert twin.paged_attention(q, host_cache, step_table.cpu(), i32(pos), i32(local_seq),
                                    1.0 / math.sqrt(d), window).equal(want)
        kinds = ["plain"] + (["mfma"] if mfma else []) + (["decode"] if mfma and max(counts) == 1 else [])
        for kind in kinds:
            rows = {"plain": 32, "mfma": 128, "decode": 16}[kind] // G
            item_seq, row0, cnt = (i32(x).to(dev()) for x in work_items(counts, max(1, rows)))
            fn = {"plain": ops().paged_attention, "mfma": ops().paged_attention_mfma,
                  "decode": ops().paged_attention_decode_mfma}[kind]
            got = fn(got_q, gpu_cache, step_table, i32(pos).to(dev()), item_seq, row0, cnt,
                     item_seq.numel(), 1.0 / math.sqrt(d), window)
            assert rel_err(got, want) < tol_of(dtype), (step_no, kind)
        if max(counts) == 1 and ops().decode_rope_fusable(qkv, nh, nkv, d, rot, adjacent, page_size,
                                                          1.0 / math.sqrt(d)):
            # the two kernels in one, from the cache as it was before the step
            got = ops().rope_attention_decode(qkv.to(dev()), i32(pos).to(dev()), i32(slots).to(dev()),
                                              qw.to(dev()), kw.to(dev()), inv_freq.to(dev()), before,
                                              step_table, nh, eps, 1.0 / math.sqrt(d), window)
            assert rel_err(got, want) < tol_of(dtype), (step_no, "both in one")
            assert rel_err(before, host_cache) < tol_of(dtype)
            fused_steps.append(step_no)
    assert fused_steps == ([2] if dtype == torch.bfloat16 and d in (64, 128) and rot == d else [])


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,L,bias", [(64, 3, False), (96, 4, True), (100, 2, True), (2048, 3, False)])
def test_kernel_short_conv_against_twin(dtype, H, L, bias):
    """Portions of three requests, several steps, state slots out of order: outputs
    and all state slots after every step."""
    w = rand((H, L), 80)
    b = rand((H,), 81) if bias else None
    host_state = torch.zeros((5, H, L))
    gpu_state = torch.zeros((5, H, L), device=dev())
    for step_no, (lens, slots) in enumerate([([19, 1, 6], [4, 0, 2]), ([1, 1, 40], [4, 0, 2]), ([2, 5], [0, 3])]):
        z = rand((sum(lens), 3 * H), 82 + step_no).to(dtype)
        starts = [0]
        for n in lens:
            starts.append(starts[-1] + n)
        token_seq = [i for i, n in enumerate(lens) for _ in range(n)]
        want = twin.short_conv(z.float(), w, b, host_state, i32(starts), i32(slots))
        got = ops().short_conv(z.to(dev()), w.t().contiguous().to(dev()), b.to(dev()) if bias else None,
                               gpu_state, i32(token_seq).to(dev()), i32(starts).to(dev()), i32(slots).to(dev()))
        assert rel_err(got, want) < tol_of(dtype), step_no
        assert rel_err(gpu_state, host_state) < F32_TOL, step_no


@pytest.mark.gpu
@pytest.mark.parametrize("vocab", [50, 1003, 65536])
def test_kernel_sampler_against_twin(vocab):
    R = 48
    logits = rand((R, vocab), 90, 3.0)
    g = torch.Generator().manual_seed(91)
    temps = torch.tensor([0.0, 0.3, 0.7, 1.0, 1.7])[torch.randint(0, 5, (R,), generator=g)]
    ks = torch.tensor([0, 1, 2, 7, 50, 1000])[torch.randint(0, 6, (R,), generator=g)].to(torch.int32)
    ps = torch.tensor([1.0, 0.95, 0.5, 0.1])[torch.randint(0, 4, (R,), generator=g)]
    u = torch.rand(R, generator=g)
    want = twin.sample(logits, temps, ks, ps, u).tolist()
    got = ops().sample(*(t.to(dev()) for t in (logits, temps, ks, ps, u))).cpu().tolist()
    assert ops().argmax(logits.to(dev())).cpu().tolist() == twin.argmax(logits).tolist()
    for r in range(R):
        if got[r] == want[r]:
            continue
        # the kernel sums 32-bit exponentials: the draw may fall within rounding of the
        # boundary between two kept tokens, and only there may the choices differ
        weight, keep = twin.sample_weights(logits[r], float(temps[r]), int(ks[r]), float(ps[r]))
        assert bool(keep[got[r]]), (r, got[r], want[r])
        cdf = torch.cumsum(weight, 0) / weight.sum()
        lo = float(cdf[got[r] - 1]) if got[r] > 0 else 0.0
        assert lo - 1e-5 <= float(u[r]) <= float(cdf[got[r]]) + 1e-5, (r, got[r], want[r])
    pairs_r, pairs_t = i32([0, 0, 3, 7]), i32([5, 9, 9, 0])
    fac = torch.tensor([1.3, 2.0, 1.1, 4.0])
    work = logits.clone().to(dev())
    ops().repetition_penalty_(work, pairs_r.to(dev()), pairs_t.to(dev()), fac.to(dev()))
    twin.repetition_penalty_(logits, pairs_r, pairs_t, fac)
    assert torch.allclose(work.cpu(), logits, rtol=1e-6, atol=0)
