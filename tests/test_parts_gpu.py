"""Each part alone, built through its registry entry with random tensors, against
the plain formulas: norm, embedding and head, SwiGLU, the ShortConv mixer with its
state slot, the attention mixer with its pages, and the block arrangement."""


import pytest
import torch

import plain_lfm2 as plain

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 5e-5, torch.bfloat16: 1.5e-2}


def dev():
    return torch.device("cuda", 0)


def rnd(shape, seed, scale=1.0):
    return torch.randn(shape, generator=torch.Generator().manual_seed(seed)) * scale


def rel_err(a, e):
    a, e = a.detach().double().cpu(), e.detach().double().cpu()
    assert a.shape == e.shape and torch.isfinite(a).all()
    return float((a - e).abs().max() / e.abs().max())


def runtime(dtype):
    from zig_ai_amd.parts import Runtime
    return Runtime(device=dev(), dtype=dtype)


def place(tensors, rules, dtype):
    """Tensors on the device in the precision their role prescribes."""
    from zig_ai_amd.weights import keep_dtype
    return {k: v.to(dev()).to(keep_dtype(dtype, rules[k].role, dtype)) for k, v in tensors.items()}


def total(y):
    """A part may return a stack of partial sums."""
    return y.sum(0) if y.dim() == 3 else y


def still_pending(residual, pending):
    """What a block leaves to be added to the stream: nothing when its last part has
    added its result itself (a decode batch in bfloat16)."""
    return torch.zeros_like(residual) if pending is None else total(pending)


def step_for(cache, entries):
    from zig_ai_amd.engine import StepEntry
    from zig_ai_amd.engine.batch import build_step
    batch = [StepEntry(r, list(range(n)), []) for r, n in entries]
    for r, n in entries:
        cache.reserve(r, n)
    return build_step(batch, cache, dev(), 10 ** 6, [1, 2, 4, 8, 16, 32, 64])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rms_norm_part(dtype):
    from zig_ai_amd.parts import lookup
    cls = lookup("norm", "rms_norm")
    params = {"width": 72, "eps": 1e-6}
    w = rnd((72,), 1) + 1
    part = cls(params, place({"weight": w}, cls.tensor_rules(params), dtype), runtime(dtype))
    x = rnd((9, 72), 2, 3.0)
    out = part.forward(x.to(dev()).to(dtype))
    assert out.dtype == dtype
    assert rel_err(out, plain.rms_norm(x.to(dtype).double(), w.double(), 1e-6)) < TOL[dtype]
    res = x.clone().to(dev())
    delta = rnd((9, 72), 3).to(dtype)
    out = part.add_forward(res, delta.to(dev()))
    h = x.double() + delta.double()
    assert rel_err(res, h) < 5e-5 and rel_err(out, plain.rms_norm(h, w.double(), 1e-6)) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embedding_and_head(dtype):
    from zig_ai_amd.parts import lookup
    emb_cls, head_cls = lookup("embedding", "token_embedding"), lookup("head", "linear_head")
    params = {"vocab_size": 301, "hidden_size": 80}
    table = rnd((301, 80), 4)
    emb = emb_cls(params, place({"weight": table}, emb_cls.tensor_rules(params), dtype), runtime(dtype))
    toks = torch.tensor([0, 300, 7, 7, 150], dtype=torch.int32)
    x = emb.forward(toks.to(dev()))
    assert x.dtype == torch.float32 and torch.equal(x.cpu(), table.to(dtype).float()[toks.long()])
    tied = head_cls({**params, "tied": True}, {}, runtime(dtype))
    assert head_cls.tensor_rules({**params, "tied": True}) == {}
    tied.weight = emb.weight
    n = rnd((5, 80), 5).to(dtype)
    logits = tied.forward(n.to(dev()))
    assert logits.dtype == torch.float32                       # logits are 32-bit in both modes
    assert rel_err(logits, n.double() @ table.to(dtype).double().T) < 5e-5
    own = rnd((301, 80), 6)
    untied = head_cls({**params, "tied": False},
                      place({"weight": own}, head_cls.tensor_rules({**params, "tied": False}), dtype),
                      runtime(dtype))
    assert rel_err(untied.forward(n.to(dev())), n.double() @ own.to(dtype).double().T) < 5e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T", [1, 9, 40, 130])
def test_swiglu_part(dtype, T):
    from zig_ai_amd.parts import lookup
    cls = lookup("feed_forward", "swiglu")
    params = {"hidden_size": 96, "intermediate_size": 176}
    w = {"gate.weight": rnd((176, 96), 7, 0.2), "up.weight": rnd((176, 96), 8, 0.2),
         "down.weight": rnd((96, 176), 9, 0.2)}
    part = cls(params, place(w, cls.tensor_rules(params), dtype), runtime(dtype))
    x = rnd((T, 96), 10).to(dtype)
    out = total(part.forward(x.to(dev()), None))
    wd = {k: v.to(dtype).double() for k, v in w.items()}
    expect = plain.swiglu_ffn(x.double(), wd["gate.weight"], wd["up.weight"], wd["down.weight"])
    assert rel_err(out, expect) < TOL[dtype]


@pytest.mark.parametrize("T", [1, 8, 16])
@pytest.mark.parametrize("adds", [False, True])
def test_swiglu_part_of_a_wide_model(T, adds):
    """Hidden 6144 with a feed-forward of 12288 in bfloat16, a decode batch: K is longer
    than one workgroup of the decode kernel covers and there are more outputs than fill
    the chip, whether the part adds to the stream itself or hands its product back."""
    from zig_ai_amd.parts import lookup
    cls = lookup("feed_forward", "swiglu")
    H, I = 6144, 12288
    params = {"hidden_size": H, "intermediate_size": I}
    w = {"gate.weight": rnd((I, H), 7, 0.02), "up.weight": rnd((I, H), 8, 0.02),
         "down.weight": rnd((H, I), 9, 0.02)}
    part = cls(params, place(w, cls.tensor_rules(params), torch.bfloat16), runtime(torch.bfloat16))
    x = rnd((T, H), 10).to(torch.bfloat16)
    wd = {k: v.to(torch.bfloat16).double() for k, v in w.items()}
    expect = plain.swiglu_ffn(x.double(), wd["gate.weight"], wd["up.weight"], wd["down.weight"])
    if adds:
        stream0 = rnd((T, H), 11)
        stream = stream0.to(dev())
        assert part.forward(x.to(dev()), None, stream=stream) is None
        assert rel_err(stream, stream0.double() + expect) < TOL[torch.bfloat16]
    else:
        out = total(part.forward(x.to(dev()), None))
        assert rel_err(out, expect) < TOL[torch.bfloat16]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("bias", [False, True])
def test_short_conv_part(dtype, bias):
    """Two requests through the mixer in portions; the carried state makes the
    portions equal to the whole."""
    from zig_ai_amd.cache import CacheManager
    from zig_ai_amd.parts import lookup
    cls = lookup("mixer", "short_conv")
    H, L = 64, 4
    params = {"hidden_size": H, "kernel_size": L, "bias": bias}
    w = {"in_proj.weight": rnd((3 * H, H), 11, 0.2), "conv.weight": rnd((H, L), 12, 0.5),
         "out_proj.weight": rnd((H, H), 13, 0.2)}
    if bias:
        w.update({"in_proj.bias": rnd((3 * H,), 14, 0.1), "conv.bias": rnd((H,), 15, 0.1),
                  "out_proj.bias": rnd((H,), 16, 0.1)})
    assert cls.cache_need(params).shape == (H, L)
    part = cls(params, place(w, cls.tensor_rules(params), dtype), runtime(dtype))
    cache = CacheManager({0: cls.cache_need(params)}, 4, 8, 3, device=dev(), dtype=dtype)
    view = cache.view(0)
    xs = {"a": rnd((23, H), 17).to(dtype), "b": rnd((6, H), 18).to(dtype)}
    wd = {k.replace(".weight", "").replace(".bias", "_bias"): v.to(dtype if v.dim() == 2 and "conv" not in k else torch.float32).double()
          for k, v in w.items()}
    expect = {r: plain.short_conv_mixer(x.double(), wd) for r, x in xs.items()}
    cuts = {"a": [5, 1, 2, 15], "b": [1, 1, 4]}
    done = {"a": 0, "b": 0}
    got = {"a": [], "b": []}
    for r in xs:
        cache.admit(r)
    for stepi in range(4):
        entries = [(r, cuts[r][stepi]) for r in ("a", "b") if stepi < len(cuts[r])]
        step = step_for(cache, entries)
        x = torch.cat([xs[r][done[r]:done[r] + n] for r, n in entries]).to(dev())
        y = total(part.forward(x, step, view)).cpu()
        row = 0
        for r, n in entries:
            got[r].append(y[row:row + n])
            row += n
            done[r] += n
            cache.commit(r, n)
    for r in xs:
        assert rel_err(torch.cat(got[r]), expect[r]) < TOL[dtype]


@pytest.mark.parametrize("bias", [False, True])
def test_short_conv_part_decoding_from_the_stream(bias, monkeypatch):
    """The mixer given rows that still await their norm, as a block gives them: two
    prompts in one step (the three kernels), then single tokens of both requests (norm,
    in_proj and convolution in one kernel when in_proj has no bias), against the plain
    norm and mixer on the whole sequences; the fused kernel is seen to run."""
    from zig_ai_amd.cache import CacheManager
    from zig_ai_amd.kernels import ops
    from zig_ai_amd.parts import lookup
    cls = lookup("mixer", "short_conv")
    H, L, eps = 512, 3, 1e-5
    params = {"hidden_size": H, "kernel_size": L, "bias": bias}
    w = {"in_proj.weight": rnd((3 * H, H), 111, 0.05), "conv.weight": rnd((H, L), 112, 0.5),
         "out_proj.weight": rnd((H, H), 113, 0.05)}
    if bias:
        w.update({"in_proj.bias": rnd((3 * H,), 114, 0.1), "conv.bias": rnd((H,), 115, 0.1)})
    nw = (rnd((H,), 116, 0.2) + 1).to(dev())
    part = cls(params, place(w, cls.tensor_rules(params), torch.bfloat16), runtime(torch.bfloat16))
    cache = CacheManager({0: cls.cache_need(params)}, 4, 16, 3, device=dev(), dtype=torch.bfloat16)
    view = cache.view(0)
    streams = {"a": rnd((11, H), 117, 2.0), "b": rnd((6, H), 118, 2.0)}
    bf = lambda t: t.to(torch.bfloat16).double()
    wd = {"in_proj": bf(w["in_proj.weight"]), "conv": w["conv.weight"].double(), "out_proj": bf(w["out_proj.weight"])}
    if bias:
        wd.update({"in_proj_bias": w["in_proj.bias"].double(), "conv_bias": w["conv.bias"].double()})
    expect = {r: plain.short_conv_mixer(plain.rms_norm(x.double(), nw.double().cpu(), eps), wd)
              for r, x in streams.items()}
    calls = []
    fused = ops.in_proj_gated_conv
    monkeypatch.setattr(ops, "in_proj_gated_conv", lambda *a, **k: (calls.append(a[0].shape[0]), fused(*a, **k))[1])
    cuts = {"a": [7, 1, 1, 1, 1], "b": [2, 1, 1, 1, 1]}
    done, got = {"a": 0, "b": 0}, {"a": [], "b": []}
    for r in streams:
        cache.admit(r)
    for stepi in range(5):
        entries = [(r, cuts[r][stepi]) for r in ("a", "b")]
        step = step_for(cache, entries)
        rows = torch.cat([streams[r][done[r]:done[r] + n] for r, n in entries]).to(dev())
        y = total(part.forward(ops.NormedRows(rows, nw, eps, torch.bfloat16), step, view)).float().cpu()
        row = 0
        for r, n in entries:
            got[r].append(y[row:row + n])
            row += n
            done[r] += n
            cache.commit(r, n)
    assert calls == ([] if bias else [2, 2, 2, 2])
    for r in streams:
        assert rel_err(torch.cat(got[r]), expect[r]) < TOL[torch.bfloat16]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh,nkv,d,window", [(4, 2, 16, 0), (3, 1, 32, 0), (8, 2, 64, 0), (8, 2, 64, 20)])
def test_attention_part(dtype, nh, nkv, d, window, monkeypatch):
    """The mixer with its pages: a prompt portion, then single tokens, against the
    plain mixer on the whole sequence.  In bfloat16 with a head size the matrix cores take,
    a step of single tokens runs norm, rotation and cache write inside its attention."""
    from zig_ai_amd.cache import CacheManager
    from zig_ai_amd.config.spec import PartSpec
    from zig_ai_amd.kernels import ops
    from zig_ai_amd.parts import lookup
    calls = []
    fused = ops.rope_attention_decode
    monkeypatch.setattr(ops, "rope_attention_decode",
                        lambda *a, **k: (calls.append(a[0].shape[0]), fused(*a, **k))[1])
    cls = lookup("mixer", "gqa_attention")
    H, theta, eps = 80, 10000.0, 1e-5
    rope = PartSpec("rope", {"head_dim": d, "rotary_dim": d, "theta": theta, "pairing": "half"})
    params = {"hidden_size": H, "num_heads": nh, "num_kv_heads": nkv, "head_dim": d, "qk_norm": True,
              "norm_eps": eps, "window": window, "softmax_scale": None, "bias": False, "position": rope}
    w = {"q_proj.weight": rnd((nh * d, H), 19, 0.3), "k_proj.weight": rnd((nkv * d, H), 20, 0.3),
         "v_proj.weight": rnd((nkv * d, H), 21, 0.2), "out_proj.weight": rnd((H, nh * d), 22, 0.2),
         "q_norm.weight": rnd((d,), 23, 0.2) + 1, "k_norm.weight": rnd((d,), 24, 0.2) + 1}
    need = cls.cache_need(params)
    assert need.is_kv and (need.planes[0], need.window) == ((nkv, d), window)
    part = cls(params, place(w, cls.tensor_rules(params), dtype), runtime(dtype))
    cache = CacheManager({0: need}, 8, 16, 2, device=dev(), dtype=dtype)
    view = cache.view(0)
    T = 45
    x = rnd((T, H), 25).to(dtype)
    wd = {k.replace(".weight", ""): v.to(dtype if v.dim() == 2 else torch.float32).double() for k, v in w.items()}
    expect = plain.attention_mixer(x.double(), wd, torch.arange(T), nh, nkv, d, eps, theta, window)
    cache.admit("r")
    got, done = [], 0
    for n in [30, 1, 1, 5, 1, 1, 1, 1, 1, 1, 1, 1]:
        step = step_for(cache, [("r", n)])
        got.append(total(part.forward(x[done:done + n].to(dev()), step, view)).cpu())
        cache.commit("r", n)
        done += n
    assert done == T
    assert rel_err(torch.cat(got), expect) < TOL[dtype]
    assert calls == ([1] * 10 if dtype == torch.bfloat16 and d == 64 else [])


@pytest.mark.parametrize("T", [12, 20])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_block_arrangement(dtype, T):
    """pre_norm_residual: h = x + mixer(norm1(x)); y = h + ffn(norm2(h)), with the adds
    deferred into the next norm; with at most 16 tokens in bfloat16 the projections
    run the norms and add to the stream themselves, and nothing is left pending."""
    from zig_ai_amd.cache import CacheManager
    from zig_ai_amd.parts import lookup
    H, L, I, eps = 64, 3, 96, 1e-5
    rt = runtime(dtype)
    norm_cls, mix_cls, ffn_cls = lookup("norm", "rms_norm"), lookup("mixer", "short_conv"), lookup("feed_forward", "swiglu")
    n1w, n2w = rnd((H,), 30, 0.2) + 1, rnd((H,), 31, 0.2) + 1
    mw = {"in_proj.weight": rnd((3 * H, H), 32, 0.2), "conv.weight": rnd((H, L), 33, 0.5),
          "out_proj.weight": rnd((H, H), 34, 0.2)}
    fw = {"gate.weight": rnd((I, H), 35, 0.2), "up.weight": rnd((I, H), 36, 0.2), "down.weight": rnd((H, I), 37, 0.2)}
    mp, fp, npar = {"hidden_size": H, "kernel_size": L, "bias": False}, {"hidden_size": H, "intermediate_size": I}, {"width": H, "eps": eps}
    block = lookup("arrangement", "pre_norm_residual")({
        "mixer_norm": norm_cls(npar, place({"weight": n1w}, norm_cls.tensor_rules(npar), dtype), rt),
        "mixer": mix_cls(mp, place(mw, mix_cls.tensor_rules(mp), dtype), rt),
        "feed_forward_norm": norm_cls(npar, place({"weight": n2w}, norm_cls.tensor_rules(npar), dtype), rt),
        "feed_forward": ffn_cls(fp, place(fw, ffn_cls.tensor_rules(fp), dtype), rt)})
    cache = CacheManager({0: mix_cls.cache_need(mp)}, 4, 4, 1, device=dev(), dtype=dtype)
    cache.admit("r")
    x = rnd((T, H), 38)
    step = step_for(cache, [("r", T)])
    residual, pending = block.forward(x.clone().to(dev()), None, step, cache.view(0))
    assert (pending is None) == (dtype == torch.bfloat16 and T <= 16)
    y = residual.double().cpu() + still_pending(residual, pending).double().cpu()
    q = lambda t: t.to(dtype).double()
    h = x.double() + plain.short_conv_mixer(
        plain.rms_norm(x.double(), n1w.double(), eps),
        {"in_proj": q(mw["in_proj.weight"]), "conv": mw["conv.weight"].double(), "out_proj": q(mw["out_proj.weight"])})
    expect = h + plain.swiglu_ffn(plain.rms_norm(h, n2w.double(), eps), q(fw["gate.weight"]), q(fw["up.weight"]),
                                  q(fw["down.weight"]))
    assert rel_err(y, expect) < TOL[dtype]
