"""What pins the plain implementation besides the reference's text: vectors the
reference's own tests hold, special cases that reduce to a library routine, and
invariants.  Each is chosen so that a plausible mistake (a wrong sign or pairing
in the rotation, a norm weight in the wrong place, an off-by-one in the
convolution or the mask) fails it."""

import math

import pytest
import torch
import torch.nn.functional as F

import engine_util as eu
import plain_lfm2 as plain
from tiny_configs import TINY_A, TINY_B

D = torch.float64


def rnd(*shape, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=D)


# ----------------------------------------------------------------------- norm
def test_rms_norm_is_the_library_routine():
    x, w = rnd(5, 24, seed=1), rnd(24, seed=2)
    assert torch.allclose(plain.rms_norm(x, w, 1e-5), F.rms_norm(x, (24,), w, 1e-5), atol=1e-12)


def test_rms_norm_reference_vectors_and_invariants():
    """norm.zig:83-103 ([1,2,3,4] and ones, weight 1)."""
    out = plain.rms_norm(torch.tensor([[1.0, 2, 3, 4], [1, 1, 1, 1]], dtype=D), torch.ones(4, dtype=D), 0.0)
    assert torch.allclose(out[0], torch.tensor([1.0, 2, 3, 4], dtype=D) / math.sqrt(7.5))
    assert torch.allclose(out[1], torch.ones(4, dtype=D))
    x, w = rnd(3, 16, seed=3), rnd(16, seed=4)
    assert torch.allclose(plain.rms_norm(7.0 * x, w, 0.0), plain.rms_norm(x, w, 0.0))   # scale-free
    # the weight multiplies after the scale (no "1 + w"): weight 0 gives 0
    assert plain.rms_norm(x, torch.zeros(16, dtype=D), 1e-5).abs().max() == 0
    # rows are independent
    assert torch.equal(plain.rms_norm(x, w, 1e-5)[1], plain.rms_norm(x[1:2], w, 1e-5)[0])
    # eps sits inside the root
    assert torch.allclose(plain.rms_norm(torch.zeros(1, 4, dtype=D) + 1e-3, torch.ones(4, dtype=D), 1.0),
                          torch.full((1, 4), 1e-3 / math.sqrt(1e-6 + 1.0), dtype=D))


# ----------------------------------------------------------------------- rope
@pytest.mark.parametrize("pairing", ["half", "adjacent"])
def test_rope_invariants(pairing):
    """rope.zig:226-253 holds the rotation to keeping the norm, for shape [1,2,4,64], base 1e4."""
    x = rnd(4, 2, 64, seed=5)
    pos = torch.tensor([0, 1, 17, 300])
    y = plain.apply_rope(x, pos, 10000.0, pairing=pairing)
    assert torch.equal(y[0], x[0])                                        # position 0: identity
    assert torch.allclose(y.norm(dim=-1), x.norm(dim=-1), atol=1e-12)     # norm kept
    # only distances count: <q(p), k(p')> depends on p - p'
    q, k = rnd(1, 1, 64, seed=6), rnd(1, 1, 64, seed=7)
    def dot(p, pp):
        a = plain.apply_rope(q, torch.tensor([p]), 10000.0, pairing=pairing)
        b = plain.apply_rope(k, torch.tensor([pp]), 10000.0, pairing=pairing)
        return float((a * b).sum())
    assert abs(dot(9, 4) - dot(105, 100)) < 1e-9
    assert abs(dot(9, 4) - dot(4, 9)) > 1e-3                              # and their sign counts


def test_rope_is_a_complex_multiplication():
    d, theta = 32, 1e6
    x = rnd(3, 2, d, seed=8)
    pos = torch.tensor([2, 50, 777])
    inv = plain.rope_inv_freq(d, theta)
    assert torch.allclose(inv, torch.tensor([theta ** (-2 * i / d) for i in range(d // 2)], dtype=D))
    rot = torch.polar(torch.ones(3, d // 2, dtype=D), pos[:, None].double() * inv[None, :])[:, None, :]
    half = torch.complex(x[..., : d // 2], x[..., d // 2:]) * rot
    want_half = torch.cat([half.real, half.imag], dim=-1)
    assert torch.allclose(plain.apply_rope(x, pos, theta, pairing="half"), want_half, atol=1e-12)
    adj = torch.view_as_complex(x.reshape(3, 2, d // 2, 2).contiguous()) * rot
    assert torch.allclose(plain.apply_rope(x, pos, theta, pairing="adjacent"),
                          torch.view_as_real(adj).reshape(3, 2, d), atol=1e-12)
    # the two pairings are different functions: picking the wrong one cannot pass
    assert not torch.allclose(want_half, torch.view_as_real(adj).reshape(3, 2, d))


def test_partial_rotation_leaves_the_rest():
    x = rnd(2, 1, 16, seed=9)
    y = plain.apply_rope(x, torch.tensor([3, 4]), 100.0, rotary_dim=8)
    assert torch.equal(y[..., 8:], x[..., 8:]) and not torch.equal(y[..., :8], x[..., :8])


# ------------------------------------------------------------------- attention
def test_gqa_head_map_reference_vectors():
    """gqa.zig:87-106."""
    assert [plain.kv_head_of(h, 32, 8) for h in (0, 3, 4, 31)] == [0, 0, 1, 7]
    assert [plain.kv_head_of(h, 8, 2) for h in range(8)] == [0, 0, 0, 0, 1, 1, 1, 1]


def test_attention_is_the_library_routine():
    T, nh, nkv, d = 9, 6, 2, 16
    q, k, v = rnd(T, nh, d, seed=10), rnd(T, nkv, d, seed=11), rnd(T, nkv, d, seed=12)
    want = F.scaled_dot_product_attention(
        q.transpose(0, 1)[None], k.repeat_interleave(nh // nkv, 1).transpose(0, 1)[None],
        v.repeat_interleave(nh // nkv, 1).transpose(0, 1)[None], is_causal=True)[0].transpose(0, 1)
    assert torch.allclose(plain.causal_attention(q, k, v), want, atol=1e-12)


def test_attention_special_cases():
    nh, nkv, d = 4, 2, 8
    q, k, v = rnd(1, nh, d, seed=13), rnd(1, nkv, d, seed=14), rnd(1, nkv, d, seed=15)
    out = plain.causal_attention(q, k, v)            # one key: softmax is 1, out = V
    for h in range(nh):                              # (hybrid_attn.zig:1207-1212)
        assert torch.allclose(out[0, h], v[0, h // 2])
    T = 6
    q, v = rnd(T, nh, d, seed=16), rnd(T, nkv, d, seed=17)
    k = torch.zeros(T, nkv, d, dtype=D)              # equal scores: the mean of the values so far
    out = plain.causal_attention(q, k, v)
    assert torch.allclose(out[4, 3], v[:5, 1].mean(0))
    # a window of 1 sees only itself; a window of T is no window
    assert torch.allclose(plain.causal_attention(q, rnd(T, nkv, d, seed=18), v, window=1)[:, 0], v[:, 0])
    kk = rnd(T, nkv, d, seed=19)
    assert torch.allclose(plain.causal_attention(q, kk, v, window=T), plain.causal_attention(q, kk, v))
    # window w: query t sees keys t-w+1 .. t
    w2 = plain.causal_attention(q, k, v, window=2)
    assert torch.allclose(w2[3, 0], v[2:4, 0].mean(0))


# ------------------------------------------------------------------------ conv
@pytest.mark.parametrize("H,L,T", [(6, 3, 10), (5, 4, 3), (4, 1, 5), (3, 2, 1)])
def test_conv_is_the_library_routine(H, L, T):
    u, w, b = rnd(T, H, seed=20), rnd(H, L, seed=21), rnd(H, seed=22)
    want = F.conv1d(u.T[None], w[:, None, :], b, padding=L - 1, groups=H)[0, :, :T].T
    assert torch.allclose(plain.causal_depthwise_conv(u, w, b), want, atol=1e-12)


def test_conv_identity_and_causality():
    H, L, T = 4, 3, 7
    u = rnd(T, H, seed=23)
    w = torch.zeros(H, L, dtype=D)
    w[:, L - 1] = 1                                   # the last tap is the current input
    assert torch.equal(plain.causal_depthwise_conv(u, w, None), u)
    w = torch.zeros(H, L, dtype=D)
    w[:, 0] = 1                                       # the first tap is the oldest input
    out = plain.causal_depthwise_conv(u, w, None)
    assert torch.equal(out[L - 1:], u[: T - L + 1]) and out[: L - 1].abs().max() == 0
    ww = rnd(H, L, seed=24)
    a = plain.causal_depthwise_conv(u, ww, None)
    u2 = u.clone()
    u2[5] += 1.0                                      # a later input changes no earlier output
    assert torch.equal(plain.causal_depthwise_conv(u2, ww, None)[:5], a[:5])


def test_short_conv_mixer_order_of_gates():
    """(B, C, x) in that order: B gates the input of the convolution, C its output.
    Seen by what each gate can reach, not by the formula again: in_proj is chosen so
    that B[t] is feature 0 of token t, C[t] feature 1 and x[t] feature 2, and the filter
    is all ones.  A token whose B is zero then vanishes from the L outputs that its
    input reaches (and those outputs no longer depend on its x); a token whose C is zero
    has a zero output of its own and nothing else changes."""
    H, T, L = 4, 9, 3
    x = rnd(T, H, seed=25) + 2.0                       # no accidental zeros
    in_proj = torch.zeros((3 * H, H), dtype=D)
    in_proj[0:H, 0] = 1.0                              # B[t, c] = x[t, 0]
    in_proj[H:2 * H, 1] = 1.0                          # C[t, c] = x[t, 1]
    in_proj[2 * H:3 * H, 2] = 1.0                      # xx[t, c] = x[t, 2]
    w = {"in_proj": in_proj, "conv": torch.ones((H, L), dtype=D), "out_proj": torch.eye(H, dtype=D)}
    y = plain.short_conv_mixer(x, w)
    for t in range(T):                                 # the definition, token by token
        want = x[t, 1] * sum(x[s, 0] * x[s, 2] for s in range(max(0, t - L + 1), t + 1))
        assert torch.allclose(y[t], want.expand(H))
    t0 = 4
    xb = x.clone()
    xb[t0, 0] = 0.0                                    # B of token t0 is zero
    yb = plain.short_conv_mixer(xb, w)
    xb2 = xb.clone()
    xb2[t0, 2] = 123.0                                 # ... so its x reaches nothing
    assert torch.equal(plain.short_conv_mixer(xb2, w), yb)
    changed = [t for t in range(T) if not torch.equal(yb[t], y[t])]
    assert changed == list(range(t0, t0 + L))          # the outputs its input reached
    xc = x.clone()
    xc[t0, 1] = 0.0                                    # C of token t0 is zero
    yc = plain.short_conv_mixer(xc, w)
    assert yc[t0].abs().max() == 0
    assert [t for t in range(T) if not torch.equal(yc[t], y[t])] == [t0]


# ------------------------------------------------------------------------- ffn
def test_swiglu_is_the_library_routine():
    """ffn.zig:83-111 checks [4,128] -> [4,128] through 256."""
    x, wg, wu, wd = rnd(4, 128, seed=28), rnd(256, 128, seed=29), rnd(256, 128, seed=30), rnd(128, 256, seed=31)
    out = plain.swiglu_ffn(x, wg, wu, wd)
    assert out.shape == (4, 128)
    assert torch.allclose(out, (F.silu(x @ wg.T) * (x @ wu.T)) @ wd.T, atol=1e-9)


def test_ffn_width():
    assert plain.ffn_width({"block_ff_dim": 12288, "block_multiple_of": 256}) == 8192
    assert plain.ffn_width({"block_ff_dim": 6656, "block_multiple_of": 256}) == 4608
    assert plain.ffn_width({"block_ff_dim": 10752, "block_multiple_of": 256}) == 7168
    assert plain.ffn_width(TINY_B) == 256 and plain.ffn_width(TINY_A) == 192


def test_embedding_reference_vector():
    """embedding.zig:53-77: tokens {0,5,10,20,30,40}: row 0 of the output is row 0 of the table."""
    table = rnd(50, 8, seed=32)
    out = plain.embedding([0, 5, 10, 20, 30, 40], table)
    assert torch.equal(out[0], table[0]) and torch.equal(out[3], table[20])


# ----------------------------------------------------------------- whole model
def test_whole_model_structure():
    folder = eu.model_folder(TINY_B, 1, torch.float32, **eu.sharp_kwargs())
    m = plain.PlainLfm2(folder)
    toks = eu.random_tokens(12, 512, 1)
    logits = m.logits(toks)
    assert logits.shape == (12, 512)
    # causal: a later token changes no earlier logits, and does change its own
    toks2 = list(toks)
    toks2[8] = (toks2[8] + 1) % 512
    l2 = m.logits(toks2)
    assert torch.equal(l2[:8], logits[:8]) and not torch.allclose(l2[8:], logits[8:])
    # every layer matters (a skipped layer would go unnoticed otherwise)
    for i in range(6):
        assert not torch.allclose(m.hidden_states(toks, upto_layer=i), m.hidden_states(toks, upto_layer=i + 1))
    # untied head: logits use lm_head, not the embedding table
    n = plain.rms_norm(m.hidden_states(toks), m.w["model.embedding_norm.weight"], m.eps)
    assert torch.allclose(logits, n @ m.w["lm_head.weight"].T)
    tied = plain.PlainLfm2(eu.model_folder(TINY_A, 0, torch.float32, **eu.sharp_kwargs()))
    t = eu.random_tokens(5, 256, 2)
    n = plain.rms_norm(tied.hidden_states(t), tied.w["model.embedding_norm.weight"], tied.eps)
    assert torch.allclose(tied.logits(t), n @ tied.w["model.embed_tokens.weight"].T)


def test_attention_layers_see_distances_only():
    """Shifting every position by the same amount leaves the hidden states where
    they are: the rotation enters through differences of positions only."""
    folder = eu.model_folder(TINY_B, 1, torch.float32, **eu.sharp_kwargs())
    m = plain.PlainLfm2(folder)
    toks = eu.random_tokens(10, 512, 3)
    assert torch.allclose(m.hidden_states(toks), m.hidden_states(toks, position_offset=1000), atol=1e-9)


# -------------------------------------------------------------------- sampling
def test_sampler():
    logits = torch.tensor([1.0, 3.0, 3.0, -1.0, 0.5], dtype=D)
    assert plain.argmax_first(logits) == 1                              # first of the tie
    assert plain.sample_token(logits, 0.0, 0.9) == 1                    # temperature 0: greedy
    assert plain.sample_token(logits, 1e-4, 0.3) == 1                   # T -> 0 tends to it
    p = torch.softmax(logits / 0.7, 0)
    cdf = torch.cumsum(p, 0)
    for u in (0.0, 0.2, 0.5, 0.77, 0.999):
        want = int((cdf >= u).nonzero()[0]) if u > 0 else 0
        assert plain.sample_token(logits, 0.7, u) == want
    n = 20000
    draws = torch.tensor([plain.sample_token(logits, 0.7, (i + 0.5) / n) for i in range(0, n, 10)])
    freq = torch.bincount(draws, minlength=5).double() / len(draws)
    assert (freq - p).abs().max() < 2e-3
    keep = plain.kept_after_top_k_top_p(logits, 2, 1.0)
    assert keep.tolist() == [False, True, True, False, False]
    keep = plain.kept_after_top_k_top_p(logits, 0, 0.5)
    assert keep.tolist() == [False, True, True, False, False]           # ties with the cut stay
    keep = plain.kept_after_top_k_top_p(logits, 0, 0.95)               # 0.894 + 0.061 reaches it
    assert keep.tolist() == [True, True, True, False, False]
    keep = plain.kept_after_top_k_top_p(logits, 0, 0.97)
    assert keep.tolist() == [True, True, True, False, True]
    assert plain.sample_token(logits, 1.0, 0.999, top_k=2) == 2
    pen = plain.apply_repetition_penalty(logits, [1, 3, 1], 2.0)        # once per occurrence
    assert pen.tolist() == [1.0, 0.75, 3.0, -2.0, 0.5]
