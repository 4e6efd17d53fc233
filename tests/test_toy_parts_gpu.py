"""Extending the framework from outside: a toy mixer with state of its own and a
toy architecture around it, both defined here, are registered, built from a
model folder, and stepped through the engine's step function, cache manager and
run order without a change to the framework's files.  Also: a run order that
names a layer twice, and a layer that reads another layer's cache; and a second
toy architecture with a feed-forward that routes tokens to experts and a position
encoding of another kind, beside the framework's own ShortConv mixer; and a norm, an
embedding and a head of another kind around the framework's own layers.
"""

import pytest
import torch

import engine_util as eu
import plain_lfm2 as plain

pytestmark = pytest.mark.gpu


# --------------------------------------------------------------- the toy mixer
def toy_classes():
    from zig_ai_amd.kernels import ops
    from zig_ai_amd.parts import Mixer, StateNeed, TensorRule, register_mixer

    class RunningMeanMixer(Mixer):
        """y[t] = W * mean(x[0..t]): needs the sum of all earlier inputs and their
        count, a state of ``width + 1`` floats per request."""
        kind = "toy_running_mean"
        kernel_sources = ("gemm",)

        @classmethod
        def tensor_rules(cls, params):
            w = int(params["width"])
            return {"mix.weight": TensorRule(((w, w),))}

        @classmethod
        def cache_need(cls, params):
            return StateNeed((int(params["width"]) + 1,))

        def __init__(self, params, tensors, runtime):
            super().__init__(params, tensors, runtime)
            self.width = int(params["width"])
            self.weight = tensors["mix.weight"]

        def forward(self, x, step, cache):
            out = torch.empty_like(x, dtype=torch.float32)
            row = 0
            for n, slot in zip(step.seq_lens_host, step.slots_host):
                state = cache.state[slot]
                xs = x[row:row + n].float()
                sums = state[: self.width] + torch.cumsum(xs, dim=0)
                counts = state[self.width] + torch.arange(1, n + 1, device=x.device)
                out[row:row + n] = sums / counts[:, None]
                state[: self.width] = sums[-1]
                state[self.width] = counts[-1]
                row += n
            return ops.linear(out.to(x.dtype), self.weight)

    class RunningMaxMixer(Mixer):
        """y[t] = W * max(x[0..t]), element by element: the state is the largest input
        so far, which for a new request is minus infinity, not zero."""
        kind = "toy_running_max"
        kernel_sources = ("gemm",)

        @classmethod
        def tensor_rules(cls, params):
            w = int(params["width"])
            return {"mix.weight": TensorRule(((w, w),))}

        @classmethod
        def cache_need(cls, params):
            return StateNeed((int(params["width"]),), init=float("-inf"))

        def __init__(self, params, tensors, runtime):
            super().__init__(params, tensors, runtime)
            self.weight = tensors["mix.weight"]

        def forward(self, x, step, cache):
            out = torch.empty_like(x, dtype=torch.float32)
            row = 0
            for n, slot in zip(step.seq_lens_host, step.slots_host):
                state = cache.state[slot]
                top = torch.cummax(torch.cat([state[None], x[row:row + n].float()]), dim=0).values[1:]
                out[row:row + n] = top
                state.copy_(top[-1])
                row += n
            return ops.linear(out.to(x.dtype), self.weight)

    register_mixer(RunningMeanMixer.kind, RunningMeanMixer)
    register_mixer(RunningMaxMixer.kind, RunningMaxMixer)
    return RunningMeanMixer


class ToyConfig:
    """A whole toy architecture: layers alternate the toy mixer and attention."""

    def __init__(self, data):
        self.data = dict(data)

    @classmethod
    def from_dict(cls, data):
        return cls(data)

    def to_dict(self):
        return dict(self.data)

    def to_spec(self):
        from zig_ai_amd.config.spec import LayerCall, LayerSpec, ModelSpec, PartSpec
        d = self.data
        H, V = d["width"], d["vocab_size"]
        layers = []
        for i, kind in enumerate(d["kinds"]):
            p = f"layers.{i}."
            if kind in ("toy", "max"):
                mixer = PartSpec("toy_running_mean" if kind == "toy" else "toy_running_max",
                                 {"width": H}, {"mix.weight": (p + "mix.weight",)})
            else:
                rope = PartSpec("rope", {"head_dim": d["head_dim"], "rotary_dim": d["head_dim"] // 2,
                                         "theta": 100.0, "pairing": "adjacent"})
                mixer = PartSpec("gqa_attention",
                                 {"hidden_size": H, "num_heads": d["heads"], "num_kv_heads": d["kv_heads"],
                                  "head_dim": d["head_dim"], "qk_norm": False, "norm_eps": 1e-5,
                                  "window": d.get("window", 0), "softmax_scale": d.get("scale"),
                                  "bias": False, "position": rope},
                                 {k + ".weight": (p + k + ".weight",)
                                  for k in ("q_proj", "k_proj", "v_proj", "out_proj")})
            ffn = PartSpec("swiglu", {"hidden_size": H, "intermediate_size": d["ffn"]},
                           {k + ".weight": (p + "ffn." + k + ".weight",) for k in ("gate", "up", "down")})
            n1 = PartSpec("rms_norm", {"width": H, "eps": 1e-5}, {"weight": (p + "norm1.weight",)})
            n2 = PartSpec("rms_norm", {"width": H, "eps": 1e-5}, {"weight": (p + "norm2.weight",)})
            layers.append(LayerSpec.pre_norm(mixer, ffn, n1, n2))
        schedule = tuple(LayerCall(*c) for c in d["schedule"])
        return ModelSpec("ToyForCausalLM", H, V,
                         PartSpec("token_embedding", {"vocab_size": V, "hidden_size": H},
                                  {"weight": ("embed.weight",)}),
                         tuple(layers), schedule,
                         PartSpec("rms_norm", {"width": H, "eps": 1e-5}, {"weight": ("norm.weight",)}),
                         PartSpec("linear_head", {"vocab_size": V, "hidden_size": H, "tied": True}, {}))


TOY = {"architectures": ["ToyForCausalLM"], "width": 48, "vocab_size": 97, "ffn": 72,
       "heads": 3, "kv_heads": 3, "head_dim": 16, "window": 9, "scale": 0.5,
       "kinds": ["toy", "attn", "toy"],
       # layer 0 runs twice (second time with a cache of its own), the last entry reads
       # the keys and values that entry 1 wrote
       "schedule": [(0, 0), (1, 1), (2, 2), (0, 3), (1, 1, False)]}


def toy_oracle(folder, tokens, d=None):
    """The toy model, whole sequence, float64, written out directly."""
    from safetensors.torch import load_file
    w = {k: v.double() for k, v in load_file(folder + "/model.safetensors").items()}
    d = d or TOY
    H, nh, hd = d["width"], d["heads"], d["head_dim"]
    x = w["embed.weight"][torch.tensor(tokens)]
    pos = torch.arange(len(tokens))
    kv_of_entry = {}
    for layer, cache, *rest in d["schedule"]:
        writes = not rest or rest[0]
        p = f"layers.{layer}."
        n1 = plain.rms_norm(x, w[p + "norm1.weight"], 1e-5)
        if d["kinds"][layer] == "toy":
            mean = torch.cumsum(n1, 0) / torch.arange(1, len(tokens) + 1)[:, None]
            m = mean @ w[p + "mix.weight"].T
        elif d["kinds"][layer] == "max":
            m = torch.cummax(n1, 0).values @ w[p + "mix.weight"].T
        else:
            T = len(tokens)
            q = (n1 @ w[p + "q_proj.weight"].T).view(T, nh, hd)
            q = plain.apply_rope(q, pos, 100.0, hd // 2, "adjacent")
            if writes:
                k = (n1 @ w[p + "k_proj.weight"].T).view(T, nh, hd)
                k = plain.apply_rope(k, pos, 100.0, hd // 2, "adjacent")
                v = (n1 @ w[p + "v_proj.weight"].T).view(T, nh, hd)
                kv_of_entry[cache] = (k, v)
            k, v = kv_of_entry[cache]
            o = plain.causal_attention(q, k, v, pos, window=d["window"], scale=d["scale"])
            m = o.reshape(T, nh * hd) @ w[p + "out_proj.weight"].T
        h = x + m
        n2 = plain.rms_norm(h, w[p + "norm2.weight"], 1e-5)
        x = h + plain.swiglu_ffn(n2, w[p + "ffn.gate.weight"], w[p + "ffn.up.weight"],
                                 w[p + "ffn.down.weight"])
    return plain.rms_norm(x, w["norm.weight"], 1e-5) @ w["embed.weight"].T


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_architecture_steps_through_the_engine(dtype):
    from zig_ai_amd.config import register_architecture
    from zig_ai_amd.engine import DecoderModel, ModelRunner
    toy_classes()
    register_architecture("ToyForCausalLM", ToyConfig)
    store = torch.float32 if dtype == "float32" else torch.bfloat16
    # query/key weights sized so that scores spread over about one unit: sharper
    # scores would turn bfloat16's rounding of q and k into percent-sized changes
    # of the softmax, which is the number format's doing, not the engine's
    folder = eu.model_folder(TOY, 11, store, std=0.2, norm_init="around_one",
                             role_std={"norm": 0.2, "q_proj.weight": 0.08, "k_proj.weight": 0.08})
    model = DecoderModel.from_folder(folder, dtype)
    # four cache entries: two states (layer 0 twice), one state (layer 2), one paged group
    assert len(model.cache_needs) == 4
    lengths = [40, 9, 23]
    prompts = [eu.random_tokens(n, 97, 600 + n) for n in lengths]
    expect = [toy_oracle(folder, p) for p in prompts]
    tol = 1e-4 if dtype == "float32" else 2.5e-2
    for schedule in (eu.whole(lengths), eu.changing_portions(lengths, 1),
                     eu.mixed(lengths, seed=3, max_live=3, decode_tail=5)):
        runner = ModelRunner(model, page_size=4, num_pages=24, num_slots=3)
        got = eu.run_schedule(runner, prompts, schedule)
        for g, e in zip(got, expect):
            assert eu.rel_err(g, e) < tol
        # the window of 9 lets pages behind it go back while the request still runs
        assert runner.cache.stats()["groups"][0]["pages_high_water"] < sum(
            (n + 3) // 4 for n in lengths)


TOY_MAX = dict(TOY, kinds=["max", "attn"], schedule=[(0, 0), (1, 1)])


def test_a_state_that_does_not_start_at_zero():
    """A mixer whose state starts at minus infinity: every request, also one that takes
    a slot another request has left, begins from that value and from nothing else."""
    from zig_ai_amd.config import register_architecture
    from zig_ai_amd.engine import DecoderModel, ModelRunner
    toy_classes()
    register_architecture("ToyForCausalLM", ToyConfig)
    folder = eu.model_folder(TOY_MAX, 12, torch.float32, std=0.2, norm_init="around_one",
                             role_std={"norm": 0.2, "q_proj.weight": 0.08, "k_proj.weight": 0.08})
    model = DecoderModel.from_folder(folder, "float32")
    lengths = [21, 9, 30, 14, 11]
    prompts = [eu.random_tokens(n, 97, 700 + n) for n in lengths]
    # every input of the first request is below zero at some channel with near
    # certainty, so a state that started at zero would show in its first tokens
    expect = [toy_oracle(folder, p, TOY_MAX) for p in prompts]
    for schedule in (eu.whole(lengths), eu.mixed(lengths, seed=5, max_live=2, decode_tail=4)):
        # two slots for five requests: each slot is used again, after a request that
        # left its running maximum there
        runner = ModelRunner(model, page_size=4, num_pages=24, num_slots=2)
        got = eu.run_schedule(runner, prompts, schedule)
        for g, e in zip(got, expect):
            assert eu.rel_err(g, e) < 1e-4


# ------------------------------ a feed-forward with routing, another position encoding
def routed_classes():
    from zig_ai_amd.kernels import ops
    from zig_ai_amd.parts import (FeedForward, PositionEncoding, TensorRule, register_feed_forward,
                                  register_position)

    class TopOneExperts(FeedForward):
        """Every token goes to the expert whose router logit is largest (the first of
        equals) and takes that expert's SwiGLU, weighted by the softmax probability
        of the choice.  Router logits and softmax in 32-bit.  The part looks at the
        choices on the host, so it is not safe to record into a graph."""
        kind = "toy_top_one_experts"
        kernel_sources = ("gemm", "activation")

        @classmethod
        def tensor_rules(cls, params):
            H, I, E = int(params["hidden_size"]), int(params["intermediate_size"]), int(params["experts"])
            rules = {"router.weight": TensorRule(((E, H),))}
            for e in range(E):
                rules[f"experts.{e}.gate_up.weight"] = TensorRule(((2 * I, H),))
                rules[f"experts.{e}.down.weight"] = TensorRule(((H, I),))
            return rules

        def __init__(self, params, tensors, runtime):
            super().__init__(params, tensors, runtime)
            self.experts = int(params["experts"])
            self.router = tensors["router.weight"].float()
            self.gate_up = [tensors[f"experts.{e}.gate_up.weight"] for e in range(self.experts)]
            self.down = [tensors[f"experts.{e}.down.weight"] for e in range(self.experts)]

        def forward(self, x, step=None):
            logits = ops.linear(x, self.router, out_dtype=torch.float32)
            prob = torch.softmax(logits, dim=-1)
            weight, choice = prob.max(dim=-1)
            out = torch.zeros((x.shape[0], x.shape[1]), dtype=torch.float32, device=x.device)
            for e in range(self.experts):
                rows = (choice == e).nonzero().view(-1)
                if rows.numel() == 0:
                    continue
                a = ops.swiglu(ops.linear(x.index_select(0, rows).contiguous(), self.gate_up[e]))
                y = ops.linear(a, self.down[e], out_dtype=torch.float32)
                out.index_copy_(0, rows, y * weight.index_select(0, rows)[:, None])
            return out.to(x.dtype)

    class AddedWaves(PositionEncoding):
        """Absolute positions: element i of every query and key head takes
        ``amplitude * sin(position * rate^i + i)``."""
        kind = "toy_added_waves"

        def __init__(self, params, tensors, runtime):
            super().__init__(params, tensors, runtime)
            d = int(params["head_dim"])
            i = torch.arange(d, dtype=torch.float32, device=runtime.device)
            self.rates = float(params["rate"]) ** i
            self.phase = i
            self.amplitude = float(params["amplitude"])

        def apply(self, q, k, positions):
            wave = self.amplitude * torch.sin(positions.float()[:, None] * self.rates + self.phase)
            return (q.float() + wave[:, None, :]).to(q.dtype), (k.float() + wave[:, None, :]).to(k.dtype)

    register_feed_forward(TopOneExperts.kind, TopOneExperts)
    register_position(AddedWaves.kind, AddedWaves)


class RoutedConfig:
    """Attention with the toy position encoding, and the framework's own ShortConv
    mixer, each followed by the routed feed-forward."""

    def __init__(self, data):
        self.data = dict(data)

    @classmethod
    def from_dict(cls, data):
        return cls(data)

    def to_dict(self):
        return dict(self.data)

    def to_spec(self):
        from zig_ai_amd.config.spec import LayerCall, LayerSpec, ModelSpec, PartSpec
        d = self.data
        H, V, E, I = d["width"], d["vocab_size"], d["experts"], d["ffn"]
        layers = []
        for i, kind in enumerate(d["kinds"]):
            p = f"layers.{i}."
            if kind == "conv":
                mixer = PartSpec("short_conv", {"hidden_size": H, "kernel_size": d["taps"], "bias": False},
                                 {k + ".weight": (p + k + ".weight",) for k in ("in_proj", "conv", "out_proj")})
            else:
                waves = PartSpec("toy_added_waves", {"head_dim": d["head_dim"], "rate": 0.7, "amplitude": 0.5})
                mixer = PartSpec("gqa_attention",
                                 {"hidden_size": H, "num_heads": d["heads"], "num_kv_heads": d["kv_heads"],
                                  "head_dim": d["head_dim"], "qk_norm": True, "norm_eps": 1e-5,
                                  "bias": False, "position": waves},
                                 {k + ".weight": (p + k + ".weight",)
                                  for k in ("q_proj", "k_proj", "v_proj", "out_proj", "q_norm", "k_norm")})
            names = {"router.weight": (p + "router.weight",)}
            for e in range(E):
                names[f"experts.{e}.gate_up.weight"] = (p + f"experts.{e}.gate_up.weight",)
                names[f"experts.{e}.down.weight"] = (p + f"experts.{e}.down.weight",)
            ffn = PartSpec("toy_top_one_experts", {"hidden_size": H, "intermediate_size": I, "experts": E}, names)
            n1 = PartSpec("rms_norm", {"width": H, "eps": 1e-5}, {"weight": (p + "norm1.weight",)})
            n2 = PartSpec("rms_norm", {"width": H, "eps": 1e-5}, {"weight": (p + "norm2.weight",)})
            layers.append(LayerSpec.pre_norm(mixer, ffn, n1, n2))
        schedule = tuple(LayerCall(i, i) for i in range(len(layers)))
        return ModelSpec("ToyRoutedForCausalLM", H, V,
                         PartSpec("token_embedding", {"vocab_size": V, "hidden_size": H},
                                  {"weight": ("embed.weight",)}),
                         tuple(layers), schedule,
                         PartSpec("rms_norm", {"width": H, "eps": 1e-5}, {"weight": ("norm.weight",)}),
                         PartSpec("linear_head", {"vocab_size": V, "hidden_size": H, "tied": True}, {}))


ROUTED = {"architectures": ["ToyRoutedForCausalLM"], "width": 40, "vocab_size": 83, "ffn": 56,
          "experts": 3, "heads": 5, "kv_heads": 1, "head_dim": 16, "taps": 2,
          "kinds": ["attn", "conv", "attn"]}


def routed_oracle(folder, tokens):
    """The routed toy model, whole sequence, float64, written out directly; also
    returns the smallest gap between the two largest router logits of any token
    (a choice within rounding of a tie is no fault of the engine's)."""
    from safetensors.torch import load_file
    w = {k: v.double() for k, v in load_file(folder + "/model.safetensors").items()}
    d = ROUTED
    H, nh, nkv, hd, L = d["width"], d["heads"], d["kv_heads"], d["head_dim"], d["taps"]
    T = len(tokens)
    x = w["embed.weight"][torch.tensor(tokens)]
    pos = torch.arange(T, dtype=torch.float64)
    i = torch.arange(hd, dtype=torch.float64)
    wave = 0.5 * torch.sin(pos[:, None] * (0.7 ** i) + i)
    gap = float("inf")
    for layer, kind in enumerate(d["kinds"]):
        p = f"layers.{layer}."
        n1 = plain.rms_norm(x, w[p + "norm1.weight"], 1e-5)
        if kind == "conv":
            z = n1 @ w[p + "in_proj.weight"].T
            u = z[:, :H] * z[:, 2 * H:]
            m = (z[:, H:2 * H] * plain.causal_depthwise_conv(u, w[p + "conv.weight"].view(H, L), None)) \
                @ w[p + "out_proj.weight"].T
        else:
            q = plain.rms_norm((n1 @ w[p + "q_proj.weight"].T).view(T, nh, hd), w[p + "q_norm.weight"], 1e-5)
            k = plain.rms_norm((n1 @ w[p + "k_proj.weight"].T).view(T, nkv, hd), w[p + "k_norm.weight"], 1e-5)
            v = (n1 @ w[p + "v_proj.weight"].T).view(T, nkv, hd)
            o = plain.causal_attention(q + wave[:, None, :], k + wave[:, None, :], v)
            m = o.reshape(T, nh * hd) @ w[p + "out_proj.weight"].T
        h = x + m
        n2 = plain.rms_norm(h, w[p + "norm2.weight"], 1e-5)
        logits = n2 @ w[p + "router.weight"].T
        top = torch.sort(logits, dim=-1, descending=True).values
        gap = min(gap, float((top[:, 0] - top[:, 1]).min()))
        prob = torch.softmax(logits, dim=-1)
        f = torch.zeros_like(h)
        for t in range(T):
            e = int(torch.argmax(logits[t]))
            gu = n2[t] @ w[p + f"experts.{e}.gate_up.weight"].T
            a = torch.nn.functional.silu(gu[: d["ffn"]]) * gu[d["ffn"]:]
            f[t] = prob[t, e] * (a @ w[p + f"experts.{e}.down.weight"].T)
        x = h + f
    return plain.rms_norm(x, w["norm.weight"], 1e-5) @ w["embed.weight"].T, gap


def test_toy_routing_and_position_parts_step_through_the_engine():
    """A feed-forward that routes and a position encoding of another kind, both
    defined here, beside the framework's own mixers: registered, built and stepped
    in 32-bit under three ways of cutting the work.  (In bfloat16 a token whose two
    best router logits lie within rounding of each other may go to the other expert,
    which no tolerance of the logits covers; the 32-bit path decides the same as the
    plain formulas as long as no gap is within 1e-4, which is asserted.)"""
    from zig_ai_amd.config import register_architecture
    from zig_ai_amd.engine import DecoderModel, ModelRunner
    routed_classes()
    register_architecture("ToyRoutedForCausalLM", RoutedConfig)
    folder = eu.model_folder(ROUTED, 13, torch.float32, std=0.2, norm_init="around_one",
                             role_std={"norm": 0.2, "filter": 0.5})
    model = DecoderModel.from_folder(folder, "float32")
    assert not model.graph_safe          # the routed feed-forward looks at its choices on the host
    lengths = [31, 6, 18]
    prompts = [eu.random_tokens(n, 83, 700 + n) for n in lengths]
    expect = []
    for p in prompts:
        logits, gap = routed_oracle(folder, p)
        assert gap > 1e-4
        expect.append(logits)
    for schedule in (eu.whole(lengths), eu.changing_portions(lengths, 2),
                     eu.mixed(lengths, seed=5, max_live=3, decode_tail=4)):
        runner = ModelRunner(model, page_size=4, num_pages=20, num_slots=3)
        assert runner.graphs is None
        got = eu.run_schedule(runner, prompts, schedule)
        for g, e in zip(got, expect):
            assert eu.rel_err(g, e) < 1e-4


# ------------------- a position encoding inside a mixer decides whether steps are recorded
class WavedLfm2Config:
    """LFM2's own parts with the attention's rotary encoding replaced by the position part
    named under ``position_kind``."""

    def __init__(self, data):
        self.data = dict(data)

    @classmethod
    def from_dict(cls, data):
        return cls(data)

    def to_dict(self):
        return dict(self.data)

    def to_spec(self):
        import dataclasses

        from zig_ai_amd.config.lfm2 import Lfm2Config
        from zig_ai_amd.config.spec import LayerSpec, PartSpec
        inner = dict(self.data, architectures=["Lfm2ForCausalLM"])
        kind = inner.pop("position_kind")
        spec = Lfm2Config.from_dict(inner).to_spec()
        waves = PartSpec(kind, {"head_dim": spec.layers[0].mixer.params.get("head_dim", 16),
                                "rate": 0.7, "amplitude": 0.5})
        layers = []
        for layer in spec.layers:
            parts = dict(layer.parts)
            if parts["mixer"].kind == "gqa_attention":
                parts["mixer"] = parts["mixer"].with_params(position=waves)
            layers.append(LayerSpec(parts, layer.arrangement))
        return dataclasses.replace(spec, architecture=self.data["architectures"][0], layers=tuple(layers))


WAVED = {"architectures": ["ToyWavedForCausalLM"], "model_type": "lfm2", "hidden_size": 64,
         "num_hidden_layers": 3, "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 16,
         "vocab_size": 97, "layer_types": ["full_attention", "conv", "full_attention"],
         "intermediate_size": 96, "rope_theta": 10000.0, "norm_eps": 1e-5, "conv_L_cache": 3,
         "conv_bias": False, "tie_embedding": True, "max_position_embeddings": 512}


def test_a_nested_position_part_decides_whether_steps_are_recorded():
    """The attention mixer holds its position encoding inside it.  The model asks nested
    parts too whether a step may be recorded: with a position part that declares nothing
    (``graph_safe`` is false unless a part says otherwise) no graph is ever made, although
    every other part of the model is the framework's own and safe; the same encoding
    declared safe is recorded, and replayed steps give the logits of steps issued one
    kernel at a time.  Nothing under the package changes for either."""
    from zig_ai_amd.config import register_architecture
    from zig_ai_amd.engine import DecoderModel, ModelRunner, StepEntry
    from zig_ai_amd.parts import lookup, register_position
    routed_classes()
    looking = lookup("position", "toy_added_waves")
    assert not looking.graph_safe

    class RecordableWaves(looking):
        """The same arithmetic; it only uses the positions on the device."""
        kind = "toy_added_waves_recordable"
        graph_safe = True

    register_position(RecordableWaves.kind, RecordableWaves)
    register_architecture("ToyWavedForCausalLM", WavedLfm2Config)
    tokens = eu.random_tokens(60, 97, 5)
    outs = {}
    for kind in ("toy_added_waves", RecordableWaves.kind):
        folder = eu.model_folder(dict(WAVED, position_kind=kind), 21, torch.float32, **eu.sharp_kwargs())
        model = DecoderModel.from_folder(folder, "float32")
        assert model.graph_safe == (kind == RecordableWaves.kind)
        runner = ModelRunner(model, page_size=4, num_pages=20, num_slots=2)
        assert (runner.graphs is not None) == model.graph_safe
        runner.admit("r")
        out = [runner.step([StepEntry("r", tokens[:20], [19])]).cpu()]
        for p in range(20, 60):
            out.append(runner.step([StepEntry("r", tokens[p:p + 1], [0])]).cpu())
            if p % 7 == 0:
                torch.cuda.synchronize()
        outs[kind] = torch.cat(out)
        if runner.graphs is not None:
            assert runner.graphs.captures >= 1 and runner.graphs.replays >= 35
    # the two models have the same tensors (same seed, same names): recorded or not, the
    # same logits
    assert eu.rel_err(outs[RecordableWaves.kind], outs["toy_added_waves"].double()) < 2e-5
    # and they are the model's: the rotary model with these weights gives other logits
    # (the encoding is really applied)
    plain_folder = eu.model_folder({k: v for k, v in dict(WAVED, architectures=["Lfm2ForCausalLM"]).items()},
                                   21, torch.float32, **eu.sharp_kwargs())
    rotary = plain.PlainLfm2(plain_folder).logits(tokens)[19:]
    assert eu.rel_err(outs["toy_added_waves"], rotary) > 1e-2


# ------------------------- another norm, another embedding and another head around LFM2's layers
def capped_classes():
    from zig_ai_amd.kernels import ops
    from zig_ai_amd.parts import (Norm, Part, TensorRule, register_embedding, register_head,
                                  register_norm)

    class CenteredNorm(Norm):
        """``(x - mean) / sqrt(var + eps) * weight + bias`` over the last axis, in 32-bit.  It
        has no fused forms: the base class adds what is pending to the stream and calls
        ``forward``; the parts behind it receive plain activations."""
        kind = "toy_centered_norm"
        graph_safe = True

        @classmethod
        def tensor_rules(cls, params):
            w = int(params["width"])
            return {"weight": TensorRule(((w,),), role="norm"), "bias": TensorRule(((w,),), role="bias")}

        def __init__(self, params, tensors, runtime):
            super().__init__(params, tensors, runtime)
            self.eps = float(params["eps"])
            self.weight, self.bias = tensors["weight"], tensors["bias"]

        def forward(self, x):
            x = x.float()
            x = x - x.mean(dim=-1, keepdim=True)
            y = x * torch.rsqrt((x * x).mean(dim=-1, keepdim=True) + self.eps)
            return (y * self.weight + self.bias).to(self.runtime.dtype)

    class ScaledEmbedding(Part):
        """The table's row times ``sqrt(width)``."""
        kind = "toy_scaled_embedding"
        graph_safe = True
        kernel_sources = ("norm",)

        @classmethod
        def tensor_rules(cls, params):
            return {"weight": TensorRule(((int(params["vocab_size"]), int(params["hidden_size"])),),
                                         role="table")}

        def __init__(self, params, tensors, runtime):
            super().__init__(params, tensors, runtime)
            self.weight = tensors["weight"]
            self.scale = float(params["hidden_size"]) ** 0.5

        def forward(self, token_ids):
            return ops.embed_gather(token_ids, self.weight) * self.scale

    class CappedHead(Part):
        """``cap * tanh(logits / cap)``: logits that cannot leave (-cap, cap)."""
        kind = "toy_capped_head"
        graph_safe = True
        kernel_sources = ("gemm",)

        @classmethod
        def tensor_rules(cls, params):
            return {"weight": TensorRule(((int(params["vocab_size"]), int(params["hidden_size"])),),
                                         role="table")}

        def __init__(self, params, tensors, runtime):
            super().__init__(params, tensors, runtime)
            self.weight = tensors["weight"]
            self.cap = float(params["cap"])

        def forward(self, x):
            logits = ops.linear(x, self.weight, out_dtype=torch.float32)
            return torch.tanh(logits / self.cap) * self.cap

    register_norm(CenteredNorm.kind, CenteredNorm)
    register_embedding(ScaledEmbedding.kind, ScaledEmbedding)
    register_head(CappedHead.kind, CappedHead)


class CappedLfm2Config:
    """LFM2's mixers and feed-forwards between a scaled embedding, centered norms with a
    bias everywhere, and a head with capped logits."""

    def __init__(self, data):
        self.data = dict(data)

    @classmethod
    def from_dict(cls, data):
        return cls(data)

    def to_dict(self):
        return dict(self.data)

    def to_spec(self):
        import dataclasses

        from zig_ai_amd.config.lfm2 import Lfm2Config
        from zig_ai_amd.config.spec import LayerSpec, PartSpec
        inner = dict(self.data, architectures=["Lfm2ForCausalLM"], tie_embedding=False)
        cap = inner.pop("logit_cap")
        spec = Lfm2Config.from_dict(inner).to_spec()

        def centered(norm):
            name = norm.tensors["weight"][0]
            return PartSpec("toy_centered_norm", dict(norm.params),
                            {"weight": (name,), "bias": (name[:-len("weight")] + "bias",)})
        layers = []
        for layer in spec.layers:
            parts = dict(layer.parts)
            for name in ("mixer_norm", "feed_forward_norm"):
                parts[name] = centered(parts[name])
            layers.append(LayerSpec(parts, layer.arrangement))
        head = PartSpec("toy_capped_head", dict(spec.lm_head.params, cap=cap), dict(spec.lm_head.tensors))
        return dataclasses.replace(
            spec, architecture=self.data["architectures"][0], layers=tuple(layers),
            embedding=PartSpec("toy_scaled_embedding", dict(spec.embedding.params),
                               dict(spec.embedding.tensors)),
            final_norm=centered(spec.final_norm), lm_head=head)


CAPPED = {"architectures": ["ToyCappedForCausalLM"], "model_type": "lfm2", "hidden_size": 72,
          "num_hidden_layers": 3, "num_attention_heads": 3, "num_key_value_heads": 1, "head_dim": 32,
          "vocab_size": 131, "layer_types": ["conv", "full_attention", "conv"],
          "intermediate_size": 104, "rope_theta": 10000.0, "norm_eps": 1e-5, "conv_L_cache": 4,
          "conv_bias": True, "max_position_embeddings": 512, "logit_cap": 3.0}


def capped_oracle(folder, tokens):
    """The model in float64, written out with the plain implementation's mixers."""
    from safetensors.torch import load_file
    w = {k: v.double() for k, v in load_file(folder + "/model.safetensors").items()}
    spec = CappedLfm2Config(CAPPED).to_spec()
    lfm2 = plain.PlainLfm2.__new__(plain.PlainLfm2)              # its naming of a layer's tensors
    lfm2.w, lfm2.H = w, CAPPED["hidden_size"]
    lfm2.kinds = ["attention" if t == "full_attention" else "conv" for t in CAPPED["layer_types"]]

    def centered(x, part):
        x = x - x.mean(dim=-1, keepdim=True)
        y = x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + CAPPED["norm_eps"])
        return y * w[part.tensors["weight"][0]] + w[part.tensors["bias"][0]]

    x = w[spec.embedding.tensors["weight"][0]][torch.tensor(tokens)] * CAPPED["hidden_size"] ** 0.5
    pos = torch.arange(len(tokens))
    for i, layer in enumerate(spec.layers):
        lw = lfm2.layer_weights(i)
        n1 = centered(x, layer.mixer_norm)
        if lfm2.kinds[i] == "attention":
            m = plain.attention_mixer(n1, lw, pos, CAPPED["num_attention_heads"], CAPPED["num_key_value_heads"],
                                      CAPPED["head_dim"], CAPPED["norm_eps"], CAPPED["rope_theta"])
        else:
            m = plain.short_conv_mixer(n1, lw)
        x = x + m
        ff = layer.feed_forward.tensors
        x = x + plain.swiglu_ffn(centered(x, layer.feed_forward_norm), w[ff["gate.weight"][0]],
                                 w[ff["up.weight"][0]], w[ff["down.weight"][0]])
    logits = centered(x, spec.final_norm) @ w[spec.lm_head.tensors["weight"][0]].T
    return torch.tanh(logits / CAPPED["logit_cap"]) * CAPPED["logit_cap"]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_another_norm_embedding_and_head(dtype):
    """A norm, an embedding and a head defined here, registered from outside, around the
    framework's own mixers and feed-forwards: built from a folder that the random model
    writer made from the same spec (it asks the parts for their tensors, the norm's bias
    among them), stepped whole, in portions and mixed, recorded and replayed."""
    from zig_ai_amd.config import register_architecture
    from zig_ai_amd.engine import DecoderModel, ModelRunner
    capped_classes()
    register_architecture("ToyCappedForCausalLM", CappedLfm2Config)
    store = torch.float32 if dtype == "float32" else torch.bfloat16
    folder = eu.model_folder(CAPPED, 31, store, std=0.2, norm_init="around_one",
                             role_std={"norm": 0.2, "bias": 0.3, "table": 0.1,
                                       "q_proj.weight": 0.08, "k_proj.weight": 0.08})
    model = DecoderModel.from_folder(folder, dtype)
    assert model.graph_safe
    lengths = [33, 7, 20]
    prompts = [eu.random_tokens(n, CAPPED["vocab_size"], 800 + n) for n in lengths]
    expect = [capped_oracle(folder, p) for p in prompts]
    assert max(float(e.abs().max()) for e in expect) > 0.7 * CAPPED["logit_cap"]   # the cap is at work
    tol = 1e-4 if dtype == "float32" else 2.5e-2
    for schedule in (eu.whole(lengths), eu.changing_portions(lengths, 1),
                     eu.mixed(lengths, seed=9, max_live=3, decode_tail=6)):
        runner = ModelRunner(model, page_size=4, num_pages=24, num_slots=3)
        got = eu.run_schedule(runner, prompts, schedule)
        for g, e in zip(got, expect):
            assert eu.rel_err(g, e) < tol
    assert runner.graphs is not None and runner.graphs.replays > 0


# ---------- another arrangement (four norms, two mixers), a mixer that pages ONE vector
def sandwich_classes():
    from zig_ai_amd.kernels import ops
    from zig_ai_amd.parts import (Mixer, PagedNeed, StateNeed, TensorRule, register_arrangement,
                                  register_mixer)

    class LatentMemoryMixer(Mixer):
        """Attention over one small vector per token: c[t] = x[t] Wd^T is all that is kept
        (ONE plane of ``latent`` elements per token, in 32-bit whatever the run's type);
        y[t] = softmax_j<=t(q[t] . c[j] / sqrt(latent)) c[j] Wu^T with q[t] = x[t] Wq^T."""
        kind = "toy_latent_memory"
        kernel_sources = ("gemm",)

        @classmethod
        def tensor_rules(cls, params):
            H, r = int(params["width"]), int(params["latent"])
            return {"down.weight": TensorRule(((r, H),)), "q.weight": TensorRule(((r, H),)),
                    "up.weight": TensorRule(((H, r),))}

        @classmethod
        def cache_need(cls, params):
            return PagedNeed(((1, int(params["latent"])),), dtype=torch.float32)

        def __init__(self, params, tensors, runtime):
            super().__init__(params, tensors, runtime)
            self.latent = int(params["latent"])
            self.down, self.q, self.up = (tensors[k + ".weight"] for k in ("down", "q", "up"))

        def forward(self, x, step, cache):
            (plane,) = cache.planes                       # [pages, 1, page_size, latent]
            assert plane.dtype == torch.float32 and cache.kv is None
            page_size = plane.shape[2]
            c = ops.linear(x, self.down, out_dtype=torch.float32)
            q = ops.linear(x, self.q, out_dtype=torch.float32)
            place = step.slot_mapping[cache.group].long()
            plane[place // page_size, 0, place % page_size] = c
            out = torch.empty((x.shape[0], self.latent), dtype=torch.float32, device=x.device)
            row = 0
            table = step.block_tables[cache.group]
            for s, (n, ctx) in enumerate(zip(step.seq_lens_host, step.ctx_lens_host)):
                total = ctx + n
                pages = table[s, : (total + page_size - 1) // page_size].long()
                memory = plane[pages, 0].reshape(-1, self.latent)[:total]
                scores = q[row:row + n] @ memory.T / self.latent ** 0.5
                seen = torch.arange(total, device=x.device)[None, :] <= \
                    (ctx + torch.arange(n, device=x.device))[:, None]
                weights = torch.softmax(scores.masked_fill(~seen, float("-inf")), dim=-1)
                out[row:row + n] = weights @ memory
                row += n
            return ops.linear(out.to(x.dtype), self.up)

    class FadingGate(Mixer):
        """A factor 1 / (1 + t / 8) for the request's t-th token: the count of tokens seen
        is its state, one 32-bit INTEGER per request."""
        kind = "toy_fading_gate"

        @classmethod
        def cache_need(cls, params):
            return StateNeed((1,), dtype=torch.int32)

        def forward(self, x, step, cache):
            assert cache.state.dtype == torch.int32
            factor = torch.empty((x.shape[0], 1), dtype=torch.float32, device=x.device)
            row = 0
            for n, slot in zip(step.seq_lens_host, step.slots_host):
                seen = int(cache.state[slot, 0])
                t = seen + torch.arange(n, device=x.device, dtype=torch.float32)
                factor[row:row + n, 0] = 1.0 / (1.0 + t / 8.0)
                cache.state[slot, 0] = seen + n
                row += n
            return factor

    class SandwichBlock:
        """Norms before AND after each of mixer and feed-forward, and a second mixer whose
        output scales the first one's:
            h = x + post1(mixer(pre1(x)) * gate(pre1(x)));  y = h + post2(ffn(pre2(h)))"""
        kind = "toy_sandwich"
        slots = {"pre_mixer_norm": "norm", "mixer": "mixer", "gate": "mixer",
                 "post_mixer_norm": "norm", "pre_feed_forward_norm": "norm",
                 "feed_forward": "feed_forward", "post_feed_forward_norm": "norm"}

        def __init__(self, parts):
            self.parts = dict(parts)

        def forward(self, residual, pending, step, cache):
            p = self.parts
            n1 = p["pre_mixer_norm"].add_forward(residual, pending)
            m = p["mixer"].forward(n1, step, cache["mixer"]).float() \
                * p["gate"].forward(n1, step, cache["gate"])
            residual += p["post_mixer_norm"].forward(m).float()
            f = p["feed_forward"].forward(p["pre_feed_forward_norm"].forward(residual), step)
            if f.dim() == 3:
                f = f.sum(dim=0)
            return residual, p["post_feed_forward_norm"].forward(f.float())

    register_mixer(LatentMemoryMixer.kind, LatentMemoryMixer)
    register_mixer(FadingGate.kind, FadingGate)
    register_arrangement(SandwichBlock.kind, SandwichBlock)


class SandwichConfig:
    def __init__(self, data):
        self.data = dict(data)

    @classmethod
    def from_dict(cls, data):
        return cls(data)

    def to_dict(self):
        return dict(self.data)

    def to_spec(self):
        from zig_ai_amd.config.spec import LayerCall, LayerSpec, ModelSpec, PartSpec
        d = self.data
        H, V = d["width"], d["vocab_size"]

        def norm(name):
            return PartSpec("rms_norm", {"width": H, "eps": 1e-5}, {"weight": (name,)})

        layers = []
        for i in range(d["layers"]):
            p = f"layers.{i}."
            layers.append(LayerSpec({
                "pre_mixer_norm": norm(p + "pre1.weight"),
                "mixer": PartSpec("toy_latent_memory", {"width": H, "latent": d["latent"]},
                                  {k + ".weight": (p + k + ".weight",) for k in ("down", "q", "up")}),
                "gate": PartSpec("toy_fading_gate", {}),
                "post_mixer_norm": norm(p + "post1.weight"),
                "pre_feed_forward_norm": norm(p + "pre2.weight"),
                "feed_forward": PartSpec("swiglu", {"hidden_size": H, "intermediate_size": d["ffn"]},
                                         {k + ".weight": (p + "ffn." + k + ".weight",)
                                          for k in ("gate", "up", "down")}),
                "post_feed_forward_norm": norm(p + "post2.weight"),
            }, "toy_sandwich"))
        return ModelSpec("ToySandwichForCausalLM", H, V,
                         PartSpec("token_embedding", {"vocab_size": V, "hidden_size": H},
                                  {"weight": ("embed.weight",)}),
                         tuple(layers), tuple(LayerCall(i, i) for i in range(d["layers"])),
                         norm("norm.weight"),
                         PartSpec("linear_head", {"vocab_size": V, "hidden_size": H, "tied": True}, {}))


SANDWICH = {"architectures": ["ToySandwichForCausalLM"], "width": 56, "vocab_size": 91, "ffn": 80,
            "latent": 24, "layers": 3}


def sandwich_oracle(folder, tokens):
    from safetensors.torch import load_file
    w = {k: v.double() for k, v in load_file(folder + "/model.safetensors").items()}
    d = SANDWICH
    T, r = len(tokens), d["latent"]
    x = w["embed.weight"][torch.tensor(tokens)]
    factor = 1.0 / (1.0 + torch.arange(T, dtype=torch.float64) / 8.0)
    for i in range(d["layers"]):
        p = f"layers.{i}."
        n1 = plain.rms_norm(x, w[p + "pre1.weight"], 1e-5)
        c, q = n1 @ w[p + "down.weight"].T, n1 @ w[p + "q.weight"].T
        scores = (q @ c.T / r ** 0.5).masked_fill(torch.ones(T, T).triu(1).bool(), float("-inf"))
        m = (torch.softmax(scores, dim=-1) @ c) @ w[p + "up.weight"].T * factor[:, None]
        h = x + plain.rms_norm(m, w[p + "post1.weight"], 1e-5)
        f = plain.swiglu_ffn(plain.rms_norm(h, w[p + "pre2.weight"], 1e-5), w[p + "ffn.gate.weight"],
                             w[p + "ffn.up.weight"], w[p + "ffn.down.weight"])
        x = h + plain.rms_norm(f, w[p + "post2.weight"], 1e-5)
    return plain.rms_norm(x, w["norm.weight"], 1e-5) @ w["embed.weight"].T


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_another_arrangement_and_a_mixer_that_pages_one_vector(dtype):
    """A block of another shape (norms before and after both parts: four norms; two
    mixers) and a mixer that keeps ONE vector per token in pages, of a storage type of
    its own, beside a mixer whose state is an integer: all defined here, registered from
    outside, built from a model folder by the framework's loader and random model writer
    (which ask the arrangement for its parts' names), and stepped whole, in portions and
    mixed, with pages used again."""
    from zig_ai_amd.config import register_architecture
    from zig_ai_amd.engine import DecoderModel, ModelRunner
    sandwich_classes()
    register_architecture("ToySandwichForCausalLM", SandwichConfig)
    store = torch.float32 if dtype == "float32" else torch.bfloat16
    folder = eu.model_folder(SANDWICH, 17, store, std=0.2, norm_init="around_one", role_std={"norm": 0.2})
    model = DecoderModel.from_folder(folder, dtype)
    assert not model.graph_safe
    # per layer a paged entry and a state entry, named (cache, part)
    assert len(model.cache_needs) == 6 and (0, "mixer") in model.cache_needs
    lengths = [37, 5, 22, 14]
    prompts = [eu.random_tokens(n, 91, 800 + n) for n in lengths]
    expect = [sandwich_oracle(folder, p) for p in prompts]
    tol = 1e-4 if dtype == "float32" else 4e-2
    for schedule in (eu.whole(lengths), eu.changing_portions(lengths, 4),
                     eu.mixed(lengths, seed=6, max_live=2, decode_tail=6)):
        pages = eu.peak_tokens(lengths, schedule, round_to=4) // 4
        runner = ModelRunner(model, page_size=4, num_pages=pages, num_slots=2)
        group = runner.cache.groups[0]
        assert group.dtype == torch.float32 and group.kv is None
        assert group.elements_per_page() == 4 * 24 and len(group.cache_ids) == 3
        got = eu.run_schedule(runner, prompts, schedule)
        for g, e in zip(got, expect):
            assert eu.rel_err(g, e) < tol
        stats = runner.cache.stats()
        assert stats["requests"] == 0 and stats["slots_high_water"] <= 2
    assert stats["pages_reused"] > 0
