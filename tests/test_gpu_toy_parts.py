"""Generality of the parts: a toy mixer that keeps a state of its own per request, a toy
feed-forward with routing and a toy position encoding, all defined HERE, are registered,
built into models beside the framework's parts, loaded from a folder and stepped (whole,
in portions, mixed with another request) without any change to the framework's files.
Also a layer order that names a layer twice and lets an execution read another one's cache."""
import json
import os

import pytest
import torch

import plain_model as pm
import replay_util as ru
import tiny

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


# ---- the toy mixer: a leaky running sum over the request's tokens -----------------------------
#   s_t = decay * s_{t-1} + W_in x_t ;  y_t = W_out s_t          (s carried across steps in a state slot)
def define_toy():
    from inferx_amd.config import ModelSpec, PartSpec, ScheduleEntry, register_architecture
    from inferx_amd.config.spec import LayerSpec
    from inferx_amd.parts import Mixer, ParamSpec, StateNeed, register_part

    class RunningSumMixer(Mixer):
        def __init__(self, hidden_size, state_size, decay):
            self.hidden_size, self.state_size, self.decay = hidden_size, state_size, decay

        def state_need(self):
            return StateNeed((self.state_size,))

        def param_specs(self):
            return [ParamSpec("in.weight", (self.state_size, self.hidden_size), std=0.3),
                    ParamSpec("out.weight", (self.hidden_size, self.state_size), std=0.3)]

        def bind(self, tensors, rt):
            self.w_in, self.w_out = tensors["in.weight"].float(), tensors["out.weight"].float()

        def forward(self, ctx, x, cache):
            batch = ctx.host  # host arrays of the step: which rows belong to which request, and its state slot
            u = x.float() @ self.w_in.T
            s_all = torch.empty_like(u)
            for r in range(batch.num_requests):
                b, e, slot = int(batch.q_start[r]), int(batch.q_start[r + 1]), int(batch.state_slots[r])
                s = cache.state[slot]
                for t in range(b, e):  # tokens of a request in order
                    s = self.decay * s + u[t]
                    s_all[t] = s
                cache.state[slot] = s
            return (s_all @ self.w_out.T).to(x.dtype)

    register_part("mixer", "toy_running_sum", RunningSumMixer)

    class ToyConfig:
        def __init__(self, raw):
            self.raw = raw

        @classmethod
        def from_dict(cls, raw):
            return cls(raw)

        def validate(self):
            pass

        def model_spec(self):
            r = self.raw
            H = r["hidden_size"]
            norm = lambda p: PartSpec("rmsnorm", {"width": H, "eps": r["eps"]}, prefix=p)
            layers = []
            for l, kind in enumerate(r["mixers"]):
                p = f"layers.{l}."
                if kind == "toy":
                    mixer = PartSpec("toy_running_sum", {"hidden_size": H, "state_size": r["state_size"],
                                                         "decay": r["decay"]}, prefix=p + "mix.")
                else:
                    mixer = PartSpec("attention", {"hidden_size": H, "num_heads": 2, "num_kv_heads": 1, "head_dim": 16,
                                                   "qkv_bias": False, "init_std": 0.2,
                                                   "position": PartSpec("rope", {"theta": 1e4, "rotary_dim": 16})},
                                     prefix=p + "attn.")
                ffn = PartSpec("dense_mlp", {"hidden_size": H, "width": r["width"], "init_std": 0.2}, prefix=p + "mlp.")
                layers.append(LayerSpec("prenorm", mixer, ffn, norm(p + "norm1."), norm(p + "norm2.")))
            return ModelSpec("ToyStateForCausalLM", H, r["vocab_size"], 0, layers,
                             [ScheduleEntry(l) for l in range(len(layers))], "embed.weight", norm("final_norm."),
                             None, init_std=0.5)

    register_architecture("ToyStateForCausalLM", ToyConfig)
    return ToyConfig


TOY = {"architectures": ["ToyStateForCausalLM"], "hidden_size": 24, "state_size": 10, "decay": 0.8, "eps": 1e-5,
       "width": 40, "vocab_size": 50, "mixers": ["toy", "attention", "toy"]}


def toy_reference(w, tokens):
    """The toy model, whole sequence, float64."""
    w = {k: v.double() for k, v in w.items()}
    T = len(tokens)
    h = w["embed.weight"][torch.tensor(tokens)]
    pos = torch.arange(T)
    for l, kind in enumerate(TOY["mixers"]):
        p = f"layers.{l}."
        x = pm.rms_norm(h, w[p + "norm1.weight"], TOY["eps"])
        if kind == "toy":
            u = x @ w[p + "mix.in.weight"].T
            s, rows = torch.zeros(TOY["state_size"], dtype=torch.float64), []
            for t in range(T):
                s = TOY["decay"] * s + u[t]
                rows.append(s)
            a = torch.stack(rows) @ w[p + "mix.out.weight"].T
        else:
            q = pm.apply_rope((x @ w[p + "attn.q_proj.weight"].T).view(T, 2, 16), pos, 1e4)
            k = pm.apply_rope((x @ w[p + "attn.k_proj.weight"].T).view(T, 1, 16), pos, 1e4)
            v = (x @ w[p + "attn.v_proj.weight"].T).view(T, 1, 16)
            a = pm.attention(q, k, v, pos, 0.25).reshape(T, 32) @ w[p + "attn.o_proj.weight"].T
        h = h + a
        x = pm.rms_norm(h, w[p + "norm2.weight"], TOY["eps"])
        h = h + pm.gated_mlp(x, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    return pm.rms_norm(h, w["final_norm.weight"], TOY["eps"]) @ w["embed.weight"].T


@pytest.mark.parametrize("dtype,tol", [("float32", ru.FP32_TOL), ("bfloat16", ru.BF16_TOL)])
def test_a_mixer_with_state_of_its_own(tmp_path, dtype, tol):
    ToyConfig = define_toy()
    from inferx_amd.engine.runner import ModelRunner
    from inferx_amd.parts import build_model
    from inferx_amd.weights import random_tensors, write_safetensors
    model = build_model(ToyConfig(TOY).model_spec())
    assert [type(b.mixer).__name__ for b in model.blocks] == ["RunningSumMixer", "PagedAttention", "RunningSumMixer"]
    weights = random_tensors(model, 3, dtype)
    write_safetensors(os.path.join(str(tmp_path), "model.safetensors"), weights)
    with open(os.path.join(str(tmp_path), "config.json"), "w") as f:
        json.dump(TOY, f)
    prompts = {"a": tiny.random_tokens(45, 50, 1), "b": tiny.random_tokens(20, 50, 2), "c": tiny.random_tokens(33, 50, 3)}
    expected = {rid: toy_reference(weights, toks) for rid, toks in prompts.items()}
    for name, steps in [("whole", ru.whole(prompts)), ("tail", ru.tail_decoded(prompts, 8)),
                        ("chunked", ru.chunked(prompts)), ("mixed", ru.mixed(prompts, seed=2, max_live=2))]:
        runner = ModelRunner.from_directory(str(tmp_path), dtype=dtype, page_size=16, num_pages=8, max_requests=2,
                                            max_seq_len=128)
        assert not runner.use_graphs  # the toy mixer plans on the host: it does not claim to be graph-safe
        assert sum(b.state is not None for b in runner.bindings) == 2 and len(runner.kv) == 1
        got = ru.replay(runner, steps)
        ru.compare(got, expected, tol, f"toy {name} {dtype}")


@pytest.mark.parametrize("dtype,tol", [("float32", ru.FP32_TOL), ("bfloat16", ru.BF16_TOL)])
def test_layer_order_is_data(tmp_path, dtype, tol):
    """Layer 1 runs twice (shared weights, caches of its own) and the last execution reads the cache of the first."""
    from inferx_amd.config import ScheduleEntry, config_from_dict
    from inferx_amd.engine.runner import ModelRunner
    from inferx_amd.engine.runtime import Runtime
    from inferx_amd.parts import build_model
    from inferx_amd.weights import load_weights
    import dataclasses
    tiny.make_folder(tiny.CONFIG_A, 21, str(tmp_path), dtype)
    cfg, weights = tiny.read_folder(str(tmp_path))
    schedule = [(0, None), (1, None), (1, None), (0, 0)]

    class Reordered:  # the same configuration with another order of execution
        def __init__(self, inner):
            self.inner = inner

        def model_spec(self):
            spec = self.inner.model_spec()
            return dataclasses.replace(spec, schedule=[ScheduleEntry(l, c) for l, c in schedule])

    config = Reordered(config_from_dict(tiny.CONFIG_A))
    rt = Runtime(dtype)
    model = build_model(config.model_spec())
    runner = ModelRunner(config, load_weights(model, str(tmp_path), rt), rt, page_size=16, num_pages=16,
                         max_requests=2, max_seq_len=128, model=model)
    assert runner.kv[0].shape[0] == 3  # three executions own a cache; the fourth reads the first one's
    prompts = {"a": tiny.random_tokens(40, 256, 7), "b": tiny.random_tokens(9, 256, 8)}
    expected = {rid: pm.forward(cfg, weights, toks, schedule=schedule) for rid, toks in prompts.items()}
    for steps in (ru.whole(prompts), ru.chunked(prompts), ru.tail_decoded(prompts, 12)):
        ru.compare(ru.replay(runner, steps), expected, tol, f"schedule {dtype}")


# ---- a toy position encoding and a toy feed-forward with routing, defined HERE -----------------
#   position: rotation by angle (position / stretch) * theta^(-2j/d)   (positions stretched, another base)
#   feed-forward: every token goes to ONE of a few small experts, the one whose router score is largest:
#                 y_t = W2[e_t] relu(W1[e_t] x_t),  e_t = argmax_e (Wr x_t)_e
def define_toy_routed():
    from inferx_amd.config import ModelSpec, PartSpec, ScheduleEntry, register_architecture
    from inferx_amd.config.spec import LayerSpec
    from inferx_amd.parts import FeedForward, LazyNorm, ParamSpec, PositionEncoding, register_part, resolve_input

    class StretchedRotary(PositionEncoding):
        def __init__(self, theta, rotary_dim, stretch):
            self.theta, self.rotary_dim, self.stretch = float(theta), int(rotary_dim), float(stretch)

        def bind(self, tensors, rt):
            j = torch.arange(self.rotary_dim // 2, dtype=torch.float64)
            self.inv_freq = torch.pow(torch.tensor(self.theta, dtype=torch.float64), -2.0 * j / self.rotary_dim).to(rt.device)

        def prepare(self, ctx):
            key = ("toy_stretched", self.theta, self.rotary_dim, self.stretch)
            if key not in ctx.memo:
                angle = ctx.positions.double()[:, None] / self.stretch * self.inv_freq[None, :]
                ctx.memo[key] = torch.stack([torch.cos(angle), torch.sin(angle)], dim=-1).float().contiguous()
            return ctx.memo[key]

    class SwitchFeedForward(FeedForward):
        def __init__(self, hidden_size, width, num_experts):
            self.hidden_size, self.width, self.num_experts = hidden_size, width, num_experts

        def param_specs(self):
            E, H, W = self.num_experts, self.hidden_size, self.width
            return [ParamSpec("router.weight", (E, H), std=1.0), ParamSpec("w1", (E, W, H), std=0.3),
                    ParamSpec("w2", (E, H, W), std=0.3)]

        def bind(self, tensors, rt):
            self.wr, self.w1, self.w2 = (tensors[n].float() for n in ("router.weight", "w1", "w2"))

        takes_lazy_norm = True  # the block hands the norm before this part over unapplied; it is applied here

        def forward(self, ctx, x):
            assert isinstance(x, LazyNorm)
            x = resolve_input(ctx, x)
            xf = x.float()
            e = torch.argmax(xf @ self.wr.T, dim=-1)
            hidden = torch.relu(torch.einsum("twh,th->tw", self.w1[e], xf))
            return torch.einsum("thw,tw->th", self.w2[e], hidden).to(x.dtype)

    register_part("position", "toy_stretched_rope", StretchedRotary)
    register_part("feed_forward", "toy_switch", SwitchFeedForward)

    class ToyRoutedConfig:
        def __init__(self, raw):
            self.raw = raw

        @classmethod
        def from_dict(cls, raw):
            return cls(raw)

        def validate(self):
            pass

        def model_spec(self):
            r = self.raw
            H = r["hidden_size"]
            norm = lambda p: PartSpec("rmsnorm", {"width": H, "eps": r["eps"]}, prefix=p)
            layers = []
            for l in range(r["layers"]):
                p = f"layers.{l}."
                position = PartSpec("toy_stretched_rope", {"theta": r["theta"], "rotary_dim": 16, "stretch": r["stretch"]})
                mixer = PartSpec("attention", {"hidden_size": H, "num_heads": 3, "num_kv_heads": 3, "head_dim": 16,
                                               "qkv_bias": False, "init_std": 0.2, "position": position},
                                 prefix=p + "attn.")
                ffn = PartSpec("toy_switch", {"hidden_size": H, "width": r["width"], "num_experts": r["experts"]},
                               prefix=p + "ffn.")
                layers.append(LayerSpec("prenorm", mixer, ffn, norm(p + "norm1."), norm(p + "norm2.")))
            return ModelSpec("ToyRoutedForCausalLM", H, r["vocab_size"], 0, layers,
                             [ScheduleEntry(l) for l in range(len(layers))], "embed.weight", norm("final_norm."),
                             None, init_std=0.5)

    register_architecture("ToyRoutedForCausalLM", ToyRoutedConfig)
    return ToyRoutedConfig


ROUTED = {"architectures": ["ToyRoutedForCausalLM"], "hidden_size": 40, "eps": 1e-5, "width": 24, "experts": 3,
          "layers": 2, "vocab_size": 60, "theta": 500.0, "stretch": 2.5}


def toy_routed_reference(w, tokens):
    """The toy model, whole sequence, float64.  Also the margin of every routing decision (best score minus
    second best, relative to the largest score), the smallest over the layers."""
    w = {k: v.double() for k, v in w.items()}
    T = len(tokens)
    h = w["embed.weight"][torch.tensor(tokens)]
    pos = torch.arange(T, dtype=torch.float64)
    j = torch.arange(8, dtype=torch.float64)
    angle = pos[:, None] / ROUTED["stretch"] * torch.pow(torch.tensor(ROUTED["theta"], dtype=torch.float64), -2.0 * j / 16)[None, :]
    c, s = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
    rotate = lambda x: torch.cat([x[..., :8] * c - x[..., 8:] * s, x[..., 8:] * c + x[..., :8] * s], dim=-1)
    margins = torch.full((T,), float("inf"), dtype=torch.float64)
    for l in range(ROUTED["layers"]):
        p = f"layers.{l}."
        x = pm.rms_norm(h, w[p + "norm1.weight"], ROUTED["eps"])
        q = rotate((x @ w[p + "attn.q_proj.weight"].T).view(T, 3, 16))
        k = rotate((x @ w[p + "attn.k_proj.weight"].T).view(T, 3, 16))
        v = (x @ w[p + "attn.v_proj.weight"].T).view(T, 3, 16)
        h = h + pm.attention(q, k, v, torch.arange(T), 0.25).reshape(T, 48) @ w[p + "attn.o_proj.weight"].T
        x = pm.rms_norm(h, w[p + "norm2.weight"], ROUTED["eps"])
        scores = x @ w[p + "ffn.router.weight"].T
        top = torch.topk(scores, 2, dim=-1).values
        margins = torch.minimum(margins, (top[:, 0] - top[:, 1]) / scores.abs().max(dim=-1).values)
        e = torch.argmax(scores, dim=-1)
        hidden = torch.relu(torch.einsum("twh,th->tw", w[p + "ffn.w1"][e], x))
        h = h + torch.einsum("thw,tw->th", w[p + "ffn.w2"][e], hidden)
    return pm.rms_norm(h, w["final_norm.weight"], ROUTED["eps"]) @ w["embed.weight"].T, margins


@pytest.mark.parametrize("dtype,tol", [("float32", ru.FP32_TOL), ("bfloat16", ru.BF16_TOL)])
def test_a_routed_feed_forward_and_another_position_encoding(tmp_path, dtype, tol):
    """Both toy parts are registered, built beside the framework's attention, loaded from a folder and stepped
    four ways, without a change to the framework's files."""
    ToyRoutedConfig = define_toy_routed()
    from inferx_amd.engine.runner import ModelRunner
    from inferx_amd.parts import build_model
    from inferx_amd.weights import random_tensors, write_safetensors
    model = build_model(ToyRoutedConfig(ROUTED).model_spec())
    assert [type(b.feed_forward).__name__ for b in model.blocks] == ["SwitchFeedForward"] * 2
    assert type(model.blocks[0].mixer.position).__name__ == "StretchedRotary"
    prompts = {"a": tiny.random_tokens(40, 60, 1), "b": tiny.random_tokens(12, 60, 2), "c": tiny.random_tokens(25, 60, 3)}
    # weights whose routing decisions are all clear in the plain implementation (a near tie would legitimately
    # fall the other way in bfloat16): the first seed that gives such weights
    for seed in range(5, 200):
        weights = random_tensors(model, seed, dtype)
        expected, clear = {}, True
        for rid, toks in prompts.items():
            expected[rid], margins = toy_routed_reference(weights, toks)
            clear = clear and float(margins.min()) >= 2 * ru.NEAR_TIE
        if clear:
            break
    assert clear, "no seed gave clear routing decisions"
    write_safetensors(os.path.join(str(tmp_path), "model.safetensors"), weights)
    with open(os.path.join(str(tmp_path), "config.json"), "w") as f:
        json.dump(ROUTED, f)
    for name, steps in [("whole", ru.whole(prompts)), ("tail", ru.tail_decoded(prompts, 8)),
                        ("chunked", ru.chunked(prompts)), ("mixed", ru.mixed(prompts, seed=4, max_live=2))]:
        runner = ModelRunner.from_directory(str(tmp_path), dtype=dtype, page_size=16, num_pages=10, max_requests=2,
                                            max_seq_len=128)
        assert not runner.use_graphs  # the toy parts do not claim to be graph-safe
        got = ru.replay(runner, steps)
        ru.compare(got, expected, tol, f"toy routed {name} {dtype}")
