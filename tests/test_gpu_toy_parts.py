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
    from inferx_amd.config import (LayerSpec, ModelSpec, PartSpec, ScheduleEntry, linear_head, register_architecture,
                                   token_embedding)
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

        # A step of one token per request only launches work on the device (its state slots come from the step's
        # device arrays), so the part may be captured into a graph; other steps walk their requests on the host,
        # which no captured step ever does.
        graph_safe = True

        def forward(self, ctx, x, cache):
            u = x.float() @ self.w_in.T
            if ctx.one_token_each:
                slots = ctx.state_slots.long()
                s_all = self.decay * cache.state.index_select(0, slots) + u
                cache.state.index_copy_(0, slots, s_all)
                return (s_all @ self.w_out.T).to(x.dtype)
            batch = ctx.host  # host arrays of the step: which rows belong to which request, and its state slot
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
                layers.append(LayerSpec("prenorm", {"mixer": mixer, "feed_forward": ffn, "mixer_norm": norm(p + "norm1."),
                                                    "feed_forward_norm": norm(p + "norm2.")}))
            V = r["vocab_size"]
            return ModelSpec("ToyStateForCausalLM", H, V, 0, layers, [ScheduleEntry(l) for l in range(len(layers))],
                             token_embedding("embed.weight", V, H, 0.5), norm("final_norm."),
                             linear_head("embed.weight", V, H, 0.5), init_std=0.5)

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
        assert runner.use_graphs  # a model with a stateful part of its own still replays its decoding steps
        assert sum(b.state is not None for bound in runner.bindings for b in bound.values()) == 2
        assert len(runner.pages) == 1 and runner.group_owners == [[(1, "mixer")]]
        got = ru.replay(runner, steps)
        ru.compare(got, expected, tol, f"toy {name} {dtype}")
        if name != "mixed":  # (a mixed trace may or may not hold a step of one token each)
            assert bool(runner._graphs) == (name == "tail"), f"{name}: graphs {list(runner._graphs)}"


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
    # three executions own a cache; the fourth reads the first one's
    assert runner.group_owners == [[(0, "mixer"), (1, "mixer"), (2, "mixer")]] and runner.pages[0]["k"].shape[0] == 3
    assert runner.bindings[3]["mixer"].k.data_ptr() == runner.bindings[0]["mixer"].k.data_ptr()
    assert not runner.bindings[3]["mixer"].writes
    prompts = {"a": tiny.random_tokens(40, 256, 7), "b": tiny.random_tokens(9, 256, 8)}
    expected = {rid: pm.forward(cfg, weights, toks, schedule=schedule) for rid, toks in prompts.items()}
    for steps in (ru.whole(prompts), ru.chunked(prompts), ru.tail_decoded(prompts, 12)):
        ru.compare(ru.replay(runner, steps), expected, tol, f"schedule {dtype}")


# ---- a toy position encoding and a toy feed-forward with routing, defined HERE -----------------
#   position: rotation by angle (position / stretch) * theta^(-2j/d)   (positions stretched, another base), of the
#             whole head or of `rotary_dim` of its elements from `begin` on
#   feed-forward: every token goes to ONE of a few small experts, the one whose router score is largest:
#                 y_t = W2[e_t] relu(W1[e_t] x_t),  e_t = argmax_e (Wr x_t)_e
def define_toy_routed():
    from inferx_amd.config import (LayerSpec, ModelSpec, PartSpec, ScheduleEntry, linear_head, register_architecture,
                                   token_embedding)
    from inferx_amd.parts import FeedForward, LazyNorm, ParamSpec, PositionEncoding, register_part, resolve_input

    class StretchedRotary(PositionEncoding):
        def __init__(self, theta, rotary_dim, stretch, begin=0):
            self.theta, self.rotary_dim, self.stretch = float(theta), int(rotary_dim), float(stretch)
            self.begin = int(begin)  # the mixer asks for `rotary_dim` and `begin`: the part of a head that is rotated

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
                position = PartSpec("toy_stretched_rope", {"theta": r["theta"], "rotary_dim": r.get("rotary_dim", 16),
                                                           "stretch": r["stretch"], "begin": r.get("begin", 0)})
                mixer = PartSpec("attention", {"hidden_size": H, "num_heads": 3, "num_kv_heads": 3, "head_dim": 16,
                                               "qkv_bias": False, "init_std": 0.2, "position": position},
                                 prefix=p + "attn.")
                ffn = PartSpec("toy_switch", {"hidden_size": H, "width": r["width"], "num_experts": r["experts"]},
                               prefix=p + "ffn.")
                layers.append(LayerSpec("prenorm", {"mixer": mixer, "feed_forward": ffn, "mixer_norm": norm(p + "norm1."),
                                                    "feed_forward_norm": norm(p + "norm2.")}))
            V = r["vocab_size"]
            return ModelSpec("ToyRoutedForCausalLM", H, V, 0, layers, [ScheduleEntry(l) for l in range(len(layers))],
                             token_embedding("embed.weight", V, H, 0.5), norm("final_norm."),
                             linear_head("embed.weight", V, H, 0.5), init_std=0.5)

    register_architecture("ToyRoutedForCausalLM", ToyRoutedConfig)
    return ToyRoutedConfig


ROUTED = {"architectures": ["ToyRoutedForCausalLM"], "hidden_size": 40, "eps": 1e-5, "width": 24, "experts": 3,
          "layers": 2, "vocab_size": 60, "theta": 500.0, "stretch": 2.5}
# the same with only elements 6 to 12 of every head of 16 rotated
ROUTED_PART = dict(ROUTED, rotary_dim=6, begin=6, theta=90.0, stretch=1.5)


def toy_routed_reference(w, tokens, ROUTED=ROUTED):
    """The toy model, whole sequence, float64.  Also the margin of every routing decision (best score minus
    second best, relative to the largest score), the smallest over the layers."""
    w = {k: v.double() for k, v in w.items()}
    T = len(tokens)
    h = w["embed.weight"][torch.tensor(tokens)]
    pos = torch.arange(T, dtype=torch.float64)
    begin, dim = ROUTED.get("begin", 0), ROUTED.get("rotary_dim", 16)
    j = torch.arange(dim // 2, dtype=torch.float64)
    angle = pos[:, None] / ROUTED["stretch"] * torch.pow(torch.tensor(ROUTED["theta"], dtype=torch.float64), -2.0 * j / dim)[None, :]
    c, s = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]

    def rotate(x):
        lo, hi = x[..., begin:begin + dim // 2], x[..., begin + dim // 2:begin + dim]
        return torch.cat([x[..., :begin], lo * c - hi * s, hi * c + lo * s, x[..., begin + dim:]], dim=-1)
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


@pytest.mark.parametrize("ROUTED", [ROUTED, ROUTED_PART], ids=["whole_heads_rotated", "a_part_of_each_head_rotated"])
@pytest.mark.parametrize("dtype,tol", [("float32", ru.FP32_TOL), ("bfloat16", ru.BF16_TOL)])
def test_a_routed_feed_forward_and_another_position_encoding(tmp_path, dtype, tol, ROUTED):
    """Both toy parts are registered, built beside the framework's attention, loaded from a folder and stepped
    four ways, without a change to the framework's files; the position encoding also where it rotates only a part
    of each head, which the framework's attention takes from its `rotary_dim` and `begin`."""
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
            expected[rid], margins = toy_routed_reference(weights, toks, ROUTED)
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


# ---- other arrangements, another kind of cache, other ends of the model: all defined HERE ----------------------
#   sandwich block: four norms     h += post1(mixer(pre1(h)));  h += post2(ffn(pre2(h)))
#   parallel block: one norm       x = norm(h);  h += mixer(x) + ffn(x)
#   latent mixer: keeps ONE array of `rank` numbers per token (c_t = Wc x_t) instead of keys and values, and reads
#       it back through the block table:  y_t = Wo sum_{j<=t} softmax_j(q_t . c_j / sqrt(rank)) c_j,  q_t = Wq x_t
#   embedding: table[id] * scale + learned_position[position];  head: cap * tanh((x . W^T + bias) / cap)
def define_toy_shapes():
    from inferx_amd.config import LayerSpec, ModelSpec, PartSpec, ScheduleEntry, register_architecture
    from inferx_amd.parts import (Block, CacheArray, CacheNeed, Embedding, Head, Mixer, ParamSpec, register_part,
                                  resolve_delta)

    class SandwichBlock(Block):
        part_kinds = {"mixer": "mixer", "feed_forward": "feed_forward", "pre_mixer": "norm", "post_mixer": "norm",
                      "pre_ffn": "norm", "post_ffn": "norm"}

        def forward(self, ctx, h, pending, caches):
            zero = lambda: torch.zeros_like(h)
            x = self.pre_mixer.forward(ctx, h, pending)
            a = resolve_delta(ctx, self.mixer.forward(ctx, x, caches.get("mixer")))
            a = self.post_mixer.forward(ctx, a.float().contiguous(), None)     # a norm of the delta, not of h
            x = self.pre_ffn.forward(ctx, h, a)
            f = resolve_delta(ctx, self.feed_forward.forward(ctx, x))
            return self.post_ffn.forward(ctx, f.float().contiguous(), None)

    class ParallelBlock(Block):
        part_kinds = {"mixer": "mixer", "feed_forward": "feed_forward", "norm": "norm"}

        def forward(self, ctx, h, pending, caches):
            x = self.norm.forward(ctx, h, pending)
            a = resolve_delta(ctx, self.mixer.forward(ctx, x, caches.get("mixer")))
            f = resolve_delta(ctx, self.feed_forward.forward(ctx, x))
            return a + f

    class LatentMixer(Mixer):
        def __init__(self, hidden_size, rank):
            self.hidden_size, self.rank = hidden_size, rank

        def cache_need(self):
            return CacheNeed((CacheArray("latent", 1, self.rank, dtype="float32"),))

        def param_specs(self):
            H, r = self.hidden_size, self.rank
            return [ParamSpec("c.weight", (r, H), std=0.15), ParamSpec("q.weight", (r, H), std=0.15),
                    ParamSpec("o.weight", (H, r), std=0.4)]

        def bind(self, tensors, rt):
            self.wc, self.wq, self.wo = (tensors[n].float() for n in ("c.weight", "q.weight", "o.weight"))

        def forward(self, ctx, x, cache):
            pages = cache.arrays["latent"]                     # [pages, 1, page_size, rank], as the need says
            page_size = pages.shape[2]
            flat = pages.view(-1, self.rank)                   # slot = page * page_size + offset
            xf = x.float()
            flat.index_copy_(0, ctx.slots[cache.group].long(), xf @ self.wc.T)
            q = xf @ self.wq.T
            batch, table = ctx.host, ctx.block_tables[cache.group]
            out = torch.empty_like(q)
            for t in range(batch.num_tokens):
                s, p = int(batch.seq_of_token[t]), int(batch.positions[t])
                keys = torch.arange(p + 1, device=x.device)
                slots = table[s, keys // page_size].long() * page_size + keys % page_size
                c = flat[slots]
                out[t] = torch.softmax(c @ q[t] / self.rank ** 0.5, 0) @ c
            return (out @ self.wo.T).to(x.dtype)

    class ScaledPositionalEmbedding(Embedding):
        def __init__(self, vocab_size, hidden_size, max_positions, scale):
            self.vocab_size, self.hidden_size, self.max_positions, self.scale = vocab_size, hidden_size, max_positions, scale

        def param_specs(self):
            return [ParamSpec("tokens.weight", (self.vocab_size, self.hidden_size), std=0.5),
                    ParamSpec("positions.weight", (self.max_positions, self.hidden_size), std=0.5)]

        def bind(self, tensors, rt):
            self.tokens, self.positions = tensors["tokens.weight"].float(), tensors["positions.weight"].float()

        def forward(self, ctx):
            return (self.tokens[ctx.token_ids.long()] * self.scale + self.positions[ctx.positions.long()]).contiguous()

    class CappedHead(Head):
        def __init__(self, vocab_size, hidden_size, cap):
            self.vocab_size, self.hidden_size, self.cap = vocab_size, hidden_size, cap

        def param_specs(self):
            return [ParamSpec("weight", (self.vocab_size, self.hidden_size), std=0.5),
                    ParamSpec("bias", (self.vocab_size,), std=0.5)]

        def bind(self, tensors, rt):
            self.weight, self.bias = tensors["weight"].float(), tensors["bias"].float()

        def forward(self, ctx, x):
            return self.cap * torch.tanh((x.float() @ self.weight.T + self.bias) / self.cap)

    register_part("block", "toy_sandwich", SandwichBlock)
    register_part("block", "toy_parallel", ParallelBlock)
    register_part("mixer", "toy_latent", LatentMixer)
    register_part("embedding", "toy_scaled_positional", ScaledPositionalEmbedding)
    register_part("head", "toy_capped", CappedHead)

    class ToyShapesConfig:
        def __init__(self, raw):
            self.raw = raw

        @classmethod
        def from_dict(cls, raw):
            return cls(raw)

        def validate(self):
            pass

        def model_spec(self):
            r = self.raw
            H, V = r["hidden_size"], r["vocab_size"]
            norm = lambda p: PartSpec("rmsnorm", {"width": H, "eps": r["eps"]}, prefix=p)
            layers = []
            for l, (block, mixer_kind) in enumerate(r["layers"]):
                p = f"layers.{l}."
                if mixer_kind == "latent":
                    mixer = PartSpec("toy_latent", {"hidden_size": H, "rank": r["rank"]}, prefix=p + "latent.")
                else:
                    mixer = PartSpec("attention", {"hidden_size": H, "num_heads": 2, "num_kv_heads": 2, "head_dim": 16,
                                                   "qkv_bias": True, "init_std": 0.2,
                                                   "position": PartSpec("rope", {"theta": 1e4, "rotary_dim": 16})},
                                     prefix=p + "attn.")
                ffn = PartSpec("dense_mlp", {"hidden_size": H, "width": r["width"], "init_std": 0.2}, prefix=p + "mlp.")
                parts = {"mixer": mixer, "feed_forward": ffn}
                if block == "toy_sandwich":
                    parts.update({n: norm(p + n + ".") for n in ("pre_mixer", "post_mixer", "pre_ffn", "post_ffn")})
                else:
                    parts["norm"] = norm(p + "norm.")
                layers.append(LayerSpec(block, parts))
            embedding = PartSpec("toy_scaled_positional", {"vocab_size": V, "hidden_size": H,
                                                           "max_positions": r["max_positions"], "scale": r["scale"]},
                                 prefix="embed.")
            head = PartSpec("toy_capped", {"vocab_size": V, "hidden_size": H, "cap": r["cap"]}, prefix="head.")
            return ModelSpec("ToyShapesForCausalLM", H, V, r["max_positions"], layers,
                             [ScheduleEntry(l) for l in range(len(layers))], embedding, norm("final_norm."), head)

    register_architecture("ToyShapesForCausalLM", ToyShapesConfig)
    return ToyShapesConfig


SHAPES = {"architectures": ["ToyShapesForCausalLM"], "hidden_size": 32, "eps": 1e-5, "width": 48, "rank": 12,
          "vocab_size": 70, "max_positions": 96, "scale": 3.0, "cap": 30.0,
          "layers": [["toy_sandwich", "latent"], ["toy_parallel", "attention"], ["toy_sandwich", "attention"],
                     ["toy_parallel", "latent"]]}


def toy_shapes_reference(w, tokens):
    """The toy model, whole sequence, float64."""
    w = {k: v.double() for k, v in w.items()}
    r, T = SHAPES, len(tokens)
    eps = r["eps"]
    pos = torch.arange(T)
    h = w["embed.tokens.weight"][torch.tensor(tokens)] * r["scale"] + w["embed.positions.weight"][pos]
    for l, (block, mixer_kind) in enumerate(r["layers"]):
        p = f"layers.{l}."

        def mixer(x):
            if mixer_kind == "latent":
                c, q = x @ w[p + "latent.c.weight"].T, x @ w[p + "latent.q.weight"].T
                rows = [torch.softmax(c[:t + 1] @ q[t] / r["rank"] ** 0.5, 0) @ c[:t + 1] for t in range(T)]
                return torch.stack(rows) @ w[p + "latent.o.weight"].T
            a = p + "attn."
            q = pm.apply_rope((x @ w[a + "q_proj.weight"].T + w[a + "q_proj.bias"]).view(T, 2, 16), pos, 1e4)
            k = pm.apply_rope((x @ w[a + "k_proj.weight"].T + w[a + "k_proj.bias"]).view(T, 2, 16), pos, 1e4)
            v = (x @ w[a + "v_proj.weight"].T + w[a + "v_proj.bias"]).view(T, 2, 16)
            return pm.attention(q, k, v, pos, 0.25).reshape(T, 32) @ w[a + "o_proj.weight"].T

        ffn = lambda x: pm.gated_mlp(x, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"],
                                     w[p + "mlp.down_proj.weight"])
        n = lambda name, x: pm.rms_norm(x, w[p + name + ".weight"], eps)
        if block == "toy_sandwich":
            h = h + n("post_mixer", mixer(n("pre_mixer", h)))
            h = h + n("post_ffn", ffn(n("pre_ffn", h)))
        else:
            x = n("norm", h)
            h = h + mixer(x) + ffn(x)
    logits = pm.rms_norm(h, w["final_norm.weight"], eps) @ w["head.weight"].T + w["head.bias"]
    return r["cap"] * torch.tanh(logits / r["cap"])


@pytest.mark.parametrize("dtype,tol", [("float32", ru.FP32_TOL), ("bfloat16", ru.BF16_TOL)])
def test_other_arrangements_caches_and_ends(tmp_path, dtype, tol):
    """Blocks with four norms and with one, a mixer whose cache is one array per token (beside attention's two, in a
    page group of its own), an embedding with a scale and learned positions and a head with a bias and a cap: all
    registered from here, built, loaded from a folder and stepped four ways without a change to the framework."""
    ToyShapesConfig = define_toy_shapes()
    from inferx_amd.engine.runner import ModelRunner
    from inferx_amd.parts import build_model
    from inferx_amd.weights import random_tensors, write_safetensors
    model = build_model(ToyShapesConfig(SHAPES).model_spec())
    assert [type(b).__name__ for b in model.blocks] == ["SandwichBlock", "ParallelBlock"] * 2
    assert sorted(model.blocks[0].parts) == ["feed_forward", "mixer", "post_ffn", "post_mixer", "pre_ffn", "pre_mixer"]
    weights = random_tensors(model, 9, dtype)
    assert "head.bias" in weights and "embed.positions.weight" in weights and "layers.0.post_ffn.weight" in weights
    write_safetensors(os.path.join(str(tmp_path), "model.safetensors"), weights)
    with open(os.path.join(str(tmp_path), "config.json"), "w") as f:
        json.dump(SHAPES, f)
    prompts = {"a": tiny.random_tokens(50, 70, 1), "b": tiny.random_tokens(19, 70, 2), "c": tiny.random_tokens(34, 70, 3)}
    expected = {rid: toy_shapes_reference(weights, toks) for rid, toks in prompts.items()}
    for name, steps in [("whole", ru.whole(prompts)), ("tail", ru.tail_decoded(prompts, 8)),
                        ("chunked", ru.chunked(prompts)), ("mixed", ru.mixed(prompts, seed=6, max_live=2))]:
        runner = ModelRunner.from_directory(str(tmp_path), dtype=dtype, page_size=16, num_pages=9, max_requests=2,
                                            max_seq_len=96)
        # two page groups, laid out from the parts' own descriptions: one float32 array of `rank` per token for the
        # latent mixers, keys and values in the run's type for attention
        assert runner.group_owners == [[(0, "mixer"), (3, "mixer")], [(1, "mixer"), (2, "mixer")]]
        assert {n: tuple(t.shape) for n, t in runner.pages[0].items()} == {"latent": (2, 9, 1, 16, 12)}
        assert runner.pages[0]["latent"].dtype == torch.float32 and runner.pages[1]["v"].shape == (2, 9, 2, 16, 16)
        assert runner.kv_bytes_per_token() == 2 * 12 * 4 + 2 * 2 * 2 * 16 * runner.pages[1]["k"].element_size()
        got = ru.replay(runner, steps)
        ru.compare(got, expected, tol, f"toy shapes {name} {dtype}")


def test_a_block_says_which_parts_it_misses_or_does_not_know():
    define_toy_shapes()
    from inferx_amd.config import PartSpec
    from inferx_amd.parts import build_block
    norm = PartSpec("rmsnorm", {"width": 8, "eps": 1e-5})
    ffn = PartSpec("dense_mlp", {"hidden_size": 8, "width": 8})
    with pytest.raises(KeyError, match=r"missing: \['mixer'\]"):
        build_block("toy_parallel", {"feed_forward": ffn, "norm": norm})
    with pytest.raises(KeyError, match=r"not known to it: \['post_ffn'\]"):
        build_block("prenorm", {"feed_forward": ffn, "mixer_norm": norm, "feed_forward_norm": norm, "post_ffn": norm,
                                "mixer": PartSpec("toy_latent", {"hidden_size": 8, "rank": 4})})
    with pytest.raises(KeyError, match="no block registered"):
        build_block("no_such_block", {})


# ---- a toy mixer that PLANS ON THE HOST for steps of one token per request, and is still replayed from a graph -----
#   the latent mixer above, but in a step of one token per request it reads, for all requests at once, the first
#   ceil(longest / page_size) pages of every block table, `longest` being a number that it takes from the host's
#   batch.  Under a recorded step there is no host batch: the number then comes from the part's own `capture_plan`,
#   which the runner calls for every part without knowing what any of them leaves in the step's memo.
def define_toy_planned():
    from inferx_amd.config import (LayerSpec, ModelSpec, PartSpec, ScheduleEntry, linear_head, register_architecture,
                                   token_embedding)
    from inferx_amd.parts import CacheArray, CacheNeed, Mixer, ParamSpec, register_part

    class PlannedLatentMixer(Mixer):
        graph_safe = True
        steps_without_host = 0   # how often a step ran from the plan alone (the recording and its warm-up)
        plans_seen = []          # the `longest` of every plan that the runner asked for

        def __init__(self, hidden_size, rank):
            self.hidden_size, self.rank = hidden_size, rank

        def cache_need(self):
            return CacheNeed((CacheArray("latent", 1, self.rank, dtype="float32"),))

        def param_specs(self):
            H, r = self.hidden_size, self.rank
            return [ParamSpec("c.weight", (r, H), std=0.15), ParamSpec("q.weight", (r, H), std=0.15),
                    ParamSpec("o.weight", (H, r), std=0.4)]

        def bind(self, tensors, rt):
            self.wc, self.wq, self.wo = (tensors[n].float() for n in ("c.weight", "q.weight", "o.weight"))

        def capture_plan(self, ctx, requests, longest):
            ctx.memo[("toy_planned_longest", self.rank)] = longest
            type(self).plans_seen.append(longest)

        def forward(self, ctx, x, cache):
            pages = cache.arrays["latent"]                     # [pages, 1, page_size, rank]
            page_size = pages.shape[2]
            flat = pages.view(-1, self.rank)
            xf = x.float()
            flat.index_copy_(0, ctx.slots[cache.group].long(), xf @ self.wc.T)
            q = xf @ self.wq.T
            table = ctx.block_tables[cache.group]
            if ctx.one_token_each:
                longest = ctx.memo.get(("toy_planned_longest", self.rank))
                if longest is None:
                    longest = int(ctx.host.seq_lens.max())     # planned on the host, from the step's batch
                if ctx.host is None:
                    type(self).steps_without_host += 1
                n_pages = min(-(-longest // page_size), table.shape[1])
                c = pages[table[:, :n_pages].long().clamp(min=0)].reshape(x.shape[0], n_pages * page_size, self.rank)
                keys = torch.arange(n_pages * page_size, device=x.device)
                scores = torch.einsum("skr,sr->sk", c, q) / self.rank ** 0.5
                scores = scores.masked_fill(keys[None, :] > ctx.positions[:, None], float("-inf"))
                # (pages beyond a request's own hold other requests' numbers or stale ones: weight exactly zero)
                out = torch.einsum("sk,skr->sr", torch.softmax(scores, -1), torch.nan_to_num(c))
                return (out @ self.wo.T).to(x.dtype)
            batch = ctx.host
            out = torch.empty_like(q)
            for t in range(batch.num_tokens):
                s, p = int(batch.seq_of_token[t]), int(batch.positions[t])
                keys = torch.arange(p + 1, device=x.device)
                slots = table[s, keys // page_size].long() * page_size + keys % page_size
                c = flat[slots]
                out[t] = torch.softmax(c @ q[t] / self.rank ** 0.5, 0) @ c
            return (out @ self.wo.T).to(x.dtype)

    register_part("mixer", "toy_planned_latent", PlannedLatentMixer)

    class ToyPlannedConfig:
        def __init__(self, raw):
            self.raw = raw

        @classmethod
        def from_dict(cls, raw):
            return cls(raw)

        def validate(self):
            pass

        def model_spec(self):
            r = self.raw
            H, V = r["hidden_size"], r["vocab_size"]
            norm = lambda p: PartSpec("rmsnorm", {"width": H, "eps": r["eps"]}, prefix=p)
            layers = []
            for l, kind in enumerate(r["mixers"]):
                p = f"layers.{l}."
                if kind == "planned":
                    mixer = PartSpec("toy_planned_latent", {"hidden_size": H, "rank": r["rank"]}, prefix=p + "latent.")
                else:
                    mixer = PartSpec("attention", {"hidden_size": H, "num_heads": 2, "num_kv_heads": 1, "head_dim": 16,
                                                   "qkv_bias": True, "init_std": 0.2,
                                                   "position": PartSpec("rope", {"theta": 1e4, "rotary_dim": 16})},
                                     prefix=p + "attn.")
                ffn = PartSpec("dense_mlp", {"hidden_size": H, "width": r["width"], "init_std": 0.2}, prefix=p + "mlp.")
                layers.append(LayerSpec("prenorm", {"mixer": mixer, "feed_forward": ffn, "mixer_norm": norm(p + "norm1."),
                                                    "feed_forward_norm": norm(p + "norm2.")}))
            return ModelSpec("ToyPlannedForCausalLM", H, V, 0, layers, [ScheduleEntry(l) for l in range(len(layers))],
                             token_embedding("embed.weight", V, H, 0.5), norm("final_norm."),
                             linear_head("embed.weight", V, H, 0.5), init_std=0.5)

    register_architecture("ToyPlannedForCausalLM", ToyPlannedConfig)
    return ToyPlannedConfig, PlannedLatentMixer


PLANNED = {"architectures": ["ToyPlannedForCausalLM"], "hidden_size": 32, "eps": 1e-5, "width": 40, "rank": 12,
           "vocab_size": 64, "mixers": ["planned", "attention", "planned"]}


def toy_planned_reference(w, tokens):
    """The toy model, whole sequence, float64."""
    w = {k: v.double() for k, v in w.items()}
    r, T = PLANNED, len(tokens)
    pos = torch.arange(T)
    h = w["embed.weight"][torch.tensor(tokens)]
    for l, kind in enumerate(r["mixers"]):
        p = f"layers.{l}."
        x = pm.rms_norm(h, w[p + "norm1.weight"], r["eps"])
        if kind == "planned":
            c, q = x @ w[p + "latent.c.weight"].T, x @ w[p + "latent.q.weight"].T
            rows = [torch.softmax(c[:t + 1] @ q[t] / r["rank"] ** 0.5, 0) @ c[:t + 1] for t in range(T)]
            a = torch.stack(rows) @ w[p + "latent.o.weight"].T
        else:
            n = p + "attn."
            q = pm.apply_rope((x @ w[n + "q_proj.weight"].T + w[n + "q_proj.bias"]).view(T, 2, 16), pos, 1e4)
            k = pm.apply_rope((x @ w[n + "k_proj.weight"].T + w[n + "k_proj.bias"]).view(T, 1, 16), pos, 1e4)
            v = (x @ w[n + "v_proj.weight"].T + w[n + "v_proj.bias"]).view(T, 1, 16)
            a = pm.attention(q, k, v, pos, 0.25).reshape(T, 32) @ w[n + "o_proj.weight"].T
        h = h + a
        x = pm.rms_norm(h, w[p + "norm2.weight"], r["eps"])
        h = h + pm.gated_mlp(x, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    return pm.rms_norm(h, w["final_norm.weight"], r["eps"]) @ w["embed.weight"].T


@pytest.mark.parametrize("dtype,tol", [("float32", ru.FP32_TOL), ("bfloat16", ru.BF16_TOL)])
def test_a_mixer_that_plans_on_the_host_is_replayed_from_a_graph(tmp_path, dtype, tol):
    """The runner asks every part for its plan of a one-token-per-request step (`capture_plan`) and knows none of
    them: a mixer defined here, whose plan is a number of its own under a memo key of its own, is recorded and
    replayed beside the framework's attention, with no change to the framework's files."""
    ToyPlannedConfig, Mixer = define_toy_planned()
    from inferx_amd.engine.runner import ModelRunner
    from inferx_amd.parts import build_model
    from inferx_amd.weights import random_tensors, write_safetensors
    model = build_model(ToyPlannedConfig(PLANNED).model_spec())
    weights = random_tensors(model, 11, dtype)
    write_safetensors(os.path.join(str(tmp_path), "model.safetensors"), weights)
    with open(os.path.join(str(tmp_path), "config.json"), "w") as f:
        json.dump(PLANNED, f)
    prompts = {"a": tiny.random_tokens(70, 64, 1), "b": tiny.random_tokens(21, 64, 2), "c": tiny.random_tokens(40, 64, 3)}
    expected = {rid: toy_planned_reference(weights, toks) for rid, toks in prompts.items()}
    for name, steps in [("whole", ru.whole(prompts)), ("tail", ru.tail_decoded(prompts, 24)),
                        ("chunked", ru.chunked(prompts)), ("mixed", ru.mixed(prompts, seed=8, max_live=2))]:
        Mixer.steps_without_host, Mixer.plans_seen = 0, []
        runner = ModelRunner.from_directory(str(tmp_path), dtype=dtype, page_size=16, num_pages=10, max_requests=2,
                                            max_seq_len=128)
        assert runner.use_graphs
        assert len(runner.pages) == 2  # the toy's latent array and attention's keys and values, a group each
        got = ru.replay(runner, steps)
        ru.compare(got, expected, tol, f"toy planned {name} {dtype}")
        if name == "tail":
            # decoding from 46 to 70 tokens, from 1 to 21 and from 16 to 40: graphs of several context buckets were
            # recorded with the toy's plan (the context rounded up to a power of two), and ran without a host batch
            assert len(runner._graphs) >= 3 and Mixer.steps_without_host > 0
            assert set(Mixer.plans_seen) >= {32, 64, 128} and all(p & (p - 1) == 0 for p in Mixer.plans_seen)
        if name == "whole":
            assert not runner._graphs and not Mixer.plans_seen
