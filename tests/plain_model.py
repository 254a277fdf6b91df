"""The plain implementation: Qwen2-MoE written the obvious way, on the CPU, in
float64, whole sequences, no cache, no batching, one function per part.

It shares no code with `inferx_amd`: it reads config.json keys and checkpoint
tensor names itself.  Every function cites the place in the reference
(divedb/InferX, paths relative to its root) whose formula it follows.  The
reference was read, not run.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence, Tuple

import torch

F64 = torch.float64


class Widened:
    """A checkpoint's tensors in float64, each widened when it is first used (of a model with many experts only
    those that some token chose).  `forward` takes plain tensors too; handing it one of these keeps the widened
    tensors from one call to the next."""

    def __init__(self, tensors: Dict[str, torch.Tensor]):
        self._stored, self._wide = tensors, {}

    def __contains__(self, name: str) -> bool:
        return name in self._stored

    def __getitem__(self, name: str) -> torch.Tensor:
        if name not in self._wide:
            self._wide[name] = self._stored[name].to(F64)
        return self._wide[name]


def no_rounding(t: torch.Tensor) -> torch.Tensor:
    return t


def to_bfloat16_and_back(t: torch.Tensor) -> torch.Tensor:
    """Rounds to bfloat16 (nearest even) and widens again: what a tensor stored in bfloat16 holds."""
    return t.to(torch.bfloat16).to(F64)


# --------------------------------------------------------------------------
def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """y_i = x_i * rsqrt(sum(x^2)/H + eps) * w_i
    src/backends/cuda/ops/layers.cu:50-76 (RmsNormKernel: sumsq / hidden + eps, rsqrtf, x*inv*w)."""
    inv = torch.rsqrt((x * x).sum(-1, keepdim=True) / x.shape[-1] + eps)
    return x * inv * weight


def rope_frequencies(theta: float, head_dim: int) -> torch.Tensor:
    """inv_freq[j] = theta^(-2j/d), j < d/2.   layers.cu:93-94 (RopeKernel).
    Rounded to float32 as a device table would hold it."""
    j = torch.arange(head_dim // 2, dtype=F64)
    return (theta ** (-2.0 * j / head_dim)).to(torch.float32).to(F64)


def apply_rope(x: torch.Tensor, positions: torch.Tensor, theta: float) -> torch.Tensor:
    """Half-split rotation: pairs (j, j + d/2);
    x'_j = x_j cos a - x_{j+d/2} sin a;  x'_{j+d/2} = x_{j+d/2} cos a + x_j sin a;  a = pos * inv_freq[j].
    layers.cu:80-115 (RopeKernel: lo*c - hi*s, hi*c + lo*s).   x: [T, heads, d]."""
    d = x.shape[-1]
    half = d // 2
    # the angle is formed in float32 (float(pos) * inv_freq), layers.cu:87, 95
    angle = (positions.to(torch.float32)[:, None] * rope_frequencies(theta, d).to(torch.float32)[None, :]).to(F64)
    c, s = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
    lo, hi = x[..., :half], x[..., half:]
    return torch.cat([lo * c - hi * s, hi * c + lo * s], dim=-1)


def apply_rope_part(x: torch.Tensor, positions: torch.Tensor, theta: float, begin: int, dim: int) -> torch.Tensor:
    """Rotation of elements [begin, begin + dim) of every head, the others unchanged: the rotated part is a vector of
    its own, with the pairing (j, j + dim/2) and the frequencies theta^(-2j/dim) of its own width.
    mla.cu:21-46 (RopeInPlaceKernel: the trailing rope_dim of a head, inv_freq by the sub-vector's width)."""
    out = x.clone()
    out[..., begin:begin + dim] = apply_rope(x[..., begin:begin + dim], positions, theta)
    return out


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, positions: torch.Tensor, scale: float,
              window: int = 0) -> torch.Tensor:
    """Causal grouped-query attention, by position, no mask tensor.
    Query head h reads kv head h // (heads // kv_heads); a query at position p reads keys [start, p],
    start = 0 or, with a window W, max(0, p + 1 - W); s_j = (q . k_j) * scale; softmax with the maximum
    subtracted; o = sum(e_j v_j) / sum(e_j).
    layers.cu:329-407 (PagedAttentionWithLseKernel; window :346-354; contiguous variant :133-191).
    q: [T, heads, d]; k, v: [T, kv_heads, d]."""
    T, heads, d = q.shape
    kv_heads = k.shape[1]
    group = heads // kv_heads
    out = torch.zeros_like(q)
    for t in range(T):
        p = int(positions[t])
        start = p + 1 - window if (window > 0 and p + 1 > window) else 0
        keys = torch.tensor([j for j in range(T) if start <= int(positions[j]) <= p])
        for h in range(heads):
            g = h // group
            s = (k[keys, g] @ q[t, h]) * scale
            e = torch.exp(s - s.max())
            out[t, h] = (e[:, None] * v[keys, g]).sum(0) / e.sum()
    return out


def silu(g: torch.Tensor) -> torch.Tensor:
    """silu(g) = g / (1 + exp(-g)).   layers.cu:512-529 (SiluMulFusedKernel)."""
    return g / (1.0 + torch.exp(-g))


def gated_mlp(x: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor,
              rnd=no_rounding) -> torch.Tensor:
    """y = (silu(x Wg^T) * (x Wu^T)) Wd^T.   src/model/qwen2.cc:1042-1048; weights [out, in], gemm.h:51-57.
    `rnd`: what a stored activation goes through (the reference stores the two products, the activation and the
    result in bfloat16; the sums themselves are 32-bit)."""
    return rnd(rnd(silu(rnd(x @ w_gate.T)) * rnd(x @ w_up.T)) @ w_down.T)


def route(x: torch.Tensor, w_router: torch.Tensor, top_k: int, renormalize: bool,
          scale: float = 1.0, rnd=no_rounding, chosen: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """p = softmax(x Wr^T) over all experts; k rounds of argmax with strict '>' (lowest index wins a tie),
    chosen weight = p_e, chosen expert masked to -inf; optional division by the sum of the chosen; times scale.
    src/backends/cuda/ops/moe.cu:36-127 (RouteTopKKernel); src/model/moe_ffn.cc:200-221.
    Returns weights [T, k] and experts [T, k], slots in descending score.  `rnd`: the reference stores the scores
    z in bfloat16 (moe_ffn.cc:200-207) before the 32-bit softmax.
    `chosen` [T, k]: the experts are given (someone else's selection, for tests that compare a run whose near ties
    fell the other way); the weights are those experts' probabilities, everything after the selection as above."""
    z = rnd(x @ w_router.T)
    T, E = z.shape
    weights = torch.zeros(T, top_k, dtype=x.dtype)
    experts = torch.zeros(T, top_k, dtype=torch.int64)
    for t in range(T):
        e = torch.exp(z[t] - z[t].max())
        inv_sum = 1.0 / e.sum()
        row = e.clone()
        total = 0.0
        for slot in range(top_k):
            if chosen is not None:
                best = int(chosen[t, slot])
                best_value = float(row[best])
            else:
                best, best_value = -1, -math.inf
                for i in range(E):
                    if float(row[i]) > best_value:
                        best_value, best = float(row[i]), i
            weights[t, slot] = best_value * inv_sum
            total += float(weights[t, slot])
            experts[t, slot] = best
            row[best] = -math.inf
        if renormalize and total > 0:
            weights[t] = weights[t] / total
        weights[t] = weights[t] * scale
    return weights, experts


def router_margin(x: torch.Tensor, w_router: torch.Tensor, top_k: int) -> torch.Tensor:
    """Per token, how far the last chosen expert is ahead of the first one left out: (p_k - p_{k+1}) / p_k
    (1 when every expert is chosen).  A run in reduced precision may legitimately choose the other one where
    this is tiny; the tests leave such places out of bfloat16 comparisons."""
    p = torch.softmax(x @ w_router.T, -1).sort(-1, descending=True).values
    if top_k >= p.shape[-1]:
        return torch.ones(p.shape[0], dtype=p.dtype)
    return (p[:, top_k - 1] - p[:, top_k]) / p[:, top_k - 1]


def moe_block(x: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str, num_experts: int, top_k: int,
              renormalize: bool, shared_width: int, rnd=no_rounding, chosen: Optional[torch.Tensor] = None,
              chosen_out: Optional[List[torch.Tensor]] = None) -> torch.Tensor:
    """Every chosen expert applied per token and summed in slot order, plus the sigmoid-gated shared expert:
    out_t = sum_slot w_{t,slot} * MLP_e(x_t)  +  sigmoid(x_t . Wsg) * MLP_shared(x_t).
    src/model/moe_ffn.cc:158-367 (route, experts, combine :305-306, shared :308-351);
    moe.cu:237-255 (CombineRowsKernel), :275-287 (AddSharedExpertKernel: 1/(1+exp(-g)))."""
    weights, experts = route(x, w[prefix + "gate.weight"], top_k, renormalize, rnd=rnd, chosen=chosen)
    if chosen_out is not None:
        chosen_out.append(experts)
    # every expert is applied once, to the tokens that chose it (rows of a product do not depend on each other) ...
    applied = {}
    for e in sorted(set(experts.flatten().tolist())):
        p = f"{prefix}experts.{e}."
        tokens = torch.nonzero((experts == e).any(dim=1)).flatten()
        y = gated_mlp(x[tokens], w[p + "gate_proj.weight"], w[p + "up_proj.weight"], w[p + "down_proj.weight"], rnd)
        applied[e] = dict(zip(tokens.tolist(), y))
    # ... and each token sums its experts' results in slot order
    out = torch.zeros_like(x)
    for t in range(x.shape[0]):
        for slot in range(top_k):
            out[t] += weights[t, slot] * applied[int(experts[t, slot])][t]
    out = rnd(out)
    if shared_width > 0:
        p = prefix + "shared_expert."
        shared = gated_mlp(x, w[p + "gate_proj.weight"], w[p + "up_proj.weight"], w[p + "down_proj.weight"], rnd)
        gate = 1.0 / (1.0 + torch.exp(-rnd(x @ w[prefix + "shared_expert_gate.weight"].T)))  # [T, 1]
        out = rnd(out + gate * shared)
    return out


# --------------------------------------------------------------------------
def is_moe_layer(cfg: dict, layer: int) -> bool:
    """Sparse unless listed in mlp_only_layers or (layer + 1) % decoder_sparse_step != 0.
    The reference's rule is another architecture's (include/inferx/model/config.h:121-126); these two keys are the
    Qwen2-MoE ones, which the reference never reads."""
    if layer in (cfg.get("mlp_only_layers") or []):
        return False
    return cfg.get("num_experts", 0) > 0 and (layer + 1) % cfg.get("decoder_sparse_step", 1) == 0


def window_of_layer(cfg: dict, layer: int) -> int:
    """Windowed iff use_sliding_window and layer >= max_window_layers (window semantics layers.cu:346-354); a
    config that lists `layer_types` names its windowed layers itself ("sliding_attention")."""
    if cfg.get("layer_types"):
        return int(cfg["sliding_window"]) if cfg["layer_types"][layer] == "sliding_attention" else 0
    if cfg.get("use_sliding_window", False) and cfg.get("sliding_window", 0) and \
            layer >= cfg.get("max_window_layers", cfg["num_hidden_layers"]):
        return int(cfg["sliding_window"])
    return 0


def forward(cfg: dict, weights: Dict[str, torch.Tensor], token_ids: Sequence[int],
            positions: Optional[Sequence[int]] = None,
            schedule: Optional[List[Tuple[int, Optional[int]]]] = None,
            margins: Optional[List[torch.Tensor]] = None, rnd=no_rounding,
            router_scores: Optional[List[torch.Tensor]] = None, experts: Optional[List[torch.Tensor]] = None,
            experts_out: Optional[List[torch.Tensor]] = None) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence.  Layer order and the place of every norm and residual:
    src/model/qwen2.cc:902-1066 (embed :902; input norm :912; qkv + bias :920-923; rope :925-926; attention
    :1021-1023; o_proj + residual :1026-1030; post norm :1036; feed-forward :1042-1048; residual :1051; final norm
    and head :1059-1066).  `schedule`: (layer, cache_from) per execution, default each layer once.
    `margins`: if a list, the router margin per token of every sparse layer run is appended to it; `router_scores`
    likewise takes the router's scores [T, experts] of every sparse layer, `experts_out` the chosen experts [T, k].
    `experts`: the chosen experts [T, k] of every sparse layer run, given from outside instead of selected here.

    `rnd` is what every stored activation goes through.  With `to_bfloat16_and_back` this is the reference's
    bfloat16 model: every tensor it keeps between kernels is bfloat16 (norm outputs layers.cu:50-76; the q/k/v
    product, then again after the bias :485-510; rotated q and k :80-115; attention output :256-318; the output
    product and the residual sum :542-548; feed-forward activations; the router's scores, moe_ffn.cc:200-207) while
    every sum inside a kernel is 32-bit.  The difference between that model and this one in float64 is the error
    that bfloat16 storage alone brings: the measure for what a bfloat16 engine may differ by (the reference derives
    its own tolerance so, scripts/gen_reference_logits.py:51-55).  The logits themselves are left unrounded."""
    w = weights if isinstance(weights, Widened) else Widened(weights)
    H = cfg["hidden_size"]
    heads = cfg["num_attention_heads"]
    kv_heads = cfg.get("num_key_value_heads", heads)
    d = cfg.get("head_dim") or H // heads
    eps = cfg.get("rms_norm_eps", 1e-6)
    theta = float(cfg.get("rope_theta", 10000.0))
    T = len(token_ids)
    pos = torch.arange(T) if positions is None else torch.tensor(list(positions))
    scale = 1.0 / math.sqrt(d)  # qwen2.cc:890
    h = rnd(w["model.embed_tokens.weight"][torch.tensor(list(token_ids))])  # layers.cu:465-481
    if schedule is None:
        schedule = [(l, None) for l in range(cfg["num_hidden_layers"])]
    kept: List[Tuple[torch.Tensor, torch.Tensor]] = []
    sparse_runs = 0
    for layer, cache_from in schedule:
        p = f"model.layers.{layer}."
        x = rnd(rms_norm(h, w[p + "input_layernorm.weight"], eps))
        a = p + "self_attn."
        q = rnd(x @ w[a + "q_proj.weight"].T)
        k = rnd(x @ w[a + "k_proj.weight"].T)
        v = rnd(x @ w[a + "v_proj.weight"].T)
        if a + "q_proj.bias" in w:  # SplitQkvKernel adds the bias after the product, layers.cu:485-510
            q, k, v = rnd(q + w[a + "q_proj.bias"]), rnd(k + w[a + "k_proj.bias"]), rnd(v + w[a + "v_proj.bias"])
        q = rnd(apply_rope(q.view(T, heads, d), pos, theta))
        k = rnd(apply_rope(k.view(T, kv_heads, d), pos, theta))  # rotated keys are what is cached, qwen2.cc:928-969
        v = v.view(T, kv_heads, d)
        if cache_from is not None:
            k, v = kept[cache_from]
        kept.append((k, v))
        att = rnd(attention(q, k, v, pos, scale, window_of_layer(cfg, layer)))
        h = rnd(h + rnd(att.reshape(T, heads * d) @ w[a + "o_proj.weight"].T))
        x = rnd(rms_norm(h, w[p + "post_attention_layernorm.weight"], eps))
        m = p + "mlp."
        if is_moe_layer(cfg, layer):
            if margins is not None:
                margins.append(router_margin(x, w[m + "gate.weight"], cfg["num_experts_per_tok"]))
            if router_scores is not None:
                router_scores.append(rnd(x @ w[m + "gate.weight"].T))
            f = moe_block(x, w, m, cfg["num_experts"], cfg["num_experts_per_tok"],
                          bool(cfg.get("norm_topk_prob", False)), cfg.get("shared_expert_intermediate_size", 0), rnd,
                          chosen=experts[sparse_runs] if experts is not None else None, chosen_out=experts_out)
            sparse_runs += 1
        else:
            f = gated_mlp(x, w[m + "gate_proj.weight"], w[m + "up_proj.weight"], w[m + "down_proj.weight"], rnd)
        h = rnd(h + f)
    x = rnd(rms_norm(h, w["model.norm.weight"], eps))
    head = w["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings", False) else w["lm_head.weight"]
    return x @ head.T


# --------------------------------------------------------------------------
def greedy(logits_row: torch.Tensor) -> int:
    """First maximum, lowest index on ties.   src/engine/host_sampling.cc:52-53; layers.cu:413-452."""
    best, best_value = 0, -math.inf
    for i, v in enumerate(logits_row.tolist()):
        if v > best_value:
            best, best_value = i, v
    return best


def sampling_support(logits_row: torch.Tensor, temperature: float, top_k: int = 0, top_p: float = 1.0,
                     min_p: float = 0.0) -> List[int]:
    """Token ids that temperature sampling with the given cut-offs may return.
    p = softmax(logits / t); sort descending (ties by index); keep the first top_k, then those with
    p >= min_p * p_max, then the smallest prefix whose mass reaches top_p.
    src/engine/host_sampling.cc:60-97."""
    p = torch.softmax(logits_row.to(F64) / temperature, dim=-1)
    order = sorted(range(p.numel()), key=lambda i: (-float(p[i]), i))
    keep = len(order)
    if top_k > 0:
        keep = min(keep, top_k)
    if min_p > 0:
        floor = min_p * float(p[order[0]])
        n = 0
        while n < keep and float(p[order[n]]) >= floor:
            n += 1
        keep = max(n, 1)
    if top_p < 1.0:
        mass, n = 0.0, 0
        while n < keep:
            mass += float(p[order[n]])
            n += 1
            if mass >= top_p:
                break
        keep = max(n, 1)
    return order[:keep]
