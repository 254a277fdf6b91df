"""Mixture-of-experts feed-forward with an optional (sigmoid-gated) shared expert.

route -> group -> gate|up of the routed experts (+SwiGLU) -> down -> weighted
sum in slot order + shared expert (reference: MoeFfn::ForwardImpl,
src/model/moe_ffn.cc:158-367; kernels src/backends/cuda/ops/moe.cu).  Expert
weights are stacked at load: w13 [E, 2*mi, H] (gate rows, then up rows, per
expert) and w2 [E, H, mi] (reference: moe_ffn.h:25-34; stacking pattern
src/model/deepseek_v2.cc:515-542).  Router scores and the shared gate are
float32 from the product on.
"""
from __future__ import annotations

from typing import List

import torch

from .. import ops
from .base import FeedForward, LazyDelta, LazyNorm, ParamSpec, register_part
from .dense_mlp import stack_rows


# From here on the shared expert runs on a second stream beside the routed ones.  Below it a step of 24 layers
# waits for the host, which the two streams' hand-overs cost 21 us a layer (measured at the A2.7B shape, beside
# against one after the other: 8.1 against 7.0 ms at 256 tokens, 8.3 against 8.3 at 512, 9.0 against 9.8 at 768,
# 15.1 against 15.4 at 2,048).
SHARED_BESIDE_TOKENS = 512
# From this width on the LDS-staged expert products run in their wide form (256 weight rows per workgroup) and the
# shared expert stays on the main stream (a wide workgroup fills a compute unit's LDS, the library's kernels find
# no place beside it).  Measured, prompt portions at a width of 3,584 (64 experts of 2,560, 8 per token): 14.9 against
# 15.5 ms for a mixed step of 1,056 tokens and 8 layers, 2.86 against 3.03 s for 193,000 tokens of long prompts; at a
# width of 2,048 (60 experts of 1,408, 4 per token) the narrow form beside the shared expert is ahead, 15.2 against
# 16.0 ms for 2,048 tokens and 24 layers.
WIDE_TILES_WIDTH = 3072
# Between the few rows of a decoding step (where routed and shared experts already share a launch) and the portions
# from which the shared expert's library products run beside the routed experts, the shared expert is cut into
# pieces of the routed experts' width, which every token "chooses" with the shared gate's value as their weight:
# grouping, the two grouped products and the weighted sum then take it along, its weights stream at the rate of the
# big launches instead of through two library products of few rows and a launch for SwiGLU.  Needs a shared width
# that is a multiple of the experts' width; keeps the shared expert's weights a second time, in that layout.
# Measured at the A2.7B shape (24 layers), with against without: decoding at batch 64 11.22 against 11.59 ms a step; a
# portion of 256 tokens 6.58 against 7.19 ms, of 512 8.16 against 9.17, of 768 9.50 against 9.47, of 1,024 10.88
# against 10.42; at the 57B shape (8 layers) 512 tokens 9.41 against 10.26 ms, 1,024 13.41 against 13.29.
FOLD_SHARED_BELOW_TOKENS = 768


class MoeFeedForward(FeedForward):
    graph_safe = True

    def __init__(self, hidden_size: int, num_experts: int, top_k: int, expert_width: int, shared_width: int = 0,
                 shared_gated: bool = True, renormalize: bool = False, routed_scale: float = 1.0,
                 init_std: float = 0.02):
        if not 0 < top_k <= num_experts:
            raise ValueError(f"top_k {top_k} must be between 1 and num_experts {num_experts}")
        if num_experts > 1024 or top_k > 32:
            raise ValueError("at most 1024 experts and top_k 32 are supported")
        self.hidden_size, self.num_experts, self.top_k = int(hidden_size), int(num_experts), int(top_k)
        self.expert_width, self.shared_width = int(expert_width), int(shared_width)
        self.shared_gated, self.renormalize = bool(shared_gated), bool(renormalize)
        self.routed_scale, self.init_std = float(routed_scale), float(init_std)
        self.wide_tiles = self.hidden_size >= WIDE_TILES_WIDTH
        # pieces of the routed experts' width that the shared expert is cut into for steps of middling size, or 0
        self.shared_pieces = self.shared_width // self.expert_width if (
            self.shared_width > 0 and self.shared_width % self.expert_width == 0
            and self.shared_width // self.expert_width <= 32) else 0
        self.w13_all = self.w2_all = None  # routed experts, then the shared expert's pieces
        self.w_router = self.w13 = self.w2 = None
        self.w_shared_gate_up = self.w_shared_down = self.w_shared_gate = None

    def param_specs(self) -> List[ParamSpec]:
        H, mi, si, s = self.hidden_size, self.expert_width, self.shared_width, self.init_std
        specs = [ParamSpec("gate.weight", (self.num_experts, H), std=s)]
        for e in range(self.num_experts):
            specs += [ParamSpec(f"experts.{e}.gate_proj.weight", (mi, H), std=s),
                      ParamSpec(f"experts.{e}.up_proj.weight", (mi, H), std=s),
                      ParamSpec(f"experts.{e}.down_proj.weight", (H, mi), std=s)]
        if si > 0:
            specs += [ParamSpec("shared_expert.gate_proj.weight", (si, H), std=s),
                      ParamSpec("shared_expert.up_proj.weight", (si, H), std=s),
                      ParamSpec("shared_expert.down_proj.weight", (H, si), std=s)]
            if self.shared_gated:
                specs.append(ParamSpec("shared_expert_gate.weight", (1, H), std=s))
        return specs

    def bind(self, tensors, rt) -> None:
        E = self.num_experts
        self.w_router = tensors["gate.weight"].contiguous()
        parts = []
        for e in range(E):
            parts += [tensors[f"experts.{e}.gate_proj.weight"], tensors[f"experts.{e}.up_proj.weight"]]
        downs = [tensors[f"experts.{e}.down_proj.weight"] for e in range(E)]
        mi, S = self.expert_width, self.shared_pieces
        fold = S > 0 and all(t.dtype == torch.bfloat16 for t in parts + downs) and all(
            tensors[f"shared_expert.{n}_proj.weight"].dtype == torch.bfloat16 for n in ("gate", "up", "down"))
        if fold:  # piece c of the shared expert: its gate rows, its up rows, and the columns of the down product
            for c in range(S):
                parts += [tensors["shared_expert.gate_proj.weight"][c * mi:(c + 1) * mi],
                          tensors["shared_expert.up_proj.weight"][c * mi:(c + 1) * mi]]
                downs.append(tensors["shared_expert.down_proj.weight"][:, c * mi:(c + 1) * mi])
        else:
            self.shared_pieces = S = 0
        self.w13_all = stack_rows(parts).view(E + S, 2 * mi, self.hidden_size)
        self.w2_all = stack_rows(downs).view(E + S, self.hidden_size, mi)
        self.w13, self.w2 = self.w13_all[:E], self.w2_all[:E]
        if self.shared_width > 0:
            self.w_shared_gate_up = stack_rows([tensors["shared_expert.gate_proj.weight"],
                                                tensors["shared_expert.up_proj.weight"]])
            self.w_shared_down = tensors["shared_expert.down_proj.weight"].contiguous()
            if self.shared_gated:
                self.w_shared_gate = tensors["shared_expert_gate.weight"].contiguous()

    # -- the steps, separately callable so tests can look between them ----
    def route(self, ctx, x, always: int = 0):
        """`always`: the shared expert's pieces follow each token's chosen experts, with the shared gate's value (or
        1) as their weight."""
        rt, T, k = ctx.rt, x.shape[0], self.top_k + always
        topk_w = rt.empty((T, k), torch.float32)
        topk_e = rt.empty((T, k), torch.int32)
        gate = rt.empty((T,), torch.float32) if self.w_shared_gate is not None else None
        ops.moe_route(x, self.w_router, self.w_shared_gate, topk_w, topk_e, gate, self.renormalize, self.routed_scale,
                      always)
        return topk_w, topk_e, gate

    def _tile_rows(self, ctx, x) -> int:
        """Rows per tile of the matrix-core product, or 0 where it does not take the shapes (then the plain one runs)."""
        ok = (x.dtype == torch.bfloat16 and self.w13.dtype == torch.bfloat16 and self.w2.dtype == torch.bfloat16
              and self.hidden_size % 8 == 0 and self.expert_width % 8 == 0)
        if not ok:
            return 0
        # A decoding step, or few rows per expert: 16-row tiles, the weights streamed by every wavefront for itself.
        # From about three rows per expert on the LDS-staged kernel is faster (60 experts, 4 per token: 174 against
        # 173 us for both products at 48 tokens, 209 against 189 at 96, 316 against 195 at 256).
        per_expert = x.shape[0] * self.top_k / self.num_experts
        return 16 if (x.shape[0] <= ctx.rt.SKINNY_ROWS or per_expert <= 3) else ops.moe_tiled_rows(self.wide_tiles)

    def dispatch(self, ctx, topk_e, tile_rows: int = 0, always: int = 0):
        rt, A, E = ctx.rt, topk_e.numel(), self.num_experts + always
        offsets = rt.empty((E + 1,), torch.int32)
        rows = rt.empty((A,), torch.int32)
        dest = rt.empty((A,), torch.int32)
        tile_map = None
        if tile_rows:
            tile_map = rt.empty((2 * ops.moe_max_tiles(A, E, tile_rows) + 1,), torch.int32)
        ops.moe_dispatch(topk_e, offsets, rows, dest, E, tile_rows, tile_map)
        return offsets, rows, dest, tile_map

    def experts(self, ctx, x, offsets, rows, tile_map=None, tile_rows: int = 0, with_shared: bool = False):
        """`with_shared`: the grouping holds the shared expert's pieces as further experts."""
        rt, A = ctx.rt, rows.numel()
        w13, w2 = (self.w13_all, self.w2_all) if with_shared else (self.w13, self.w2)
        act = rt.empty((A, self.expert_width))
        y = rt.empty((A, self.hidden_size))
        if tile_rows == ops.moe_tiled_rows(self.wide_tiles):  # many rows per expert: operands staged through LDS
            ops.moe_grouped_tiled(x, w13, act, offsets, rows, tile_map, True, self.wide_tiles)
            ops.moe_grouped_tiled(act, w2, y, offsets, None, tile_map, False, self.wide_tiles)
        elif tile_rows:
            # few rows: the weights are the traffic, the reduction is split over a workgroup's four wavefronts
            ops.moe_grouped_mfma(x, w13, act, offsets, rows, tile_map, tile_rows, True, 4)
            ops.moe_grouped_mfma(act, w2, y, offsets, None, tile_map, tile_rows, False, 4)
        else:
            ops.moe_grouped_plain(x, w13, act, offsets, rows, gate_up=True)
            ops.moe_grouped_plain(act, w2, y, offsets, None, gate_up=False)
        return y

    def _one_launch(self, ctx, x, tile_rows: int) -> bool:
        """Few tokens (decoding): routed and shared experts go into one launch per product."""
        return (tile_rows == 16 and self.shared_width > 0 and self.shared_width % 8 == 0
                and x.shape[0] <= ctx.rt.SKINNY_ROWS and self.w_shared_gate_up.dtype == torch.bfloat16
                and self.w_shared_down.dtype == torch.bfloat16)

    def experts_and_shared(self, ctx, x, offsets, rows, tile_map, tile_rows):
        rt, A, T = ctx.rt, rows.numel(), x.shape[0]
        act, sact = rt.empty((A, self.expert_width)), rt.empty((T, self.shared_width))
        ops.moe_grouped_dual(x, self.w13, act, offsets, rows, tile_map, tile_rows, x, self.w_shared_gate_up, sact, True)
        y, sout = rt.empty((A, self.hidden_size)), rt.empty((T, self.hidden_size))
        ops.moe_grouped_dual(act, self.w2, y, offsets, None, tile_map, tile_rows, sact, self.w_shared_down, sout, False)
        return y, sout

    def shared(self, ctx, x):
        rt = ctx.rt
        return rt.linear(rt.gated_linear(x, self.w_shared_gate_up), self.w_shared_down)

    def route_and_dispatch(self, ctx, x, tile_rows: int, norm=None, always: int = 0):
        """`route` then `dispatch`; for the few tokens of a decoding step in one launch, and the norm before the
        feed-forward with them: `norm` = (h, delta, weight, eps, x), x still to be filled.  `always`: see `route`
        (the chosen experts are then the first `top_k` columns of what is returned)."""
        rt, T, k, E = ctx.rt, x.shape[0], self.top_k, self.num_experts
        if always or not ops.route_one_launch_fits(T, self.hidden_size, E):
            assert norm is None
            topk_w, topk_e, gate = self.route(ctx, x, always)
            return (topk_w, topk_e, gate) + self.dispatch(ctx, topk_e, tile_rows, always)
        topk_w = rt.empty((T, k), torch.float32)
        topk_e = rt.empty((T, k), torch.int32)
        gate = rt.empty((T,), torch.float32) if self.w_shared_gate is not None else None
        offsets = rt.empty((E + 1,), torch.int32)
        rows = rt.empty((T * k,), torch.int32)
        dest = rt.empty((T * k,), torch.int32)
        tile_map = rt.empty((2 * ops.moe_max_tiles(T * k, E, tile_rows) + 1,), torch.int32) if tile_rows else None
        ops.moe_route_dispatch(None if norm else x, self.w_router, self.w_shared_gate, topk_w, topk_e, gate,
                               self.renormalize, self.routed_scale, offsets, rows, dest, tile_rows, tile_map, norm)
        return topk_w, topk_e, gate, offsets, rows, dest, tile_map

    takes_lazy_norm = True

    def forward(self, ctx, x):
        norm = None
        if isinstance(x, LazyNorm):
            # a decoding step: the norm is applied by the router's kernel, which every token's row passes anyway
            rms = x.rms_operands()
            if rms is not None and ops.route_one_launch_fits(x.h.shape[0], self.hidden_size, self.num_experts):
                lazy, x = x, ctx.rt.empty(tuple(x.h.shape))
                norm = (lazy.h, lazy.delta, rms[0], rms[1], x)
            else:
                x = x.materialize(ctx)
        tile_rows = self._tile_rows(ctx, x)
        one_launch = self._one_launch(ctx, x, tile_rows)
        if (self.shared_pieces and tile_rows and not one_launch and norm is None
                and ctx.rt.SKINNY_ROWS < x.shape[0] < FOLD_SHARED_BELOW_TOKENS):
            # a step of middling size: the shared expert rides along as pieces that every token chooses
            topk_w, _, _, offsets, rows, dest, tile_map = self.route_and_dispatch(ctx, x, tile_rows,
                                                                                  always=self.shared_pieces)
            y = self.experts(ctx, x, offsets, rows, tile_map, tile_rows, with_shared=True)
            return MoeSum(y, dest, topk_w, None, None, self.hidden_size)
        shared = join = None
        if (not one_launch and self.shared_width > 0 and tile_rows == ops.MOE_TILED_ROWS and not self.wide_tiles
                and x.shape[0] >= SHARED_BESIDE_TOKENS and ctx.rt.can_run_beside()):
            # a prompt portion: the shared expert's library products are bound by the matrix cores, the routed
            # experts' kernels by memory, so the two run beside each other on two streams
            shared, join = ctx.rt.run_beside(lambda: self.shared(ctx, x))
        topk_w, topk_e, gate, offsets, rows, dest, tile_map = self.route_and_dispatch(ctx, x, tile_rows, norm)
        if one_launch:
            y, shared = self.experts_and_shared(ctx, x, offsets, rows, tile_map, tile_rows)
        else:
            y = self.experts(ctx, x, offsets, rows, tile_map, tile_rows)
            if join is not None:
                join()
            elif self.shared_width > 0:
                shared = self.shared(ctx, x)
        return MoeSum(y, dest, topk_w, shared, gate, self.hidden_size)


class MoeSum(LazyDelta):
    """sum_s topk_w[t, s] * y[dest[t, s]] + gate[t] * shared[t], formed by whoever consumes it."""

    def __init__(self, y, dest, topk_w, shared, gate, width):
        self.y, self.dest, self.topk_w, self.shared, self.gate, self.width = y, dest, topk_w, shared, gate, width

    def materialize(self, ctx):
        out = ctx.rt.empty((self.topk_w.shape[0], self.width))
        ops.moe_combine(self.y, self.dest, self.topk_w, self.shared, self.gate, out)
        return out

    def add_rmsnorm(self, ctx, h, weight, eps, rows, out) -> bool:
        if self.width * 4 > 60 * 1024:
            return False
        ops.moe_combine_add_rmsnorm(h, self.y, self.dest, self.topk_w, self.shared, self.gate, weight, out, eps, rows)
        return True


register_part("feed_forward", "moe", MoeFeedForward)
