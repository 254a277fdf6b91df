"""What a run is made of besides the model: device, the activations' type, the
library matrix product, and the per-step context that parts read.

Library matrix products stand where the reference calls its vendor library
(`CublasLtGemm::LinearBF16`, include/inferx/ops/gemm.h:68-80: y = x . W^T with
weights [out, in] as on disk, float32 accumulation).  In a float32 run every
product is true float32: reduced-precision matrix modes are switched off.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

import torch


def _dtype_of(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name in (torch.float32, torch.bfloat16):
            return name
    table = {"float32": torch.float32, "fp32": torch.float32, "float": torch.float32,
             "bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "auto": torch.bfloat16}
    if name in table:
        return table[name]
    raise ValueError(f"dtype {name!r} is not one of float32, bfloat16")


class Runtime:
    def __init__(self, dtype="bfloat16", device: str = "cuda:0"):
        self.dtype = _dtype_of(dtype)
        self.device = torch.device(device)
        if self.device.type != "cuda" or not torch.cuda.is_available():
            raise RuntimeError("inferx_amd runs on a GPU only: no HIP device is visible (there is no CPU path)")
        torch.cuda.set_device(self.device)
        # true 32-bit products: no TF32-like or reduced-precision reduction modes
        torch.backends.cuda.matmul.allow_tf32 = False
        torch.backends.cudnn.allow_tf32 = False
        torch.set_float32_matmul_precision("highest")
        if hasattr(torch.backends.cuda.matmul, "allow_bf16_reduced_precision_reduction"):
            torch.backends.cuda.matmul.allow_bf16_reduced_precision_reduction = False
        from .. import ops
        ops.lib()  # fail now, loudly, if the HIP library cannot be had
        self._mm_out_dtype_ok: Optional[bool] = None
        self._skinny_plans: Dict[int, Any] = {}
        self._side_stream: Optional[torch.cuda.Stream] = None

    @property
    def is_fp32(self) -> bool:
        return self.dtype == torch.float32

    # ---- work beside the main stream ------------------------------------------------------------------
    def can_run_beside(self) -> bool:
        """Not while a graph is being captured: a captured step stays on one stream."""
        return not torch.cuda.is_current_stream_capturing()

    def run_beside(self, fn):
        """Runs fn() on a second stream (of the default priority) that starts from the main stream's present
        state, and returns (fn's tensor, join): the main stream goes on at once, and `join()` makes it wait for
        fn's work.  What fn allocates belongs to the second stream; the tensor it returns is marked as used by
        the main stream too, so that its memory is not given out again before the main stream is done with it."""
        main = torch.cuda.current_stream(self.device)
        if self._side_stream is None:
            self._side_stream = torch.cuda.Stream(self.device)
        side = self._side_stream
        side.wait_stream(main)
        with torch.cuda.stream(side):
            out = fn()
        out.record_stream(main)

        def join():
            main.wait_stream(side)
        return out, join

    def empty(self, shape, dtype=None) -> torch.Tensor:
        return torch.empty(shape, dtype=dtype or self.dtype, device=self.device)

    def place(self, t: torch.Tensor) -> torch.Tensor:
        """A loaded tensor on the device in the type it keeps for this run: in a
        float32 run everything becomes float32 (exact); in a bfloat16 run bfloat16
        stays, a tensor stored in 32 bits stays so, float16 is widened to float32."""
        if t.dtype in (torch.int32, torch.int64, torch.int16, torch.int8, torch.uint8):
            return t.to(self.device, torch.int32)
        if self.is_fp32 or t.dtype in (torch.float32, torch.float16, torch.float64):
            return t.to(self.device, torch.float32)
        return t.to(self.device, torch.bfloat16)

    # ---- few rows (decoding): the weights are the traffic, so they are streamed by the matrix-core kernel
    # that also serves the experts (one "expert", one row tile), instead of a library product tuned for tiles
    # Up to two 16-row tiles: a decode step of 6 layers at batch 17 / 24 / 32 took 1477 / 1642 / 1822 us against
    # 1566 / 1691 / 1837 us through the library's products; from 48 rows on the library is faster (1966 against 2120).
    SKINNY_ROWS = 32

    def _skinny_ok(self, x: torch.Tensor, w: torch.Tensor) -> bool:
        return (x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and 0 < x.shape[0] <= self.SKINNY_ROWS
                and x.shape[1] % 8 == 0 and x.is_contiguous() and w.is_contiguous())

    def _skinny(self, x: torch.Tensor, w: torch.Tensor, gate_up: bool) -> torch.Tensor:
        from .. import ops
        T = x.shape[0]
        plan = self._skinny_plans.get(T)
        if plan is None:
            tile_rows = 16 if T <= 16 else (32 if T <= 32 else 64)
            mt = ops.moe_max_tiles(T, 1, tile_rows)
            tile_map = torch.tensor([0] * (2 * mt) + [1], dtype=torch.int32, device=self.device)
            offsets = torch.tensor([0, T], dtype=torch.int32, device=self.device)
            plan = self._skinny_plans[T] = (offsets, tile_map, tile_rows)
        offsets, tile_map, tile_rows = plan
        n_out = w.shape[0] // 2 if gate_up else w.shape[0]
        out = self.empty((T, n_out))
        ops.moe_grouped_mfma(x, w.unsqueeze(0), out, offsets, None, tile_map, tile_rows, gate_up, 4)
        return out

    def linear(self, x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
        """x [T, in] . w[out, in]^T -> [T, out] in the run's type, float32 accumulation.
        A weight kept in float32 during a bfloat16 run is multiplied in float32."""
        if w.dtype == x.dtype:
            if self._skinny_ok(x, w):
                return self._skinny(x, w, False)
            if x.dtype == torch.bfloat16 and x.shape[0] > 0 and x.is_contiguous() and w.is_contiguous():
                # the vendor library's product, called through its C interface (half the host time of the call
                # through the tensor library, the same kernel and bits)
                from .. import ops
                out = self.empty((x.shape[0], w.shape[0]))
                if ops.gemm_bf16(x, w, out):
                    return out
            return torch.matmul(x, w.t())
        return torch.matmul(x.to(torch.float32), w.to(torch.float32).t()).to(self.dtype)

    def gated_linear(self, x: torch.Tensor, w_gate_up: torch.Tensor) -> torch.Tensor:
        """silu(x . Wg^T) * (x . Wu^T) for w_gate_up = [Wg; Wu] of shape [2 n, in] -> [T, n]."""
        from .. import ops
        if self._skinny_ok(x, w_gate_up):
            return self._skinny(x, w_gate_up, True)
        gate_up = self.linear(x, w_gate_up)
        act = self.empty((x.shape[0], w_gate_up.shape[0] // 2))
        ops.silu_mul(gate_up, act)
        return act

    def linear_f32(self, x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
        """As `linear`, result float32 (the logits)."""
        if x.dtype == torch.float32 and w.dtype == torch.float32:
            return torch.matmul(x, w.t())
        if x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16:
            if self._skinny_ok(x, w):  # few rows: the vocabulary's weights are the traffic
                from .. import ops
                out = self.empty((x.shape[0], w.shape[0]), torch.float32)
                ops.linear_skinny_f32(x, w, out)
                return out
            if x.shape[0] > 0 and x.is_contiguous() and w.is_contiguous():
                from .. import ops
                out = self.empty((x.shape[0], w.shape[0]), torch.float32)
                if ops.gemm_bf16(x, w, out):
                    return out
            if self._mm_out_dtype_ok is not False:
                try:
                    out = torch.mm(x, w.t(), out_dtype=torch.float32)
                    self._mm_out_dtype_ok = True
                    return out
                except (TypeError, RuntimeError):
                    if self._mm_out_dtype_ok:  # it worked before: a real failure
                        raise
                    self._mm_out_dtype_ok = False
            return torch.matmul(x, w.t()).to(torch.float32)
        return torch.matmul(x.to(torch.float32), w.to(torch.float32).t())


@dataclass
class CacheBinding:
    """What one part of one layer execution sees of the cache manager's memory."""

    group: int = -1
    arrays: Dict[str, torch.Tensor] = field(default_factory=dict)  # by the names of the part's `CacheNeed`
    writes: bool = True                    # False: reads another execution's cache
    state: Optional[torch.Tensor] = None   # [slots, *shape]

    @property
    def k(self) -> Optional[torch.Tensor]:
        """Attention's keys: [pages, kv_heads, page_size, head_dim]."""
        return self.arrays.get("k")

    @property
    def v(self) -> Optional[torch.Tensor]:
        """Attention's values, transposed within a page: [pages, kv_heads, head_dim, page_size]."""
        return self.arrays.get("v")


@dataclass
class StepContext:
    rt: Runtime
    num_tokens: int
    num_requests: int
    token_ids: torch.Tensor
    positions: torch.Tensor
    seq_of_token: torch.Tensor
    q_start: torch.Tensor
    seq_lens: torch.Tensor
    state_slots: torch.Tensor
    logits_rows: torch.Tensor
    slots: List[torch.Tensor]
    block_tables: List[torch.Tensor]
    host: Any = None                       # the StepBatch (host arrays), for parts that plan on the host
    one_token_each: bool = False           # every request brings exactly one token (a decoding step)
    memo: Dict[Any, Any] = field(default_factory=dict)  # per-step results shared between layers
