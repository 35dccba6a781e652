"""Gated feed-forward: down( act(gate x) * up x ), act = SiLU
(/root/reference/crates/nnis-model/src/runtime.rs:1054-1087;
/root/reference/crates/nnis-model/src/fused_swiglu.rs:14-28), the tanh form
of GELU, or ReLU.  Gate and up are one fused projection whose first ``inner`` output
columns are the gate."""

from __future__ import annotations

import torch

from ..errors import Unsupported
from .base import FeedForward, TensorSpec, register_part
from .linear import Projection


class GatedFeedForward(FeedForward):
    graph_safe = True

    def __init__(self, width, inner, gate, up, down, activation="silu"):
        if activation not in ("silu", "gelu_tanh", "relu"):
            raise Unsupported(f"gated feed-forward activation {activation!r}; silu, gelu_tanh and relu are built")
        self.activation = activation
        self.width, self.inner = int(width), int(inner)
        self.names = {"gate": gate, "up": up, "down": down}
        self.gate_up = None
        self.down = None

    def tensors(self):
        return [
            TensorSpec(self.names["gate"], (self.inner, self.width)),
            TensorSpec(self.names["up"], (self.inner, self.width)),
            TensorSpec(self.names["down"], (self.width, self.inner)),
        ]

    def bind(self, weights, rt):
        if rt.dtype == torch.bfloat16:
            rt.ops.unit_rows(rt.device)  # (made here, outside any captured step)
        self.gate_up = Projection(torch.cat([weights[self.names["gate"]], weights[self.names["up"]]], dim=0), rt)
        self.down = Projection(weights[self.names["down"]], rt)

    def weight_bytes(self):
        return self.gate_up.weight_bytes() + self.down.weight_bytes()

    takes_pending_norm = True
    adds_to_residual = True

    def forward(self, x, ctx, rt, into=None):
        from .lazy import PendingNorm

        if isinstance(x, PendingNorm) and self.activation == "silu" and x.can_fuse(self.gate_up.weight):
            # (residual sum,) norm, both projections and the gating in one kernel
            hidden = x.fused(self.gate_up.weight, rt.empty(x.rows, self.inner), rt.ops.EPILOGUE_SILU)
        else:
            if isinstance(x, PendingNorm):
                x = x.materialize()
            ops = rt.ops
            if (rt.dtype == torch.bfloat16 and x.dtype == torch.bfloat16 and isinstance(self.gate_up.weight, ops.PackedWeight)
                    and 0 < x.shape[0] <= ops.UNIT_ROWS_MOST and x.is_contiguous() and x.data_ptr() % 16 == 0):
                # both projections with the gating in their epilogue, on rows that are normed already
                hidden = ops.gated_linear(x, self.gate_up.weight, rt.empty(x.shape[0], self.inner), self.activation)
            else:
                gate_up = self.gate_up(x, rt)
                hidden = ops.gated_act(gate_up, rt.empty(x.shape[0], self.inner), self.activation)
        if into is not None and into.can_take(hidden, self.down.weight):
            return into.take(hidden, self.down.weight)  # the down projection adds to the stream itself
        return self.down(hidden, rt)


register_part("feed_forward", "gated", GatedFeedForward)
