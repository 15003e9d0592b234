"""Feed-forwards.  "swiglu", the dense gated one: down(act(gate(x)) * up(x)), no biases, act = silu
(engine/model.py:317-320 of the reference) or another of `kernels.lib.ACTIVATIONS` by the spec's
`activation`.  gate and up are one product over
concatenated weights; the gate is applied in float32 and rounded once.  "dense", the plain
one: down(act(up(x))), act one of `kernels.lib.ACTIVATIONS`, applied in float32."""

from __future__ import annotations

import torch

from ..kernels import lib as K
from .base import OwedRows, Part, plain_rows, register_feed_forward
from .linear import Linear, rows_a_graph_may_hold


@register_feed_forward("swiglu")
class SwiGLU(Part):
    graph_safe = True
    takes_owed_rows = True
    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        if spec.activation not in K.ACTIVATIONS:
            raise ValueError(f"activation '{spec.activation}' is not one of {', '.join(K.ACTIVATIONS)}")
        self.silu = spec.activation == "silu"  # the activation the few-row product's gated epilogue knows

    @property
    def graph_max_rows(self):
        return rows_a_graph_may_hold(self.dtype, self.spec.hidden_size, self.spec.intermediate_size)

    def tensors(self, prefix):
        s = self.spec
        return {prefix + s.gate_name + s.weight_suffix: (s.intermediate_size, s.hidden_size),
                prefix + s.up_name + s.weight_suffix: (s.intermediate_size, s.hidden_size),
                prefix + s.down_name + s.weight_suffix: (s.hidden_size, s.intermediate_size)}

    BLOCK = 8  # gate and up rows alternate in blocks of this many (the skinny product's gated epilogue)

    def bind(self, prefix, weights):
        s = self.spec
        gate, up = weights[prefix + s.gate_name + s.weight_suffix], weights[prefix + s.up_name + s.weight_suffix]
        inter, hidden = gate.shape
        self.block = self.BLOCK if (self.dtype == torch.bfloat16 and inter % self.BLOCK == 0) else 0
        if self.block:
            b = self.block
            gate_up = torch.stack([gate.view(inter // b, b, hidden), up.view(inter // b, b, hidden)], dim=1)
            gate_up = gate_up.reshape(2 * inter, hidden)
        else:
            gate_up = torch.cat([gate, up], dim=0)
        self.gate_up = Linear(self.matrix(gate_up))
        self.down = Linear(self.matrix(weights[prefix + s.down_name + s.weight_suffix]))

    def decode_fusable(self, rows: int, block_size: int) -> bool:
        s = self.spec
        return (self.silu and self.dtype == torch.bfloat16 and bool(self.block) and 0 < rows <= K.program_max_rows()
                and s.hidden_size % 8 == 0 and s.intermediate_size % 8 == 0
                and K.program_takes_product(rows, s.hidden_size,
                                            K.whole_sum_splits(2 * s.intermediate_size, s.hidden_size, rows))
                and K.program_takes_product(rows, s.intermediate_size,
                                            K.residual_splits(s.hidden_size, s.intermediate_size, rows)))

    def forward(self, ctx, x):
        """`x`: normalised activations, or `OwedRows` (the gated product then pays their scale)."""
        act = torch.empty((x.shape[0], self.spec.intermediate_size), dtype=x.dtype, device=x.device)
        rows = x.rows if isinstance(x, OwedRows) else x
        if self.silu and self.block and x.shape[0] and K.skinny_supported(rows, self.gate_up.weight):
            splits = K.whole_sum_splits(2 * self.spec.intermediate_size, self.spec.hidden_size, x.shape[0])
            K.gemm_skinny(act, rows, self.gate_up.weight, None, K.EPI_SWIGLU, splits,
                          row_scale=x.row_scale if isinstance(x, OwedRows) else None)
        elif self.block and x.shape[0] and K.skinny_supported(rows, self.gate_up.weight) and not isinstance(x, OwedRows):
            # another activation: the same product and layout, the activation by name in its epilogue
            splits = K.whole_sum_splits(2 * self.spec.intermediate_size, self.spec.hidden_size, x.shape[0])
            K.gemm_skinny_gated(act, rows, self.gate_up.weight, self.spec.activation, splits)
        elif self.silu:
            K.swiglu(act, self.gate_up(plain_rows(x)), self.block)
        else:
            K.gated_act(act, self.gate_up(plain_rows(x)), self.spec.activation, self.block)
        return self.down.branch(act, getattr(ctx, "sink", None))


@register_feed_forward("dense")
class DenseFeedForward(Part):
    """down(act(up(x))), no gate, no biases.  `spec.activation`: "gelu" (the exact one, by erf),
    "gelu_tanh" or "silu"."""

    graph_safe = True

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        if spec.activation not in K.ACTIVATIONS:
            raise ValueError(f"activation '{spec.activation}' is not one of {', '.join(K.ACTIVATIONS)}")

    @property
    def graph_max_rows(self):
        return rows_a_graph_may_hold(self.dtype, self.spec.hidden_size, self.spec.intermediate_size)

    def tensors(self, prefix):
        s = self.spec
        return {prefix + s.up_name + s.weight_suffix: (s.intermediate_size, s.hidden_size),
                prefix + s.down_name + s.weight_suffix: (s.hidden_size, s.intermediate_size)}

    def bind(self, prefix, weights):
        s = self.spec
        self.up = Linear(self.matrix(weights[prefix + s.up_name + s.weight_suffix]))
        self.down = Linear(self.matrix(weights[prefix + s.down_name + s.weight_suffix]))

    def forward(self, ctx, x):
        """Up to 64 rows the activation runs in the up product's epilogue, on its float32 sums; above,
        the platform library's product is followed by the activation kernel."""
        x = plain_rows(x)
        if x.shape[0] and K.skinny_supported(x, self.up.weight):
            act = torch.empty((x.shape[0], self.spec.intermediate_size), dtype=x.dtype, device=x.device)
            splits = K.whole_sum_splits(self.spec.intermediate_size, self.spec.hidden_size, x.shape[0])
            K.gemm_skinny_act(act, x, self.up.weight, self.spec.activation, splits)
        else:
            act = self.up(x)
            K.activation(act, self.spec.activation)
        return self.down.branch(act, getattr(ctx, "sink", None))
