"""The gated delta rule: a recurrent mixer that keeps, per request, one matrix per head and the
last inputs of its short convolutions, instead of keys and values per token.

Per token, with h the mixer's input:  q = W_q h and k = W_k h (G heads of D), v = W_v h (H heads
of V); each passes a causal convolution over time (one filter per channel) and SiLU; q and k
become unit vectors per head (q also times D^-1/2); beta = sigmoid(W_b h) and
decay = exp(-exp(A_log) * softplus(W_a h + dt_bias)), one of each per head.  Head j, which reads
q/k head j // (H / G), then moves its state S [D, V] on:

    S <- decay S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q

and o is divided by its root mean square over V, multiplied by a weight shared by the heads and by
silu(W_g h), and projected out by W_o.

The six projections are one product over concatenated weights.  The state (the matrices, and the
last taps - 1 inputs of the convolutions) lives in the cache manager's per-request slots as two
named float32 tensors; a request's slot is zeroed when it is taken, which is the design's start
state.  Everything after the projections runs in float32 inside `kernels.lib.delta_rule_step`.
The mixer keeps nothing per token, so a model made of such mixers alone needs no pages.
"""

from __future__ import annotations

import torch

from ..cache.manager import StateSpec
from ..kernels import lib as K
from .base import Part, ScaleShape, StepShape, plain_rows, register_mixer
from .linear import Linear, rows_a_graph_may_hold

SEQ_RUNS = "runs of the step's sequences"


def sequence_runs(shape: StepShape):
    """For every sequence of the step (first flat row, rows, tokens held before the step, 0)."""
    return {"runs": ([x for start, n, past in zip(shape.q_starts, shape.q_lens, shape.past_lens)
                      for x in (start, n, past, 0)], 4)}


@register_mixer("gated_delta")
class GatedDeltaMixer(Part):
    graph_safe = True

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        if spec.num_heads % spec.num_kv_heads:
            raise ValueError(f"{spec.num_heads} value heads over {spec.num_kv_heads} query/key heads")
        if not 0 < spec.key_dim <= 1024:
            raise ValueError(f"key_dim {spec.key_dim}: the recurrence kernel takes up to 1024")
        if not 1 <= spec.conv_taps <= 64:
            raise ValueError(f"conv_taps {spec.conv_taps} is outside 1..64")
        if not 0 < spec.value_dim <= 1024:
            raise ValueError(f"value_dim {spec.value_dim}: the kernels take up to 1024")

    @property
    def channels(self) -> int:
        s = self.spec
        return 2 * s.num_kv_heads * s.key_dim + s.num_heads * s.value_dim

    @property
    def graph_max_rows(self):
        s = self.spec
        return rows_a_graph_may_hold(self.dtype, s.hidden_size, s.num_heads * s.value_dim)

    def state_spec(self):
        s = self.spec
        return (StateSpec((s.num_heads, s.value_dim, s.key_dim), torch.float32, "matrices"),
                StateSpec((s.conv_taps - 1, self.channels), torch.float32, "conv_tail"))

    def step_lists_key(self, block_size: int):
        return SEQ_RUNS

    def step_lists(self, shape: StepShape):
        return sequence_runs(shape)

    def _projections(self):
        """(name, rows) of the six projections in the order of the product's columns."""
        s = self.spec
        qk, hv = s.num_kv_heads * s.key_dim, s.num_heads * s.value_dim
        return ((s.q_name, qk), (s.k_name, qk), (s.v_name, hv), (s.gate_name, hv), (s.beta_name, s.num_heads),
                (s.decay_name, s.num_heads))

    def tensors(self, prefix):
        s = self.spec
        out = {prefix + name + s.weight_suffix: (rows, s.hidden_size) for name, rows in self._projections()}
        for name, rows in self._projections()[:3]:
            out[prefix + name + s.conv_suffix] = (rows, s.conv_taps)
        out[prefix + s.a_log_name] = (s.num_heads,)
        out[prefix + s.dt_bias_name] = (s.num_heads,)
        out[prefix + s.norm_name] = ScaleShape((s.value_dim,))
        out[prefix + s.o_name + s.weight_suffix] = (s.hidden_size, s.num_heads * s.value_dim)
        return out

    def bind(self, prefix, weights):
        s = self.spec
        self.proj = Linear(self.matrix(torch.cat([weights[prefix + name + s.weight_suffix]
                                                  for name, _ in self._projections()], dim=0)))
        f32 = dict(device=self.device, dtype=torch.float32)
        # what enters the recurrence is float32 whatever it is stored in
        self.conv = torch.cat([weights[prefix + name + s.conv_suffix] for name, _ in self._projections()[:3]],
                              dim=0).to(**f32).contiguous()
        self.a_log = weights[prefix + s.a_log_name].to(**f32).contiguous()
        self.dt_bias = weights[prefix + s.dt_bias_name].to(**f32).contiguous()
        self.norm = self.vector(weights[prefix + s.norm_name])
        self.out = Linear(self.matrix(weights[prefix + s.o_name + s.weight_suffix]))

    def forward(self, ctx, x):
        s = self.spec
        if not ctx.writes_cache:
            raise ValueError("a recurrent mixer cannot borrow another stop's state")
        x = plain_rows(x)
        proj = self.proj(x)
        state = ctx.cache.state_of(ctx.cache_entry)
        runs = ctx.memo[SEQ_RUNS]["runs"]
        out = torch.empty((x.shape[0], s.num_heads * s.value_dim), dtype=x.dtype, device=x.device)
        K.delta_rule_step(proj, out, ctx.tok_seq, ctx.positions, runs, ctx.slots, self.conv, state["conv_tail"],
                          state["matrices"], self.a_log, self.dt_bias, self.norm, s.num_kv_heads, s.num_heads,
                          s.key_dim, s.value_dim, s.conv_taps, s.unit_eps, s.norm_eps)
        return self.out.branch(out, ctx.sink)
