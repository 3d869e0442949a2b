"""Gated delta rule: a recurrent mixer with one state matrix per head and sequence.

For token t, value head h and its query/key head h // (heads / kv_heads), with x the
mixer's input (all of the recurrence in float32):

    q, k, v  = silu(conv(W_q x)), silu(conv(W_k x)), silu(conv(W_v x))    short causal
               convolutions over time, one filter a channel, zeros before the sequence
    q, k     = unit vectors per head (x / sqrt(sum x^2 + unit_eps)); q also / sqrt(key_dim)
    beta     = sigmoid(W_beta x)                                          one per head
    g        = exp(-exp(decay_log_rate) * softplus(W_decay x + decay_bias))
    S       <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q
    y        = W_o (o / sqrt(mean(o^2) + eps) * out_norm * silu(W_gate x))

The six input projections are one fused matrix [q | k | v | beta | decay | gate].  Per
sequence the cache holds one float32 row (`StateRequest`): S of every head, then the last
taps - 1 inputs of every convolved channel, so a prompt may arrive whole, in portions of
any size or token by token.  The row has two versions: a step reads one and writes the whole
other one, and the session makes that one current when the step is committed, so a failed
step costs nothing and no copy of the state is ever taken.  Kernels: `csrc/delta_rule.hip`.
"""
from __future__ import annotations

import torch

from ..csrc import lib
from ..weights.loader import ParamSpec
from .base import StateRequest
from .linear import Linear


class GatedDelta:
    @property
    def capture_safe(self):
        """Only this library's kernels, nothing allocated per step, what varies read from the
        step's metadata on the device: as long as its products say the same."""
        return self.proj.capture_safe and self.o.capture_safe

    @property
    def capture_rows(self):
        return min(self.proj.capture_rows, self.o.capture_rows)

    @classmethod
    def shape_of(cls, spec) -> lib.DeltaShape:
        return lib.DeltaShape(spec.n_heads, spec.n_kv_heads, spec.key_dim, spec.value_dim,
                              spec.conv_taps)

    @classmethod
    def parameters(cls, spec, hidden):
        taps = spec.conv_taps
        return {
            "q_proj.weight": ParamSpec((spec.qk_width, hidden)),
            "k_proj.weight": ParamSpec((spec.qk_width, hidden)),
            "v_proj.weight": ParamSpec((spec.v_width, hidden)),
            "q_conv.weight": ParamSpec((spec.qk_width, taps), scale=0.5),
            "k_conv.weight": ParamSpec((spec.qk_width, taps), scale=0.5),
            "v_conv.weight": ParamSpec((spec.v_width, taps), scale=0.5),
            "beta_proj.weight": ParamSpec((spec.n_heads, hidden)),
            "decay_proj.weight": ParamSpec((spec.n_heads, hidden)),
            "decay_log_rate": ParamSpec((spec.n_heads,), init="uniform", low=-3.0, high=0.5),
            "decay_bias": ParamSpec((spec.n_heads,), init="uniform", low=-4.0, high=0.0),
            "gate_proj.weight": ParamSpec((spec.v_width, hidden)),
            "out_norm.weight": ParamSpec((spec.value_dim,), init="norm"),
            "o_proj.weight": ParamSpec((hidden, spec.v_width)),
        }

    @classmethod
    def cache_request(cls, spec):
        # (S is a megabyte a layer and sequence at real sizes: two versions instead of copies)
        return StateRequest(shape=(cls.shape_of(spec).state_floats,), two_versions=True)

    @classmethod
    def kernel_libraries(cls, spec, dtype):
        return ("delta_rule", *Linear.kernel_libraries(dtype))

    @classmethod
    def check(cls, spec):
        if spec.n_heads < 1 or spec.n_kv_heads < 1 or spec.n_heads % spec.n_kv_heads:
            raise ValueError("gated_delta: n_heads must be a multiple of n_kv_heads")
        if not 1 <= spec.key_dim <= 256:
            raise ValueError(f"gated_delta: key_dim must lie in 1..256, got {spec.key_dim}")
        if spec.value_dim < 1:
            raise ValueError("gated_delta: value_dim must be positive")
        if not 1 <= spec.conv_taps <= 32:
            raise ValueError(f"gated_delta: conv_taps must lie in 1..32, got {spec.conv_taps}")

    def __init__(self, spec, hidden, params, dtype, device, positions=None):
        self.check(spec)
        self.spec = spec
        self.shape = self.shape_of(spec)
        fused = torch.cat([params[f"{name}.weight"] for name in
                           ("q_proj", "k_proj", "v_proj", "beta_proj", "decay_proj", "gate_proj")],
                          dim=0)
        self.proj = Linear(fused, dtype, device)
        self.o = Linear(params["o_proj.weight"], dtype, device)

        def f32(tensor):
            return tensor.to(device=device, dtype=torch.float32).contiguous()
        self.conv_w = f32(torch.cat([params["q_conv.weight"], params["k_conv.weight"],
                                     params["v_conv.weight"]], dim=0))
        self.decay_log_rate = f32(params["decay_log_rate"])
        self.decay_bias = f32(params["decay_bias"])
        self.out_norm = f32(params["out_norm.weight"])
        self.q_scale = float(spec.key_dim) ** -0.5

    def forward(self, ctx, x, entry):
        if not entry.writes_cache:
            raise ValueError("gated_delta: a run that only reads another run's state is not "
                             "implemented")
        shape, meta = self.shape, ctx.meta
        n = x.shape[0]
        state = ctx.cache.state(entry.cache)                 # [2 (slots + 1), state_floats]
        rows_in = meta.seq_state_in                          # a sequence's state, and the row
        rows_out = meta.seq_state_out                        # the step writes
        proj = self.proj.forward(ctx, x, "delta.proj")
        conv = ctx.buffer("delta.conv", (n, shape.channels), torch.float32)
        # a decode step (one row a sequence) renews the convolution's tails in the same kernel
        renew = ctx.decode and shape.taps <= lib.DELTA_FEW_TAPS
        lib.delta_conv(proj, self.conv_w, state, shape, meta.row_pos, meta.row_seq,
                       rows_in, rows_out, meta.seq_start, conv, renew_tail=renew)
        if not renew:
            lib.delta_tail(proj, state, shape, n, rows_in, rows_out, meta.seq_count,
                           meta.seq_row0)
        o_raw = ctx.buffer("delta.o_raw", (n, shape.v_width), torch.float32)
        lib.delta_rule(conv, proj, self.decay_log_rate, self.decay_bias, state, shape,
                       rows_in, rows_out, meta.seq_count, meta.seq_row0, o_raw, self.q_scale,
                       self.spec.unit_eps)
        ctx.release(conv)
        gated = ctx.buffer("delta.gated", (n, shape.v_width))
        lib.delta_out(o_raw, proj, self.out_norm, self.spec.out_norm_eps, shape, meta.row_seq,
                      gated)
        ctx.release(o_raw, proj)
        delta = self.o.forward(ctx, gated, "delta.o")
        ctx.release(gated)
        return delta
