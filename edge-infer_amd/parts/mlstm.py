"""Matrix memory with exponential gates (the mLSTM cell): a recurrent mixer with one state
matrix, one normaliser vector and one running maximum per head and sequence.

For token t and head a, with x the mixer's input, d the key size and c the gates' cap (the
gates and the whole recurrence in float32):

    q, k, v  = W_q x / sqrt(d), W_k x, W_v x
    i        = c tanh((w_i . x + b_i) / c)                      log input gate
    f        = logsigmoid(c tanh((w_f . x + b_f) / c))          log forget gate
    m_t      = max(f + m_{t-1}, i)                              m_0 = 0
    S_t      = e^(f + m_{t-1} - m_t) S_{t-1} + e^(i - m_t) k v^T      n_t alike, with k alone
    o        = S_t^T q / (max(|n_t . q|, e^(-m_t)) + bottom_eps)
    y        = W_o (o / sqrt(mean(o^2) + eps) per head * out_norm * sigmoid(W_g x))

The six input projections are one fused matrix [q | k | v | i | f | g]; the two gate biases go
to the kernel, which adds them in float32.  Per sequence the cache holds one float32 row
(`StateRequest`): per head S transposed, n and m, so a prompt may arrive whole, in portions of
any size or token by token.  The row has two versions: a step reads one and writes the whole
other one, and the session makes that one current when the step is committed.  Kernels:
`csrc/mlstm.hip`.
"""
from __future__ import annotations

import torch

from ..csrc import lib
from ..weights.loader import ParamSpec
from .base import StateRequest
from .linear import Linear


class MatrixMemory:
    @property
    def capture_safe(self):
        """Only this library's kernels, nothing allocated per step, what varies read from the
        step's metadata on the device: as long as its products say the same."""
        return self.proj.capture_safe and self.o.capture_safe

    @property
    def capture_rows(self):
        return min(self.proj.capture_rows, self.o.capture_rows)

    @classmethod
    def parameters(cls, spec, hidden):
        return {
            "q_proj.weight": ParamSpec((spec.qk_width, hidden)),
            "k_proj.weight": ParamSpec((spec.qk_width, hidden)),
            "v_proj.weight": ParamSpec((spec.v_width, hidden)),
            "in_gate.weight": ParamSpec((spec.n_heads, hidden)),
            "in_gate.bias": ParamSpec((spec.n_heads,), init="uniform", low=-1.0, high=1.0),
            "forget_gate.weight": ParamSpec((spec.n_heads, hidden)),
            "forget_gate.bias": ParamSpec((spec.n_heads,), init="uniform", low=1.0, high=4.0),
            "gate_proj.weight": ParamSpec((spec.v_width, hidden)),
            "out_norm.weight": ParamSpec((spec.v_width,), init="norm"),
            "o_proj.weight": ParamSpec((hidden, spec.v_width)),
        }

    @classmethod
    def cache_request(cls, spec):
        floats = lib.mlstm_state_floats(spec.n_heads, spec.key_dim, spec.value_dim)
        return StateRequest(shape=(floats,), two_versions=True)

    @classmethod
    def kernel_libraries(cls, spec, dtype):
        return ("mlstm", *Linear.kernel_libraries(dtype))

    @classmethod
    def check(cls, spec):
        if spec.n_heads < 1 or spec.value_dim < 1:
            raise ValueError("mlstm: heads and value_dim must be positive")
        if not 1 <= spec.key_dim <= 256:
            raise ValueError(f"mlstm: key_dim must lie in 1..256, got {spec.key_dim}")
        if not spec.gate_cap > 0:
            raise ValueError("mlstm: the cap of the gates must be positive")

    def __init__(self, spec, hidden, params, dtype, device, positions=None):
        self.check(spec)
        self.spec = spec
        fused = torch.cat([params[f"{name}.weight"] for name in
                           ("q_proj", "k_proj", "v_proj", "in_gate", "forget_gate", "gate_proj")],
                          dim=0)
        self.proj = Linear(fused, dtype, device)
        self.o = Linear(params["o_proj.weight"], dtype, device)

        def f32(tensor):
            return tensor.to(device=device, dtype=torch.float32).contiguous()
        self.in_bias = f32(params["in_gate.bias"])
        self.forget_bias = f32(params["forget_gate.bias"])
        self.out_norm = f32(params["out_norm.weight"])
        self.q_scale = float(spec.key_dim) ** -0.5

    def forward(self, ctx, x, entry):
        if not entry.writes_cache:
            raise ValueError("mlstm: a run that only reads another run's state is not implemented")
        spec, meta = self.spec, ctx.meta
        n = x.shape[0]
        state = ctx.cache.state(entry.cache)                 # [2 (slots + 1), state floats]
        proj = self.proj.forward(ctx, x, "mlstm.proj")
        o_raw = ctx.buffer("mlstm.o_raw", (n, spec.v_width), torch.float32)
        lib.mlstm_walk(proj, self.in_bias, self.forget_bias, state, meta.seq_state_in,
                       meta.seq_state_out, meta.seq_count, meta.seq_row0, o_raw, spec.n_heads,
                       spec.key_dim, spec.value_dim, spec.gate_cap, self.q_scale, spec.bottom_eps)
        gated = ctx.buffer("mlstm.gated", (n, spec.v_width))
        lib.mlstm_out(o_raw, proj, self.out_norm, spec.out_norm_eps, meta.row_seq, gated,
                      spec.n_heads, spec.key_dim, spec.value_dim)
        ctx.release(o_raw, proj)
        delta = self.o.forward(ctx, gated, "mlstm.o")
        ctx.release(gated)
        return delta
