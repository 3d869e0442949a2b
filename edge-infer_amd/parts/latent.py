"""Causal attention over a latent cache: per position one normed latent vector c [kv_rank],
from which every head's unrotated key and its value are up-projections, and one rotated key
part [rot_dim] that all heads share.  The cache holds nothing but c and that part.

With x the mixer's input, head a, W_uk,a [head_dim, kv_rank] and W_uv,a [value_dim, kv_rank]
the head's rows of the two up-projections:

    c_q      = rmsnorm(W_dq x) * w_dq                     the queries' latent
    q_a      = (W_uq c_q)_a = [q_plain (head_dim) | q_turn (rot_dim)]
    [c | t]  = W_dkv x;  c <- rmsnorm(c) * w_dkv;  t and q_turn are rotated by the position
    score    = (q_plain . W_uk,a c_j + q_turn . t_j) * scale
             = ((W_uk,a^T q_plain) . c_j + q_turn . t_j) * scale
    out_a    = W_uv,a (sum_j p_j c_j) * sigmoid(w_g,a . x)

so the up-projections never touch the cache: a head's query is carried into the latent's space
([W_uk,a^T q_plain | q_turn], kv_rank + rot_dim wide), attention runs with one shared "kv head"
whose key is the cached row [c | t] and whose value is that row's first kv_rank elements, and
the value up-projection is applied to the head's weighted sum of latents.  The softmax's
denominator may hold a learned sink per head.  Projections of x are one fused matrix
[dq | dkv | g].  Kernels: `csrc/head_ops.hip`; attention in bfloat16 on the matrix cores
(`csrc/attention_wide.hip`: cache rows a multiple of 32 wide, latents a multiple of 16),
otherwise, and in float32, `csrc/attention_generic.hip`.
"""
from __future__ import annotations

import numpy as np
import torch

from ..csrc import lib
from ..csrc.lib import PAGE_TOKENS
from ..weights.loader import ParamSpec
from .attention import MATRIX_CORE_ATTENTION, MAX_SLICES, _decode_items
from .base import KVRequest
from .linear import Linear


class LatentAttention:
    @property
    def capture_safe(self):
        return self.down.capture_safe and self.up_q.capture_safe and self.o.capture_safe

    @property
    def capture_rows(self):
        # (beyond the few-rows products' rows the per-head products are the library's as well)
        return min(self.down.capture_rows, self.up_q.capture_rows, self.o.capture_rows,
                   lib.SKINNY_ROWS)

    @classmethod
    def parameters(cls, spec, hidden):
        params = {
            "q_down.weight": ParamSpec((spec.q_rank, hidden)),
            "q_down_norm.weight": ParamSpec((spec.q_rank,), init="norm"),
            "q_up.weight": ParamSpec((spec.q_width, spec.q_rank), scale=0.1),
            "kv_down.weight": ParamSpec((spec.cache_width, hidden)),
            "kv_down_norm.weight": ParamSpec((spec.kv_rank,), init="norm"),
            "k_up.weight": ParamSpec((spec.n_heads * spec.head_dim, spec.kv_rank), scale=0.1),
            "v_up.weight": ParamSpec((spec.n_heads * spec.value_dim, spec.kv_rank), scale=0.1),
            "o_proj.weight": ParamSpec((hidden, spec.out_width)),
        }
        if spec.sink:
            params["sink"] = ParamSpec((spec.n_heads,), init="uniform", low=-1.0, high=1.0)
        if spec.output_gate:
            params["gate_proj.weight"] = ParamSpec((spec.n_heads, hidden))
        return params

    @classmethod
    def cache_request(cls, spec):
        # one row [latent | rotated key part] a position and no value pages: the values are the
        # row's first kv_rank elements
        return KVRequest(n_kv_heads=1, head_dim=spec.cache_width, value_dim=0)

    @classmethod
    def on_matrix_cores(cls, spec, dtype) -> bool:
        return MATRIX_CORE_ATTENTION and lib.attention_wide_supported(
            dtype, spec.cache_width, spec.cache_width, spec.kv_rank)

    @classmethod
    def kernel_libraries(cls, spec, dtype):
        attention = "attention_wide" if cls.on_matrix_cores(spec, dtype) else "attention_generic"
        return ("head_ops", attention, *Linear.kernel_libraries(dtype))

    @classmethod
    def check(cls, spec):
        if min(spec.n_heads, spec.head_dim, spec.value_dim, spec.kv_rank, spec.q_rank) < 1:
            raise ValueError("latent_attention: every size must be positive")
        if spec.rot_dim < 0 or spec.rot_dim % 2:
            raise ValueError("latent_attention: rot_dim must be even")
        if spec.rot_dim and (spec.position.kind != "rope_pairs" or spec.position.dim != spec.rot_dim):
            raise ValueError("latent_attention: the rotation is of neighbouring pairs over the "
                             "whole rotated part")
        if spec.cache_width > 1024 or spec.kv_rank > 512:
            raise ValueError("latent_attention: kv_rank may be 512 and kv_rank + rot_dim 1024 at "
                             f"most, got {spec.kv_rank} and {spec.cache_width}")

    def __init__(self, spec, hidden, params, dtype, device, positions):
        self.check(spec)
        self.spec = spec
        self.dtype = dtype
        H, d, r, e = spec.n_heads, spec.head_dim, spec.rot_dim, spec.value_dim
        fused = [params["q_down.weight"], params["kv_down.weight"]]
        if spec.output_gate:
            fused.append(params["gate_proj.weight"])
        self.down = Linear(torch.cat(fused, dim=0), dtype, device)
        self.up_q = Linear(params["q_up.weight"], dtype, device)
        self.o = Linear(params["o_proj.weight"], dtype, device)

        def f32(tensor):
            return tensor.to(device=device, dtype=torch.float32).contiguous()
        self.q_norm = f32(params["q_down_norm.weight"])
        self.c_norm = f32(params["kv_down_norm.weight"])
        # per head [in, out]: W_uk,a as stored is [head_dim, kv_rank]; W_uv,a is transposed
        self.k_up = params["k_up.weight"].to(device=device, dtype=dtype) \
            .reshape(H, d, spec.kv_rank).contiguous()
        self.v_up = params["v_up.weight"].to(device=device, dtype=dtype) \
            .reshape(H, e, spec.kv_rank).transpose(1, 2).contiguous()
        self.sinks = f32(params["sink"]) if spec.sink else None
        self.frequencies = positions(spec.position).frequencies if r else None
        self.scale = spec.scale if spec.scale is not None else float(d + r) ** -0.5
        self.compute_units = lib.compute_units(device)
        self.wide = self.on_matrix_cores(spec, dtype)
        self.positions_per_item = (lib.attention_wide_positions(H) if self.wide
                                   else lib.attention_positions_per_item(H))

    @property
    def plan_key(self):
        return ("latent_attention", self.positions_per_item, self.wide)

    def plan_step(self, plan):
        """Work items of the attention kernel, [3, items]: sequence, first row, positions."""
        if plan.decode:
            return {"attention.decode_items": _decode_items(plan.n_seqs, plan.n_live_seqs)}
        size = self.positions_per_item
        items = []
        for index, seq in enumerate(plan.seqs):
            for p0 in range(0, seq.count, size):
                npos = min(size, seq.count - p0)
                items.append((-(seq.start + p0 + npos), index, seq.row0 + p0, npos))
        items.sort()
        return {f"latent.items{size}": np.asarray([item[1:] for item in items],
                                                  dtype=np.int32).T.copy()}

    def decode_slices(self, n_seqs: int, context: int) -> int:
        """Slices of the key range in a decode step: enough blocks for about two a compute
        unit, never more than there are pages."""
        pages = max(1, (context + PAGE_TOKENS - 1) // PAGE_TOKENS)
        if self.wide:         # blocks of up to 64 heads, about two a compute unit
            blocks = n_seqs * ((self.spec.n_heads + 63) // 64)
            wanted = max(1, 2 * self.compute_units // blocks)
        else:
            blocks = n_seqs * ((self.spec.n_heads + 15) // 16)
            wanted = (2 * self.compute_units + blocks - 1) // blocks
        return max(1, min(wanted, pages, MAX_SLICES))

    def _per_head(self, ctx, x, matrices, y, x_head, x_first, y_head, y_first, name):
        """y[n, h, y_first ..] = x[n, h, x_first ..] . matrices[h]: the library's batched product
        for the many rows of a bfloat16 prompt step (as the framework's other products of many
        rows), this package's kernel otherwise."""
        heads, inner, outer = matrices.shape
        rows = y.shape[0]
        if self.dtype == torch.bfloat16 and rows > lib.SKINNY_ROWS and x.dim() == 2:
            taken = x.view(rows, heads, x_head)[:, :, x_first:x_first + inner].transpose(0, 1)
            made = ctx.buffer(name, (heads, rows, outer))
            torch.bmm(taken, matrices, out=made)
            y.view(rows, heads, y_head)[:, :, y_first:y_first + outer].copy_(made.transpose(0, 1))
            ctx.release(made)
        else:
            lib.head_matmul(x, matrices, y, heads, x_head=x_head, x_first=x_first, y_head=y_head,
                            y_first=y_first)

    def forward(self, ctx, x, entry):
        spec, meta = self.spec, ctx.meta
        H, d, r, rank = spec.n_heads, spec.head_dim, spec.rot_dim, spec.kv_rank
        n = x.shape[0]
        group_index, k_pages, _ = ctx.cache.kv(entry.cache)
        page_table = meta.page_table(group_index)
        n_gate = H if spec.output_gate else 0

        down = self.down.forward(ctx, x, "latent.down")
        q_latent = ctx.buffer("latent.cq", (n, spec.q_rank))
        gate = ctx.buffer("latent.gate", (n, H), torch.float32) if n_gate else None
        lib.latent_down_store(down, self.q_norm, self.c_norm, spec.norm_eps, self.frequencies,
                              meta.row_pos, meta.row_seq, page_table, q_latent, k_pages, gate,
                              spec.q_rank, rank, r, n_gate, write_cache=entry.writes_cache)
        ctx.release(down)
        q = self.up_q.forward(ctx, q_latent, "latent.q")
        ctx.release(q_latent)
        # the queries in the latent's space: [W_uk^T q_plain | rotated q_turn] a head
        q_wide = ctx.buffer("latent.q_wide", (n, H * spec.cache_width))
        self._per_head(ctx, q, self.k_up, q_wide, d + r, 0, spec.cache_width, 0, "latent.q_made")
        if r:
            lib.rotate_pairs(q, self.frequencies, meta.row_pos, q_wide, H, r, x_head=d + r,
                             x_first=d, y_head=spec.cache_width, y_first=rank)
        ctx.release(q)
        mixed = ctx.buffer("latent.mixed", (n, H * rank))
        common = dict(window=None, scale=self.scale, value_dim=rank, sinks=self.sinks,
                      values_in_keys=True, gate=gate)
        part_o = part_ml = None
        if ctx.decode:
            splits = self.decode_slices(ctx.n_seqs, ctx.context_bound)
            if splits > 1:
                part_o = ctx.buffer("latent.part_o", (n * H * splits * rank,), torch.float32)
                part_ml = ctx.buffer("latent.part_ml", (n * H * splits * 2,), torch.float32)
            section = meta.section("attention.decode_items")
            common.update(n_splits=splits, part_o=part_o, part_ml=part_ml)
        else:
            section = meta.section(f"latent.items{self.positions_per_item}")
        count = section.numel() // 3
        kernel = lib.attention_wide if self.wide else lib.attention
        kernel(q_wide, k_pages, None, section[:count], section[count:2 * count],
               section[2 * count:], count, meta.row_pos, meta.row_seq, page_table, mixed,
               H, 1, spec.cache_width, **common)
        ctx.release(q_wide, gate, part_o, part_ml)
        out = ctx.buffer("latent.out", (n, spec.out_width))
        self._per_head(ctx, mixed, self.v_up, out, rank, 0, spec.value_dim, 0, "latent.v_made")
        ctx.release(mixed)
        delta = self.o.forward(ctx, out, "latent.o")
        ctx.release(out)
        return delta
