"""Latent attention: causal attention whose keys and values are all made from one small row per position.

With h the mixer's input, H heads, per head `dim` plain and `rot` rotated query/key dims, values of `vdim`, a latent row
of `rank` values:

    q = W_q h                        per head [dim plain | rot rotated]
    [c_raw | kr_raw] = W_dkv h       rank + rot values
    c = rms_norm(c_raw) * w_c        the latent row;   kr = rotate(kr_raw), one rotated key part shared by all heads
    key of head n    = [W_uk[n] c | kr],   value of head n = W_uv[n] c
    score            = (q_plain . key_plain + rotate(q_rot) . kr) * scale          causal: position i sees j <= i
    weights          = exp(score) / (sum over j of exp(score) + exp(sink[n]))      the sink has no key and no value
    out              = W_o concat over n of sigmoid(W_g h)[n] * sum_j weights_j value_j

Only [c | kr] is kept, one row a position (a paged need without value pages; bfloat16 runs keep c a second time, transposed
inside a page, where the matrix-core kernel reads a latent column's keys side by side).  W_uk and W_uv never meet the kept rows:
since q_plain . (W_uk[n] c) = (W_uk[n]^T q_plain) . c and sum_j w_j W_uv[n] c_j = W_uv[n] sum_j w_j c_j, the query is carried
into the latent dims before the attention kernel and its result out of them after, both as small products per (token, head),
and the kernel attends over the rows as they are kept, all heads reading the same ones.  The gate, one number a head, is
applied to the latent sum inside the attention kernel.

q, dkv and g are one stacked product.  Norm, rotation, scores, weights and sums are float32 in every precision mode.
"""

from __future__ import annotations

import math

import torch

from ..kernels import ops
from .attention import GQAAttention
from .base import PagedKVNeed, Part, PartSpec, TensorSpec, create, length_class, register
from .linear import linear, materialize, rows_of


class LatentAttention(Part):
    graph_safe = True
    plan_safe = True
    can_overwrite = True        # forward(..., accumulate=False) stores its output
    wants_query_groups = True   # bfloat16 steps go to a kernel that walks groups of a request's consecutive tokens

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, rot_dim: int, value_dim: int, kv_rank: int, *,
                 position: PartSpec = PartSpec("none"), norm_eps: float = 1e-6, scale: float | None = None, sink: bool = False,
                 gate: bool = False, window: int | None = None):
        for name, value in (("hidden_size", hidden_size), ("num_heads", num_heads), ("head_dim", head_dim), ("value_dim", value_dim), ("kv_rank", kv_rank)):
            if value <= 0:
                raise ValueError(f"{name} must be positive, got {value}")
        if rot_dim < 0 or rot_dim % 2:
            raise ValueError(f"rot_dim must be even and not negative, got {rot_dim}")
        if scale is not None and (not math.isfinite(scale) or scale <= 0):
            raise ValueError(f"scale must be finite and positive, got {scale}")
        if window is not None and window <= 0:
            raise ValueError(f"window must be positive when given, got {window}")
        if norm_eps <= 0:
            raise ValueError(f"norm_eps must be positive, got {norm_eps}")
        self.hidden_size, self.num_heads, self.head_dim, self.rot_dim = hidden_size, num_heads, head_dim, rot_dim
        self.value_dim, self.kv_rank, self.norm_eps, self.window = value_dim, kv_rank, norm_eps, window
        self.position = create("position", position)
        if getattr(self.position, "rotary_dim", rot_dim) != rot_dim:
            raise ValueError(f"the position part rotates {self.position.rotary_dim} dims, the mixer's rotated part has {rot_dim}")
        self.scale = 1.0 / math.sqrt(head_dim + rot_dim) if scale is None else scale
        self.has_sink, self.has_gate = sink, gate
        self.w_in = self.w_uk = self.w_uv = self.w_o = self.latent_norm = self.sink = None

    # ------------------------------------------------------------------ weights
    @property
    def width(self) -> int:
        """Values kept per position."""
        return self.kv_rank + self.rot_dim

    def tensors(self):
        h, n, r = self.hidden_size, self.num_heads, self.kv_rank
        specs = {
            "q_proj.weight": TensorSpec((n * (self.head_dim + self.rot_dim), h)),
            "dkv_proj.weight": TensorSpec((self.width, h)),
            "dkv_norm.weight": TensorSpec((r,), role="norm"),
            "uk_proj.weight": TensorSpec((n * self.head_dim, r)),
            "uv_proj.weight": TensorSpec((n * self.value_dim, r)),
            "o_proj.weight": TensorSpec((h, n * self.value_dim)),
        }
        if self.has_sink:
            specs["sink"] = TensorSpec((n,), role="bias")
        if self.has_gate:
            specs["g_proj.weight"] = TensorSpec((n, h))
        return specs

    def bind(self, weights, dtype):
        n = self.num_heads
        stacked = [weights["q_proj.weight"], weights["dkv_proj.weight"]] + ([weights["g_proj.weight"]] if self.has_gate else [])
        w_in = torch.cat(stacked, 0).to(dtype)
        pad = -w_in.shape[0] % 16             # whole groups of 16 output columns suit every product kernel
        if pad:
            w_in = torch.cat((w_in, w_in.new_zeros(pad, self.hidden_size)), 0)
        self.w_in = w_in.contiguous()
        self.kv_col = n * (self.head_dim + self.rot_dim)
        self.gate_col = self.kv_col + self.width
        # a head's two small matrices: [outputs, inputs] for the matrix-core product of bfloat16 runs, [inputs, outputs] for the
        # float32 one, whose threads then read side by side
        w_uk = weights["uk_proj.weight"].to(dtype).reshape(n, self.head_dim, self.kv_rank)          # inputs: a head's plain dims
        w_uv = weights["uv_proj.weight"].to(dtype).reshape(n, self.value_dim, self.kv_rank)         # inputs: the latent dims
        self.by_outputs = dtype == torch.bfloat16
        self.w_uk = (w_uk.transpose(1, 2) if self.by_outputs else w_uk).contiguous()
        self.w_uv = (w_uv if self.by_outputs else w_uv.transpose(1, 2)).contiguous()
        # bfloat16 runs of shapes the matrix-core kernel takes keep the latent values a second time, transposed inside a page
        self.keeps_columns = dtype == torch.bfloat16 and self.kv_rank <= 512 and self.width % 8 == 0
        self.w_o = weights["o_proj.weight"].to(dtype).contiguous()
        self.latent_norm = weights["dkv_norm.weight"]
        self.sink = weights["sink"].float().contiguous() if self.has_sink else None

    def weight_bytes(self):
        return (self.w_in.numel() + self.w_uk.numel() + self.w_uv.numel() + self.w_o.numel()) * self.w_o.element_size()

    def flops(self, tokens, pairs):
        if self.window is not None:
            pairs = min(pairs, tokens * self.window)
        # the projections (the two per-head ones count their matrices once a token, as the others), then scores over the
        # kept rows and the weighted sum of their latent part, per pair and head
        return super().flops(tokens, pairs) + 2.0 * pairs * self.num_heads * (self.width + self.kv_rank)

    def cache_need(self):
        return PagedKVNeed(1, self.width, self.window, value_dim=self.kv_rank if getattr(self, "keeps_columns", False) else 0)

    # ------------------------------------------------------------------ forward
    def forward(self, ctx, x, residual, cache, then_norm=None, accumulate: bool = True):
        if cache is None:
            raise ValueError("latent attention needs a paged cache")
        t, n, r = rows_of(x), self.num_heads, self.kv_rank
        x = materialize(ctx, x)
        group = ctx.group(cache.group)
        proj = ctx.scratch("latent_proj", (t, self.w_in.shape[0]), ctx.dtype)
        linear(ctx, proj, x, self.w_in)
        tables = self.position.tables(ctx) if self.rot_dim else None
        cos, sin = tables if tables is not None else (None, None)
        queries = ctx.scratch("latent_queries", (t, n, self.width), ctx.dtype)
        fast = cache.v_pages is not None and ops.latent_attention_groups_takes(ctx.dtype, r, self.width, group.page_size)
        ops.latent_prep(proj, 0, self.kv_col, n, self.head_dim, self.rot_dim, r, self.latent_norm, self.norm_eps, cos, sin,
                        cache.k_pages, group.slots, queries, value_pages=cache.v_pages if fast else None)
        plain = proj[:, :self.kv_col].view(t, n, self.head_dim + self.rot_dim)[:, :, :self.head_dim]
        ops.head_gemm(queries[:, :, :r], plain, self.w_uk, transposed=not self.by_outputs)
        latent = ctx.scratch("latent_out", (t, n * r), ctx.dtype)
        gate = proj[:, self.gate_col:self.gate_col + n] if self.has_gate else None
        if fast:
            self._attend_groups(ctx, latent, queries, gate, cache, group)
        else:
            ops.latent_attention(latent, queries, cache.k_pages, group.block_table, ctx.token_slot, ctx.positions, r, self.scale,
                                 sink=self.sink, gate=gate, window=self.window or 0)
        heads_out = ctx.scratch("latent_heads_out", (t, n, self.value_dim), ctx.dtype)
        ops.head_gemm(heads_out, latent.view(t, n, r), self.w_uv, transposed=not self.by_outputs)
        return linear(ctx, residual, heads_out.view(t, n * self.value_dim), self.w_o, accumulate=accumulate, then_norm=then_norm)


    @staticmethod
    def _splits_alone(workgroups: int, longest: int) -> int:
        """Into how many workgroups the keys of a single token are divided: towards two workgroups a compute unit, at least
        64 keys each (two tiles; a power of two that follows the length's class, so that eager steps and graph replays agree);
        a workgroup walks its tiles one after the other, so a long context in few workgroups is a matter of latency."""
        units = ops.compute_units()
        if workgroups >= 2 * units:
            return 1
        return max(1, min(-(-2 * units // workgroups), length_class(longest) // 64, 64))

    def _attend_groups(self, ctx, latent, queries, gate, cache, group):
        """The matrix-core kernel: decode steps token by token, the single tokens at the head of a mixed step likewise, the
        rest by the step's query groups.  The keys of a group are divided between workgroups where the groups alone leave
        compute units idle, by the rules of the grouped-query kernels (a workgroup here is 64 (token, head) rows)."""
        t, n, r = latent.shape[0], self.num_heads, self.kv_rank
        window = self.window or 0
        tiles = -(-n // 64)

        def parts(name, rows, splits):
            if splits == 1:
                return None, None
            return (ctx.scratch(f"latent_{name}_o", (rows, n * splits * r), torch.float32), ctx.scratch(f"latent_{name}_ml", (rows, n * splits * 2), torch.float32))

        def alone(rows):
            longest = ctx.max_k if ctx.all_decode else ctx.max_k_bound
            if self.window is not None:
                longest = min(longest, self.window + 32)
            splits = self._splits_alone(rows * tiles, longest)
            part_o, part_ml = parts("single", rows, splits)
            ops.latent_attention_groups(latent[:rows], queries[:rows], cache.k_pages, cache.v_pages, group.block_table, ctx.token_slot, ctx.positions,
                                        None, None, 1, r, self.scale, sink=self.sink, gate=None if gate is None else gate[:rows], window=window,
                                        splits=splits, part_o=part_o, part_ml=part_ml)

        if ctx.all_decode:
            return alone(t)
        singles = ctx.single_rows
        if singles:
            alone(singles)
        rest = ctx.memo.get("rows_after_singles")
        if rest is None:
            rest = ctx.memo["rows_after_singles"] = (ctx.token_slot[singles:], ctx.positions[singles:])
        longest = ctx.max_k_bound if self.window is None else min(ctx.max_k_bound, self.window + 64)
        rows_a_group = ctx.max_qblock * n
        splits = GQAAttention._prefill_splits(ctx.num_qblocks * -(-rows_a_group // 64), longest, (t - singles) * n * r, 4, t - singles)
        part_o, part_ml = parts("group", t - singles, splits)
        ops.latent_attention_groups(latent[singles:], queries[singles:], cache.k_pages, cache.v_pages, group.block_table, rest[0], rest[1],
                                    ctx.qblock_token0, ctx.qblock_count, ctx.max_qblock, r, self.scale, sink=self.sink,
                                    gate=None if gate is None else gate[singles:], window=window, splits=splits, part_o=part_o, part_ml=part_ml)


register("mixer", "latent_attention", LatentAttention)
