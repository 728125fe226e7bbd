"""Grouped-query softmax attention over a paged cache (the mixer of this architecture).

    qkv = h @ qkv_w^T;  q, k <- per-head norm (optional), rotation (optional)
    k, v -> cache pages at the tokens' slots, written before attending
    o = softmax(q k^T * scale over the keys a query may see) v;  out = o @ o_w^T

(reference atomserve/model.py:292-336).  Every size, the scale, the window, the norm
and the position encoding arrive through the spec.  A run that only reads another
run's cache computes q alone and stores nothing.
"""

import torch

from atomserve_amd.kernels import ops
from atomserve_amd.parts.base import GatedDelta, Mixer, PagedCacheRequest, PendingNorm, SplitSums, WeightDecl, build, register

# Rows with at most SHORT_ROW new tokens are attended as that many single queries
# (reference atomserve/runner.py:31-34); longer rows go through the prefill kernel in work items of
# TILE_Q consecutive queries.  The step's batch sorts its rows so because this mixer asks for it.
SHORT_ROW = 8
TILE_Q = ops.PREFILL_TILE_QUERIES


class Attention(Mixer):
    takes_pending_norm = True
    adds_to_residual = True

    @property
    def capturable(self) -> bool:
        return self.position is None or self.position.capturable

    def __init__(self, spec, env):
        super().__init__(spec, env)
        s = spec
        if s.num_heads % s.num_kv_heads:
            raise ValueError(f"{s.num_heads} query heads do not divide over {s.num_kv_heads} kv heads")
        chunk = 4 if env.dtype == torch.float32 else 8
        if s.head_dim % chunk or s.head_dim > ops.SINGLE_QUERY_MAX_HEAD_DIM:
            raise ValueError(
                f"head_dim {s.head_dim} is not supported by the attention kernels "
                f"(a multiple of {chunk}, at most {ops.SINGLE_QUERY_MAX_HEAD_DIM})"
            )
        # What the kernels compute and nothing else: a per-head RMSNorm, and a rotation of the pairs
        # (i, i + R/2) of a head's first R coordinates by angles that the position part tabulates.
        if s.qk_norm is not None and s.qk_norm.kind != "rmsnorm":
            raise ValueError(f"the attention kernels norm heads by 'rmsnorm' only, not by {s.qk_norm.kind!r}")
        if s.qk_norm is not None and s.qk_norm.size != s.head_dim:
            raise ValueError(f"the per-head norm has {s.qk_norm.size} gains, a head {s.head_dim} coordinates")
        self.position = build("position", s.position, env) if s.position is not None else None
        if self.position is not None and getattr(self.position, "pairs", None) != "half":
            raise ValueError(
                f"the attention kernels rotate the pairs (i, i + R/2) by a table of cosines and sines "
                f"(a position part that declares pairs = 'half'); {s.position.kind!r} declares "
                f"{getattr(self.position, 'pairs', None)!r}"
            )
        self.q_norm_weight = self.k_norm_weight = None

    def weight_decls(self) -> dict:
        s = self.spec
        decls = {
            "qkv.weight": WeightDecl(((s.num_heads + 2 * s.num_kv_heads) * s.head_dim, s.hidden_size)),
            "o.weight": WeightDecl((s.hidden_size, s.num_heads * s.head_dim)),
        }
        if s.qk_norm is not None:
            decls["q_norm.weight"] = WeightDecl((s.head_dim,), role="vector")
            decls["k_norm.weight"] = WeightDecl((s.head_dim,), role="vector")
        return decls

    def bind(self, tensors: dict) -> None:
        super().bind(tensors)
        # what the products of a decode step stream: the matrices with their copies in wave order
        self.qkv = ops.Streamed(self.qkv_weight, self.env.stream_copies)
        self.o = ops.Streamed(self.o_weight, self.env.stream_copies)

    def streamed(self) -> list:
        return [self.qkv, self.o]

    def cache_request(self):
        s = self.spec
        return PagedCacheRequest(s.num_kv_heads, s.head_dim, s.window)

    def row_split(self):
        return (SHORT_ROW, TILE_Q)

    def forward(self, h, step, cache, residual=None, next_norm=None):
        """h [T, hidden] compute dtype (or the norm left pending on the stream) -> [T, hidden], or the
        pending `next_norm` after adding the output into `residual`.  cache: a PagedLayerView (pages
        of this run's cache, its group's slots and block tables for this step, whether to store)."""
        s, env = self.spec, self.env
        pending = isinstance(h, PendingNorm)
        T, device = (h.x.shape[0], h.x.device) if pending else (h.shape[0], h.device)
        H, KV, D = s.num_heads, s.num_kv_heads, s.head_dim
        qkv = torch.empty((T, (H + 2 * KV) * D), dtype=env.dtype, device=device)
        if pending:
            h.gemm(self.qkv, qkv)
        else:
            ops.gemm(h, self.qkv, qkv, env.products)
        cos_sin = self.position.prepare(step) if self.position is not None else None
        eps = s.qk_norm.eps if s.qk_norm is not None else 0.0
        rotary = 2 * cos_sin.shape[1] if cos_sin is not None else 0
        if step.decode_only and ops.attn_decode_fresh_supported(env.dtype, H, KV, D, cache.block_size, rotary,
                                                                s.qk_norm is not None):  # fmt: skip
            # a decode step: norm, rotation, the cache store and attention in one kernel
            out = torch.empty((T, H, D), dtype=env.dtype, device=device)
            ops.attn_decode_fresh(
                qkv.view(T, H + 2 * KV, D), self.q_norm_weight, self.k_norm_weight, cos_sin, cache.slots, eps,
                cache.writes, cache.k_pages, cache.v_pages, step.positions, cache.block_tables, out, H, s.scale,
                s.window, step.max_context, order=step.all_tokens,
            )  # fmt: skip
        else:
            q = torch.empty((T, H, D), dtype=env.dtype, device=device)
            ops.qk_norm_rope_store(
                qkv.view(T, H + 2 * KV, D), self.q_norm_weight, self.k_norm_weight, cos_sin, cache.slots, q,
                cache.k_pages, cache.v_pages, H, KV, eps, store_kv=cache.writes,
            )  # fmt: skip
            out = torch.empty((T, H, D), dtype=env.dtype, device=device)
            self.attend(q, out, step, cache)
        if residual is not None and next_norm is not None:
            link = next_norm.absorb(out.view(T, H * D), self.o, residual)
            if link is not None:
                return link
            if next_norm.takes_split_sums:
                plan = ops.gemm_split_plan(T, s.hidden_size, out.view(T, H * D).shape[1], env.dtype)
                if plan is not None:
                    return SplitSums(ops.gemm_split(out.view(T, H * D), self.o, plan))
        y = torch.empty((T, s.hidden_size), dtype=env.dtype, device=device)
        ops.gemm(out.view(T, H * D), self.o, y, env.products)
        return y

    def attend(self, q, out, step, cache) -> None:
        attend(q, out, step, cache, self.spec.scale, self.spec.window, self.row_split())


def attend(q, out, step, cache, scale: float, window: int, split) -> None:
    """Attention of a step's queries q [T, H, D] over the pages of `cache` (which hold the step's own keys
    already) into out [T, H, D]; `split`: the (short, tile) under which the step sorted its rows for this."""
    # fp32, and shapes the prefill kernel does not take: every token is a single query.
    # Otherwise short rows are single queries and long rows go through the prefill kernel.
    if step.decode_only:  # token t is row t: the kernels need no maps from one to the other
        ops.attn_single_query(q, cache.k_pages, cache.v_pages, step.all_tokens, step.positions, None,
                              cache.block_tables, out, scale, window, step.max_context)  # fmt: skip
        return
    if not ops.attn_prefill_supported(q.dtype, q.shape[2], cache.block_size):
        ops.attn_single_query(q, cache.k_pages, cache.v_pages, step.all_tokens, step.positions, step.tok_row,
                              cache.block_tables, out, scale, window, step.max_context)  # fmt: skip
        return
    rows = step.split(split)
    if rows.num_short_tokens:
        ops.attn_single_query(q, cache.k_pages, cache.v_pages, rows.short_tokens, step.positions, step.tok_row,
                              cache.block_tables, out, scale, window, rows.max_short_context)  # fmt: skip
    if rows.num_long_tiles:
        ops.attn_prefill(q, cache.k_pages, cache.v_pages, rows.long_tiles, cache.block_tables, out, scale,
                         window, step.max_context, tile_keys=rows.tile_keys)  # fmt: skip


register("mixer", "attention", Attention)


class MixedHeadsAttention(Mixer):
    """Softmax attention whose heads see each other's scores:

        q = W_q h,  k = W_k h,  v = k as projected (spec.values "keys") or W_v h ("own")
        q, k turned by the position part (their first R coordinates, pairs (i, i + R/2)); v never
        raw_g = scale q_g . k_kv(g);  s_h = sum_g M[h, g] raw_g  (spec.mix_heads)
        j visible from i: j <= i and (i - j < window or j < keep_first)   (window 0: every j <= i)
        out = W_o [softmax(s_h) v_kv(h)]_h

    q, k (v) and, with spec.out_gate, the logits of the output gate are rows of one input matrix.  A workgroup
    of the kernel owns all heads of up to `tile` consecutive queries; single tokens are items of one query."""

    def __init__(self, spec, env):
        super().__init__(spec, env)
        s = spec
        if s.num_heads % s.num_kv_heads:
            raise ValueError(f"{s.num_heads} query heads do not divide over {s.num_kv_heads} kv heads")
        if s.values not in ("keys", "own"):
            raise ValueError(f"values are 'keys' or 'own', not {s.values!r}")
        self.position = build("position", s.position, env) if s.position is not None else None
        if self.position is not None and getattr(self.position, "pairs", None) != "half":
            raise ValueError(f"the kernel turns the pairs (i, i + R/2) by a table of cosines and sines; "
                             f"{s.position.kind!r} declares {getattr(self.position, 'pairs', None)!r}")  # fmt: skip
        if s.position is not None and s.position.rotary_dim > s.head_dim:
            raise ValueError(f"{s.position.rotary_dim} turned coordinates in a head of {s.head_dim}")
        self.padded_dim = -(-s.head_dim // 8) * 8  # what the kernel reads 16 bytes at a time; the rest is zero
        self.tile = ops.attn_headmix_rows(s.num_heads, s.num_kv_heads, self.padded_dim, env.dtype)
        if self.tile < 1:
            raise ValueError(f"{s.num_heads} heads of {s.head_dim} are more than the mixed-heads kernel keeps at once")
        self.kv_rows = s.num_kv_heads * s.head_dim
        self.gate_off = s.num_heads * s.head_dim + (1 if s.values == "keys" else 2) * self.kv_rows
        self.mix_f32 = None

    @property
    def capturable(self) -> bool:
        return self.position is None or self.position.capturable

    def weight_decls(self) -> dict:
        s = self.spec
        decls = {
            "in.weight": WeightDecl((self.gate_off + (s.hidden_size if s.out_gate else 0), s.hidden_size)),
            "o.weight": WeightDecl((s.hidden_size, s.num_heads * s.head_dim)),
        }
        if s.mix_heads:
            decls["mix"] = WeightDecl((s.num_heads, s.num_heads))
        if s.out_gate:
            decls["gate_bias"] = WeightDecl((s.hidden_size,), role="vector")
        return decls

    def bind(self, tensors: dict) -> None:
        super().bind(tensors)
        self.win = ops.Streamed(self.in_weight, self.env.stream_copies)
        self.o = ops.Streamed(self.o_weight, self.env.stream_copies)
        if self.spec.mix_heads:
            self.mix_f32 = self.mix.float().contiguous()  # exact: what the file holds in 16 bits widens

    def streamed(self) -> list:
        return [self.win, self.o]

    def cache_request(self):
        s = self.spec
        return PagedCacheRequest(s.num_kv_heads, self.padded_dim, s.window, s.keep_first if s.window > 0 else 0)

    def row_split(self):
        return (1, self.tile)

    def forward(self, h, step, cache):
        s, env = self.spec, self.env
        T, dev = h.shape[0], h.device
        H, KV, D, Dp = s.num_heads, s.num_kv_heads, s.head_dim, self.padded_dim
        proj = torch.empty((T, self.in_weight.shape[0]), dtype=env.dtype, device=dev)
        ops.gemm(h, self.win, proj, env.products)
        cos_sin = self.position.prepare(step) if self.position is not None else None
        q = torch.empty((T, H, Dp), dtype=env.dtype, device=dev)
        k_off = H * D
        v_off = k_off if s.values == "keys" else k_off + self.kv_rows
        ops.head_norm_store(proj, 0, k_off, v_off, H, KV, D, D, None, None, 0.0, cache.slots, q, cache.k_pages,
                            cache.v_pages, store_kv=cache.writes, cos_sin=cos_sin)  # fmt: skip
        out = torch.empty((T, H, D), dtype=env.dtype, device=dev)
        args = (cache.block_tables, self.mix_f32, out, s.scale, s.window, s.keep_first)
        if step.decode_only:  # token t is row t
            ops.attn_headmix(q, cache.k_pages, cache.v_pages, step.all_tokens, 1, step.positions, None, *args,
                             max_context=step.max_context)  # fmt: skip
        else:
            rows = step.split(self.row_split())
            if rows.num_short_tokens:
                ops.attn_headmix(q, cache.k_pages, cache.v_pages, rows.short_tokens, 1, step.positions, step.tok_row, *args,
                                 max_context=rows.max_short_context)  # fmt: skip
            if rows.num_long_tiles:
                ops.attn_headmix(q, cache.k_pages, cache.v_pages, rows.long_tiles, self.tile, None, None, *args,
                                 max_context=step.max_context)  # fmt: skip
        y = torch.empty((T, s.hidden_size), dtype=env.dtype, device=dev)
        ops.gemm(out.view(T, H * D), self.o, y, env.products)
        if s.out_gate:
            return GatedDelta(y, proj, self.gate_off, self.gate_bias)
        return y


register("mixer", "mixed_heads_attention", MixedHeadsAttention)
