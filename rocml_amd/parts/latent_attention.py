"""Softmax attention whose keys and values are expanded from one small latent vector per position.

Per token the layer projects its input ``h`` to a query latent ``c_q = norm(W_dq h)``, a
key/value latent ``c = norm(W_dkv h)[:kv_rank]`` and one rotated key part ``k_r`` that all heads
share; head ``a`` then has ``q_a = W_uq,a c_q = [q_a^n, q_a^r]`` (the second part rotated),
``k_a(j) = [W_uk,a c_j, k_r(j)]`` and ``v_a(j) = W_uv,a c_j``.  The cache holds ``[c_j, k_r(j)]``
and nothing per head.  The attention never expands the keys: since

    q_a^n . (W_uk,a c_j) = (W_uk,a^T q_a^n) . c_j        and
    sum_j p_j W_uv,a c_j = W_uv,a (sum_j p_j c_j),

every head asks one shared key/value "head" whose keys are the cache rows ``[c_j, k_r(j)]`` and
whose values are the first ``kv_rank`` numbers of the same rows, with the query
``[W_uk,a^T q_a^n, q_a^r]``; the head's output is ``W_uv,a`` times what the attention returns.
Both small products run once per token and head, whatever the number of keys.  Long prompt steps in
bfloat16 take the other road (``_expanded_prompt``): keys and values per head, expanded for the
positions the step sees, which costs a third of the operations per (query, key) pair at the usual
sizes; the cache is the same rows either way.

Launches of a step: one product for the three projections of ``h`` (query latent, key/value
latent with its rotated part, output gate), one kernel that norms both latents, rotates and
appends to the cache, the product ``W_uq``, the rotation of the queries' rotated parts, the
per-head products with ``W_uk^T``, the attention, the per-head products with ``W_uv`` (the gate is
their epilogue in bfloat16), and the output product whose epilogue is the residual sum.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .. import ops
from ..config.spec import LatentAttentionSpec
from ..errors import ConfigError
from .base import BuildContext, LatentCacheRequest, Mixer, ParamSpec
from .registry import build_position, register_mixer
from .residual import stream


class LatentAttention(Mixer):
    adds_only = True
    # A prompt step of at least so many tokens expands keys and values per head for the positions its
    # queries see and runs the attention kernels for separate heads: a (query, key) pair then costs
    # 2 (head_dim + rot_dim) + 2 v_head_dim operations instead of 2 (kv_rank + rot_dim) + 2 kv_rank.
    EXPANDED_PROMPT_MIN_TOKENS = 256

    def __init__(self, spec: LatentAttentionSpec, ctx: BuildContext):
        for norm in (spec.q_norm, spec.kv_norm):
            if norm.kind != "rmsnorm" or getattr(norm, "unit_offset", False):
                # the latents are normed inside the kernel that appends to the cache, which knows one kind
                raise ConfigError("the latents' norms must be plain root-mean-square norms")
        if spec.q_norm.size != spec.q_rank or spec.kv_norm.size != spec.kv_rank:
            raise ConfigError("the latents' norms must span the latents")
        if spec.q_norm.eps != spec.kv_norm.eps:
            raise ConfigError("the two latent norms share one eps")
        if spec.window is not None and spec.window <= 0:
            raise ConfigError(f"window must be positive, got {spec.window}")
        self.spec = spec
        self.dtype = ctx.dtype
        self.position = build_position(spec.position, ctx)
        if getattr(self.position, "pairing", "halves") != "halves" or self.position.rot_dim > spec.rot_dim:
            raise ConfigError("the rotated part turns in pairs (i, i + n/2) of its first n numbers, n at most its size")
        self.graph_safe = getattr(self.position, "graph_safe", True)
        self.prompt_graph_safe = self.graph_safe and getattr(self.position, "prompt_graph_safe", False)
        self.qk_dim = spec.head_dim + spec.rot_dim             # a head's query as the projection gives it
        self.row = spec.kv_rank + spec.rot_dim                 # a cache row, and a head's query as the attention takes it
        self.o_dim = spec.n_heads * spec.v_head_dim
        # columns of the first projection: query latent, key/value latent, rotated key part, gate
        self.first_cols = spec.q_rank + self.row + (self.o_dim if spec.gate else 0)
        self.w_first: Optional[torch.Tensor] = None
        self.w_uq: Optional[torch.Tensor] = None
        self.w_uk_t: Optional[torch.Tensor] = None
        self.w_uv: Optional[torch.Tensor] = None
        self.w_o: Optional[torch.Tensor] = None
        self.q_gain: Optional[torch.Tensor] = None
        self.kv_gain: Optional[torch.Tensor] = None
        self.w_expand: Optional[torch.Tensor] = None
        self._ident = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        s = self.spec
        specs = {"dq.weight": ParamSpec((s.q_rank, s.hidden)),
                 "dq_norm.weight": ParamSpec((s.q_rank,), role="gain", init="gain"),
                 "uq.weight": ParamSpec((s.n_heads * self.qk_dim, s.q_rank)),
                 "dkv.weight": ParamSpec((self.row, s.hidden)),
                 "dkv_norm.weight": ParamSpec((s.kv_rank,), role="gain", init="gain"),
                 "uk.weight": ParamSpec((s.n_heads * s.head_dim, s.kv_rank)),
                 "uv.weight": ParamSpec((self.o_dim, s.kv_rank)),
                 "o_proj.weight": ParamSpec((s.hidden, self.o_dim))}
        if s.gate:
            specs["g.weight"] = ParamSpec((self.o_dim, s.hidden))
        return specs

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        s = self.spec
        first = [tensors["dq.weight"], tensors["dkv.weight"]] + ([tensors["g.weight"]] if s.gate else [])
        self.w_first = torch.cat(first, dim=0).contiguous()
        self.w_uq = tensors["uq.weight"]
        # per head [kv_rank, head_dim]: the transposed key expansion, applied to the queries
        self.w_uk_t = tensors["uk.weight"].view(s.n_heads, s.head_dim, s.kv_rank).transpose(1, 2).contiguous()
        self.w_uv = tensors["uv.weight"].view(s.n_heads, s.v_head_dim, s.kv_rank).contiguous()
        self.w_o = tensors["o_proj.weight"]
        self.q_gain = tensors["dq_norm.weight"]
        self.kv_gain = tensors["dkv_norm.weight"]
        if self._expandable():
            # One matrix that turns a cache row [c, k_r] into every head's key [W_uk,a c, k_r] and value
            # [W_uv,a c, zeros up to the key's size]: rows of W_uk and W_uv against c, an identity against k_r.
            D, H = self.qk_dim, s.n_heads
            w = torch.zeros((2 * H, D, self.row), dtype=self.dtype, device=self.w_o.device)
            w[:H, :s.head_dim, :s.kv_rank] = tensors["uk.weight"].view(H, s.head_dim, s.kv_rank)
            w[:H, s.head_dim:, s.kv_rank:] = torch.eye(s.rot_dim, dtype=self.dtype, device=w.device)
            w[H:, :s.v_head_dim, :s.kv_rank] = tensors["uv.weight"].view(H, s.v_head_dim, s.kv_rank)
            self.w_expand = w.view(2 * H * D, self.row).contiguous()

    def _expandable(self) -> bool:
        """Whether prompts may take the expanded form: bfloat16, a head (unrotated and rotated part) of a
        size the matrix-core attention kernels know, values no wider than that."""
        return (self.dtype == torch.bfloat16 and self.qk_dim in ops.PREFILL_FUSED_HEAD_DIMS
                and self.spec.v_head_dim <= self.qk_dim and self.row % 8 == 0)

    def matrix_elements(self) -> int:
        # (the expansion matrix is built from uk and uv: no parameters of its own)
        return super().matrix_elements()

    def flops(self, new_counts, starts) -> int:
        s = self.spec
        keys = 0
        for n, s0 in zip(new_counts, starts):
            if s.window is None:
                keys += n * s0 + n * (n + 1) // 2
            else:
                keys += sum(min(s0 + i + 1, s.window) for i in range(n))
        return 2 * sum(new_counts) * self.matrix_elements() + 2 * s.n_heads * (self.row + s.kv_rank) * keys

    def activation_bytes(self, n_tokens: int) -> int:
        s = self.spec
        size = 2 if self.dtype == torch.bfloat16 else 4
        total = n_tokens * ((self.first_cols + s.n_heads * self.qk_dim) * 4
                            + (s.q_rank + s.n_heads * (self.row + s.kv_rank) + self.o_dim) * size
                            + self.position.rot_dim * 4)
        if self._expandable():
            # a prompt step's expanded keys and values (the step's tokens and a window before each sequence),
            # as the product leaves them and as pages, and the queries and outputs of separate heads
            keys = 2 * n_tokens + (s.window or 0)
            total += keys * (self.row + 4 * s.n_heads * self.qk_dim) * size + 2 * n_tokens * s.n_heads * self.qk_dim * size
        return total

    def cache_request(self) -> LatentCacheRequest:
        return LatentCacheRequest(self.row, self.spec.window)

    def forward(self, step, xn, x_accum, cache, owns_cache: bool) -> None:
        s = self.spec
        n = step.n_tokens
        ws = step.workspace
        if stream(step).row_scale is not None:
            raise ConfigError("the latent attention was handed an input without its norm's scale")
        first = ws.get("latent.first", (n, self.first_cols), torch.float32)
        ops.gemm(xn, self.w_first, first, workspace=ws.scratch())
        cos, sin = self.position.tables(step)
        dims = self.position.rot_dim
        cq = ws.get("latent.cq", (n, s.q_rank), self.dtype)
        ops.latent_prepare(first, s.q_rank, s.kv_rank, s.rot_dim, dims, self.q_gain, self.kv_gain, s.q_norm.eps,
                           cos, sin, cq, cache.k, cache.block_table, step.token_seq, step.token_pos,
                           write_cache=owns_cache)
        q = ws.get("latent.q", (n, s.n_heads * self.qk_dim), torch.float32)
        ops.gemm(cq, self.w_uq, q, workspace=ws.scratch())
        # the queries as the attention takes them: per head [W_uk^T q^n, rotated q^r]
        qa = ws.get("latent.qa", (n, s.n_heads * self.row), self.dtype)
        expanded = (self.w_expand is not None and step.max_new > 1 and n >= self.EXPANDED_PROMPT_MIN_TOKENS
                    and step.cu_seqlens is not None and cache.k.shape[1] == ops.PREFILL_FUSED_PAGE)
        if expanded:
            self._expanded_prompt(step, q, first, cos, sin, dims, cache, x_accum)
            return
        ops.gemm_batched(q, self.qk_dim, self.w_uk_t, qa, self.row)
        ops.rope_heads(q, s.n_heads, self.qk_dim, s.head_dim, s.rot_dim, dims, cos, sin, qa, self.row, s.kv_rank)
        ol = ws.get("latent.ol", (n, s.n_heads * s.kv_rank), self.dtype)
        ops.attention(qa, ol, cache.k.unsqueeze(1), None, cache.block_table, step.token_seq, step.token_pos,
                      s.n_heads, 1, self.row, s.scale, s.window, workspace=ws.scratch(),
                      cu_seqlens=step.cu_seqlens, max_new=step.max_new, q_counts=step.new_counts,
                      max_len=step.max_len, v_head_dim=s.kv_rank, values_in_keys=True)
        o = ws.get("latent.o", (n, self.o_dim), self.dtype)
        gate = first[:, s.q_rank + self.row:] if s.gate else None
        if gate is not None and ops.gemm_batched_gate_fusable(self.w_uv, ol) and s.kv_rank % 8 == 0:
            ops.gemm_batched(ol, s.kv_rank, self.w_uv, o, s.v_head_dim, gate=gate)      # the gate is the product's epilogue
        else:
            ops.gemm_batched(ol, s.kv_rank, self.w_uv, o, s.v_head_dim)
            if gate is not None:
                ops.sigmoid_gate(o, gate)
        stream(step).add_product(o, self.w_o, x_accum)


    def _expanded_prompt(self, step, q, first, cos, sin, dims, cache, x_accum) -> None:
        """A prompt step in the expanded form.  The cache rows the step's queries see (its own tokens, which
        ``latent_prepare`` has appended, and up to window - 1 before them per sequence) are gathered into a
        dense matrix in scratch-page order, one product turns them into every head's key and value, the
        append kernel lays those out as pages of keys and transposed values, and the attention kernel for
        separate heads runs over them with a block table of scratch pages.  Nothing of it is kept."""
        s = self.spec
        n, H, D = step.n_tokens, s.n_heads, self.qk_dim
        ws = step.workspace
        page = cache.k.shape[1]
        span = s.window if s.window is not None else step.max_len
        pages = sum(min((c + span) // page + 2, step.max_len // page + 1) for c in step.new_counts)
        width = cache.block_table.shape[1]
        table = ws.get("latent.x.table", (len(step.new_counts), width), torch.int32)
        plan = ws.get("latent.x.plan", (4, pages), torch.int32)
        ops.latent_window_plan(step.cu_seqlens, step.token_pos, cache.block_table, s.window, page, table, plan)
        rows = ws.get("latent.x.rows", (pages * page, self.row), self.dtype)
        ops.latent_window_gather(cache.k, plan, rows)
        kv = ws.get("latent.x.kv", (pages * page, 2 * H * D), self.dtype)
        ops.gemm(rows, self.w_expand, kv, workspace=ws.scratch())
        ks = ws.get("latent.x.k", (pages, H, page, D), self.dtype)
        vs = ws.get("latent.x.v", (pages, H, D, page), self.dtype)
        if self._ident is None or self._ident[0].numel() < pages * page:
            dev = kv.device
            self._ident = (torch.arange(pages * page, dtype=torch.int32, device=dev),
                           torch.zeros(pages * page, dtype=torch.int32, device=dev),
                           torch.arange(pages, dtype=torch.int32, device=dev).view(1, pages))
        pos_id, seq_id, table_id = self._ident
        ops.qk_norm_rope_append(kv, 0, H, D, None, None, 1.0, None, None, 0, None, ks, vs, table_id[:, :pages].contiguous(),
                                seq_id[:pages * page], pos_id[:pages * page], write_kv=True)
        qf = ws.get("latent.x.q", (n, H * D), self.dtype)
        ops.rope_heads(q, H, D, s.head_dim, s.rot_dim, dims, cos, sin, qf, D, 0, lead=s.head_dim)
        of = ws.get("latent.x.o", (n, H * D), self.dtype)
        ops.attention(qf, of, ks, vs, table, step.token_seq, step.token_pos, H, H, D, s.scale, s.window,
                      workspace=ws.scratch(), cu_seqlens=step.cu_seqlens, max_new=step.max_new, q_counts=step.new_counts,
                      max_len=step.max_len)
        o = ws.get("latent.o", (n, self.o_dim), self.dtype)
        ops.gate_heads(of, D, first[:, s.q_rank + self.row:] if s.gate else None, o, H, s.v_head_dim)
        stream(step).add_product(o, self.w_o, x_accum)


register_mixer("latent_attention", LatentAttention)
