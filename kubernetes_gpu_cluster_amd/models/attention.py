"""Paged attention layer + the per-step forward context.

A step's tokens are laid out prefill-chunks first, then one token per decoding
sequence (``AttnMetadata``).  The attention layer splits ``q`` accordingly and
runs the prefill kernel (K2) on the first part and the split-context decode
kernel (K1) on the rest, both reading the layer's paged KV cache, after the
fused RoPE + KV-write kernel (K3/K5/K6) has stored the step's new keys/values.
"""
from __future__ import annotations

import dataclasses
from typing import Optional

import torch
import torch.nn as nn

from .. import ops


@dataclasses.dataclass
class AttnMetadata:
    slot_mapping: torch.Tensor                     # [T] int64, -1 = padding
    num_prefill_tokens: int = 0
    num_prefills: int = 0
    num_decodes: int = 0
    # prefill part (sequence i: query rows [qsl[i], qsl[i+1]) of the prefill tokens)
    prefill_block_tables: Optional[torch.Tensor] = None   # [P, max_blocks] int32
    query_start_loc: Optional[torch.Tensor] = None        # [P+1] int32
    prefill_seq_lens: Optional[torch.Tensor] = None       # [P] int32 (context incl. chunk)
    work_seq: Optional[torch.Tensor] = None
    work_mblk: Optional[torch.Tensor] = None
    # decode part
    decode_block_tables: Optional[torch.Tensor] = None    # [D, max_blocks] int32
    decode_ctx_lens: Optional[torch.Tensor] = None        # [D] int32
    decode_grid_z: int = 1
    decode_workspace: Optional[tuple] = None
    # prefill-only TP step split into two token halves for comm/compute overlap:
    # (a, meta of tokens [0, a), meta of tokens [a, T)) -- engine/model_runner.py
    split: Optional[tuple] = None
    # recurrent layers: the state slot of every step sequence (prefill chunks first, then
    # decode rows; < 0: a graph padding row) -- int32 [P + D]
    state_slots: Optional[torch.Tensor] = None


@dataclasses.dataclass
class ForwardContext:
    attn: AttnMetadata
    kv_caches: list                                    # per local layer: (k_cache, v_cache)
    cos_sin: Optional[torch.Tensor] = None
    k_scale: float = 1.0                               # fp8 KV: cache holds fp8(x / scale)
    v_scale: float = 1.0
    # per recurrent layer: its state tensors, one slot per running sequence
    states: Optional[list] = None


class PagedAttention(nn.Module):
    def __init__(self, num_heads: int, num_kv_heads: int, head_dim: int, layer_idx: int,
                 scale: Optional[float] = None):
        super().__init__()
        self.nq, self.nkv, self.d = num_heads, num_kv_heads, head_dim
        self.layer_idx = layer_idx
        self.scale = head_dim ** -0.5 if scale is None else scale

    def forward(self, q: torch.Tensor, ctx: ForwardContext) -> torch.Tensor:
        """q [T, nq, d] (rotated, K/V already in cache) -> [T, nq*d]."""
        m = ctx.attn
        kc, vc = ctx.kv_caches[self.layer_idx]
        out = torch.empty_like(q)
        tp = m.num_prefill_tokens
        if tp:
            o = ops.prefill_attention(q[:tp], kc, vc, m.prefill_block_tables, m.query_start_loc,
                                      m.prefill_seq_lens, self.scale, m.work_seq, m.work_mblk,
                                      out=out[:tp], k_scale=ctx.k_scale, v_scale=ctx.v_scale)
            if o.data_ptr() != out.data_ptr():
                out[:tp].copy_(o)
        if m.num_decodes:
            dst = out[tp:tp + m.num_decodes]
            o = ops.paged_attention_decode(q[tp:tp + m.num_decodes], kc, vc,
                                           m.decode_block_tables, m.decode_ctx_lens, self.scale,
                                           m.decode_workspace, m.decode_grid_z, out=dst,
                                           k_scale=ctx.k_scale, v_scale=ctx.v_scale)
            if o.data_ptr() != dst.data_ptr():
                dst.copy_(o)
        return out.view(q.shape[0], self.nq * self.d)


class WindowedAttention(nn.Module):
    """Attention mixer of the hybrid decoders: GQA with separate query/key and value
    sizes, rotary on the first ``rot_dims`` dimensions of a head, a sliding window that
    keeps the first tokens visible, softmax in fp32, and a per-head sigmoid output gate
    computed from the mixer's input.  Keys and values live in a plain-layout paged cache
    (k [nb, G, bs, dim], v [nb, G, bs, vdim]) indexed by the engine's block tables, so
    chunked prefill and decode rows of one step run through the same kernels."""

    def __init__(self, hidden: int, spec, cache_idx: int, dtype, device):
        super().__init__()
        from ..parallel.layers import ReplicatedLinear
        self.spec, self.cache_idx = spec, cache_idx
        H, G, dk, dv = spec.heads, spec.kv_heads, spec.dim, spec.vdim
        assert H % G == 0, "query heads must be a multiple of key/value heads"
        assert spec.rot_dims % 2 == 0 and spec.rot_dims <= dk
        self.qkv_proj = ReplicatedLinear(hidden, H * dk + G * dk + G * dv, dtype=dtype,
                                         device=device)
        self.o_proj = ReplicatedLinear(H * dv, hidden, dtype=dtype, device=device)
        self.gate = (nn.Parameter(torch.zeros(H, hidden, dtype=dtype, device=device),
                                  requires_grad=False) if spec.head_gate else None)
        self.scale = spec.dim ** -0.5 if spec.scale is None else spec.scale
        self.rope = None            # [max_pos, rot_dims] fp32, set by prepare()

    def prepare(self, tables: dict, max_pos: int, device) -> None:
        sp = self.spec
        if not sp.rot_dims:
            return
        key = (sp.rot_dims, sp.rot_base)
        if key not in tables:
            tables[key] = ops.ref.rope_table(sp.rot_dims, max_pos, sp.rot_base).to(device)
        self.rope = tables[key]

    def forward(self, h: torch.Tensor, positions: torch.Tensor, ctx: ForwardContext):
        sp = self.spec
        kc, vc = ctx.kv_caches[self.cache_idx]
        qkv = self.qkv_proj(h)
        gate = (ops.gate_proj(h, self.gate, None, ops.GATE_SIGMOID)
                if self.gate is not None else None)
        q = ops.rope_kv_store(qkv, positions, self.rope, kc, vc, ctx.attn.slot_mapping,
                              sp.heads, sp.kv_heads, sp.dim, sp.vdim)
        w = sp.window
        o = ops.window_attention(q, kc, vc, positions, ctx.attn, self.scale,
                                 w.size if w else 0, w.keep_first if w else 0, gate)
        return self.o_proj(o)


class LatentAttention(nn.Module):
    """Attention over a compressed cache: per token the cache row is one RMS-normed latent
    c (``kv_rank`` wide) followed by one rotary key part (``rot_dims``) that all heads
    share.  A head's key is [W_uk c | rotary part] and its value W_uv c, so
        score = q_u . (W_uk c) + q_r . k_r = (W_uk^T q_u) . c + q_r . k_r
    and   out = W_uv (sum_j p_j c_j):
    the unrotated query part is multiplied into latent space (one batched GEMM per step),
    all heads then attend the same rows as one key/value group -- keys are whole cache
    rows, values their latent columns -- and a second batched GEMM lifts the result to the
    heads' value size.  Prefill chunks and decode rows take the same path.  Sliding window,
    softmax in fp32, ``scale`` as given; the concatenated heads are multiplied by
    sigmoid(W_g h) before the output projection.

    One merged projection yields q | latent + rotary key | gate.  The cache of a layer run
    is chosen at call time (a looped layer has one per pass)."""

    def __init__(self, hidden: int, spec, eps: float, dtype, device):
        super().__init__()
        from ..parallel.layers import ReplicatedLinear
        self.spec, self.eps = spec, eps
        H, d, r, dv, rank = spec.heads, spec.dim, spec.rot_dims, spec.vdim, spec.kv_rank
        assert r % 2 == 0
        self.n_q, self.n_kv, self.n_g = H * (d + r), rank + r, H * dv
        self.proj = ReplicatedLinear(hidden, self.n_q + self.n_kv + self.n_g, dtype=dtype,
                                     device=device)
        self.o_proj = ReplicatedLinear(H * dv, hidden, dtype=dtype, device=device)
        z = lambda *s: nn.Parameter(torch.zeros(*s, dtype=dtype, device=device),   # noqa: E731
                                    requires_grad=False)
        self.w_uk = z(H, d, rank)          # [head, unrotated dim, latent]: q_u -> latent space
        self.w_uv = z(H, rank, dv)         # [head, latent, value dim]
        self.norm_weight = nn.Parameter(torch.ones(rank, dtype=torch.float32, device=device),
                                        requires_grad=False)
        self.scale = (d + r) ** -0.5 if spec.scale is None else spec.scale
        self.rope = None

    def prepare(self, tables: dict, max_pos: int, device) -> None:
        rs = self.spec.rotary
        if rs is None:
            return
        key = (rs.dims, rs.base, rs.yarn)
        if key not in tables:
            tables[key] = ops.ref.rope_table_yarn(rs.dims, max_pos, rs.base, rs.yarn).to(device)
        self.rope = tables[key]

    def forward(self, h: torch.Tensor, positions: torch.Tensor, ctx: ForwardContext,
                cache_idx: int):
        sp = self.spec
        H, d, r, dv, rank = sp.heads, sp.dim, sp.rot_dims, sp.vdim, sp.kv_rank
        T = h.shape[0]
        cache = ctx.kv_caches[cache_idx][0]                 # [nb, 1, bs, rank + r]
        proj = self.proj(h)
        qu = proj[:, : self.n_q].view(T, H, d + r)[:, :, :d].transpose(0, 1)   # [H, T, d]
        q_lat = torch.bmm(qu, self.w_uk)                                       # [H, T, rank]
        q = ops.latent_rope_store(proj, q_lat, positions, self.rope, self.norm_weight, self.eps,
                                  cache, ctx.attn.slot_mapping, H, d, r, rank)
        w = sp.window
        o = ops.window_attention(q, cache, cache[..., :rank], positions, ctx.attn, self.scale,
                                 w.size if w else 0, 0, None)                  # [T, H * rank]
        o = torch.bmm(o.view(T, H, rank).transpose(0, 1), self.w_uv)           # [H, T, dv]
        return self.o_proj(ops.gate_mul(o.transpose(0, 1), proj[:, self.n_q + self.n_kv:]))


class AttentionCore(nn.Module):
    """The part of a softmax attention mixer between its projections, for mixers whose
    projections are merged with a neighbour's (a parallel mixer): reads q | k | v (| the
    gate pre-activation) from columns ``col0 ..`` of a wider projection, rotates q and k
    (pairs (i, i + dims/2), or (2i, 2i + 1) when ``spec.rotary.interleaved``), stores k and
    v in the paged cache chosen at call time, attends causally (``spec.window`` when set)
    with scores q.k * scale that pass cap * tanh(. / cap) when ``spec.softcap`` > 0,
    multiplies the concatenated heads by sigmoid of the gate columns (``spec.elem_gate``)
    and by ``out_scale`` -- both in the attention kernels' epilogue -- and writes them into a
    column slice of the output projection's input.  Softmax, scores and rotation are fp32.

    With ``spec.conv`` taps, q | k | v first pass a causal convolution over time per channel
    (no bias, no activation; the last taps - 1 projected rows are per-sequence state).
    ``spec.qk_unit`` / ``spec.v_unit`` divide each head's q and k / v by its root mean square
    (v is cached so), and ``spec.q_temp`` = (coef, every) multiplies q at position p by
    1 + coef * ln(floor((p + 1) / every) + 1); these take the place of the rotation."""

    def __init__(self, spec, out_scale: float = 1.0, eps: float = 1e-6, device=None):
        super().__init__()
        self.spec, self.out_scale, self.eps = spec, float(out_scale), eps
        H, G, dk, dv = spec.heads, spec.kv_heads, spec.dim, spec.vdim
        assert H % G == 0, "query heads must be a multiple of key/value heads"
        assert spec.rot_dims % 2 == 0 and spec.rot_dims <= dk
        self.n_qkv = H * dk + G * dk + G * dv
        self.n_in = self.n_qkv + (H * dv if spec.elem_gate else 0)
        self.n_out = H * dv
        self.scale = spec.dim ** -0.5 if spec.scale is None else spec.scale
        self.rope = None            # [max_pos, rot_dims] fp32, set by prepare()
        self.unit = bool(spec.qk_unit or spec.v_unit or spec.q_temp)
        assert not (self.unit and spec.rot_dims), "unit-RMS inputs take the rotation's place"
        self.conv_w = (nn.Parameter(torch.zeros(self.n_qkv, spec.conv, dtype=torch.float32,
                                                device=device), requires_grad=False)
                       if spec.conv else None)

    def state_shapes(self) -> tuple:
        """Per-slot shapes of the state tensors: the convolution's last inputs, if any."""
        sp = self.spec
        return ((max(sp.conv - 1, 1), self.n_qkv),) if sp.conv else ()

    def prepare(self, tables: dict, max_pos: int, device) -> None:
        sp = self.spec
        if not sp.rot_dims:
            return
        key = (sp.rot_dims, sp.rot_base)
        if key not in tables:
            tables[key] = ops.ref.rope_table(sp.rot_dims, max_pos, sp.rot_base).to(device)
        self.rope = tables[key]

    def forward(self, proj: torch.Tensor, col0: int, positions: torch.Tensor,
                ctx: ForwardContext, cache_idx: int, out: torch.Tensor,
                state: tuple = ()) -> None:
        sp = self.spec
        kc, vc = ctx.kv_caches[cache_idx]
        qkv = proj[:, col0: col0 + self.n_qkv]
        if self.conv_w is not None:
            qkv = ops.causal_conv(qkv, self.conv_w, None, state[0], ctx.attn, False)
        if self.unit:
            q = ops.norm_kv_store(qkv.float(), positions, kc, vc, ctx.attn.slot_mapping, sp.heads,
                                  sp.kv_heads, sp.dim, sp.vdim, self.eps, sp.qk_unit, sp.v_unit,
                                  sp.q_temp, proj.dtype)
        else:
            q = ops.rope_kv_store(qkv.to(proj.dtype), positions, self.rope, kc, vc,
                                  ctx.attn.slot_mapping, sp.heads, sp.kv_heads, sp.dim, sp.vdim,
                                  bool(sp.rotary and sp.rotary.interleaved))
        w = sp.window
        g = proj[:, col0 + self.n_qkv: col0 + self.n_in] if sp.elem_gate else None
        ops.window_attention(q, kc, vc, positions, ctx.attn, self.scale, w.size if w else 0,
                             w.keep_first if w else 0, None, sp.softcap, self.out_scale, out=out,
                             elem_gate=g)
