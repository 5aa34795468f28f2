"""Pure-PyTorch reference implementations of every fused op.

These are the numerics oracles for the HIP kernels in ``csrc/kernels`` and the
CPU execution path (tiny models, the OPT-125m CPU plumbing pod).  They are
written for clarity, in fp32, not speed.

KV-cache layout (shared with the HIP kernels, chosen for CDNA4 MFMA operand
loads, see csrc/kernels/attention_decode.hip):
  k_cache: [num_blocks, num_kv_heads, block_size, head_dim]   (key rows contiguous)
  v_cache: [num_blocks, num_kv_heads, block_size/8, head_dim, 8]
           (V^T in 8-key groups: the 8 consecutive keys of one dim are 16 contiguous
            bytes -- the MFMA A-operand fragment of O^T = V^T.P^T -- and the 16 dims
            of one 16-row tile are 256 contiguous bytes)
"""
from __future__ import annotations

import math
import struct
from typing import Optional

import torch


# ---------------------------------------------------------------- norms / act
def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    xf = x.float()
    var = xf.pow(2).mean(-1, keepdim=True)
    return (xf * torch.rsqrt(var + eps) * w.float()).to(x.dtype)


def fused_add_rms_norm(x: torch.Tensor, residual: torch.Tensor, w: torch.Tensor,
                       eps: float) -> tuple[torch.Tensor, torch.Tensor]:
    """residual' = x + residual ; out = rms_norm(residual') * w.  Returns (out, residual')."""
    r = (x.float() + residual.float()).to(residual.dtype)
    return rms_norm(r, w, eps), r


def layer_norm(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, eps: float = 1e-5):
    return torch.nn.functional.layer_norm(x.float(), (x.shape[-1],), w.float(), b.float(),
                                          eps).to(x.dtype)


def silu_mul(x: torch.Tensor) -> torch.Tensor:
    d = x.shape[-1] // 2
    xf = x.float()
    return (torch.nn.functional.silu(xf[..., :d]) * xf[..., d:]).to(x.dtype)


# ---------------------------------------------------------------- rope
def _llama3_inv_freq(inv_freq: torch.Tensor, sc: dict) -> torch.Tensor:
    factor = sc["factor"]
    lo, hi = sc.get("low_freq_factor", 1.0), sc.get("high_freq_factor", 4.0)
    old = sc.get("original_max_position_embeddings", 8192)
    lo_wl, hi_wl = old / lo, old / hi
    wl = 2 * math.pi / inv_freq
    smooth = (old / wl - lo) / (hi - lo)
    scaled = torch.where(wl > lo_wl, inv_freq / factor, inv_freq)
    mid = (1 - smooth) * inv_freq / factor + smooth * inv_freq
    is_mid = (wl <= lo_wl) & (wl >= hi_wl)
    return torch.where(is_mid, mid, scaled)


def rope_cos_sin_cache(head_dim: int, max_pos: int, theta: float,
                       scaling: Optional[dict] = None) -> torch.Tensor:
    """[max_pos, head_dim] fp32: first half cos, second half sin (NeoX layout)."""
    inv = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float64) / head_dim))
    if scaling and scaling.get("rope_type", scaling.get("type")) == "llama3":
        inv = _llama3_inv_freq(inv, scaling)
    t = torch.arange(max_pos, dtype=torch.float64)
    freqs = torch.outer(t, inv)
    return torch.cat([freqs.cos(), freqs.sin()], dim=-1).float()


def apply_rope(x: torch.Tensor, positions: torch.Tensor, cos_sin: torch.Tensor) -> torch.Tensor:
    """x [T, n, d]; NeoX rotate-half."""
    d = x.shape[-1]
    cs = cos_sin[positions.long()]                 # [T, d]
    cos = cs[:, None, : d // 2]
    sin = cs[:, None, d // 2:]
    xf = x.float()
    x1, x2 = xf[..., : d // 2], xf[..., d // 2:]
    return torch.cat([x1 * cos - x2 * sin, x2 * cos + x1 * sin], dim=-1).to(x.dtype)


def rope_qk_kv_write(qkv: torch.Tensor, positions: torch.Tensor, cos_sin: torch.Tensor,
                     k_cache: torch.Tensor, v_cache: torch.Tensor, slot_mapping: torch.Tensor,
                     num_heads: int, num_kv_heads: int, head_dim: int,
                     q_norm_w: Optional[torch.Tensor] = None,
                     k_norm_w: Optional[torch.Tensor] = None, eps: float = 1e-6,
                     use_rope: bool = True, k_scale: float = 1.0,
                     v_scale: float = 1.0) -> torch.Tensor:
    """K3+K5(+K6): split fused qkv [T, (nq+2nkv)*d], optional per-head q/k RMSNorm,
    RoPE on q,k, scatter k,v into the paged cache at slot_mapping (-1 = skip).
    Returns rotated q as a contiguous [T, nq, d] tensor."""
    T = qkv.shape[0]
    qs, ks = num_heads * head_dim, num_kv_heads * head_dim
    q = qkv[:, :qs].reshape(T, num_heads, head_dim)
    k = qkv[:, qs:qs + ks].reshape(T, num_kv_heads, head_dim)
    v = qkv[:, qs + ks:qs + 2 * ks].reshape(T, num_kv_heads, head_dim)
    if q_norm_w is not None:
        q = rms_norm(q, q_norm_w, eps)
        k = rms_norm(k, k_norm_w, eps)
    if use_rope:
        q = apply_rope(q, positions, cos_sin)
        k = apply_rope(k, positions, cos_sin)
    kv_cache_write(k, v, k_cache, v_cache, slot_mapping, k_scale, v_scale)
    return q.contiguous()


FP8_MAX = 448.0


def to_cache(x: torch.Tensor, cache_dtype: torch.dtype, scale: float = 1.0) -> torch.Tensor:
    """Value -> cache element: the cache dtype itself, or fp8 e4m3 of (x / scale) with
    saturation (the kernels clamp to +-448 before the hardware conversion)."""
    if cache_dtype == torch.float8_e4m3fn:
        return (x.float() / scale).clamp(-FP8_MAX, FP8_MAX).to(cache_dtype)
    return x.to(cache_dtype)


def kv_cache_write(k: torch.Tensor, v: torch.Tensor, k_cache: torch.Tensor,
                   v_cache: torch.Tensor, slot_mapping: torch.Tensor,
                   k_scale: float = 1.0, v_scale: float = 1.0) -> None:
    bs = k_cache.shape[2]
    sm = slot_mapping.long()
    valid = sm >= 0
    if not bool(valid.any()):
        return
    sm = sm[valid]
    blk, off = sm // bs, sm % bs
    # an fp8 cache stores the activation-dtype-rounded value, quantised
    k_cache[blk, :, off, :] = to_cache(k[valid].to(k.dtype), k_cache.dtype, k_scale)
    v_cache[blk, :, off // 8, :, off % 8] = to_cache(v[valid].to(v.dtype), v_cache.dtype, v_scale)


# ---------------------------------------------------------------- attention
def _gather_kv(k_cache, v_cache, block_table, ctx_len, k_scale=1.0, v_scale=1.0):
    bs = k_cache.shape[2]
    nb = (ctx_len + bs - 1) // bs
    blocks = block_table[:nb].long()
    k = k_cache[blocks]                                   # [nb, nkv, bs, d]
    k = k.permute(0, 2, 1, 3).reshape(nb * bs, k.shape[1], k.shape[3])[:ctx_len]
    v = v_cache[blocks]                                   # [nb, nkv, bs/8, d, 8]
    v = v.permute(0, 2, 4, 1, 3).reshape(nb * bs, v.shape[1], v.shape[3])[:ctx_len]
    return k.float() * k_scale, v.float() * v_scale      # [ctx, nkv, d]


def paged_attention_decode(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                           block_tables: torch.Tensor, context_lens: torch.Tensor,
                           scale: float, k_scale: float = 1.0, v_scale: float = 1.0) -> torch.Tensor:
    """K1: q [B, nq, d] -> out [B, nq, d], one query token per sequence."""
    B, nq, d = q.shape
    nkv = k_cache.shape[1]
    g = nq // nkv
    out = torch.empty_like(q)
    for b in range(B):
        L = int(context_lens[b])
        k, v = _gather_kv(k_cache, v_cache, block_tables[b], L, k_scale, v_scale)
        qb = q[b].float().view(nkv, g, d)
        s = torch.einsum("hgd,lhd->hgl", qb, k) * scale
        p = torch.softmax(s, dim=-1)
        o = torch.einsum("hgl,lhd->hgd", p, v)
        out[b] = o.reshape(nq, d).to(q.dtype)
    return out


def prefill_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                      block_tables: torch.Tensor, query_start_loc: torch.Tensor,
                      seq_lens: torch.Tensor, scale: float, k_scale: float = 1.0,
                      v_scale: float = 1.0) -> torch.Tensor:
    """K2: varlen causal attention for packed prompt chunks.  Sequence i owns query
    rows [qsl[i], qsl[i+1]); its keys are cache positions [0, seq_lens[i]) and its
    queries sit at absolute positions seq_lens[i]-qlen .. seq_lens[i]-1."""
    T, nq, d = q.shape
    nkv = k_cache.shape[1]
    g = nq // nkv
    out = torch.empty_like(q)
    for i in range(len(seq_lens)):
        a, b = int(query_start_loc[i]), int(query_start_loc[i + 1])
        ql, L = b - a, int(seq_lens[i])
        if ql == 0:
            continue
        k, v = _gather_kv(k_cache, v_cache, block_tables[i], L, k_scale, v_scale)
        qi = q[a:b].float().view(ql, nkv, g, d)
        s = torch.einsum("qhgd,lhd->hgql", qi, k) * scale
        qpos = torch.arange(L - ql, L)[:, None]
        kpos = torch.arange(L)[None, :]
        s = s.masked_fill(kpos > qpos, float("-inf"))
        p = torch.softmax(s, dim=-1)
        o = torch.einsum("hgql,lhd->qhgd", p, v)
        out[a:b] = o.reshape(ql, nq, d).to(q.dtype)
    return out


def dense_causal_attention(q, k, v, scale):
    """Plain causal attention over one sequence: q [S, nq, d], k/v [S, nkv, d]."""
    S, nq, d = q.shape
    g = nq // k.shape[1]
    k = k.float().repeat_interleave(g, dim=1)
    v = v.float().repeat_interleave(g, dim=1)
    s = torch.einsum("qhd,khd->hqk", q.float(), k) * scale
    mask = torch.triu(torch.ones(S, S, dtype=torch.bool), 1)
    s = s.masked_fill(mask, float("-inf"))
    return torch.einsum("hqk,khd->qhd", torch.softmax(s, -1), v).to(q.dtype)


# ---------------------------------------------------------------- sampling
_M32 = 0xFFFFFFFF


def _mix32(x: torch.Tensor) -> torch.Tensor:
    """lowbias32 integer hash on int64 tensors holding uint32 values."""
    x = x & _M32
    x = x ^ (x >> 16)
    x = (x * 0x7FEB352D) & _M32
    x = x ^ (x >> 15)
    x = (x * 0x846CA68B) & _M32
    x = x ^ (x >> 16)
    return x


def _row_key(seeds: torch.Tensor) -> torch.Tensor:
    """Per-row stream key from both halves of the int64 seed (sampling.hip row_key)."""
    s = seeds.long()
    hi = _mix32(((s >> 32) + 0x632BE5AB) & _M32)
    return _mix32((s & _M32) ^ hi)


def uniform_noise(seeds: torch.Tensor, vocab: int) -> torch.Tensor:
    """Counter-based uniform(0,1) noise, identical to the HIP sampler's generator.
    seeds: [B] int64 (per-row stream key) -> [B, V] fp32."""
    return uniform_noise_cols(seeds, 0, vocab)


def uniform_noise_cols(seeds: torch.Tensor, col0: int, n: int) -> torch.Tensor:
    """``uniform_noise`` restricted to the global columns col0 .. col0 + n - 1."""
    col = torch.arange(col0, col0 + n, dtype=torch.int64)
    h = _mix32(_row_key(seeds)[:, None] ^ ((col[None, :] * 0x9E3779B9) & _M32))
    return ((h >> 9).double() + 0.5).float() * (1.0 / 8388608.0)    # 23 bits: u < 1 exactly


_LN2 = 0.69314718


def gumbel(u: torch.Tensor) -> torch.Tensor:
    """-ln(-ln u) as sampling.hip gumbel computes it (fp32): -ln2 * log2(-ln2 * log2 u)."""
    ln2 = torch.tensor(_LN2, dtype=torch.float32)
    return -(ln2 * torch.log2(-(ln2 * torch.log2(u.float()))))


_VP_BIAS = 1 << 63


def _ord_key(v: float) -> int:
    b = struct.unpack("<I", struct.pack("<f", v))[0]
    return (~b & 0xFFFFFFFF) if b & 0x80000000 else (b | 0x80000000)


def sample_vp_partial(logits: torch.Tensor, temperature: torch.Tensor, seeds: torch.Tensor,
                      vocab_off: int) -> torch.Tensor:
    """Vocab-parallel sampler, one shard: per row the packed (ord(value) << 32 | ~global
    index) of the shard's (Gumbel-)argmax, biased to a signed int64 so that a MAX
    all-reduce over the shards yields the unsharded sampler's pick (ties -> lower
    index).  Rows must not use top-k / top-p."""
    B, V = logits.shape
    x = logits.float().cpu()
    u = uniform_noise_cols(seeds.cpu(), vocab_off, V)
    out = torch.empty(B, dtype=torch.int64)
    for b in range(B):
        t = float(temperature[b])
        row = x[b] if t <= 1e-5 else x[b] / t + gumbel(u[b])
        i = int(torch.argmax(row))                       # first index on ties
        packed = (_ord_key(float(row[i])) << 32) | (~(i + vocab_off) & 0xFFFFFFFF)
        out[b] = packed - _VP_BIAS                       # == (packed ^ bias) as int64
    return out.to(logits.device)


def sample_vp_unpack(packed: torch.Tensor) -> torch.Tensor:
    out = torch.empty_like(packed)
    for b, v in enumerate(packed.tolist()):
        u64 = v + _VP_BIAS
        idx = ~u64 & 0xFFFFFFFF
        out[b] = 0 if (u64 == 0 or idx >= 0x7FFFFFFF) else idx
    return out


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor,
           top_p: torch.Tensor, seeds: torch.Tensor) -> torch.Tensor:
    """K10: greedy when temperature==0, else Gumbel-max over the top-k/top-p support.
    Returns int64 token ids [B]."""
    B, V = logits.shape
    x = logits.float()
    out = torch.empty(B, dtype=torch.int64)
    u = uniform_noise(seeds.cpu(), V)
    for b in range(B):
        row = x[b].cpu()
        t = float(temperature[b])
        if t <= 1e-5:
            out[b] = int(torch.argmax(row))
            continue
        row = row / t
        drop = torch.zeros(V, dtype=torch.bool)
        k = int(top_k[b])
        if 0 < k < V:
            kth = torch.topk(row, k).values[-1]
            drop |= row < kth
        p = float(top_p[b])
        if p < 1.0:
            probs = torch.softmax(row.masked_fill(drop, float("-inf")), -1)
            sp, idx = torch.sort(probs, descending=True)
            cum = torch.cumsum(sp, 0)
            keep = (cum - sp) < p
            thr = sp[keep][-1]
            drop |= probs < thr
        # noise first, then the mask: a dropped column is -inf whatever its noise
        out[b] = int(torch.argmax((row + gumbel(u[b])).masked_fill(drop, float("-inf"))))
    return out.to(logits.device)


# ---------------------------------------------------------------- MoE
def moe_topk_softmax(router_logits: torch.Tensor, k: int, renormalize: bool = True):
    """K13: softmax over experts, top-k; returns (weights fp32 [T,k], ids int32 [T,k])."""
    p = torch.softmax(router_logits.float(), dim=-1)
    w, ids = torch.topk(p, k, dim=-1)
    if renormalize:
        w = w / w.sum(-1, keepdim=True)
    return w, ids.to(torch.int32)


def moe_mlp_local(x: torch.Tensor, w13: torch.Tensor, w2: torch.Tensor, topk_w: torch.Tensor,
                  topk_ids: torch.Tensor, expert_offset: int = 0) -> torch.Tensor:
    """K14 over the experts held locally (global ids offset by ``expert_offset``); pairs
    routed elsewhere contribute nothing.  Expert outputs are rounded to x.dtype before
    the fp32 weighted combine, like the kernel."""
    T, H = x.shape
    out = torch.zeros(T, H, dtype=torch.float32, device=x.device)
    for e in range(w13.shape[0]):
        tok, slot = torch.nonzero(topk_ids == e + expert_offset, as_tuple=True)
        if tok.numel() == 0:
            continue
        h = silu_mul((x[tok].float() @ w13[e].float().t()).to(x.dtype).float())
        y = (h.to(x.dtype).float() @ w2[e].float().t()).to(x.dtype)
        out.index_add_(0, tok, y.float() * topk_w[tok, slot, None].float())
    return out.to(x.dtype)


def moe_mlp(x: torch.Tensor, w13: torch.Tensor, w2: torch.Tensor, topk_w: torch.Tensor,
            topk_ids: torch.Tensor) -> torch.Tensor:
    """K14: per-expert SwiGLU MLP, weighted combine.  w13 [E, 2I, H], w2 [E, H, I]."""
    T, H = x.shape
    out = torch.zeros(T, H, dtype=torch.float32, device=x.device)
    for e in range(w13.shape[0]):
        tok, slot = torch.nonzero(topk_ids == e, as_tuple=True)
        if tok.numel() == 0:
            continue
        h = x[tok].float() @ w13[e].float().t()
        h = silu_mul(h)
        y = h @ w2[e].float().t()
        out.index_add_(0, tok, y * topk_w[tok, slot, None].float())
    return out.to(x.dtype)


# ---------------------------------------------------------------- hybrid decoders
# (grouped RMSNorm, depth-weighted averaging, xIELU, small gate projections, windowed
# attention with kept first tokens over a plain-layout paged cache, mLSTM state scan)
def group_rms_norm(x: torch.Tensor, w: torch.Tensor, groups: int, eps: float,
                   out_dtype: torch.dtype) -> torch.Tensor:
    """Each of ``groups`` equal consecutive parts of a row is divided by its own
    sqrt(mean(part^2) + eps); the whole row is then multiplied by w.  fp32 math."""
    T, W = x.shape
    xg = x.float().view(T, groups, W // groups)
    xg = xg * torch.rsqrt(xg.pow(2).mean(-1, keepdim=True) + eps)
    return (xg.view(T, W) * w.float()).to(out_dtype)


def depth_mix(hist: torch.Tensor, n: int, coef: torch.Tensor, T: int) -> torch.Tensor:
    """sum_j coef[j] * hist[j, :T] over the first n layer results (fp32)."""
    return torch.einsum("j,jtw->tw", coef[:n].float(), hist[:n, :T].float())


def xielu(z: torch.Tensor, ab: torch.Tensor) -> torch.Tensor:
    """z > 0: a z^2 + z/2;  z <= 0: b (exp(z) - 1 - z) + z/2, with ab = (a, b) fp32."""
    zf = z.float()
    a, b = ab[0], ab[1]
    return torch.where(zf > 0, a * zf * zf + 0.5 * zf,
                       b * (torch.expm1(torch.clamp(zf, max=0.0)) - zf) + 0.5 * zf).to(z.dtype)


GATE_SIGMOID, GATE_CAP_TANH, GATE_LOGSIG_CAP_TANH, GATE_NONE = 0, 1, 2, 3


def _gate_act(y: torch.Tensor, kind: int, cap: float) -> torch.Tensor:
    if kind == GATE_SIGMOID:
        return torch.sigmoid(y)
    if kind == GATE_NONE:
        return y
    y = cap * torch.tanh(y / cap)
    return y if kind == GATE_CAP_TANH else torch.nn.functional.logsigmoid(y)


def gate_proj(h: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], kind_a: int,
              kind_b: int, split: int, cap: float) -> torch.Tensor:
    """fp32 [T, N]: act(h . w^T + bias), rows < split of w with kind_a, the rest kind_b.
    The dot products accumulate in fp32 and are never rounded to 16 bits."""
    y = h.float() @ w.float().t()
    if bias is not None:
        y = y + bias.float()
    return torch.cat([_gate_act(y[:, :split], kind_a, cap), _gate_act(y[:, split:], kind_b, cap)],
                     dim=1)


def rope_table(rot_dims: int, max_pos: int, base: float) -> torch.Tensor:
    """[max_pos, rot_dims] fp32: cos | sin of p * base^(-2i/rot_dims), i < rot_dims/2,
    with the frequencies, the angles and cos / sin all evaluated in fp32."""
    f = torch.tensor(base, dtype=torch.float32) ** (
        -2.0 * torch.arange(rot_dims // 2, dtype=torch.float32) / rot_dims)
    a = torch.arange(max_pos, dtype=torch.float32)[:, None] * f[None]
    return torch.cat([a.cos(), a.sin()], dim=-1)


def rope_kv_store(qkv: torch.Tensor, positions: torch.Tensor, table: Optional[torch.Tensor],
                  k_cache: torch.Tensor, v_cache: torch.Tensor, slot_mapping: torch.Tensor,
                  H: int, G: int, dk: int, dv: int, interleaved: bool = False) -> torch.Tensor:
    """qkv [T, H*dk + G*dk + G*dv] -> rotated q [T, H, dk]; rotated k and v go to the
    plain-layout paged cache (k_cache [nb, G, bs, dk], v_cache [nb, G, bs, dv]) at
    ``slot_mapping`` (< 0: no write).  Rotation pairs dim i with i + rot/2 (interleaved:
    2i with 2i + 1) over the first rot = table.shape[1] dims of a head (fp32 math); the
    rest pass unchanged."""
    T = qkv.shape[0]
    q = qkv[:, : H * dk].float().view(T, H, dk)
    k = qkv[:, H * dk: (H + G) * dk].float().view(T, G, dk)
    v = qkv[:, (H + G) * dk: (H + G) * dk + G * dv].view(T, G, dv)
    if table is not None:
        r = table.shape[1]
        cs = table[positions.long()]
        c, s = cs[:, None, : r // 2], cs[:, None, r // 2:]

        def rot(x):
            if interleaved:
                a, b = x[..., 0:r:2], x[..., 1:r:2]
                ab = torch.stack([a * c - b * s, b * c + a * s], dim=-1).flatten(-2)
                return torch.cat([ab, x[..., r:]], dim=-1)
            a, b = x[..., : r // 2], x[..., r // 2: r]
            return torch.cat([a * c - b * s, b * c + a * s, x[..., r:]], dim=-1)
        q, k = rot(q), rot(k)
    bs = k_cache.shape[2]
    ok = slot_mapping >= 0
    sl = slot_mapping[ok].long()
    k_cache[sl // bs, :, sl % bs] = k[ok].to(k_cache.dtype)
    v_cache[sl // bs, :, sl % bs] = v[ok].to(v_cache.dtype)
    return q.to(qkv.dtype)


def window_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                     positions: torch.Tensor, row_tables: torch.Tensor, scale: float,
                     window: int, keep_first: int,
                     gate: Optional[torch.Tensor], softcap: float = 0.0,
                     out_scale: float = 1.0,
                     elem_gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """q [T, H, dk] (rotated; the step's k / v already stored) -> [T, H*dv].  Row t at
    position p = positions[t] attends the cached keys j <= p with p - j < window or
    j < keep_first (window <= 0: all of them) of the sequence whose block table is
    row_tables[t]; scores q.k * scale, then softcap * tanh(score / softcap) when
    softcap > 0; softmax and the weighted sum in fp32; each head's output times
    gate[t, head] (fp32) when given, the concatenated heads times sigmoid(elem_gate
    [T, H*dv]) when given, and times out_scale."""
    T, H, dk = q.shape
    G, bs, dv = k_cache.shape[1], k_cache.shape[2], v_cache.shape[3]
    out = torch.zeros(T, H, dv, dtype=torch.float32)
    for t in range(T):
        p = int(positions[t])
        if p < 0:
            continue
        j = torch.arange(p + 1)
        if window > 0:
            j = j[(p - j < window) | (j < keep_first)]
        blk = row_tables[t].long()[j // bs]
        k = k_cache[blk, :, j % bs].float()           # [n, G, dk]
        v = v_cache[blk, :, j % bs].float()
        qt = q[t].float().view(G, H // G, dk)
        s = torch.einsum("ghd,ngd->ghn", qt, k) * scale
        if softcap > 0:
            s = softcap * torch.tanh(s / softcap)
        pr = torch.softmax(s, dim=-1)
        out[t] = torch.einsum("ghn,ngv->ghv", pr, v).reshape(H, dv)
    if gate is not None:
        out = out * gate.float()[:, :, None]
    if elem_gate is not None:
        out = out * torch.sigmoid(elem_gate.float()).view(T, H, dv)
    if out_scale != 1.0:
        out = out * out_scale
    return out.view(T, H * dv).to(q.dtype)


def mlstm_scan(qkvg: torch.Tensor, gates: torch.Tensor, S: torch.Tensor, n: torch.Tensor,
               m: torch.Tensor, seq_start: list, seq_len: list, seq_pos: list, seq_slot: list,
               H: int, d: int, dv: int) -> torch.Tensor:
    """The mLSTM recurrence over each step sequence's tokens, from (and back into) its
    state slot: S [slots, H, d, dv], n [slots, H, d], m [slots, H], all fp32.  A sequence
    whose first token is at position 0 starts from zero state (m = 0).  qkvg [T, >= 2Hd+Hdv]:
    q | k | v (| ...); gates [T, 2H] fp32: log input gate | log forget gate.  With
    m' = max(f + m, i):  S' = exp(f + m - m') S + exp(i - m') k v^T, n' likewise with k;
    o = S'^T q / (max(|n'.q|, exp(-m')) + 1e-6), q scaled by d^-1/2.  -> fp32 [T, H*dv]."""
    T = qkvg.shape[0]
    out = torch.zeros(T, H, dv, dtype=torch.float32)
    qs = d ** -0.5
    for a, ln, p0, slot in zip(seq_start, seq_len, seq_pos, seq_slot):
        if slot < 0:
            continue
        if p0 == 0:
            Sx = torch.zeros(H, d, dv)
            nx = torch.zeros(H, d)
            mx = torch.zeros(H)
        else:
            Sx, nx, mx = S[slot].clone(), n[slot].clone(), m[slot].clone()
        for t in range(a, a + ln):
            q = qkvg[t, : H * d].float().view(H, d) * qs
            k = qkvg[t, H * d: 2 * H * d].float().view(H, d)
            v = qkvg[t, 2 * H * d: 2 * H * d + H * dv].float().view(H, dv)
            ig, fg = gates[t, :H], gates[t, H:]
            mn = torch.maximum(fg + mx, ig)
            fa, ia = torch.exp(fg + mx - mn), torch.exp(ig - mn)
            Sx = fa[:, None, None] * Sx + ia[:, None, None] * k[:, :, None] * v[:, None, :]
            nx = fa[:, None] * nx + ia[:, None] * k
            mx = mn
            den = torch.maximum((nx * q).sum(-1).abs(), torch.exp(-mx)) + 1e-6
            out[t] = torch.einsum("hdv,hd->hv", Sx, q) / den[:, None]
        S[slot], n[slot], m[slot] = Sx, nx, mx
    return out.view(T, H * dv)


def head_norm_gate(o: torch.Tensor, g: torch.Tensor, w: torch.Tensor, H: int, eps: float,
                   out_dtype: torch.dtype) -> torch.Tensor:
    """o fp32 [T, H*dv]: each head divided by its root mean square, times w, times
    sigmoid(g) (g [T, H*dv], any float dtype); fp32 math -> out_dtype."""
    T, N = o.shape
    oh = o.float().view(T, H, N // H)
    oh = oh * torch.rsqrt(oh.pow(2).mean(-1, keepdim=True) + eps)
    return (oh.view(T, N) * w.float() * torch.sigmoid(g.float())).to(out_dtype)


# ---------------------------------------------------------------- Konovik-style decoders
# (scaled residual + norm, token shift, minGRU scan, latent-attention cache rows with
# YaRN / interleaved rotary, sigmoid routing with a choice correction, squared-ReLU
# experts, per-token side input)
def rope_table_yarn(rot_dims: int, max_pos: int, base: float, yarn=None) -> torch.Tensor:
    """[max_pos, rot_dims] fp32: cos | sin of p * f_i, i < rot_dims/2.  ``yarn`` =
    (factor, original, fast, slow): f_i = base^(-2i/dims) is slowed by ``factor`` for the
    pairs past the ramp between the dimensions that make ``fast`` and ``slow`` turns over
    ``original`` positions, and cos / sin are scaled by 0.1 ln(factor) + 1."""
    i = torch.arange(rot_dims // 2, dtype=torch.float32)
    f = torch.tensor(base, dtype=torch.float32) ** (-2.0 * i / rot_dims)
    mag = 1.0
    if yarn is not None:
        factor, orig, fast, slow = yarn

        def turn_dim(turns):
            return rot_dims * math.log(orig / (2 * math.pi * turns)) / (2 * math.log(base))
        lo = max(math.floor(turn_dim(fast)), 0)
        hi = min(math.ceil(turn_dim(slow)), rot_dims - 1)
        ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
        f = f / factor * ramp + f * (1 - ramp)
        mag = 0.1 * math.log(factor) + 1.0
    a = torch.arange(max_pos, dtype=torch.float32)[:, None] * f[None]
    return torch.cat([a.cos() * mag, a.sin() * mag], dim=-1)


def residual_norm(x: torch.Tensor, add: Optional[torch.Tensor], mult: float,
                  w: Optional[torch.Tensor], eps: float, out_dtype: Optional[torch.dtype],
                  add_norm_w: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """x (fp32, in place) += mult * a, with a = add, or add / rms(add) * add_norm_w when
    that weight is given; then returns x / rms(x) * w (w None: x itself) in out_dtype
    (None: nothing).  rms(v) = sqrt(mean(v^2) + eps); fp32 math."""
    if add is not None:
        a = add.float()
        if add_norm_w is not None:
            a = a * torch.rsqrt(a.pow(2).mean(-1, keepdim=True) + eps) * add_norm_w.float()
        x += mult * a
    if out_dtype is None:
        return None
    if w is None:
        return x.to(out_dtype)
    return (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w.float()).to(out_dtype)


def step_sequences(meta) -> list:
    """[(first row, rows, position of the first row, state slot)] of a step's sequences:
    prefill chunks, then decode rows."""
    P, D, tp = meta.num_prefills, meta.num_decodes, meta.num_prefill_tokens
    seqs = []
    slots = meta.state_slots[: P + D].tolist()
    if P:
        qsl, sl = meta.query_start_loc.tolist(), meta.prefill_seq_lens.tolist()
        for i in range(P):
            n = qsl[i + 1] - qsl[i]
            seqs.append((qsl[i], n, sl[i] - n, slots[i]))
    if D:
        ctx = meta.decode_ctx_lens.tolist()
        for i in range(D):
            seqs.append((tp + i, 1, ctx[i] - 1, slots[P + i]))
    return seqs


def token_shift(h: torch.Tensor, mu: torch.Tensor, state: torch.Tensor, seqs: list,
                out_dtype: torch.dtype) -> torch.Tensor:
    """h fp32 [T, W] -> h + (prev - h) * mu, prev the sequence's previous row (before this
    replacement): the row above, or for a chunk's first row state[slot] (zeros at position
    0).  state[slot] then holds the chunk's last row.  Rows of slot < 0 give zeros."""
    out = torch.zeros_like(h)
    for a, n, p0, slot in seqs:
        if slot < 0:
            continue
        first = torch.zeros_like(h[:1]) if p0 == 0 else state[slot][None]
        prev = torch.cat([first, h[a:a + n - 1]], 0)
        out[a:a + n] = h[a:a + n] + (prev - h[a:a + n]) * mu.float()
        state[slot] = h[a + n - 1]
    return out.to(out_dtype)


def mingru_scan(zxg: torch.Tensor, bias: torch.Tensor, state: torch.Tensor, seqs: list,
                width: int, out_dtype: torch.dtype) -> torch.Tensor:
    """zxg [T, 3 width]: pre-activations of the update gate | candidate | output gate;
    bias fp32 [2 width] for the first two.  z = sigmoid(.), u -> u + 1/2 (u >= 0) or
    sigmoid(u); S = (1 - z) S + z cand per sequence from state[slot] (zeros at position
    0), written back; -> S * silu(g) [T, width].  fp32 math."""
    T = zxg.shape[0]
    zx = zxg[:, : 2 * width].float() + bias.float()
    z = torch.sigmoid(zx[:, :width])
    u = zx[:, width:]
    cand = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    g = zxg[:, 2 * width: 3 * width].float()
    out = torch.zeros(T, width, dtype=torch.float32, device=zxg.device)
    for a, n, p0, slot in seqs:
        if slot < 0:
            continue
        S = torch.zeros(width) if p0 == 0 else state[slot].clone()
        for t in range(a, a + n):
            S = (1 - z[t]) * S + z[t] * cand[t]
            out[t] = S
        state[slot] = S
    return (out * g * torch.sigmoid(g)).to(out_dtype)


def _rot_pairs(x: torch.Tensor, cs: torch.Tensor) -> torch.Tensor:
    """x [..., r] with pairs (2i, 2i+1); cs [..., r] = cos | sin."""
    r = x.shape[-1]
    c, s = cs[..., : r // 2], cs[..., r // 2:]
    u, v = x[..., 0::2], x[..., 1::2]
    return torch.stack([u * c - v * s, v * c + u * s], dim=-1).flatten(-2)


def latent_rope_store(proj: torch.Tensor, q_lat: torch.Tensor, positions: torch.Tensor,
                      table: Optional[torch.Tensor], norm_w: torch.Tensor, eps: float,
                      cache: torch.Tensor, slot_mapping: torch.Tensor, H: int, d: int, r: int,
                      rank: int) -> torch.Tensor:
    """proj [T, H (d + r) + rank + r + ...]: per head the query's d unrotated and r rotary
    columns, then the latent pre-activation (rank) and the shared rotary key part (r).
    q_lat [H, T, rank]: the unrotated query parts already multiplied into latent space.
    Writes the cache row [RMS-normed latent * norm_w | rotated key part] at slot_mapping
    (< 0: none) into cache [nb, 1, bs, rank + r] and returns the query rows
    [T, H, rank + r] = [q_lat | rotated query part] in proj's dtype.  Pairs are (2i, 2i+1)."""
    T = proj.shape[0]
    q = proj[:, : H * (d + r)].float().view(T, H, d + r)[..., d:]
    dkv = proj[:, H * (d + r): H * (d + r) + rank + r].float()
    c = dkv[:, :rank]
    c = c * torch.rsqrt(c.pow(2).mean(-1, keepdim=True) + eps) * norm_w.float()
    kr = dkv[:, rank:]
    if r:
        cs = table[positions.long()]
        q = _rot_pairs(q, cs[:, None, :])
        kr = _rot_pairs(kr, cs)
    bs = cache.shape[2]
    ok = slot_mapping >= 0
    sl = slot_mapping[ok].long()
    cache[sl // bs, 0, sl % bs] = torch.cat([c, kr], -1)[ok].to(cache.dtype)
    return torch.cat([q_lat.float().transpose(0, 1), q], -1).to(proj.dtype)


def gate_mul(o: torch.Tensor, g: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """o [T, H, dv] (any strides) * sigmoid(g [T, H dv]) * scale -> [T, H dv] in g's dtype."""
    T = o.shape[0]
    y = o.float().reshape(T, -1) * torch.sigmoid(g.float())
    return (y * scale if scale != 1.0 else y).to(g.dtype)


def relu_sq(z: torch.Tensor) -> torch.Tensor:
    return torch.relu(z.float()).pow(2).to(z.dtype)


def moe_route_sigmoid(scores: torch.Tensor, correction: torch.Tensor, k: int, scale: float):
    """scores fp32 [T, >= E]: sigmoid router scores in the first E = len(correction)
    columns.  The k experts with the largest score + correction (lowest index first among
    equals); weights = their scores / (sum + 1e-20) * scale.  -> (fp32 [T, k], int32 [T, k])."""
    E = correction.numel()
    s = scores[:, :E].float()
    ids = torch.topk(s + correction.float(), k, dim=-1).indices
    w = torch.gather(s, 1, ids)
    return w / (w.sum(-1, keepdim=True) + 1e-20) * scale, ids.to(torch.int32)


def moe_finish(routed: Optional[torch.Tensor], dense: Optional[torch.Tensor],
               topk_w: Optional[torch.Tensor], topk_ids: Optional[torch.Tensor],
               shared: Optional[torch.Tensor], gate: Optional[torch.Tensor]) -> torch.Tensor:
    """The routed experts' weighted sum -- ``routed`` [T, W] already combined, or gathered
    from ``dense`` [E, T, W] (every expert's output for every token) with topk_w / topk_ids
    -- plus gate[t] * shared[t] (gate fp32 [T], any stride)."""
    if routed is not None:
        out = routed.float()
    else:
        T = dense.shape[1]
        ids = topk_ids.long()
        ids = torch.where((ids < 0) | (ids >= dense.shape[0]), torch.zeros_like(ids), ids)
        y = dense.float()[ids, torch.arange(T, device=dense.device)[:, None]]
        out = (y * topk_w.float()[:, :, None]).sum(1)
    if shared is not None:
        out = out + gate.float()[:, None] * shared.float()
    return out.to(shared.dtype if shared is not None else (routed if routed is not None else dense).dtype)


def side_gate(pre: torch.Tensor, ids: torch.Tensor, table: torch.Tensor, col0: int) -> torch.Tensor:
    """gelu_tanh(pre [T, n]) * table[ids, col0:col0 + n] in pre's dtype."""
    n = pre.shape[1]
    z = pre.float()
    g = 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))
    return (g * table[ids.long(), col0:col0 + n].float()).to(pre.dtype)


# ---------------------------------------------------------------- parallel mixers
# (short causal convolutions over per-sequence state, the Mamba-2 recurrence, the gated
# delta rule, RMS norms combined with a SiLU gate)
def causal_conv(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor],
                state: torch.Tensor, seqs: list, silu: bool = True,
                out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """Per-channel causal convolution over time: y[t, c] = sum_j w[c, j] * x[t - (K-1) + j, c]
    (+ bias[c]), the last tap on the current token, then SiLU.  x [T, C] (a column slice of
    a projection), w fp32 [C, K].  state fp32 [slots, K-1, C] holds each sequence's last
    K-1 inputs (oldest first; zeros before position 0) and is updated.  -> [T, C] in
    ``out_dtype`` (fp32 math)."""
    T, C = x.shape
    K = w.shape[1]
    out = torch.zeros(T, C, dtype=torch.float32, device=x.device)
    wf = w.float()
    for a, n, p0, slot in seqs:
        if slot < 0:
            continue
        prev = torch.zeros(K - 1, C) if p0 == 0 else state[slot][: K - 1].clone()
        xs = torch.cat([prev, x[a:a + n].float()], 0)              # [K-1+n, C]
        y = torch.zeros(n, C)
        for j in range(K):
            y = y + xs[j:j + n] * wf[:, j]
        if bias is not None:
            y = y + bias.float()
        out[a:a + n] = y
        if K > 1:
            state[slot] = xs[n:]
    return (out * torch.sigmoid(out) if silu else out).to(out_dtype)


def ssd_scan(xbc: torch.Tensor, dt: torch.Tensor, a_log: torch.Tensor, dt_bias: torch.Tensor,
             dskip: torch.Tensor, state: torch.Tensor, seqs: list, H: int, P: int, N: int,
             G: int) -> torch.Tensor:
    """The Mamba-2 recurrence.  xbc fp32 [T, H P + 2 G N] = x | B | C (after convolution
    and SiLU), dt [T, H] raw step sizes; per head h (group g = h // (H / G)):
        d = softplus(dt + dt_bias_h);  S = exp(-exp(a_log_h) d) S + d B_g x_h^T  (S [N, P])
        y_h = S^T C_g + dskip_h x_h
    from state[slot] [H, N, P] fp32 (zeros at position 0), written back.  -> fp32 [T, H P]."""
    T = xbc.shape[0]
    x = xbc[:, : H * P].float().view(T, H, P)
    B = xbc[:, H * P: H * P + G * N].float().view(T, G, N).repeat_interleave(H // G, dim=1)
    C = xbc[:, H * P + G * N: H * P + 2 * G * N].float().view(T, G, N).repeat_interleave(H // G, dim=1)
    d = torch.nn.functional.softplus(dt.float() + dt_bias.float())
    decay = torch.exp(-torch.exp(a_log.float()) * d)
    out = torch.zeros(T, H, P, dtype=torch.float32)
    for a, n, p0, slot in seqs:
        if slot < 0:
            continue
        S = torch.zeros(H, N, P) if p0 == 0 else state[slot].clone()
        for t in range(a, a + n):
            S = decay[t, :, None, None] * S + (d[t, :, None] * B[t])[:, :, None] * x[t][:, None, :]
            out[t] = torch.einsum("hnp,hn->hp", S, C[t]) + dskip.float()[:, None] * x[t]
        state[slot] = S
    return out.view(T, H * P)


def gated_delta_scan(qkv: torch.Tensor, ba: torch.Tensor, a_log: torch.Tensor,
                     dt_bias: torch.Tensor, state: torch.Tensor, seqs: list, H: int, G: int,
                     d: int, dv: int) -> torch.Tensor:
    """The gated delta rule.  qkv fp32 [T, 2 G d + H dv] = q | k | v (after convolution and
    SiLU), ba [T, 2 H]: pre-activations of the write strength | of the decay.  q and k
    become unit vectors per head (x / sqrt(sum x^2 + 1e-6)), q times d^-1/2.  Per head h
    (q / k head h // (H / G)), with beta = sigmoid(b), g = exp(-exp(a_log_h) softplus(a + dt_bias_h)):
        S = g S;  u = beta (v - S^T k);  S = S + k u^T;  o = S^T q         (S [d, dv])
    from state[slot] [H, d, dv] fp32 (zeros at position 0), written back.  -> fp32 [T, H dv]."""
    T = qkv.shape[0]
    q = qkv[:, : G * d].float().view(T, G, d)
    k = qkv[:, G * d: 2 * G * d].float().view(T, G, d)
    v = qkv[:, 2 * G * d: 2 * G * d + H * dv].float().view(T, H, dv)
    q = q * torch.rsqrt(q.pow(2).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
    k = k * torch.rsqrt(k.pow(2).sum(-1, keepdim=True) + 1e-6)
    q, k = q.repeat_interleave(H // G, dim=1), k.repeat_interleave(H // G, dim=1)
    beta = torch.sigmoid(ba[:, :H].float())
    g = torch.exp(-torch.exp(a_log.float()) *
                  torch.nn.functional.softplus(ba[:, H: 2 * H].float() + dt_bias.float()))
    out = torch.zeros(T, H, dv, dtype=torch.float32)
    for a, n, p0, slot in seqs:
        if slot < 0:
            continue
        S = torch.zeros(H, d, dv) if p0 == 0 else state[slot].clone()
        for t in range(a, a + n):
            S = g[t, :, None, None] * S
            u = beta[t, :, None] * (v[t] - torch.einsum("hdv,hd->hv", S, k[t]))
            S = S + k[t][:, :, None] * u[:, None, :]
            out[t] = torch.einsum("hdv,hd->hv", S, q[t])
        state[slot] = S
    return out.view(T, H * dv)


def gated_rms_norm(y: torch.Tensor, gate: torch.Tensor, w: torch.Tensor, groups: int,
                   eps: float, gate_first: bool, out_dtype: torch.dtype) -> torch.Tensor:
    """y fp32 [T, n] in ``groups`` equal parts, each divided by its own root mean square and
    the row multiplied by w [n], with a SiLU gate silu(gate [T, n]): applied to y before
    the norm (gate_first) or to the normed, weighted result.  fp32 math -> out_dtype."""
    T, n = y.shape
    g = gate.float()
    g = g * torch.sigmoid(g)
    v = y.float() * g if gate_first else y.float()
    vg = v.view(T, groups, n // groups)
    v = (vg * torch.rsqrt(vg.pow(2).mean(-1, keepdim=True) + eps)).view(T, n) * w.float()
    return (v if gate_first else v * g).to(out_dtype)


# ---------------------------------------------------------------- Lorenex-style decoders
# (gated linear attention with a decay per key channel, the selective scan, attention inputs
# made unit-RMS vectors with a position-dependent query factor, PolyNorm, clamped gated
# experts, softmax routing over all router outputs with a choice correction)
def embed_pos(ids: torch.Tensor, positions: torch.Tensor, table: torch.Tensor, scale: float,
              pos_table: Optional[torch.Tensor], out: torch.Tensor) -> torch.Tensor:
    """out fp32 [T, W] = table[ids] * scale (+ pos_table[positions])."""
    x = table[ids.long()].float() * scale
    if pos_table is not None:
        x = x + pos_table[positions.long().clamp(0, pos_table.shape[0] - 1)].float()
    out.copy_(x)
    return out


def gla_scan(proj: torch.Tensor, low: torch.Tensor, a2: torch.Tensor, a2_bias: torch.Tensor,
             state: torch.Tensor, seqs: list, H: int, d: int, dv: int, tau: float) -> torch.Tensor:
    """Gated linear attention.  proj [T, >= 2 H d + H dv] = q | k | v (| ...); low [T, r] the
    decay bottleneck; a2 fp32 [H d, r], a2_bias fp32 [H d].  Per head, with
    ln alpha = logsigmoid(a2 low + a2_bias) / tau (one decay per key channel) and q times
    d^-1/2:   S = diag(alpha) S + k v^T;  o = S^T q      (S [d, dv])
    from state[slot] [H, d, dv] fp32 (zeros at position 0), written back.  -> fp32 [T, H dv]."""
    T = proj.shape[0]
    q = proj[:, : H * d].float().view(T, H, d) * d ** -0.5
    k = proj[:, H * d: 2 * H * d].float().view(T, H, d)
    v = proj[:, 2 * H * d: 2 * H * d + H * dv].float().view(T, H, dv)
    z = low.float() @ a2.float().t() + a2_bias.float()
    alpha = torch.exp(torch.nn.functional.logsigmoid(z) / tau).view(T, H, d)
    out = torch.zeros(T, H, dv, dtype=torch.float32)
    for a, n, p0, slot in seqs:
        if slot < 0:
            continue
        S = torch.zeros(H, d, dv) if p0 == 0 else state[slot].clone()
        for t in range(a, a + n):
            S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
            out[t] = torch.einsum("hdv,hd->hv", S, q[t])
        state[slot] = S
    return out.view(T, H * dv)


def selective_scan(x: torch.Tensor, dt: torch.Tensor, bc: torch.Tensor, At: torch.Tensor,
                   dt_bias: torch.Tensor, dskip: torch.Tensor, z: torch.Tensor,
                   state: torch.Tensor, seqs: list, out_scale: float,
                   out_dtype: torch.dtype) -> torch.Tensor:
    """The selective scan.  x [T, I] (after convolution and SiLU), dt [T, I] raw step sizes,
    bc [T, 2 N] = B | C, At fp32 [N, I] (negative; states by channels), z [T, I] the gate
    pre-activation.  With d = softplus(dt + dt_bias), per channel c and state n:
        S[n, c] = exp(d_c At[n, c]) S[n, c] + d_c x_c B_n;   y_c = sum_n S[n, c] C_n + dskip_c x_c
    from state[slot] [N, I] fp32 (zeros at position 0), written back.
    -> y * silu(z) * out_scale in out_dtype [T, I]."""
    T, I = x.shape
    N = At.shape[0]
    xf = x.float()
    d = torch.nn.functional.softplus(dt.float() + dt_bias.float())
    B, C = bc[:, :N].float(), bc[:, N: 2 * N].float()
    y = torch.zeros(T, I, dtype=torch.float32)
    for a, n, p0, slot in seqs:
        if slot < 0:
            continue
        S = torch.zeros(N, I) if p0 == 0 else state[slot].clone()
        for t in range(a, a + n):
            S = torch.exp(d[t][None, :] * At.float()) * S + B[t][:, None] * (d[t] * xf[t])[None, :]
            y[t] = C[t] @ S + dskip.float() * xf[t]
        state[slot] = S
    zf = z.float()
    return (y * (zf * torch.sigmoid(zf)) * out_scale).to(out_dtype)


def norm_kv_store(qkv: torch.Tensor, positions: torch.Tensor, k_cache: torch.Tensor,
                  v_cache: torch.Tensor, slot_mapping: torch.Tensor, H: int, G: int, dk: int,
                  dv: int, eps: float, qk_unit: bool, v_unit: bool, q_temp,
                  out_dtype: torch.dtype) -> torch.Tensor:
    """qkv fp32 [T, H dk + G dk + G dv] -> q [T, H, dk] in out_dtype; k and v go to the
    plain-layout paged cache at ``slot_mapping`` (< 0: no write).  ``qk_unit`` / ``v_unit``:
    each head's vector is divided by sqrt(mean(x^2) + eps).  ``q_temp`` = (coef, every): q at
    position p times 1 + coef * ln(floor((p + 1) / every) + 1).  fp32 math."""
    T = qkv.shape[0]
    q = qkv[:, : H * dk].float().view(T, H, dk)
    k = qkv[:, H * dk: (H + G) * dk].float().view(T, G, dk)
    v = qkv[:, (H + G) * dk: (H + G) * dk + G * dv].float().view(T, G, dv)

    def unit(x):
        return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)
    if qk_unit:
        q, k = unit(q), unit(k)
    if v_unit:
        v = unit(v)
    if q_temp is not None:
        coef, every = q_temp
        p = positions.clamp(min=0)
        f = 1.0 + coef * torch.log((torch.div(p + 1, every, rounding_mode="floor") + 1).float())
        q = q * f[:, None, None]
    bs = k_cache.shape[2]
    ok = slot_mapping >= 0
    sl = slot_mapping[ok].long()
    k_cache[sl // bs, :, sl % bs] = k[ok].to(k_cache.dtype)
    v_cache[sl // bs, :, sl % bs] = v[ok].to(v_cache.dtype)
    return q.to(out_dtype)


def polynorm(z: torch.Tensor, coef: torch.Tensor, eps: float) -> torch.Tensor:
    """a N(z) + b N(z^2) + c N(z^3) + e over rows of z [T, F]: powers element by element,
    N(v) = v / sqrt(mean(v^2) + eps), coef fp32 [4] = (a, b, c, e).  fp32 math."""
    zf = z.float()

    def n(v):
        return v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps)
    c = coef.float()
    return (c[0] * n(zf) + c[1] * n(zf * zf) + c[2] * n(zf * zf * zf) + c[3]).to(z.dtype)


def swiglu_clamp(x: torch.Tensor, limit: float, alpha: float = 1.702) -> torch.Tensor:
    """x [rows, 2 I] = gate | up  ->  g sigmoid(alpha g) (u + 1) with g = min(gate, limit),
    u = clamp(up, -limit, limit)."""
    I = x.shape[-1] // 2
    g = x[..., :I].float().clamp(max=limit)
    u = x[..., I:].float().clamp(-limit, limit)
    return (g * torch.sigmoid(alpha * g) * (u + 1.0)).to(x.dtype)


def moe_route_softmax_all(logits: torch.Tensor, correction: torch.Tensor, k: int, n_real: int):
    """logits fp32 [T, E]: s = softmax over all E router outputs; the k outputs with the
    largest s + correction are chosen (lowest index first among equals) and weighted by s as
    it is.  Outputs >= n_real name identity experts: their pairs get weight 0 here and their
    scores are summed per token.  -> (weights fp32 [T, k], ids int32 [T, k], identity weight
    fp32 [T])."""
    E = correction.numel()
    s = torch.softmax(logits[:, :E].float(), dim=-1)
    ids = torch.topk(s + correction.float(), k, dim=-1).indices
    w = torch.gather(s, 1, ids)
    ident = ids >= n_real
    idw = (w * ident).sum(-1)
    return w.masked_fill(ident, 0.0), ids.to(torch.int32), idw
