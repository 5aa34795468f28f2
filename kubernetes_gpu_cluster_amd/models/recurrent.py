"""Recurrent token mixers: layers whose memory is a fixed-size per-sequence state
instead of a growing KV cache.

The engine gives every running sequence a state slot (the sequence's block-table row
index, ``engine/block_manager.py``); a layer's state tensors hold one entry per slot
(``ModelRunner.init_kv_cache``), and a step's ``AttnMetadata.state_slots`` names the slot
of each step sequence.  A sequence's first token (position 0) starts from the zero state,
so a slot is reused, and a preempted sequence recomputed, without any clearing pass.
State is fp32 and carried from step to step: chunked prefill and decode rows run through
the same scan kernel.
"""
from __future__ import annotations

import torch
import torch.nn as nn

from .. import ops
from ..parallel.layers import ReplicatedLinear
from .attention import ForwardContext


class MLSTMMixer(nn.Module):
    """Matrix-memory LSTM (the mLSTM of xLSTM): per head a [dim, vdim] memory S, a
    normaliser n and a running log-scale m (starting at 0).  With capped log gates
    i = cap tanh((W_i h + b_i) / cap) and f = logsigmoid(cap tanh((W_f h + b_f) / cap)):
        m' = max(f + m, i);  S' = e^(f + m - m') S + e^(i - m') k v^T;  n' likewise with k
        o  = S'^T q / (max(|n'.q|, e^(-m')) + 1e-6),   q scaled by dim^-1/2
    then each head's o over its RMS, times a learned weight, times sigmoid(W_g h), and the
    output projection.  The gates, the scan and the head norm run in fp32."""

    def __init__(self, hidden: int, spec, state_idx: int, eps: float, dtype, device):
        super().__init__()
        self.spec, self.state_idx, self.eps = spec, state_idx, eps
        H, d, dv = spec.heads, spec.dim, spec.vdim
        # q | k | v | output-gate pre-activation, one GEMM
        self.qkvg_proj = ReplicatedLinear(hidden, 2 * H * d + 2 * H * dv, dtype=dtype,
                                          device=device)
        self.o_proj = ReplicatedLinear(H * dv, hidden, dtype=dtype, device=device)
        # log input gates | log forget gates
        self.if_weight = nn.Parameter(torch.zeros(2 * H, hidden, dtype=dtype, device=device),
                                      requires_grad=False)
        self.if_bias = nn.Parameter(torch.zeros(2 * H, dtype=torch.float32, device=device),
                                    requires_grad=False)
        self.norm_weight = nn.Parameter(torch.ones(H * dv, dtype=torch.float32, device=device),
                                        requires_grad=False)

    def state_shapes(self) -> tuple:
        """Per-slot shapes of the state tensors S, n, m."""
        sp = self.spec
        return ((sp.heads, sp.dim, sp.vdim), (sp.heads, sp.dim), (sp.heads,))

    def forward(self, h: torch.Tensor, positions: torch.Tensor, ctx: ForwardContext):
        sp = self.spec
        H, d, dv = sp.heads, sp.dim, sp.vdim
        qkvg = self.qkvg_proj(h)
        gates = ops.gate_proj(h, self.if_weight, self.if_bias, ops.GATE_CAP_TANH,
                              ops.GATE_LOGSIG_CAP_TANH, H, sp.gate_cap)
        o = ops.mlstm_scan(qkvg, gates, ctx.states[self.state_idx], ctx.attn, H, d, dv)
        g = qkvg[:, 2 * H * d + H * dv:]
        return self.o_proj(ops.head_norm_gate(o, g, self.norm_weight, H, self.eps, h.dtype))


class MinGRUMixer(nn.Module):
    """minGRU: an element-wise gated recurrence whose gates read only the current token.
    z = sigmoid(W_z h + b_z); u = W_x h + b_x; candidate = u + 1/2 (u >= 0) or sigmoid(u);
    S_t = (1 - z) S_(t-1) + z candidate; output W_o (S_t * silu(W_g h)).  One merged
    projection yields z | u | g; biases, gates and the state (fp32 [slots, width]) stay in
    fp32.  The state slot tensor of a layer run is chosen at call time."""

    def __init__(self, hidden: int, spec, dtype, device):
        super().__init__()
        self.spec = spec
        n = spec.width
        self.zxg_proj = ReplicatedLinear(hidden, 3 * n, dtype=dtype, device=device)
        self.o_proj = ReplicatedLinear(n, hidden, dtype=dtype, device=device)
        self.zx_bias = nn.Parameter(torch.zeros(2 * n, dtype=torch.float32, device=device),
                                    requires_grad=False)

    def state_shapes(self) -> tuple:
        return ((self.spec.width,),)

    def forward(self, h: torch.Tensor, positions: torch.Tensor, ctx: ForwardContext,
                state: torch.Tensor):
        y = ops.mingru_scan(self.zxg_proj(h), self.zx_bias, state, ctx.attn, self.spec.width,
                            h.dtype)
        return self.o_proj(y)


class Mamba2Core(nn.Module):
    """The Mamba-2 (state-space duality) mixer between its projections.  Its projection
    columns are z | x | B | C | dt (inner = heads * vdim for z and x, groups * N each for B
    and C, one dt per head).  x | B | C pass a causal convolution with bias and SiLU (the
    last taps - 1 inputs are per-sequence state); per head, with d = softplus(dt + dt_bias)
    and a = exp(-exp(A_log) d):  S = a S + d B x^T,  y = S^T C + D x  (S [N, vdim], fp32,
    per-sequence state); y * silu(z) is RMS-normed in ``inner_norm_groups`` parts, times a
    weight (times ``out_scale``), and written into a column slice of the output
    projection's input."""

    def __init__(self, spec, eps: float, device, out_scale: float = 1.0):
        super().__init__()
        self.spec, self.eps, self.out_scale = spec, eps, float(out_scale)
        H, P, N, G = spec.heads, spec.vdim, spec.dim, spec.kv_heads
        assert H % G == 0 and (H * P) % spec.inner_norm_groups == 0
        self.inner = H * P
        self.n_conv = self.inner + 2 * G * N
        self.n_in = self.inner + self.n_conv + H
        self.n_out = self.inner
        f = lambda *s: nn.Parameter(torch.zeros(*s, dtype=torch.float32, device=device),  # noqa: E731
                                    requires_grad=False)
        self.conv_w, self.conv_b = f(self.n_conv, spec.conv), f(self.n_conv)
        self.dt_bias, self.a_log, self.dskip = f(H), f(H), f(H)
        self.norm_weight = f(self.inner)         # the checkpoint's weight times out_scale

    def state_shapes(self) -> tuple:
        """Per-slot shapes: the convolution's last inputs, the recurrent state."""
        sp = self.spec
        return ((max(sp.conv - 1, 1), self.n_conv), (sp.heads, sp.dim, sp.vdim))

    def forward(self, proj: torch.Tensor, col0: int, ctx: ForwardContext, state: tuple,
                out: torch.Tensor) -> None:
        sp = self.spec
        z = proj[:, col0: col0 + self.inner]
        xbc = ops.causal_conv(proj[:, col0 + self.inner: col0 + self.inner + self.n_conv],
                              self.conv_w, self.conv_b, state[0], ctx.attn)
        dt = proj[:, col0 + self.inner + self.n_conv: col0 + self.n_in]
        y = ops.ssd_scan(xbc, dt, self.a_log, self.dt_bias, self.dskip, state[1], ctx.attn,
                         sp.heads, sp.vdim, sp.dim, sp.kv_heads)
        ops.gated_rms_norm(y, z, self.norm_weight, sp.inner_norm_groups, self.eps, True, out)


class GatedDeltaCore(nn.Module):
    """The gated delta rule mixer between its projections.  Its projection columns are
    q | k (kv_heads * dim each) | v | output gate (heads * vdim each) | b | a (one per
    head).  q | k | v pass a causal convolution without bias and SiLU; q and k become unit
    vectors per head, q times dim^-1/2; with beta = sigmoid(b) and
    g = exp(-exp(A_log) softplus(a + dt_bias)):  S = g S;  u = beta (v - S^T k);
    S = S + k u^T;  o = S^T q  (S [dim, vdim], fp32, per-sequence state).  Each head's o
    over its RMS, times a weight shared by the heads (times ``out_scale``), times
    silu(output gate), into a column slice of the output projection's input."""

    def __init__(self, spec, eps: float, device, out_scale: float = 1.0):
        super().__init__()
        self.spec, self.eps, self.out_scale = spec, eps, float(out_scale)
        H, G, d, dv = spec.heads, spec.kv_heads, spec.dim, spec.vdim
        assert H % G == 0
        self.n_conv = 2 * G * d + H * dv
        self.n_in = self.n_conv + H * dv + 2 * H
        self.n_out = H * dv
        f = lambda *s: nn.Parameter(torch.zeros(*s, dtype=torch.float32, device=device),  # noqa: E731
                                    requires_grad=False)
        self.conv_w = f(self.n_conv, spec.conv)
        self.dt_bias, self.a_log = f(H), f(H)
        self.norm_weight = f(H * dv)             # the shared weight per head, times out_scale

    def state_shapes(self) -> tuple:
        sp = self.spec
        return ((max(sp.conv - 1, 1), self.n_conv), (sp.heads, sp.dim, sp.vdim))

    def forward(self, proj: torch.Tensor, col0: int, ctx: ForwardContext, state: tuple,
                out: torch.Tensor) -> None:
        sp = self.spec
        qkv = ops.causal_conv(proj[:, col0: col0 + self.n_conv], self.conv_w, None, state[0],
                              ctx.attn)
        g = proj[:, col0 + self.n_conv: col0 + self.n_conv + self.n_out]
        ba = proj[:, col0 + self.n_conv + self.n_out: col0 + self.n_in]
        o = ops.gated_delta_scan(qkv, ba, self.a_log, self.dt_bias, state[1], ctx.attn,
                                 sp.heads, sp.kv_heads, sp.dim, sp.vdim)
        ops.gated_rms_norm(o, g, self.norm_weight, sp.heads, self.eps, False, out)


class GLAMixer(nn.Module):
    """Gated linear attention: per head a [dim, vdim] fp32 state with one decay per key
    channel.  q = W_q h * dim^-1/2, k = W_k h, v = W_v h;
    alpha = sigmoid(W_a2 (W_a1 h) + b)^(1 / tau), laid out heads x dim;
        S = diag(alpha) S + k v^T,   o = S^T q
    then each head's o over its RMS, times a weight shared by the heads, the concatenated
    heads times silu(W_g h), and the output projection.  One merged projection yields
    q | k | v | g | the decay bottleneck; the second decay projection (a few columns wide)
    runs inside the scan kernel in fp32, so the decay's logarithm never passes 16 bits."""

    def __init__(self, hidden: int, spec, eps: float, dtype, device):
        super().__init__()
        self.spec, self.eps = spec, eps
        H, d, dv, r = spec.heads, spec.dim, spec.vdim, spec.decay_rank
        assert r >= 1
        self.n_qkv, self.n_g = 2 * H * d + H * dv, H * dv
        self.proj = ReplicatedLinear(hidden, self.n_qkv + self.n_g + r, dtype=dtype, device=device)
        self.o_proj = ReplicatedLinear(H * dv, hidden, dtype=dtype, device=device)
        f = lambda *s: nn.Parameter(torch.zeros(*s, dtype=torch.float32, device=device),  # noqa: E731
                                    requires_grad=False)
        self.a2, self.a2_bias = f(H * d, r), f(H * d)
        self.norm_weight = f(H * dv)            # the shared per-head weight, repeated

    def state_shapes(self) -> tuple:
        sp = self.spec
        return ((sp.heads, sp.dim, sp.vdim),)

    def cache_shape(self):
        return None

    def forward(self, h: torch.Tensor, positions: torch.Tensor, ctx: ForwardContext,
                cache_idx: int, state: tuple) -> torch.Tensor:
        sp = self.spec
        proj = self.proj(h)
        o = ops.gla_scan(proj, proj[:, self.n_qkv + self.n_g:], self.a2, self.a2_bias, state[0],
                         ctx.attn, sp.heads, sp.dim, sp.vdim, sp.decay_tau)
        feats = torch.empty(h.shape[0], self.n_g, dtype=h.dtype, device=h.device)
        ops.gated_rms_norm(o, proj[:, self.n_qkv: self.n_qkv + self.n_g], self.norm_weight,
                           sp.heads, self.eps, False, feats)
        return self.o_proj(feats)


class MambaCore(nn.Module):
    """The selective-scan (Mamba) mixer between its outer projections.  Its projection
    columns are x | z (``width`` channels each).  x passes a causal convolution with bias and
    SiLU (the last taps - 1 inputs are per-sequence state); W_x x = dt | B | C (dt_rank, N,
    N); d = softplus(W_dt dt + dt_bias) per channel; with A = -exp(A_log) [width, N]:
        S[c, n] = exp(d_c A[c, n]) S[c, n] + d_c x_c B_n,   y_c = S[c, :] . C + D_c x_c
    (S fp32, per-sequence state, kept as [N, width] like A so that loads run along the
    channels); y * silu(z) (times ``out_scale``) is written into a column
    slice of the output projection's input.  The two inner projections are GEMMs; step
    sizes, decays and the state are fp32."""

    def __init__(self, spec, eps: float, device, out_scale: float = 1.0, dtype=torch.bfloat16):
        super().__init__()
        self.spec, self.out_scale = spec, float(out_scale)
        I, N, R = spec.width, spec.dim, spec.dt_rank
        self.n_in, self.n_out = 2 * I, I
        self.x_proj = ReplicatedLinear(I, R + 2 * N, dtype=dtype, device=device)
        self.dt_proj = ReplicatedLinear(R, I, dtype=dtype, device=device)
        f = lambda *s: nn.Parameter(torch.zeros(*s, dtype=torch.float32, device=device),  # noqa: E731
                                    requires_grad=False)
        self.conv_w, self.conv_b = f(I, spec.conv), f(I)
        self.A = f(N, I)                         # -exp(A_log), states by channels
        self.dt_bias, self.dskip = f(I), f(I)

    def state_shapes(self) -> tuple:
        """Per-slot shapes: the convolution's last inputs, the recurrent state."""
        sp = self.spec
        return ((max(sp.conv - 1, 1), sp.width), (sp.dim, sp.width))

    def forward(self, proj: torch.Tensor, col0: int, ctx: ForwardContext, state: tuple,
                out: torch.Tensor) -> None:
        sp = self.spec
        I, R = sp.width, sp.dt_rank
        x = ops.causal_conv(proj[:, col0: col0 + I], self.conv_w, self.conv_b, state[0],
                            ctx.attn, True, proj.dtype)
        dbc = self.x_proj(x)
        dt = self.dt_proj(dbc[:, :R])
        ops.selective_scan(x, dt, dbc[:, R:], self.A, self.dt_bias, self.dskip,
                           proj[:, col0 + I: col0 + 2 * I], state[1], ctx.attn, self.out_scale,
                           out)
