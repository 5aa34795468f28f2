"""Nolesun: a decoder whose every layer runs an attention and a recurrence side by side.

On an fp32 residual stream x (width W), E the scaled embedding of the step's tokens:
  x = embed[token] * embed_scale
  layers [start, stop) of the loop run ``times`` times in a row with the same weights (own
  cache and state per pass); before the first layer of pass t:  x = W_in [x; E] + step[t]
  per layer run:
    h = RMSNorm(x) (1 + w_1);   y = left_scale * attention(h) + right_scale * recurrence(h)
    x += RMSNorm(y) (1 + w_1b) * ls_1
    h = RMSNorm(x) (1 + w_2);   x += RMSNorm(ff(h)) (1 + w_2b) * ls_2
  logits = head(RMSNorm(x) (1 + w_f))
Layer type "parallel": attention (pairs (i, i + dims/2)) beside Mamba-2; "parallel_2":
attention with biases, pairs (2i, 2i + 1), capped scores and an element-wise sigmoid output
gate beside the gated delta rule.  Feed-forward: down(relu(up h)^2), or softmax-routed
gated SiLU experts.  Norm weights are kept as 1 + w, and the post-norm weights times the
layer scale, so the row kernels are the ones other decoders use.  Projections run in the
activation dtype with fp32 accumulation; the stream, every norm, the loop's input mix,
rotation, softmax, routing, and everything of the recurrences past their convolutions are
fp32.

Kernel sequence per layer run (ops/__init__.py, "parallel mixers"):
  residual_norm (the previous sublayer's normed result joins x; norm) -> ONE merged
  projection GEMM for both mixers -> rope_kv_store -> window_attention (gate in its epilogue) |
  causal_conv -> ssd_scan / gated_delta_scan -> gated_rms_norm, both writing column slices
  of one buffer -> ONE output GEMM over [left | right] (the mixers' scales ride on the
  activations) -> residual_norm -> feed-forward (up GEMM -> relu_sq -> down GEMM | gate_proj
  -> moe_topk_softmax -> expert GEMMs with silu_mul).
One GPU per replica (TP = PP = 1).
"""
from __future__ import annotations

import re
from typing import Iterable, Optional

import torch
import torch.nn as nn

from .. import ops
from ..parallel.layers import ParallelLMHead, ReplicatedLinear, VocabParallelEmbedding
from ..parallel.state import get_state
from .attention import AttentionCore, ForwardContext
from .configs import ModelConfig
from .moe import SoftmaxRoutedExperts
from .recurrent import GatedDeltaCore, Mamba2Core, MambaCore


def _f32(shape, device, fill=0.0):
    return nn.Parameter(torch.full(shape, fill, dtype=torch.float32, device=device),
                        requires_grad=False)


class ReluSqMLP(nn.Module):
    """down(relu(up h)^2)."""

    def __init__(self, hidden: int, ff: int, dtype, device):
        super().__init__()
        self.up_proj = ReplicatedLinear(hidden, ff, dtype=dtype, device=device)
        self.down_proj = ReplicatedLinear(ff, hidden, dtype=dtype, device=device)

    def forward(self, h):
        return self.down_proj(ops.relu_sq(self.up_proj(h)))


class ParallelMixer(nn.Module):
    """An attention (left) and a recurrence (right) on the same input:
    left_scale * left(h) + right_scale * right(h).  Both mixers' input projections are one
    GEMM (left columns first), and both output projections one GEMM over the concatenated
    [left | right] features; the scales are applied to those features in fp32 before they
    are rounded, so the weights stay the checkpoint's.  The right mixer is Mamba-2, the gated
    delta rule or the selective scan; a layer run's state tensors are the left mixer's (its
    convolution inputs, if it has any) followed by the right mixer's."""

    def __init__(self, hidden: int, spec, eps: float, dtype, device):
        super().__init__()
        self.spec = spec
        l, r = spec.left, spec.right
        self.left = AttentionCore(l, spec.left_scale, eps, device)
        if r.kind == "mamba":
            self.right = MambaCore(r, eps, device, spec.right_scale, dtype)
        else:
            core = Mamba2Core if r.kind == "mamba2" else GatedDeltaCore
            self.right = core(r, eps, device, spec.right_scale)
        o_bias = l.bias if l.out_bias is None else l.out_bias
        self.in_proj = ReplicatedLinear(hidden, self.left.n_in + self.right.n_in, bias=l.bias,
                                        dtype=dtype, device=device)
        self.o_proj = ReplicatedLinear(self.left.n_out + self.right.n_out, hidden, bias=o_bias,
                                       dtype=dtype, device=device)
        if l.bias:                  # only the left mixer's columns carry a bias
            self.in_proj.bias.data.zero_()
        if o_bias:
            self.o_proj.bias.data.zero_()
        self.n_left_state = len(self.left.state_shapes())

    def cache_shape(self) -> tuple:
        l = self.spec.left
        return (l.kv_heads, l.dim, l.vdim)

    def state_shapes(self) -> tuple:
        return self.left.state_shapes() + self.right.state_shapes()

    def forward(self, h: torch.Tensor, positions: torch.Tensor, ctx: ForwardContext,
                cache_idx: int, state: tuple) -> torch.Tensor:
        proj = self.in_proj(h)
        feats = torch.empty(h.shape[0], self.left.n_out + self.right.n_out, dtype=h.dtype,
                            device=h.device)
        nl = self.n_left_state
        self.left(proj, 0, positions, ctx, cache_idx, feats[:, : self.left.n_out], state[:nl])
        self.right(proj, self.left.n_in, ctx, state[nl:], feats[:, self.left.n_out:])
        return self.o_proj(feats)


class NolesunLayer(nn.Module):
    def __init__(self, cfg: ModelConfig, idx: int, dtype, device):
        super().__init__()
        sp = cfg.layer_specs[idx]
        W = cfg.hidden_size
        self.idx = idx
        self.norm1 = _f32((W,), device, 1.0)        # 1 + the checkpoint's weight
        self.post1 = _f32((W,), device, 1.0)        # (1 + w_1b) * ls_1
        self.mix = ParallelMixer(W, sp, cfg.rms_eps, dtype, device)
        f = sp.mlp
        if f is None:
            self.norm2 = self.post2 = self.mlp = None
        else:
            self.norm2 = _f32((W,), device, 1.0)
            self.post2 = _f32((W,), device, 1.0)
            self.mlp = (ReluSqMLP(W, f.ff, dtype, device) if f.kind == "dense"
                        else SoftmaxRoutedExperts(W, f, dtype, device))


class NolesunForCausalLM(nn.Module):
    def __init__(self, cfg: ModelConfig, dtype=torch.bfloat16, device=None):
        super().__init__()
        s = get_state()
        assert s.tp_size == 1 and s.pp_size == 1, "Nolesun runs on one GPU per replica"
        self.cfg, self.dtype = cfg, dtype
        self.start, self.end = 0, cfg.num_layers
        self.first = self.last = True
        W, L = cfg.hidden_size, cfg.num_layers
        self.embed_tokens = VocabParallelEmbedding(cfg.vocab_size, W, dtype, device)
        self.layers = nn.ModuleList([NolesunLayer(cfg, i, dtype, device) for i in range(L)])
        self.final_norm = _f32((W,), device, 1.0)
        self.lm_head = ParallelLMHead(cfg.vocab_size, W, dtype, device)
        # execution order: (layer, run index = cache and state index, pass number when the
        # run opens a pass of the loop, else -1)
        lp = cfg.layer_loop
        order = []
        if lp:
            a, b, times = lp
            order = [(i, -1) for i in range(a)]
            for t in range(times):
                order += [(i, t if i == a else -1) for i in range(a, b)]
            order += [(i, -1) for i in range(b, L)]
            self.loop_in_x = _f32((W, W), device)       # W_in's columns for x
            self.loop_in_e = _f32((W, W), device)       # ... and for the embedding output
            self.loop_step = _f32((lp[2], W), device)
        else:
            order = [(i, -1) for i in range(L)]
            self.loop_in_x = self.loop_in_e = self.loop_step = None
        self.runs = [(i, n, t) for n, (i, t) in enumerate(order)]
        self._w_parts: dict = {}     # checkpoint tensors that combine into one parameter
        self.stream = self.embed_out = None     # [Tcap, W] fp32 step buffers

    # ------------------------------------------------------------------ engine hooks
    @property
    def num_local_layers(self) -> int:
        return len(self.runs)

    def local_kv_heads(self) -> int:
        return max(sp.left.kv_heads for sp in self.cfg.layer_specs)

    def cache_layout(self) -> list:
        """(kv heads, key size, value size) of every layer run's paged cache."""
        return [self.layers[i].mix.cache_shape() for i, _, _ in self.runs]

    def state_layout(self) -> list:
        """Per layer run, the per-slot shapes of its state tensors (convolution inputs,
        recurrent state)."""
        return [self.layers[i].mix.state_shapes() for i, _, _ in self.runs]

    def prepare(self, max_pos: int, max_tokens: int, device) -> None:
        """Rotary tables for ``max_pos`` positions and the step buffers for ``max_tokens``
        rows (static, so captured decode graphs replay over them)."""
        tables: dict = {}
        for l in self.layers:
            l.mix.left.prepare(tables, max_pos, device)
        W = self.cfg.hidden_size
        self.stream = torch.zeros(max_tokens, W, dtype=torch.float32, device=device)
        self.embed_out = (torch.zeros(max_tokens, W, dtype=torch.float32, device=device)
                          if self.loop_step is not None else None)

    @torch.no_grad()
    def init_random(self, seed: int = 0, std: float = 0.02) -> None:
        """Random weights for benchmarking: projections ~ N(0, std), norm weights near 1,
        decays and step sizes in the range trained models use."""
        g = torch.Generator(device="cpu").manual_seed(seed)

        def rnd(p, scale, base=0.0):
            p.copy_((torch.randn(p.shape, generator=g) * scale + base).to(p.device, p.dtype))
        W = self.cfg.hidden_size
        for name, p in self.named_parameters():
            leaf = name.rsplit(".", 1)[-1]
            if leaf in ("norm1", "norm2", "final_norm", "norm_weight"):
                rnd(p, 0.05, 1.0)
            elif leaf in ("post1", "post2"):
                rnd(p, 0.02, 0.5)
            elif leaf == "a_log":
                p.copy_(torch.log(1.0 + 7.0 * torch.rand(p.shape, generator=g)).to(p.device))
            elif leaf == "dt_bias":
                rnd(p, 0.5, -2.0)
            elif leaf == "dskip":
                rnd(p, 0.1, 1.0)
            elif leaf == "conv_w":
                rnd(p, 0.3)
            elif leaf in ("conv_b", "router_bias", "loop_step", "bias"):
                rnd(p, 0.02)
            elif leaf in ("loop_in_x", "loop_in_e"):
                rnd(p, 0.5 * W ** -0.5)
                p.diagonal().add_(0.5)
            elif leaf == "router":
                rnd(p, 0.2)
            else:
                rnd(p, std)

    # ------------------------------------------------------------------ forward
    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor, ctx: ForwardContext,
                hidden=None, residual=None, taps: Optional[list] = None):
        """-> the final-normed hidden rows.  ``taps``: the residual stream after every
        layer run is appended (fp32 copies; debugging and tests)."""
        cfg = self.cfg
        T = input_ids.shape[0]
        if self.stream is None or self.stream.shape[0] < T:
            self.prepare(cfg.max_position, max(T, 1), input_ids.device)
        eps, dt = cfg.rms_eps, self.dtype
        x = self.stream[:T]
        torch.mul(self.embed_tokens(input_ids), cfg.embed_scale, out=x)
        side = None
        if self.loop_step is not None:
            self.embed_out[:T].copy_(x)
            # W_in [x; E] = W_x x + W_e E: the second product is the same for every pass
            side = self.embed_out[:T] @ self.loop_in_e.t()
        y = post = None                     # a sublayer result that has not joined x yet
        for i, n, t in self.runs:
            layer = self.layers[i]
            if t >= 0:
                if y is not None:
                    ops.residual_norm(x, y, 1.0, None, eps, None, add_norm_w=post)
                    y = post = None
                x.copy_(torch.addmm(side + self.loop_step[t], x, self.loop_in_x.t()))
            h = ops.residual_norm(x, y, 1.0, layer.norm1, eps, dt, add_norm_w=post)
            y, post = layer.mix(h, positions, ctx, n, ctx.states[n]), layer.post1
            if layer.mlp is not None:
                h = ops.residual_norm(x, y, 1.0, layer.norm2, eps, dt, add_norm_w=post)
                y, post = layer.mlp(h), layer.post2
            if taps is not None:
                ops.residual_norm(x, y, 1.0, None, eps, None, add_norm_w=post)
                y = post = None
                taps.append(x.clone())
        return ops.residual_norm(x, y, 1.0, self.final_norm, eps, dt, add_norm_w=post)

    def compute_logits(self, hidden: torch.Tensor, gather: bool = True) -> torch.Tensor:
        return self.lm_head(hidden, gather)

    # ------------------------------------------------------------------ weights
    def load_weights(self, weights: Iterable[tuple[str, torch.Tensor]]) -> int:
        """Checkpoint names: ``embed``, ``head``, ``final.norm``, ``loop.in``, ``loop.step``
        and per layer i ``l<i>.norm1|norm1b|norm2|norm2b|ls1|ls2``, ``l<i>.mix.left.*``,
        ``l<i>.mix.right.*``, ``l<i>.mlp.*``.  Returns the number loaded and raises on a
        name it does not know."""
        n = 0
        for name, w in weights:
            if not self._load_one(name, w):
                raise KeyError(f"unexpected tensor {name!r} in a Nolesun checkpoint")
            n += 1
        return n

    def _combine(self, key: str, a: str, b: str, w: torch.Tensor, which: str, tgt, fn) -> bool:
        """Two checkpoint tensors (``a`` and ``b``) that form one parameter: keep the first
        that arrives, write ``fn(a, b)`` when both are there."""
        parts = self._w_parts.setdefault(key, {})
        parts[which] = w.float()
        if a in parts and b in parts:
            tgt.data.copy_(fn(parts[a], parts[b]).to(tgt.device))
            del self._w_parts[key]
        return True

    def _load_one(self, name: str, w: torch.Tensor) -> bool:
        dt = self.dtype
        if name == "embed":
            self.embed_tokens.weight.weight_loader(self.embed_tokens.weight, w.to(dt))
            return True
        if name == "head":
            self.lm_head.weight.weight_loader(self.lm_head.weight, w.to(dt))
            return True
        if name == "final.norm":
            self.final_norm.data.copy_(1.0 + w.float())
            return True
        if name == "loop.in" and self.loop_step is not None:
            W = self.cfg.hidden_size
            self.loop_in_x.data.copy_(w.float()[:, :W])
            self.loop_in_e.data.copy_(w.float()[:, W:])
            return True
        if name == "loop.step" and self.loop_step is not None:
            self.loop_step.data.copy_(w.float())
            return True
        mm = re.match(r"l(\d+)\.(.*)", name)
        if mm is None or int(mm.group(1)) >= len(self.layers):
            return False
        layer, rest = self.layers[int(mm.group(1))], mm.group(2)
        sp, mix = self.cfg.layer_specs[layer.idx], layer.mix
        if rest in ("norm1", "norm2"):
            p = getattr(layer, rest)
            if p is None:
                return False
            p.data.copy_(1.0 + w.float())
            return True
        for nb, ls, post in (("norm1b", "ls1", layer.post1), ("norm2b", "ls2", layer.post2)):
            if rest in (nb, ls):
                return post is not None and self._combine(
                    f"{layer.idx}.{nb}", nb, ls, w, rest, post, lambda a, b: (1.0 + a) * b)
        if rest.startswith("mix.left."):
            return self._load_left(mix, sp, rest[9:], w)
        if rest.startswith("mix.right."):
            return self._load_right(layer.idx, mix, sp, rest[10:], w)
        if not rest.startswith("mlp.") or layer.mlp is None:
            return False
        f, mlp, leaf = sp.mlp, layer.mlp, rest[4:]
        if f.kind == "dense":
            tgt = {"up": mlp.up_proj.weight, "down": mlp.down_proj.weight}.get(leaf)
            if tgt is None:
                return False
            tgt.data.copy_(w.to(dt))
            return True
        me = re.match(r"e(\d+)\.(gate|up|down)$", leaf)
        if me:
            e, which = int(me.group(1)), me.group(2)
            if e >= f.experts:
                return False
            if which == "down":
                mlp.w2.data[e].copy_(w.to(dt))
            else:
                mlp.w13.data[e].narrow(0, 0 if which == "gate" else f.ff, f.ff).copy_(w.to(dt))
            return True
        if leaf == "router":
            mlp.router.data.copy_(w.to(dt))
        elif leaf == "router.b":
            mlp.router_bias.data.copy_(w.float())
        else:
            return False
        return True

    def _load_left(self, mix: ParallelMixer, sp, leaf: str, w: torch.Tensor) -> bool:
        dt, l = self.dtype, sp.left
        H, G, dk, dv = l.heads, l.kv_heads, l.dim, l.vdim
        off = {"q": (0, H * dk), "k": (H * dk, G * dk), "v": ((H + G) * dk, G * dv)}
        if l.elem_gate:
            off["g"] = ((H + G) * dk + G * dv, H * dv)
        base = leaf[:-2] if leaf.endswith(".b") else leaf
        if base in off and (leaf == base or (l.bias and base != "g")):
            a, n = off[base]
            tgt = mix.in_proj.weight if leaf == base else mix.in_proj.bias
            tgt.data.narrow(0, a, n).copy_(w.to(dt))
            return True
        if leaf == "o":
            mix.o_proj.weight.data[:, : mix.left.n_out].copy_(w.to(dt))
            return True
        if leaf == "o.b" and l.bias:
            # left_scale * (W_o f + b) = W_o (left_scale f) + left_scale b
            mix.o_proj.bias.data.copy_((sp.left_scale * w.float()).to(dt))
            return True
        return False

    def _load_right(self, idx: int, mix: ParallelMixer, sp, leaf: str, w: torch.Tensor) -> bool:
        dt, r, core = self.dtype, sp.right, mix.right
        c0 = mix.left.n_in
        P = mix.in_proj.weight.data
        if leaf == "o":
            mix.o_proj.weight.data[:, mix.left.n_out:].copy_(w.to(dt))
            return True
        if leaf in ("dt_bias", "A_log"):
            (core.dt_bias if leaf == "dt_bias" else core.a_log).data.copy_(w.float())
            return True
        if r.kind == "mamba2":
            if leaf == "in":
                P[c0: c0 + core.n_in].copy_(w.to(dt))
            elif leaf == "conv":
                core.conv_w.data.copy_(w.float())
            elif leaf == "conv.b":
                core.conv_b.data.copy_(w.float())
            elif leaf == "D":
                core.dskip.data.copy_(w.float())
            elif leaf == "norm":
                core.norm_weight.data.copy_(w.float() * sp.right_scale)
            else:
                return False
            return True
        H, G, d, dv = r.heads, r.kv_heads, r.dim, r.vdim
        nc = core.n_conv
        off = {"q": (0, G * d), "k": (G * d, G * d), "v": (2 * G * d, H * dv), "g": (nc, H * dv),
               "b": (nc + H * dv, H), "a": (nc + H * dv + H, H)}
        if leaf in off:
            a, n = off[leaf]
            P[c0 + a: c0 + a + n].copy_(w.to(dt))
        elif leaf.endswith(".conv") and leaf[:-5] in ("q", "k", "v"):
            a, n = off[leaf[:-5]]
            core.conv_w.data[a: a + n].copy_(w.float())
        elif leaf == "norm":
            core.norm_weight.data.copy_((w.float() * sp.right_scale).repeat(H))
        else:
            return False
        return True
