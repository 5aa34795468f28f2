"""Built-in model architectures (offline: no HF download on the GPU box).

The reference deploys these models through its Helm values files
(`values-01-minimal-example.yaml:7` OPT-125m, `values-01-minimal-example2.yaml:8`
Qwen3-0.6B, `…4.yaml:8` Qwen-7B, `…5.yaml:8` Qwen3-4B, `…8.yaml:8` Qwen2.5-7B,
`…9.yaml:8` Qwen3-14B) and the north-star configs add Llama-3-8B/70B and
Mixtral-8x7B.  Dimensions are the public HF config values.

A model is resolved from (in order): a preset name, a local directory holding
an HF ``config.json`` (weights loaded from safetensors if present), or an HF
id whose basename matches a preset (``Qwen/Qwen3-0.6B`` -> ``qwen3-0.6b``).
"""
from __future__ import annotations

import dataclasses
import json
import os
from typing import Optional


@dataclasses.dataclass(frozen=True)
class WindowSpec:
    """Sliding-window visibility with kept first tokens: query i sees key j when
    j <= i and (i - j < size or j < keep_first)."""
    size: int
    keep_first: int = 0


@dataclasses.dataclass(frozen=True)
class RotarySpec:
    """Rotary embedding of ``dims`` dimensions: pair i turns by p * base^(-2i/dims).
    ``interleaved``: the pair is (2i, 2i + 1) instead of (i, i + dims/2).  ``yarn``
    (factor, original length, fast turns, slow turns): YaRN frequency interpolation --
    pairs that complete fewer than ``slow`` turns over the original length are slowed by
    ``factor``, pairs above ``fast`` turns keep their frequency, a linear ramp between --
    and cos / sin are scaled by 0.1 ln(factor) + 1."""
    dims: int
    base: float = 10000.0
    interleaved: bool = False
    yarn: Optional[tuple] = None


@dataclasses.dataclass(frozen=True)
class FeedForwardSpec:
    """A layer's feed-forward.  kind "dense": gated, down(act(gate h) * up h).  kind "moe":
    ``experts`` ungated experts down(act(up h)) of which a token uses ``top``: sigmoid
    router scores, the choice made on score + a per-expert correction, the weights the
    chosen scores over their sum times ``route_scale``; ``shared_ff`` > 0 adds an expert
    every token uses, scaled by a per-token sigmoid gate."""
    kind: str
    ff: int
    act: str = "silu"
    experts: int = 0
    top: int = 0
    route_scale: float = 1.0
    shared_ff: int = 0
    # gated: down(act(gate h) * up h); not gated: down(act(up h)).  None: the kind's usual
    # form (dense: gated, moe: ungated)
    gated: Optional[bool] = None
    # "sigmoid": the routing described above; "softmax": logits W_r h + b_r, the ``top``
    # largest chosen, their weights the softmax over the chosen logits only; "softmax_all":
    # scores = softmax over all router outputs, the choice made on score + a per-output
    # correction, the weights the chosen scores as they are
    router: str = "sigmoid"
    # act "polynorm" (dense, not gated): a N(z) + b N(z^2) + c N(z^3) + e with N = division
    # by the row's root mean square and four learned numbers.  act "swiglu_clamp" (gated):
    # g = min(gate h, limit), u = clamp(up h, -limit, limit), g sigmoid(1.702 g) (u + 1)
    limit: float = 0.0
    # the last ``identity`` router outputs (beyond ``experts``) name experts without weights
    # whose output is their input
    identity: int = 0


@dataclasses.dataclass(frozen=True)
class MixerSpec:
    """One layer of a hybrid decoder: its token mixer and (optional) feed-forward.

    kind "attention": softmax attention over a paged KV cache (GQA, per-head query/key
    size ``dim`` and value size ``vdim``, rotary on the first ``rot_dims`` dimensions,
    an optional window, an optional per-head sigmoid output gate).
    kind "mlstm": matrix-memory recurrence (one [dim, vdim] fp32 state per head and
    sequence, exponential gating capped at ``gate_cap``).
    kind "latent_attention": softmax attention whose keys and values are up-projections
    of one ``kv_rank``-wide normed latent per token; a head's query / key has ``dim``
    unrotated dimensions plus ``rot_dims`` rotated ones, the rotated key part shared by
    all heads.  The paged cache holds the latent and the rotated key part only.
    kind "mingru": an element-wise gated recurrence of ``width`` channels (one fp32 state
    vector per sequence) with a SiLU output gate.
    kind "parallel": two mixers side by side on the same input, ``left`` (an "attention"
    spec) and ``right`` (a "mamba2" or "gated_delta" spec); the result is
    left_scale * left + right_scale * right.
    kind "mamba2": the state-space-duality recurrence, ``heads`` heads of ``vdim`` channels
    with a [dim, vdim] fp32 state each (dim: the state size N), B / C shared by the heads
    of one of ``kv_heads`` groups, a causal convolution of ``conv`` taps with bias on
    x | B | C, a SiLU gate before an RMS norm in ``inner_norm_groups`` parts.
    kind "gated_delta": the gated delta rule, ``heads`` value heads over ``kv_heads``
    query / key heads, a [dim, vdim] fp32 state per head, convolutions of ``conv`` taps
    without bias on q, k and v, a per-head RMS norm and a SiLU gate after it.
    kind "gla": gated linear attention, per head S = diag(alpha) S + k v^T, o = S^T q with a
    decay per key channel alpha = sigmoid(W_a2 W_a1 h + b)^(1 / decay_tau) through a
    bottleneck of ``decay_rank``; a per-head RMS norm and a SiLU gate after it.
    kind "mamba": the selective scan, ``width`` channels with ``dim`` states each
    (S[c, n] = exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n, y_c = S[c, :] . C + D_c x_c), step
    sizes through a bottleneck of ``dt_rank``, a causal convolution of ``conv`` taps with
    bias and SiLU on x, a SiLU gate on the result."""
    kind: str
    heads: int
    dim: int
    vdim: int
    kv_heads: int = 0
    scale: Optional[float] = None
    rot_dims: int = 0
    rot_base: float = 10000.0
    window: Optional[WindowSpec] = None
    head_gate: bool = False
    gate_cap: float = 0.0
    ff: int = 0                  # 0: the layer has no feed-forward sublayer
    ff_kind: str = "dense"
    kv_rank: int = 0             # latent_attention: width of the cached latent
    width: int = 0               # mingru: recurrent channels
    rotary: Optional[RotarySpec] = None     # latent_attention (rot_dims = rotary.dims)
    mlp: Optional[FeedForwardSpec] = None   # feed-forwards other than the plain dense one
    # attention inside a parallel mixer: biases on q, k, v and the output projection, a
    # tanh cap on the scaled scores (0: none), an element-wise sigmoid gate sigmoid(W_g h)
    # on the concatenated heads; ``rotary.interleaved`` chooses the pair layout
    bias: bool = False
    softcap: float = 0.0
    elem_gate: bool = False
    conv: int = 0                # mamba2 / gated_delta: taps of the causal convolution
    inner_norm_groups: int = 1   # mamba2: parts of the gated RMS norm
    # attention inside a parallel mixer: a causal convolution of ``conv`` taps (no bias, no
    # activation) on q, k and v right after the projection; q and k (``qk_unit``) and v
    # (``v_unit``) divided by their root mean square per head; q times
    # 1 + coef * ln(floor((p + 1) / every) + 1) at position p (``q_temp`` = (coef, every));
    # ``out_bias``: whether the output projection has a bias (None: as ``bias``)
    qk_unit: bool = False
    v_unit: bool = False
    q_temp: Optional[tuple] = None
    out_bias: Optional[bool] = None
    decay_tau: float = 1.0       # gla
    decay_rank: int = 0
    dt_rank: int = 0             # mamba
    left: Optional["MixerSpec"] = None      # parallel
    right: Optional["MixerSpec"] = None
    left_scale: float = 1.0
    right_scale: float = 1.0

    @property
    def is_attention(self) -> bool:
        return self.kind in ("attention", "latent_attention")


@dataclasses.dataclass
class ModelConfig:
    name: str
    arch: str                    # "llama" | "qwen2" | "qwen3" | "qwen" | "opt" | "mixtral"
    num_layers: int
    hidden_size: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    intermediate_size: int
    vocab_size: int
    max_position: int = 8192
    rope_theta: float = 10000.0
    rope_scaling: Optional[dict] = None
    rms_eps: float = 1e-5
    tie_embeddings: bool = False
    qkv_bias: bool = False
    qk_norm: bool = False        # Qwen3 per-head q/k RMSNorm (kernel K6)
    # OPT
    norm_type: str = "rms"       # "rms" | "layer"
    act: str = "silu"            # "silu" (SwiGLU) | "relu" (OPT)
    learned_pos: bool = False
    pos_offset: int = 0
    mlp_bias: bool = False
    o_bias: bool = False
    # MoE
    num_experts: int = 0
    top_k_experts: int = 0
    bos_token_id: int = 1
    eos_token_id: int = 2
    # hybrid decoders (arch "dilavik"): one MixerSpec per layer, a grouped RMSNorm, a
    # scaled embedding and learned depth-weighted averaging of the layer results
    layer_specs: Optional[tuple] = None
    norm_groups: int = 1
    embed_scale: float = 1.0
    # arch "konovik": sublayer outputs join the stream times ``residual_mult``; layers
    # [start, stop) of ``layer_loop`` = (start, stop, times) run ``times`` times in a row
    # (own cache and state per pass); ``side_dim`` > 0: a per-layer, per-token embedding
    # of that many columns gates a small projection after every layer; every mixer input
    # is lerped towards the previous token's (``token_shift``, per-sequence state)
    residual_mult: float = 1.0
    layer_loop: Optional[tuple] = None
    side_dim: int = 0
    token_shift: bool = False
    # arch "nolesun": every sublayer's result is RMS-normed and scaled per channel before
    # it joins the stream (norm weights stored around zero); before each pass of the loop
    # x <- W_in [x; embedding output] + step[pass]
    loop_mix: bool = False
    # arch "lorenex": sublayers read the stream itself and their RMS-normed results join it
    # times ``residual_mult``; a learned position vector is added to the scaled embedding;
    # layer i runs with the weights of layer ``weights_of[i]`` (cache and state its own)
    weights_of: Optional[tuple] = None

    @property
    def q_size(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_kv_heads * self.head_dim

    @property
    def is_moe(self) -> bool:
        return self.num_experts > 0

    @property
    def has_recurrent_state(self) -> bool:
        """A layer carries per-sequence state outside the paged KV cache: cached prefix
        blocks cannot stand in for computing the prefix."""
        return self.token_shift or any(not sp.is_attention for sp in (self.layer_specs or ()))

    def layer_runs(self) -> list:
        """[(layer index, first layer of a repeated pass)] in execution order."""
        n = len(self.layer_specs) if self.layer_specs else self.num_layers
        if not self.layer_loop:
            return [(i, False) for i in range(n)]
        a, b, times = self.layer_loop
        runs = [(i, False) for i in range(a)]
        for k in range(times):
            runs += [(i, k > 0 and i == a) for i in range(a, b)]
        return runs + [(i, False) for i in range(b, n)]

    def num_params(self) -> int:
        h, i, L = self.hidden_size, self.intermediate_size, self.num_layers
        if self.layer_specs:
            n = 2 * self.vocab_size * h
            for li, sp in enumerate(self.layer_specs):
                if self.weights_of and self.weights_of[li] != li:
                    continue                # a layer that runs with another layer's tensors
                if sp.kind == "latent_attention":
                    n += h * (sp.heads * (sp.dim + sp.rot_dims) + sp.kv_rank + sp.rot_dims)
                    n += sp.kv_rank * sp.heads * (sp.dim + sp.vdim) + 2 * h * sp.heads * sp.vdim
                elif sp.kind == "mingru":
                    n += 4 * h * sp.width
                elif sp.kind == "parallel":
                    l, r = sp.left, sp.right
                    n += h * (l.heads * l.dim + l.kv_heads * (l.dim + l.vdim))
                    n += l.heads * l.vdim * h * (2 if l.elem_gate else 1)
                    if r.kind == "mamba2":
                        n += h * (3 * r.heads * r.vdim + 2 * r.kv_heads * r.dim + r.heads)
                    elif r.kind == "mamba":
                        n += 3 * h * r.width + r.width * (2 * r.dt_rank + 3 * r.dim)
                    else:
                        n += h * (2 * r.kv_heads * r.dim + 3 * r.heads * r.vdim + 2 * r.heads)
                elif sp.kind == "attention":
                    n += h * (sp.heads * sp.dim + sp.kv_heads * (sp.dim + sp.vdim) + sp.heads)
                elif sp.kind == "gla":
                    n += h * (2 * sp.heads * sp.dim + 3 * sp.heads * sp.vdim)
                    n += sp.decay_rank * (h + sp.heads * sp.dim)
                else:
                    n += h * (2 * sp.heads * sp.dim + 2 * sp.heads * sp.vdim + 2 * sp.heads)
                if sp.kind in ("attention", "mlstm"):
                    n += sp.heads * sp.vdim * h
                f = sp.mlp
                if f is None:
                    n += 2 * h * sp.ff
                elif f.kind == "dense":
                    n += (2 if f.gated is False else 3) * h * f.ff
                else:
                    n += ((3 if f.gated else 2) * h * f.experts * f.ff + 2 * h * f.shared_ff
                          + h * (f.experts + f.identity + 1))
                n += 2 * h * self.side_dim
            return n + self.vocab_size * self.side_dim * len(self.layer_specs)
        attn = h * (self.q_size + 2 * self.kv_size) + self.q_size * h
        if self.act == "silu":
            mlp = 3 * h * i
        else:
            mlp = 2 * h * i
        if self.is_moe:
            mlp = mlp * self.num_experts + h * self.num_experts
        emb = self.vocab_size * h * (1 if self.tie_embeddings else 2)
        return L * (attn + mlp) + emb

    def kv_bytes_per_token(self, dtype_bytes: int = 2) -> int:
        if self.layer_specs:
            n = {i: 0 for i in range(len(self.layer_specs))}
            for i, _ in self.layer_runs():
                n[i] += 1
            att = [(i, sp.left if sp.kind == "parallel" else sp)
                   for i, sp in enumerate(self.layer_specs) if sp.is_attention or sp.kind == "parallel"]
            return sum(n[i] * dtype_bytes * (sp.kv_rank + sp.rot_dims if sp.kind == "latent_attention"
                                             else sp.kv_heads * (sp.dim + sp.vdim))
                       for i, sp in att)
        return 2 * self.num_layers * self.num_kv_heads * self.head_dim * dtype_bytes

    def shrink(self, **kw) -> "ModelConfig":
        return dataclasses.replace(self, **kw)


_LLAMA3_SCALING = {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0,
                   "high_freq_factor": 4.0, "original_max_position_embeddings": 8192}

PRESETS: dict[str, ModelConfig] = {
    # north-star model (BASELINE configs 2, 5)
    "llama-3-8b": ModelConfig("llama-3-8b", "llama", 32, 4096, 32, 8, 128, 14336, 128256,
                              max_position=8192, rope_theta=500000.0, bos_token_id=128000,
                              eos_token_id=128001),
    "llama-3.1-8b": ModelConfig("llama-3.1-8b", "llama", 32, 4096, 32, 8, 128, 14336, 128256,
                                max_position=131072, rope_theta=500000.0,
                                rope_scaling=_LLAMA3_SCALING, bos_token_id=128000,
                                eos_token_id=128001),
    "llama-3-70b": ModelConfig("llama-3-70b", "llama", 80, 8192, 64, 8, 128, 28672, 128256,
                               max_position=8192, rope_theta=500000.0, bos_token_id=128000,
                               eos_token_id=128001),
    "mixtral-8x7b": ModelConfig("mixtral-8x7b", "mixtral", 32, 4096, 32, 8, 128, 14336, 32000,
                                max_position=32768, rope_theta=1e6, num_experts=8,
                                top_k_experts=2),
    # reference values-file models
    "opt-125m": ModelConfig("opt-125m", "opt", 12, 768, 12, 12, 64, 3072, 50272,
                            max_position=2048, norm_type="layer", act="relu",
                            learned_pos=True, pos_offset=2, qkv_bias=True, mlp_bias=True,
                            o_bias=True, tie_embeddings=True, bos_token_id=2, eos_token_id=2),
    "qwen3-0.6b": ModelConfig("qwen3-0.6b", "qwen3", 28, 1024, 16, 8, 128, 3072, 151936,
                              max_position=40960, rope_theta=1e6, rms_eps=1e-6,
                              tie_embeddings=True, qk_norm=True, bos_token_id=151643,
                              eos_token_id=151645),
    "qwen3-4b": ModelConfig("qwen3-4b", "qwen3", 36, 2560, 32, 8, 128, 9728, 151936,
                            max_position=40960, rope_theta=1e6, rms_eps=1e-6,
                            tie_embeddings=True, qk_norm=True, bos_token_id=151643,
                            eos_token_id=151645),
    "qwen3-14b": ModelConfig("qwen3-14b", "qwen3", 40, 5120, 40, 8, 128, 17408, 151936,
                             max_position=40960, rope_theta=1e6, rms_eps=1e-6,
                             qk_norm=True, bos_token_id=151643, eos_token_id=151645),
    "qwen2.5-7b": ModelConfig("qwen2.5-7b", "qwen2", 28, 3584, 28, 4, 128, 18944, 152064,
                              max_position=32768, rope_theta=1e6, rms_eps=1e-6, qkv_bias=True,
                              bos_token_id=151643, eos_token_id=151643),
    "qwen-7b": ModelConfig("qwen-7b", "qwen", 32, 4096, 32, 32, 128, 11008, 151936,
                           max_position=8192, rope_theta=10000.0, rms_eps=1e-6, qkv_bias=True,
                           bos_token_id=151643, eos_token_id=151643),
    # tiny configs for tests / CPU plumbing
    "tiny-llama": ModelConfig("tiny-llama", "llama", 2, 256, 4, 2, 64, 512, 1024,
                              max_position=2048, rope_theta=10000.0, bos_token_id=1,
                              eos_token_id=2),
    "tiny-qwen3": ModelConfig("tiny-qwen3", "qwen3", 2, 256, 4, 2, 64, 512, 1024,
                              max_position=2048, rope_theta=1e6, rms_eps=1e-6, qk_norm=True,
                              tie_embeddings=True),
    "tiny-qwen2": ModelConfig("tiny-qwen2", "qwen2", 2, 256, 4, 2, 64, 512, 1024,
                              max_position=2048, rope_theta=1e6, rms_eps=1e-6, qkv_bias=True),
    "tiny-opt": ModelConfig("tiny-opt", "opt", 2, 128, 4, 4, 32, 512, 1024, max_position=512,
                            norm_type="layer", act="relu", learned_pos=True, pos_offset=2,
                            qkv_bias=True, mlp_bias=True, o_bias=True, tie_embeddings=True),
    # TP = 8 rehearsals: 16 q / 2 kv heads of 64 (each kv head replicated on 4 ranks at
    # TP = 8; GPU kernels take head_dim 64 / 128), and Llama-3-70B's head layout (64 q / 8
    # kv, intermediate 3.5 x hidden) scaled down to head_dim 16 (CPU oracle path only)
    "tiny-llama-gqa8": ModelConfig("tiny-llama-gqa8", "llama", 2, 1024, 16, 2, 64, 2048, 1024,
                                   max_position=2048, rope_theta=500000.0, bos_token_id=1,
                                   eos_token_id=2),
    "tiny-llama-70b-shape": ModelConfig("tiny-llama-70b-shape", "llama", 2, 1024, 64, 8, 16,
                                        3584, 1024, max_position=2048, rope_theta=500000.0,
                                        rope_scaling=_LLAMA3_SCALING, bos_token_id=1,
                                        eos_token_id=2),
    "tiny-mixtral": ModelConfig("tiny-mixtral", "mixtral", 2, 256, 4, 2, 64, 384, 1024,
                                max_position=2048, rope_theta=1e6, num_experts=4,
                                top_k_experts=2),
}

def _hybrid(name: str, width: int, pattern: str, att: dict, rec: dict, ff: int, vocab: int = 32000,
            groups: int = 1) -> ModelConfig:
    """A Dilavik-architecture preset: ``pattern`` is one letter per layer ("m": mLSTM,
    "a": windowed attention); every layer has a dense feed-forward of ``ff``."""
    specs = tuple(
        MixerSpec("attention", att["heads"], att["dim"], att["vdim"], kv_heads=att["kv"],
                  scale=att["dim"] ** -0.5, rot_dims=att["rot"], rot_base=att.get("base", 1e4),
                  window=WindowSpec(att["window"], att["keep"]), head_gate=True, ff=ff)
        if c == "a" else
        MixerSpec("mlstm", rec["heads"], rec["dim"], rec["vdim"], gate_cap=rec.get("cap", 15.0), ff=ff)
        for c in pattern)
    return ModelConfig(name, "dilavik", len(specs), width, att["heads"], att["kv"], att["dim"], ff,
                       vocab, max_position=8192, layer_specs=specs, norm_groups=groups,
                       embed_scale=width ** 0.5, bos_token_id=1, eos_token_id=2)


# Benchmark pairs of equal width, depth, head layout and (to ~5 %) parameter count: a hybrid
# and the Llama-style decoder closest to it (bench.py --mode compare).  The hybrid's dense
# two-matrix feed-forward is 1.5 x the gated one's intermediate size.
PRESETS.update({
    "dilavik-w2048": _hybrid("dilavik-w2048", 2048, "maam" * 3,
                             dict(heads=16, kv=4, dim=128, vdim=128, rot=64, window=1024, keep=4),
                             dict(heads=4, dim=256, vdim=512), ff=8256),
    "llama-w2048": ModelConfig("llama-w2048", "llama", 12, 2048, 16, 4, 128, 5504, 32000,
                               max_position=8192, rope_theta=10000.0),
    "dilavik-w4096": _hybrid("dilavik-w4096", 4096, "maam" * 2,
                             dict(heads=32, kv=8, dim=128, vdim=128, rot=64, window=2048, keep=4),
                             dict(heads=8, dim=256, vdim=512), ff=21504, groups=2),
    "llama-w4096": ModelConfig("llama-w4096", "llama", 8, 4096, 32, 8, 128, 14336, 32000,
                               max_position=8192, rope_theta=500000.0),
    # tests / CPU plumbing
    "tiny-dilavik": _hybrid("tiny-dilavik", 128, "maam",
                            dict(heads=4, kv=2, dim=32, vdim=16, rot=16, window=24, keep=2),
                            dict(heads=2, dim=16, vdim=32), ff=192, vocab=1024, groups=2),
})


def _konovik(name: str, width: int, pattern: str, heads: int, gru_width: int, dense_ff: int,
             expert_ff: int, shared_ff: int, loop: Optional[tuple], window: int = 1024,
             vocab: int = 32000, rank: int = 192, dim: int = 128, rot: int = 64, vdim: int = 128,
             experts: int = 8, top: int = 2, side: int = 64) -> ModelConfig:
    """A Konovik-architecture preset: ``pattern`` is one letter per layer ("a": latent
    attention, "g": minGRU); attention layers carry the gated dense feed-forward, minGRU
    layers the routed experts (+ a shared one)."""
    rs = RotarySpec(rot, 10000.0, interleaved=True, yarn=(8.0, 4096.0, 16.0, 2.0))
    moe = FeedForwardSpec("moe", expert_ff, act="relu2", experts=experts, top=top,
                          route_scale=2.5, shared_ff=shared_ff)
    specs = tuple(
        MixerSpec("latent_attention", heads, dim, vdim, kv_heads=1, scale=(dim + rot) ** -0.5,
                  rot_dims=rot, window=WindowSpec(window), ff=dense_ff, kv_rank=rank, rotary=rs,
                  mlp=FeedForwardSpec("dense", dense_ff))
        if c == "a" else
        MixerSpec("mingru", 1, gru_width, gru_width, ff=expert_ff, width=gru_width, mlp=moe)
        for c in pattern)
    return ModelConfig(name, "konovik", len(specs), width, heads, 1, dim, dense_ff, vocab,
                       max_position=8192, rms_eps=1e-6, layer_specs=specs, residual_mult=0.5,
                       layer_loop=loop, side_dim=side, token_shift=True, bos_token_id=1,
                       eos_token_id=2)


# Konovik presets beside the equal-width hybrid / Llama presets above: the same number of
# layer runs (a looped pair counts twice), 16 / 32 heads, and a feed-forward whose ACTIVE
# parameters per token (two of eight experts + the shared one, or the gated dense one) are
# those of the Llama preset's; the cache row (192 + 64) is what the matrix-core prefill
# kernel of the windowed attention covers.
PRESETS.update({
    "konovik-w2048": _konovik("konovik-w2048", 2048, "agagagagag", 16, 4096, 5504, 2048, 1536,
                              (2, 4, 2)),
    "konovik-w4096": _konovik("konovik-w4096", 4096, "agagag", 32, 8192, 14336, 4096, 4096,
                              (2, 4, 2), window=2048),
    "tiny-konovik": _konovik("tiny-konovik", 128, "agag", 4, 192, 256, 128, 128, (1, 3, 2),
                             window=24, vocab=1024, rank=32, dim=16, rot=16, vdim=16, experts=4,
                             side=16),
})


def _nolesun(name: str, width: int, pattern: str, att: dict, ssm: dict, gdn: dict, dense_ff: int,
             expert_ff: int, loop: Optional[tuple], experts: int = 8, top: int = 2,
             vocab: int = 32000) -> ModelConfig:
    """A Nolesun-architecture preset: ``pattern`` is one letter per layer ("m": attention
    beside Mamba-2, "d": biased, capped, gated attention beside the gated delta rule; a
    capital letter: routed experts instead of the dense feed-forward)."""
    dense = FeedForwardSpec("dense", dense_ff, act="relu2", gated=False)
    moe = FeedForwardSpec("moe", expert_ff, act="silu", gated=True, experts=experts, top=top,
                          router="softmax")
    specs = []
    for c in pattern:
        two = c.lower() == "d"
        rs = RotarySpec(att["rot"], att.get("base", 1e4), interleaved=two)
        left = MixerSpec("attention", att["heads"], att["dim"], att["vdim"], kv_heads=att["kv"],
                         scale=att["dim"] ** -0.5, rot_dims=rs.dims, rot_base=rs.base, rotary=rs,
                         bias=two, softcap=30.0 if two else 0.0, elem_gate=two)
        right = (MixerSpec("gated_delta", gdn["heads"], gdn["dim"], gdn["vdim"], kv_heads=gdn["kv"],
                           conv=gdn.get("conv", 4)) if two else
                 MixerSpec("mamba2", ssm["heads"], ssm["state"], ssm["vdim"],
                           kv_heads=ssm.get("groups", 1), conv=ssm.get("conv", 4),
                           inner_norm_groups=ssm.get("norm_groups", 1)))
        mlp = moe if c.isupper() else dense
        specs.append(MixerSpec("parallel", left.heads, left.dim, left.vdim, kv_heads=left.kv_heads,
                               ff=mlp.ff, mlp=mlp, left=left, right=right,
                               left_scale=1.0, right_scale=1.0))
    return ModelConfig(name, "nolesun", len(specs), width, att["heads"], att["kv"], att["dim"],
                       dense_ff, vocab, max_position=8192, rms_eps=1e-6, layer_specs=tuple(specs),
                       embed_scale=width ** 0.5, layer_loop=loop, loop_mix=loop is not None,
                       bos_token_id=1, eos_token_id=2)


# Nolesun presets beside the equal-width hybrid / Llama presets above: the same number of
# layer runs (a looped pair counts twice), 16 / 32 attention heads of 128, and a feed-forward
# whose active parameters per token are those of the Llama preset's (the two-matrix dense one
# 1.5 x as wide as the gated one; two of eight gated experts of half its size).  Every layer
# also carries a recurrence as wide as the model (Mamba-2: heads of 64 with a state of 128;
# gated delta rule: heads of 128 x 128), so a layer has about twice a Llama layer's mixer.
PRESETS.update({
    "nolesun-w2048": _nolesun("nolesun-w2048", 2048, "mDmDmDmDmD",
                              dict(heads=16, kv=4, dim=128, vdim=128, rot=64),
                              dict(heads=32, vdim=64, state=128, groups=1),
                              dict(heads=16, kv=8, dim=128, vdim=128), 8256, 2752, (2, 4, 2)),
    "nolesun-w4096": _nolesun("nolesun-w4096", 4096, "mDmDmD",
                              dict(heads=32, kv=8, dim=128, vdim=128, rot=64),
                              dict(heads=64, vdim=64, state=128, groups=1),
                              dict(heads=32, kv=16, dim=128, vdim=128), 21504, 7168, (2, 4, 2)),
    "tiny-nolesun": _nolesun("tiny-nolesun", 128, "mDdM",
                             dict(heads=4, kv=2, dim=32, vdim=16, rot=16),
                             dict(heads=4, vdim=16, state=16, groups=2, conv=3, norm_groups=2),
                             dict(heads=4, kv=2, dim=16, vdim=16, conv=4), 192, 64, (1, 3, 2),
                             experts=4, vocab=1024),
})


def _lorenex(name: str, width: int, pattern: str, gla: dict, att: dict, ssm: dict, dense_ff: int,
             expert_ff: int, experts: int = 8, top: int = 2, identity: int = 1,
             vocab: int = 32000, share: Optional[dict] = None, max_pos: int = 8192) -> ModelConfig:
    """A Lorenex-architecture preset: ``pattern`` is one letter per layer ("g": gated linear
    attention, "p": attention beside the selective scan; a capital letter: routed experts
    instead of the dense feed-forward); ``share`` maps a layer to the layer whose weights
    it runs with."""
    dense = FeedForwardSpec("dense", dense_ff, act="polynorm", gated=False)
    moe = FeedForwardSpec("moe", expert_ff, act="swiglu_clamp", gated=True, experts=experts,
                          top=top, router="softmax_all", limit=7.0, identity=identity)
    specs = []
    for c in pattern:
        mlp = moe if c.isupper() else dense
        if c.lower() == "g":
            specs.append(MixerSpec("gla", gla["heads"], gla["dim"], gla["vdim"], ff=mlp.ff, mlp=mlp,
                                   decay_tau=gla.get("tau", 16.0), decay_rank=gla.get("rank", 16)))
            continue
        left = MixerSpec("attention", att["heads"], att["dim"], att["vdim"], kv_heads=att["kv"],
                         scale=att.get("scale", 1.0), bias=True, out_bias=False,
                         conv=att.get("conv", 4), qk_unit=True, v_unit=True,
                         q_temp=(att.get("coef", 0.5), att.get("every", 1024)))
        right = MixerSpec("mamba", 1, ssm["state"], ssm["inner"], width=ssm["inner"],
                          conv=ssm.get("conv", 4), dt_rank=ssm["dt_rank"])
        specs.append(MixerSpec("parallel", left.heads, left.dim, left.vdim, kv_heads=left.kv_heads,
                               ff=mlp.ff, mlp=mlp, left=left, right=right, left_scale=1.0,
                               right_scale=1.0))
    share = share or {}
    return ModelConfig(name, "lorenex", len(specs), width, att["heads"], att["kv"], att["dim"],
                       dense_ff, vocab, max_position=max_pos, rms_eps=1e-5, tie_embeddings=True,
                       learned_pos=True, layer_specs=tuple(specs), embed_scale=width ** 0.5,
                       residual_mult=0.5,
                       weights_of=tuple(share.get(i, i) for i in range(len(specs))),
                       bos_token_id=1, eos_token_id=2)


# Lorenex presets beside the equal-width hybrid / Llama presets above: the same number of
# layers, 16 / 32 attention heads of 128, a feed-forward whose active parameters per token are
# those of the Llama preset's (the two-matrix dense one 1.5 x as wide as the gated one; two of
# eight gated experts of half its size, plus an identity expert).  Gated-linear-attention
# layers have key size width / 2 and value size width; the selective scan beside the
# attention is as wide as the model with 16 states per channel.
PRESETS.update({
    "lorenex-w2048": _lorenex("lorenex-w2048", 2048, "gPgPgPgPgPgP",
                              dict(heads=8, dim=128, vdim=256, rank=16),
                              dict(heads=16, kv=4, dim=128, vdim=128, scale=12.0),
                              dict(inner=2048, state=16, dt_rank=128), 8256, 2752),
    "lorenex-w4096": _lorenex("lorenex-w4096", 4096, "gPgPgPgP",
                              dict(heads=16, dim=128, vdim=256, rank=16),
                              dict(heads=32, kv=8, dim=128, vdim=128, scale=12.0),
                              dict(inner=4096, state=16, dt_rank=256), 21504, 7168),
    "tiny-lorenex": _lorenex("tiny-lorenex", 128, "gPpG",
                             dict(heads=2, dim=16, vdim=32, rank=4, tau=8.0),
                             dict(heads=4, kv=2, dim=32, vdim=16, scale=6.0, conv=3, every=16),
                             dict(inner=96, state=8, dt_rank=6, conv=3), 192, 64, experts=4,
                             vocab=1024, share={2: 1}, max_pos=2048),
})


# HF repo basenames (lower-cased) -> preset
_ALIASES = {
    "meta-llama-3-8b": "llama-3-8b", "meta-llama-3-8b-instruct": "llama-3-8b",
    "llama-3-8b-instruct": "llama-3-8b", "meta-llama-3.1-8b": "llama-3.1-8b",
    "llama-3.1-8b-instruct": "llama-3.1-8b", "meta-llama-3.1-8b-instruct": "llama-3.1-8b",
    "meta-llama-3-70b": "llama-3-70b", "meta-llama-3-70b-instruct": "llama-3-70b",
    "mixtral-8x7b-v0.1": "mixtral-8x7b", "mixtral-8x7b-instruct-v0.1": "mixtral-8x7b",
    "qwen2.5-7b-instruct": "qwen2.5-7b", "qwen3-0.6b-base": "qwen3-0.6b",
}


def _mixer_spec(entry: dict) -> MixerSpec:
    """One entry of a hybrid config's ``layers`` list -> MixerSpec."""
    kind, m, mlp = entry["type"], entry["mixer"], entry.get("mlp")
    ff = int(mlp["ff"]) if mlp else 0
    ff_kind = mlp.get("kind", "dense") if mlp else "dense"
    if ff and ff_kind != "dense":
        raise ValueError(f"unsupported feed-forward kind {ff_kind!r}")
    if kind == "attention":
        rot, mask = m.get("rot"), m.get("mask")
        return MixerSpec("attention", int(m["heads"]), int(m["dim"]), int(m["vdim"]),
                         kv_heads=int(m.get("kv_heads", m["heads"])), scale=float(m["scale"]),
                         rot_dims=int(rot["dims"]) if rot else 0,
                         rot_base=float(rot["base"]) if rot else 10000.0,
                         window=WindowSpec(int(mask["size"]), int(mask.get("keep_first", 0)))
                         if mask else None,
                         head_gate=True, ff=ff, ff_kind=ff_kind)
    if kind == "mlstm":
        return MixerSpec("mlstm", int(m["heads"]), int(m["dim"]), int(m["vdim"]),
                         gate_cap=float(m["gate_cap"]), ff=ff, ff_kind=ff_kind)
    raise ValueError(f"unknown mixer type {kind!r}")


def dilavik_config(d: dict, name: str) -> ModelConfig:
    """A Dilavik config.json (``architecture``, ``width``, ``vocab``, ``layers``, ``norm``,
    ``embedding``) -> ModelConfig.  The flat attention fields describe the first attention
    layer (reporting only); the engine sizes caches and state from ``layer_specs``."""
    specs = tuple(_mixer_spec(e) for e in d["layers"])
    att = next((sp for sp in specs if sp.kind == "attention"), specs[0])
    return ModelConfig(
        name, "dilavik", len(specs), int(d["width"]), att.heads, att.kv_heads or att.heads,
        att.dim, max((sp.ff for sp in specs), default=0), int(d["vocab"]),
        max_position=int(d.get("max_position", 8192)), rope_theta=att.rot_base,
        rms_eps=float(d["norm"]["eps"]), layer_specs=specs,
        norm_groups=int(d["norm"].get("groups", 1)),
        embed_scale=float(d.get("embedding", {}).get("scale", 1.0)),
        bos_token_id=int(d.get("bos_token_id", 0)), eos_token_id=int(d.get("eos_token_id", -1)))


def _feed_forward_spec(mlp: Optional[dict]) -> Optional[FeedForwardSpec]:
    if not mlp:
        return None
    kind = mlp.get("kind", "dense")
    if kind == "dense":
        return FeedForwardSpec("dense", int(mlp["ff"]), act="silu")
    if kind == "moe":
        rt, sh = mlp["router"], mlp.get("shared")
        return FeedForwardSpec("moe", int(mlp["expert"]["ff"]), act="relu2",
                               experts=int(rt["experts"]), top=int(rt["top"]),
                               route_scale=float(rt.get("scale", 1.0)),
                               shared_ff=int(sh["ff"]) if sh else 0)
    raise ValueError(f"unsupported feed-forward kind {kind!r}")


def _konovik_spec(entry: dict) -> MixerSpec:
    kind, m = entry["type"], entry["mixer"]
    mlp = _feed_forward_spec(entry.get("mlp"))
    ff = mlp.ff if mlp else 0
    if kind == "latent_attention":
        r = int(m.get("rot_dim", 0))
        rot, mask = m.get("rot"), m.get("mask")
        rs = None
        if r:
            sc = rot.get("scaling")
            rs = RotarySpec(r, float(rot["base"]), interleaved=True,
                            yarn=(float(sc["factor"]), float(sc["original"]), float(sc["fast"]),
                                  float(sc["slow"])) if sc else None)
        return MixerSpec("latent_attention", int(m["heads"]), int(m["dim"]), int(m["vdim"]),
                         kv_heads=1, scale=float(m["scale"]), rot_dims=r,
                         rot_base=rs.base if rs else 10000.0,
                         window=WindowSpec(int(mask["size"])) if mask else None,
                         ff=ff, kv_rank=int(m["kv_rank"]), rotary=rs, mlp=mlp)
    if kind == "mingru":
        return MixerSpec("mingru", 1, int(m["width"]), int(m["width"]), ff=ff,
                         width=int(m["width"]), mlp=mlp)
    raise ValueError(f"unknown mixer type {kind!r}")


def konovik_config(d: dict, name: str) -> ModelConfig:
    """A Konovik config.json (``architecture``, ``width``, ``vocab``, ``layers``, ``loop``,
    ``norm``, ``residual_mult``, ``token_side``) -> ModelConfig."""
    specs = tuple(_konovik_spec(e) for e in d["layers"])
    att = next((sp for sp in specs if sp.is_attention), specs[0])
    lp, side = d.get("loop"), d.get("token_side")
    loop = (int(lp["start"]), int(lp["stop"]), int(lp["times"])) if lp else None
    if loop and not (0 <= loop[0] <= loop[1] <= len(specs) and loop[2] >= 1):
        raise ValueError(f"bad layer loop {loop}")
    return ModelConfig(
        name, "konovik", len(specs), int(d["width"]), att.heads, 1, att.dim,
        max((sp.ff for sp in specs), default=0), int(d["vocab"]),
        max_position=int(d.get("max_position", 8192)), rope_theta=att.rot_base,
        rms_eps=float(d["norm"]["eps"]), layer_specs=specs,
        residual_mult=float(d.get("residual_mult", 1.0)), layer_loop=loop,
        side_dim=int(side["dim"]) if side else 0, token_shift=True,
        bos_token_id=int(d.get("bos_token_id", 0)), eos_token_id=int(d.get("eos_token_id", -1)))


def _nolesun_ff(mlp: Optional[dict]) -> Optional[FeedForwardSpec]:
    if not mlp:
        return None
    kind = mlp.get("kind", "dense")
    if kind == "dense":
        return FeedForwardSpec("dense", int(mlp["ff"]), act="relu2", gated=False)
    if kind == "moe":
        rt = mlp["router"]
        return FeedForwardSpec("moe", int(mlp["expert"]["ff"]), act="silu", gated=True,
                               experts=int(rt["experts"]), top=int(rt["top"]), router="softmax")
    raise ValueError(f"unsupported feed-forward kind {kind!r}")


def _nolesun_spec(entry: dict) -> MixerSpec:
    """One entry of a Nolesun ``layers`` list.  Type "parallel": attention (pairs
    (i, i + dims/2)) beside Mamba-2; type "parallel_2": attention with biases, pairs
    (2i, 2i + 1), a score cap and an element-wise output gate beside the gated delta rule."""
    kind, m = entry["type"], entry["mixer"]
    if kind not in ("parallel", "parallel_2"):
        raise ValueError(f"unknown mixer type {kind!r}")
    two = kind == "parallel_2"
    mlp = _nolesun_ff(entry.get("mlp"))
    l, r = m["left"], m["right"]
    rot = l.get("rot")
    rs = (RotarySpec(int(rot["dims"]), float(rot["base"]), interleaved=two)
          if rot and int(rot["dims"]) else None)
    H = int(l["heads"])
    left = MixerSpec("attention", H, int(l["dim"]), int(l["vdim"]),
                     kv_heads=int(l.get("kv_heads", H)), scale=float(l["scale"]),
                     rot_dims=rs.dims if rs else 0, rot_base=rs.base if rs else 10000.0,
                     rotary=rs, bias=two, softcap=float(l.get("softcap", 0.0)) if two else 0.0,
                     elem_gate=two)
    Hr = int(r["heads"])
    if two:
        right = MixerSpec("gated_delta", Hr, int(r["dim"]), int(r["vdim"]),
                          kv_heads=int(r.get("kv_heads", Hr)), conv=int(r["conv"]))
    else:
        right = MixerSpec("mamba2", Hr, int(r["state"]), int(r["vdim"]),
                          kv_heads=int(r.get("groups", 1)), conv=int(r["conv"]),
                          inner_norm_groups=int(r.get("norm_groups", 1)))
    if left.heads % left.kv_heads or right.heads % right.kv_heads:
        raise ValueError("heads must be a multiple of the key/value heads (groups)")
    return MixerSpec("parallel", H, left.dim, left.vdim, kv_heads=left.kv_heads,
                     ff=mlp.ff if mlp else 0, mlp=mlp, left=left, right=right,
                     left_scale=float(m.get("left_scale", 1.0)),
                     right_scale=float(m.get("right_scale", 1.0)))


def nolesun_config(d: dict, name: str) -> ModelConfig:
    """A Nolesun config.json (``architecture``, ``width``, ``vocab``, ``layers``, ``loop``,
    ``norm``, ``embedding``) -> ModelConfig."""
    specs = tuple(_nolesun_spec(e) for e in d["layers"])
    lp = d.get("loop")
    loop = (int(lp["start"]), int(lp["stop"]), int(lp["times"])) if lp else None
    if loop and not (0 <= loop[0] < loop[1] <= len(specs) and loop[2] >= 1):
        raise ValueError(f"bad layer loop {loop}")
    a = specs[0].left
    return ModelConfig(
        name, "nolesun", len(specs), int(d["width"]), a.heads, a.kv_heads, a.dim,
        max((sp.ff for sp in specs), default=0), int(d["vocab"]),
        max_position=int(d.get("max_position", 8192)), rope_theta=a.rot_base,
        rms_eps=float(d["norm"]["eps"]), layer_specs=specs,
        embed_scale=float(d.get("embedding", {}).get("scale", 1.0)), layer_loop=loop,
        loop_mix=loop is not None,
        bos_token_id=int(d.get("bos_token_id", 0)), eos_token_id=int(d.get("eos_token_id", -1)))


def _lorenex_ff(mlp: Optional[dict]) -> Optional[FeedForwardSpec]:
    if not mlp:
        return None
    kind = mlp.get("kind", "dense")
    if kind == "dense":
        return FeedForwardSpec("dense", int(mlp["ff"]), act="polynorm", gated=False)
    if kind == "moe":
        rt, ex = mlp["router"], mlp["expert"]
        return FeedForwardSpec("moe", int(ex["ff"]), act="swiglu_clamp", gated=True,
                               experts=int(rt["experts"]), top=int(rt["top"]),
                               router="softmax_all", limit=float(ex["limit"]),
                               identity=int(rt.get("identity", 0)))
    raise ValueError(f"unsupported feed-forward kind {kind!r}")


def _lorenex_spec(entry: dict, rank: Optional[int]) -> MixerSpec:
    """One entry of a Lorenex ``layers`` list.  ``rank``: the bottleneck of a gated-linear-
    attention layer's decay projection, which only its tensors' shapes give."""
    kind, m = entry["type"], entry["mixer"]
    mlp = _lorenex_ff(entry.get("mlp"))
    ff = mlp.ff if mlp else 0
    if kind == "gla":
        rank = int(m["rank"]) if "rank" in m else rank
        if not rank:
            raise ValueError("a gla layer needs its decay bottleneck: mixer.rank in the config, "
                             "or the checkpoint whose <layer>.mix.a1 has that many rows")
        return MixerSpec("gla", int(m["heads"]), int(m["dim"]), int(m["vdim"]), ff=ff, mlp=mlp,
                         decay_tau=float(m["tau"]), decay_rank=rank)
    if kind != "parallel":
        raise ValueError(f"unknown mixer type {kind!r}")
    l, r = m["left"], m["right"]
    qt = l.get("q_temp")
    H = int(l["heads"])
    left = MixerSpec("attention", H, int(l["dim"]), int(l["vdim"]),
                     kv_heads=int(l.get("kv_heads", H)), scale=float(l["scale"]), bias=True,
                     out_bias=False, conv=int(l.get("conv", 0)), qk_unit=True, v_unit=True,
                     q_temp=(float(qt["coef"]), int(qt["every"])) if qt else None)
    if left.heads % left.kv_heads:
        raise ValueError("heads must be a multiple of the key/value heads")
    right = MixerSpec("mamba", 1, int(r["state"]), int(r["inner"]), width=int(r["inner"]),
                      conv=int(r["conv"]), dt_rank=int(r["dt_rank"]))
    return MixerSpec("parallel", H, left.dim, left.vdim, kv_heads=left.kv_heads, ff=ff, mlp=mlp,
                     left=left, right=right, left_scale=float(m.get("left_scale", 1.0)),
                     right_scale=float(m.get("right_scale", 1.0)))


def lorenex_config(d: dict, name: str, shapes: Optional[dict] = None) -> ModelConfig:
    """A Lorenex config.json (``architecture``, ``width``, ``vocab``, ``max_positions``,
    ``layers``, ``norm``, ``embedding``, ``residual_mult``) -> ModelConfig.  ``shapes``:
    tensor name -> shape of the checkpoint beside it, for the sizes config.json leaves to
    the tensors."""
    layers = d["layers"]
    share = []
    for i, e in enumerate(layers):
        j, seen = i, set()
        while "weights_of" in layers[j] and int(layers[j]["weights_of"]) != j:
            seen.add(j)                     # a layer may point at one that points further
            j = int(layers[j]["weights_of"])
            if not 0 <= j < len(layers) or j in seen:
                raise ValueError(f"layer {i}: bad weights_of")
        if layers[j]["type"] != e["type"]:
            raise ValueError(f"layer {i} runs with the weights of layer {j}, of another type")
        share.append(j)
    share = tuple(share)
    specs = []
    for i, e in enumerate(layers):
        a1 = (shapes or {}).get(f"l{share[i]}.mix.a1")
        specs.append(_lorenex_spec(e, int(a1[0]) if a1 else None))
    a = next((sp.left for sp in specs if sp.kind == "parallel"), specs[0])
    return ModelConfig(
        name, "lorenex", len(specs), int(d["width"]), a.heads, a.kv_heads or a.heads, a.dim,
        max((sp.ff for sp in specs), default=0), int(d["vocab"]),
        max_position=int(d.get("max_positions") or (shapes or {}).get("pos", (8192,))[0]),
        rms_eps=float(d["norm"]["eps"]),
        tie_embeddings=True, learned_pos=True, layer_specs=tuple(specs),
        embed_scale=float(d.get("embedding", {}).get("scale", 1.0)),
        residual_mult=float(d.get("residual_mult", 1.0)), weights_of=share,
        bos_token_id=int(d.get("bos_token_id", 0)), eos_token_id=int(d.get("eos_token_id", -1)))


def _tensor_shapes(path: str) -> dict:
    """Tensor name -> shape from the headers of the safetensors files in ``path``."""
    import glob
    import struct
    shapes = {}
    for fn in sorted(glob.glob(os.path.join(path, "*.safetensors"))):
        with open(fn, "rb") as f:
            (n,) = struct.unpack("<Q", f.read(8))
            for k, v in json.loads(f.read(n)).items():
                if k != "__metadata__":
                    shapes[k] = tuple(v["shape"])
    return shapes


def _from_hf_config(d: dict, name: str, path: Optional[str] = None) -> ModelConfig:
    """Map an HF config.json dict onto ModelConfig."""
    if d.get("architecture") == "Lorenex":
        return lorenex_config(d, name, _tensor_shapes(path) if path else None)
    if d.get("architecture") == "Nolesun":
        return nolesun_config(d, name)
    if d.get("architecture") == "Dilavik":
        return dilavik_config(d, name)
    if d.get("architecture") == "Konovik":
        return konovik_config(d, name)
    mt = d.get("model_type", "llama")
    if mt == "opt":
        h = d["hidden_size"]
        return ModelConfig(name, "opt", d["num_hidden_layers"], h, d["num_attention_heads"],
                           d["num_attention_heads"], h // d["num_attention_heads"], d["ffn_dim"],
                           d["vocab_size"], max_position=d.get("max_position_embeddings", 2048),
                           norm_type="layer", act="relu", learned_pos=True, pos_offset=2,
                           qkv_bias=True, mlp_bias=True, o_bias=True,
                           tie_embeddings=d.get("tie_word_embeddings", True),
                           bos_token_id=d.get("bos_token_id", 2),
                           eos_token_id=d.get("eos_token_id", 2))
    if mt == "qwen":  # Qwen v1 (trust-remote-code arch)
        h = d["hidden_size"]
        nh = d["num_attention_heads"]
        return ModelConfig(name, "qwen", d["num_hidden_layers"], h, nh, nh, h // nh,
                           d["intermediate_size"] // 2, d["vocab_size"],
                           max_position=d.get("seq_length", 8192),
                           rope_theta=d.get("rotary_emb_base", 10000.0),
                           rms_eps=d.get("layer_norm_epsilon", 1e-6), qkv_bias=True)
    nh = d["num_attention_heads"]
    h = d["hidden_size"]
    arch = {"llama": "llama", "qwen2": "qwen2", "qwen3": "qwen3", "mistral": "llama",
            "mixtral": "mixtral"}.get(mt, "llama")
    eos = d.get("eos_token_id", 2)
    if isinstance(eos, list):
        eos = eos[0]
    return ModelConfig(
        name, arch, d["num_hidden_layers"], h, nh, d.get("num_key_value_heads", nh),
        d.get("head_dim") or h // nh, d["intermediate_size"], d["vocab_size"],
        max_position=d.get("max_position_embeddings", 8192),
        rope_theta=float(d.get("rope_theta", 10000.0)), rope_scaling=d.get("rope_scaling"),
        rms_eps=d.get("rms_norm_eps", 1e-6), tie_embeddings=d.get("tie_word_embeddings", False),
        qkv_bias=(arch == "qwen2") or d.get("attention_bias", False), qk_norm=(arch == "qwen3"),
        num_experts=d.get("num_local_experts", 0), top_k_experts=d.get("num_experts_per_tok", 0),
        bos_token_id=d.get("bos_token_id", 1) or 1, eos_token_id=eos)


def resolve_model(model: str) -> tuple[ModelConfig, Optional[str]]:
    """Return (config, weights_dir_or_None) for a preset name, local dir or HF id."""
    key = model.lower().rstrip("/")
    if key in PRESETS:
        return PRESETS[key], None
    if os.path.isdir(model) and os.path.isfile(os.path.join(model, "config.json")):
        with open(os.path.join(model, "config.json")) as f:
            cfg = _from_hf_config(json.load(f), os.path.basename(model.rstrip("/")), model)
        return cfg, model
    base = os.path.basename(key)
    base = _ALIASES.get(base, base)
    if base in PRESETS:
        return PRESETS[base], None
    raise ValueError(f"unknown model {model!r}: not a preset ({sorted(PRESETS)}) and no "
                     f"config.json found at that path")
