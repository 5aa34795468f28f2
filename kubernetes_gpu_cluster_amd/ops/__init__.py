"""Fused ops: gfx950 HIP kernels (``torch.ops.kgc``) for GPU tensors, the
pure-PyTorch reference (``ops.reference``) for CPU tensors.

There is exactly one GPU implementation per op.  If a GPU tensor reaches an op
and the in-tree extension ``_kgc_ops.so`` is not loadable, the op raises: there
is no silent eager fallback on the GPU path.
"""
from __future__ import annotations

import math
import os
from typing import Optional

import torch

from . import reference as ref

# KGC_HIP_DEBUG=1: the bounds-checking build (``KGC_HIP_DEBUG=1 python csrc/build.py``)
DEBUG = os.environ.get("KGC_HIP_DEBUG", "0") not in ("", "0")
_SO = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))),
                   "_kgc_ops_debug.so" if DEBUG else "_kgc_ops.so")
# KGC_OPS_SO=path: another build of the same library (same-box A/B of two kernel builds)
_SO = os.environ.get("KGC_OPS_SO") or _SO
_loaded: Optional[bool] = None
_load_err: Optional[str] = None


def load_extension(strict: bool = False) -> bool:
    """Load the HIP kernel library once.  strict=True raises if unavailable."""
    global _loaded, _load_err
    if _loaded is None:
        try:
            if not os.path.exists(_SO):
                raise FileNotFoundError(f"{_SO} not built (run `python csrc/build.py`)")
            torch.ops.load_library(_SO)
            _loaded = True
        except Exception as e:  # noqa: BLE001 - report reason on use
            _loaded, _load_err = False, f"{type(e).__name__}: {e}"
    if strict and not _loaded:
        raise RuntimeError(f"kgc HIP extension unavailable: {_load_err}")
    return bool(_loaded)


def extension_path() -> str:
    return _SO


class KernelDebugCheckFailed(RuntimeError):
    """A debug-build kernel read an out-of-range block-table entry, slot or length."""


def debug_check() -> None:
    """Debug build: raise if any K1/K2/K3 bounds check tripped since the last call (the
    kernel printed the offending value and clamped it).  No-op in release builds."""
    if not DEBUG or not load_extension():
        return
    torch.cuda.synchronize()
    err = int(torch.ops.kgc.debug_errors())
    if err:
        which = [n for b, n in ((1, "paged decode (K1)"), (2, "prefill attention (K2)"),
                                (4, "rope / KV write (K3)")) if err & b]
        raise KernelDebugCheckFailed(f"device bounds check failed in {', '.join(which)}; "
                                     f"see the kernel's printf above")


def _k():
    load_extension(strict=True)
    return torch.ops.kgc


def _gpu(t: torch.Tensor) -> bool:
    return t.is_cuda


def fused_small_m_enabled() -> bool:
    """KGC_FUSED_SMALL_M=0 turns off the fused small-batch decoder layer (models/llama.py)."""
    return os.environ.get("KGC_FUSED_SMALL_M", "1") != "0"


# ------------------------------------------------------------------ norms
def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float,
             out: Optional[torch.Tensor] = None) -> torch.Tensor:
    if not _gpu(x):
        r = ref.rms_norm(x, w, eps)
        if out is not None:
            out.copy_(r)
            return out
        return r
    x2 = x.reshape(-1, x.shape[-1]) if x.is_contiguous() else x
    out = torch.empty(x2.shape, dtype=x.dtype, device=x.device) if out is None else out
    _k().rms_norm(out.view(x2.shape), x2, None, w, eps)
    return out.view(x.shape)


def fused_add_rms_norm(x: torch.Tensor, residual: torch.Tensor, w: torch.Tensor,
                       eps: float) -> tuple[torch.Tensor, torch.Tensor]:
    """In place: residual += x; x = rms_norm(residual) * w.  Returns (x, residual)."""
    if not _gpu(x):
        o, r = ref.fused_add_rms_norm(x, residual, w, eps)
        x.copy_(o)
        residual.copy_(r)
        return x, residual
    x2 = x.view(-1, x.shape[-1])
    _k().rms_norm(x2, x2, residual.view(-1, x.shape[-1]), w, eps)
    return x, residual


def layer_norm(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, eps: float = 1e-5):
    if not _gpu(x):
        return ref.layer_norm(x, w, b, eps)
    x2 = x.reshape(-1, x.shape[-1]).contiguous()
    out = torch.empty_like(x2)
    _k().layer_norm(out, x2, w, b, eps)
    return out.view(x.shape)


def silu_mul(x: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    if not _gpu(x):
        return ref.silu_mul(x)
    I = x.shape[-1] // 2
    x2 = x.view(-1, x.shape[-1])
    if out is None:
        out = torch.empty(x2.shape[0], I, dtype=x.dtype, device=x.device)
    _k().silu_mul(out, x2)
    return out.view(*x.shape[:-1], I)


# ------------------------------------------------------------------ rope + kv cache
def rope_kv_write(qkv: torch.Tensor, positions: torch.Tensor, cos_sin: torch.Tensor,
                  k_cache: torch.Tensor, v_cache: torch.Tensor, slot_mapping: torch.Tensor,
                  num_heads: int, num_kv_heads: int, head_dim: int,
                  q_norm_w: Optional[torch.Tensor] = None,
                  k_norm_w: Optional[torch.Tensor] = None, eps: float = 1e-6,
                  use_rope: bool = True, k_scale: float = 1.0,
                  v_scale: float = 1.0, dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """k_cache / v_cache may be fp8 (torch.float8_e4m3fn): values are stored as
    fp8(x / scale).  On the GPU ``qkv`` may also be the K9m split-K slices of the QKV
    projection (fp32 [S, T, N], ops/gemm.py linear_qkv): the kernel sums them, and
    ``dtype`` names the activation dtype of q."""
    if not _gpu(qkv):
        return ref.rope_qk_kv_write(qkv, positions, cos_sin, k_cache, v_cache, slot_mapping,
                                    num_heads, num_kv_heads, head_dim, q_norm_w, k_norm_w, eps,
                                    use_rope, k_scale, v_scale)
    sl = qkv.dim() == 3
    T = qkv.shape[1] if sl else qkv.shape[0]
    q = torch.empty(T, num_heads, head_dim, dtype=(dtype or qkv.dtype) if sl else qkv.dtype,
                    device=qkv.device)
    _k().rope_kv_write(qkv, positions, cos_sin, q, k_cache, v_cache, slot_mapping, q_norm_w,
                       k_norm_w, num_heads, num_kv_heads, head_dim, eps, use_rope, k_scale,
                       v_scale)
    return q


def kv_write_rope(qkv: torch.Tensor, positions: torch.Tensor, cos_sin: torch.Tensor,
                  k_cache: torch.Tensor, v_cache: torch.Tensor, slot_mapping: torch.Tensor,
                  num_heads: int, num_kv_heads: int, head_dim: int,
                  k_norm_w: Optional[torch.Tensor] = None, eps: float = 1e-6,
                  k_scale: float = 1.0, v_scale: float = 1.0) -> None:
    """rope_kv_write for k / v only (GPU, bf16 / f16 qkv [T, N]): the q part is left to
    ``prefill_attention_rope``, which rotates it as it loads it."""
    q = torch.empty(0, dtype=qkv.dtype, device=qkv.device)
    _k().rope_kv_write(qkv, positions, cos_sin, q, k_cache, v_cache, slot_mapping,
                       k_norm_w, k_norm_w, num_heads, num_kv_heads, head_dim, eps, True,
                       k_scale, v_scale)


# ------------------------------------------------------------------ attention
DECODE_PARTITION = 64        # tokens per wave-iteration of the 4-wave decode kernel
DECODE_CHUNK = 32            # tokens per pipelined step of K1w
DECODE_TARGET_WAVES = 2048   # K1w: 8 resident waves per CU (2 per SIMD at 256 VGPRs)
DECODE_WAVE_MIN_PAIRS = 64   # attention_decode.hip DEC_WAVE_MIN_PAIRS
DECODE_LONG_PAIRS = 256      # attention_decode.hip DEC_LONG_PAIRS
DECODE_LONG_TARGET_WAVES = 1024
PREFILL_BLOCK_M = 128


def decode_wave_kernel() -> bool:
    """K1w (one wave per (seq, kv-head, z-slice), csrc/kernels/attention_decode.hip) unless
    KGC_DECODE_WAVE=0 selects the 4-wave workgroup kernel; the C++ launcher reads the same
    variable, so the Z chosen here and the kernel that runs always agree."""
    return os.environ.get("KGC_DECODE_WAVE", "1") != "0"


def decode_uses_wave(batch: int, num_kv_heads: int) -> bool:
    """The kernel a launch of this grid takes: K1w from DECODE_WAVE_MIN_PAIRS (seq, kv-head)
    pairs up (at B = 1 the 4-wave kernel's 4x finer context split wins: 9.3 vs 12.3 us)."""
    lim = int(os.environ.get("KGC_DECODE_WAVE_MIN_PAIRS", DECODE_WAVE_MIN_PAIRS))
    return decode_wave_kernel() and batch * num_kv_heads >= lim


def decode_max_z(max_blocks: int, block_size: int) -> int:
    """The largest Z either kernel picks for this context capacity."""
    ctx = max_blocks * block_size
    wave = math.ceil(math.ceil(ctx / DECODE_CHUNK) / 2)     # >= 2 chunks per K1w slice
    four = math.ceil(math.ceil(ctx / DECODE_PARTITION) / 4)
    return max(1, min(1024, max(wave if decode_wave_kernel() else 1, four)))


def decode_partials(batch: int, num_heads: int, head_dim: int, max_blocks: int,
                    block_size: int, device) -> tuple:
    """Per-z-slice (max, sum, O) partials of the split-context decode kernels (static:
    graph-capturable), flat: row (seq, q-head) * Z + z, for every Z ``decode_grid_z`` picks
    at any batch <= ``batch`` (Z <= decode_max_z, and B * Z bounded by the wave targets:
    K1w B * nkv * Z <= 2 x 2048, the 4-wave kernel B * nkv * 4 * Z <= 2 x 4096).  Unused
    when the grid has a single z-slice."""
    Z = decode_max_z(max_blocks, block_size)
    rows = min(batch * Z, 2 * 4096 + batch)
    ml = torch.empty(rows * num_heads, dtype=torch.float32, device=device)
    es = torch.empty(rows * num_heads, dtype=torch.float32, device=device)
    tmp = torch.empty(rows * num_heads, head_dim, dtype=torch.float32, device=device)
    return ml, es, tmp


def _decode_z_cap(ws, B: int, nq: int) -> int:
    """Largest Z the workspace holds for a batch of B rows of nq heads."""
    return max(1, min(1024, ws[0].numel() // max(1, B * nq)))


def decode_grid_z(batch: int, num_kv_heads: int, max_ctx: int, target_waves: int = 0) -> int:
    """z-slices of the decode grid: enough waves to fill 256 CUs, bounded by the
    context (K1w: two 32-token chunks per wave; 4-wave kernel: 64-token partitions) and by
    the 1024 slices the reduce kernel merges.  Z == 1 (large batches) lets the kernel
    write its output directly."""
    pairs = max(1, batch * num_kv_heads)
    if decode_uses_wave(batch, num_kv_heads):
        chunks = max(1, math.ceil(max_ctx / DECODE_CHUNK))
        # from DECODE_LONG_PAIRS pairs up: ~4 waves per CU of longer slices (the kernel
        # also keeps those slices >= 10 chunks, attention_decode.hip DEC_LONG_MIN_CHUNKS)
        tgt = target_waves or (DECODE_LONG_TARGET_WAVES if pairs >= DECODE_LONG_PAIRS
                               else DECODE_TARGET_WAVES)
        want = math.ceil(tgt / pairs)
        return max(1, min(want, math.ceil(chunks / 2), 1024))
    parts = max(1, math.ceil(max_ctx / DECODE_PARTITION))
    want = math.ceil((target_waves or 4096) / (pairs * 4))
    return max(1, min(want, math.ceil(parts / 4), 1024))


def paged_attention_decode(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                           block_tables: torch.Tensor, context_lens: torch.Tensor, scale: float,
                           workspace=None, grid_z: int = 1,
                           out: Optional[torch.Tensor] = None, k_scale: float = 1.0,
                           v_scale: float = 1.0) -> torch.Tensor:
    if not _gpu(q):
        return ref.paged_attention_decode(q, k_cache, v_cache, block_tables, context_lens, scale,
                                          k_scale, v_scale)
    B, nq, d = q.shape
    if out is None:
        out = torch.empty_like(q)
    if workspace is None:
        workspace = decode_partials(B, nq, d, block_tables.shape[1], k_cache.shape[2], q.device)
    ml, es, tmp = workspace
    grid_z = min(grid_z, _decode_z_cap(workspace, B, nq))
    _k().paged_decode(out, q, k_cache, v_cache, block_tables, context_lens, ml, es, tmp,
                      grid_z, scale, k_scale, v_scale)
    return out


def paged_attention_decode_rope(qkv: torch.Tensor, positions: torch.Tensor,
                                cos_sin: torch.Tensor, k_cache: torch.Tensor,
                                v_cache: torch.Tensor, slot_mapping: torch.Tensor,
                                num_heads: int, num_kv_heads: int, head_dim: int,
                                block_tables: torch.Tensor, context_lens: torch.Tensor,
                                scale: float, q_norm_w: Optional[torch.Tensor] = None,
                                k_norm_w: Optional[torch.Tensor] = None, eps: float = 1e-6,
                                use_rope: bool = True, workspace=None, grid_z: int = 1,
                                k_scale: float = 1.0, v_scale: float = 1.0,
                                dtype: Optional[torch.dtype] = None,
                                row_scale: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``rope_kv_write`` + ``paged_attention_decode`` of a decode-only batch in ONE
    launch (K1 with K3/K5/K6 as its prologue): q is built in registers from the QKV
    projection (or its K9m fp32 split-K slices [S, B, N]), the new token's k / v are
    written to the cache by the workgroup that reads them back.  -> [B, nq, d].
    ``row_scale`` [B] fp32: projection row b is scaled by it before its rounding (the
    norm-free layer's rsqrt(mean(x^2) + eps) over a gamma-folded QKV weight)."""
    if not _gpu(qkv):
        if row_scale is not None:
            qkv = (qkv.float().sum(0) if qkv.dim() == 3 else qkv.float()) * row_scale[:, None]
            qkv = qkv.to(dtype or torch.float32)
        q = ref.rope_qk_kv_write(qkv, positions, cos_sin, k_cache, v_cache, slot_mapping,
                                 num_heads, num_kv_heads, head_dim, q_norm_w, k_norm_w, eps,
                                 use_rope, k_scale, v_scale)
        return ref.paged_attention_decode(q, k_cache, v_cache, block_tables, context_lens, scale,
                                          k_scale, v_scale)
    sl = qkv.dim() == 3
    B = qkv.shape[1] if sl else qkv.shape[0]
    out = torch.empty(B, num_heads, head_dim, dtype=(dtype or qkv.dtype) if sl else qkv.dtype,
                      device=qkv.device)
    if workspace is None:
        workspace = decode_partials(B, num_heads, head_dim, block_tables.shape[1],
                                    k_cache.shape[2], qkv.device)
    ml, es, tmp = workspace
    grid_z = min(grid_z, _decode_z_cap(workspace, B, num_heads))
    _k().paged_decode_rope(out, qkv, positions, cos_sin, k_cache, v_cache, slot_mapping,
                           q_norm_w, k_norm_w, block_tables, context_lens, ml, es, tmp,
                           num_heads, grid_z, scale, eps, use_rope, k_scale, v_scale,
                           row_scale)
    return out


def prefill_work_list(query_lens: list[int], seq_lens: list[int]) -> tuple[list[int], list[int]]:
    """(seq, 128-row block) work items, heaviest (most keys) first."""
    items = []
    for i, (ql, sl) in enumerate(zip(query_lens, seq_lens)):
        ctx0 = sl - ql
        for mb in range((ql + PREFILL_BLOCK_M - 1) // PREFILL_BLOCK_M):
            last = ctx0 + min((mb + 1) * PREFILL_BLOCK_M, ql)
            items.append((-last, i, mb))
    items.sort()
    return [i for _, i, _ in items], [m for _, _, m in items]


def prefill_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                      block_tables: torch.Tensor, query_start_loc: torch.Tensor,
                      seq_lens: torch.Tensor, scale: float, work_seq: torch.Tensor = None,
                      work_mblk: torch.Tensor = None,
                      out: Optional[torch.Tensor] = None, k_scale: float = 1.0,
                      v_scale: float = 1.0) -> torch.Tensor:
    if not _gpu(q):
        return ref.prefill_attention(q, k_cache, v_cache, block_tables, query_start_loc,
                                     seq_lens, scale, k_scale, v_scale)
    if work_seq is None:
        qsl = query_start_loc.tolist()
        ws, wm = prefill_work_list([qsl[i + 1] - qsl[i] for i in range(len(qsl) - 1)],
                                   seq_lens.tolist())
        work_seq = torch.tensor(ws, dtype=torch.int32, device=q.device)
        work_mblk = torch.tensor(wm, dtype=torch.int32, device=q.device)
    if out is None:
        out = torch.empty_like(q)
    _k().prefill_attention(out, q, k_cache, v_cache, block_tables, query_start_loc, seq_lens,
                           work_seq, work_mblk, scale, k_scale, v_scale)
    return out


def prefill_attention_rope(qkv: torch.Tensor, cos_sin: torch.Tensor, k_cache: torch.Tensor,
                           v_cache: torch.Tensor, block_tables: torch.Tensor,
                           query_start_loc: torch.Tensor, seq_lens: torch.Tensor, scale: float,
                           num_heads: int, head_dim: int, work_seq: Optional[torch.Tensor] = None,
                           work_mblk: Optional[torch.Tensor] = None,
                           out: Optional[torch.Tensor] = None,
                           k_scale: float = 1.0, v_scale: float = 1.0) -> torch.Tensor:
    """K2 on a prefill-only step whose q is still the unrotated QKV projection row: NeoX
    RoPE (position = context start + row, as the engine numbers tokens) is applied as the
    kernel loads q, so q is never written or re-read (k / v: ``kv_write_rope``)."""
    T = qkv.shape[0]
    if work_seq is None:
        qsl = query_start_loc.tolist()
        ws, wm = prefill_work_list([qsl[i + 1] - qsl[i] for i in range(len(qsl) - 1)],
                                   seq_lens.tolist())
        work_seq = torch.tensor(ws, dtype=torch.int32, device=qkv.device)
        work_mblk = torch.tensor(wm, dtype=torch.int32, device=qkv.device)
    if out is None:
        out = torch.empty(T, num_heads, head_dim, dtype=qkv.dtype, device=qkv.device)
    _k().prefill_attention_rope(out, qkv, cos_sin, k_cache, v_cache, block_tables,
                                query_start_loc, seq_lens, work_seq, work_mblk, num_heads, scale,
                                k_scale, v_scale)
    return out


# ------------------------------------------------------------------ sampling
def sample(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor,
           top_p: torch.Tensor, seeds: torch.Tensor,
           out: Optional[torch.Tensor] = None, thresholds: bool = True) -> torch.Tensor:
    """K10.  ``thresholds=False`` promises that no row uses top-k / top-p (the caller
    knows from the host-side plan): the single-pass kernel then runs; otherwise the
    cooperative kernel splits each row's threshold passes over its workgroups."""
    if not _gpu(logits):
        return ref.sample(logits, temperature, top_k, top_p, seeds)
    B = logits.shape[0]
    if out is None:
        out = torch.empty(B, dtype=torch.int64, device=logits.device)
    _k().sample(out, logits, temperature, top_k, top_p, seeds, thresholds)
    return out


class SamplerFailed(RuntimeError):
    """The cooperative top-k / top-p sampler's row barrier timed out: the step's
    thresholds (and tokens) are invalid."""


class SamplerHealth:
    """The cooperative sampler's sticky error word (sampling.hip ``g_smp_err``), checked
    like the peer-memory collectives' words: ``enqueue_err_read`` queues a copy into a
    pinned host slot and a clear of the device word behind the step, and returns the slot;
    ``raise_if_failed(slot)`` (after that step completed) raises instead of letting its
    tokens be served.  Every in-flight step copies into its OWN slot (a ring): with async
    scheduling step N + 1 is launched before N's tokens are read, and N + 1's copy of the
    just-cleared word must not overwrite N's flag."""

    SLOTS = 8      # > steps in flight (async: 2; PP: one per stage, <= 8)

    def __init__(self, device: torch.device):
        with torch.cuda.device(device):
            self.addr = int(_k().sample_err_addr())
        self.host = torch.zeros(self.SLOTS, dtype=torch.int32, pin_memory=True)
        self._next = 0

    def enqueue_err_read(self) -> int:
        slot = self._next
        self._next = (slot + 1) % self.SLOTS
        self.host[slot] = 0
        _k().u32_copy_async(self.addr, self.host, slot)
        _k().u32_clear_async(self.addr)
        return slot

    def failed(self, slot: int) -> bool:
        """The flag of `slot` (its step must have completed)."""
        return bool(int(self.host[slot]))

    def raise_if_failed(self, slot: Optional[int] = None) -> None:
        if slot is None:
            slot = (self._next - 1) % self.SLOTS
        if int(self.host[slot]):
            self.host[slot] = 0
            raise SamplerFailed("top-k / top-p sampler: a row's workgroups were not co-resident "
                                "and its barrier timed out; the step's tokens are invalid")


def sample_vp_partial(logits: torch.Tensor, V: int, temperature: torch.Tensor,
                      seeds: torch.Tensor, vocab_off: int,
                      out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Vocab-parallel K10 (rows without top-k / top-p): this rank's packed (value,
    global index) candidate per row over its shard ``logits[:, :V]`` (columns
    ``vocab_off ..``), as int64 ordered for a MAX all-reduce over the TP group; then
    ``sample_vp_finish``.  The result equals ``sample`` on the unsharded logits."""
    B = logits.shape[0]
    if not _gpu(logits):
        return ref.sample_vp_partial(logits[:, :V], temperature[:B], seeds[:B], vocab_off)
    if out is None:
        out = torch.empty(B, dtype=torch.int64, device=logits.device)
    _k().sample_vp(out, logits, V, temperature, seeds, vocab_off)
    return out


def sample_vp_finish(packed: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Token ids from the all-reduced packed candidates."""
    if not _gpu(packed):
        return ref.sample_vp_unpack(packed)
    if out is None:
        out = torch.empty_like(packed)
    _k().sample_vp_unpack(out, packed)
    return out


__all__ = ["load_extension", "rms_norm", "fused_add_rms_norm", "layer_norm", "silu_mul",
           "rope_kv_write", "paged_attention_decode", "paged_attention_decode_rope", "prefill_attention", "sample", "sample_vp_partial", "sample_vp_finish",
           "decode_partials", "decode_grid_z", "moe_pack", "moe_packable", "prefill_work_list", "ref"]


# ------------------------------------------------------------------ MoE (K13 / K14)
MOE_GATE_FUSED_MAX_T = 1024  # tokens up to which the router GEMM runs inside the top-k kernel
MOE_NATIVE_MAX_ROWS = 128   # mean rows per expert above which hipBLASLt per expert wins


def moe_supported(n: int, k: int) -> bool:
    """Shapes the grouped GEMM tiles cover: N % 128 == 0 and K % 64 == 0."""
    return n % 128 == 0 and k % 64 == 0


def moe_topk_softmax(router_logits: torch.Tensor, k: int, renormalize: bool = True):
    """K13: (weights fp32 [T, k], expert ids int32 [T, k])."""
    if not _gpu(router_logits):
        return ref.moe_topk_softmax(router_logits, k, renormalize)
    T = router_logits.shape[0]
    w = torch.empty(T, k, dtype=torch.float32, device=router_logits.device)
    ids = torch.empty(T, k, dtype=torch.int32, device=router_logits.device)
    _k().moe_route(w, ids, router_logits, renormalize)
    return w, ids


def moe_gate_topk(x: torch.Tensor, wg: torch.Tensor, k: int,
                  renormalize: bool = True) -> Optional[tuple]:
    """K13 with the router GEMM folded in: (weights fp32 [T, k], expert ids int32 [T, k])
    of x [T, H] . wg [E, H]^T in one launch, or None where the fused kernel does not apply
    (CPU, E > 16, H % 512 != 0): the caller then runs the GEMM and ``moe_topk_softmax``."""
    if (not _gpu(x) or x.dim() != 2 or wg.shape[0] > 16 or x.shape[1] % 512
            or x.dtype not in (torch.bfloat16, torch.float16) or wg.dtype != x.dtype
            or x.stride(1) != 1 or x.stride(0) % 8):
        return None
    T = x.shape[0]
    w = torch.empty(T, k, dtype=torch.float32, device=x.device)
    ids = torch.empty(T, k, dtype=torch.int32, device=x.device)
    _k().moe_gate_route(w, ids, x, wg.contiguous(), renormalize)
    return w, ids


def moe_splitk(npairs: int, E: int, N: int, K: int, bm: int) -> int:
    """K-slices for the down projection: enough workgroups to fill 256 CUs twice over,
    each slice still >= 16 K-tiles of 64.  The row-block count is bounded without a host
    sync (at most npairs/bm + E blocks carry rows)."""
    if os.environ.get("KGC_MOE_SPLITK") is not None:
        return max(1, int(os.environ["KGC_MOE_SPLITK"]))
    wgs = min((npairs + bm - 1) // bm + E, npairs) * (N // 128)
    S = 1
    while S < 8 and wgs * S < 1024 and K // 64 // (2 * S) >= 16:
        S *= 2
    return S


def moe_pack(w: torch.Tensor, silu: bool) -> torch.Tensor:
    """Per-expert K9m packed copy [E, N/128, K/64, 8192] of an expert weight stack
    [E, N, K] (``dgemm_pack`` per expert; w13 SiLU-packed: gate / up 16-row groups
    interleaved per 128-row tile), the operand of ``moe_dgemm`` (K14m)."""
    E, N, K = w.shape
    p = torch.empty(E, N // 128, K // 64, 8192, dtype=w.dtype, device=w.device)
    for e in range(E):
        _k().dgemm_pack(p[e], w[e], silu)
    return p


def moe_packable(w13: torch.Tensor, w2: torch.Tensor) -> bool:
    """Shapes K14m's packed tiles cover: 2I % 128, I % 64, H % 128, K % 64."""
    I2, H = w13.shape[1], w13.shape[2]
    return I2 % 128 == 0 and (I2 // 2) % 64 == 0 and H % 128 == 0 and w2.shape[2] % 64 == 0


def moe_k14m_bm(npairs: int, E: int) -> int:
    """K14m row block for a call of ``npairs`` (token, expert) pairs over E local experts:
    the smallest of 64 / 96 / 128 that holds a typical expert's pairs in ONE block (an
    expert with more rows than a block streams its weights once per block): routed
    uniformly, a bucket is ~npairs / E +- 3 sd (Mixtral 8x7B decode at batch 256: 64 per
    expert, max ~80 -> 96)."""
    mean = npairs / max(1, E)
    if mean <= 44:
        return 64
    return 96 if mean <= 72 else 128


def moe_k14m_bn() -> int:
    """K14m column tile: 256 (KGC_MOE_BN=128 for A/B)."""
    return 128 if os.environ.get("KGC_MOE_BN") == "128" else 256


def moe_dgemm_splitk(npairs: int, E: int, N: int, K: int, bm: int, bn: int = 128) -> int:
    """K-slices of K14m's down projection: the used row blocks (at most npairs/bm + E)
    times N/bn column tiles times S near one workgroup per CU, each slice >= 8 K-steps
    (KGC_MOE_SPLITK overrides, as for the register-staged kernel)."""
    if os.environ.get("KGC_MOE_SPLITK") is not None:
        return max(1, int(os.environ["KGC_MOE_SPLITK"]))
    blocks = min((npairs + bm - 1) // bm + E, max(1, npairs))
    wgs = blocks * (N // bn)
    S = 1
    while S < 16 and wgs * S * 2 <= 320 and K // 64 // (2 * S) >= 8:
        S *= 2
    return S


def fused_moe(x: torch.Tensor, w13: torch.Tensor, w2: torch.Tensor, topk_w: torch.Tensor,
              topk_ids: torch.Tensor, expert_offset: int = 0,
              all_local: bool = True, w13p: Optional[torch.Tensor] = None,
              w2p: Optional[torch.Tensor] = None, rows_hint: Optional[int] = None,
              combine: bool = True) -> torch.Tensor:
    """K14: sum_j topk_w[t, j] * MLP_{topk_ids[t, j]}(x[t]) for the experts held here
    (global ids ``expert_offset .. expert_offset + w13.shape[0]``).  x [T, H];
    w13 [E, 2I, H] (gate rows then up rows); w2 [E, H, I].  No host synchronisation:
    bucket sizes stay on the device, so the block is captured in decode graphs.
    ``w13p`` / ``w2p`` (``moe_pack``): K14m -- both projections on the K9m LDS-DMA
    pipeline over packed per-expert tiles, the SiLU in the gate_up epilogue (no [rows, 2I]
    intermediate, no silu_mul launch); else the register-staged grouped GEMM.

    ``rows_hint``: the number of pairs expected to carry rows when ``topk_ids`` has room
    for more (the EP owner's receive slots: NR x C slots, ~T x k of them used); it sizes
    the row block and the down projection's split-K.  ``combine=False`` returns the down
    projection's output per pair instead of the weighted sum -- [npairs, H] in x's dtype,
    or its fp32 split-K slices [S, npairs, H] -- for a consumer that sums the slices
    itself (``ep_return``)."""
    if not _gpu(x):
        return ref.moe_mlp_local(x, w13, w2, topk_w, topk_ids, expert_offset)
    k = _k()
    T, H = x.shape
    E, I2 = w13.shape[0], w13.shape[1]
    topk = topk_ids.shape[1]
    npairs = T * topk
    used = min(npairs, rows_hint) if rows_hint else npairs
    packed = w13p is not None and w2p is not None
    bm = int(os.environ.get("KGC_MOE_BM", 0)) or (moe_k14m_bm(used, E) if packed else
                                                  (64 if used <= 40 * E else 128))
    if bm == 96 and not packed:
        bm = 128                    # the register-staged kernel has 64 / 128-row tiles only
    rows = (npairs + E * (bm - 1) + bm - 1) // bm * bm
    dev = x.device
    sorted_ids = torch.empty(rows, dtype=torch.int32, device=dev)
    block_expert = torch.empty(rows // bm, dtype=torch.int32, device=dev)
    meta = torch.empty(1, dtype=torch.int32, device=dev)
    ids = topk_ids.contiguous()
    k.moe_align(sorted_ids, block_expert, meta, ids, expert_offset, E, bm)
    if packed:
        bn = moe_k14m_bn()
        act = torch.empty(rows, I2 // 2, dtype=x.dtype, device=dev)
        k.moe_dgemm(act, x.contiguous(), w13p, sorted_ids, block_expert, meta, npairs, topk,
                    bm, 1, bn if I2 % bn == 0 else 128)
        bn2 = bn if H % bn == 0 else 128
        S = moe_dgemm_splitk(used, E, H, I2 // 2, bm, bn2)
        alloc = torch.empty if all_local else torch.zeros
        if S > 1:
            y = alloc(S, npairs, H, dtype=torch.float32, device=dev)
        else:
            y = alloc(npairs, H, dtype=x.dtype, device=dev)
        k.moe_dgemm(y, act, w2p, sorted_ids, block_expert, meta, npairs, topk, bm, 2, bn2)
        if not combine:
            return y
        out = torch.empty(T, H, dtype=x.dtype, device=dev)
        k.moe_combine(out, y, topk_w.contiguous().float())
        return out
    inter = torch.empty(rows, I2, dtype=x.dtype, device=dev)
    k.moe_gemm(inter, x.contiguous(), w13, sorted_ids, block_expert, meta, npairs, topk, bm,
               True, False)
    act = silu_mul(inter)
    S = moe_splitk(used, E, H, w2.shape[2], bm)
    alloc = torch.empty if all_local else torch.zeros   # EP: pairs of remote experts add 0
    if S > 1:
        y = alloc(S, npairs, H, dtype=torch.float32, device=dev)
    else:
        y = alloc(npairs, H, dtype=x.dtype, device=dev)
    k.moe_gemm(y, act, w2, sorted_ids, block_expert, meta, npairs, topk, bm, False, True, S)
    if not combine:
        return y
    out = torch.empty(T, H, dtype=x.dtype, device=dev)
    k.moe_combine(out, y, topk_w.contiguous().float())
    return out


# ------------------------------------------------------------------ hybrid decoders
# Grouped RMSNorm over an fp32 residual stream, depth-weighted averaging of the layer
# results, xIELU, small fp32 gate projections, windowed attention with kept first tokens
# over a plain-layout paged cache (per-layer query/key and value sizes), and the mLSTM
# matrix-memory scan over per-sequence state slots.  ``meta`` is the step's AttnMetadata.
GATE_SIGMOID, GATE_CAP_TANH, GATE_LOGSIG_CAP_TANH, GATE_NONE = (
    ref.GATE_SIGMOID, ref.GATE_CAP_TANH, ref.GATE_LOGSIG_CAP_TANH, ref.GATE_NONE)


def group_rms_norm(x: torch.Tensor, w: torch.Tensor, groups: int, eps: float,
                   out_dtype: torch.dtype, add: Optional[torch.Tensor] = None) -> torch.Tensor:
    """h = grouped RMSNorm(x) * w in ``out_dtype``; x [T, W] is the fp32 residual stream.
    ``add`` [T, W]: x += add first, in place (the sublayer's output joins the stream)."""
    if not _gpu(x):
        if add is not None:
            x += add.float()
        return ref.group_rms_norm(x, w, groups, eps, out_dtype)
    out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
    _k().residual_group_norm(out, x, add, w, groups, eps)
    return out


def depth_mix_norm(x: torch.Tensor, hist: torch.Tensor, layer: int, y: torch.Tensor,
                   coef: torch.Tensor, w: torch.Tensor, groups: int, eps: float,
                   out_dtype: torch.dtype) -> torch.Tensor:
    """End of layer ``layer`` of a depth-averaged decoder, in one pass over the rows:
    hist[layer + 1, :T] = x + y (the layer's result); x = sum_j coef[j] * hist[j, :T] over
    j <= layer + 1 (in place: what the next layer reads); returns grouped RMSNorm(x) * w
    (the next layer's first norm, or the model's final one).  hist [L + 1, Tcap, W] and x
    are fp32; coef fp32 [layer + 2]."""
    T = x.shape[0]
    if not _gpu(x):
        hist[layer + 1, :T] = x + y.float()
        x.copy_(ref.depth_mix(hist, layer + 2, coef, T))
        return ref.group_rms_norm(x, w, groups, eps, out_dtype)
    out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
    _k().depth_mix_norm(out, x, hist, y, coef, w, layer, groups, eps)
    return out


def xielu(z: torch.Tensor, ab: torch.Tensor) -> torch.Tensor:
    """ab fp32 [2] = (softplus(p), 1/2 + softplus(q)) of the layer's two parameters."""
    if not _gpu(z):
        return ref.xielu(z, ab)
    out = torch.empty_like(z)
    _k().xielu(out, z, ab)
    return out


def gate_proj(h: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], kind_a: int,
              kind_b: int = 0, split: Optional[int] = None, cap: float = 1.0) -> torch.Tensor:
    """fp32 [T, N] gate values act(h . w^T + bias) for a few output rows N (per-head
    gates): the products accumulate and stay in fp32."""
    split = w.shape[0] if split is None else split
    if not _gpu(h):
        return ref.gate_proj(h, w, bias, kind_a, kind_b, split, cap)
    out = torch.empty(h.shape[0], w.shape[0], dtype=torch.float32, device=h.device)
    _k().gate_proj(out, h, w, bias, kind_a, kind_b, split, cap)
    return out


def rope_kv_store(qkv: torch.Tensor, positions: torch.Tensor, table: Optional[torch.Tensor],
                  k_cache: torch.Tensor, v_cache: torch.Tensor, slot_mapping: torch.Tensor,
                  H: int, G: int, dk: int, dv: int, interleaved: bool = False) -> torch.Tensor:
    if not _gpu(qkv):
        return ref.rope_kv_store(qkv, positions, table, k_cache, v_cache, slot_mapping, H, G,
                                 dk, dv, interleaved)
    q = torch.empty(qkv.shape[0], H, dk, dtype=qkv.dtype, device=qkv.device)
    _k().rope_kv_store(qkv, positions, table, q, k_cache, v_cache, slot_mapping, H, G, dk, dv,
                       interleaved)
    return q


def _row_tables(meta, T: int) -> torch.Tensor:
    """CPU path: the block-table row of every token of the step."""
    rows = []
    if meta.num_prefills:
        qsl = meta.query_start_loc.tolist()
        for i in range(meta.num_prefills):
            rows.append(meta.prefill_block_tables[i:i + 1].expand(qsl[i + 1] - qsl[i], -1))
    if meta.num_decodes:
        rows.append(meta.decode_block_tables[: meta.num_decodes])
    return torch.cat(rows, 0)[:T]


def window_attention_fast() -> bool:
    """KGC_WINDOW_ATTN=simple runs every row on the one-wave-per-(row, head) kernel; by
    default prefill chunks take the MFMA tile kernel (16-bit activations, head sizes it
    covers) and decode rows the 8-wave kernel, the one-wave kernel taking what is left."""
    return os.environ.get("KGC_WINDOW_ATTN", "fast") != "simple"


def window_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                     positions: torch.Tensor, meta, scale: float, window: int, keep_first: int,
                     gate: Optional[torch.Tensor] = None, softcap: float = 0.0,
                     out_scale: float = 1.0, out: Optional[torch.Tensor] = None,
                     elem_gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Prefill chunks and decode rows of one step alike: row t sees the cached keys
    j <= p with p - j < window or j < keep_first (p = positions[t]; window <= 0: plain
    causal).  Decode padding rows (context length 0) give zeros.  ``softcap`` > 0: the
    scaled scores pass softcap * tanh(. / softcap).  The result is multiplied by
    sigmoid(``elem_gate`` [T, H * dv], a column slice of a projection) when given and by
    ``out_scale``, and may go to ``out`` [T, H * dv], a column slice of a wider buffer."""
    T, H, _ = q.shape
    dv = v_cache.shape[3]
    if not _gpu(q):
        pos = positions.clone()
        if meta.num_decodes:
            tp = meta.num_prefill_tokens
            pos[tp:tp + meta.num_decodes] = meta.decode_ctx_lens[: meta.num_decodes].long() - 1
        r = ref.window_attention(q, k_cache, v_cache, pos, _row_tables(meta, T), scale,
                                 window, keep_first, gate, softcap, out_scale, elem_gate)
        if out is not None:
            out.copy_(r)
            return out
        return r
    if out is None:
        out = torch.empty(T, H * dv, dtype=q.dtype, device=q.device)
    ws, wb = getattr(meta, "work_seq", None), getattr(meta, "work_mblk", None)
    if meta.num_prefills and ws is None:
        qsl = meta.query_start_loc.tolist()
        a, b = prefill_work_list([qsl[i + 1] - qsl[i] for i in range(meta.num_prefills)],
                                 meta.prefill_seq_lens.tolist())
        ws = torch.tensor(a, dtype=torch.int32, device=q.device)
        wb = torch.tensor(b, dtype=torch.int32, device=q.device)
    _k().window_attention(out, q, k_cache, v_cache, meta.query_start_loc,
                          meta.prefill_seq_lens, meta.prefill_block_tables,
                          meta.decode_ctx_lens, meta.decode_block_tables, ws, wb,
                          meta.num_prefills, meta.num_decodes, meta.num_prefill_tokens,
                          scale, window, keep_first, gate, window_attention_fast(),
                          float(softcap), float(out_scale), elem_gate)
    return out


def mlstm_scan(qkvg: torch.Tensor, gates: torch.Tensor, state: tuple, meta, H: int, d: int,
               dv: int) -> torch.Tensor:
    """fp32 [T, H*dv]: the matrix-memory recurrence over every step sequence's tokens,
    read from and written back to its state slot (``meta.state_slots``; < 0: a padding
    row, skipped).  state = (S [slots, H, d, dv], n [slots, H, d], m [slots, H]) fp32."""
    S, n, m = state
    T = qkvg.shape[0]
    P, D, tp = meta.num_prefills, meta.num_decodes, meta.num_prefill_tokens
    if not _gpu(qkvg):
        start, ln, pos = [], [], []
        if P:
            qsl, sl = meta.query_start_loc.tolist(), meta.prefill_seq_lens.tolist()
            for i in range(P):
                start.append(qsl[i])
                ln.append(qsl[i + 1] - qsl[i])
                pos.append(sl[i] - ln[-1])
        if D:
            ctx = meta.decode_ctx_lens.tolist()
            for i in range(D):
                start.append(tp + i)
                ln.append(1)
                pos.append(ctx[i] - 1)
        return ref.mlstm_scan(qkvg, gates, S, n, m, start, ln, pos,
                              meta.state_slots[: P + D].tolist(), H, d, dv)
    out = torch.empty(T, H * dv, dtype=torch.float32, device=qkvg.device)
    _k().mlstm_scan(out, qkvg, gates, S, n, m, meta.query_start_loc, meta.prefill_seq_lens,
                    meta.decode_ctx_lens, meta.state_slots, P, D, tp, H, d, dv)
    return out


def head_norm_gate(o: torch.Tensor, g: torch.Tensor, w: torch.Tensor, H: int, eps: float,
                   out_dtype: torch.dtype) -> torch.Tensor:
    """Per-head RMS normalisation of the recurrence output o (fp32 [T, H*dv]), times w,
    times sigmoid(g) (g: a [T, H*dv] column slice of the merged projection)."""
    if not _gpu(o):
        return ref.head_norm_gate(o, g, w, H, eps, out_dtype)
    out = torch.empty(o.shape, dtype=out_dtype, device=o.device)
    _k().head_norm_gate(out, o, g, w, H, eps)
    return out


# ------------------------------------------------------------------ Konovik-style decoders
# A residual stream scaled per sublayer, token shift and minGRU over per-sequence state
# slots, latent attention (the paged cache holds one normed latent + one rotary key part
# per token; values are the latent columns of the same rows), sigmoid routing with a
# choice correction over squared-ReLU experts, and a per-token side input.
def residual_norm(x: torch.Tensor, add: Optional[torch.Tensor], mult: float,
                  w: Optional[torch.Tensor], eps: float, out_dtype: Optional[torch.dtype],
                  add_norm_w: Optional[torch.Tensor] = None,
                  out: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """x fp32 [T, W], in place: x += mult * a (a = add, or RMS-normed add times
    add_norm_w); returns RMSNorm(x) * w (w None: x) in out_dtype (None: no output).
    ``out`` may be x itself (fp32): the stream is replaced by its normed value."""
    if not _gpu(x):
        r = ref.residual_norm(x, add, mult, w, eps, out_dtype, add_norm_w)
        if out is not None and r is not None:
            out.copy_(r)
            return out
        return r
    if out is None and out_dtype is not None:
        out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
    _k().residual_norm(out, x, add, add_norm_w, w, float(mult), eps)
    return out


def token_shift(h: torch.Tensor, mu: torch.Tensor, state: torch.Tensor, meta,
                out_dtype: torch.dtype) -> torch.Tensor:
    """h fp32 [T, W] -> h + (previous row of the sequence - h) * mu in out_dtype; the row
    before a chunk's first comes from state [slots, W] (zeros at position 0), which then
    takes the chunk's last row."""
    if not _gpu(h):
        return ref.token_shift(h, mu, state, ref.step_sequences(meta), out_dtype)
    out = torch.empty(h.shape, dtype=out_dtype, device=h.device)
    _k().token_shift(out, h, mu, state, meta.query_start_loc, meta.prefill_seq_lens,
                     meta.decode_ctx_lens, meta.state_slots, meta.num_prefills,
                     meta.num_decodes, meta.num_prefill_tokens)
    return out


def mingru_scan(zxg: torch.Tensor, bias: torch.Tensor, state: torch.Tensor, meta, width: int,
                out_dtype: torch.dtype) -> torch.Tensor:
    """The minGRU recurrence over every step sequence's rows from / into state
    [slots, width] fp32, times silu of the output-gate columns: zxg [T, 3 width] holds the
    update-gate | candidate | output-gate pre-activations, bias fp32 [2 width].  Long chunks
    of few sequences run block-parallel (KGC_MINGRU_SCAN=token keeps the token-order scan)."""
    if not _gpu(zxg):
        return ref.mingru_scan(zxg, bias, state, ref.step_sequences(meta), width, out_dtype)
    out = torch.empty(zxg.shape[0], width, dtype=out_dtype, device=zxg.device)
    _k().mingru_scan(out, zxg, bias, state, meta.query_start_loc, meta.prefill_seq_lens,
                     meta.decode_ctx_lens, meta.state_slots, meta.num_prefills,
                     meta.num_decodes, meta.num_prefill_tokens, width,
                     os.environ.get("KGC_MINGRU_SCAN", "block") != "token")
    return out


def latent_rope_store(proj: torch.Tensor, q_lat: torch.Tensor, positions: torch.Tensor,
                      table: Optional[torch.Tensor], norm_w: torch.Tensor, eps: float,
                      cache: torch.Tensor, slot_mapping: torch.Tensor, H: int, d: int, r: int,
                      rank: int) -> torch.Tensor:
    """Cache rows [normed latent | rotated key part] of the step's tokens, and their query
    rows [T, H, rank + r] = [q_lat (H, T, rank) | rotated query part]; see
    ``ref.latent_rope_store``."""
    if not _gpu(proj):
        return ref.latent_rope_store(proj, q_lat, positions, table, norm_w, eps, cache,
                                     slot_mapping, H, d, r, rank)
    q = torch.empty(proj.shape[0], H, rank + r, dtype=proj.dtype, device=proj.device)
    _k().latent_rope_store(q, proj, q_lat, positions, table, norm_w, eps, cache, slot_mapping,
                           H, d, r, rank)
    return q


def gate_mul(o: torch.Tensor, g: torch.Tensor, scale: float = 1.0,
             out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """o [T, H, dv] (any token / head strides) * sigmoid(g [T, H dv], a column slice) *
    scale, into ``out`` [T, H dv] (a column slice of a wider buffer) when given."""
    if not _gpu(o):
        r = ref.gate_mul(o, g, scale)
        if out is not None:
            out.copy_(r)
            return out
        return r
    T, H, dv = o.shape
    if out is None:
        out = torch.empty(T, H * dv, dtype=g.dtype, device=g.device)
    _k().gate_mul(out, o, g, float(scale))
    return out


def relu_sq(z: torch.Tensor) -> torch.Tensor:
    if not _gpu(z):
        return ref.relu_sq(z)
    out = torch.empty_like(z)
    _k().relu_sq(out, z.contiguous())
    return out


def moe_route_sigmoid(scores: torch.Tensor, correction: torch.Tensor, k: int, scale: float):
    """(weights fp32 [T, k], expert ids int32 [T, k]) from sigmoid scores fp32 [T, >= E]."""
    if not _gpu(scores):
        return ref.moe_route_sigmoid(scores, correction, k, scale)
    T = scores.shape[0]
    w = torch.empty(T, k, dtype=torch.float32, device=scores.device)
    ids = torch.empty(T, k, dtype=torch.int32, device=scores.device)
    _k().moe_route_sigmoid(w, ids, scores, correction, float(scale))
    return w, ids


def grouped_experts(x: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor,
                    topk_w: torch.Tensor, topk_ids: torch.Tensor, act,
                    all_local: bool = True) -> torch.Tensor:
    """sum_j topk_w[t, j] * down_e(act(up_e x[t])), e = topk_ids[t, j], on the grouped MFMA
    GEMM (``moe_align`` buckets, rows gathered for the up projection and scattered back
    by the down projection, ``moe_combine``): experts w_up [E, I, H] (gated: [E, 2 I, H],
    ``act`` halving the columns), w_down [E, H, I] with the activation ``act`` between.
    ``all_local=False``: ids outside [0, E) are allowed and add nothing.  No host
    synchronisation."""
    k = _k()
    T, H = x.shape
    E, I = w_up.shape[0], w_up.shape[1]
    topk = topk_ids.shape[1]
    npairs = T * topk
    bm = 64 if npairs <= 40 * E else 128
    rows = (npairs + E * (bm - 1) + bm - 1) // bm * bm
    dev = x.device
    sorted_ids = torch.empty(rows, dtype=torch.int32, device=dev)
    block_expert = torch.empty(rows // bm, dtype=torch.int32, device=dev)
    meta = torch.empty(1, dtype=torch.int32, device=dev)
    k.moe_align(sorted_ids, block_expert, meta, topk_ids.contiguous(), 0, E, bm)
    inter = torch.empty(rows, I, dtype=x.dtype, device=dev)
    k.moe_gemm(inter, x.contiguous(), w_up, sorted_ids, block_expert, meta, npairs, topk, bm,
               True, False)
    a = act(inter)
    S = moe_splitk(npairs, E, H, a.shape[1], bm)
    alloc = torch.empty if all_local else torch.zeros
    if S > 1:
        y = alloc(S, npairs, H, dtype=torch.float32, device=dev)
    else:
        y = alloc(npairs, H, dtype=x.dtype, device=dev)
    k.moe_gemm(y, a, w_down, sorted_ids, block_expert, meta, npairs, topk, bm, False, True, S)
    out = torch.empty(T, H, dtype=x.dtype, device=dev)
    k.moe_combine(out, y, topk_w.contiguous().float())
    return out


def moe_finish(routed, dense, topk_w, topk_ids, shared, gate) -> torch.Tensor:
    """Weighted sum of the chosen experts (``routed`` [T, W], or gathered from ``dense``
    [E, T, W]) + gate[t] * shared[t]."""
    src = routed if routed is not None else dense
    if not _gpu(src):
        return ref.moe_finish(routed, dense, topk_w, topk_ids, shared, gate)
    T, W = src.shape[-2], src.shape[-1]
    out = torch.empty(T, W, dtype=src.dtype, device=src.device)
    _k().moe_finish(out, routed, dense, topk_w, topk_ids, shared, gate)
    return out


def side_gate(pre: torch.Tensor, ids: torch.Tensor, table: torch.Tensor, col0: int) -> torch.Tensor:
    """gelu_tanh(pre [T, n]) * table[ids, col0:col0 + n]."""
    if not _gpu(pre):
        return ref.side_gate(pre, ids, table, col0)
    out = torch.empty_like(pre)
    _k().side_gate(out, pre.contiguous(), ids, table, col0)
    return out


def side_input(x: torch.Tensor, y: Optional[torch.Tensor], mult: float, gate_w: torch.Tensor,
               proj_w: torch.Tensor, ids: torch.Tensor, table: torch.Tensor, col0: int,
               side_w: torch.Tensor, next_w: Optional[torch.Tensor], eps: float,
               out_dtype: Optional[torch.dtype]) -> Optional[torch.Tensor]:
    """The end of a layer with a per-token side input, on the fp32 stream x [T, W] in place:
    x += mult * y (the feed-forward's output);  v = proj_w (gelu_tanh(gate_w x) *
    table[ids, col0:col0 + n]);  x += mult * v / rms(v) * side_w;  returns x / rms(x) * next_w
    in out_dtype (None: nothing).  Decode-size batches of 16-bit activations run as one
    kernel; otherwise a cast, two GEMMs, ``side_gate`` and ``residual_norm``."""
    from .gemm import linear
    if _gpu(x) and x.shape[0] <= 256 and os.environ.get("KGC_SIDE_INPUT", "fused") != "gemm":
        out = (torch.empty(x.shape, dtype=out_dtype, device=x.device)
               if out_dtype is not None and next_w is not None else None)
        if _k().side_input_rows(out, x, y, gate_w, proj_w, ids, table, col0, side_w,
                                next_w if out is not None else None, float(mult), eps):
            return out
    xb = residual_norm(x, y, mult, None, eps, gate_w.dtype)
    g = side_gate(linear(xb, gate_w), ids, table, col0)
    if next_w is None:
        out_dtype = None
    return residual_norm(x, linear(g, proj_w), mult, next_w, eps, out_dtype, add_norm_w=side_w)


# ------------------------------------------------------------------ parallel mixers
# An attention and a recurrence side by side on one input: short causal convolutions over
# per-sequence state, the Mamba-2 recurrence, the gated delta rule, and RMS norms combined
# with a SiLU gate.  State tensors hold one fp32 entry per sequence slot; a chunk that
# starts at position 0 starts from zeros, and rows of slot < 0 (graph padding) are skipped.
def causal_conv(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor],
                state: torch.Tensor, meta, silu: bool = True,
                out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """[T, C] in ``out_dtype`` (fp32, or x's dtype): y[t, c] = act(sum_j w[c, j]
    x[t - (K - 1) + j, c] + bias[c]) per sequence; x [T, C] is a column slice of a
    projection, w fp32 [C, K], state fp32 [slots, K - 1, C] each sequence's last K - 1
    inputs (read, then replaced)."""
    if not _gpu(x):
        return ref.causal_conv(x, w, bias, state, ref.step_sequences(meta), silu, out_dtype)
    out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
    ws, wb = getattr(meta, "work_seq", None), getattr(meta, "work_mblk", None)
    if meta.num_prefills and ws is None:
        qsl = meta.query_start_loc.tolist()
        a, b = prefill_work_list([qsl[i + 1] - qsl[i] for i in range(meta.num_prefills)],
                                 meta.prefill_seq_lens.tolist())
        ws = torch.tensor(a, dtype=torch.int32, device=x.device)
        wb = torch.tensor(b, dtype=torch.int32, device=x.device)
    _k().causal_conv(out, x, w, bias, state, meta.query_start_loc, meta.prefill_seq_lens,
                     meta.decode_ctx_lens, meta.state_slots, ws, wb, meta.num_prefills,
                     meta.num_decodes, meta.num_prefill_tokens, silu)
    return out


def ssd_scan(xbc: torch.Tensor, dt: torch.Tensor, a_log: torch.Tensor, dt_bias: torch.Tensor,
             dskip: torch.Tensor, state: torch.Tensor, meta, H: int, P: int, N: int,
             G: int) -> torch.Tensor:
    """fp32 [T, H P]: the Mamba-2 recurrence over every step sequence's rows from / into
    state [slots, H, N, P]; xbc fp32 [T, H P + 2 G N] = x | B | C, dt [T, H] (a column
    slice of the projection); see ``ref.ssd_scan``."""
    if not _gpu(xbc):
        return ref.ssd_scan(xbc, dt, a_log, dt_bias, dskip, state, ref.step_sequences(meta),
                            H, P, N, G)
    out = torch.empty(xbc.shape[0], H * P, dtype=torch.float32, device=xbc.device)
    _k().ssd_scan(out, xbc, dt, a_log, dt_bias, dskip, state, meta.query_start_loc,
                  meta.prefill_seq_lens, meta.decode_ctx_lens, meta.state_slots,
                  meta.num_prefills, meta.num_decodes, meta.num_prefill_tokens, H, P, N, G)
    return out


def gated_delta_scan(qkv: torch.Tensor, ba: torch.Tensor, a_log: torch.Tensor,
                     dt_bias: torch.Tensor, state: torch.Tensor, meta, H: int, G: int, d: int,
                     dv: int) -> torch.Tensor:
    """fp32 [T, H dv]: the gated delta rule over every step sequence's rows from / into
    state [slots, H, d, dv]; qkv fp32 [T, 2 G d + H dv] = q | k | v, ba [T, 2 H] (a column
    slice of the projection) = write strength | decay pre-activations; see
    ``ref.gated_delta_scan``."""
    if not _gpu(qkv):
        return ref.gated_delta_scan(qkv, ba, a_log, dt_bias, state, ref.step_sequences(meta),
                                    H, G, d, dv)
    out = torch.empty(qkv.shape[0], H * dv, dtype=torch.float32, device=qkv.device)
    _k().gated_delta_scan(out, qkv, ba, a_log, dt_bias, state, meta.query_start_loc,
                          meta.prefill_seq_lens, meta.decode_ctx_lens, meta.state_slots,
                          meta.num_prefills, meta.num_decodes, meta.num_prefill_tokens, H, G,
                          d, dv)
    return out


def gated_rms_norm(y: torch.Tensor, gate: torch.Tensor, w: torch.Tensor, groups: int,
                   eps: float, gate_first: bool, out: torch.Tensor) -> torch.Tensor:
    """out [T, n] (a column slice of a wider buffer) = RMS norm of y (fp32 [T, n]) in
    ``groups`` parts, times w, with silu(gate [T, n], a column slice) applied before the
    norm (gate_first) or after it."""
    if not _gpu(y):
        out.copy_(ref.gated_rms_norm(y, gate, w, groups, eps, gate_first, out.dtype))
        return out
    _k().gated_rms_norm(out, y, gate, w, groups, eps, gate_first)
    return out


# ------------------------------------------------------------------ Lorenex-style decoders
# Gated linear attention with a decay per key channel and the selective scan over
# per-sequence state slots, attention inputs made unit-RMS vectors with a position-dependent
# query factor, PolyNorm, clamped gated experts, softmax routing over all router outputs
# with a choice correction and identity experts.
def embed_pos(ids: torch.Tensor, positions: torch.Tensor, table: torch.Tensor, scale: float,
              pos_table: Optional[torch.Tensor], out: torch.Tensor) -> torch.Tensor:
    """out fp32 [T, W] = table[ids] * scale (+ pos_table[positions]): the start of an fp32
    residual stream with a scaled embedding and learned positions."""
    if not _gpu(out):
        return ref.embed_pos(ids, positions, table, scale, pos_table, out)
    _k().embed_pos(out, ids, positions, table, pos_table, float(scale))
    return out


def gla_scan(proj: torch.Tensor, low: torch.Tensor, a2: torch.Tensor, a2_bias: torch.Tensor,
             state: torch.Tensor, meta, H: int, d: int, dv: int, tau: float) -> torch.Tensor:
    """fp32 [T, H dv]: gated linear attention over every step sequence's rows from / into
    state [slots, H, d, dv]; proj [T, >= 2 H d + H dv] = q | k | v, low [T, r] (a column slice)
    the decay bottleneck, a2 fp32 [H d, r], a2_bias fp32 [H d]; see ``ref.gla_scan``."""
    if not _gpu(proj):
        return ref.gla_scan(proj, low, a2, a2_bias, state, ref.step_sequences(meta), H, d, dv, tau)
    out = torch.empty(proj.shape[0], H * dv, dtype=torch.float32, device=proj.device)
    _k().gla_scan(out, proj, low, a2, a2_bias, state, meta.query_start_loc,
                  meta.prefill_seq_lens, meta.decode_ctx_lens, meta.state_slots,
                  meta.num_prefills, meta.num_decodes, meta.num_prefill_tokens, H, d, dv,
                  float(tau))
    return out


def selective_scan(x: torch.Tensor, dt: torch.Tensor, bc: torch.Tensor, At: torch.Tensor,
                   dt_bias: torch.Tensor, dskip: torch.Tensor, z: torch.Tensor,
                   state: torch.Tensor, meta, out_scale: float, out: torch.Tensor) -> torch.Tensor:
    """out [T, I] (a column slice of a wider buffer) = y * silu(z) * out_scale, y the
    selective scan over every step sequence's rows from / into state [slots, N, I]; x, dt
    [T, I], bc [T, 2 N] and z [T, I] (column slices), At fp32 [N, I]; see
    ``ref.selective_scan``."""
    if not _gpu(x):
        out.copy_(ref.selective_scan(x, dt, bc, At, dt_bias, dskip, z, state,
                                     ref.step_sequences(meta), out_scale, out.dtype))
        return out
    _k().selective_scan(out, x, dt.contiguous(), bc, At, dt_bias, dskip, z, state,
                        meta.query_start_loc,
                        meta.prefill_seq_lens, meta.decode_ctx_lens, meta.state_slots,
                        meta.num_prefills, meta.num_decodes, meta.num_prefill_tokens,
                        float(out_scale))
    return out


def norm_kv_store(qkv: torch.Tensor, positions: torch.Tensor, k_cache: torch.Tensor,
                  v_cache: torch.Tensor, slot_mapping: torch.Tensor, H: int, G: int, dk: int,
                  dv: int, eps: float, qk_unit: bool, v_unit: bool, q_temp,
                  out_dtype: torch.dtype) -> torch.Tensor:
    """q [T, H, dk] in ``out_dtype`` from qkv fp32 [T, H dk + G dk + G dv], k and v into the
    paged cache: head vectors divided by their root mean square (``qk_unit``, ``v_unit``),
    q times 1 + coef * ln(floor((p + 1) / every) + 1) (``q_temp`` = (coef, every) or None)."""
    if not _gpu(qkv):
        return ref.norm_kv_store(qkv, positions, k_cache, v_cache, slot_mapping, H, G, dk, dv,
                                 eps, qk_unit, v_unit, q_temp, out_dtype)
    q = torch.empty(qkv.shape[0], H, dk, dtype=out_dtype, device=qkv.device)
    coef, every = q_temp if q_temp is not None else (0.0, 1)
    _k().norm_kv_store(qkv, positions, q, k_cache, v_cache, slot_mapping, H, G, dk, dv,
                       float(eps), qk_unit, v_unit, float(coef), int(every))
    return q


def polynorm(z: torch.Tensor, coef: torch.Tensor, eps: float) -> torch.Tensor:
    """a N(z) + b N(z^2) + c N(z^3) + e per row of z [T, F], coef fp32 [4]."""
    if not _gpu(z):
        return ref.polynorm(z, coef, eps)
    out = torch.empty_like(z)
    _k().polynorm(out, z, coef, float(eps))
    return out


def swiglu_clamp(x: torch.Tensor, limit: float, alpha: float = 1.702) -> torch.Tensor:
    """x [..., 2 I] = gate | up -> min(gate, limit) sigmoid(alpha .) (clamp(up, +-limit) + 1)."""
    if not _gpu(x):
        return ref.swiglu_clamp(x, limit, alpha)
    I = x.shape[-1] // 2
    x2 = x.reshape(-1, 2 * I)
    out = torch.empty(x2.shape[0], I, dtype=x.dtype, device=x.device)
    _k().swiglu_clamp(out, x2, float(limit), float(alpha))
    return out.view(*x.shape[:-1], I)


def moe_route_softmax_all(logits: torch.Tensor, correction: torch.Tensor, k: int, n_real: int):
    """(weights fp32 [T, k], expert ids int32 [T, k], identity weight fp32 [T]) from router
    logits fp32 [T, >= E]; see ``ref.moe_route_softmax_all``."""
    if not _gpu(logits):
        return ref.moe_route_softmax_all(logits, correction, k, n_real)
    T = logits.shape[0]
    w = torch.empty(T, k, dtype=torch.float32, device=logits.device)
    ids = torch.empty(T, k, dtype=torch.int32, device=logits.device)
    idw = torch.empty(T, dtype=torch.float32, device=logits.device)
    _k().moe_route_softmax_all(w, ids, idw, logits, correction, int(n_real))
    return w, ids, idw
