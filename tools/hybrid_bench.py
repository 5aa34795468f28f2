"""Microbenchmarks of the hybrid-decoder kernels beside the Llama-path kernel each one is
closest to, at the layer shapes of the dilavik-w2048 / konovik-w2048 / nolesun-w2048 /
llama-w2048 presets (``--only nolesun``: the parallel mixers' kernels; ``--only lorenex``: gated
linear attention, the selective scan, unit-RMS attention inputs, PolyNorm, clamped experts).

    python tools/hybrid_bench.py [--reps 20] > profiles/hybrid_kernels.jsonl

One JSON line per kernel and shape: microseconds per call (events around `reps` calls) and
the bytes or FLOPs the call has to move or do at least, as GB/s or TFLOP/s.  Prefill shape:
32 chunks of 512 tokens (16384 rows); decode shapes: 64 and 256 rows at context 544."""
import argparse
import json
import types

import torch

from kubernetes_gpu_cluster_amd import ops
from kubernetes_gpu_cluster_amd.ops import reference as ref

DEV = torch.device("cuda")
BF = torch.bfloat16


def timed(fn, reps):
    for _ in range(3):
        fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(reps):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) * 1e3 / reps


def emit(name, shape, us, gbytes=None, tflop=None, like=None):
    r = {"kernel": name, "shape": shape, "us": round(us, 1)}
    if gbytes is not None:
        r["GB_s"] = round(gbytes / us * 1e6, 0)
    if tflop is not None:
        r["TFLOP_s"] = round(tflop / us * 1e6, 1)
    if like:
        r["like"] = like
    print(json.dumps(r), flush=True)


def meta(P_q, P_sl, D_ctx, bs, dev, slots=None):
    m = types.SimpleNamespace()
    P, D = len(P_q), len(D_ctx)
    lens = P_sl + D_ctx
    mb = max(lens) // bs + 1
    tables = (torch.arange(len(lens) * mb, dtype=torch.int32).view(len(lens), mb) + 1).to(dev)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)   # noqa: E731
    qsl = [0]
    for q in P_q:
        qsl.append(qsl[-1] + q)
    m.num_prefills, m.num_decodes, m.num_prefill_tokens = P, D, qsl[-1]
    m.query_start_loc = i32(qsl) if P else None
    m.prefill_seq_lens = i32(P_sl) if P else None
    m.prefill_block_tables = tables[:P].contiguous() if P else None
    m.decode_ctx_lens = i32(D_ctx) if D else None
    m.decode_block_tables = tables[P:].contiguous() if D else None
    m.state_slots = i32(slots) if slots is not None else None
    if P:
        ws, wb = ops.prefill_work_list(P_q, P_sl)
        m.work_seq, m.work_mblk = i32(ws), i32(wb)
    return m, tables, len(lens) * mb + 1


def attention(reps):
    H, G, d, bs, W, keep = 16, 4, 128, 32, 1024, 4
    for name, P_q, P_sl, D_ctx in (("prefill 32x512", [512] * 32, [512] * 32, []),
                                   ("prefill 8x2048", [2048] * 8, [2048] * 8, []),
                                   ("decode 64 @544", [], [], [544] * 64),
                                   ("decode 256 @544", [], [], [544] * 256)):
        m, tables, nb = meta(P_q, P_sl, D_ctx, bs, DEV)
        T = sum(P_q) + len(D_ctx)
        q = torch.randn(T, H, d, device=DEV, dtype=BF)
        kc = torch.randn(nb, G, bs, d, device=DEV, dtype=BF)
        vc = torch.randn(nb, G, bs, d, device=DEV, dtype=BF)
        gate = torch.rand(T, H, device=DEV)
        pos = torch.zeros(T, dtype=torch.int64, device=DEV)
        us = timed(lambda: ops.window_attention(q, kc, vc, pos, m, 0.09, W, keep, gate), reps)
        # visible (query, key) pairs -> 2 * pairs * (dk + dv) FLOPs per head; decode: K/V bytes
        pairs = sum(sum(min(p + 1, W) + max(0, min(keep, p + 1 - W)) for p in range(sl - ql, sl))
                    for ql, sl in zip(P_q, P_sl))
        if P_q:
            emit("window_attention (MFMA tile)", name, us, tflop=2 * pairs * 2 * d * H / 1e12)
            kc2 = kc
            vc2 = torch.randn(nb, G, bs // 8, d, 8, device=DEV, dtype=BF)
            us2 = timed(lambda: ops.prefill_attention(q, kc2, vc2, m.prefill_block_tables,
                                                      m.query_start_loc, m.prefill_seq_lens, 0.09,
                                                      m.work_seq, m.work_mblk), reps)
            full = sum(sum(p + 1 for p in range(sl - ql, sl)) for ql, sl in zip(P_q, P_sl))
            emit("prefill_attention (K2, causal)", name, us2, tflop=2 * full * 2 * d * H / 1e12,
                 like="window_attention")
        else:
            gb = sum(min(c, W + keep) for c in D_ctx) * G * 2 * d * 2 / 1e9
            emit("window_attention (8-wave decode)", name, us, gbytes=gb)
            vc2 = torch.randn(nb, G, bs // 8, d, 8, device=DEV, dtype=BF)
            z = ops.decode_grid_z(len(D_ctx), G, max(D_ctx))
            ws = ops.decode_partials(len(D_ctx), H, d, tables.shape[1], bs, DEV)
            us2 = timed(lambda: ops.paged_attention_decode(q, kc, vc2, m.decode_block_tables,
                                                           m.decode_ctx_lens, 0.09, ws, z), reps)
            emit("paged_attention_decode (K1)", name, us2, gbytes=sum(D_ctx) * G * 2 * d * 2 / 1e9,
                 like="window_attention")


def recurrent(reps):
    H, d, dv = 4, 256, 512
    N = 2 * H * d + 2 * H * dv
    for name, P_q, D_ctx in (("prefill 32x512", [512] * 32, []), ("decode 64", [], [100] * 64),
                             ("decode 256", [], [100] * 256)):
        n = len(P_q) + len(D_ctx)
        m, _, _ = meta(P_q, list(P_q), D_ctx, 32, DEV, slots=list(range(n)))
        T = sum(P_q) + len(D_ctx)
        qkvg = torch.randn(T, N, device=DEV, dtype=BF)
        gates = torch.cat([torch.randn(T, H, device=DEV), -torch.rand(T, H, device=DEV)], 1)
        st = (torch.zeros(n, H, d, dv, device=DEV), torch.zeros(n, H, d, device=DEV),
              torch.zeros(n, H, device=DEV))
        us = timed(lambda: ops.mlstm_scan(qkvg, gates, st, m, H, d, dv), reps)
        # per token and head: S update + read-out = 4 d dv FLOPs; per step: state read + write
        emit("mlstm_scan", name, us, gbytes=2 * n * H * d * dv * 4 / 1e9,
             tflop=4 * T * H * d * dv / 1e12)


def rows(reps):
    W, L = 2048, 12
    for T in (16384, 64, 256):
        x = torch.randn(T, W, device=DEV)
        y = torch.randn(T, W, device=DEV, dtype=BF)
        w = torch.ones(W, device=DEV)
        hist = torch.randn(L + 1, T, W, device=DEV)
        coef = torch.randn(L + 1, device=DEV)
        us = timed(lambda: ops.group_rms_norm(x, w, 1, 1e-5, BF, add=y), reps)
        emit("group_rms_norm(add)", f"{T}x{W}", us, gbytes=T * W * (4 + 4 + 2 + 2) / 1e9)
        xb, rb, wb = y.clone(), y.clone(), torch.ones(W, device=DEV, dtype=BF)
        us = timed(lambda: ops.fused_add_rms_norm(xb, rb, wb, 1e-5), reps)
        emit("fused_add_rms_norm (K4)", f"{T}x{W}", us, gbytes=T * W * 8 / 1e9,
             like="group_rms_norm(add)")
        for layer in (0, 5, 11):
            us = timed(lambda: ops.depth_mix_norm(x, hist, layer, y, coef, w, 1, 1e-5, BF), reps)
            emit(f"depth_mix_norm layer {layer}", f"{T}x{W}", us,
                 gbytes=T * W * (4 * (layer + 1) + 4 + 4 + 4 + 2 + 2) / 1e9)
        z = torch.randn(T, 8256, device=DEV, dtype=BF)
        ab = torch.tensor([0.7, 1.2], device=DEV)
        us = timed(lambda: ops.xielu(z, ab), reps)
        emit("xielu", f"{T}x8256", us, gbytes=T * 8256 * 4 / 1e9)
        gu = torch.randn(T, 2 * 5504, device=DEV, dtype=BF)
        us = timed(lambda: ops.silu_mul(gu), reps)
        emit("silu_mul (K7)", f"{T}x5504", us, gbytes=T * 5504 * 6 / 1e9, like="xielu")
        h = torch.randn(T, W, device=DEV, dtype=BF)
        wg = torch.randn(16, W, device=DEV, dtype=BF)
        us = timed(lambda: ops.gate_proj(h, wg, None, ops.GATE_SIGMOID), reps)
        emit("gate_proj N=16", f"{T}x{W}", us, gbytes=T * W * 2 / 1e9)
        o = torch.randn(T, 2048, device=DEV)
        g = torch.randn(T, 2048, device=DEV, dtype=BF)
        us = timed(lambda: ops.head_norm_gate(o, g, w, 4, 1e-5, BF), reps)
        emit("head_norm_gate", f"{T}x2048", us, gbytes=T * 2048 * 8 / 1e9)
        # rotary + cache store
        H, G, d, bs = 16, 4, 128, 32
        nb = T // bs + 2
        qkv = torch.randn(T, (H + 2 * G) * d, device=DEV, dtype=BF)
        kc = torch.zeros(nb, G, bs, d, device=DEV, dtype=BF)
        vc = torch.zeros(nb, G, bs, d, device=DEV, dtype=BF)
        pos = (torch.arange(T, device=DEV) % 512).to(torch.int64)
        slots = torch.arange(T, device=DEV, dtype=torch.int64) + bs
        table = ref.rope_table(64, 4096, 1e4).to(DEV)
        us = timed(lambda: ops.rope_kv_store(qkv, pos, table, kc, vc, slots, H, G, d, d), reps)
        emit("rope_kv_store", f"{T} rows", us, gbytes=T * (H + 2 * G) * d * 4 / 1e9)
        cs = ref.rope_cos_sin_cache(d, 4096, 1e4).to(DEV)
        vc2 = torch.zeros(nb, G, bs // 8, d, 8, device=DEV, dtype=BF)
        us = timed(lambda: ops.rope_kv_write(qkv, pos, cs, kc, vc2, slots, H, G, d), reps)
        emit("rope_kv_write (K3)", f"{T} rows", us, gbytes=T * (H + 2 * G) * d * 4 / 1e9,
             like="rope_kv_store")


def konovik(reps):
    """The Konovik-style kernels at the konovik-w2048 layer shapes, each beside the kernel of
    the other hybrid decoder (or of the Llama / Mixtral path) it is closest to."""
    # ---- latent attention: 16 heads over one cache row of 192 + 64 per token, window 1024
    H, rank, r, bs, Wn = 16, 192, 64, 32, 1024
    dk = rank + r
    for name, P_q, P_sl, D_ctx in (("prefill 32x512", [512] * 32, [512] * 32, []),
                                   ("prefill 8x2048", [2048] * 8, [2048] * 8, []),
                                   ("decode 64 @544", [], [], [544] * 64),
                                   ("decode 256 @544", [], [], [544] * 256)):
        m, tables, nb = meta(P_q, P_sl, D_ctx, bs, DEV)
        T = sum(P_q) + len(D_ctx)
        q = torch.randn(T, H, dk, device=DEV, dtype=BF)
        cache = torch.randn(nb, 1, bs, dk, device=DEV, dtype=BF)
        pos = torch.zeros(T, dtype=torch.int64, device=DEV)
        us = timed(lambda: ops.window_attention(q, cache, cache[..., :rank], pos, m, 0.07, Wn, 0,
                                                None), reps)
        pairs = sum(sum(min(p + 1, Wn) for p in range(sl - ql, sl)) for ql, sl in zip(P_q, P_sl))
        if P_q:
            emit("window_attention, latent rows (MFMA tile)", name, us,
                 tflop=2 * pairs * (dk + rank) * H / 1e12, like="window_attention (MFMA tile)")
        else:
            emit("window_attention, latent rows (8-wave decode)", name, us,
                 gbytes=sum(min(c, Wn) for c in D_ctx) * dk * 2 / 1e9,
                 like="window_attention (8-wave decode)")
    # ---- minGRU scan (width 4096) beside the mLSTM scan of the same rows
    n_ch = 4096
    for name, P_q, D_ctx in (("prefill 32x512", [512] * 32, []), ("prefill 2x8192", [8192] * 2, []),
                             ("decode 64", [], [100] * 64), ("decode 256", [], [100] * 256)):
        n = len(P_q) + len(D_ctx)
        m, _, _ = meta(P_q, list(P_q), D_ctx, 32, DEV, slots=list(range(n)))
        T = sum(P_q) + len(D_ctx)
        zxg = torch.randn(T, 3 * n_ch, device=DEV, dtype=BF)
        bias = torch.randn(2 * n_ch, device=DEV)
        st = torch.zeros(n, n_ch, device=DEV)
        us = timed(lambda: ops.mingru_scan(zxg, bias, st, m, n_ch, BF), reps)
        emit("mingru_scan", name, us, gbytes=(T * n_ch * 8 + 2 * n * n_ch * 4) / 1e9, like="mlstm_scan")
    W = 2048
    for T in (16384, 64, 256):
        x = torch.randn(T, W, device=DEV)
        y = torch.randn(T, W, device=DEV, dtype=BF)
        w = torch.ones(W, device=DEV)
        us = timed(lambda: ops.residual_norm(x, y, 0.3, w, 1e-6, BF), reps)
        emit("residual_norm (add, norm -> 16 bit)", f"{T}x{W}", us, gbytes=T * W * 12 / 1e9,
             like="group_rms_norm(add)")
        us = timed(lambda: ops.residual_norm(x, y, 0.3, w, 1e-6, torch.float32, add_norm_w=w), reps)
        emit("residual_norm (normed add, norm -> fp32)", f"{T}x{W}", us, gbytes=T * W * 14 / 1e9,
             like="group_rms_norm(add)")
        n = 64 if T > 256 else T
        P_q, D_ctx = ([T // n] * n, []) if T > 256 else ([], [100] * T)
        m, _, _ = meta(P_q, list(P_q), D_ctx, 32, DEV, slots=list(range(n)))
        h = torch.randn(T, W, device=DEV)
        st = torch.zeros(n, W, device=DEV)
        us = timed(lambda: ops.token_shift(h, w, st, m, BF), reps)
        emit("token_shift", f"{T}x{W}", us, gbytes=T * W * (4 + 4 + 2) / 1e9, like="group_rms_norm(add)")
        # latent cache rows + query rows beside rotary + store of the windowed attention
        d = 128
        proj = torch.randn(T, H * (d + r) + dk + H * d, device=DEV, dtype=BF)
        q_lat = torch.randn(H, T, rank, device=DEV, dtype=BF)
        nb = T // bs + 2
        cache = torch.zeros(nb, 1, bs, dk, device=DEV, dtype=BF)
        pos = (torch.arange(T, device=DEV) % 512).to(torch.int64)
        slots = torch.arange(T, device=DEV, dtype=torch.int64) + bs
        table = ref.rope_table_yarn(r, 4096, 1e4, (8.0, 4096.0, 16.0, 2.0)).to(DEV)
        us = timed(lambda: ops.latent_rope_store(proj, q_lat, pos, table, torch.ones(rank, device=DEV),
                                                 1e-6, cache, slots, H, d, r, rank), reps)
        emit("latent_rope_store", f"{T} rows", us,
             gbytes=T * (H * r * 2 + H * rank * 2 + H * dk * 2 + 2 * dk * 2) / 1e9, like="rope_kv_store")
        o = torch.randn(H, T, d, device=DEV, dtype=BF)
        g = torch.randn(T, H * d, device=DEV, dtype=BF)
        us = timed(lambda: ops.gate_mul(o.transpose(0, 1), g), reps)
        emit("gate_mul", f"{T}x{H * d}", us, gbytes=T * H * d * 6 / 1e9, like="head_norm_gate")
        z = torch.randn(T * 2, 2048, device=DEV, dtype=BF)
        us = timed(lambda: ops.relu_sq(z), reps)
        emit("relu_sq", f"{2 * T}x2048", us, gbytes=T * 2 * 2048 * 4 / 1e9, like="silu_mul (K7)")
        # routing: 8 experts + the shared gate, top 2
        hb = torch.randn(T, W, device=DEV, dtype=BF)
        wg = torch.randn(9, W, device=DEV, dtype=BF)
        us = timed(lambda: ops.gate_proj(hb, wg, None, ops.GATE_SIGMOID), reps)
        emit("gate_proj N=9 (router scores)", f"{T}x{W}", us, gbytes=T * W * 2 / 1e9, like="gate_proj N=16")
        sc = torch.rand(T, 9, device=DEV)
        corr = torch.randn(8, device=DEV) * 0.1
        us = timed(lambda: ops.moe_route_sigmoid(sc, corr, 2, 1.5), reps)
        emit("moe_route_sigmoid", f"{T}x8 top 2", us, gbytes=T * (36 + 16) / 1e9)
        lg = torch.randn(T, 8, device=DEV, dtype=BF)
        us = timed(lambda: ops.moe_topk_softmax(lg, 2), reps)
        emit("moe_topk_softmax (K13)", f"{T}x8 top 2", us, gbytes=T * (16 + 16) / 1e9,
             like="moe_route_sigmoid")
        routed = torch.randn(T, W, device=DEV, dtype=BF)
        shared = torch.randn(T, W, device=DEV, dtype=BF)
        us = timed(lambda: ops.moe_finish(routed, None, None, None, shared, sc[:, 8]), reps)
        emit("moe_finish (routed + gated shared)", f"{T}x{W}", us, gbytes=T * W * 6 / 1e9,
             like="silu_mul (K7)")
        if T <= 256:
            import os
            wsg = torch.randn(64, W, device=DEV, dtype=BF) / 45
            wsp = torch.randn(W, 64, device=DEV, dtype=BF) / 8
            tab2 = torch.randn(32000, 640, device=DEV, dtype=BF)
            ids2 = torch.randint(0, 32000, (T,), device=DEV)
            for mode in ("fused", "gemm"):
                os.environ["KGC_SIDE_INPUT"] = mode
                us = timed(lambda: ops.side_input(x, y, 0.3, wsg, wsp, ids2, tab2, 128, w, w, 1e-6,
                                                  torch.float32), reps)
                emit(f"side_input ({'one kernel' if mode == 'fused' else 'cast, 2 GEMMs, gate, add + norm'})",
                     f"{T}x{W}", us)
            os.environ.pop("KGC_SIDE_INPUT")
        pre = torch.randn(T, 64, device=DEV, dtype=BF)
        ids = torch.randint(0, 32000, (T,), device=DEV)
        tab = torch.randn(32000, 640, device=DEV, dtype=BF)
        us = timed(lambda: ops.side_gate(pre, ids, tab, 128), reps)
        emit("side_gate", f"{T}x64", us, gbytes=T * 64 * 6 / 1e9)


def nolesun(reps):
    """The parallel mixers' kernels at the nolesun-w2048 layer shapes: the causal convolution,
    both scans, the gated norms, and the attention with capped scores writing a column slice."""
    W = 2048
    shapes = (("prefill 32x512", [512] * 32, []), ("prefill 2x8192", [8192] * 2, []),
              ("decode 64", [], [544] * 64), ("decode 256", [], [544] * 256))
    for name, P_q, D_ctx in shapes:
        n = len(P_q) + len(D_ctx)
        m, _, _ = meta(P_q, list(P_q), D_ctx, 32, DEV, slots=list(range(n)))
        T = sum(P_q) + len(D_ctx)
        # Mamba-2: 32 heads of 64, state 128, one group, 4 taps
        H, V, N, G, K = 32, 64, 128, 1, 4
        C = H * V + 2 * G * N
        proj = torch.randn(T, 2 * H * V + 2 * G * N + H, device=DEV, dtype=BF)
        cw, cb = torch.randn(C, K, device=DEV) * 0.3, torch.randn(C, device=DEV) * 0.1
        cst = torch.zeros(n, K - 1, C, device=DEV)
        us = timed(lambda: ops.causal_conv(proj[:, H * V: H * V + C], cw, cb, cst, m), reps)
        emit("causal_conv (x | B | C, 4 taps)", name, us, gbytes=T * C * 6 / 1e9, like="token_shift")
        xbc = torch.randn(T, C, device=DEV)
        par = (torch.rand(H, device=DEV), torch.randn(H, device=DEV) - 2, torch.ones(H, device=DEV))
        S = torch.zeros(n, H, N, V, device=DEV)
        us = timed(lambda: ops.ssd_scan(xbc, proj[:, -H:], *par, S, m, H, V, N, G), reps)
        emit("ssd_scan", name, us, gbytes=2 * n * H * N * V * 4 / 1e9, tflop=4 * T * H * N * V / 1e12,
             like="mlstm_scan")
        y = torch.randn(T, H * V, device=DEV)
        feats = torch.empty(T, 2 * W, device=DEV, dtype=BF)
        nw = torch.ones(H * V, device=DEV)
        us = timed(lambda: ops.gated_rms_norm(y, proj[:, : H * V], nw, 1, 1e-6, True, feats[:, W:]), reps)
        emit("gated_rms_norm (gate, then norm of the row)", f"{T}x{H * V}", us,
             gbytes=T * H * V * 8 / 1e9, like="head_norm_gate")
        # gated delta rule: 16 heads of 128 x 128 over 8 query / key heads, 4 taps
        H, G, d, V = 16, 8, 128, 128
        C = 2 * G * d + H * V
        proj = torch.randn(T, C + H * V + 2 * H, device=DEV, dtype=BF)
        cw = torch.randn(C, K, device=DEV) * 0.3
        cst = torch.zeros(n, K - 1, C, device=DEV)
        us = timed(lambda: ops.causal_conv(proj[:, :C], cw, None, cst, m), reps)
        emit("causal_conv (q | k | v, 4 taps)", name, us, gbytes=T * C * 6 / 1e9, like="token_shift")
        qkv = torch.randn(T, C, device=DEV)
        S = torch.zeros(n, H, d, V, device=DEV)
        us = timed(lambda: ops.gated_delta_scan(qkv, proj[:, -2 * H:], par[0][:H], par[1][:H], S, m,
                                                H, G, d, V), reps)
        emit("gated_delta_scan", name, us, gbytes=2 * n * H * d * V * 4 / 1e9,
             tflop=6 * T * H * d * V / 1e12, like="mlstm_scan")
        o = torch.randn(T, H * V, device=DEV)
        nw = torch.ones(H * V, device=DEV)
        us = timed(lambda: ops.gated_rms_norm(o, proj[:, C: C + H * V], nw, H, 1e-6, False,
                                              feats[:, W:]), reps)
        emit("gated_rms_norm (norm per head, then gate)", f"{T}x{H * V}", us,
             gbytes=T * H * V * 8 / 1e9, like="head_norm_gate")
    # attention: plain causal with a score cap, into a column slice, beside the windowed kernel
    H, G, d, bs = 16, 4, 128, 32
    for name, P_q, P_sl, D_ctx in (("prefill 32x512", [512] * 32, [512] * 32, []),
                                   ("prefill 8x2048", [2048] * 8, [2048] * 8, []),
                                   ("decode 64 @544", [], [], [544] * 64),
                                   ("decode 256 @544", [], [], [544] * 256)):
        m, tables, nb = meta(P_q, P_sl, D_ctx, bs, DEV)
        T = sum(P_q) + len(D_ctx)
        q = torch.randn(T, H, d, device=DEV, dtype=BF)
        kc = torch.randn(nb, G, bs, d, device=DEV, dtype=BF)
        vc = torch.randn(nb, G, bs, d, device=DEV, dtype=BF)
        pos = torch.zeros(T, dtype=torch.int64, device=DEV)
        feats = torch.empty(T, 2 * H * d, device=DEV, dtype=BF)
        keys = sum(s * (s + 1) // 2 for s in P_sl) if P_q else sum(D_ctx)
        for cap in (0.0, 30.0):
            us = timed(lambda: ops.window_attention(q, kc, vc, pos, m, 0.09, 0, 0, None, cap, 1.2,
                                                    out=feats[:, : H * d]), reps)
            emit("window_attention (causal%s, into a slice)" % (", capped" if cap else ""), name, us,
                 gbytes=None if P_q else keys * G * 2 * d * 2 / 1e9,
                 tflop=keys * H * 4 * d / 1e12 if P_q else None, like="window_attention")


def lorenex(reps):
    """The Lorenex kernels at the lorenex-w2048 layer shapes, each beside the closest kernel of
    the other decoders at the same shape (``like``)."""
    W = 2048
    shapes = (("prefill 32x512", [512] * 32, []), ("prefill 2x8192", [8192] * 2, []),
              ("decode 64", [], [544] * 64), ("decode 256", [], [544] * 256))
    for name, P_q, D_ctx in shapes:
        n = len(P_q) + len(D_ctx)
        m, _, nb = meta(P_q, list(P_q), D_ctx, 32, DEV, slots=list(range(n)))
        T = sum(P_q) + len(D_ctx)
        pos = torch.arange(T, dtype=torch.int64, device=DEV) % 512
        slots = torch.arange(T, dtype=torch.int64, device=DEV) + 32
        # gated linear attention: 8 heads of 128 x 256, decay bottleneck 16
        H, d, V, R = 8, 128, 256, 16
        proj = torch.randn(T, 2 * H * d + 2 * H * V + R, device=DEV, dtype=BF)
        a2, a2b = torch.randn(H * d, R, device=DEV) * 0.3, torch.randn(H * d, device=DEV) + 3
        S = torch.zeros(n, H, d, V, device=DEV)
        us = timed(lambda: ops.gla_scan(proj, proj[:, -R:], a2, a2b, S, m, H, d, V, 16.0), reps)
        emit("gla_scan", name, us, gbytes=2 * n * H * d * V * 4 / 1e9,
             tflop=4 * T * H * d * V / 1e12, like="gated_delta_scan")
        S2 = torch.zeros(n, 16, 128, 128, device=DEV)
        qkv = torch.randn(T, 2 * 8 * 128 + 16 * 128, device=DEV)
        par = (torch.rand(16, device=DEV), torch.randn(16, device=DEV) - 2)
        us = timed(lambda: ops.gated_delta_scan(qkv, proj[:, :32], *par, S2, m, 16, 8, 128, 128), reps)
        emit("gated_delta_scan (same state bytes)", name, us, gbytes=2 * n * 16 * 128 * 128 * 4 / 1e9,
             tflop=6 * T * 16 * 128 * 128 / 1e12)
        # attention inputs: 16 query / 4 key-value heads of 128, 4 taps, unit-RMS vectors
        Hq, G, dk, K = 16, 4, 128, 4
        C = (Hq + 2 * G) * dk
        aproj = torch.randn(T, C + 2 * W, device=DEV, dtype=BF)
        cw = torch.randn(C, K, device=DEV) * 0.3
        cst = torch.zeros(n, K - 1, C, device=DEV)
        us = timed(lambda: ops.causal_conv(aproj[:, :C], cw, None, cst, m, False), reps)
        emit("causal_conv (q | k | v, 4 taps, no activation)", name, us, gbytes=T * C * 6 / 1e9,
             like="causal_conv")
        conv = torch.randn(T, C, device=DEV)
        kc = torch.zeros(nb + 2, G, 32, dk, device=DEV, dtype=BF)
        vc = torch.zeros(nb + 2, G, 32, dk, device=DEV, dtype=BF)
        us = timed(lambda: ops.norm_kv_store(conv, pos, kc, vc, slots, Hq, G, dk, dk, 1e-5, True, True,
                                             (0.5, 1024), BF), reps)
        emit("norm_kv_store", name, us, gbytes=T * C * 6 / 1e9, like="rope_kv_store")
        rope = ref.rope_table(64, 1024, 1e4).to(DEV)
        us = timed(lambda: ops.rope_kv_store(aproj[:, :C], pos, rope, kc, vc, slots, Hq, G, dk, dk), reps)
        emit("rope_kv_store (same heads)", name, us, gbytes=T * C * 4 / 1e9)
        # selective scan: 2048 channels of 16 states, 4 taps, gate in the epilogue
        I, N = W, 16
        xw, xb = torch.randn(I, K, device=DEV) * 0.3, torch.randn(I, device=DEV) * 0.1
        xst = torch.zeros(n, K - 1, I, device=DEV)
        us = timed(lambda: ops.causal_conv(aproj[:, C: C + I], xw, xb, xst, m, True, BF), reps)
        emit("causal_conv (x, 4 taps, 16-bit out)", name, us, gbytes=T * I * 4 / 1e9, like="causal_conv")
        x = torch.randn(T, I, device=DEV, dtype=BF)
        dt = torch.randn(T, I, device=DEV, dtype=BF)
        dbc = torch.randn(T, 128 + 2 * N, device=DEV, dtype=BF)
        At = -(1 + 15 * torch.rand(N, I, device=DEV))
        dtb, D = torch.randn(I, device=DEV) - 3, torch.ones(I, device=DEV)
        Ss = torch.zeros(n, N, I, device=DEV)
        feats = torch.empty(T, 2 * W, device=DEV, dtype=BF)
        us = timed(lambda: ops.selective_scan(x, dt, dbc[:, 128:], At, dtb, D, aproj[:, C + I:], Ss, m,
                                              1.0, feats[:, W:]), reps)
        emit("selective_scan (+ gate)", name, us, gbytes=(2 * n * N * I * 4 + T * I * 8) / 1e9,
             tflop=6 * T * N * I / 1e12, like="ssd_scan")
        # feed-forwards: PolyNorm on 8256 columns, clamped gated experts of 2752, routing over 9
        z = torch.randn(T, 8256, device=DEV, dtype=BF)
        coef = torch.tensor([1.0, 0.3, 0.1, 0.0], device=DEV)
        us = timed(lambda: ops.polynorm(z, coef, 1e-5), reps)
        emit("polynorm", f"{T}x8256", us, gbytes=T * 8256 * 4 / 1e9, like="relu_sq")
        us = timed(lambda: ops.relu_sq(z), reps)
        emit("relu_sq (same shape)", f"{T}x8256", us, gbytes=T * 8256 * 4 / 1e9)
        gu = torch.randn(2 * T, 2 * 2752, device=DEV, dtype=BF)
        us = timed(lambda: ops.swiglu_clamp(gu, 7.0), reps)
        emit("swiglu_clamp", f"{2 * T}x2752", us, gbytes=2 * T * 2752 * 6 / 1e9, like="silu_mul")
        us = timed(lambda: ops.silu_mul(gu), reps)
        emit("silu_mul (same shape)", f"{2 * T}x2752", us, gbytes=2 * T * 2752 * 6 / 1e9)
        logits = torch.randn(T, 9, device=DEV)
        corr = torch.randn(9, device=DEV) * 0.01
        us = timed(lambda: ops.moe_route_softmax_all(logits, corr, 2, 8), reps)
        emit("moe_route_softmax_all", f"{T}x9", us, like="moe_topk_softmax")
        us = timed(lambda: ops.moe_topk_softmax(logits[:, :8].contiguous(), 2), reps)
        emit("moe_topk_softmax (8 experts)", f"{T}x8", us)
        ids = torch.randint(0, 32000, (T,), device=DEV)
        tab = torch.randn(32000, W, device=DEV, dtype=BF)
        ptab = torch.randn(8192, W, device=DEV)
        xs = torch.empty(T, W, device=DEV)
        us = timed(lambda: ops.embed_pos(ids, pos, tab, 45.0, ptab, xs), reps)
        emit("embed_pos", f"{T}x{W}", us, gbytes=T * W * 10 / 1e9)


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--reps", type=int, default=20)
    ap.add_argument("--only", default="attention,recurrent,rows,konovik")
    a = ap.parse_args()
    ops.load_extension(strict=True)
    for part in a.only.split(","):
        {"attention": attention, "recurrent": recurrent, "rows": rows, "konovik": konovik,
         "nolesun": nolesun, "lorenex": lorenex}[part](a.reps)
