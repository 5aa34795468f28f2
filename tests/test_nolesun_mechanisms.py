"""Each mechanism of the Nolesun decoder alone (the product's op or module) against the
numpy oracle's function for it, on the CPU reference ops and, with ``-m gpu``, on the HIP
kernels: rotary layouts, attention with a planted stand-out key (far back, at page borders,
the first token; capped scores), the causal convolution and both recurrences over portions
of every size with state carried in slots, the gated norms, both feed-forwards, and the
whole parallel mixer."""
import types

import numpy as np
import pytest
import torch

import nolesun_oracle as oracle
from kubernetes_gpu_cluster_amd import ops
from kubernetes_gpu_cluster_amd.models.attention import ForwardContext
from kubernetes_gpu_cluster_amd.models.configs import FeedForwardSpec, _nolesun_spec
from kubernetes_gpu_cluster_amd.models.moe import SoftmaxRoutedExperts
from kubernetes_gpu_cluster_amd.models.nolesun import ParallelMixer, ReluSqMLP

DEV = [pytest.param("cpu", id="cpu"), pytest.param("cuda", marks=pytest.mark.gpu, id="gpu")]
PAGE = 8


def dev_of(name):
    if name == "cuda" and not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device(name)


def f32(a, dev):
    return torch.tensor(np.asarray(a), dtype=torch.float32, device=dev)


def meta_for(chunks, decodes, tables, dev, slots=None):
    """chunks: [(first position, length)], decodes: [position] -> (metadata, positions)."""
    m = types.SimpleNamespace()
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)   # noqa: E731
    P, D = len(chunks), len(decodes)
    qsl = np.concatenate([[0], np.cumsum([n for _, n in chunks])]).astype(int).tolist()
    m.num_prefills, m.num_decodes, m.num_prefill_tokens = P, D, qsl[-1]
    m.query_start_loc = i32(qsl) if P else None
    m.prefill_seq_lens = i32([a + n for a, n in chunks]) if P else None
    m.prefill_block_tables = tables[:P].contiguous().to(dev) if P and tables is not None else None
    m.decode_ctx_lens = i32([p + 1 for p in decodes]) if D else None
    m.decode_block_tables = tables[P:P + D].contiguous().to(dev) if D and tables is not None else None
    m.state_slots = i32(slots) if slots is not None else None
    m.work_seq = m.work_mblk = None
    pos = [p for a, n in chunks for p in range(a, a + n)] + list(decodes)
    m.slot_mapping = None
    return m, torch.tensor(pos, dtype=torch.int64, device=dev)


def steps_of(n, cuts):
    """[(lo, hi, is a decode row)] for a sequence fed in portions `cuts` (the last repeats)."""
    out, lo, i = [], 0, 0
    while lo < n:
        c = cuts[min(i, len(cuts) - 1)]
        i += 1
        hi = min(n, lo + c)
        out.append((lo, hi, hi - lo == 1 and lo > 0))
        lo = hi
    return out


def over_steps(n, cuts, dev, fn, slot=2, other=None):
    """Run ``fn(rows lo..hi, meta) -> [hi - lo, ...]`` over the portions of one sequence in
    state slot ``slot``.  ``other`` = (n2, fn2 rows -> None): a second sequence in slot 0
    that decodes one token per step beside it (its rows come last in a prefill step and
    first never: prefill chunks precede decode rows)."""
    got = []
    for lo, hi, dec in steps_of(n, cuts):
        m, _ = meta_for([] if dec else [(lo, hi - lo)], [lo] if dec else [], None, dev, [slot])
        got.append(fn(lo, hi, m).cpu().numpy())
    return np.concatenate(got)


CUTS = [[200], [1], [2], [3, 1, 2, 70, 1, 1, 40, 2], [64, 65, 1], [17, 16, 15, 1]]


# ---------------------------------------------------------------- convolution
@pytest.mark.parametrize("dev", DEV)
@pytest.mark.parametrize("K,bias", [(4, False), (3, True), (2, True), (5, False), (1, True)])
@pytest.mark.parametrize("C,off,pad", [(37, 3, 5), (72, 8, 4)], ids=["odd", "aligned"])
def test_causal_conv_over_steps(dev, K, bias, C, off, pad):
    """Columns of a wider matrix at an odd offset, and at an offset, width and row stride
    that are multiples of four (the GPU kernel then walks four channels per thread)."""
    dev = dev_of(dev)
    rng = np.random.default_rng(K)
    n = 150
    x, w = rng.normal(size=(n, C)), rng.normal(size=(C, K))
    b = rng.normal(size=C) if bias else None
    want = oracle.silu(oracle.short_conv(x, w, b))
    wide = f32(np.concatenate([rng.normal(size=(n, off)), x, rng.normal(size=(n, pad))], 1), dev)
    for cuts in CUTS:
        state = torch.full((4, max(K - 1, 1), C), 9.0, device=dev)    # another request's leftovers
        got = over_steps(n, cuts, dev, lambda lo, hi, m: ops.causal_conv(
            wide[lo:hi, off:off + C], f32(w, dev), f32(b, dev) if bias else None, state, m))
        np.testing.assert_allclose(got, want, rtol=2e-5, atol=2e-5, err_msg=str(cuts))
        if K > 1:     # the state holds the last K - 1 inputs, oldest first
            np.testing.assert_allclose(state[2].cpu().numpy(), x[n - (K - 1):], rtol=1e-6, atol=1e-6)
            assert float(state[1].min()) == 9.0


@pytest.mark.parametrize("dev", DEV)
def test_causal_conv_batch_of_unequal_sequences(dev):
    """Three prompts' portions and two decode rows in one step, against each alone."""
    dev = dev_of(dev)
    rng = np.random.default_rng(7)
    C, K = 70, 4
    w = rng.normal(size=(C, K))
    seqs = {s: rng.normal(size=(n, C)) for s, n in ((0, 140), (1, 9), (2, 30), (3, 12), (4, 3))}
    want = {s: oracle.silu(oracle.short_conv(x, w)) for s, x in seqs.items()}
    state = torch.zeros(5, K - 1, C, device=dev)
    # step 1: prompts 0, 1, 2 in part; sequences 3 and 4 up to their last token
    m, _ = meta_for([(0, 130), (0, 2), (0, 30), (0, 11), (0, 2)], [], None, dev, [0, 1, 2, 3, 4])
    rows = [seqs[0][:130], seqs[1][:2], seqs[2], seqs[3][:11], seqs[4][:2]]
    got = ops.causal_conv(f32(np.concatenate(rows), dev), f32(w, dev), None, state, m).cpu().numpy()
    o = 0
    for s, r in zip(range(5), rows):
        np.testing.assert_allclose(got[o:o + len(r)], want[s][:len(r)], rtol=2e-5, atol=2e-5)
        o += len(r)
    # step 2: the rest of 0 and 1 as portions, 3 and 4 as decode rows
    m, _ = meta_for([(130, 10), (2, 7)], [11, 2], None, dev, [0, 1, 3, 4])
    rows = [seqs[0][130:], seqs[1][2:], seqs[3][11:], seqs[4][2:]]
    got = ops.causal_conv(f32(np.concatenate(rows), dev), f32(w, dev), None, state, m).cpu().numpy()
    o = 0
    for s, lo, r in zip((0, 1, 3, 4), (130, 2, 11, 2), rows):
        np.testing.assert_allclose(got[o:o + len(r)], want[s][lo:lo + len(r)], rtol=2e-5, atol=2e-5)
        o += len(r)


# ---------------------------------------------------------------- recurrences
def ssd_oracle(x, B, C, dt, a_log, dt_bias, D, H, V, N, G):
    T = x.shape[0]
    x, B, C = x.reshape(T, H, V), B.reshape(T, G, N), C.reshape(T, G, N)
    step = oracle.softplus(dt + dt_bias)
    y = np.zeros((T, H, V))
    for h in range(H):
        S = np.zeros((N, V))
        for t in range(T):
            S = np.exp(-np.exp(a_log[h]) * step[t, h]) * S + step[t, h] * np.outer(B[t, h // (H // G)], x[t, h])
            y[t, h] = C[t, h // (H // G)] @ S + D[h] * x[t, h]
    return y.reshape(T, H * V)


@pytest.mark.parametrize("dev", DEV)
@pytest.mark.parametrize("H,V,N,G", [(4, 8, 12, 2), (2, 80, 20, 1), (3, 5, 9, 3), (2, 64, 128, 2)])
def test_ssd_scan_over_steps(dev, H, V, N, G):
    dev = dev_of(dev)
    rng = np.random.default_rng(H * V)
    n = 120
    xbc = rng.normal(size=(n, H * V + 2 * G * N))
    dt, a_log, dtb, D = rng.normal(size=(n, H)), rng.normal(size=H) * 0.5, rng.normal(size=H), rng.normal(size=H)
    want = ssd_oracle(xbc[:, :H * V], xbc[:, H * V:H * V + G * N], xbc[:, H * V + G * N:], dt, a_log,
                      dtb, D, H, V, N, G)
    dtw = f32(np.concatenate([rng.normal(size=(n, 2)), dt], 1), dev)
    for cuts in CUTS[1:] if N == 128 else CUTS:
        state = torch.full((4, H, N, V), 5.0, device=dev)
        got = over_steps(n, cuts, dev, lambda lo, hi, m: ops.ssd_scan(
            f32(xbc[lo:hi], dev), dtw[lo:hi, 2:], f32(a_log, dev), f32(dtb, dev), f32(D, dev),
            state, m, H, V, N, G))
        np.testing.assert_allclose(got, want, rtol=2e-4, atol=2e-4 * np.abs(want).max(), err_msg=str(cuts))


def delta_oracle(q, k, v, b, a, a_log, dt_bias, H, G, d, V):
    T = q.shape[0]
    q, k, v = q.reshape(T, G, d), k.reshape(T, G, d), v.reshape(T, H, V)
    q = q / np.sqrt((q * q).sum(-1, keepdims=True) + 1e-6) / np.sqrt(d)
    k = k / np.sqrt((k * k).sum(-1, keepdims=True) + 1e-6)
    beta, keep = oracle.logistic(b), np.exp(-np.exp(a_log) * oracle.softplus(a + dt_bias))
    o = np.zeros((T, H, V))
    for h in range(H):
        g = h // (H // G)
        S = np.zeros((d, V))
        for t in range(T):
            S = keep[t, h] * S
            u = beta[t, h] * (v[t, h] - k[t, g] @ S)
            S = S + np.outer(k[t, g], u)
            o[t, h] = q[t, g] @ S
    return o.reshape(T, H * V)


@pytest.mark.parametrize("dev", DEV)
@pytest.mark.parametrize("H,G,d,V", [(4, 2, 10, 6), (2, 2, 24, 72), (6, 3, 7, 11), (2, 1, 128, 64)])
def test_gated_delta_scan_over_steps(dev, H, G, d, V):
    dev = dev_of(dev)
    rng = np.random.default_rng(H * d)
    n = 120
    qkv = rng.normal(size=(n, 2 * G * d + H * V))
    ba, a_log, dtb = rng.normal(size=(n, 2 * H)), rng.normal(size=H) * 0.5, rng.normal(size=H)
    want = delta_oracle(qkv[:, :G * d], qkv[:, G * d:2 * G * d], qkv[:, 2 * G * d:], ba[:, :H],
                        ba[:, H:], a_log, dtb, H, G, d, V)
    baw = f32(np.concatenate([rng.normal(size=(n, 1)), ba], 1), dev)
    for cuts in CUTS[1:] if d == 128 else CUTS:
        state = torch.full((4, H, d, V), 5.0, device=dev)
        got = over_steps(n, cuts, dev, lambda lo, hi, m: ops.gated_delta_scan(
            f32(qkv[lo:hi], dev), baw[lo:hi, 1:], f32(a_log, dev), f32(dtb, dev), state, m, H, G, d, V))
        np.testing.assert_allclose(got, want, rtol=2e-4, atol=2e-4 * np.abs(want).max(), err_msg=str(cuts))


@pytest.mark.parametrize("dev", DEV)
def test_delta_rule_overwrites_a_key(dev):
    """With full write strength and no decay, writing key k twice leaves only the second
    value under it: the read-out with q = k returns the second value (times d^-1/2)."""
    dev = dev_of(dev)
    d, V = 16, 8
    rng = np.random.default_rng(3)
    k = rng.normal(size=d)
    v1, v2 = rng.normal(size=V), rng.normal(size=V)
    qkv = np.stack([np.concatenate([k, k, v1]), np.concatenate([k, k, v2])])
    ba = np.array([[40.0, -40.0], [40.0, -40.0]])          # beta = 1; softplus(-40) = 0: keep = 1
    state = torch.zeros(1, 1, d, V, device=dev)
    m, _ = meta_for([(0, 2)], [], None, dev, [0])
    got = ops.gated_delta_scan(f32(qkv, dev), f32(ba, dev), f32([0.0], dev), f32([0.0], dev),
                               state, m, 1, 1, d, V).cpu().numpy()
    np.testing.assert_allclose(got[0], v1 / np.sqrt(d), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(got[1], v2 / np.sqrt(d), rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("dev", DEV)
def test_scans_in_a_batch_with_padding_rows(dev):
    """Two decode rows and a padding row (slot -1) beside a prompt: each sequence's result
    equals its own run, the padding row gives zeros and touches no state."""
    dev = dev_of(dev)
    rng = np.random.default_rng(11)
    H, V, N, G = 2, 8, 6, 1
    xa, xb = rng.normal(size=(20, H * V + 2 * G * N)), rng.normal(size=(5, H * V + 2 * G * N))
    da, db = rng.normal(size=(20, H)), rng.normal(size=(5, H))
    par = [f32(rng.normal(size=H) * 0.5, dev), f32(rng.normal(size=H), dev), f32(rng.normal(size=H), dev)]
    alone = {}
    for key, x, dtv in (("a", xa, da), ("b", xb, db)):
        st = torch.zeros(3, H, N, V, device=dev)
        m, _ = meta_for([(0, len(x))], [], None, dev, [1])
        alone[key] = (ops.ssd_scan(f32(x, dev), f32(dtv, dev), *par, st, m, H, V, N, G).cpu().numpy(),
                      st[1].clone())
    st = torch.full((3, H, N, V), 3.0, device=dev)
    m, _ = meta_for([(0, 19), (0, 4)], [], None, dev, [2, 0])
    ops.ssd_scan(f32(np.concatenate([xa[:19], xb[:4]]), dev), f32(np.concatenate([da[:19], db[:4]]), dev),
                 *par, st, m, H, V, N, G)
    m, _ = meta_for([], [19, 4, 0], None, dev, [2, 0, -1])
    m.decode_ctx_lens[2] = 0
    got = ops.ssd_scan(f32(np.stack([xa[19], xb[4], xa[0]]), dev), f32(np.stack([da[19], db[4], da[0]]), dev),
                       *par, st, m, H, V, N, G).cpu().numpy()
    np.testing.assert_allclose(got[0], alone["a"][0][19], rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(got[1], alone["b"][0][4], rtol=1e-5, atol=1e-5)
    assert np.all(got[2] == 0)
    np.testing.assert_allclose(st[2].cpu().numpy(), alone["a"][1].cpu().numpy(), rtol=1e-5, atol=1e-5)
    assert float(st[1].min()) == 3.0 and float(st[1].max()) == 3.0


@pytest.mark.parametrize("dev", DEV)
def test_scans_with_many_sequences_and_heads(dev):
    """Sixteen prompts of unequal length and 32 heads in one step: the grid size at which the
    GPU kernels keep 16 value columns per wave (smaller steps keep 4)."""
    dev = dev_of(dev)
    rng = np.random.default_rng(13)
    lens = [1, 2, 3, 5, 8, 13, 16, 17, 21, 30, 31, 32, 33, 34, 40, 47]
    T, off = sum(lens), np.concatenate([[0], np.cumsum(lens)])
    m, _ = meta_for([(0, n) for n in lens], [], None, dev, list(range(16)))
    H, V, N, G = 32, 24, 20, 4
    xbc, dt = rng.normal(size=(T, H * V + 2 * G * N)), rng.normal(size=(T, H))
    a_log, dtb, D = rng.normal(size=H) * 0.5, rng.normal(size=H), rng.normal(size=H)
    st = torch.full((16, H, N, V), 2.0, device=dev)
    got = ops.ssd_scan(f32(xbc, dev), f32(dt, dev), f32(a_log, dev), f32(dtb, dev), f32(D, dev), st, m,
                       H, V, N, G).cpu().numpy()
    for i in (0, 1, 7, 12, 15):
        x = xbc[off[i]:off[i + 1]]
        want = ssd_oracle(x[:, :H * V], x[:, H * V:H * V + G * N], x[:, H * V + G * N:],
                          dt[off[i]:off[i + 1]], a_log, dtb, D, H, V, N, G)
        np.testing.assert_allclose(got[off[i]:off[i + 1]], want, rtol=2e-4, atol=2e-4 * np.abs(want).max())
    H, G, d, V = 32, 8, 20, 24
    qkv, ba = rng.normal(size=(T, 2 * G * d + H * V)), rng.normal(size=(T, 2 * H))
    st = torch.full((16, H, d, V), 2.0, device=dev)
    got = ops.gated_delta_scan(f32(qkv, dev), f32(ba, dev), f32(a_log, dev), f32(dtb, dev), st, m,
                               H, G, d, V).cpu().numpy()
    for i in (0, 1, 7, 12, 15):
        x, b = qkv[off[i]:off[i + 1]], ba[off[i]:off[i + 1]]
        want = delta_oracle(x[:, :G * d], x[:, G * d:2 * G * d], x[:, 2 * G * d:], b[:, :H], b[:, H:],
                            a_log, dtb, H, G, d, V)
        np.testing.assert_allclose(got[off[i]:off[i + 1]], want, rtol=2e-4, atol=2e-4 * np.abs(want).max())


# ---------------------------------------------------------------- gated norms
@pytest.mark.parametrize("dev", DEV)
@pytest.mark.parametrize("n,groups", [(96, 3), (128, 1), (2048, 2), (66, 6)])
def test_gated_rms_norm(dev, n, groups):
    dev = dev_of(dev)
    rng = np.random.default_rng(n)
    y, g, w = rng.normal(size=(9, n)) * 2, rng.normal(size=(9, n)), rng.normal(size=n)
    gw = f32(np.concatenate([rng.normal(size=(9, 5)), g], 1), dev)
    for first in (True, False):
        out = torch.zeros(9, n + 6, device=dev)
        ops.gated_rms_norm(f32(y, dev), gw[:, 5:], f32(w, dev), groups, 1e-4, first, out[:, 2:2 + n])
        v = y * oracle.silu(g) if first else y
        v = oracle.unit_rms(v.reshape(9, groups, n // groups), 1e-4).reshape(9, n) * w
        want = v if first else v * oracle.silu(g)
        np.testing.assert_allclose(out[:, 2:2 + n].cpu().numpy(), want, rtol=3e-5, atol=3e-5)
        assert float(out[:, :2].abs().max()) == 0 and float(out[:, 2 + n:].abs().max()) == 0


# ---------------------------------------------------------------- rotary layouts, attention
def cache_for(G, dk, dv, pages, dev, dtype=torch.float32):
    return (torch.zeros(pages, G, PAGE, dk, dtype=dtype, device=dev),
            torch.zeros(pages, G, PAGE, dv, dtype=dtype, device=dev))


def attend(q, k, v, H, G, dk, dv, rot, base, inter, scale, cap, dev, cuts, out_scale=1.0):
    """q [n, H dk], k [n, G dk], v [n, G dv] through rope_kv_store + window_attention over
    pages handed out in a scrambled order; -> [n, H dv]."""
    n = q.shape[0]
    pages = -(-n // PAGE)
    order = np.random.default_rng(5).permutation(pages) + 1
    table = torch.tensor([order.tolist()], dtype=torch.int32, device=dev)
    kc, vc = cache_for(G, dk, dv, pages + 1, dev)
    rope = ops.ref.rope_table(rot, n + 1, base).to(dev) if rot else None
    qkv = f32(np.concatenate([q, k, v], 1), dev)
    got = []
    for lo, hi, dec in steps_of(n, cuts):
        m, pos = meta_for([] if dec else [(lo, hi - lo)], [lo] if dec else [], table, dev)
        slots = torch.tensor([int(order[p // PAGE]) * PAGE + p % PAGE for p in range(lo, hi)],
                             dtype=torch.int64, device=dev)
        qr = ops.rope_kv_store(qkv[lo:hi], pos, rope, kc, vc, slots, H, G, dk, dv, inter)
        out = torch.zeros(hi - lo, H * dv + 3, device=dev)
        ops.window_attention(qr, kc, vc, pos, m, scale, 0, 0, None, cap, out_scale, out=out[:, 3:])
        got.append(out[:, 3:].cpu().numpy())
    return np.concatenate(got)


def attention_oracle(q, k, v, H, G, dk, dv, rot, base, inter, scale, cap):
    n = q.shape[0]
    W = {"q": np.eye(H * dk), "k": np.eye(G * dk), "v": np.eye(G * dv), "o": np.eye(H * dv)}
    m = {"heads": H, "kv_heads": G, "dim": dk, "vdim": dv, "scale": scale,
         "rot": {"dims": rot, "base": base}}
    # the oracle's attention takes the mixer input and its projections: feed q | k | v as
    # the input and pick them out again
    h = np.concatenate([q, k, v], 1)
    Wp = {"a.q": np.eye(H * dk, h.shape[1]), "a.k": np.eye(G * dk, h.shape[1], H * dk),
          "a.v": np.eye(G * dv, h.shape[1], (H + G) * dk), "a.o": np.eye(H * dv)}
    if inter or cap:
        m["softcap"] = cap
        z = np.zeros
        Wp.update({"a.q.b": z(H * dk), "a.k.b": z(G * dk), "a.v.b": z(G * dv), "a.o.b": z(H * dv),
                   "a.g": z((H * dv, h.shape[1]))})
        return 2.0 * oracle.attention(h, Wp, "a.", m, True)        # the zero gate halves
    return oracle.attention(h, Wp, "a.", m, False)


@pytest.mark.parametrize("dev", DEV)
@pytest.mark.parametrize("inter,cap", [(False, 0.0), (True, 0.0), (True, 3.0)])
@pytest.mark.parametrize("H,G,dk,dv,rot", [(4, 2, 12, 10, 8), (2, 2, 16, 8, 16), (3, 1, 10, 6, 2), (8, 2, 64, 32, 32)])
def test_attention_layouts_and_portions(dev, inter, cap, H, G, dk, dv, rot):
    dev = dev_of(dev)
    rng = np.random.default_rng(dk)
    n = 75
    q, k, v = rng.normal(size=(n, H * dk)), rng.normal(size=(n, G * dk)), rng.normal(size=(n, G * dv))
    want = attention_oracle(q, k, v, H, G, dk, dv, rot, 50.0, inter, 0.4, cap)
    for cuts in ([75], [30, 1], [2], [7, 9, 1, 1, 20, 3]):
        got = attend(q, k, v, H, G, dk, dv, rot, 50.0, inter, 0.4, cap, dev, cuts)
        np.testing.assert_allclose(got, want, rtol=3e-4, atol=3e-4, err_msg=str(cuts))
    got = attend(q, k, v, H, G, dk, dv, rot, 50.0, inter, 0.4, cap, dev, [40, 1], out_scale=1.7)
    np.testing.assert_allclose(got, 1.7 * want, rtol=3e-4, atol=3e-4)


@pytest.mark.parametrize("dev", DEV)
@pytest.mark.parametrize("cap", [0.0, 25.0])
@pytest.mark.parametrize("target", [0, 1, 7, 8, 63, 64, 250, 383, 384, 398])
def test_attention_finds_a_planted_key(dev, cap, target):
    """One key among 400 carries a score far above the rest (no rotary, so it is exact);
    the last prompt row and a decoded row must both return its value, whether it is the
    first token, hundreds of tokens back, or at a page's or key tile's border."""
    dev = dev_of(dev)
    rng = np.random.default_rng(target)
    n, H, G, dk, dv = 400, 2, 1, 16, 8
    q, k, v = rng.normal(size=(n, H * dk)) * 0.1, rng.normal(size=(n, G * dk)) * 0.1, rng.normal(size=(n, G * dv))
    mark = rng.normal(size=dk)
    mark *= 6.0 / np.linalg.norm(mark)
    k[target] = mark
    for row in (n - 2, n - 1):
        q[row] = np.concatenate([mark, mark])
    got = attend(q, k, v, H, G, dk, dv, 0, 1.0, False, 1.0, cap, dev, [n - 1, 1])
    if cap == 0.0:            # score 36 against |others| < 3: weights below e^-30
        for row in (n - 2, n - 1):
            np.testing.assert_allclose(got[row].reshape(H, dv), np.stack([v[target]] * H), atol=1e-4)
    else:                      # capped at 25 tanh(36 / 25): still far above the rest
        want = attention_oracle(q, k, v, H, G, dk, dv, 0, 1.0, True, 1.0, cap)
        np.testing.assert_allclose(got[n - 2:], want[n - 2:], rtol=2e-4, atol=2e-4)
        assert np.abs(got[n - 1].reshape(H, dv) - v[target]).max() < 1e-3


# ---------------------------------------------------------------- feed-forwards
@pytest.mark.parametrize("dev", DEV)
def test_relu_squared_feed_forward(dev):
    dev = dev_of(dev)
    rng = np.random.default_rng(2)
    W = {"f.up": rng.normal(size=(40, 24)) / 5, "f.down": rng.normal(size=(24, 40)) / 6}
    mlp = ReluSqMLP(24, 40, torch.float32, dev)
    mlp.up_proj.weight.data.copy_(f32(W["f.up"], dev))
    mlp.down_proj.weight.data.copy_(f32(W["f.down"], dev))
    h = rng.normal(size=(11, 24))
    np.testing.assert_allclose(mlp(f32(h, dev)).cpu().numpy(),
                               oracle.feed_forward(h, W, "f.", {"kind": "dense"}), rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("dev", DEV)
@pytest.mark.parametrize("E,top,ff,width", [(6, 2, 20, 24), (2, 1, 16, 16), (5, 5, 8, 30), (8, 3, 64, 128)])
def test_softmax_routed_experts(dev, E, top, ff, width):
    """Chosen experts, softmax over the chosen logits only, the router bias; a bias that
    lifts one expert above all others makes every token use it."""
    dev = dev_of(dev)
    rng = np.random.default_rng(E)
    f = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": E, "top": top}}
    W = {"f.router": rng.normal(size=(E, width)), "f.router.b": rng.normal(size=E)}
    for e in range(E):
        W["f.e%d.gate" % e] = rng.normal(size=(ff, width)) / 4
        W["f.e%d.up" % e] = rng.normal(size=(ff, width)) / 4
        W["f.e%d.down" % e] = rng.normal(size=(width, ff)) / 4
    spec = FeedForwardSpec("moe", ff, act="silu", gated=True, experts=E, top=top, router="softmax")
    mod = SoftmaxRoutedExperts(width, spec, torch.float32, dev)
    mod.router.data.copy_(f32(W["f.router"], dev))
    for e in range(E):
        mod.w13.data[e, :ff].copy_(f32(W["f.e%d.gate" % e], dev))
        mod.w13.data[e, ff:].copy_(f32(W["f.e%d.up" % e], dev))
        mod.w2.data[e].copy_(f32(W["f.e%d.down" % e], dev))
    h = rng.normal(size=(13, width))
    for lift in (None, E - 1):
        b = W["f.router.b"].copy()
        if lift is not None:
            b[lift] += 100.0
        mod.router_bias.data.copy_(f32(b, dev))
        margins = []
        want = oracle.feed_forward(h, dict(W, **{"f.router.b": b}), "f.", f, margins)
        got = mod(f32(h, dev)).cpu().numpy()
        firm = margins[0] > 1e-3
        np.testing.assert_allclose(got[firm], want[firm], rtol=2e-4, atol=2e-4)
        if lift is not None and top == 1:
            pe = "f.e%d." % lift
            only = (oracle.silu(h @ W[pe + "gate"].T) * (h @ W[pe + "up"].T)) @ W[pe + "down"].T
            np.testing.assert_allclose(got, only, rtol=2e-4, atol=2e-4)


# ---------------------------------------------------------------- the whole mixer
def mixer_weights(layer, width, rng):
    m, W = layer["mixer"], {}
    a, r = m["left"], m["right"]
    two = layer["type"] == "parallel_2"

    def lin(name, out, inp, gain=1.0):
        W[name] = (rng.normal(size=(out, inp)) * gain / np.sqrt(inp)).astype(np.float32).astype(np.float64)

    def vec(name, n, base, spread):
        W[name] = (base + spread * rng.normal(size=n)).astype(np.float32).astype(np.float64)
    H, G, d, dv = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
    lin("left.q", H * d, width, 2.0), lin("left.k", G * d, width, 2.0), lin("left.v", G * dv, width)
    lin("left.o", width, H * dv)
    if two:
        lin("left.g", H * dv, width, 2.0)
        for nme, sz in (("q.b", H * d), ("k.b", G * d), ("v.b", G * dv), ("o.b", width)):
            vec("left." + nme, sz, 0.0, 0.3)
        H, G, d, dv, K = r["heads"], r["kv_heads"], r["dim"], r["vdim"], r["conv"]
        for nme, sz in (("q", G * d), ("k", G * d), ("v", H * dv)):
            lin("right." + nme, sz, width, 2.0)
            W["right." + nme + ".conv"] = rng.normal(size=(sz, K)) * 0.6
        lin("right.g", H * dv, width, 2.0), lin("right.b", H, width, 2.0), lin("right.a", H, width, 2.0)
        vec("right.A_log", H, -0.5, 0.7), vec("right.dt_bias", H, -1.0, 0.7), vec("right.norm", dv, 1.0, 0.2)
        lin("right.o", width, H * dv)
    else:
        H, V, N, G, K = r["heads"], r["vdim"], r["state"], r["groups"], r["conv"]
        lin("right.in", 2 * H * V + 2 * G * N + H, width, 2.0)
        W["right.conv"] = rng.normal(size=(H * V + 2 * G * N, K)) * 0.6
        vec("right.conv.b", H * V + 2 * G * N, 0.0, 0.3)
        vec("right.A_log", H, -0.5, 0.7), vec("right.dt_bias", H, -1.0, 0.7), vec("right.D", H, 0.5, 0.5)
        vec("right.norm", H * V, 1.0, 0.2)
        lin("right.o", width, H * V)
    return W


LAYERS = [
    {"type": "parallel", "mlp": None, "mixer": {
        "left": {"heads": 4, "kv_heads": 2, "dim": 12, "vdim": 10, "scale": 0.3, "rot": {"dims": 8, "base": 100.0}},
        "right": {"heads": 4, "vdim": 8, "state": 12, "groups": 2, "conv": 3, "norm_groups": 2},
        "left_scale": 1.3, "right_scale": 0.8}},
    {"type": "parallel_2", "mlp": None, "mixer": {
        "left": {"heads": 3, "kv_heads": 1, "dim": 8, "vdim": 6, "scale": 0.4, "softcap": 5.0,
                 "rot": {"dims": 6, "base": 40.0}},
        "right": {"heads": 4, "kv_heads": 2, "dim": 10, "vdim": 6, "conv": 4},
        "left_scale": 0.6, "right_scale": 1.4}},
]


@pytest.mark.parametrize("dev", DEV)
@pytest.mark.parametrize("layer", LAYERS, ids=["mamba2", "gated_delta"])
@pytest.mark.parametrize("cuts", [[50], [20, 1], [2], [5, 3, 1, 1, 17, 2]])
def test_parallel_mixer(dev, layer, cuts):
    """The module the model uses, loaded through the model's own weight mapping."""
    from kubernetes_gpu_cluster_amd.models.nolesun import NolesunForCausalLM
    dev = dev_of(dev)
    width, n, eps = 40, 50, 1e-5
    rng = np.random.default_rng(9)
    W = mixer_weights(layer, width, rng)
    spec = _nolesun_spec(layer)
    mix = ParallelMixer(width, spec, eps, torch.float32, dev)
    host = types.SimpleNamespace(dtype=torch.float32)
    for name, w in W.items():
        side, leaf = name.split(".", 1)
        fn = NolesunForCausalLM._load_left if side == "left" else NolesunForCausalLM._load_right
        args = (host, mix, spec, leaf, torch.tensor(w)) if side == "left" else \
            (host, 0, mix, spec, leaf, torch.tensor(w))
        assert fn(*args), name
    h = rng.normal(size=(n, width))
    want = oracle.mixer(h, {"m." + k: v for k, v in W.items()}, "m.", layer, eps)
    pages = -(-n // PAGE)
    order = np.random.default_rng(6).permutation(pages) + 1
    table = torch.tensor([order.tolist()], dtype=torch.int32, device=dev)
    G, dk, dv = mix.cache_shape()
    caches = [cache_for(G, dk, dv, pages + 1, dev)]
    state = tuple(torch.full((2,) + s, 4.0, device=dev) for s in mix.state_shapes())
    mix.left.prepare({}, n + 1, dev)
    got = []
    for lo, hi, dec in steps_of(n, cuts):
        m, pos = meta_for([] if dec else [(lo, hi - lo)], [lo] if dec else [], table, dev, [1])
        m.slot_mapping = torch.tensor([int(order[p // PAGE]) * PAGE + p % PAGE for p in range(lo, hi)],
                                      dtype=torch.int64, device=dev)
        ctx = ForwardContext(m, caches, states=[state])
        got.append(mix(f32(h[lo:hi], dev), pos, ctx, 0, state).cpu().numpy())
    np.testing.assert_allclose(np.concatenate(got), want, rtol=3e-4, atol=3e-4 * np.abs(want).max())
