"""Each mechanism of the Lorenex decoder alone (the product's op or module) against the
numpy oracle's function for it, on the CPU reference ops and, with ``-m gpu``, on the HIP
kernels: the scaled embedding with learned positions, gated linear attention and the
selective scan over portions of every size with state carried in slots, unit-RMS attention
inputs with the query factor and a planted stand-out key (far back, at page borders, the
first token, on both sides of a step of the query factor), the convolution in the
activation dtype, PolyNorm, the clamped gated activation, routing with a lifted correction
and identity experts, and the routed-experts module on both of its GEMM paths."""
import types

import numpy as np
import pytest
import torch

import lorenex_oracle as oracle
from kubernetes_gpu_cluster_amd import ops
from kubernetes_gpu_cluster_amd.models.configs import FeedForwardSpec
from kubernetes_gpu_cluster_amd.models.moe import SoftmaxAllRoutedExperts

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


def over_steps(n, cuts, dev, fn, slot=2):
    got = []
    for lo, hi, dec in steps_of(n, cuts):
        m, _ = meta_for([] if dec else [(lo, hi - lo)], [lo] if dec else [], None, dev, [slot])
        got.append(fn(lo, hi, m).float().cpu().numpy())
    return np.concatenate(got)


CUTS = [[200], [1], [2], [3, 1, 2, 70, 1, 1, 40, 2], [64, 65, 1], [17, 16, 15, 1]]


# ---------------------------------------------------------------- embedding
@pytest.mark.parametrize("dev", DEV)
def test_embedding_scale_and_positions(dev):
    dev = dev_of(dev)
    rng = np.random.default_rng(0)
    table, pos = rng.normal(size=(50, 37)), rng.normal(size=(20, 37))
    ids, p = rng.integers(0, 50, 13), rng.integers(0, 20, 13)
    out = torch.zeros(13, 37, device=dev)
    ops.embed_pos(torch.tensor(ids, device=dev), torch.tensor(p, device=dev), f32(table, dev), 3.5,
                  f32(pos, dev), out)
    np.testing.assert_allclose(out.cpu().numpy(), table[ids] * 3.5 + pos[p], rtol=1e-6, atol=1e-6)
    ops.embed_pos(torch.tensor(ids, device=dev), torch.tensor(p, device=dev), f32(table, dev), 1.0,
                  None, out)
    np.testing.assert_allclose(out.cpu().numpy(), table[ids], rtol=1e-6, atol=1e-6)


# ---------------------------------------------------------------- gated linear attention
def gla_inputs(rng, n, H, d, V, R, off=3):
    proj = rng.normal(size=(n, off + 2 * H * d + H * V + 5 + R))
    a2, b = rng.normal(size=(H * d, R)), rng.normal(size=H * d) + 2.0
    return proj, a2, b


def gla_want(proj, a2, b, H, d, V, R, tau, off=3):
    n = proj.shape[0]
    body = proj[:, off:]
    q = body[:, : H * d].reshape(n, H, d) * d ** -0.5
    k = body[:, H * d: 2 * H * d].reshape(n, H, d)
    v = body[:, 2 * H * d: 2 * H * d + H * V].reshape(n, H, V)
    z = proj[:, -R:] @ a2.T + b
    alpha = (oracle.sigmoid(z) ** (1.0 / tau)).reshape(n, H, d)
    return oracle.gla_scan(q, k, v, alpha).reshape(n, H * V)


@pytest.mark.parametrize("dev", DEV)
@pytest.mark.parametrize("H,d,V,R,tau", [(2, 12, 10, 5, 4.0), (1, 16, 16, 1, 1.0), (3, 40, 7, 16, 16.0),
                                         (2, 64, 80, 8, 8.0), (1, 130, 20, 4, 2.0)])
def test_gla_scan_over_steps(dev, H, d, V, R, tau):
    dev = dev_of(dev)
    rng = np.random.default_rng(H * d)
    n = 150
    proj, a2, b = gla_inputs(rng, n, H, d, V, R)
    want = gla_want(proj, a2, b, H, d, V, R, tau)
    pt = f32(proj, dev)
    for cuts in CUTS:
        state = torch.full((4, H, d, V), 7.0, device=dev)       # another request's leftovers
        got = over_steps(n, cuts, dev, lambda lo, hi, m: ops.gla_scan(
            pt[lo:hi, 3:], pt[lo:hi, proj.shape[1] - R:], f32(a2, dev), f32(b, dev), state, m, H, d,
            V, tau))
        np.testing.assert_allclose(got, want, rtol=3e-4, atol=3e-4, err_msg=str(cuts))
        assert float(state[1].min()) == 7.0 and float(state[3].max()) == 7.0


@pytest.mark.parametrize("dev", DEV)
def test_gla_decay_keeps_and_forgets_per_channel(dev):
    """Key channel 0 never decays (alpha = 1) and channel 1 forgets at once (alpha = 0): a
    query on channel 0 still returns the first token's value 300 tokens later, a query on
    channel 1 only the current token's."""
    dev = dev_of(dev)
    n, H, d, V, R = 300, 1, 4, 6, 2
    rng = np.random.default_rng(3)
    v = rng.normal(size=(n, V))
    k = np.zeros((n, d))
    k[0, 0] = 2.0                       # only the first token writes channel 0
    k[:, 1] = 1.0                       # every token writes channel 1
    q = np.zeros((n, d))
    q[:, 0], q[-1, 0], q[-1, 1] = 1.0, 0.0, 1.0
    low = np.zeros((n, R))
    low[:, 0] = 1.0
    a2 = np.zeros((d, R))
    a2[0, 0], a2[1, 0] = 60.0, -60.0    # sigmoid(+-60)
    proj = f32(np.concatenate([q, k, v, low], 1), dev)
    for cuts in ([n], [n - 40, 1], [7, 2]):
        state = torch.zeros(3, H, d, V, device=dev)
        got = over_steps(n, cuts, dev, lambda lo, hi, m: ops.gla_scan(
            proj[lo:hi], proj[lo:hi, 2 * d + V:], f32(a2, dev), torch.zeros(d, device=dev), state, m,
            H, d, V, 1.0))
        np.testing.assert_allclose(got[n - 2], v[0] * 2.0 * d ** -0.5, rtol=1e-5, atol=1e-5)
        np.testing.assert_allclose(got[n - 1], v[n - 1] * d ** -0.5, rtol=1e-5, atol=1e-5)


# ---------------------------------------------------------------- selective scan
def sel_inputs(rng, n, I, N):
    x, dt = rng.normal(size=(n, I)), rng.normal(size=(n, I))
    bc, z = rng.normal(size=(n, 3 + 2 * N)), rng.normal(size=(n, I + 2))
    A = -np.exp(rng.normal(size=(I, N)))
    return x, dt, bc, z, A, rng.normal(size=I) - 1.0, rng.normal(size=I)


def sel_want(x, dt, bc, z, A, dtb, D, N, scale):
    y = oracle.selective_scan(x, oracle.softplus(dt + dtb), A, bc[:, 3:3 + N], bc[:, 3 + N:], D)
    return y * oracle.silu(z[:, 2:]) * scale


@pytest.mark.parametrize("dev", DEV)
@pytest.mark.parametrize("I,N", [(37, 5), (64, 16), (96, 32), (20, 1), (130, 70)])
def test_selective_scan_over_steps(dev, I, N):
    dev = dev_of(dev)
    rng = np.random.default_rng(I + N)
    n = 150
    x, dt, bc, z, A, dtb, D = sel_inputs(rng, n, I, N)
    want = sel_want(x, dt, bc, z, A, dtb, D, N, 0.8)
    t = {k: f32(a, dev) for k, a in dict(x=x, dt=dt, bc=bc, z=z, At=A.T.copy(), dtb=dtb, D=D).items()}
    for cuts in CUTS:
        state = torch.full((4, N, I), 7.0, device=dev)
        out = torch.zeros(n, I + 4, device=dev)

        def fn(lo, hi, m):
            ops.selective_scan(t["x"][lo:hi], t["dt"][lo:hi], t["bc"][lo:hi, 3:], t["At"], t["dtb"],
                               t["D"], t["z"][lo:hi, 2:], state, m, 0.8, out[lo:hi, 1:1 + I])
            return out[lo:hi, 1:1 + I]
        got = over_steps(n, cuts, dev, fn)
        np.testing.assert_allclose(got, want, rtol=3e-4, atol=3e-4, err_msg=str(cuts))
        assert float(out[:, 0].abs().max()) == 0 and float(out[:, 1 + I:].abs().max()) == 0
        assert float(state[1].min()) == 7.0


@pytest.mark.parametrize("dev", DEV)
def test_selective_scan_keeps_and_forgets_per_channel(dev):
    """Channel 0 has A ~ 0 (its state never decays) and channel 1 a large |A| (it forgets at
    once): 300 tokens after the only input, channel 0 still returns it, channel 1 returns only
    the current token's -- in one prompt, in decode rows and in two-token portions."""
    dev = dev_of(dev)
    n, I, N = 300, 2, 1
    x = np.zeros((n, I))
    x[0] = [1.0, 1.0]
    x[-1] = [0.0, 2.0]
    dt = np.ones((n, I))
    step = oracle.softplus(1.0)
    bc = np.ones((n, 2 * N))
    z = np.full((n, I), 30.0)                     # silu(30) = 30
    At = f32(np.array([[-1e-9, -50.0]]), dev)
    zero = torch.zeros(I, device=dev)
    t = {k: f32(a, dev) for k, a in dict(x=x, dt=dt, bc=bc, z=z).items()}
    for cuts in ([n], [n - 40, 1], [7, 2]):
        state = torch.full((3, N, I), 5.0, device=dev)
        out = torch.zeros(n, I, device=dev)

        def fn(lo, hi, m):
            ops.selective_scan(t["x"][lo:hi], t["dt"][lo:hi], t["bc"][lo:hi], At, zero, zero,
                               t["z"][lo:hi], state, m, 1.0, out[lo:hi])
            return out[lo:hi]
        got = over_steps(n, cuts, dev, fn)
        np.testing.assert_allclose(got[n - 2], [30.0 * step, 0.0], rtol=1e-5, atol=1e-5)
        np.testing.assert_allclose(got[n - 1], [30.0 * step, 60.0 * step], rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("dev", DEV)
def test_scans_in_a_batch_with_padding_rows(dev):
    """Two prompts' portions and three decode rows (one a padding row of slot -1) in one
    step, against each sequence alone; slots handed out in no particular order."""
    dev = dev_of(dev)
    rng = np.random.default_rng(11)
    H, d, V, R, I, N = 2, 12, 10, 3, 24, 6
    lens = {0: 40, 1: 9, 2: 13, 3: 5}
    slot = {0: 3, 1: 0, 2: 4, 3: 1}
    g = {s: gla_inputs(rng, n, H, d, V, R, off=0) for s, n in lens.items()}
    a2, b = g[0][1], g[0][2]
    gw = {s: gla_want(g[s][0], a2, b, H, d, V, R, 4.0, off=0) for s in lens}
    se = {s: sel_inputs(rng, n, I, N) for s, n in lens.items()}
    A, dtb, D = se[0][4], se[0][5], se[0][6]
    sw = {s: sel_want(*se[s][:4], A, dtb, D, N, 1.0) for s in lens}
    gs = torch.zeros(5, H, d, V, device=dev)
    ss = torch.zeros(5, N, I, device=dev)

    def run(rows, m):
        cat = lambda i: f32(np.concatenate([r[i] for r in rows]), dev)     # noqa: E731
        proj = cat(0)
        o1 = ops.gla_scan(proj, proj[:, proj.shape[1] - R:], f32(a2, dev), f32(b, dev), gs, m, H, d,
                          V, 4.0).cpu().numpy()
        out = torch.zeros(proj.shape[0], I, device=dev)
        ops.selective_scan(cat(1), cat(2), cat(3)[:, 3:], f32(A.T.copy(), dev), f32(dtb, dev),
                           f32(D, dev), cat(4)[:, 2:], ss, m, 1.0, out)
        return o1, out.cpu().numpy()

    def part(s, lo, hi):
        return (g[s][0][lo:hi],) + tuple(a[lo:hi] for a in se[s][:4])
    # step 1: prompts 0 and 1 in part, 2 and 3 up to their last token
    m, _ = meta_for([(0, 33), (0, 2), (0, 12), (0, 4)], [], None, dev, [slot[s] for s in range(4)])
    o1, o2 = run([part(0, 0, 33), part(1, 0, 2), part(2, 0, 12), part(3, 0, 4)], m)
    o = 0
    for s, n in zip(range(4), (33, 2, 12, 4)):
        np.testing.assert_allclose(o1[o:o + n], gw[s][:n], rtol=3e-4, atol=3e-4)
        np.testing.assert_allclose(o2[o:o + n], sw[s][:n], rtol=3e-4, atol=3e-4)
        o += n
    # step 2: the rest of 0 and 1 as portions; 2, a padding row and 3 as decode rows
    m, _ = meta_for([(33, 7), (2, 7)], [12, 0, 4], None, dev, [slot[0], slot[1], slot[2], -1, slot[3]])
    o1, o2 = run([part(0, 33, 40), part(1, 2, 9), part(2, 12, 13), part(3, 0, 1), part(3, 4, 5)], m)
    for s, lo, n, o in ((0, 33, 7, 0), (1, 2, 7, 7), (2, 12, 1, 14), (3, 4, 1, 16)):
        np.testing.assert_allclose(o1[o:o + n], gw[s][lo:lo + n], rtol=3e-4, atol=3e-4)
        np.testing.assert_allclose(o2[o:o + n], sw[s][lo:lo + n], rtol=3e-4, atol=3e-4)
    assert float(np.abs(o1[15]).max()) == 0 and float(np.abs(o2[15]).max()) == 0
    assert float(gs[2].abs().max()) == 0 and float(ss[2].abs().max()) == 0


@pytest.mark.parametrize("dev", DEV)
def test_convolution_in_the_activation_dtype(dev):
    """The convolution may write the activation dtype (the scan's and a GEMM's input) and
    may leave the activation out; its state stays fp32."""
    dev = dev_of(dev)
    rng = np.random.default_rng(5)
    n, C, K = 90, 40, 3
    x, w, b = rng.normal(size=(n, C)), rng.normal(size=(C, K)), rng.normal(size=C)
    for silu, bias in ((True, b), (False, None)):
        y = oracle.causal_conv(x, w, bias)
        want = oracle.silu(y) if silu else y
        for dt, tol in ((torch.float32, 2e-5), (torch.bfloat16, 2e-2)):
            xs = f32(x, dev).to(dt)
            ref = oracle.causal_conv(xs.float().cpu().numpy().astype(np.float64), w, bias)
            ref = oracle.silu(ref) if silu else ref
            state = torch.full((4, K - 1, C), 9.0, device=dev)
            got = over_steps(n, [31, 2, 1], dev, lambda lo, hi, m: ops.causal_conv(
                xs[lo:hi], f32(w, dev), f32(bias, dev) if bias is not None else None, state, m,
                silu, dt))
            np.testing.assert_allclose(got, ref if dt != torch.float32 else want, rtol=tol, atol=tol)


# ---------------------------------------------------------------- unit-RMS attention inputs
def attend(q, k, v, H, G, dk, dv, scale, qt, dev, cuts, eps=1e-5, out_scale=1.0, unit=(True, True)):
    """q [n, H dk], k [n, G dk], v [n, G dv] through norm_kv_store + window_attention over
    pages handed out in a scrambled order; -> [n, H dv]."""
    n = q.shape[0]
    pages = -(-n // PAGE)
    order = np.random.default_rng(5).permutation(pages) + 1
    table = torch.tensor([order.tolist()], dtype=torch.int32, device=dev)
    kc = torch.zeros(pages + 1, G, PAGE, dk, device=dev)
    vc = torch.zeros(pages + 1, G, PAGE, dv, device=dev)
    qkv = f32(np.concatenate([q, k, v], 1), dev)
    got = []
    for lo, hi, dec in steps_of(n, cuts):
        m, pos = meta_for([] if dec else [(lo, hi - lo)], [lo] if dec else [], table, dev)
        slots = torch.tensor([int(order[p // PAGE]) * PAGE + p % PAGE for p in range(lo, hi)],
                             dtype=torch.int64, device=dev)
        qr = ops.norm_kv_store(qkv[lo:hi], pos, kc, vc, slots, H, G, dk, dv, eps, unit[0], unit[1],
                               qt, torch.float32)
        out = torch.zeros(hi - lo, H * dv + 3, device=dev)
        ops.window_attention(qr, kc, vc, pos, m, scale, 0, 0, None, 0.0, out_scale, out=out[:, 3:])
        got.append(out[:, 3:].cpu().numpy())
    return np.concatenate(got)


def attention_want(q, k, v, H, G, dk, dv, scale, qt, eps=1e-5):
    n = q.shape[0]
    temp = oracle.query_temperature(n, {"coef": qt[0], "every": qt[1]} if qt else None)
    qq = oracle.rms(q.reshape(n, H, dk), eps) * temp[:, None, None]
    return oracle.softmax_attention(qq, oracle.rms(k.reshape(n, G, dk), eps),
                                    oracle.rms(v.reshape(n, G, dv), eps), scale).reshape(n, H * dv)


@pytest.mark.parametrize("dev", DEV)
@pytest.mark.parametrize("H,G,dk,dv,qt", [(4, 2, 12, 10, (0.5, 16)), (2, 2, 16, 8, (1.5, 1)),
                                          (3, 1, 10, 6, None), (8, 2, 64, 32, (0.3, 7)),
                                          (4, 2, 48, 40, (0.5, 16)),
                                          (2, 1, 70, 130, (0.5, 1000))])
def test_unit_norm_attention_and_portions(dev, H, G, dk, dv, qt):
    dev = dev_of(dev)
    rng = np.random.default_rng(dk)
    n = 75
    q, k, v = rng.normal(size=(n, H * dk)) * 3, rng.normal(size=(n, G * dk)) * 0.2, rng.normal(size=(n, G * dv))
    want = attention_want(q, k, v, H, G, dk, dv, 0.4, qt)
    for cuts in ([75], [30, 1], [2], [7, 9, 1, 1, 20, 3]):
        got = attend(q, k, v, H, G, dk, dv, 0.4, qt, dev, cuts)
        np.testing.assert_allclose(got, want, rtol=3e-4, atol=3e-4, err_msg=str(cuts))
    got = attend(q, k, v, H, G, dk, dv, 0.4, qt, dev, [40, 1], out_scale=1.7)
    np.testing.assert_allclose(got, 1.7 * want, rtol=3e-4, atol=3e-4)
    # norms switched off: the vectors pass as they are
    got = attend(q, k, v, H, G, dk, dv, 0.05, None, dev, [40, 1], unit=(False, False))
    plain = oracle.softmax_attention(q.reshape(n, H, dk), k.reshape(n, G, dk), v.reshape(n, G, dv), 0.05)
    np.testing.assert_allclose(got, plain.reshape(n, H * dv), rtol=3e-4, atol=3e-4)


@pytest.mark.parametrize("dev", DEV)
@pytest.mark.parametrize("target", [0, 1, 7, 8, 63, 64, 250, 383, 384, 398])
def test_attention_finds_a_planted_key(dev, target):
    """One key among 400 points along the last queries, every other key across them: with
    unit-RMS vectors its score is scale * dk against ~0, so the last prompt row and a decoded
    row must both return its (unit-RMS) value, whether it is the first token, hundreds of
    tokens back, or at a page's or key tile's border."""
    dev = dev_of(dev)
    rng = np.random.default_rng(target)
    n, H, G, dk, dv = 400, 2, 1, 16, 8
    mark = rng.normal(size=dk)
    k = rng.normal(size=(n, dk))
    k -= np.outer(k @ mark, mark) / (mark @ mark)          # across the mark
    k[target] = mark * 0.3
    q = rng.normal(size=(n, H * dk))
    for row in (n - 2, n - 1):
        q[row] = np.concatenate([mark, mark]) * 5.0
    v = rng.normal(size=(n, G * dv))
    got = attend(q, k, v, H, G, dk, dv, 2.5, (0.5, 64), dev, [n - 1, 1])
    vt = oracle.rms(v[target], 1e-5)                         # score 2.5 * 16 * 3.4 against 0
    for row in (n - 2, n - 1):
        np.testing.assert_allclose(got[row].reshape(H, dv), np.stack([vt] * H), atol=1e-4)


@pytest.mark.parametrize("dev", DEV)
def test_query_factor_steps_at_multiples_of_every(dev):
    """The factor is 1 + coef ln(floor((p + 1) / every) + 1): constant within a block of
    `every` positions that starts at p = every - 1, and a step up at that position, in a
    prompt row and in a decoded row alike."""
    dev = dev_of(dev)
    H, G, dk, dv, every, coef = 1, 1, 8, 4, 16, 0.75
    n = 3 * every + 2
    rng = np.random.default_rng(1)
    qkv = f32(rng.normal(size=(n, 2 * dk + dv)), dev)
    kc = torch.zeros(n // PAGE + 2, G, PAGE, dk, device=dev)
    vc = torch.zeros(n // PAGE + 2, G, PAGE, dv, device=dev)
    none = torch.full((n,), -1, dtype=torch.int64, device=dev)
    pos = torch.arange(n, device=dev)
    base = ops.norm_kv_store(qkv, pos, kc, vc, none, H, G, dk, dv, 1e-5, True, True, None, torch.float32)
    got = ops.norm_kv_store(qkv, pos, kc, vc, none, H, G, dk, dv, 1e-5, True, True, (coef, every),
                            torch.float32)
    ratio = (got / base).cpu().numpy()[:, 0, :].mean(-1)
    want = 1.0 + coef * np.log(np.floor((np.arange(n) + 1) / every) + 1.0)
    np.testing.assert_allclose(ratio, want, rtol=1e-5)
    assert ratio[every - 2] == pytest.approx(1.0) and ratio[every - 1] > 1.5
    assert float(kc.abs().max()) == 0            # slot -1: nothing stored
    one = ops.norm_kv_store(qkv[every - 1:every], pos[every - 1:every], kc, vc, none[:1], H, G, dk, dv,
                            1e-5, True, True, (coef, every), torch.float32)
    np.testing.assert_allclose(one.cpu().numpy(), got[every - 1:every].cpu().numpy(), rtol=1e-6)


# ---------------------------------------------------------------- feed-forwards
@pytest.mark.parametrize("dev", DEV)
@pytest.mark.parametrize("F", [40, 37, 1024, 3000])
def test_polynorm(dev, F):
    dev = dev_of(dev)
    rng = np.random.default_rng(F)
    z = rng.normal(size=(9, F)) * 1.5
    coef = np.array([0.9, -0.4, 0.25, 0.1])
    want = (coef[0] * oracle.rms(z, 1e-5) + coef[1] * oracle.rms(z ** 2, 1e-5)
            + coef[2] * oracle.rms(z ** 3, 1e-5) + coef[3])
    got = ops.polynorm(f32(z, dev), f32(coef, dev), 1e-5)
    np.testing.assert_allclose(got.cpu().numpy(), want, rtol=2e-5, atol=2e-5)
    zb = f32(z, dev).bfloat16()
    zr = zb.float().cpu().numpy().astype(np.float64)
    want = (coef[0] * oracle.rms(zr, 1e-5) + coef[1] * oracle.rms(zr ** 2, 1e-5)
            + coef[2] * oracle.rms(zr ** 3, 1e-5) + coef[3])
    got = ops.polynorm(zb, f32(coef, dev), 1e-5)
    np.testing.assert_allclose(got.float().cpu().numpy(), want, rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("dev", DEV)
@pytest.mark.parametrize("I", [24, 19, 512])
def test_clamped_gated_activation(dev, I):
    dev = dev_of(dev)
    rng = np.random.default_rng(I)
    x = rng.normal(size=(7, 2 * I)) * 3.0
    g, u = np.minimum(x[:, :I], 2.0), np.clip(x[:, I:], -2.0, 2.0)
    want = g * oracle.sigmoid(1.702 * g) * (u + 1.0)
    np.testing.assert_allclose(ops.swiglu_clamp(f32(x, dev), 2.0).cpu().numpy(), want, rtol=2e-5, atol=2e-5)
    got = ops.swiglu_clamp(f32(x, dev).bfloat16(), 2.0).float().cpu().numpy()
    xr = f32(x, dev).bfloat16().float().cpu().numpy().astype(np.float64)
    g, u = np.minimum(xr[:, :I], 2.0), np.clip(xr[:, I:], -2.0, 2.0)
    np.testing.assert_allclose(got, g * oracle.sigmoid(1.702 * g) * (u + 1.0), rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("dev", DEV)
@pytest.mark.parametrize("E,ident,top", [(6, 2, 3), (4, 0, 1), (70, 3, 5), (2, 1, 3)])
def test_routing_scores_correction_and_identity(dev, E, ident, top):
    """The choice is made on softmax score + correction, the weights are the scores as they
    are: an output lifted by its correction is chosen with its small score; identity outputs
    get weight 0 in the pairs and their scores are summed per token."""
    dev = dev_of(dev)
    rng = np.random.default_rng(E)
    n, En = 40, E + ident
    logits = rng.normal(size=(n, En)) * 2.0
    corr = rng.normal(size=En) * 0.05
    corr[1] = 5.0                                           # always chosen
    W = {"r.router": np.eye(En), "r.correction": corr}
    w, ids = oracle.route(logits, W, "r.", top)
    gw, gi, gs = ops.moe_route_softmax_all(f32(logits, dev), f32(corr, dev), top, E)
    gw, gi, gs = gw.cpu().numpy(), gi.cpu().numpy(), gs.cpu().numpy()
    assert (gi[:, 0] == 1).all()
    np.testing.assert_array_equal(gi, ids)
    np.testing.assert_allclose(gw, np.where(ids >= E, 0.0, w), rtol=2e-5, atol=1e-7)
    np.testing.assert_allclose(gs, (w * (ids >= E)).sum(-1), rtol=2e-5, atol=1e-7)
    s = np.exp(logits - logits.max(-1, keepdims=True))
    np.testing.assert_allclose(w[:, 0], (s / s.sum(-1, keepdims=True))[:, 1], rtol=1e-6)   # not renormalised


@pytest.mark.parametrize("dev", DEV)
@pytest.mark.parametrize("E,ident,top,ff,width,dtype", [
    (5, 2, 3, 20, 24, torch.float32), (3, 0, 2, 16, 40, torch.float32),
    (8, 2, 3, 64, 128, torch.bfloat16), (4, 1, 4, 64, 128, torch.bfloat16)])
def test_routed_experts_module(dev, E, ident, top, ff, width, dtype):
    """The module against the oracle: gathered batched GEMMs (fp32, small sizes) and the
    grouped GEMM (bf16 on the GPU, sizes its tiles cover), with identity experts."""
    dev = dev_of(dev)
    rng = np.random.default_rng(E * ff)
    cfgd = {"width": width, "vocab": 8, "max_positions": 4, "layers": [
        {"type": "gla", "mixer": {"heads": 1, "dim": 4, "vdim": 4, "tau": 1.0},
         "mlp": {"kind": "moe", "expert": {"ff": ff, "limit": 1.5},
                 "router": {"experts": E, "identity": ident, "top": top}}}]}
    Wt = oracle.random_weights(cfgd, seed=E)
    spec = FeedForwardSpec("moe", ff, act="swiglu_clamp", gated=True, experts=E, top=top,
                           router="softmax_all", limit=1.5, identity=ident)
    mod = SoftmaxAllRoutedExperts(width, spec, dtype, dev)
    t = lambda a: torch.tensor(a, dtype=dtype, device=dev)      # noqa: E731
    for e in range(E):
        mod.w13.data[e, :ff] = t(Wt[f"l0.mlp.e{e}.gate"])
        mod.w13.data[e, ff:] = t(Wt[f"l0.mlp.e{e}.up"])
        mod.w2.data[e] = t(Wt[f"l0.mlp.e{e}.down"])
    mod.router.data.copy_(t(Wt["l0.mlp.router"]))
    mod.correction.data.copy_(f32(Wt["l0.mlp.correction"], dev))
    h = rng.normal(size=(50, width))
    hr = t(h).float().cpu().numpy().astype(np.float64)
    want = oracle.moe_mlp(hr, Wt, "l0.mlp.", cfgd["layers"][0]["mlp"])
    got = mod(t(h)).float().cpu().numpy()
    if dtype == torch.float32:
        np.testing.assert_allclose(got, want, rtol=3e-4, atol=3e-4)
    else:       # a close routing call may flip in bf16: most rows must agree closely
        err = np.abs(got - want).max(-1) / np.abs(want).max()
        assert np.median(err) < 0.02 and (err < 0.05).mean() > 0.85, err
