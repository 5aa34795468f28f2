"""Lorenex through the engine (registry, safetensors loading, block manager, state slots,
step packing, kernels) against the plain numpy oracle in ``lorenex_oracle.py``.

Every test writes its own small config.json + model.safetensors (random bf16 weights) and
drives the engine with the teacher-forced replayer or the generation entry points.  CPU runs
use the reference ops in fp32; ``-m gpu`` runs use the HIP kernels in fp32 and bf16.  Pages
are 8 tokens, so prompts cross many page borders, and the recurrences carry every earlier
token: a key wrongly hidden, a lost state, a convolution input taken from the wrong step or
a layer run on the wrong weights changes the logits far beyond the tolerances."""
import json
import os

import numpy as np
import pytest
import torch

import lorenex_oracle as oracle
from kubernetes_gpu_cluster_amd.engine.config import EngineConfig
from kubernetes_gpu_cluster_amd.engine.llm_engine import LLM, LLMEngine
from kubernetes_gpu_cluster_amd.engine.replay import TraceReplayer
from kubernetes_gpu_cluster_amd.engine.sequence import SamplingParams
from kubernetes_gpu_cluster_amd.models.configs import PRESETS, resolve_model

CPU = pytest.param("cpu", "float32", id="cpu-fp32")
GPU32 = pytest.param("cuda", "float32", marks=pytest.mark.gpu, id="gpu-fp32")
GPU16 = pytest.param("cuda", "bfloat16", marks=pytest.mark.gpu, id="gpu-bf16")
DEVICES = [CPU, GPU32, GPU16]
# Row error: rms of the logit difference over the rms of the logits, means taken off.
# fp32: every row within 3e-4.  bf16: rounding moves a row by a few percent (the PyTorch
# reference ops in bf16 do the same) -- except where rounding flips a routing choice: a token
# whose choice scores the oracle itself separates by less than MARGIN is a close call, and such
# a row (and, through the recurrent state, the few after it) is only held to 2.0.
TOL = {"float32": 3e-4, "bfloat16": 0.5}
TOL_MEDIAN = {"float32": 3e-4, "bfloat16": 0.08}
MARGIN, AFTER = 0.05, 4


def gla(heads=2, dim=12, vdim=10, tau=4.0, rank=5):
    return {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau, "_rank": rank}


def att(heads=4, kv=2, dim=12, vdim=10, conv=3, scale=0.6, coef=0.5, every=16):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "conv": conv, "scale": scale,
         "q_temp": {"coef": coef, "every": every}}
    if not conv:
        del m["conv"]                    # no convolution on q, k and v at all
    return m


def ssm(inner=24, state=6, dt_rank=3, conv=3):
    return {"inner": inner, "state": state, "dt_rank": dt_rank, "conv": conv}


def glal(m, mlp=None, **kw):
    return dict({"type": "gla", "mixer": m, "mlp": mlp}, **kw)


def par(left, right, mlp=None, ls=1.2, rs=0.9, **kw):
    return dict({"type": "parallel", "mlp": mlp,
                 "mixer": {"left": left, "right": right, "left_scale": ls, "right_scale": rs}}, **kw)


def dense(ff=48):
    return {"kind": "dense", "ff": ff}


def moe(experts=6, top=2, ff=20, identity=1, limit=1.5):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit},
            "router": {"experts": experts, "top": top, "identity": identity}}


def config(layers, width=64, vocab=160, eps=1e-5, scale=3.0, mult=0.5, max_pos=512):
    return {"architecture": "Lorenex", "vocab": vocab, "width": width, "layers": layers,
            "norm": {"eps": eps}, "embedding": {"scale": scale}, "residual_mult": mult,
            "max_positions": max_pos}


MIXED = config([glal(gla(), dense()), par(att(), ssm(), moe()),
                glal(gla(), dense(), weights_of=0), par(att(), ssm(), moe(), weights_of=1),
                par(att(heads=3, kv=1, dim=8, vdim=16, conv=2, scale=0.9, every=5),
                    ssm(inner=20, state=9, dt_rank=1, conv=4), dense(40), ls=0.7, rs=1.3),
                glal(gla(heads=3, dim=8, vdim=16, tau=16.0, rank=2), moe(top=3, identity=2))])
# values a model may make equal or 1, and parts it may leave out: one head, one state, one
# expert used of two, no identity expert, no feed-forward, a convolution of one tap, of two and
# none,
# scales and the residual multiplier 1, a query factor that steps at every position, value
# size = key size, a layer that runs with the weights of one that itself names another, the
# parallel layer first
PLAIN = config([par(att(heads=1, kv=1, dim=16, vdim=16, conv=1, scale=1.0, coef=0.25, every=1),
                    ssm(inner=16, state=1, dt_rank=1, conv=1), dense(32), ls=1.0, rs=1.0),
                glal(gla(heads=1, dim=16, vdim=16, tau=1.0, rank=1), moe(experts=2, top=1, ff=16, identity=0)),
                par(att(heads=1, kv=1, dim=16, vdim=16, conv=1, scale=1.0, coef=0.25, every=1),
                    ssm(inner=16, state=1, dt_rank=1, conv=1), dense(32), ls=1.0, rs=1.0, weights_of=0),
                glal(gla(heads=2, dim=8, vdim=8, tau=2.0, rank=3)),
                par(att(heads=1, kv=1, dim=16, vdim=16, conv=1, scale=1.0, coef=0.25, every=1),
                    ssm(inner=16, state=1, dt_rank=1, conv=1), dense(32), ls=1.0, rs=1.0, weights_of=2),
                par(att(heads=2, kv=2, dim=8, vdim=8, conv=0, scale=0.7, coef=0.0, every=3),
                    ssm(inner=8, state=4, dt_rank=2, conv=2))],
               width=48, vocab=96, scale=1.0, mult=1.0)
# sizes the matrix-core prefill kernel, the 16-byte decode paths and the grouped expert GEMM
# take (attention heads of 64 with values of 32; experts of 64 on a width of 128; linear-
# attention states of 64 x 64; 128 scan channels of 16 states), prompts over several key
# tiles and row blocks
WIDE = config([par(att(heads=8, kv=2, dim=64, vdim=32, conv=4, scale=0.2, every=64),
                   ssm(inner=128, state=16, dt_rank=8, conv=4), moe(experts=8, top=3, ff=64, identity=2)),
               glal(gla(heads=2, dim=64, vdim=64, tau=16.0, rank=16), dense(96)),
               par(att(heads=8, kv=2, dim=64, vdim=32, conv=4, scale=0.2, every=64),
                   ssm(inner=128, state=16, dt_rank=8, conv=4), moe(experts=8, top=3, ff=64, identity=2),
                   weights_of=0)],
              width=128, vocab=200, scale=8.0)
# sizes that are multiples of nothing: odd vocabulary and width, heads whose bytes are no
# multiple of 16, five experts, five taps
ODD = config([glal(gla(heads=3, dim=10, vdim=14, tau=3.0, rank=7), moe(experts=5, top=2, ff=18, identity=3)),
              par(att(heads=6, kv=2, dim=6, vdim=4, conv=5, scale=1.1, coef=0.3, every=7),
                  ssm(inner=22, state=9, dt_rank=5, conv=5), dense(26), ls=0.6, rs=1.1),
              par(att(heads=3, kv=3, dim=10, vdim=14, conv=3, scale=0.5, coef=2.0, every=2),
                  ssm(inner=30, state=3, dt_rank=2, conv=2), moe(experts=3, top=3, ff=10, identity=1))],
             width=70, vocab=251, eps=1e-6, scale=0.5, mult=0.8)


def write_model(path, cfg, seed):
    """Random bf16 weights in the checkpoint's naming; returns them as float64 arrays."""
    from safetensors.torch import save_file
    wts = oracle.random_weights(cfg, seed)
    os.makedirs(path, exist_ok=True)
    clean = json.loads(json.dumps(cfg))
    for L in clean["layers"]:
        L["mixer"].pop("_rank", None)        # only the tensors' shapes give it
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(clean, f)
    save_file({k: torch.tensor(v, dtype=torch.float32).to(torch.bfloat16).contiguous()
               for k, v in wts.items()}, os.path.join(path, "model.safetensors"))
    return wts


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    root = tmp_path_factory.mktemp("lorenex")
    out = {}
    for name, cfg, seed in (("mixed", MIXED, 41), ("plain", PLAIN, 42), ("wide", WIDE, 43),
                            ("odd", ODD, 44)):
        d = str(root / name)
        out[name] = (d, cfg, write_model(d, cfg, seed))
    return out


_engines = {}


@pytest.fixture(scope="module", autouse=True)
def _release_engines():
    """Engines are shared by the tests of this module and released after the last one."""
    yield
    for eng in _engines.values():
        eng.shutdown()
    _engines.clear()
    import gc
    gc.collect()
    if torch.cuda.is_available():
        torch.cuda.empty_cache()


def engine(models, name, device, dtype, pages=24, page=8, seqs=4, **kw):
    if device == "cuda" and not torch.cuda.is_available():
        pytest.skip("no GPU")
    key = (name, device, dtype, pages, page, seqs, tuple(sorted(kw.items())))
    if key not in _engines:
        d = models[name][0]
        _engines[key] = LLMEngine(EngineConfig(
            model=d, dtype=dtype, device=device, block_size=page, max_num_seqs=seqs,
            max_model_len=pages * page, max_num_batched_tokens=pages * page,
            num_gpu_blocks_override=pages + 1, cuda_graph_max_bs=seqs, **kw))
    return _engines[key]


def row_errs(got, want):
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    d = got - want
    d = d - d.mean(-1, keepdims=True)
    w = want - want.mean(-1, keepdims=True)
    return np.sqrt((d ** 2).mean(-1) / (w ** 2).mean(-1))


class Verdict:
    def __init__(self, ok, text):
        self.ok, self.text = ok, text

    def __bool__(self):
        return self.ok

    def __repr__(self):
        return self.text


class Expected:
    def __init__(self, logits, shaky):
        self.logits, self.shaky = logits, shaky

    def __getitem__(self, key):
        return Expected(self.logits[key], self.shaky[key])


_expected = {}


def expected(cfg, wts, toks):
    """The oracle's logits, with the rows marked whose routing was a close call."""
    key = (id(wts), tuple(toks))
    if key not in _expected:
        margins = []
        lg = oracle.forward(cfg, wts, toks, margins=margins)
        shaky = np.zeros(len(toks), dtype=bool)
        if margins:
            for t in np.where(np.min(np.stack(margins), axis=0) < MARGIN)[0]:
                shaky[t:t + 1 + AFTER] = True
        _expected[key] = Expected(lg, shaky)
    return _expected[key]


def close(got, want, dtype):
    e = row_errs(got, want.logits)
    firm = ~want.shaky if dtype != "float32" else np.ones(len(e), dtype=bool)
    text = "rows %d (%d firm): median %.2g, worst firm %.2g, worst %.2g" % (
        len(e), firm.sum(), np.median(e), e[firm].max() if firm.any() else 0.0, e.max())
    ok = e.max() < (TOL[dtype] if dtype == "float32" else 2.0)
    ok = ok and (not firm.any() or e[firm].max() < TOL[dtype])
    if len(e) >= 8:
        ok = ok and np.median(e) < TOL_MEDIAN[dtype]
    return Verdict(bool(ok), text)


def tokens_for(cfg, n, seed):
    return np.random.default_rng(seed).integers(0, cfg["vocab"], n).tolist()


def run_alone(rp, rid, toks, cuts):
    """Feed `toks` in portions of the sizes `cuts` (the last size repeats); all logits."""
    out, lo, i = [], 0, 0
    while lo < len(toks):
        n = cuts[min(i, len(cuts) - 1)]
        i += 1
        hi = min(len(toks), lo + n)
        lg = rp.step([{"id": rid, "tokens": toks[lo:hi], "want": list(range(hi - lo))}],
                     [rid] if hi == len(toks) else [])
        out.append(lg.cpu().numpy())
        lo = hi
    return np.concatenate(out)


# ---------------------------------------------------------------- whole prompts, decode, portions
@pytest.mark.parametrize("device,dtype", DEVICES)
@pytest.mark.parametrize("name", ["mixed", "plain", "wide", "odd"])
def test_whole_prompt_matches_oracle(models, name, device, dtype):
    _, cfg, wts = models[name]
    eng = engine(models, name, device, dtype)
    rp = TraceReplayer(eng)
    toks = tokens_for(cfg, 150 if name == "wide" else 61, 1)
    want = expected(cfg, wts, toks)
    got = run_alone(rp, "w", toks, [len(toks)])
    assert close(got, want, dtype)
    # the first tokens of a sequence, and a one-token prompt
    assert close(got[:3], want[:3], dtype)
    one = run_alone(rp, "o", toks[:1], [1])
    assert close(one, want[:1], dtype)


@pytest.mark.parametrize("device,dtype", DEVICES)
@pytest.mark.parametrize("name", ["mixed", "plain", "wide", "odd"])
def test_prefill_then_token_by_token(models, name, device, dtype):
    _, cfg, wts = models[name]
    eng = engine(models, name, device, dtype)
    rp = TraceReplayer(eng)
    toks = tokens_for(cfg, 130 if name == "wide" else 70, 2)
    want = expected(cfg, wts, toks)
    if name == "wide":                             # portions across 64-row blocks and key tiles
        assert close(run_alone(rp, "c", toks, [70, 3, 45, 2, 1]), want, dtype)
    got = run_alone(rp, "d", toks, [20, 1])
    assert close(got, want, dtype)
    if name != "wide" or device != "cpu":          # decoding from the very first token
        got = run_alone(rp, "e", toks, [1])
        assert close(got, want, dtype)


@pytest.mark.parametrize("device,dtype", DEVICES)
@pytest.mark.parametrize("cuts", [[2], [3, 2, 7, 2, 11, 5, 1], [8], [9, 16, 2, 1], [1, 2, 1, 3]])
def test_portions(models, device, dtype, cuts):
    """Portions down to two tokens (shorter than the convolutions' taps - 1, so a portion's
    convolution state keeps inputs of the portion before it) and cut inside pages."""
    _, cfg, wts = models["mixed"]
    eng = engine(models, "mixed", device, dtype)
    rp = TraceReplayer(eng)
    toks = tokens_for(cfg, 45, 3)
    want = expected(cfg, wts, toks)
    assert close(run_alone(rp, "p", toks, cuts), want, dtype)
    _, cfg, wts = models["odd"]                     # five taps: four inputs of state
    rp = TraceReplayer(engine(models, "odd", device, dtype))
    toks = tokens_for(cfg, 31, 7)
    assert close(run_alone(rp, "q", toks, cuts), expected(cfg, wts, toks), dtype)


@pytest.mark.parametrize("device,dtype", DEVICES)
def test_long_decode(models, device, dtype):
    _, cfg, wts = models["plain"]
    eng = engine(models, "plain", device, dtype, pages=40)
    rp = TraceReplayer(eng)
    toks = tokens_for(cfg, 150, 4)
    want = expected(cfg, wts, toks)
    got = run_alone(rp, "l", toks, [5, 1])
    assert close(got[-20:], want[-20:], dtype)
    assert close(got, want, dtype)


@pytest.mark.parametrize("device,dtype", DEVICES)
def test_long_prompt(models, device, dtype):
    """A prompt of several hundred tokens in one step (many row blocks of the convolution
    and many staged token blocks of the scans, several steps of the query factor), then a
    second portion and decoded tokens that continue its state."""
    _, cfg, wts = models["mixed"]
    eng = engine(models, "mixed", device, dtype, pages=60)
    rp = TraceReplayer(eng)
    toks = tokens_for(cfg, 440, 6)
    want = expected(cfg, wts, toks)
    got = run_alone(rp, "L", toks, [300, 130, 1])
    assert close(got[-40:], want[-40:], dtype)
    assert close(got, want, dtype)


# ---------------------------------------------------------------- batches, pages and slots reused
@pytest.mark.parametrize("device,dtype", DEVICES)
@pytest.mark.parametrize("name", ["mixed", "wide"])
def test_mixed_batches_and_reuse(models, name, device, dtype):
    """Four live requests of unequal length, portions beside decode rows, requests that
    sit out steps; the pool (14 pages) and the four slots are used again by later
    requests.  Every row must match the request run alone (the oracle)."""
    _, cfg, wts = models[name]
    eng = engine(models, name, device, dtype, pages=14)
    rp = TraceReplayer(eng)
    lens = {"a": 30, "b": 9, "c": 41, "d": 2, "e": 25, "f": 17, "g": 33}
    toks = {k: tokens_for(cfg, n, 10 + i) for i, (k, n) in enumerate(lens.items())}
    want = {k: expected(cfg, wts, v) for k, v in toks.items()}
    at = {k: 0 for k in lens}
    got = {k: [] for k in lens}
    # (request, tokens) per step; a request is freed when its tokens are used up
    plan = [[("a", 7), ("b", 3)], [("a", 1), ("b", 1), ("c", 12)], [("a", 1), ("c", 2), ("d", 2)],
            [("b", 5), ("c", 1), ("a", 9)], [("a", 1), ("c", 1)], [("a", 11), ("c", 25), ("e", 4)],
            [("e", 1), ("f", 17)], [("e", 1), ("g", 8)], [("e", 19), ("g", 1)], [("g", 24)]]
    used_pages, used_slots = [], []
    for step in plan:
        entries, end = [], []
        for k, n in step:
            lo = at[k]
            entries.append({"id": k, "tokens": toks[k][lo:lo + n], "want": list(range(n))})
            at[k] += n
            if at[k] == lens[k]:
                end.append(k)
        assert len(rp.seqs) <= 4
        lg = rp.step(entries, end).cpu().numpy()
        for s in rp.seqs.values():
            used_pages += s.block_ids
        o = 0
        for k, n in step:
            got[k].append(lg[o:o + n])
            o += n
    assert len(used_pages) > len(set(used_pages))          # pages were handed out again
    for k in lens:
        assert at[k] == lens[k]
        assert close(np.concatenate(got[k]), want[k], dtype), k


@pytest.mark.parametrize("device,dtype", DEVICES)
def test_slot_reuse_starts_from_zero_state(models, device, dtype):
    """A request that takes over the slot (state tensors, convolution inputs) and the pages
    of a finished one must not see anything of it."""
    _, cfg, wts = models["mixed"]
    eng = engine(models, "mixed", device, dtype, pages=8, seqs=1)
    rp = TraceReplayer(eng)
    for i in range(3):
        toks = tokens_for(cfg, 37 + i, 20 + i)
        got = run_alone(rp, "r%d" % i, toks, [11, 1])
        assert close(got, expected(cfg, wts, toks), dtype), i


@pytest.mark.parametrize("device,dtype", [CPU, GPU32])
@pytest.mark.parametrize("name", ["mixed", "plain"])
def test_residual_stream_after_every_layer(models, name, device, dtype):
    """The fp32 stream after each layer run against the oracle's (a shared layer counts each
    time it runs)."""
    _, cfg, wts = models[name]
    eng = engine(models, name, device, dtype)
    rp = TraceReplayer(eng)
    toks = tokens_for(cfg, 29, 9)
    want = []
    oracle.forward(cfg, wts, toks, taps=want)
    model = eng.executor.runner.model
    taps = []
    orig = model.forward
    model.forward = lambda *a, **k: orig(*a, taps=taps, **k)
    try:
        run_alone(rp, "t", toks, [len(toks)])
    finally:
        model.forward = orig
    assert len(taps) == len(want) == len(cfg["layers"])
    for i, (g, w) in enumerate(zip(taps, want)):
        np.testing.assert_allclose(g.cpu().numpy(), w, rtol=5e-4, atol=6e-4, err_msg="layer %d" % i)


# ---------------------------------------------------------------- generation, presets, config
@pytest.mark.parametrize("device,dtype", [CPU, GPU32])
def test_greedy_generation_through_the_scheduler(models, device, dtype):
    """LLM.generate (scheduler, chunked prefill, sampling kernel at temperature 0, decode
    graphs on the GPU) picks the oracle's arg-max token at every step."""
    if device == "cuda" and not torch.cuda.is_available():
        pytest.skip("no GPU")
    d, cfg, wts = models["mixed"]
    llm = LLM(model=d, dtype=dtype, device=device, block_size=8, max_num_seqs=3, max_model_len=96,
              max_num_batched_tokens=16, num_gpu_blocks_override=40, cuda_graph_max_bs=3)
    try:
        prompts = [tokens_for(cfg, n, 30 + n) for n in (19, 5, 33)]
        outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True))
        for p, o in zip(prompts, outs):
            seq = list(p)
            gen = list(o.output_token_ids)
            assert len(gen) == 12
            for tok in gen:
                lg = oracle.forward(cfg, wts, seq)[-1]
                top2 = np.sort(lg)[-2:]
                if top2[1] - top2[0] > 1e-3 * np.abs(lg).max():      # a clear arg-max
                    assert tok == int(np.argmax(lg))
                seq.append(tok)
    finally:
        llm.shutdown()


@pytest.mark.parametrize("device,dtype", [CPU, GPU16])
def test_preset_runs_through_sampling(device, dtype):
    if device == "cuda" and not torch.cuda.is_available():
        pytest.skip("no GPU")
    llm = LLM(model="tiny-lorenex", dtype=dtype, device=device, random_init=True, seed=3,
              block_size=8, max_num_seqs=4, max_model_len=64, num_gpu_blocks_override=40)
    try:
        outs = llm.generate([[1, 5, 9, 200], [7] * 11],
                            SamplingParams(temperature=0.8, top_k=20, max_tokens=6, ignore_eos=True))
        assert len(outs) == 2 and all(len(o.output_token_ids) == 6 for o in outs)
        assert all(0 <= t < 1024 for o in outs for t in o.output_token_ids)
    finally:
        llm.shutdown()


def test_config_reader(models):
    d, cfg, _ = models["mixed"]
    mc, wdir = resolve_model(d)
    assert wdir == d and mc.arch == "lorenex" and mc.weights_of == (0, 1, 0, 1, 4, 5)
    assert mc.learned_pos and mc.tie_embeddings and mc.residual_mult == 0.5
    g, p = mc.layer_specs[0], mc.layer_specs[1]
    assert (g.kind, g.decay_rank, g.decay_tau) == ("gla", 5, 4.0)         # rank: from a1's shape
    assert mc.layer_specs[5].decay_rank == 2
    assert p.left.q_temp == (0.5, 16) and p.left.conv == 3 and p.left.qk_unit and p.left.v_unit
    assert (p.right.kind, p.right.width, p.right.dim, p.right.dt_rank) == ("mamba", 24, 6, 3)
    assert (p.mlp.router, p.mlp.identity, p.mlp.limit) == ("softmax_all", 1, 1.5)
    mc2, _ = resolve_model(models["plain"][0])
    assert mc2.weights_of == (0, 1, 0, 3, 0, 5) and mc2.layer_specs[3].mlp is None
    assert mc.has_recurrent_state and PRESETS["tiny-lorenex"].weights_of[2] == 1
    bad = json.loads(json.dumps(cfg))
    bad["layers"][2]["weights_of"] = 1                                     # another type
    with pytest.raises(ValueError):
        from kubernetes_gpu_cluster_amd.models.configs import lorenex_config
        lorenex_config(bad, "bad", {"l0.mix.a1": (5, 64), "l5.mix.a1": (2, 64)})
