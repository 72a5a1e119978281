"""Gagorax through the engine against the plain per-token oracle
(tests/gagorax_oracle.py): every mixer alone, prompt portions of many
sizes, decoding through the cache and state, mixed batches, reuse of pages
and slots, odd sizes, and greedy generation through LLMEngine.generate.

Each case writes a small random checkpoint, builds an engine on it and
replays a step plan with the product's trace replay; the CPU cases run the
reference ops, the gpu-marked ones the HIP kernels in float32 and bfloat16.
"""

import io
import json
import os

import numpy as np
import pytest
import torch

from gagorax_oracle import Oracle, random_weights

CASES = [
    pytest.param("cpu", "float32", id="cpu-f32"),
    pytest.param("cuda", "float32", id="gpu-f32", marks=pytest.mark.gpu),
    pytest.param("cuda", "bfloat16", id="gpu-bf16", marks=pytest.mark.gpu),
]
# rms of the logit difference over rms of the logits
TOL = {"float32": 2e-4, "bfloat16": 6e-2}


def attn(heads=4, kv=2, dim=16, vdim=16, rot=None, base=10000.0, scale=None, mlp=None):
    return {"type": "attention", "mlp": mlp, "mixer": {
        "heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim,
        "rot": {"base": base, "dims": dim if rot is None else rot},
        "scale": dim ** -0.5 if scale is None else scale}}


def lightning(heads=2, dim=16, vdim=16, decay=(0.9, 0.99), mlp=None):
    return {"type": "lightning", "mlp": mlp, "mixer": {
        "heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}}


def mamba(inner=96, state=8, dt_rank=6, conv=4, mlp=None):
    return {"type": "mamba1", "mlp": mlp, "mixer": {
        "inner": inner, "state": state, "dt_rank": dt_rank, "conv": conv}}


def model_cfg(layers, width=64, vocab=96, eps=1e-5, logit_scale=1.5):
    return {"architecture": "Gagorax", "layers": layers, "logit_scale": logit_scale,
            "norm": {"eps": eps}, "vocab": vocab, "width": width}


FF = {"kind": "dense", "ff": 80}
MIXED = model_cfg([attn(mlp=FF), lightning(), mamba(), attn(heads=2, kv=1, dim=24, vdim=8, rot=12)])


def write_checkpoint(path, cfg, seed=0, weights=None):
    from safetensors.torch import save_file

    os.makedirs(path, exist_ok=True)
    w = weights if weights is not None else random_weights(cfg, seed)
    save_file({k: v.contiguous() for k, v in w.items()},
              os.path.join(path, "model.safetensors"))
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    return w


def make_engine(path, device, dtype, max_tokens=256, **kw):
    from arks_amd.config import EngineConfig
    from arks_amd.engine import LLMEngine

    cfg = EngineConfig(model_path=str(path), device=device, dtype=dtype,
                       kv_cache_blocks=-(-max_tokens // 16), max_num_seqs=4,
                       max_model_len=max_tokens, max_num_batched_tokens=max_tokens,
                       enable_prefix_caching=False, **kw)
    return LLMEngine(cfg)


def replay(engine, tmp_path, steps):
    """steps: list of lists of (request id, tokens, end?). Logits of every
    token are asked for. Returns {id: [n_tokens, vocab] array}."""
    from arks_amd.engine.trace import replay as trace_replay

    out = tmp_path / "out"
    out.mkdir(exist_ok=True)
    lines = []
    for n, step in enumerate(steps):
        lines.append(json.dumps({
            "step": n,
            "entries": [{"id": i, "tokens": t, "want": list(range(len(t)))}
                        for i, t, _ in step],
            "end": [i for i, _, e in step if e]}))
    trace_replay(engine, lines, str(out), log=io.StringIO())
    got = {}
    V = engine.model_cfg.vocab_size
    for n, step in enumerate(steps):
        arr = np.fromfile(out / f"{n}.f32", dtype="<f4").reshape(-1, V)
        at = 0
        for i, t, _ in step:
            got.setdefault(i, []).append(arr[at:at + len(t)])
            at += len(t)
    return {i: np.concatenate(v) for i, v in got.items()}


def rel_err(got, want):
    want = want.numpy() if isinstance(want, torch.Tensor) else want
    d = got - want
    return float(np.sqrt((d ** 2).mean(-1)).max() / np.sqrt((want ** 2).mean()))


def portions(tokens, sizes):
    out, at, k = [], 0, 0
    while at < len(tokens):
        n = sizes[k % len(sizes)]
        out.append(tokens[at:at + n])
        at += n
        k += 1
    return out


def toks(n, vocab=96, seed=1):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("layers", [
    [attn()], [attn(mlp=FF)], [lightning()], [mamba()], [mamba(mlp=FF)],
], ids=["attention", "attention+ff", "lightning", "mamba1", "mamba1+ff"])
def test_each_mixer_alone(tmp_path, device, dtype, layers):
    cfg = model_cfg(layers)
    w = write_checkpoint(tmp_path / "m", cfg)
    t = toks(37)
    want = Oracle(cfg, w).run(t)
    eng = make_engine(tmp_path / "m", device, dtype)
    got = replay(eng, tmp_path, [[("a", t, True)]])["a"]
    assert rel_err(got, want) < TOL[dtype]


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("sizes", [[100], [29, 1, 1, 1], [2], [3, 17, 2, 5, 1, 16, 32]],
                         ids=["whole", "decode", "twos", "uneven"])
def test_portions_and_decode_match_whole_prompt(tmp_path, device, dtype, sizes):
    w = write_checkpoint(tmp_path / "m", MIXED)
    t = toks(61)
    want = Oracle(MIXED, w).run(t)
    eng = make_engine(tmp_path / "m", device, dtype)
    parts = portions(t, sizes)
    steps = [[("a", p, k == len(parts) - 1)] for k, p in enumerate(parts)]
    got = replay(eng, tmp_path, steps)["a"]
    assert rel_err(got, want) < TOL[dtype]


@pytest.mark.parametrize("device,dtype", CASES)
def test_mixed_batch_equals_each_alone_and_reuses_pages_and_slots(tmp_path, device, dtype):
    w = write_checkpoint(tmp_path / "m", MIXED)
    orc = Oracle(MIXED, w)
    reqs = {i: toks(n, seed=10 + k) for k, (i, n) in enumerate(
        [("a", 50), ("b", 7), ("c", 33), ("d", 1), ("e", 40), ("f", 18), ("g", 21)])}
    want = {i: orc.run(t) for i, t in reqs.items()}
    # pool of 9 pages and 4 slots: requests come and go, at most 4 live
    plan = [
        [("a", 0, 20), ("b", 0, 2), ("c", 0, 33)],
        [("a", 20, 21), ("b", 2, 3), ("d", 0, 1)],          # c, d end
        [("a", 21, 37), ("b", 3, 4), ("e", 0, 17)],
        [("b", 4, 7), ("a", 37, 38), ("e", 17, 19)],        # b ends
        [("a", 38, 50), ("e", 19, 40), ("f", 0, 18)],       # a, e, f end
        [("g", 0, 2)], [("g", 2, 3)], [("g", 3, 21)],
    ]
    steps = [[(i, reqs[i][lo:hi], hi == len(reqs[i])) for i, lo, hi in st] for st in plan]
    eng = make_engine(tmp_path / "m", device, dtype, max_tokens=144)
    got = replay(eng, tmp_path, steps)
    for i in reqs:
        assert rel_err(got[i], want[i]) < TOL[dtype], i
    assert eng.scheduler.allocator.num_free == eng.runner.num_blocks
    assert eng.runner.state_slots.num_free == 4


@pytest.mark.parametrize("device,dtype", CASES)
def test_long_decode_crosses_pages(tmp_path, device, dtype):
    w = write_checkpoint(tmp_path / "m", MIXED)
    t = toks(90, seed=5)
    want = Oracle(MIXED, w).run(t)
    eng = make_engine(tmp_path / "m", device, dtype)
    steps = [[("a", t[:3], False)]] + [[("a", [x], k == 86)] for k, x in enumerate(t[3:])]
    got = replay(eng, tmp_path, steps)["a"]
    assert rel_err(got, want) < TOL[dtype]


ODD = [
    # heads == kv_heads, partial rotary, vdim != dim, width not a multiple of 64
    model_cfg([attn(heads=3, kv=3, dim=20, vdim=12, rot=8, base=500.0, scale=0.3, mlp={"kind": "dense", "ff": 50}),
               lightning(heads=3, dim=8, vdim=20, decay=(0.5, 0.97, 1.0)),
               mamba(inner=50, state=5, dt_rank=3, conv=2)], width=72, vocab=70, logit_scale=0.7),
    # one kv head, long conv, state beyond one lane group, every layer with ff
    model_cfg([mamba(inner=40, state=20, dt_rank=1, conv=5, mlp=FF),
               attn(heads=4, kv=1, dim=8, vdim=32, rot=2, mlp=FF),
               lightning(heads=1, dim=40, vdim=8, decay=(0.8,), mlp=FF)], width=48, eps=1e-3),
    # a conv of one tap (no history at all)
    model_cfg([mamba(inner=32, state=4, dt_rank=2, conv=1), attn(heads=2, kv=2, dim=4, vdim=2)], width=32),
]


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("which", range(len(ODD)))
def test_other_sizes(tmp_path, device, dtype, which):
    cfg = ODD[which]
    w = write_checkpoint(tmp_path / "m", cfg, seed=which + 3)
    V = cfg["vocab"]
    ta, tb = toks(45, V, seed=2), toks(19, V, seed=3)
    orc = Oracle(cfg, w)
    eng = make_engine(tmp_path / "m", device, dtype)
    steps = [[("a", ta[:17], False), ("b", tb[:1], False)],
             [("a", ta[17:18], False), ("b", tb[1:2], False)],
             [("a", ta[18:20], False), ("b", tb[2:], True)],
             [("a", ta[20:], True)]]
    got = replay(eng, tmp_path, steps)
    assert rel_err(got["a"], orc.run(ta)) < TOL[dtype]
    assert rel_err(got["b"], orc.run(tb)) < TOL[dtype]


@pytest.mark.parametrize("device,dtype", CASES)
def test_greedy_generation_through_the_scheduler(tmp_path, device, dtype):
    from arks_amd.engine import SamplingParams

    w = write_checkpoint(tmp_path / "m", MIXED, seed=9)
    orc = Oracle(MIXED, w)
    prompts = [toks(23, seed=21), toks(5, seed=22), toks(40, seed=23)]
    # a 16-token budget cuts the prompts into portions and mixes them with
    # the decoding of earlier requests
    eng = make_engine(tmp_path / "m", device, dtype)
    eng.scheduler.max_num_batched_tokens = 16
    outs = eng.generate(prompts, SamplingParams(max_tokens=12, ignore_eos=True))
    for p, o in zip(prompts, outs):
        st = orc.new_state()
        for t in p[:-1]:
            orc.token(st, t)
        cur, n_diff = p[-1], 0
        for got_tok in o:
            logits = orc.token(st, cur)
            top2 = torch.topk(logits, 2).values
            if int(logits.argmax()) != got_tok:
                # only a near-tie may flip under rounding
                assert float(logits.max() - logits[got_tok]) < (
                    1e-3 if dtype == "float32" else 0.15), (top2, got_tok)
            cur = got_tok  # follow the engine's choice
    assert eng.scheduler.allocator.num_free == eng.runner.num_blocks


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("dim,heads,kv", [(32, 4, 2), (64, 8, 1), (96, 2, 2), (128, 4, 2),
                                           (256, 2, 1), (64, 9, 1)])
def test_attention_head_sizes_of_the_mfma_kernels(tmp_path, device, dtype, dim, heads, kv):
    """Equal q/k and value sizes the matrix-core kernels are built for: a
    long prompt (the 256-row kernel where it exists), short portions (the
    64-row kernel), single tokens (flash decode) and mixes of them."""
    cfg = model_cfg([attn(heads=heads, kv=kv, dim=dim, vdim=dim, rot=dim // 2, mlp=FF),
                     attn(heads=heads, kv=kv, dim=dim, vdim=dim)], width=64)
    w = write_checkpoint(tmp_path / "m", cfg, seed=dim)
    ta, tb = toks(330, seed=4), toks(40, seed=6)
    orc = Oracle(cfg, w)
    eng = make_engine(tmp_path / "m", device, dtype, max_tokens=512)
    steps = [[("a", ta[:300], False)],
             [("a", ta[300:301], False), ("b", tb[:30], False)],
             [("a", ta[301:302], False), ("b", tb[30:31], False)],
             [("a", ta[302:303], False), ("b", tb[31:32], False)],
             [("a", ta[303:330], True), ("b", tb[32:33], False)],
             [("b", tb[33:], True)]]
    got = replay(eng, tmp_path, steps)
    assert rel_err(got["a"], orc.run(ta)) < TOL[dtype]
    assert rel_err(got["b"], orc.run(tb)) < TOL[dtype]


@pytest.mark.parametrize("device,dtype", CASES)
def test_long_portions_cross_the_recurrent_chunks(tmp_path, device, dtype):
    """Portions longer than one chunk of the chunk-parallel recurrent
    prefill (64 rows): one row more, exact multiples, one row less, beside
    a second request and single tokens."""
    cfg = model_cfg(MIXED["layers"] + [lightning(heads=2, dim=32, vdim=32, decay=(0.95, 1.0))])
    w = write_checkpoint(tmp_path / "m", cfg, seed=4)
    orc = Oracle(cfg, w)
    ta, tb = toks(330, seed=31), toks(200, seed=32)
    eng = make_engine(tmp_path / "m", device, dtype, max_tokens=576)
    cuts_a = [65, 128, 1, 63, 73]
    steps, at = [], 0
    for k, n in enumerate(cuts_a):
        st = [("a", ta[at:at + n], at + n == 330)]
        if k == 1:
            st.append(("b", tb[:129], False))
        if k == 2:
            st.append(("b", tb[129:130], False))
        if k == 3:
            st.append(("b", tb[130:], True))
        steps.append(st)
        at += n
    got = replay(eng, tmp_path, steps)
    assert rel_err(got["a"], orc.run(ta)) < TOL[dtype]
    assert rel_err(got["b"], orc.run(tb)) < TOL[dtype]


def random_model(seed):
    """A random layer list with sizes off the beaten path: widths that are
    not multiples of 8 or 64, head sizes with and without a matrix-core
    kernel, unequal q/k and value sizes, large and tiny state sizes, dt
    ranks on both sides of the GEMM threshold, 1 to 5 conv taps."""
    import random

    r = random.Random(seed)
    width = r.choice([40, 56, 100, 128, 192])
    layers = []
    for _ in range(r.randint(2, 5)):
        mlp = r.choice([None, {"kind": "dense", "ff": r.choice([24, 72, 160])}])
        kind = r.choice(["attention", "lightning", "mamba1"])
        if kind == "attention":
            kv = r.choice([1, 2, 3])
            heads = kv * r.choice([1, 2, 4, 9])
            dim = r.choice([8, 32, 40, 64, 96])
            vdim = r.choice([dim, dim, 16, 48])
            layers.append(attn(heads=heads, kv=kv, dim=dim, vdim=vdim,
                               rot=r.choice([0, 2, dim // 2, dim]),
                               base=r.choice([100.0, 10000.0, 1e6]),
                               scale=r.choice([dim ** -0.5, 0.05, 0.4]), mlp=mlp))
        elif kind == "lightning":
            heads = r.choice([1, 2, 5])
            dim, vdim = r.choice([(8, 8), (32, 32), (64, 64), (24, 40), (64, 128), (32, 64)])
            layers.append(lightning(heads=heads, dim=dim, vdim=vdim,
                                    decay=[r.choice([1.0, 0.999, 0.9, 0.3]) for _ in range(heads)],
                                    mlp=mlp))
        else:
            layers.append(mamba(inner=r.choice([24, 64, 136]), state=r.choice([1, 4, 16, 48, 80]),
                                dt_rank=r.choice([1, 4, 8, 24]), conv=r.randint(1, 5), mlp=mlp))
    return model_cfg(layers, width=width, vocab=r.choice([64, 200]),
                     eps=r.choice([1e-6, 1e-5, 1e-2]), logit_scale=r.choice([0.5, 1.0, 3.0]))


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("seed", range(8))
def test_random_models(tmp_path, device, dtype, seed):
    cfg = random_model(seed)
    w = write_checkpoint(tmp_path / "m", cfg, seed=seed)
    V = cfg["vocab"]
    ta, tb = toks(150, V, seed=40 + seed), toks(70, V, seed=60 + seed)
    orc = Oracle(cfg, w)
    eng = make_engine(tmp_path / "m", device, dtype, max_tokens=256)
    steps = [[("a", ta[:130], False)],
             [("a", ta[130:131], False), ("b", tb[:66], False)],
             [("a", ta[131:132], False), ("b", tb[66:67], False)],
             [("a", ta[132:133], False)], [("a", ta[133:134], False)],
             [("a", ta[134:], True), ("b", tb[67:], True)]]
    got = replay(eng, tmp_path, steps)
    # five random recurrent layers in a row amplify bf16 rounding (the same
    # error with every kernel path); float32 stays at the tight bound
    tol = 2 * TOL[dtype] if dtype == "bfloat16" else TOL[dtype]
    assert rel_err(got["a"], orc.run(ta)) < tol
    assert rel_err(got["b"], orc.run(tb)) < tol


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("dim", [64, 128])
def test_long_prompt_deep_kv(tmp_path, device, dtype, dim):
    """A prompt long enough that the 256-row attention kernel splits its key
    range into parts (the sink must count once) and decoding reads many
    pages in several partitions."""
    cfg = model_cfg([attn(heads=2, kv=1, dim=dim, vdim=dim, mlp=FF), lightning(heads=1, dim=32, vdim=32, decay=(0.99,)),
                     mamba(inner=64, state=16, dt_rank=8, conv=4)], width=64)
    w = write_checkpoint(tmp_path / "m", cfg, seed=dim + 1)
    t = toks(1210, seed=8)
    want = Oracle(cfg, w).run(t)
    eng = make_engine(tmp_path / "m", device, dtype, max_tokens=1280)
    steps = [[("a", t[:1200], False)]] + [[("a", [x], k == 9)] for k, x in enumerate(t[1200:])]
    got = replay(eng, tmp_path, steps)["a"]
    assert rel_err(got, want) < TOL[dtype]


def test_preemption_recomputes_state(tmp_path):
    """A page pool too small for all requests: sequences are preempted
    (pages and state slot given back) and recomputed; the tokens must equal
    those of an engine with room for everything."""
    from arks_amd.engine import SamplingParams

    write_checkpoint(tmp_path / "m", MIXED, seed=12)
    prompts = [toks(30, seed=70 + i) for i in range(3)]
    sp = SamplingParams(max_tokens=40, ignore_eos=True)
    big = make_engine(tmp_path / "m", "cpu", "float32", max_tokens=512)
    want = big.generate(prompts, sp)
    small = make_engine(tmp_path / "m", "cpu", "float32", max_tokens=160)
    got = small.generate(prompts, sp)
    assert small.scheduler.num_preemptions > 0
    assert got == want
    assert small.runner.state_slots.num_free == 4
    assert small.scheduler.allocator.num_free == small.runner.num_blocks
