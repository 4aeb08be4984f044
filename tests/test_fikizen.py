"""The Fikizen layer-list decoder against the plain oracle of tests/fikizen_oracle.py: every
mechanism alone (whole rows, portions, one token from the cache / state), and the engine (paged
cache, state slots, batching, scheduler) against whole-sequence oracle logits: prefill vs
token-by-token decoding, prompt portions down to two tokens, unequal requests in one batch,
freed pages and slots used again, window edges, far keys across page borders, first tokens, long
decoding, other sizes, shared weights, greedy generation.
The same tests run on the CPU (reference ops) and, marked gpu, on the HIP kernels in bf16 and fp32."""
import pytest
import torch

from hipserve.config import EngineConfig, FikizenConfig
from hipserve.engine.llm_engine import LLMEngine
from hipserve.engine.request import SamplingParams
from hipserve.engine.trace import TraceSession, build_engine
from hipserve.models.llama import AttnMeta
from hipserve.models.mixers import DenseFF, make_mixer
from hipserve.ops import get_ops
from hipserve.parallel.comm import TPGroup

from . import fikizen_oracle as O

CPU = ("cpu", "float32")
TARGETS = [pytest.param(CPU, id="cpu-f32"),
           pytest.param(("cuda", "float32"), id="gpu-f32", marks=pytest.mark.gpu),
           pytest.param(("cuda", "bfloat16"), id="gpu-bf16", marks=pytest.mark.gpu)]
TOL = {"float32": 2e-4, "bfloat16": 1e-1}   # bf16: rounding of six layers, the worst of all rows
EPS = 1e-5


def rel_err(got, want):
    """rms of the difference over rms of the reference, both with their mean over the last axis taken off."""
    got, want = torch.as_tensor(got).float().cpu(), torch.as_tensor(want).float().cpu()
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    w = want - want.mean(-1, keepdim=True)
    return float((d.pow(2).mean(-1).sqrt() / w.pow(2).mean(-1).sqrt().clamp_min(1e-9)).max())


def tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def base_config(**kw):
    f = O.dense()
    layers = [O.attn_layer(mlp=f), O.delta_layer(conv=4)]
    layers += [O.shared(layers, 0), O.parallel_layer(left=dict(heads=6, kv_heads=3, window=9), mlp=f),
               O.delta_layer(heads=2, kv_heads=2, dim=5, vdim=70)]
    layers += [O.shared(layers, 3)]
    return O.make_config(layers, **kw)


def session(tmp_path, cfg, W, target, max_tokens=512, name="m"):
    path = O.save_checkpoint(str(tmp_path / name), cfg, W)
    eng = build_engine(path, target[1], max_tokens, target[0])
    if target[0] == "cuda":  # the HIP kernels are the path that runs
        assert eng.runner.ops.name == "hip" and hasattr(torch.ops.hipserve_delta, "window_attention")
    return TraceSession(eng)


def replay(sess, steps):
    """steps: list of [(id, tokens, want, ends)] -> {(id, absolute position): logits row}."""
    out, at = {}, {}
    for step in steps:
        entries = [{"id": i, "tokens": t, "want": w} for i, t, w, _ in step]
        lg = sess.step(entries, [i for i, _, _, e in step if e])
        k = 0
        for i, t, w, _ in step:
            for x in w:
                out[(i, at.get(i, 0) + x)] = lg[k]
                k += 1
            at[i] = at.get(i, 0) + len(t)
    return out


def portions(toks, sizes, rid="a"):
    """One request cut into the given portion sizes (the rest one token at a time), all positions wanted."""
    steps, p = [], 0
    sizes = list(sizes)
    while p < len(toks):
        n = min(sizes.pop(0) if sizes else 1, len(toks) - p)
        steps.append([(rid, toks[p:p + n], list(range(n)), p + n == len(toks))])
        p += n
    return steps


def check_all(got, rid, ref, tol):
    """fp32: every row within tol. bf16 (tol >= 0.01): the rows' error as a whole within tol / 2 and no single
    row beyond 3 tol: the rounding of a tiny model's six layers now and then lands on a row whose logits vary
    little, while a wrong key, state or window moves many rows by far more."""
    rows = sorted(p for i, p in got if i == rid)
    assert rows == list(range(ref.shape[0]))
    g = torch.stack([torch.as_tensor(got[(rid, p)]) for p in rows]).float().cpu()
    if tol < 0.01:
        err = rel_err(g, ref)
        assert err < tol, err
        return
    r = torch.as_tensor(ref).float()
    d = (g - r) - (g - r).mean(-1, keepdim=True)
    w = r - r.mean(-1, keepdim=True)
    whole = float(d.pow(2).mean().sqrt() / w.pow(2).mean().sqrt())
    assert whole < tol / 2 and rel_err(g, ref) < 3 * tol, (whole, rel_err(g, ref))


# ---------------------------------------------------------------- mechanisms alone
def one_seq_meta(T, dev, start=0, block_size=4, slot=0, perm_seed=0, total=160):
    """Step metadata of one sequence's rows start .. start+T-1 of a sequence of up to `total` tokens
    whose pages are scattered in the pool (the same page table at every call)."""
    nblk = -(-total // block_size)
    g = torch.Generator().manual_seed(perm_seed)
    pages = (torch.randperm(nblk + 3, generator=g)[:nblk]).to(torch.int32)
    pos = torch.arange(start, start + T)
    slots = pages.long()[pos // block_size] * block_size + pos % block_size
    dec = T == 1 and start > 0
    return AttnMeta(num_prefill_tokens=0 if dec else T, num_decode=1 if dec else 0, positions=pos.to(dev),
                    slot_mapping=slots.to(dev), seq_cu=torch.tensor([0, T], dtype=torch.int32, device=dev),
                    seq_ctx=torch.tensor([start + T], dtype=torch.int32, device=dev),
                    seq_bt=pages.view(1, -1).to(dev), seq_state=torch.tensor([slot], dtype=torch.int32, device=dev),
                    max_q=T), nblk + 3


def run_mixer(layer, W, h, target, cuts, width=24, slot=1):
    """The layer's mixer on rows h, cut into the given row ranges, each run from what the one before left in
    the cache / state (whose slot held garbage before the first)."""
    dev, dt = torch.device(target[0]), getattr(torch, target[1])
    spec = FikizenConfig.from_dict(O.make_config([layer], width=width)).layers[0].mixer
    mix = make_mixer(spec, width, EPS, dev, dt, get_ops(dev))
    mix.load(lambda k: W[k], "l0.mix.")
    _, nblk = one_seq_meta(1, dev)
    cache = torch.zeros(nblk, 4, mix.cache_dim, device=dev, dtype=dt) if mix.cache_dim else None
    state = None
    if mix.state_shapes:
        state = [torch.full(s, 7.0, device=dev, dtype=torch.float32) for s in mix.state_shapes(3)]
    parts = []
    for a, b in cuts:
        meta, _ = one_seq_meta(b - a, dev, start=a, slot=slot)
        parts.append(mix.forward(h[a:b].to(dev, dt), meta, cache, state))
    return torch.cat(parts)


CUTS = [[(0, 90)], [(0, 37), (37, 89), (89, 90)], [(0, 1), (1, 3), (3, 5), (5, 64), (64, 66), (66, 90)]]


def rows(T, width, seed):
    return torch.randn(T, width, generator=torch.Generator().manual_seed(seed)).bfloat16().float()


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("shape", [dict(), dict(heads=5, kv_heads=5, dim=16, vdim=3, window=1, rot_dims=16),
                                   dict(heads=1, kv_heads=1, dim=6, rot_dims=2, window=3),
                                   dict(heads=36, kv_heads=2, window=70, rot_dims=4),
                                   dict(heads=3, kv_heads=1, dim=80, vdim=130, window=200, rot_dims=80, base=1e6)])
def test_gated_sink_attention_alone(target, shape):
    l = O.attn_layer(**shape)
    W = O.make_weights(O.make_config([l], width=24), seed=3)
    h = rows(90, 24, 1).double()
    want = O.attention_mixer(h, l["mixer"], {k: v.double() for k, v in W.items()}, "l0.mix.", EPS, True, False, False)
    for cuts in CUTS:
        assert rel_err(run_mixer(l, W, h.float(), target, cuts), want) < TOL[target[1]]


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("shape", [dict(), dict(heads=2, dim=40, left=dict(heads=2, kv_heads=1, dim=20, vdim=7, window=33)),
                                   dict(heads=1, dim=70, left_scale=1.0, right_scale=0.3)])
def test_parallel_mixer_alone(target, shape):
    """Biased projections, whole-projection q / k norm, unit-rms values and the sink on the left; decay
    bottleneck, removal rate, unit key and the state on the right; one output projection for both."""
    l = O.parallel_layer(**shape)
    W = O.make_weights(O.make_config([l], width=24), seed=4)
    h = rows(90, 24, 2).double()
    W64 = {k: v.double() for k, v in W.items()}
    want = O.parallel_mixer(h, l["mixer"], W64, "l0.mix.", EPS)
    for cuts in CUTS:
        assert rel_err(run_mixer(l, W, h.float(), target, cuts), want) < TOL[target[1]]
    # each half really contributes with its own scale
    left = O.attention_mixer(h, l["mixer"]["left"], W64, "l0.mix.left.", EPS, False, True, True)
    right = O.delta_rule_mixer(h, l["mixer"]["right"], W64, "l0.mix.right.", EPS)
    assert rel_err(left, want) > 0.1 and rel_err(right, want) > 0.1


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("shape", [dict(), dict(heads=6, kv_heads=1, dim=33, vdim=5, conv=2),
                                   dict(heads=1, kv_heads=1, dim=4, vdim=100, conv=7),
                                   dict(heads=2, kv_heads=2, dim=70, vdim=8, conv=1)])
def test_gated_delta_alone(target, shape):
    l = O.delta_layer(**shape)
    W = O.make_weights(O.make_config([l], width=24), seed=5)
    h = rows(90, 24, 3).double()
    want = O.gated_delta_mixer(h, l["mixer"], {k: v.double() for k, v in W.items()}, "l0.mix.", EPS)
    for cuts in CUTS:
        assert rel_err(run_mixer(l, W, h.float(), target, cuts), want) < TOL[target[1]]


@pytest.mark.parametrize("target", TARGETS)
def test_state_is_carried_not_reset_and_slots_are_separate(target):
    """Two sequences take turns in two slots; a lost or mixed-up state (or convolution tail) would show."""
    for l in (O.delta_layer(), O.parallel_layer()):
        W = O.make_weights(O.make_config([l], width=24), seed=6)
        dev, dt = torch.device(target[0]), getattr(torch, target[1])
        spec = FikizenConfig.from_dict(O.make_config([l], width=24)).layers[0].mixer
        mix = make_mixer(spec, 24, EPS, dev, dt, get_ops(dev))
        mix.load(lambda k: W[k], "l0.mix.")
        hs = [rows(30, 24, 10), rows(30, 24, 11)]
        W64 = {k: v.double() for k, v in W.items()}
        fn = O.gated_delta_mixer if l["type"] == "delta" else O.parallel_mixer
        wants = [fn(h.double(), l["mixer"], W64, "l0.mix.", EPS) for h in hs]
        _, nblk = one_seq_meta(1, dev)
        caches = [torch.zeros(nblk, 4, mix.cache_dim, device=dev, dtype=dt) if mix.cache_dim else None for _ in hs]
        state = [torch.zeros(s, device=dev, dtype=torch.float32) for s in mix.state_shapes(3)]
        got = [[], []]
        for a, b in ((0, 7), (7, 8), (8, 21), (21, 30)):
            for k in (0, 1):
                meta, _ = one_seq_meta(b - a, dev, start=a, slot=2 - k)
                got[k].append(mix.forward(hs[k][a:b].to(dev, dt), meta, caches[k], state))
        for k in (0, 1):
            assert rel_err(torch.cat(got[k]), wants[k]) < TOL[target[1]]
        assert rel_err(torch.cat(got[0]), wants[1]) > 0.3


@pytest.mark.parametrize("target", TARGETS)
def test_feed_forward_activation_and_residual_update_alone(target):
    dev, dt = torch.device(target[0]), getattr(torch, target[1])
    ops = get_ops(dev)
    l = O.attn_layer(mlp=O.dense(ff=50))
    cfg = O.make_config([l], width=24)
    W = O.make_weights(cfg, seed=7)
    W["l0.mlp.act"] = torch.tensor([0.75, -1.25])
    h = (rows(40, 24, 4) * 3).double()
    want = O.feed_forward(h, {k: v.double() for k, v in W.items()}, "l0.mlp.")
    ff = DenseFF(FikizenConfig.from_dict(cfg).layers[0].mlp, 24, dev, dt, ops)
    ff.load(lambda k: W[k], "l0.mlp.")
    assert rel_err(ff.forward(h.to(dev, dt)), want) < TOL[target[1]]
    # both branches of the activation, far from zero too
    z = torch.linspace(-30, 30, 241).view(1, -1)
    got = torch.empty_like(z, device=dev)
    ops.activation(got, z.to(dev), "xielu", ff.c0, ff.c1)
    assert rel_err(got, O.xielu(z.double(), W["l0.mlp.act"][0].double(), W["l0.mlp.act"][1].double())) < 1e-5
    # x <- x + y, then the weighted RMS norm: 32-bit stream
    res = rows(40, 24, 5).to(dev)
    y = rows(40, 24, 6)
    w = 1 + 0.1 * rows(1, 24, 7)[0]
    out = torch.empty(40, 24, device=dev, dtype=dt)
    x2 = res.cpu().double() + y.double()
    ops.scaled_add_group_rmsnorm(out, res, w.to(dev), 1, EPS, y.to(dev, dt))
    assert torch.allclose(res.cpu().double(), x2, atol=1e-6)
    assert rel_err(out, O.rms(x2, EPS) * w.double()) < (1e-5 if target[1] == "float32" else 1e-2)


# ---------------------------------------------------------------- engine
@pytest.mark.parametrize("target", TARGETS)
def test_prefill_and_long_decoding(tmp_path, target):
    cfg = base_config()
    W = O.make_weights(cfg, seed=11)
    toks = tokens(70, cfg["vocab"], 1)
    streams = []
    ref = O.forward(cfg, W, toks, streams)
    sess = session(tmp_path, cfg, W, target)
    model = sess.engine.runner.model
    model.capture = []
    check_all(replay(sess, portions(toks, [len(toks)])), "a", ref, TOL[target[1]])   # the whole prompt at once
    for got, want in zip(model.capture, streams):                                    # the stream after every layer
        assert rel_err(got, want) < TOL[target[1]]
    assert len(model.capture) == len(streams) == 6
    model.capture = None
    # a short prompt, then 60 tokens one by one: the windows (6 and 9) pass over decoded tokens many times
    check_all(replay(sess, portions(toks, [10])), "a", ref, TOL[target[1]])
    check_all(replay(sess, portions(toks, [1])), "a", ref, TOL[target[1]])           # from the very first token


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("sizes", [[2] * 40, [3, 2, 17, 2, 5, 31, 2], [16, 16, 16, 16], [33, 2, 2, 2]])
def test_portions(tmp_path, target, sizes):
    cfg = base_config()
    W = O.make_weights(cfg, seed=12)
    toks = tokens(83, cfg["vocab"], 2)
    ref = O.forward(cfg, W, toks)
    check_all(replay(session(tmp_path, cfg, W, target), portions(toks, sizes)), "a", ref, TOL[target[1]])


@pytest.mark.parametrize("target", TARGETS)
def test_unequal_requests_in_one_batch_and_reuse(tmp_path, target):
    """Up to four live requests of unequal length, portions beside single tokens; finished requests
    give pages and slots back and later ones take them; the pool is small enough that they must."""
    cfg = base_config()
    W = O.make_weights(cfg, seed=13)
    V = cfg["vocab"]
    reqs = {f"r{k}": tokens(n, V, 20 + k) for k, n in enumerate([61, 1, 23, 40, 2, 35, 50, 18])}
    refs = {k: O.forward(cfg, W, t) for k, t in reqs.items()}
    sess = session(tmp_path, cfg, W, target, max_tokens=64 * 4)
    order = list(reqs)
    live, at, steps, cuts = [], {}, [], [5, 1, 2, 9, 1, 1, 3, 16, 1, 2]
    n = 0
    while order or live:
        while order and len(live) < 4:
            live.append(order.pop(0))
        step = []
        for j, rid in enumerate(list(live)):
            if (n + j) % 5 == 4 and len(live) > 1:
                continue  # a request may be left out of a step
            a = at.get(rid, 0)
            c = min(cuts[(n + 3 * j) % len(cuts)], len(reqs[rid]) - a)
            end = a + c == len(reqs[rid])
            step.append((rid, reqs[rid][a:a + c], list(range(c)), end))
            at[rid] = a + c
            if end:
                live.remove(rid)
        if step:
            steps.append(step)
        n += 1
    got = replay(sess, steps)
    for rid, ref in refs.items():
        check_all(got, rid, ref, TOL[target[1]])
    assert sess.engine.blocks.num_free() == sess.engine.blocks.num_blocks
    assert sess.engine.states.num_free() == 4


@pytest.mark.parametrize("target", TARGETS)
def test_window_edges_and_sink_matter_and_are_right(tmp_path, target):
    """With windows of 4 and 5 every key weighs enough that a window one token too long or short moves
    the logits far beyond the tolerance, and so does a softmax without the one in its denominator; the
    engine must agree with the right one."""
    f = O.dense(ff=24)
    lay = lambda d: [O.attn_layer(window=4 + d, mlp=f), O.parallel_layer(left=dict(window=5 + d, scale=1.5), mlp=f)]
    cfg = O.make_config(lay(0))
    W = O.make_weights(cfg, seed=14)
    toks = tokens(40, cfg["vocab"], 3)
    ref = O.forward(cfg, W, toks)
    for d in (-1, 1):
        assert rel_err(O.forward(O.make_config(lay(d)), W, toks)[8:], ref[8:]) > 0.05
    plain = O.sink_softmax
    try:
        O.sink_softmax = lambda s: torch.softmax(s, -1)
        assert rel_err(O.forward(cfg, W, toks), ref) > 0.05
    finally:
        O.sink_softmax = plain
    sess = session(tmp_path, cfg, W, target)
    check_all(replay(sess, portions(toks, [40])), "a", ref, TOL[target[1]])           # edges inside a prompt
    check_all(replay(sess, portions(toks, [6, 3, 2, 5])), "a", ref, TOL[target[1]])   # across portions and decoded


@pytest.mark.parametrize("target", TARGETS)
def test_far_key_across_pages(tmp_path, target):
    """A sharp softmax (large scale) and windows longer than a few pages: most of the weight of a late
    query sits on single keys hundreds of tokens back, in other pages of the cache. (bf16 runs a less
    sharp softmax: at scale 6 the rounding of the scores alone moves the weights.)"""
    sc, gain = (6.0, 1.5) if target[1] == "float32" else (1.0, 1.0)
    lay = lambda w: [O.attn_layer(window=w, scale=sc, heads=2, kv_heads=1),
                     O.parallel_layer(left=dict(window=w, scale=sc, heads=2, kv_heads=2))]
    cfg = O.make_config(lay(1000))
    W = O.make_weights(cfg, seed=15, gain=gain)
    toks = tokens(330, cfg["vocab"], 4)
    ref = O.forward(cfg, W, toks)
    assert rel_err(O.forward(O.make_config(lay(200)), W, toks)[300:], ref[300:]) > 0.05   # the far keys carry the result
    sess = session(tmp_path, cfg, W, target)
    check_all(replay(sess, portions(toks, [330])), "a", ref, TOL[target[1]])
    check_all(replay(sess, portions(toks, [129, 64, 100])), "a", ref, TOL[target[1]])   # the rest decoded


@pytest.mark.parametrize("target", TARGETS)
def test_window_edge_at_a_page_border_in_a_long_prompt(tmp_path, target):
    """Window 64 = four pages of the replay engine. The key weights are the first head's query weights with
    their columns reversed and there is no rotation, so a query scores highest against the key of the token
    whose embedding is its own reversed. The query at 164 is paired so with the token at 100, the newest key
    it must NOT see (the last slot of a page); the query at 173 with the token at 110, among the oldest it
    must see. A window one longer or shorter moves those rows."""
    lay = lambda w: [O.attn_layer(window=w, heads=2, kv_heads=1, scale=1.0, rot_dims=0)]
    cfg = O.make_config(lay(64), softcap=0.0)
    W = O.make_weights(cfg, seed=16)
    W["l0.mix.k"] = W["l0.mix.q"][:12].flip(1).clone()
    W["l0.norm1"] = torch.ones_like(W["l0.norm1"])
    W["embed"][91], W["embed"][93] = W["embed"][90].flip(0), W["embed"][92].flip(0)
    toks = [t % 90 for t in tokens(200, cfg["vocab"], 6)]
    toks[100], toks[164] = 90, 91       # token ids used nowhere else
    toks[110], toks[173] = 92, 93
    ref = O.forward(cfg, W, toks)
    wider, narrower = O.forward(O.make_config(lay(65), softcap=0.0), W, toks), O.forward(O.make_config(lay(63), softcap=0.0), W, toks)
    assert rel_err(wider[164:165], ref[164:165]) > 0.1 and rel_err(narrower[164:165], ref[164:165]) < 1e-3
    assert rel_err(narrower[173:174], ref[173:174]) > 0.1 and rel_err(wider[173:174], ref[173:174]) < 1e-3
    sess = session(tmp_path, cfg, W, target)
    tol = TOL[target[1]] * (1 if target[1] == "float32" else 2)   # scores near 50: bf16 rounds them by 0.1 and more
    check_all(replay(sess, portions(toks, [200])), "a", ref, tol)
    check_all(replay(sess, portions(toks, [101, 60, 2])), "a", ref, tol)   # 164 and 173 are decoded alone


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("variant", ["one_head", "no_mlp", "shared_delta", "no_rotation_no_cap", "wide_heads"])
def test_other_sizes(tmp_path, target, variant):
    f = O.dense(ff=8)
    if variant == "one_head":         # everything 1 that can be; a window longer than the sequence
        layers = [O.attn_layer(heads=1, kv_heads=1, window=64, mlp=f), O.delta_layer(heads=1, kv_heads=1, conv=2, mlp=f),
                  O.parallel_layer(left=dict(heads=1, kv_heads=1, window=2), heads=1, mlp=None)]
        cfg = O.make_config(layers, width=16, vocab=50)
    elif variant == "no_mlp":
        layers = [O.parallel_layer(), O.attn_layer(heads=7, kv_heads=7, dim=4, rot_dims=4, vdim=20, window=7)]
        cfg = O.make_config(layers, width=48, softcap=3.0)
    elif variant == "shared_delta":   # a recurrent layer run three times with one set of weights, states apart
        layers = [O.delta_layer(mlp=f)]
        layers += [O.shared(layers, 0), O.parallel_layer(mlp=f), O.shared(layers, 0)]
        layers += [O.shared(layers, 2)]
        cfg = O.make_config(layers, width=36)
    elif variant == "no_rotation_no_cap":
        layers = [O.attn_layer(rot_dims=0, dim=5, vdim=9, mlp=f), O.parallel_layer(left=dict(rot_dims=12, dim=12))]
        cfg = O.make_config(layers, width=24, softcap=0.0)
    else:
        layers = [O.attn_layer(heads=2, kv_heads=1, dim=72, vdim=136, rot_dims=36, window=11, mlp=O.dense(ff=70)),
                  O.delta_layer(heads=2, kv_heads=1, dim=66, vdim=72), O.parallel_layer(heads=2, dim=68)]
        cfg = O.make_config(layers, width=24)
    W = O.make_weights(cfg, seed=17)
    toks = tokens(45, cfg["vocab"], 5)
    ref = O.forward(cfg, W, toks)
    sess = session(tmp_path, cfg, W, target)
    check_all(replay(sess, portions(toks, [45])), "a", ref, TOL[target[1]])
    check_all(replay(sess, portions(toks, [4, 9, 2, 13])), "a", ref, TOL[target[1]])


def test_config_reader():
    cfg = base_config(softcap=12.5)
    c = FikizenConfig.from_dict(cfg)
    assert c.logit_softcap == 12.5 and c.num_layers == 6 and [r[0] for r in c.runs()] == [0, 1, 0, 3, 4, 3]
    a = c.layers[0].mixer
    assert (a.sink, a.gate, a.bias, a.qk_norm, a.v_norm) == (True, True, False, False, False) and a.window == 6
    p = c.layers[3].mixer
    assert (p.left.gate, p.left.bias, p.left.qk_norm, p.left.v_norm) == (False, True, True, True)
    assert (p.left_scale, p.right_scale, p.right.heads) == (0.7, 1.2, 3)
    bad = base_config()
    bad["layers"][2] = dict(bad["layers"][2], weights_of=2)
    with pytest.raises(ValueError):
        FikizenConfig.from_dict(bad)


@pytest.mark.parametrize("target", TARGETS)
def test_greedy_generation_through_the_scheduler(tmp_path, target):
    """LLMEngine.generate: the scheduler's own chunked prefill (a 24-token budget), batching of three
    prompts of unequal length and the sampler; every generated token is an argmax of the oracle's
    logits over the tokens before it."""
    cfg = base_config()
    W = O.make_weights(cfg, seed=18)
    path = O.save_checkpoint(str(tmp_path / "g"), cfg, W)
    dev = target[0]
    ecfg = EngineConfig(model=path, dtype=target[1], device=dev, max_num_seqs=4, max_num_batched_tokens=24,
                        num_kv_blocks=64, max_model_len=256, enforce_eager=True)
    eng = LLMEngine(ecfg, tp=TPGroup(0, 1, None, torch.device("cuda", 0)) if dev == "cuda" else TPGroup())
    assert eng.states is not None and not eng.blocks.prefix_caching
    prompts = [tokens(n, cfg["vocab"], 30 + n) for n in (50, 3, 29)]
    res = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True))
    # the GPU sampler holds a logits row as bf16 (steps of 1/32 between 4 and 8), whatever the model's dtype
    slack = 1e-3 if target == CPU else (0.07 if target[1] == "float32" else 0.15)
    for p, (out, _text, reason) in zip(prompts, res):
        assert len(out) == 12 and reason == "length"
        lg = O.forward(cfg, W, p + out)
        for k, t in enumerate(out):
            row = lg[len(p) + k - 1]
            assert row[t] >= row.max() - slack, (k, t, int(row.argmax()))
    assert eng.states.num_free() == 4 and eng.blocks.num_free() == eng.blocks.num_blocks


@pytest.mark.gpu
def test_graph_decode_matches_eager_gpu(tmp_path):
    """Decode-only steps replay a captured hipGraph (state slots and block tables staged per step): same
    greedy tokens as the eager engine, and argmaxes of the oracle."""
    cfg = base_config()
    W = O.make_weights(cfg, seed=23)
    path = O.save_checkpoint(str(tmp_path / "gd"), cfg, W)
    prompts = [tokens(n, cfg["vocab"], 40 + n) for n in (37, 5, 21, 2, 30)]
    sp = SamplingParams(temperature=0.0, max_tokens=20, ignore_eos=True)
    outs = []
    for eager in (True, False):
        ecfg = EngineConfig(model=path, dtype="bfloat16", device="cuda", max_num_seqs=4, max_num_batched_tokens=64,
                            num_kv_blocks=64, max_model_len=128, enforce_eager=eager)
        eng = LLMEngine(ecfg, tp=TPGroup(0, 1, None, torch.device("cuda", 0)))
        assert eng.runner.use_graphs != eager
        outs.append([r[0] for r in eng.generate(prompts, sp)])
        if not eager:
            assert eng.runner.stats["graph_steps"] > 0
    for p, out in zip(prompts, outs[1]):
        lg = O.forward(cfg, W, p + out)
        for k, t in enumerate(out):
            row = lg[len(p) + k - 1]
            assert row[t] >= row.max() - 0.15, (k, t, int(row.argmax()))
    same = sum(a == b for a, b in zip(outs[0], outs[1]))
    assert same >= len(prompts) - 1, (outs[0], outs[1])  # bf16 near-ties may flip one continuation


def test_preset_and_cli_model_resolution(tmp_path):
    from hipserve.config import resolve_model_config
    from hipserve.models.registry import model_class

    cfg = base_config()
    path = O.save_checkpoint(str(tmp_path / "c"), cfg, O.make_weights(cfg, seed=1))
    m = resolve_model_config(path)
    assert isinstance(m, FikizenConfig) and model_class(m).__name__ == "FikizenModel"
    assert isinstance(resolve_model_config("tiny-fikizen"), FikizenConfig)
