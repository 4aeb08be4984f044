"""The Kesirax layer-list decoder against the plain oracle of tests/kesirax_oracle.py: every
mechanism alone, and the engine (paged latent cache, state slots, batching, scheduler) against
whole-sequence oracle logits: prefill vs token-by-token decoding, prompt portions down to two
tokens, unequal requests in one batch, freed pages and slots used again, window edges, far
keys across page borders, first tokens, long decoding, odd sizes, greedy generation.
The same tests run on the CPU (reference ops) and, marked gpu, on the HIP kernels in bf16 and fp32."""
import pytest
import torch

from hipserve.config import EngineConfig, HybridConfig
from hipserve.engine.llm_engine import LLMEngine
from hipserve.engine.request import SamplingParams
from hipserve.engine.trace import TraceSession, build_engine
from hipserve.models.llama import AttnMeta
from hipserve.models.mixers import LatentAttention, MinGRU, TableMoE
from hipserve.ops import get_ops
from hipserve.parallel.comm import TPGroup

from . import kesirax_oracle as O

CPU = ("cpu", "float32")
TARGETS = [pytest.param(CPU, id="cpu-f32"),
           pytest.param(("cuda", "float32"), id="gpu-f32", marks=pytest.mark.gpu),
           pytest.param(("cuda", "bfloat16"), id="gpu-bf16", marks=pytest.mark.gpu)]
TOL = {"float32": 2e-4, "bfloat16": 6e-2}


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
    f = O.moe()
    layers = [O.attn_layer(mlp=f), O.gru_layer(mlp=f), O.gru_layer(width=40, mlp=f), O.attn_layer(window=9, mlp=f)]
    return O.make_config(layers, loop=(1, 3, 2), **kw)


def session(tmp_path, cfg, W, target, max_tokens=512, name="m"):
    path = O.save_checkpoint(str(tmp_path / name), cfg, W)
    eng = build_engine(path, target[1], max_tokens, target[0])
    if target[0] == "cuda":  # the HIP kernels are the path that runs
        assert eng.runner.ops.name == "hip" and hasattr(torch.ops.hipserve_seq, "latent_attention")
    return TraceSession(eng)


def replay(sess, steps):
    """steps: list of [(id, tokens, want, ends)] -> {(id, absolute position): logits row}."""
    out, at = {}, {}
    for n, step in enumerate(steps):
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
    rows = sorted(p for i, p in got if i == rid)
    assert rows == list(range(ref.shape[0]))
    err = rel_err(torch.stack([torch.as_tensor(got[(rid, p)]) for p in rows]), ref)
    assert err < tol, err


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


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("shape", [dict(), dict(heads=5, dim=16, rot_dim=8, vdim=12, q_rank=20, kv_rank=72, window=0),
                                   dict(heads=1, rot_dim=8, rot_dims=4, window=3), dict(heads=18, window=70),
                                   dict(heads=3, rot_dim=64, kv_rank=1024, window=11), dict(heads=70, kv_rank=264)])
def test_latent_attention_alone(target, shape):
    dev, dt = torch.device(target[0]), getattr(torch, target[1])
    l = O.attn_layer(**shape)
    cfg = O.make_config([l], width=24)
    W = O.make_weights(cfg, seed=3)
    T = 90
    h = torch.randn(T, 24, generator=torch.Generator().manual_seed(1)).bfloat16().float()
    want = O.latent_attention(h, W, "l0.mix.", l["mixer"], 1e-6)
    spec = HybridConfig.from_dict(cfg).layers[0].mixer
    mix = LatentAttention(spec, 24, 1e-6, dev, dt, get_ops(dev))
    mix.load(lambda k: W[k], "l0.mix.")
    meta, nblk = one_seq_meta(T, dev)
    cache = torch.zeros(mix.cache_shape(nblk, 4), device=dev, dtype=dt)
    got = mix.forward(h.to(dev, dt), meta, cache)
    assert rel_err(got, want) < TOL[target[1]]
    # the same rows in two portions and then one token alone, from the cache the first portion left
    cache.zero_()
    parts = []
    for a, b in ((0, 37), (37, T - 1), (T - 1, T)):
        m2, _ = one_seq_meta(b - a, dev, start=a)
        parts.append(mix.forward(h[a:b].to(dev, dt), m2, cache))
    assert rel_err(torch.cat(parts), want) < TOL[target[1]]


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("width", [24, 100])
def test_mingru_alone(target, width):
    dev, dt = torch.device(target[0]), getattr(torch, target[1])
    l = O.gru_layer(width=width)
    cfg = O.make_config([l], width=24)
    W = O.make_weights(cfg, seed=5)
    T = 150
    h = torch.randn(T, 24, generator=torch.Generator().manual_seed(2)).bfloat16().float()
    want, last = O.mingru(h, W, "l0.mix.", l["mixer"])
    mix = MinGRU(HybridConfig.from_dict(cfg).layers[0].mixer, 24, 1e-6, dev, dt, get_ops(dev))
    mix.load(lambda k: W[k], "l0.mix.")
    state = torch.full(mix.state_shape(3), 7.0, device=dev)  # a dirty slot: position 0 must start from zero
    parts = []
    for a, b in ((0, 70), (70, 72), (72, 73), (73, T)):  # long and short segments, one token alone
        meta, _ = one_seq_meta(b - a, dev, start=a, slot=1)
        parts.append(mix.forward(h[a:b].to(dev, dt), meta, state))
    assert rel_err(torch.cat(parts), want) < TOL[target[1]]
    assert rel_err(state[1], last) < TOL[target[1]]
    assert bool((state[0] == 7.0).all()) and bool((state[2] == 7.0).all())


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("top,experts,ff", [(1, 3, 12), (2, 4, 20), (3, 5, 70), (2, 130, 8)])
def test_table_moe_and_residual_update_alone(target, top, experts, ff):
    dev, dt = torch.device(target[0]), getattr(torch, target[1])
    f = O.moe(experts=experts, top=top, ff=ff)
    cfg = O.make_config([O.gru_layer(mlp=f)], width=40, groups=5)
    W = O.make_weights(cfg, seed=7)
    T = 77
    toks = tokens(T, cfg["vocab"], 4)
    g = torch.Generator().manual_seed(3)
    h = torch.randn(T, 40, generator=g).bfloat16().float()
    x = torch.randn(T, 40, generator=g)
    mixo = torch.randn(T, 40, generator=g).bfloat16().float()
    extra = torch.randn(T, 40, generator=g).bfloat16().float()
    ff_want = O.table_moe(h, toks, W, "l0.mlp.", f)
    x_want = x + mixo * W["l0.ls1"] + ff_want * W["l0.ls2"] + extra
    h_want = O.group_rms(x_want, W["l0.norm1"], 5, 1e-6)
    ops = get_ops(dev)
    moe = TableMoE(HybridConfig.from_dict(cfg).layers[0].mlp, 40, cfg["vocab"], dev, dt, ops)
    moe.load(lambda k: W[k], "l0.mlp.")
    y, pair_slot = moe.forward(h.to(dev, dt), torch.tensor(toks, device=dev))
    res = x.to(dev).clone()
    out = torch.empty(T, 40, device=dev, dtype=dt)
    ops.scaled_add_group_rmsnorm(out, res, W["l0.norm1"].to(dev), 5, 1e-6, mixo.to(dev, dt), W["l0.ls1"].to(dev),
                                 y, pair_slot, top, W["l0.ls2"].to(dev), extra=extra.to(dev, dt))
    assert rel_err(res, x_want) < TOL[target[1]]
    assert rel_err(out, h_want) < TOL[target[1]]


# ---------------------------------------------------------------- the engine against whole-sequence logits
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
    for got, want in zip(model.capture, streams):                                    # the stream after every layer run
        assert rel_err(got, want) < TOL[target[1]]
    assert len(model.capture) == len(streams) == len(O.layer_runs(cfg)) == 6
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
def test_window_edges_matter_and_are_right(tmp_path, target):
    """With windows of 4 and 5 every key weighs enough that a window one token too long or short
    moves the logits far beyond the tolerance; the engine must agree with the right one."""
    f = O.moe(top=1)
    cfg = O.make_config([O.attn_layer(window=4, mlp=f), O.attn_layer(window=5, scale=1.5, mlp=f)], groups=1)
    W = O.make_weights(cfg, seed=14)
    toks = tokens(40, cfg["vocab"], 3)
    ref = O.forward(cfg, W, toks)
    for delta in (-1, 1):
        other = O.make_config([O.attn_layer(window=4 + delta, mlp=f), O.attn_layer(window=5 + delta, scale=1.5, mlp=f)],
                              groups=1)
        assert rel_err(O.forward(other, W, toks)[8:], ref[8:]) > 50 * TOL[target[1]] or target[1] == "bfloat16"
        assert rel_err(O.forward(other, W, toks)[8:], ref[8:]) > 0.05
    sess = session(tmp_path, cfg, W, target)
    check_all(replay(sess, portions(toks, [40])), "a", ref, TOL[target[1]])           # edges inside a prompt
    check_all(replay(sess, portions(toks, [6, 3, 2, 5])), "a", ref, TOL[target[1]])   # across portions and decoded


@pytest.mark.parametrize("target", TARGETS)
def test_far_key_across_pages(tmp_path, target):
    """A sharp softmax (large scale) and a window longer than the prompt: most of the weight of a
    late query sits on single keys hundreds of tokens back, in other pages of the cache. (bf16 runs a
    less sharp softmax: at scale 6 the rounding of the scores alone moves the weights.)"""
    sc, gain = (6.0, 1.5) if target[1] == "float32" else (1.0, 1.0)
    cfg = O.make_config([O.attn_layer(window=1000, scale=sc, heads=2), O.attn_layer(window=0, scale=sc, heads=2)],
                        groups=1)
    W = O.make_weights(cfg, seed=15, gain=gain)
    toks = tokens(330, cfg["vocab"], 4)
    ref = O.forward(cfg, W, toks)
    near = O.make_config([O.attn_layer(window=200, scale=sc, heads=2), O.attn_layer(window=200, scale=sc, heads=2)],
                         groups=1)
    assert rel_err(O.forward(near, W, toks)[300:], ref[300:]) > 0.05   # the far keys carry the result
    sess = session(tmp_path, cfg, W, target)
    check_all(replay(sess, portions(toks, [330])), "a", ref, TOL[target[1]])
    check_all(replay(sess, portions(toks, [129, 64, 100])), "a", ref, TOL[target[1]])   # the rest decoded


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("variant", ["plain", "no_mlp_one_pass", "loop_tail", "three_passes"])
def test_other_sizes(tmp_path, target, variant):
    f1, f3 = O.moe(experts=2, top=1, ff=8), O.moe(experts=6, top=3, ff=36)
    if variant == "plain":          # one group, one expert per token, a window longer than the sequence
        cfg = O.make_config([O.attn_layer(heads=1, window=64, mlp=f1)], width=16, vocab=50, groups=1, logit_scale=1.0)
    elif variant == "no_mlp_one_pass":
        cfg = O.make_config([O.gru_layer(width=8), O.attn_layer(heads=7, dim=4, rot_dim=8, rot_dims=4, vdim=20,
                                                                 q_rank=5, kv_rank=24, window=7)],
                            width=48, loop=(0, 1, 1), groups=3)
    elif variant == "loop_tail":    # the loop covers the last layers, a recurrent layer inside it
        cfg = O.make_config([O.attn_layer(mlp=f3), O.gru_layer(mlp=f1), O.attn_layer(window=3, mlp=f3)],
                            width=36, loop=(1, 3, 2), groups=4, logit_scale=2.0)
    else:
        cfg = O.make_config([O.gru_layer(width=70, mlp=f3), O.attn_layer(kv_rank=72, vdim=4, mlp=None)],
                            width=24, loop=(0, 2, 3), groups=8)
    W = O.make_weights(cfg, seed=16)
    toks = tokens(45, cfg["vocab"], 5)
    ref = O.forward(cfg, W, toks)
    sess = session(tmp_path, cfg, W, target)
    check_all(replay(sess, portions(toks, [45])), "a", ref, TOL[target[1]])
    check_all(replay(sess, portions(toks, [4, 9, 2, 13])), "a", ref, TOL[target[1]])


@pytest.mark.parametrize("target", TARGETS)
def test_greedy_generation_through_the_scheduler(tmp_path, target):
    """LLMEngine.generate: the scheduler's own chunked prefill (a 24-token budget), batching of three
    prompts of unequal length and the sampler; every generated token is an argmax of the oracle's
    logits over the tokens before it."""
    cfg = base_config()
    W = O.make_weights(cfg, seed=17)
    path = O.save_checkpoint(str(tmp_path / "g"), cfg, W)
    dev = target[0]
    ecfg = EngineConfig(model=path, dtype=target[1], device=dev, max_num_seqs=4, max_num_batched_tokens=24,
                        num_kv_blocks=64, max_model_len=256, enforce_eager=True)
    eng = LLMEngine(ecfg, tp=TPGroup(0, 1, None, torch.device("cuda", 0)) if dev == "cuda" else TPGroup())
    assert eng.states is not None and not eng.blocks.prefix_caching
    prompts = [tokens(n, cfg["vocab"], 30 + n) for n in (50, 3, 29)]
    res = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True))
    slack = 1e-3 if target[1] == "float32" else 0.15
    for p, (out, _text, reason) in zip(prompts, res):
        assert len(out) == 12 and reason == "length"
        lg = O.forward(cfg, W, p + out)
        for k, t in enumerate(out):
            row = lg[len(p) + k - 1]
            assert row[t] >= row.max() - slack, (k, t, int(row.argmax()))
    assert eng.states.num_free() == 4 and eng.blocks.num_free() == eng.blocks.num_blocks


@pytest.mark.gpu
def test_table_moe_large_batch_gpu():
    """bf16 batches with many rows per expert take the packed-layout grouped GEMM (squared ReLU in its
    epilogue); same result as the plain experts."""
    from hipserve.models import mixers

    dev = torch.device("cuda")
    f = O.moe(experts=2, top=1, ff=256)
    cfg = O.make_config([O.gru_layer(mlp=f)], width=256, vocab=64, groups=1)
    W = O.make_weights(cfg, seed=21)
    T = 640
    toks = tokens(T, 64, 9)
    h = torch.randn(T, 256, generator=torch.Generator().manual_seed(5)).bfloat16().float()
    want = O.table_moe(h, toks, W, "l0.mlp.", f)
    moe = TableMoE(HybridConfig.from_dict(cfg).layers[0].mlp, 256, 64, dev, torch.bfloat16, get_ops(dev))
    moe.load(lambda k: W[k], "l0.mlp.")
    assert moe._packed_ok(h.to(dev, torch.bfloat16), T)
    y, pair_slot = moe.forward(h.to(dev, torch.bfloat16), torch.tensor(toks, device=dev))
    assert moe.packed is not None
    got = y.float().index_select(0, pair_slot.long())
    assert rel_err(got, want) < TOL["bfloat16"]
    assert mixers.MOE_PACKED_MIN_PAIRS_PER_EXPERT * 2 <= T


@pytest.mark.gpu
def test_graph_decode_matches_eager_gpu(tmp_path):
    """Decode-only steps replay a captured hipGraph (state slots and block tables staged per step, the
    lookahead ids resolved on the device): same greedy tokens as the eager engine, and argmaxes of the oracle."""
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


@pytest.mark.gpu
@pytest.mark.parametrize("kv_rank,window", [(64, 300), (136, 0)])
def test_latent_attention_long_prompt_gpu(kv_rank, window):
    """A prompt portion with tens of thousands of (token, head) rows on the matrix-core kernel: many key
    tiles per row, two sequences of unequal length and interleaved pages in one step."""
    dev, dt = torch.device("cuda"), torch.bfloat16
    l = O.attn_layer(heads=16, dim=16, rot_dim=8, vdim=16, q_rank=24, kv_rank=kv_rank, window=window)
    cfg = O.make_config([l], width=32)
    W = O.make_weights(cfg, seed=31)
    n = (1500, 700)
    g = torch.Generator().manual_seed(7)
    hs = [torch.randn(k, 32, generator=g).bfloat16().float() for k in n]
    want = torch.cat([O.latent_attention(h, W, "l0.mix.", l["mixer"], 1e-6) for h in hs])
    mix = LatentAttention(HybridConfig.from_dict(cfg).layers[0].mixer, 32, 1e-6, dev, dt, get_ops(dev))
    mix.load(lambda k: W[k], "l0.mix.")
    bs, T = 16, sum(n)
    nb = [-(-k // bs) for k in n]
    bt = torch.zeros(2, max(nb), dtype=torch.int32)
    bt[0, :nb[0]] = torch.arange(nb[0], dtype=torch.int32) * 2 + 1     # interleaved pages
    bt[1, :nb[1]] = torch.arange(nb[1], dtype=torch.int32) * 2
    pos = torch.cat([torch.arange(k) for k in n])
    seq = torch.cat([torch.full((k,), i) for i, k in enumerate(n)])
    slots = bt.long()[seq, pos // bs] * bs + pos % bs
    meta = AttnMeta(num_prefill_tokens=T, num_decode=0, positions=pos.to(dev), slot_mapping=slots.to(dev),
                    seq_cu=torch.tensor([0, n[0], T], dtype=torch.int32, device=dev),
                    seq_ctx=torch.tensor(n, dtype=torch.int32, device=dev), seq_bt=bt.to(dev), max_q=max(n),
                    max_ctx=max(n))
    cache = torch.zeros(mix.cache_shape(2 * max(nb) + 2, bs), device=dev, dtype=dt)
    got = mix.forward(torch.cat(hs).to(dev, dt), meta, cache)
    assert rel_err(got, want) < TOL["bfloat16"]


def test_openai_server_and_cli_config(tmp_path):
    """The engine command line resolves a checkpoint folder of this design (model class by config.json) and
    the OpenAI server completes, streams and samples with penalties and logprobs on it."""
    import asyncio

    import aiohttp
    from aiohttp import web

    from hipserve.server.api_server import OpenAIServer
    from hipserve.server.async_engine import AsyncEngine
    from hipserve.server.cli import build_parser, config_from_args

    cfg = base_config()
    path = O.save_checkpoint(str(tmp_path / "srv"), cfg, O.make_weights(cfg, seed=41))
    a = build_parser().parse_args(["--model", path, "--served-model-name", "kx", "--device", "cpu", "--dtype", "float32",
                                   "--max-model-len", "256", "--max-num-seqs", "4", "--num-kv-blocks", "64",
                                   "--max-num-batched-tokens", "32"])
    ecfg = config_from_args(a)

    async def main():
        eng = LLMEngine(ecfg, tp=TPGroup())
        assert type(eng.runner.model).__name__ == "KesiraxModel" and eng.states is not None
        ae = AsyncEngine(eng)
        ae.start(asyncio.get_running_loop())
        runner = web.AppRunner(OpenAIServer(ae, "kx", eng.max_model_len).app())
        await runner.setup()
        site = web.TCPSite(runner, "127.0.0.1", 0)
        await site.start()
        port = site._server.sockets[0].getsockname()[1]
        try:
            async with aiohttp.ClientSession() as s:
                body = {"model": "kx", "prompt": [5, 9, 33, 70, 2, 41] * 9, "max_tokens": 6, "temperature": 0.7,
                        "top_p": 0.9, "seed": 3, "presence_penalty": 0.5, "logprobs": 2}
                async with s.post(f"http://127.0.0.1:{port}/v1/completions", json=body) as r:
                    assert r.status == 200
                    d = await r.json()
                    assert d["usage"]["completion_tokens"] == 6 and d["usage"]["prompt_tokens"] == 54
                async with s.post(f"http://127.0.0.1:{port}/v1/completions", json=body) as r:
                    assert (await r.json())["choices"][0]["text"] == d["choices"][0]["text"]   # seeded: repeatable
        finally:
            await runner.cleanup()
            ae.stop() if hasattr(ae, "stop") else None

    asyncio.run(main())


def test_preemption_recomputes_state(tmp_path):
    """A cache pool too small for all running requests: the scheduler preempts (blocks and state slot freed,
    recomputed later from position 0 in whichever slot is free) and the outputs stay the oracle's argmaxes."""
    cfg = base_config()
    W = O.make_weights(cfg, seed=43)
    path = O.save_checkpoint(str(tmp_path / "pre"), cfg, W)
    ecfg = EngineConfig(model=path, dtype="float32", device="cpu", max_num_seqs=4, max_num_batched_tokens=32,
                        num_kv_blocks=13, max_model_len=128, enforce_eager=True)
    eng = LLMEngine(ecfg, tp=TPGroup())
    prompts = [tokens(n, cfg["vocab"], 60 + n) for n in (40, 33, 45, 38)]
    res = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=24, ignore_eos=True))
    assert eng.scheduler.num_preemptions > 0
    for p, (out, _text, reason) in zip(prompts, res):
        assert len(out) == 24 and reason == "length"
        lg = O.forward(cfg, W, p + out)
        for k, t in enumerate(out):
            row = lg[len(p) + k - 1]
            assert row[t] >= row.max() - 1e-3, (k, t, int(row.argmax()))
    assert eng.states.num_free() == 4 and eng.blocks.num_free() == eng.blocks.num_blocks


def random_config(seed):
    """A random small model: sizes, layer order, loop, windows and constants drawn per seed."""
    import random

    r = random.Random(seed)
    groups = r.choice([1, 2, 3, 4])
    width = groups * r.choice([8, 12, 20])
    vocab = r.choice([37, 64, 101])

    def mlp():
        if r.random() < 0.2:
            return None
        e = r.choice([1, 2, 3, 5, 6])
        return O.moe(experts=e, top=r.randint(1, min(e, 3)), ff=r.choice([4, 10, 24, 33]))

    layers = []
    for _ in range(r.randint(2, 5)):
        if r.random() < 0.5:
            layers.append(O.gru_layer(width=r.choice([8, 36, 70, 130]), mlp=mlp()))
        else:
            rot = r.choice([2, 4, 8, 16])
            layers.append(O.attn_layer(heads=r.randint(1, 9), dim=r.choice([4, 8, 16, 24]), rot_dim=rot,
                                       rot_dims=r.choice([rot, rot, max(2, rot // 2)]), vdim=r.choice([4, 8, 20]),
                                       q_rank=r.choice([6, 16, 28]), kv_rank=r.choice([8, 24, 40, 72]),
                                       window=r.choice([0, 2, 5, 17, 64]), base=r.choice([10.0, 1e4, 5e5]),
                                       scale=r.choice([None, 0.3, 0.05]), mlp=mlp()))
    a = r.randint(0, len(layers) - 1)
    b = r.randint(a, len(layers))
    return O.make_config(layers, width=width, vocab=vocab, loop=(a, b, r.randint(1, 3)), groups=groups,
                         logit_scale=r.choice([0.25, 1.0, 3.0]), eps=r.choice([1e-6, 1e-5]))


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("seed", range(8))
def test_random_models(tmp_path, target, seed):
    """Random sizes and layer orders: whole prompts, random portions with decoded tails, and two requests
    interleaved in one batch, against whole-sequence oracle logits."""
    import random

    cfg = random_config(seed)
    W = O.make_weights(cfg, seed=100 + seed)
    r = random.Random(1000 + seed)
    ta, tb = tokens(r.randint(30, 60), cfg["vocab"], 200 + seed), tokens(r.randint(3, 40), cfg["vocab"], 300 + seed)
    ra, rb = O.forward(cfg, W, ta), O.forward(cfg, W, tb)
    sess = session(tmp_path, cfg, W, target, max_tokens=256)
    check_all(replay(sess, portions(ta, [len(ta)])), "a", ra, TOL[target[1]])
    check_all(replay(sess, portions(ta, [r.randint(2, 9) for _ in range(5)])), "a", ra, TOL[target[1]])
    steps, pa, pb = [], 0, 0
    while pa < len(ta) or pb < len(tb):
        step = []
        for rid, t, p in (("a", ta, pa), ("b", tb, pb)):
            if p < len(t) and r.random() < 0.8:
                n = min(r.choice([1, 1, 2, 3, 7]), len(t) - p)
                step.append((rid, t[p:p + n], list(range(n)), p + n == len(t)))
                if rid == "a":
                    pa += n
                else:
                    pb += n
        if step:
            steps.append(step)
    got = replay(sess, steps)
    check_all(got, "a", ra, TOL[target[1]])
    check_all(got, "b", rb, TOL[target[1]])
