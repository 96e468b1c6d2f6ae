"""Pafivik through the engine against the plain implementation (tests/plain/pafivik_plain.py): each mechanism alone,
every way of cutting the work, first tokens, far tokens, long decoding, slots and pages used again, other sizes,
generation through the scheduler.  Backend "host" runs the engine's own code on the CPU with the kernels' plain
references in their place; backend "gpu" runs the HIP kernels."""
import copy
import json
import os

import pytest
import torch

import replay_util as U
from conftest import seeded_tokens
from plain import pafivik_plain as plain


# ----------------------------------------------------------------------------------------------------------------
# configurations: none has the sizes of any model that is shipped anywhere; each differs from the others in every size
# ----------------------------------------------------------------------------------------------------------------
def lightning(heads=2, dim=16, vdim=8, decay=None):
    return dict(type="lightning", mixer=dict(heads=heads, dim=dim, vdim=vdim,
                                             decay=decay or [0.5 + 0.49 * (h + 1) / heads for h in range(heads)]))


def delta(heads=4, kv_heads=2, dim=8, vdim=16, conv=3, decay_rank=6, gate_rank=5):
    return dict(type="channel_delta", mixer=dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, conv=conv, decay_rank=decay_rank,
                                                 gate_rank=gate_rank))


def attention(heads=4, kv_heads=2, dim=16, vdim=16, dims=None, base=10000.0, scale=None, rot=True):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale if scale is not None else dim ** -0.5)
    if rot:
        m["rot"] = dict(base=base, dims=dim if dims is None else dims)
    return dict(type="attention", mixer=m)


def dense(ff=40):
    return dict(kind="dense", ff=ff)


def moe(ff=24, experts=4, top=2, shared=16):
    m = dict(kind="moe", expert=dict(ff=ff), router=dict(experts=experts, top=top))
    if shared:
        m["shared"] = dict(ff=shared)
    return m


def config(layers, width=32, vocab=97, eps=1e-5, mult=0.4, scale=2.0):
    return dict(architecture="Pafivik", vocab=vocab, width=width, norm=dict(eps=eps), embedding=dict(scale=scale), residual_mult=mult,
                layers=layers)


def with_mlp(layer, mlp):
    return dict(layer, mlp=mlp)


# every mixer and both feed-forwards; grouped heads in the delta rule and in the attention; part of a head turned; a layer
# without a feed-forward
CFG_P = config([with_mlp(lightning(2, 16, 8), dense(40)), with_mlp(delta(4, 2, 8, 16, 3), moe(24, 4, 2, 16)),
                with_mlp(attention(4, 2, 16, 16, dims=8), dense(24)), with_mlp(delta(2, 2, 16, 8, 2, 4, 7), None)],
               width=32, vocab=97)
# other sizes: one head; values wider and narrower than keys; a head size that no 16 divides; one tap; an attention without
# turned dimensions; one expert of three without a shared one, all five experts with one; another order of layers
CFG_Q = config([with_mlp(attention(3, 1, 24, 40, dims=24, base=300.0, scale=0.31), moe(16, 3, 1, None)),
                with_mlp(lightning(1, 40, 24, [0.97]), None),
                with_mlp(delta(1, 1, 40, 8, 1, 3, 9), dense(20)),
                with_mlp(attention(2, 2, 8, 4, rot=False), moe(40, 5, 5, 8)),
                with_mlp(lightning(3, 8, 16), dense(56))],
               width=48, vocab=131, eps=1e-6, mult=1.0, scale=1.0)
# sizes that are multiples of nothing (the kernels' paths for single numbers): a width of 36, heads of 6 and 10, five taps
CFG_R = config([with_mlp(delta(2, 1, 6, 10, 5, 2, 3), moe(12, 2, 2, 20)), with_mlp(attention(2, 1, 10, 6, dims=4), dense(9)),
                with_mlp(lightning(2, 6, 10), moe(8, 6, 3, None))], width=36, vocab=61, mult=0.15, scale=5.0)
CONFIGS = {"P": (CFG_P, 31), "Q": (CFG_Q, 32), "R": (CFG_R, 33)}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    from denno_beta_amd.weights import write_model_folder
    made = {}

    def get(name, dtype="float32", cfg=None, seed=None, change=None):
        key = (name, dtype)
        if key not in made:
            c, s = CONFIGS[name] if cfg is None else (cfg, seed)
            d = str(tmp_path_factory.mktemp(f"pafivik{name}_{dtype}"))
            write_model_folder(d, c, s, dtype)
            if change is not None:
                from safetensors.torch import load_file, save_file
                path = os.path.join(d, "model.safetensors")
                stored = load_file(path)
                tensors = {k: v.float() for k, v in stored.items()}
                change(tensors)
                save_file({k: v.to(stored[k].dtype).contiguous() for k, v in tensors.items()}, path)
            made[key] = d
        return made[key]
    return get


def runner_for(folder, dtype, device, cache_tokens, max_live=4, page_size=16):
    from denno_beta_amd.config import EngineOptions
    from denno_beta_amd.engine import ModelRunner
    return ModelRunner.from_folder(folder, EngineOptions(dtype=dtype, device=device, page_size=page_size,
                                                         cache_tokens=cache_tokens, max_live=max_live))


_plain = {}


def plain_logits(folder, seq, streams=None):
    key = (folder, tuple(seq))
    if key not in _plain or streams is not None:
        from safetensors.torch import load_file
        with open(os.path.join(folder, "config.json")) as f:
            cfg = json.load(f)
        _plain[key] = plain.forward(cfg, load_file(os.path.join(folder, "model.safetensors")), seq, torch.float64, streams)
    return _plain[key]


def row_errors(got, want):
    """Per position: the root mean square of the difference (its mean taken off) over the spread of the wanted row."""
    d = got.double() - want.double()
    d = d - d.mean(dim=1, keepdim=True)
    return torch.sqrt((d * d).mean(dim=1)) / want.double().std(dim=1)


# bfloat16, in models 32 to 48 wide: a typical row is off by 0.01 of its spread and a row in a few hundred by several times
# that, so one row in fifty may pass the bound, none by more than two and a half times; a fault moves rows by 0.2 and more
BOUND = {"float32": 2e-5, "bfloat16": 0.06}
BF16_OVER, BF16_WORST = 0.02, 0.15
# bfloat16: a router's choice between two experts whose scores are close may fall the other way under rounding, which
# moves that row, and through states and keys later rows, by as much as a fault would.  The bfloat16 models of these
# tests therefore let every token use all its experts (`all_experts`): the same kernels run, no choice can turn, and
# every row keeps the bound.  The choice itself is tested in 32-bit.


def assert_rows(got, want, dtype, what, bound=None):
    e = row_errors(got, want)
    b = bound or BOUND[dtype]
    if dtype == "bfloat16" and bound is None:
        over = int((e > b).sum())
        assert over <= max(1, BF16_OVER * len(e)) and e.max() <= BF16_WORST, (
            f"{what}: {over} of {len(e)} positions are off by more than {b} of their row's spread, the worst (position "
            f"{int(e.argmax())}) by {e.max().item():.3g}")
        return
    assert bool((e <= b).all()), f"{what}: position {int(e.argmax())} is off by {e.max().item():.3g} of its row's spread (bound {b})"


def seqs_for(cfg, lengths, seed=3):
    return [seeded_tokens(seed + i, n, cfg["vocab"]) for i, n in enumerate(lengths)]


def all_experts(cfg):
    cfg = copy.deepcopy(cfg)
    for layer in cfg["layers"]:
        if layer.get("mlp") and layer["mlp"]["kind"] == "moe":
            layer["mlp"]["router"]["top"] = layer["mlp"]["router"]["experts"]
    return cfg


# ----------------------------------------------------------------------------------------------------------------
# the plain implementation against itself: what its pieces must satisfy whatever the weights
# ----------------------------------------------------------------------------------------------------------------
def test_plain_pieces():
    g = torch.Generator().manual_seed(0)
    z = torch.randn(50, generator=g, dtype=torch.float64) * 3
    pq = torch.tensor([0.3, -0.2], dtype=torch.float64)
    y = plain.xielu(z, pq)
    a, b = torch.log1p(torch.exp(pq[0])), 0.5 + torch.log1p(torch.exp(pq[1]))
    for zi, yi in zip(z.tolist(), y.tolist()):
        want = a * zi * zi + zi / 2 if zi > 0 else b * (torch.exp(torch.tensor(zi, dtype=torch.float64)) - 1 - zi) + zi / 2
        assert abs(yi - float(want)) < 1e-12
    # both branches meet at 0 with the same slope
    eps = torch.tensor([-1e-7, 1e-7], dtype=torch.float64)
    d = plain.xielu(eps, pq)
    assert abs(float(d[1] - d[0]) / 2e-7 - 0.5) < 1e-6
    # the delta rule with beta = 1 and no decay stores a value under a unit key exactly: reading with that key returns it
    H, dk, dv = 1, 4, 3
    k = torch.nn.functional.normalize(torch.randn(dk, generator=g, dtype=torch.float64), dim=0)
    v = torch.randn(dv, generator=g, dtype=torch.float64)
    S = torch.randn(dk, dv, generator=g, dtype=torch.float64)
    S = S + torch.outer(k, 1.0 * (v - S.T @ k))
    assert torch.allclose(S.T @ k, v, atol=1e-12)
    # the convolution's last column weighs the token itself
    x = torch.randn(5, 2, generator=g, dtype=torch.float64)
    w = torch.zeros(2, 3, dtype=torch.float64)
    w[:, 2] = 1.0
    assert torch.equal(plain.causal_taps(x, w), x)
    w = torch.zeros(2, 3, dtype=torch.float64)
    w[:, 0] = 1.0
    assert torch.equal(plain.causal_taps(x, w)[2:], x[:3]) and float(plain.causal_taps(x, w)[:2].abs().sum()) == 0.0


# ----------------------------------------------------------------------------------------------------------------
# each mechanism alone
# ----------------------------------------------------------------------------------------------------------------
ALONE = {
    "lightning": [with_mlp(lightning(3, 8, 12), None)],
    "lightning_one_head": [with_mlp(lightning(1, 24, 8, [0.9]), None)],
    "delta": [with_mlp(delta(2, 2, 8, 12, 4), None)],
    "delta_shared_keys": [with_mlp(delta(6, 2, 8, 4, 2), None)],
    "delta_one_tap": [with_mlp(delta(1, 1, 20, 12, 1), None)],
    "attention": [with_mlp(attention(4, 2, 8, 8), None)],
    "attention_wide_values": [with_mlp(attention(2, 1, 12, 20, dims=6), None)],
    "attention_narrow_values": [with_mlp(attention(3, 3, 16, 8, rot=False), None)],
    "dense": [with_mlp(lightning(1, 8, 8), dense(28))],
    "experts": [with_mlp(lightning(1, 8, 8), moe(12, 6, 3, None))],
    "experts_with_shared": [with_mlp(lightning(1, 8, 8), moe(12, 5, 1, 20))],
    "two_layers_averaged": [with_mlp(lightning(2, 8, 8), dense(12)), with_mlp(attention(2, 2, 8, 8), None)],
}


@pytest.mark.parametrize("what", sorted(ALONE))
def test_each_mechanism_alone(backend, folders, what):
    cfg = config(ALONE[what], width=24, vocab=53, mult=0.7, scale=1.5)
    folder = folders(f"alone_{what}", "float32", cfg, 5)
    seq = seqs_for(cfg, [29])[0]
    streams = []
    want = plain_logits(folder, seq, streams)
    r = runner_for(folder, "float32", backend, 64)
    got = U.replay(r, U.whole_trace([seq]))["r0"]
    assert_rows(got, want, "float32", what)


def test_what_the_model_fixes_matters(folders):
    """The constants and orders that the plain model is built from change its logits: a test against it would see them."""
    from safetensors.torch import load_file
    cfg = CFG_P
    folder = folders("P", "float32")
    W = load_file(os.path.join(folder, "model.safetensors"))
    seq = seqs_for(cfg, [25])[0]
    want = plain_logits(folder, seq)
    for change in ("mult", "scale", "dwa", "ls", "act", "sg", "decay"):
        other, weights = copy.deepcopy(cfg), dict(W)
        if change == "mult":
            other["residual_mult"] = 1.0
        elif change == "scale":
            other["embedding"]["scale"] = 1.0
        elif change == "decay":
            other["layers"][0]["mixer"]["decay"] = [1.0, 1.0]
        elif change == "dwa":
            weights["l1.dwa"] = torch.tensor([0.0, 0.0, 1.0])
        elif change == "ls":
            weights["l0.ls1"] = torch.ones_like(W["l0.ls1"])
        elif change == "act":
            weights["l0.mlp.act"] = torch.zeros(2)
        else:
            weights["l1.mlp.shared.sg"] = torch.zeros_like(W["l1.mlp.shared.sg"])
        assert row_errors(plain.forward(other, weights, seq, torch.float64), want).max() > 1e-3, change


# ----------------------------------------------------------------------------------------------------------------
# every way of cutting the work
# ----------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("name,dtype", [("P", "float32"), ("Q", "float32"), ("R", "float32"), ("P", "bfloat16"), ("Q", "bfloat16"),
                                        ("R", "bfloat16")])
def test_every_cutting_matches_the_plain_implementation(backend, folders, name, dtype):
    cfg = CONFIGS[name][0]
    lengths = (1, 2, 37, 70, 23) if backend == "cpu" else (1, 2, 37, 150, 23, 301)
    if dtype == "bfloat16":
        cfg = all_experts(cfg)
    folder = folders(name, dtype, cfg, CONFIGS[name][1])
    seqs = seqs_for(cfg, lengths)
    want = [plain_logits(folder, s) for s in seqs]
    traces = {"whole": U.whole_trace(seqs), "tail": U.tail_decode_trace(seqs, 20),
              "chunks": U.chunk_trace(seqs, sizes=(2, 3, 5, 17, 2, 16, 7, 32, 2, 31)), "mixed": U.mixed_trace(seqs, seed=5, max_live=3)}
    results = {}
    for kind, steps in traces.items():
        tokens = U.max_live_tokens(steps)
        r = runner_for(folder, dtype, backend, cache_tokens=tokens, max_live=3)
        got = U.replay(r, steps)
        r.cache.manager.check()
        assert r.cache.manager.live() == 0
        if kind == "mixed":
            assert r.cache.manager.reuse_count(r.cache.paged_groups()[0]) > 0, "the pool was too large: no page was used again"
        for i in range(len(seqs)):
            assert_rows(got[f"r{i}"], want[i], dtype, f"{name} {dtype} {kind} request {i}")
        results[kind] = got
    for kind in ("tail", "chunks", "mixed"):
        for i in range(len(seqs)):
            a, b = results["whole"][f"r{i}"], results[kind][f"r{i}"]
            assert_rows(b, a, dtype, f"{name} {dtype} {kind} against whole, request {i}", 1e-5 if dtype == "float32" else None)


def test_the_stream_after_every_layer(backend, folders):
    """Layer by layer: what goes on behind each layer (after the average over depth), read from the engine's own buffers."""
    cfg = CONFIGS["P"][0]
    folder = folders("P", "float32")
    seq = seqs_for(cfg, [19], seed=11)[0]
    streams = []
    plain_logits(folder, seq, streams)
    from denno_beta_amd.kernels import ops
    r = runner_for(folder, "float32", backend, 64)
    seen = []
    real = ops.depth_mix

    def spy(hist, n, weights, out):
        res = real(hist, n, weights, out)
        seen.append(res.detach().cpu().clone())
        return res
    ops.depth_mix = spy
    try:
        U.replay(r, U.whole_trace([seq]))
    finally:
        ops.depth_mix = real
    assert len(seen) == len(cfg["layers"]) + 1          # (the first: the embedded rows on their way to layer 0)
    for i, want in enumerate(streams):
        d = (seen[i + 1].double() - want).abs().max() / want.abs().max()
        assert d < 2e-5, f"the stream behind layer {i} differs by {d:.3g} of its largest entry"


# ----------------------------------------------------------------------------------------------------------------
# far tokens: weights made so that losing one shows
# ----------------------------------------------------------------------------------------------------------------
MARKER = 7      # the token that the crafted layers look for


def _directions(tensors, seed):
    """Every token's row becomes a random vector of length about 1 plus 0.7 along a common direction u; the marker's row
    alone has a part along m (at right angles to u and to every other row)."""
    g = torch.Generator().manual_seed(seed)
    V, W = tensors["embed"].shape
    unit = lambda n: torch.nn.functional.normalize(torch.randn(n, generator=g), dim=0)   # noqa: E731
    u, m = unit(W), unit(W)
    m = torch.nn.functional.normalize(m - (m @ u) * u, dim=0)
    e = torch.randn(V, W, generator=g) / W ** 0.5
    e = e - torch.outer(e @ m, m) - torch.outer(e @ u, u)
    tensors["embed"] = e + 0.7 * u
    tensors["embed"][MARKER] += 2.0 * m
    tensors["l0.norm1"] = torch.ones_like(tensors["l0.norm1"])
    return u, m, g


def needle(tensors):
    """An attention whose first head looks for one token wherever it lies: every query points along d (made from the
    common direction u), the marker's key alone has a large part along d (made from m); d lies in the pair of
    dimensions that the position turns slowest.  A key that is lost, misplaced or read from a wrong page changes the
    rows after it as much as one head can."""
    u, m, g = _directions(tensors, 1)
    q, k = tensors["l0.mix.q"], tensors["l0.mix.k"]
    dk = k.shape[0]
    d = torch.zeros(dk)
    d[-2:] = torch.tensor([0.6, 0.8])
    q[:dk] = 8.0 * torch.outer(d, u)
    k[:dk] = 4.0 * torch.outer(d, m)
    tensors["l0.mix.q.b"].zero_(), tensors["l0.mix.k.b"].zero_()
    tensors["l0.mix.v"] = tensors["l0.mix.v"] * 20.0
    tensors["l0.mix.o"] = tensors["l0.mix.o"] * 20.0


def imprint(tensors):
    """Recurrent layers that keep what one token wrote.  In the lightning layer (decays 0.999 and 1) the marker's key is
    many times an ordinary one, so its product with its value stays a large part of the state; in the delta layer the
    decay is nearly one (A_log far below zero), beta is small for ordinary tokens and nearly one for the marker, whose
    value is large: what it wrote stays and is read by every later token.  A state that is lost, started anew or taken
    from another slot changes every later row."""
    u, m, g = _directions(tensors, 2)
    n = tensors["l0.mix.k"].shape[0]
    tensors["l0.mix.k"] = tensors["l0.mix.k"] + 3.0 * torch.outer(torch.rand(n, generator=g) + 0.5, m)
    tensors["l1.norm1"] = torch.ones_like(tensors["l1.norm1"])
    tensors["l1.mix.A_log"] = torch.full_like(tensors["l1.mix.A_log"], -9.0)
    H = tensors["l1.mix.b"].shape[0]
    tensors["l1.mix.b"] = torch.outer(torch.ones(H), -1.5 * u + 1.5 * m)
    nv = tensors["l1.mix.v"].shape[0]
    tensors["l1.mix.v"] = tensors["l1.mix.v"] + 4.0 * torch.outer(torch.rand(nv, generator=g) + 0.5, m)


FAR = {"attention": (config([with_mlp(attention(2, 1, 16, 16, dims=16, base=1e6), None), with_mlp(attention(2, 2, 8, 8), None)],
                            width=32, vocab=71, mult=1.5, scale=1.0), needle),
       "states": (config([with_mlp(lightning(2, 16, 16, [0.999, 1.0]), None), with_mlp(delta(2, 1, 16, 16, 3), None)], width=32, vocab=71,
                         mult=1.5, scale=1.0), imprint)}


@pytest.mark.parametrize("what", sorted(FAR))
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_far_tokens_count(backend, folders, what, dtype):
    cfg, change = FAR[what]
    n = 90 if backend == "cpu" else 400
    folder = folders(f"far_{what}", dtype, cfg, 9, change)
    ordinary = [t if t != MARKER else MARKER + 1 for t in seqs_for(cfg, [n], seed=40)[0]]
    # the marker at the first place, at a page's last and first place, and in the middle of one
    for at in (0, 15, 16, 37):
        seq = list(ordinary)
        seq[at] = MARKER
        want = plain_logits(folder, seq)
        # the test's own check: with an ordinary token there the last rows differ by far more than the bound allows
        without = plain_logits(folder, ordinary)
        assert row_errors(without[-8:], want[-8:]).min() > 0.15, "the marked token does not reach the last rows"
        for kind, steps in (("whole", U.whole_trace([seq])), ("tail", U.tail_decode_trace([seq], 40)),
                            ("chunks", U.chunk_trace([seq], sizes=(15, 2, 16, 33, 1, 17))),
                            ("pages", U.chunk_trace([seq], sizes=(16, 16, 32, 1, 15, 48)))):
            if at not in (0, 16) and kind in ("chunks", "pages") and backend == "cpu":
                continue          # (the host backend is slow)
            r = runner_for(folder, dtype, backend, U.max_live_tokens(steps))
            # (32-bit: these weights are large on purpose, and so are the sums' rounding errors)
            assert_rows(U.replay(r, steps)["r0"], want, dtype, f"far {what} {dtype} {kind}, the marker at {at}",
                        1e-4 if dtype == "float32" else None)


# ----------------------------------------------------------------------------------------------------------------
# the first tokens; slots given out again; a request beside others
# ----------------------------------------------------------------------------------------------------------------
def test_first_tokens_one_by_one(backend, folders):
    """Every token alone from the first: the convolutions' histories are shorter than their taps, the states start at
    zero, the first rows are averaged with the embedded rows only."""
    cfg = CONFIGS["R"][0]
    folder = folders("R", "float32")
    seq = seqs_for(cfg, [9], seed=77)[0]
    want = plain_logits(folder, seq)
    steps = U.tail_decode_trace([seq], 9)
    r = runner_for(folder, "float32", backend, 64)
    assert_rows(U.replay(r, steps)["r0"], want, "float32", "token by token from the first")


def test_a_slot_given_out_again_starts_from_nothing(backend, folders):
    cfg = CONFIGS["P"][0]
    folder = folders("P", "float32")
    a, b, c = seqs_for(cfg, [33, 21, 18], seed=90)
    r = runner_for(folder, "float32", backend, 64, max_live=1)
    steps = U.whole_trace([a]) + [dict(s, step=1 + i) for i, s in enumerate(U.chunk_trace([b], sizes=(5, 2, 9)))]
    for i, s in enumerate(steps[1:]):      # (other names than the first request's)
        s["entries"][0]["id"], s["end"] = "second", (["second"] if s["end"] else [])
    got = U.replay(r, steps)
    assert_rows(got["second"], plain_logits(folder, b), "float32", "the second request in the first one's slot")
    got = U.replay(r, [dict(U.whole_trace([c])[0], step=99)])
    assert_rows(got["r0"], plain_logits(folder, c), "float32", "the third")
    r.cache.manager.check()


def test_unequal_requests_together_equal_each_alone(backend, folders):
    cfg = CONFIGS["Q"][0]
    folder = folders("Q", "float32")
    seqs = seqs_for(cfg, [5, 40, 1, 17], seed=123)
    r = runner_for(folder, "float32", backend, 4 * 64)
    together = U.replay(r, [{"step": 0, "entries": [{"id": f"r{i}", "tokens": s, "want": list(range(len(s)))} for i, s in enumerate(seqs)],
                             "end": [f"r{i}" for i in range(len(seqs))]}])
    alone = U.replay(runner_for(folder, "float32", backend, 64), U.whole_trace(seqs))
    for i in range(len(seqs)):
        if backend == "cpu":     # (the host's library products sum in an order that depends on the batch)
            assert_rows(together[f"r{i}"], alone[f"r{i}"], "float32", f"request {i} beside the others", 1e-5)
        else:                    # every kernel sums a row in one order whatever else the step holds
            assert torch.equal(together[f"r{i}"], alone[f"r{i}"]), f"request {i}: 32-bit logits depend on the batch"


# ----------------------------------------------------------------------------------------------------------------
# generation through the engine's own entry point and scheduler
# ----------------------------------------------------------------------------------------------------------------
def test_greedy_generation_through_the_scheduler(backend, folders):
    from denno_beta_amd.config import EngineOptions
    from denno_beta_amd.engine import Engine, SamplingParams
    cfg = CONFIGS["P"][0]
    folder = folders("P", "float32")
    prompts = seqs_for(cfg, [3, 19, 11], seed=300)
    n_new = 10
    eng = Engine.from_folder(folder, EngineOptions(dtype="float32", device=backend, cache_tokens=4 * 64, max_live=2,
                                                   prefill_chunk=7, max_batch_tokens=16))
    got = eng.generate(prompts, SamplingParams(max_tokens=n_new, temperature=0.0))
    for p, g in zip(prompts, got):
        seq = list(p)
        for n, tok in enumerate(g):
            row = plain_logits(folder, seq)[-1]
            top = row.topk(2)
            if tok != int(top.indices[0]):
                assert float(top.values[0] - top.values[1]) < 1e-4 * float(row.std()), f"token {n} of {g}: the plain model says {int(top.indices[0])}"
            seq.append(tok)
        assert len(g) == n_new


# ----------------------------------------------------------------------------------------------------------------
# configuration and weights
# ----------------------------------------------------------------------------------------------------------------
def test_config_is_read_with_errors_that_name_the_key(folders):
    from denno_beta_amd.config import ConfigError, load_config, resolve_architecture
    from denno_beta_amd.models.pafivik import PafivikConfig
    assert resolve_architecture({"architecture": "Pafivik"}).config_cls is PafivikConfig
    for path, match in ((("layers", 1, "mixer", "kv_heads"), "kv_heads"), (("layers", 0, "mixer", "decay"), "decay"),
                        (("residual_mult",), "residual_mult"), (("embedding",), "embedding"), (("layers", 2, "mixer", "scale"), "scale"),
                        (("layers", 1, "mlp", "router"), "router")):
        bad = copy.deepcopy(CFG_P)
        d = bad
        for key in path[:-1]:
            d = d[key]
        del d[path[-1]]
        with pytest.raises(ConfigError, match=match):
            PafivikConfig.from_dict(bad)
    bad = copy.deepcopy(CFG_P)
    bad["layers"][0]["type"] = "something"
    with pytest.raises(ConfigError, match="type"):
        PafivikConfig.from_dict(bad)
    bad = copy.deepcopy(CFG_P)
    bad["layers"][2]["mixer"]["rot"]["dims"] = 18
    with pytest.raises(ConfigError, match="rot.dims"):
        PafivikConfig.from_dict(bad)
    # sizes that only the tensors give: the inner sizes of the small matrices come from the file, whatever config.json holds
    folder = folders("P", "float32")
    with open(os.path.join(folder, "config.json")) as f:
        stored = json.load(f)
    for key in ("decay_rank", "gate_rank"):
        del stored["layers"][1]["mixer"][key]
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(stored, f)
    _, cfg = load_config(folder)
    assert (cfg.layers[1]["mixer"]["decay_rank"], cfg.layers[1]["mixer"]["gate_rank"]) == (6, 5)
    assert (cfg.layers[3]["mixer"]["decay_rank"], cfg.layers[3]["mixer"]["gate_rank"]) == (4, 7)


def test_a_checkpoint_that_does_not_fit_is_reported_whole(folders, tmp_path):
    from safetensors.torch import load_file, save_file
    from denno_beta_amd.config import EngineOptions
    from denno_beta_amd.engine import ModelRunner
    from denno_beta_amd.weights import CheckpointError
    import shutil
    d = str(tmp_path / "m")
    shutil.copytree(folders("R", "float32"), d)
    tensors = load_file(os.path.join(d, "model.safetensors"))
    del tensors["l0.mlp.e1.up"]
    tensors["l2.dwa"] = tensors["l2.dwa"][:3].contiguous()
    tensors["stray"] = torch.zeros(3)
    save_file(tensors, os.path.join(d, "model.safetensors"))
    with pytest.raises(CheckpointError) as e:
        ModelRunner.from_folder(d, EngineOptions(dtype="float32", device="cpu", cache_tokens=64, max_live=1))
    assert "l0.mlp.e1.up" in e.value.missing and "stray" in e.value.unexpected and e.value.wrong_shape[0][0] == "l2.dwa"


# ----------------------------------------------------------------------------------------------------------------
# the command line and the trace runner as child processes; a long run of decoded tokens
# ----------------------------------------------------------------------------------------------------------------
def plain_greedy(folder, prompt, n):
    seq = list(prompt)
    for _ in range(n):
        seq.append(int(plain_logits(folder, seq)[-1].argmax()))
    return seq[len(prompt):]


@pytest.mark.gpu
def test_command_line_generates_what_the_plain_model_does(folders):
    import subprocess
    import sys
    from conftest import ROOT
    folder = folders("R", "float32")
    prompt = seqs_for(CONFIGS["R"][0], [7], seed=410)[0]
    want = plain_greedy(folder, prompt, 6)
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "denno"), "generate", folder, "--prompt-ids",
                          ",".join(map(str, prompt)), "--max-tokens", "6", "--temperature", "0", "--quant", "fp32", "--raw",
                          "--cache-tokens", "128"], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr
    assert [int(t) for t in out.stdout.strip().split(",")] == want


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_as_a_child_process(folders, tmp_path, dtype):
    """bin/trace_run on a mixed trace with four state slots: the files it writes against the plain implementation."""
    import subprocess
    from conftest import ROOT
    cfg = CONFIGS["P"][0] if dtype == "float32" else all_experts(CONFIGS["P"][0])
    folder = folders("P", dtype, cfg, CONFIGS["P"][1])
    seqs = seqs_for(cfg, [90, 3, 41, 17, 64, 29, 5], seed=500)
    steps = U.mixed_trace(seqs, seed=3, max_live=4)
    out = str(tmp_path / "out")
    p = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype, "--out", out, "--max-tokens",
                        str(U.max_live_tokens(steps))], input="\n".join(json.dumps(s) for s in steps) + "\n",
                       capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done ")] == [f"done {s['step']}" for s in steps]
    got = U.collect_files(out, steps, cfg["vocab"])
    for i, s in enumerate(seqs):
        assert_rows(got[f"r{i}"], plain_logits(folder, s), dtype, f"trace_run {dtype} request {i}")


def test_two_hundred_decoded_tokens(backend, folders):
    """A short prompt, then token after token for long: pages fill and new ones are taken, the states run on."""
    cfg = CONFIGS["P"][0]
    folder = folders("P", "float32")
    n = 60 if backend == "cpu" else 230
    seq = seqs_for(cfg, [n], seed=600)[0]
    steps = U.tail_decode_trace([seq], n - 4)
    r = runner_for(folder, "float32", backend, U.max_live_tokens(steps))
    assert_rows(U.replay(r, steps)["r0"], plain_logits(folder, seq), "float32", "long decoding")
