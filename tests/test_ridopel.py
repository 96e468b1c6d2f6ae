"""Ridopel through the engine against the plain implementation (tests/plain/ridopel_plain.py): each mixer alone,
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
from plain import ridopel_plain as plain


# ----------------------------------------------------------------------------------------------------------------
# configurations: none has the sizes of any model that is shipped anywhere; each differs from the others in every size
# ----------------------------------------------------------------------------------------------------------------
def latent(heads=2, dim=16, rot_dim=8, vdim=16, kv_rank=24, dims=None, base=10000.0, scale=None, keep=None):
    m = dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=kv_rank,
             scale=scale if scale is not None else (dim + rot_dim) ** -0.5, rot=dict(base=base, dims=rot_dim if dims is None else dims))
    if keep:
        m["keep"] = keep      # (what the cache holds: the latent, or every head's own keys and values)
    return dict(type="latent_attention", mixer=m)


def wkv(heads=2, dim=16, rank=8):
    return dict(type="wkv", mixer=dict(heads=heads, dim=dim, decay_rank=rank))


def hgrn2(heads=2, dim=16, vdim=8):
    return dict(type="hgrn2", mixer=dict(heads=heads, dim=dim, vdim=vdim))


def moe(ff=24, experts=4, top=2, limit=3.0):
    return dict(kind="moe", expert=dict(ff=ff, limit=limit), router=dict(experts=experts, top=top))


def config(layers, width=32, vocab=97, taps=3, loop=None, eps=1e-5, softcap=12.0):
    c = dict(architecture="Ridopel", vocab=vocab, width=width, norm=dict(eps=eps), layers=layers)
    if taps:
        c["canon"] = dict(taps=taps)
    if loop:
        c["loop"] = dict(zip(("start", "stop", "times"), loop))
    if softcap:
        c["logit_softcap"] = softcap
    return c


def with_mlp(layer, mlp):
    return dict(layer, mlp=mlp)


# three mixers in a loop that starts at the second layer; a layer without a feed-forward
CFG_P = config([with_mlp(wkv(2, 16, 8), moe(24, 4, 2)), with_mlp(latent(2, 16, 8, 16, 24), moe(24, 4, 2)),
                with_mlp(hgrn2(2, 16, 8), None), with_mlp(latent(2, 16, 8, 16, 24), moe(24, 4, 2))],
               width=32, vocab=97, taps=3, loop=(1, 3, 2))
# other sizes: one head, values wider than keys, fewer turned dimensions than rot_dim, a kept key that is no multiple of
# 16 (40 + 12), a latent attention that keeps every head's keys, four taps, one expert of three, all five experts, three
# passes over one layer, no soft cap
CFG_Q = config([with_mlp(hgrn2(3, 8, 24), moe(16, 3, 1, 1.5)), with_mlp(latent(1, 24, 12, 40, 40, dims=8, base=300.0), moe(40, 5, 5, 2.5)),
                with_mlp(wkv(1, 40, 5), moe(16, 3, 1, 1.5)), with_mlp(latent(3, 8, 4, 8, 12, base=50000.0, keep="heads"), None)],
               width=48, vocab=131, taps=4, loop=(0, 1, 3), eps=1e-6, softcap=0)
# no loop, no convolution
CFG_R = config([with_mlp(latent(4, 8, 8, 8, 8), moe(8, 2, 1)), with_mlp(wkv(4, 8, 4), moe(8, 2, 2))], width=32, vocab=61, taps=0)
CONFIGS = {"P": (CFG_P, 21), "Q": (CFG_Q, 22), "R": (CFG_R, 23)}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    from denno_beta_amd.weights import write_model_folder
    made = {}

    def get(name, dtype="float32", cfg=None, seed=None, change=None):
        key = (name, dtype)
        if key not in made:
            c, s = CONFIGS[name] if cfg is None else (cfg, seed)
            d = str(tmp_path_factory.mktemp(f"ridopel{name}_{dtype}"))
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


def plain_logits(folder, seq, keep_layers=False):
    key = (folder, tuple(seq), keep_layers)
    if key not in _plain:
        from safetensors.torch import load_file
        with open(os.path.join(folder, "config.json")) as f:
            cfg = json.load(f)
        _plain[key] = plain.forward(cfg, load_file(os.path.join(folder, "model.safetensors")), seq, torch.float64, keep_layers)
    return _plain[key]


def row_errors(got, want):
    """Per position: the root mean square of the difference (its mean taken off) over the spread of the wanted row."""
    d = got.double() - want.double()
    d = d - d.mean(dim=1, keepdim=True)
    return torch.sqrt((d * d).mean(dim=1)) / want.double().std(dim=1)


# bfloat16, in models 32 to 48 wide: a typical row is off by 0.01 of its spread and a row in a few hundred by up to 0.09,
# so one row in fifty may pass the bound, none by more than two and a half times; a fault moves rows by 0.2 and more
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


# ----------------------------------------------------------------------------------------------------------------
# each mechanism alone
# ----------------------------------------------------------------------------------------------------------------
ALONE = {
    "latent": [with_mlp(latent(3, 8, 8, 16, 16), None)],
    "latent_part_turned": [with_mlp(latent(2, 12, 12, 4, 20, dims=6), None)],
    "latent_heads_kept": [with_mlp(latent(2, 12, 4, 24, 20, keep="heads"), None)],
    "latent_heads_kept_narrow_values": [with_mlp(latent(3, 8, 8, 8, 16, dims=4, keep="heads"), None)],
    "wkv": [with_mlp(wkv(3, 8, 6), None)],
    "hgrn2": [with_mlp(hgrn2(2, 24, 8), None)],
    "experts": [with_mlp(hgrn2(1, 8, 8), moe(12, 6, 3, 0.7))],
}


@pytest.mark.parametrize("what", sorted(ALONE))
@pytest.mark.parametrize("taps", [0, 2])
def test_each_mechanism_alone(backend, folders, what, taps):
    cfg = config(ALONE[what], width=24, vocab=53, taps=taps, loop=(0, 1, 1) if what == "wkv" else None)
    folder = folders(f"alone_{what}_{taps}", "float32", cfg, 5)
    seq = seqs_for(cfg, [29])[0]
    want, streams = plain_logits(folder, seq, keep_layers=True)
    r = runner_for(folder, "float32", backend, 64)
    got = U.replay(r, U.whole_trace([seq]))["r0"]
    assert_rows(got, want, "float32", f"{what}, {taps} taps")
    # the limit of an expert's gate and the soft cap must matter in this model, or the test would not see them
    if what == "experts":
        loose = copy.deepcopy(cfg)
        loose["layers"][0]["mlp"]["expert"]["limit"] = 100.0
        from safetensors.torch import load_file
        other = plain.forward(loose, load_file(os.path.join(folder, "model.safetensors")), seq, torch.float64)
        assert row_errors(other, want).max() > 1e-3


# ----------------------------------------------------------------------------------------------------------------
# every way of cutting the work
# ----------------------------------------------------------------------------------------------------------------
def all_experts(cfg):
    cfg = copy.deepcopy(cfg)
    for layer in cfg["layers"]:
        if layer.get("mlp"):
            layer["mlp"]["router"]["top"] = layer["mlp"]["router"]["experts"]
    return cfg


@pytest.mark.parametrize("name,dtype", [("P", "float32"), ("Q", "float32"), ("R", "float32"), ("P", "bfloat16"), ("Q", "bfloat16")])
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


# ----------------------------------------------------------------------------------------------------------------
# far tokens: weights made so that losing one shows
# ----------------------------------------------------------------------------------------------------------------
MARKER = 7      # the token that the crafted attention looks for


def needle(tensors):
    """A model whose first layer's first head looks for one token wherever it lies.  Every token's row gets a common
    direction u, the marker's row a direction m of its own; the head's plain queries are beta (u . h) d for every
    token, the latent of the marker's key leans towards c, and W_uk carries c to d: the marker's score stands far
    above all others, so every later row takes that head's value from the marker's position, and a key that is lost,
    misplaced or read from a wrong page changes the rows after it as much as one head can."""
    g = torch.Generator().manual_seed(1)
    W = tensors["embed"].shape[1]
    unit = lambda n: torch.nn.functional.normalize(torch.randn(n, generator=g), dim=0)   # noqa: E731
    u, m = unit(W), unit(W)
    m = torch.nn.functional.normalize(m - (m @ u) * u, dim=0)
    tensors["embed"] = tensors["embed"] + 1.5 * u
    tensors["embed"][MARKER] += 3.0 * m
    q, dkv, uk = tensors["l0.mix.q"], tensors["l0.mix.dkv"], tensors["l0.mix.uk"]
    rank, dn = uk.shape[1], 16
    d, c = unit(dn), unit(rank)
    q[:dn] = 40.0 * torch.outer(d, u)
    dkv[:rank] += 4.0 * torch.outer(c, m)
    uk[:dn] = 3.0 * torch.outer(d, c)
    tensors["l0.mix.o"] = tensors["l0.mix.o"] * 4.0


def imprint(tensors):
    """Recurrent layers that keep what one token wrote.  No token's row but the marker's has anything along m.  In the
    wkv layer the decay stays near 0.9975 a token and the marker's key is some thirty times an ordinary one, so the state
    is the marker's key-value product long after; in the hgrn2 layer the forget gate is nearly one for ordinary tokens
    (they keep the state and write almost nothing) and nearly zero for the marker, which replaces the state by its
    value.  A state that is lost, started anew or taken from another slot changes every later row."""
    g = torch.Generator().manual_seed(2)
    W = tensors["embed"].shape[1]
    m = torch.nn.functional.normalize(torch.randn(W, generator=g), dim=0)
    tensors["embed"] = tensors["embed"] - torch.outer(tensors["embed"] @ m, m)
    tensors["embed"][MARKER] += 3.0 * m
    tensors["l0.mix.w0"] = torch.full_like(tensors["l0.mix.w0"], -6.0)
    tensors["l0.mix.w2"] = tensors["l0.mix.w2"] * 0.05
    n = tensors["l0.mix.k"].shape[0]
    tensors["l0.mix.k"] = tensors["l0.mix.k"] + 8.0 * torch.outer(torch.randn(n, generator=g), m)
    tensors["l1.mix.lower"] = torch.zeros_like(tensors["l1.mix.lower"])
    tensors["l1.mix.f.b"] = torch.full_like(tensors["l1.mix.f.b"], 10.0)
    tensors["l1.mix.f"] = tensors["l1.mix.f"] - 8.0 * torch.outer(torch.ones(tensors["l1.mix.f"].shape[0]), m)
    for k in ("l0.mix.o", "l1.mix.o"):
        tensors[k] = tensors[k] * 5.0


FAR = {"latent": (config([with_mlp(latent(2, 16, 16, 8, 24, base=1000.0), None)] * 2, width=32, vocab=71, taps=2, softcap=0), needle),
       "states": (config([with_mlp(wkv(2, 16, 4), None), with_mlp(hgrn2(2, 16, 16), None)], width=32, vocab=71, taps=2, softcap=0), imprint)}


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
        assert row_errors(without[-8:], want[-8:]).min() > 0.2, "the marked token does not reach the last rows"
        for kind, steps in (("whole", U.whole_trace([seq])), ("tail", U.tail_decode_trace([seq], 40)),
                            ("chunks", U.chunk_trace([seq], sizes=(15, 2, 16, 33, 1, 17))),
                            ("pages", U.chunk_trace([seq], sizes=(16, 16, 32, 1, 15, 48)))):
            if at not in (0, 16) and kind in ("chunks", "pages") and backend == "cpu":
                continue          # (the host backend is slow)
            r = runner_for(folder, dtype, backend, U.max_live_tokens(steps))
            assert_rows(U.replay(r, steps)["r0"], want, dtype, f"far {what} {dtype} {kind}, the marker at {at}")


# ----------------------------------------------------------------------------------------------------------------
# the first tokens; slots given out again; a request beside others
# ----------------------------------------------------------------------------------------------------------------
def test_first_tokens_one_by_one(backend, folders):
    """Every token alone from the first: the convolution's history is shorter than its taps, the row before the first
    is zero, the states start at zero."""
    cfg = CONFIGS["Q"][0]
    folder = folders("Q", "float32")
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
    from denno_beta_amd.models.ridopel import RidopelConfig
    assert resolve_architecture({"architecture": "Ridopel"}).config_cls is RidopelConfig
    bad = copy.deepcopy(CFG_P)
    del bad["layers"][1]["mixer"]["kv_rank"]
    with pytest.raises(ConfigError, match="kv_rank"):
        RidopelConfig.from_dict(bad)
    bad = copy.deepcopy(CFG_P)
    bad["loop"]["stop"] = 9
    with pytest.raises(ConfigError, match="loop"):
        RidopelConfig.from_dict(bad)
    bad = copy.deepcopy(CFG_P)
    bad["layers"][0]["type"] = "something"
    with pytest.raises(ConfigError, match="type"):
        RidopelConfig.from_dict(bad)
    # the order of the runs: layer 0, then layers 1 and 2 twice, then layer 3; a pass starts at layer 1
    assert RidopelConfig.from_dict(CFG_P).run_order() == [(0, False), (1, True), (2, False), (1, True), (2, False), (3, False)]
    # a size that only the tensors give: the decay's inner size comes from the file, whatever config.json holds
    folder = folders("P", "float32")
    with open(os.path.join(folder, "config.json")) as f:
        stored = json.load(f)
    del stored["layers"][0]["mixer"]["decay_rank"]
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(stored, f)
    _, cfg = load_config(folder)
    assert cfg.layers[0]["mixer"]["decay_rank"] == 8


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
    tensors["l1.mix.mu.r"] = tensors["l1.mix.mu.r"][:5].contiguous()
    tensors["stray"] = torch.zeros(3)
    save_file(tensors, os.path.join(d, "model.safetensors"))
    with pytest.raises(CheckpointError) as e:
        ModelRunner.from_folder(d, EngineOptions(dtype="float32", device="cpu", cache_tokens=64, max_live=1))
    assert "l0.mlp.e1.up" in e.value.missing and "stray" in e.value.unexpected and e.value.wrong_shape[0][0] == "l1.mix.mu.r"


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
