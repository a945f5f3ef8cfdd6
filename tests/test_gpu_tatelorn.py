"""The Tatelorn design on the GPU against the plain implementation of tests/plain/tatelorn_plain.py:
every mechanism alone, whole models of several shapes, prompts cut into portions, token-by-token
decoding, batches of unequal requests on a cache that is used again, one key planted far away and at
both sides of page borders (the design's attention sees every key), a sink that must take its weight, long decoding
through the recorded decode step, and greedy generation through the Python entry point, the command
line and the replay program."""
import json
import os

import numpy as np
import pytest
import torch

import helpers
from helpers import run_batch, run_tail_one_by_one, run_whole
from plain import tatelorn_plain as T
from test_tatelorn_config import att, moe

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
F32, BF16 = torch.float32, torch.bfloat16
DTYPES = ["float32", "bfloat16"]
TORCH_DT = {"float32": F32, "bfloat16": BF16}
CODES = 8          # channels at the end of the stream that carry a code of the token for the routers


def config(vocab, width, positions, layers, eps=1e-5, embed_scale=1.0, logit_scale=1.0):
    return {"architecture": "Tatelorn", "vocab": vocab, "width": width, "max_positions": positions,
            "logit_scale": logit_scale, "embedding": {"scale": embed_scale}, "norm": {"eps": eps}, "layers": layers}


# P: sizes in sixteens (the matrix-core attention and products in bfloat16); the first layer does not mix values,
#    the second starts, one layer has no feed-forward, one expert a row and three a row, with and without the
#    expert that every row takes, as many kv heads as heads in one layer and one kv head in another.
# Q: sizes that are no multiple of 8 or 16 (plain products, the plain attention kernel), no cap in one layer, no
#    layer that mixes values, an embedding multiplier of 1.
# R: a dense layer between routed ones, every layer mixing, values larger than keys.
CONFIGS = {
    "P": config(160, 96, 400, [
        att(4, 2, 32, 16, 0.55, 6.0, False, moe(4, 1, 48, 1.25)),
        att(2, 2, 16, 48, 0.8, 11.0, True, {"kind": "dense", "ff": 80}),
        att(6, 2, 16, 48, 0.7, 4.0, True, None),
        att(3, 1, 48, 32, 0.4, 9.0, False, moe(6, 3, 32, 0.8, shared=(64, 2.0))),
        att(8, 2, 32, 48, 0.6, 25.0, True, moe(5, 2, 16, 3.0, shared=(16, 0.5))),
    ], eps=3e-4, embed_scale=5.0, logit_scale=0.3),
    "Q": config(131, 60, 350, [
        att(3, 3, 10, 14, 1.2, 0.0, False, {"kind": "dense", "ff": 52}),
        att(2, 1, 24, 6, 0.9, 3.0, False, moe(3, 2, 20, 1.0, shared=(36, 1.5))),
        att(5, 1, 6, 10, 1.5, 7.5, False, moe(7, 4, 12, 2.0)),
    ], eps=1e-6, embed_scale=1.0, logit_scale=1.7),
    "R": config(200, 64, 600, [
        att(2, 1, 16, 64, 0.7, 8.0, True, moe(8, 2, 24, 1.5, shared=(40, 1.0))),
        att(4, 1, 32, 64, 0.5, 15.0, True, {"kind": "dense", "ff": 136}),
        att(1, 1, 64, 64, 0.3, 5.0, True, moe(2, 2, 56, 0.6)),
    ], eps=1e-5, embed_scale=12.0, logit_scale=1.0),
}
SEEDS = {"P": 21, "Q": 22, "R": 23}
_FOLDERS, _PLAIN, _ENGINES, _WANT = {}, {}, {}, {}


def coded_routers(cfg, w, rng):
    """Routers whose choice does not hang on a close call.  The plain implementation sums in float64
    and the bfloat16 path rounds what the router reads: two scores a hair apart would be ordered
    differently by the two, and the rows would take other experts.  So the last CODES channels of the
    stream carry a code of the token (one of them 2, the others 0) that no sublayer writes to (their
    norms' multipliers are zero there), and the routers read those channels alone, with levels chosen so
    that the scores of every code lie far apart.  Every expert is still chosen by some code."""
    d = cfg["width"]
    r = slice(d - CODES, d)
    code = np.zeros((cfg["vocab"], CODES))
    code[np.arange(cfg["vocab"]), np.arange(cfg["vocab"]) % CODES] = 2.0
    w["embed"][:, r] = code / cfg["embedding"]["scale"]
    w["pos"][:, r] = 0.0
    w["embed.norm"][r] = 0.0
    for i, layer in enumerate(cfg["layers"]):
        w[f"l{i}.norm1"][r] = -1.0
        f = layer["mlp"]
        if f is None:
            continue
        w[f"l{i}.norm2"][r] = -1.0
        if f["kind"] != "moe":
            continue
        e = f["router"]["experts"]
        # [experts, codes]: code c ranks the experts c - 1 - i, c - 2 - i, ... (mod experts) from the top
        levels = ((np.arange(e)[:, None] - np.arange(CODES)[None, :] + i) % e).astype(np.float64)
        router = np.zeros((e, d))
        router[:, r] = levels * 3.0
        w[f"l{i}.mlp.router"] = router
    return w


def sharpen(cfg, w, seed, coded=True):
    """Random N(0, 0.02) weights give sublayer results whose norm then blows up rounding, gates near zero
    and experts far inside their limits.  Scale the projections so that scores spread over several
    units (the configurations' `scale` does the rest), the experts' clamps bite and the mixing numbers lie
    inside (0, 1); norm weights spread around zero."""
    rng = np.random.default_rng(seed)
    out = {}
    for name, a in w.items():
        a = np.array(a, dtype=np.float64)
        if name.endswith((".mix.q", ".mix.k", ".mix.v", ".mix.o")):
            a = a * 8.0
        elif name.endswith((".gate", ".up", ".down", ".sg")):
            a = a * 3.0
        elif name.endswith((".q.norm", ".k.norm")):
            a = 1.0 + (a - 1.0) * 6.0
        elif name.endswith(("norm1", "norm2", "embed.norm", "final.norm")):
            a = a * 8.0
        elif name.endswith(".vmix"):
            a = np.asarray(rng.uniform(0.2, 0.8))
        elif name in ("embed", "pos"):
            a = a * 20.0
        elif name.endswith(".router"):
            a = a * 40.0
        out[name] = a
    return coded_routers(cfg, out, rng) if coded else out


def make_folder(tmp_path_factory, name, cfg, seed, coded=True):
    from safetensors.torch import load_file, save_file
    from sonicboom_amd.weights import write_random_model
    folder = str(tmp_path_factory.mktemp(f"tatelorn_{name}"))
    write_random_model(folder, json.loads(json.dumps(cfg)), seed=seed, dtype="bfloat16", device=None)
    path = os.path.join(folder, "model.safetensors")
    w = sharpen(cfg, {k: v.float().numpy() for k, v in load_file(path).items()}, seed, coded)
    save_file({k: torch.from_numpy(np.asarray(v, dtype=np.float32)).to(BF16).contiguous() for k, v in w.items()}, path,
              metadata={"format": "pt"})
    plain = {k: v.float().numpy().astype(np.float64) for k, v in load_file(path).items()}
    return folder, plain


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    """name -> folder with config.json and bfloat16 weights (sharpened, routers coded as above)."""
    for name, cfg in CONFIGS.items():
        if name not in _FOLDERS:
            _FOLDERS[name], _PLAIN[name] = make_folder(tmp_path_factory, name, cfg, SEEDS[name])
    return _FOLDERS


def engine_for(folder, dtype, max_tokens=64 * 24, **kw):
    from sonicboom_amd.engine import DecoderModel, Engine
    key = (folder, dtype, max_tokens, tuple(sorted(kw.items())))
    if key not in _ENGINES:
        _ENGINES[key] = Engine(DecoderModel.from_folder(folder, dtype), max_tokens, **kw)
    return _ENGINES[key]


def want_logits(name, tokens):
    key = (name, tuple(tokens))
    if key not in _WANT:
        _WANT[key] = T.forward(CONFIGS[name], _PLAIN[name], list(tokens))
    return _WANT[key]


def prompts(name, lengths, seed=0):
    rng = np.random.default_rng(seed)
    return [[int(t) for t in rng.integers(0, CONFIGS[name]["vocab"], size=n)] for n in lengths]


# Bounds.  float32 differs from the plain implementation (float64) by the rounding of float32 sums.
# bfloat16 is measured in spreads of the logits (their standard deviation): the largest difference
# and the root mean square of all differences of a request.
F32_BOUND = 3e-4
BF16_WORST, BF16_RMS = 0.165, 0.021      # what the whole file measured (0.1169 and 0.0146: the models are sharpened) times 1.4
helpers.BF16_MAX["normed outputs and experts"], helpers.BF16_RMS["normed outputs and experts"] = BF16_WORST, BF16_RMS


def close(got, want, dtype, what):
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape, f"{what}: shape {got.shape} vs {want.shape}"
    assert np.isfinite(got).all(), f"{what}: not finite"
    spread = max(float(want.std()), 1e-30)
    err = np.abs(got - want) / spread
    if dtype in ("float32", F32):
        assert err.max() <= F32_BOUND, f"{what}: differs by {err.max():.3g} spreads at {np.unravel_index(err.argmax(), err.shape)}"
    else:
        rms = float(np.sqrt((err ** 2).mean()))
        seen = helpers.BF16_SEEN.setdefault("normed outputs and experts", [0.0, 0.0])
        seen[0], seen[1] = max(seen[0], float(err.max())), max(seen[1], rms)
        assert err.max() <= BF16_WORST and rms <= BF16_RMS, \
            f"{what}: differs by {err.max():.3g} spreads at {np.unravel_index(err.argmax(), err.shape)}, rms {rms:.3g}"


def run_cuts(engine, tokens, cuts):
    """One request fed in portions of the given sizes; logits of every position."""
    from sonicboom_amd.engine import StepEntry
    assert sum(cuts) == len(tokens)
    s = engine.alloc_slot()
    try:
        rows, at = [], 0
        for n in cuts:
            rows.append(engine.step([StepEntry(s, tokens[at:at + n], range(n))]).cpu().numpy())
            at += n
        return np.concatenate(rows, axis=0)
    finally:
        engine.free_slot(s)


# ---- whole models -------------------------------------------------------------------------------
def test_the_routers_of_these_models_make_no_close_calls(folders):
    for name, cfg in CONFIGS.items():
        tokens = prompts(name, [120], seed=3)[0]
        x = T.start(cfg, _PLAIN[name], tokens)
        for i, layer in enumerate(cfg["layers"]):
            f = layer["mlp"]
            if f is None or f["kind"] != "moe":
                continue
            z = np.sort(T.linear(x, _PLAIN[name][f"l{i}.mlp.router"]), axis=1)[:, ::-1]      # the code channels never change
            top = f["router"]["top"]
            if top < z.shape[1]:
                assert (z[:, top - 1] - z[:, top]).min() > 0.05 * z.std(), (name, i)
            chosen, _ = T.route(T.linear(x, _PLAIN[name][f"l{i}.mlp.router"]), top)
            assert len(np.unique(chosen)) == f["router"]["experts"], "every expert is chosen by some token"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_whole_requests_and_the_first_tokens(folders, name, dtype):
    eng = engine_for(folders[name], dtype)
    for tokens in prompts(name, [1, 2, 3, 17, 63, 64, 65, 200]):
        close(run_whole(eng, tokens), want_logits(name, tokens), dtype, f"{name} whole n={len(tokens)}")
    assert eng.cache.held_pages() == 0 and not eng.cache.live_slots


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_random_routers_in_32_bit(tmp_path_factory, name):
    """The same models with routers of plain random weights (scores as close as chance makes them)."""
    folder, plain = make_folder(tmp_path_factory, name + "_random", CONFIGS[name], SEEDS[name] + 100, coded=False)
    eng = engine_for(folder, "float32")
    for tokens in prompts(name, [90, 5], seed=4):
        close(run_whole(eng, tokens), T.forward(CONFIGS[name], plain, tokens), "float32", f"{name} random routers")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_prompt_against_token_by_token(folders, name, dtype):
    eng = engine_for(folders[name], dtype)
    for tokens in prompts(name, [40, 150], seed=1):
        got = run_tail_one_by_one(eng, tokens, tail=len(tokens) - 3)
        close(got, want_logits(name, tokens), dtype, f"{name} one by one n={len(tokens)}")
        if dtype == "float32":
            assert np.array_equal(got, run_whole(eng, tokens)), "in 32-bit the cut must not matter by a bit"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_portions_of_several_sizes(folders, name, dtype):
    eng = engine_for(folders[name], dtype)
    tokens = prompts(name, [331], seed=2)[0]
    whole = run_whole(eng, tokens)
    for cuts in ([2] * 20 + [291], [64, 64, 64, 139], [63, 2, 65, 1, 127, 3, 70], [130, 2, 2, 129, 68], [1, 330]):
        got = run_cuts(eng, tokens, cuts)
        close(got, want_logits(name, tokens), dtype, f"{name} cuts {cuts[:4]}")
        if dtype == "float32":
            assert np.array_equal(got, whole), f"cuts {cuts[:4]} change bits"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_unequal_batches_on_a_cache_that_is_used_again(folders, name, dtype):
    """Nine pages: every batch fills eight of them, the next gets used pages and slots."""
    eng = engine_for(folders[name], dtype, max_tokens=64 * 9, max_slots=5)
    lens = [(1, 9), (70, 4), (5, 30), (130, 12), (33, 1)]
    for round_ in range(3):
        reqs = prompts(name, [p + d for p, d in lens], seed=20 + round_)
        got = run_batch(eng, reqs, [p for p, _ in lens])
        for r, (p, _), g in zip(reqs, lens, got):
            close(g, want_logits(name, r), dtype, f"{name} batch, request of {len(r)}")
        if dtype == "float32":
            alone = run_tail_one_by_one(eng, reqs[3], tail=lens[3][1])
            assert np.array_equal(got[3], alone), "in 32-bit the batch must not matter by a bit"
        assert eng.cache.held_pages() == 0 and not eng.cache.live_slots


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_step_that_runs_in_portions(folders, dtype):
    """A step of more rows than the engine takes at once is cut inside sequences; the values that later
    layers mix in are those of the portion's own rows."""
    eng = engine_for(folders["P"], dtype, max_tokens=64 * 12, max_step_rows=100)
    reqs = prompts("P", [130, 7, 220], seed=5)
    got = run_batch(eng, reqs, [130, 7, 220])
    for r, g in zip(reqs, got):
        close(g, want_logits("P", r), dtype, f"portions, request of {len(r)}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["P", "R"])
def test_long_decoding_through_the_decode_loop(folders, name, dtype):
    """150 single-token steps of two sequences past page borders, kernel by kernel and then replayed
    from the recorded step; logits of every step against the plain implementation."""
    eng = engine_for(folders[name], dtype)
    reqs = prompts(name, [60 + 150, 3 + 150], seed=7)
    heads = [60, 3]
    from sonicboom_amd.engine import StepEntry
    slots = [eng.alloc_slot() for _ in reqs]
    try:
        eng.step([StepEntry(s, r[:h], ()) for s, r, h in zip(slots, reqs, heads)])
        loop = eng.decode_loop()
        assert loop.use_graph, "every part of the model says its step can be recorded"
        loop.start(slots, [r[h] for r, h in zip(reqs, heads)])
        rows = [[], []]
        for k in range(150):
            logits = loop.step_logits([r[h + k] for r, h in zip(reqs, heads)]).cpu().numpy()
            for i in range(2):
                rows[i].append(logits[i])
        for r, h, got in zip(reqs, heads, rows):
            close(np.stack(got), want_logits(name, r)[h:], dtype, f"{name} long decoding")
    finally:
        for s in slots:
            eng.free_slot(s)


def test_greedy_generation_through_the_entry_point(folders):
    from sonicboom_amd.api import Model
    for name in ("P", "Q"):
        ps = prompts(name, [4, 70, 19], seed=9)
        session = Model.load(folders[name], dtype="float32").session(max_tokens=64 * 8)
        got = session.generate(ps, max_tokens=12, stop_tokens=())
        assert got == [T.greedy(CONFIGS[name], _PLAIN[name], p, 12) for p in ps]
        assert [session.generate([p], max_tokens=12, stop_tokens=())[0] for p in ps] == got
        assert not session.engine.cache.live_slots
        # bfloat16: every chosen token is the plain implementation's best or within rounding of it
        session = Model.load(folders[name], dtype="bfloat16").session(max_tokens=64 * 8)
        for p, out in zip(ps, session.generate(ps, max_tokens=12, stop_tokens=())):
            logits = want_logits(name, p + out)
            for i, t in enumerate(out):
                row = logits[len(p) - 1 + i]
                assert row[t] >= row.max() - 2 * BF16_WORST * row.std(), (name, i)


def test_positions_past_the_table_are_refused(folders):
    from sonicboom_amd.engine import StepEntry, StepError
    eng = engine_for(folders["Q"], "float32", max_tokens=64 * 8)
    s = eng.alloc_slot()
    try:
        with pytest.raises(StepError, match="positions"):
            eng.step([StepEntry(s, [1] * (CONFIGS["Q"]["max_positions"] + 1), ())])
    finally:
        eng.free_slot(s)


def test_command_line_and_trace_replay(folders, tmp_path):
    """The command line generates from a folder of this design; the replay program feeds a prompt, then
    its next tokens one by one beside a second request, frees one and goes on, and writes the logits
    the plain implementation gives."""
    import subprocess
    import sys
    from conftest import ROOT
    name = "Q"
    ps = prompts(name, [4, 10], seed=9)
    tokens = tmp_path / "prompts.txt"
    tokens.write_text("\n".join(" ".join(map(str, p)) for p in ps) + "\n")
    cmd = [sys.executable, os.path.join(ROOT, "bin", "sb-gen"), "-m", folders[name], "--tokens", str(tokens), "-n", "6",
           "--dtype", "fp32", "--stop", ""]
    out = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr
    got = [[int(t) for t in line.split()] for line in out.stdout.strip().splitlines()]
    assert got == [T.greedy(CONFIGS[name], _PLAIN[name], p, 6) for p in ps]
    a, b = prompts(name, [75, 12], seed=10)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:70], "want": [0, 69]}, {"id": "b", "tokens": b[:9], "want": [8]}], "end": []}]
    for k in range(3):
        steps.append({"step": k + 1, "entries": [{"id": "a", "tokens": [a[70 + k]], "want": [0]},
                                                 {"id": "b", "tokens": [b[9 + k]], "want": [] if k == 1 else [0]}],
                      "end": ["b"] if k == 2 else []})
    steps.append({"step": 4, "entries": [{"id": "a", "tokens": a[73:75], "want": [1]}], "end": ["a"]})
    for dtype in DTYPES:
        outdir = tmp_path / f"out_{dtype}"
        run = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folders[name], "--dtype", dtype,
                              "--out", str(outdir), "--max-tokens", "256"], input="\n".join(json.dumps(x) for x in steps) + "\n",
                             capture_output=True, text=True, timeout=300)
        assert run.returncode == 0, run.stderr
        assert [ln for ln in run.stdout.splitlines() if ln.startswith("done")] == [f"done {i}" for i in range(5)]
        wa, wb = want_logits(name, a), want_logits(name, b)
        vocab = CONFIGS[name]["vocab"]
        read = lambda i: np.fromfile(outdir / f"{i}.f32", dtype="<f4").reshape(-1, vocab)
        close(read(0), np.stack([wa[0], wa[69], wb[8]]), dtype, "replay, prompts")
        close(read(1), np.stack([wa[70], wb[9]]), dtype, "replay, first single tokens")
        close(read(2), wa[71:72], dtype, "replay, a step where one request wants nothing")
        close(read(3), np.stack([wa[72], wb[11]]), dtype, "replay, last step of the short request")
        close(read(4), wa[74:75], dtype, "replay, two more tokens alone")


# ---- mechanisms alone ---------------------------------------------------------------------------
def runtime(dtype, fast=True):
    from sonicboom_amd.parts import Runtime
    return Runtime(torch.device(DEV), TORCH_DT[dtype], fast)


def rand(*shape, scale=1.0, seed=0):
    g = torch.Generator().manual_seed(1000 * seed + sum(shape) + len(shape))
    return torch.randn(tuple(shape), generator=g) * scale


def part_tensors(spec, dtype, seed=0, scale=0.3):
    dev, ref = {}, {}
    for i, t in enumerate(spec.all_tensors()):
        a = (rand(*t.shape, scale=scale, seed=seed + i) + t.init[0]).to(TORCH_DT[dtype])
        dev[t.name], ref[t.name] = a.to(DEV), a.float().numpy().astype(np.float64)
    return dev, ref


def part_close(got, want, dtype, what, bf16=2.5e-2):
    got, want = got.detach().float().cpu().numpy().astype(np.float64), np.asarray(want, dtype=np.float64)
    scale = max(float(np.abs(want).max()), 1e-30)
    assert got.shape == want.shape, f"{what}: shape {got.shape} vs {want.shape}"
    err = np.abs(got - want).max() / scale
    assert err <= (2e-5 if dtype == "float32" else bf16), f"{what}: off by {err:.3g} of the largest value"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width", [96, 60, 35, 520, 4096])
def test_norm_with_an_offset_and_the_pass_that_ends_a_sublayer(dtype, width):
    from sonicboom_amd import ops
    from sonicboom_amd.parts import build_part
    from sonicboom_amd.parts.norm import rmsnorm_spec
    spec = rmsnorm_spec("n", width, 2e-3, offset=1.0)
    dev, ref = part_tensors(spec, dtype)
    norm = build_part(spec, dev, runtime(dtype))
    assert not norm.fusable, "the fused passes of other blocks multiply by the weight as it is"
    x = rand(7, width, scale=3.0)
    part_close(norm.forward(x.to(DEV), TORCH_DT[dtype]), T.unit_norm(x.numpy(), ref["n"], 2e-3), dtype, "norm")
    rows = torch.tensor([5, 0, 5], dtype=torch.int32, device=DEV)
    part_close(norm.forward(x.to(DEV), TORCH_DT[dtype], rows=rows), T.unit_norm(x.numpy()[[5, 0, 5]], ref["n"], 2e-3), dtype,
               "norm of picked rows")
    # x += un(sum of slices): whole, in slices, and pairs with weights plus an extra addend with a gate
    y = rand(3, 7, width, seed=2)
    xd = x.to(DEV).clone()
    copy = ops.norm_add(xd, y.to(DEV), dev["n"], 2e-3, 1.0, TORCH_DT[dtype])
    want = x.numpy() + T.unit_norm(y.numpy().astype(np.float64).sum(0), ref["n"], 2e-3)
    part_close(xd, want, "float32", "slices, normed, added")
    part_close(copy, want, dtype, "the stream in the activation type")
    pairs, pw, extra = rand(7, 3, width, seed=3), rand(7, 5, seed=4).abs(), rand(7, width, seed=5)
    xd = x.to(DEV).clone()
    pwd = pw.to(DEV)
    ops.norm_add(xd, pairs.to(DEV), dev["n"], 2e-3, 1.0, None, part_weights=pwd[:, :3], extra=extra.to(DEV),
                 extra_weights=pwd[:, 4:], by_row=True)
    s = (pairs.numpy().astype(np.float64) * pw.numpy()[:, :3, None]).sum(1) + extra.numpy() * pw.numpy()[:, 4:]
    part_close(xd, x.numpy() + T.unit_norm(s, ref["n"], 2e-3), "float32", "weighted pairs and an extra addend")


@pytest.mark.parametrize("dtype", DTYPES)
def test_embedding_with_positions_and_norm(dtype):
    from sonicboom_amd.parts import build_part
    from sonicboom_amd.parts.embedding import positional_embedding_spec
    spec = positional_embedding_spec("embed", 50, 72, 7.0, "pos", 30, "embed.norm", 1e-4, 1.0)
    dev, ref = part_tensors(spec, dtype, scale=0.5)
    emb = build_part(spec, dev, runtime(dtype))

    class Ctx:
        row_pos = torch.tensor([0, 1, 2, 29, 5, 6], dtype=torch.int32, device=DEV)
    ids = torch.tensor([3, 3, 49, 0, 7, 3], dtype=torch.int32, device=DEV)
    cfg = {"embedding": {"scale": 7.0}, "norm": {"eps": 1e-4}}
    want = np.concatenate([T.start(cfg, ref, [3, 3, 49]), T.start(cfg, ref, [0], 29), T.start(cfg, ref, [7, 3], 5)])
    got = emb.forward(ids, Ctx)
    part_close(got, want, "float32", "embedding")
    assert not np.allclose(got[0].cpu().numpy(), got[1].cpu().numpy()), "the same token at another position"
    Ctx.row_pos = torch.tensor([0, 1, 2, 30, 5, 6], dtype=torch.int32, device=DEV)
    assert torch.isnan(emb.forward(ids, Ctx)[3]).all(), "a position outside the table gives no numbers"


def mixer_harness(mixer, rt, n_tokens_cap=64 * 20):
    """A cache for one mixer alone, and a function that feeds rows of one sequence in cuts and returns
    what the mixer hands to its block."""
    from sonicboom_amd.cache import PagedCache, group_entries
    from sonicboom_amd.engine.model import LayerBinding
    from sonicboom_amd.engine.step import StepContext, StepEntry
    cs = mixer.cache_spec()
    cache = PagedCache(group_entries({0: cs.key()}), n_tokens_cap, rt.cache_dtype, rt.device, None, max_slots=4)
    tiles = getattr(mixer, "row_tile", None) or ()
    tiles = (tiles,) if isinstance(tiles, int) else tuple(tiles)

    def feed(h_rows, cuts, shared=None):
        k, v, g = cache.entry_views(0)
        binding = LayerBinding(0, g, k, v, True, None)
        slot = cache.alloc_slot()
        outs, at = [], 0
        try:
            for n in cuts:
                cache.reserve([slot], [n])
                ctx = StepContext(cache, [StepEntry(slot, [0] * n, ())], rt.device, tiles)
                ctx.shared = {} if shared is None else {key: t[at:at + n].contiguous() for key, t in shared.items()}
                y = mixer.produce(h_rows[at:at + n].to(DEV).contiguous(), ctx, binding)
                outs.append(y.sum(0) if y.dim() == 3 else y)
                cache.advance([slot], [n])
                at += n
        finally:
            cache.free_slot(slot)
        return torch.cat(outs)
    return feed


def attention_mixer(dtype, heads, kv_heads, dim, vdim, scale, softcap, mix=None, width=64, seed=0, fast=True, eps=1e-5):
    from sonicboom_amd.architectures.tatelorn import MIX_NAMES
    from sonicboom_amd.parts import PartSpec, build_part
    from sonicboom_amd.parts.attention import attention_spec
    spec = attention_spec("a.", width, heads, kv_heads, dim, PartSpec("position", "none"), scale=scale, qkv_bias=False,
                          v_dim=vdim, qk_norm=True, qk_norm_eps=eps, softcap=softcap, sink=True, value_mix=mix,
                          names=MIX_NAMES)
    dev, ref = part_tensors(spec, dtype, seed=seed, scale=0.5)
    rt = runtime(dtype, fast)
    mx = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "softcap": softcap,
          "v_mix": mix is not None}
    return build_part(spec, dev, rt), rt, ref, mx


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, kv_heads, dim, vdim, softcap", [
    (4, 2, 32, 16, 6.0), (3, 3, 10, 14, 2.0), (5, 1, 16, 64, 30.0), (2, 1, 24, 6, 4.0), (8, 1, 64, 48, 9.0), (1, 1, 128, 128, 12.0)])
def test_attention_alone(dtype, heads, kv_heads, dim, vdim, softcap):
    """Head norms, scores capped, the sink, values of their own size: whole, in portions and token by token."""
    mixer, rt, ref, mx = attention_mixer(dtype, heads, kv_heads, dim, vdim, 3.0 / np.sqrt(dim), softcap)
    feed = mixer_harness(mixer, rt)
    n = 200
    h = rand(n, 64).to(TORCH_DT[dtype])
    want, _ = T.attention(mx, 1e-5, ref, "a.", h.float().numpy())
    for cuts in ([n], [70, 2, 60] + [1] * 68):
        part_close(feed(h, cuts), want, dtype, f"attention cuts {cuts[:3]}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_mixed_values_are_what_the_cache_keeps(dtype):
    """A later mixing layer: the values of the first one come with the step's rows; what is decoded later
    reads the mixed values of earlier steps from the cache."""
    mixer, rt, ref, mx = attention_mixer(dtype, 4, 2, 16, 32, 0.6, 8.0, mix="mix")
    ref["a.vmix"] = np.asarray(0.3125)
    mixer.lam.fill_(0.3125)
    feed = mixer_harness(mixer, rt)
    n = 150
    h = rand(n, 64).to(TORCH_DT[dtype])
    v_first = rand(n, 2 * 32, seed=7)
    want, _ = T.attention(mx, 1e-5, ref, "a.", h.float().numpy(), v_first.numpy().astype(np.float64))
    for cuts in ([n], [64, 3] + [1] * 83):
        part_close(feed(h, cuts, shared={"values": v_first.to(DEV)}), want, dtype, f"mixed values, cuts {cuts[:2]}")
    plain, _ = T.attention(dict(mx, v_mix=False), 1e-5, ref, "a.", h.float().numpy())
    assert np.abs(plain - want).max() > 0.1 * np.abs(want).max(), "the mixing does not show: the test shows nothing"


@pytest.mark.parametrize("heads, kv_heads, dim, vdim", [(4, 1, 32, 16), (6, 2, 64, 64), (16, 2, 128, 64), (5, 5, 16, 48), (9, 1, 48, 32)])
def test_matrix_core_attention_equals_the_plain_kernel(heads, kv_heads, dim, vdim):
    """bfloat16: a prompt, portions and single rows over several pages (the pages of a step of few rows
    are shared out over blocks and merged) against the kernel of one wave per (row, head).  The steps of
    700 and 560 rows also take the head norms' form for long steps (eight numbers a lane)."""
    n = 700
    h = rand(n, 64).to(BF16)
    outs = {}
    for fast in (True, False):
        mixer, rt, ref, mx = attention_mixer("bfloat16", heads, kv_heads, dim, vdim, 2.0 / np.sqrt(dim), 10.0, fast=fast)
        feed = mixer_harness(mixer, rt)
        outs[fast] = [feed(h, cuts) for cuts in ([n], [560, 17, 3] + [1] * 120)]
    want, _ = T.attention(mx, 1e-5, ref, "a.", h.float().numpy())
    for a, b in zip(outs[True], outs[False]):
        part_close(a, b.float().cpu().numpy(), "bfloat16", "matrix cores against the plain kernel", bf16=1.5e-2)
        part_close(a, want, "bfloat16", "matrix cores against the plain implementation")


def planted_mixer(dtype, dim=16, vdim=16, width=48, gain=12.0, softcap=50.0, fast=True):
    """An attention mixer whose weights are set by hand: keys read the input's numbers 1..dim, queries the
    numbers behind them; both carry a constant 1 in their first number (input number 0 and dim+1), so that
    the head norm does not blow a silent row up.  A row whose input has number dim+2 set asks for keys whose
    input has number 1 set: the score of that pair is large, every other score is the small product of the
    constants.  Values and output are random."""
    mixer, rt, ref, mx = attention_mixer(dtype, 2, 1, dim, vdim, 1.0, softcap, width=width, fast=fast, eps=1e-6)
    t = {k: torch.zeros(v.shape) for k, v in ref.items()}
    for d in range(dim):
        t["a.k"][d, d] = 1.0
        for a in range(2):
            t["a.q"][a * dim + d, dim + d] = 1.0
    t["a.q.norm"][:], t["a.k.norm"][:] = 1.0, 1.0
    t["a.v"], t["a.o"] = rand(vdim, width, seed=1), rand(width, 2 * vdim, scale=0.3, seed=3)
    from sonicboom_amd.parts import PartSpec, build_part
    from sonicboom_amd.parts.attention import attention_spec
    from sonicboom_amd.architectures.tatelorn import MIX_NAMES
    spec = attention_spec("a.", width, 2, 1, dim, PartSpec("position", "none"), scale=gain / dim, qkv_bias=False,
                          v_dim=vdim, qk_norm=True, qk_norm_eps=1e-6, softcap=softcap, sink=True, names=MIX_NAMES)
    dev = {k: v.to(TORCH_DT[dtype]).to(DEV) for k, v in t.items()}
    ref = {k: v.to(TORCH_DT[dtype]).float().numpy().astype(np.float64) for k, v in t.items()}
    mx = dict(mx, scale=gain / dim)
    return build_part(spec, dev, rt), rt, ref, mx, width


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("fast", [True, False])
def test_one_key_stands_out_and_the_sink_takes_its_weight(dtype, fast):
    """A prompt of 700 rows in which the last row asks and one row answers: the query's weight falls on that
    key however far back it lies: the row before, at both sides of page borders, hundreds of rows away, the
    very first row.  The query runs as the last row of a prompt, as a single decoded row, and behind a
    portion of two rows.  With no key that answers, most of the weight goes to the sink and the result is
    small: leaving the sink out would show as a result several times larger."""
    if fast and dtype == "float32":
        pytest.skip("the 32-bit path has one attention kernel")
    dim = 16
    mixer, rt, ref, mx, width = planted_mixer(dtype, dim=dim, fast=fast)
    feed = mixer_harness(mixer, rt)
    n = 700
    t = n - 1
    shows = 0
    for b in [1, 2, 63, 64, 65, 127, 128, 129, 500, 636, 699]:
        j = t - b
        h = rand(n, width, seed=b) * 0.05
        h[:, 0] = 1.0                     # every key's constant number
        h[:, 1:dim] = 0.0                 # no key answers ...
        h[:, dim] = 1.0                   # every query's constant number
        h[:, dim + 1:2 * dim] = 0.0       # ... and no row asks,
        h[j, 1], h[t, dim + 1] = 3.0, 3.0  # but for these two
        h = h.to(TORCH_DT[dtype])
        hn = h.float().numpy()
        want, _ = T.attention(mx, 1e-6, ref, "a.", hn)
        for cuts in ([n], [n - 1, 1], [300, 336, 61, 2, 1]):
            part_close(feed(h, cuts)[t:], want[t:], dtype, f"key {b} back, cuts {cuts}")
        hidden = hn.copy()
        hidden[j, 1] = 0.0
        other, _ = T.attention(mx, 1e-6, ref, "a.", hidden)
        if np.abs(other[t] - want[t]).max() > 0.3 * np.abs(want[t]).max():
            shows += 1
    assert shows >= 10, "the planted key does not decide the result: the test shows nothing"
    # nobody answers: the sink holds most of the weight
    h = rand(n, width, seed=99) * 0.05
    h[:, 0], h[:, dim] = 1.0, -1.0        # every row asks for the opposite of what the keys hold: scores far below 0
    h[:, 1:dim], h[:, dim + 1:2 * dim] = 0.0, 0.0
    h = h.to(TORCH_DT[dtype])
    hn = h.float().numpy()
    want, _ = T.attention(mx, 1e-6, ref, "a.", hn)
    got = feed(h, [n - 1, 1])
    part_close(got[t:], want[t:], dtype, "no key answers")
    q = T.head_norm(T.linear(hn, ref["a.q"]).reshape(n, 2, dim), ref["a.q.norm"], 1e-6)
    k = T.head_norm(T.linear(hn, ref["a.k"]).reshape(n, 1, dim), ref["a.k.norm"], 1e-6)
    s = T.capped_scores(q[t:, 0], k[:, 0], mx["scale"], mx["softcap"])
    no_sink = np.exp(s - s.max())
    no_sink = (no_sink / no_sink.sum()) @ T.linear(hn, ref["a.v"])
    with_sink = T.sink_softmax(s, np.ones_like(s, dtype=bool)) @ T.linear(hn, ref["a.v"])
    assert np.abs(no_sink).max() > 3 * np.abs(with_sink).max(), "the sink does not show: the test shows nothing"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows", [1, 3, 70, 300])
@pytest.mark.parametrize("experts, top, inner, shared", [(4, 1, 48, 0), (6, 3, 32, 64), (3, 3, 20, 36), (9, 2, 136, 16)])
def test_routed_experts_alone(dtype, rows, experts, top, inner, shared):
    """The router's choice and weights, the experts' products (grouped by expert on the matrix cores in
    bfloat16 when the sizes allow, else a thread an output), the shared expert and its gate, and the pass
    that adds them up."""
    from sonicboom_amd import ops
    from sonicboom_amd.parts import build_part
    from sonicboom_amd.parts.moe import moe_ffn_spec
    width = 72 if inner % 8 else 64
    spec = moe_ffn_spec("m.", width, experts, top, inner, 0.9, 1.702, shared, 1.4)
    dev, ref = part_tensors(spec, dtype, scale=0.4)
    # routers apart by construction: the first `experts` input numbers decide, in levels
    g = torch.Generator().manual_seed(rows + experts)
    h = rand(rows, width, scale=1.0, seed=rows)
    h[:, :experts] = torch.stack([torch.randperm(experts, generator=g).float() for _ in range(rows)]) * 2.0
    router = torch.zeros(experts, width)
    router[:, :experts] = torch.eye(experts) * 2.0
    dev["m.router"], ref["m.router"] = router.to(TORCH_DT[dtype]).to(DEV), router.numpy().astype(np.float64)
    ffn = build_part(spec, dev, runtime(dtype))
    h = h.to(TORCH_DT[dtype])
    b = ffn.produce(h.to(DEV), None)
    cfg = {"router": {"experts": experts, "top": top}, "expert": {"ff": inner, "limit": 0.9},
           "shared": {"ff": shared, "limit": 1.4} if shared else None}
    want = T.moe_ff(cfg, ref, "m.", h.float().numpy())
    x = torch.zeros(rows, width, dtype=F32, device=DEV)
    ops.norm_add(x, b.part, None, 0.0, 0.0, None, part_weights=b.part_weights, extra=b.extra, extra_weights=b.extra_weights,
                 by_row=True, norm=False)
    part_close(x, want, dtype, "routed experts")
    x2 = torch.zeros(rows, width, dtype=F32, device=DEV)
    ffn.forward(h.to(DEV), x2, None)
    assert torch.equal(x, x2)
    # the clamps bite in this test: without them the result is another
    loose = T.moe_ff(dict(cfg, expert={"ff": inner, "limit": 1e9}), ref, "m.", h.float().numpy())
    assert np.abs(loose - want).max() > 0.05 * np.abs(want).max()


def test_the_router_kernel_orders_like_the_plain_one():
    from sonicboom_amd import ops
    z = rand(500, 11, seed=3)
    z[5, 2] = z[5, 7]                       # a tie goes to the lower number
    z[6] = 0.0
    for top in (1, 2, 5, 11):
        ids, w = ops.moe_route(torch.cat([z, rand(500, 1, seed=4)], dim=1).contiguous().to(DEV), 11, top, True)
        chosen, weight = T.route(z.numpy().astype(np.float64), top)
        assert np.array_equal(ids.cpu().numpy(), chosen)
        assert np.allclose(w[:, :top].cpu().numpy(), weight, atol=1e-6)
        assert np.allclose(w[:, top].cpu().numpy(), T.sigmoid(rand(500, 1, seed=4).numpy()[:, 0]), atol=1e-6)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows", [3, 70, 300])
def test_dense_feed_forward_with_a_relu_gate(dtype, rows):
    from sonicboom_amd.parts import build_part
    from sonicboom_amd.parts.ffn import gated_ffn_spec
    spec = gated_ffn_spec("m.", 72, 200, activation="relu", names=("gate", "up", "down"))
    dev, ref = part_tensors(spec, dtype)
    ffn = build_part(spec, dev, runtime(dtype))
    h = rand(rows, 72, scale=2.0).to(TORCH_DT[dtype])
    y = ffn.produce(h.to(DEV), None)
    part_close(y.sum(0) if y.dim() == 3 else y, T.dense_ff(ref, "m.", h.float().numpy()), dtype, "feed-forward")
