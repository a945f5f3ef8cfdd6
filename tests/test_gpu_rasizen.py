"""The Rasizen design on the GPU against the plain implementation of tests/plain/rasizen_plain.py:
every mechanism alone, whole models of several shapes, prompts cut into portions, token-by-token
decoding, batches of unequal requests on a cache that is used again, keys planted far away, at
page borders and at both sides of a window's edge, long decoding through the recorded decode
step, and greedy generation through the Python entry point."""
import json
import os

import numpy as np
import pytest
import torch

import helpers
from helpers import run_batch, run_tail_one_by_one, run_whole
from plain import rasizen_plain as R

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
F32, BF16 = torch.float32, torch.bfloat16
DTYPES = ["float32", "bfloat16"]
TORCH_DT = {"float32": F32, "bfloat16": BF16}


# ---- configurations ------------------------------------------------------------------------------
def latent(heads, dim, rot_dim, vdim, rank, scale, window, base=10000.0, dims=None, kv_from=None, mlp=None):
    mx = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank, "scale": scale,
          "rot": {"base": base, "dims": rot_dim if dims is None else dims}}
    if window:
        mx["mask"] = {"size": window}
    if kv_from is not None:
        mx["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": mx, "mlp": None if mlp is None else {"kind": "dense", "ff": mlp}}


def gru(width, mlp=None):
    return {"type": "mingru", "mixer": {"width": width}, "mlp": None if mlp is None else {"kind": "dense", "ff": mlp}}


def config(vocab, width, layers, groups=1, eps=1e-5, mult=1.0):
    return {"architecture": "Rasizen", "vocab": vocab, "width": width, "residual_mult": mult,
            "norm": {"eps": eps, "groups": groups}, "layers": layers}


# K: attention first, two readers of one latent (one with a wider window than the writer, one that sees
# everything), recurrences with and without a feed-forward, part of the rotated numbers passing unturned.
# L: one group, no multiplier, a window of one page and one token, a layer without a window, one head.
# M: sizes that are no multiple of 8 (the projections then take the plain product), three groups.
CONFIGS = {
    "K": config(160, 96, [
        latent(4, 16, 8, 24, 40, 0.2, 37, base=500.0, dims=4, mlp=80),
        gru(64, mlp=112),
        latent(2, 24, 8, 16, 40, 0.15, 70, base=500.0, dims=4, kv_from=0),
        gru(136),
        latent(3, 8, 8, 8, 40, 0.3, 0, base=500.0, dims=4, kv_from=0, mlp=64),
    ], groups=4, eps=3e-4, mult=0.6),
    "L": config(200, 64, [
        gru(64),
        latent(1, 32, 16, 48, 24, 0.125, 65, base=1e6),
        latent(5, 8, 2, 8, 16, 0.4, 0, base=20.0, mlp=96),
        latent(2, 8, 2, 16, 16, 0.5, 1, base=20.0, kv_from=2),
    ], groups=1, eps=1e-6, mult=1.0),
    "M": config(131, 60, [
        latent(3, 10, 6, 14, 20, 0.3, 9, base=100.0, mlp=52),
        gru(44, mlp=36),
        latent(2, 6, 6, 10, 20, 0.25, 130, base=100.0, kv_from=0),
    ], groups=3, eps=1e-5, mult=0.35),
}
SEEDS = {"K": 11, "L": 12, "M": 13}
_FOLDERS, _PLAIN, _ENGINES, _WANT = {}, {}, {}, {}


def sharpen(w):
    """Random N(0, 0.02) projections give scores and gates near zero, where a softmax is flat and a
    sigmoid is 1/2.  Scale what feeds them so that scores spread over several units and the gates
    of the recurrence move: a wrong window, position or state then shows in the logits."""
    out = {}
    for name, a in w.items():
        f = 1.0
        if name.endswith((".mix.q", ".mix.dkv", ".mix.z", ".mix.x", ".mix.g")):
            f = 12.0
        elif name.endswith((".mix.uk", ".mix.uv", ".mix.o", ".mlp.up", ".mlp.down")):
            f = 5.0
        elif name.endswith((".z.b", ".x.b")):
            f = 30.0
        out[name] = a * f if f != 1.0 else a
    return out


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    """name -> folder with config.json and bfloat16 weights (sharpened as above)."""
    from safetensors.torch import load_file, save_file
    from sonicboom_amd.weights import write_random_model
    for name, cfg in CONFIGS.items():
        if name in _FOLDERS:
            continue
        folder = str(tmp_path_factory.mktemp(f"rasizen_{name}"))
        write_random_model(folder, json.loads(json.dumps(cfg)), seed=SEEDS[name], dtype="bfloat16", device=None)
        path = os.path.join(folder, "model.safetensors")
        w = sharpen({k: v.float() for k, v in load_file(path).items()})
        save_file({k: v.to(BF16).contiguous() for k, v in w.items()}, path, metadata={"format": "pt"})
        _FOLDERS[name] = folder
        _PLAIN[name] = {k: v.float().numpy().astype(np.float64) for k, v in load_file(path).items()}
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
        _WANT[key] = R.forward(CONFIGS[name], _PLAIN[name], list(tokens))
    return _WANT[key]


def prompts(name, lengths, seed=0):
    rng = np.random.default_rng(seed)
    return [[int(t) for t in rng.integers(0, CONFIGS[name]["vocab"], size=n)] for n in lengths]


# Bounds.  float32 differs from the plain implementation (float64) by the rounding of float32 sums.
# bfloat16 is measured in spreads of the logits (their standard deviation): the largest difference
# and the root mean square of all differences of a request.
F32_BOUND = 2e-4
BF16_WORST, BF16_RMS = 0.28, 0.019      # what the whole file measured (0.2007 and 0.0135: the models are sharpened) times 1.4
helpers.BF16_MAX["recurrent and latent"], helpers.BF16_RMS["recurrent and latent"] = BF16_WORST, BF16_RMS


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
        seen = helpers.BF16_SEEN.setdefault("recurrent and latent", [0.0, 0.0])      # the test run's summary prints them
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
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_whole_requests_and_the_first_tokens(folders, name, dtype):
    eng = engine_for(folders[name], dtype)
    for tokens in prompts(name, [1, 2, 3, 63, 64, 65, 200]):
        close(run_whole(eng, tokens), want_logits(name, tokens), dtype, f"{name} whole n={len(tokens)}")
    assert eng.cache.held_pages() == 0 and not eng.cache.live_slots


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
    """Nine pages: every batch fills eight of them, the next gets used pages, slots and state rows."""
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
    """A step of more rows than the engine takes at once is cut inside sequences; state and rows go on."""
    eng = engine_for(folders["K"], dtype, max_tokens=64 * 12, max_step_rows=100)
    reqs = prompts("K", [130, 7, 220], seed=5)
    got = run_batch(eng, reqs, [130, 7, 220])
    for r, g in zip(reqs, got):
        close(g, want_logits("K", r), dtype, f"portions, request of {len(r)}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["K", "L"])
def test_long_decoding_through_the_decode_loop(folders, name, dtype):
    """150 single-token steps of two sequences past windows and page borders, kernel by kernel and then
    replayed from the recorded step; logits of every step against the plain implementation."""
    eng = engine_for(folders[name], dtype)
    reqs = prompts(name, [60 + 150, 3 + 150], seed=7)
    heads = [60, 3]
    from sonicboom_amd.engine import StepEntry
    slots = [eng.alloc_slot() for _ in reqs]
    try:
        eng.step([StepEntry(s, r[:h], ()) for s, r, h in zip(slots, reqs, heads)])
        loop = eng.decode_loop()
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
    for name in ("K", "M"):
        ps = prompts(name, [4, 70, 19], seed=9)
        session = Model.load(folders[name], dtype="float32").session(max_tokens=64 * 8)
        got = session.generate(ps, max_tokens=12, stop_tokens=())
        assert got == [R.greedy(CONFIGS[name], _PLAIN[name], p, 12) for p in ps]
        assert [session.generate([p], max_tokens=12, stop_tokens=())[0] for p in ps] == got
        assert not session.engine.cache.live_slots
        # bfloat16: every chosen token is the plain implementation's best or within rounding of it
        session = Model.load(folders[name], dtype="bfloat16").session(max_tokens=64 * 8)
        for p, out in zip(ps, session.generate(ps, max_tokens=12, stop_tokens=())):
            logits = want_logits(name, p + out)
            for i, t in enumerate(out):
                row = logits[len(p) - 1 + i]
                assert row[t] >= row.max() - 2 * BF16_WORST * row.std(), (name, i)


def test_command_line_and_trace_replay(folders, tmp_path):
    """The command line generates from a folder and from a configuration file of this design; the
    replay program feeds a prompt, then its next tokens one by one beside a second request, frees
    one and goes on, and writes the logits the plain implementation gives."""
    import subprocess
    import sys
    from conftest import ROOT
    name = "M"
    ps = prompts(name, [4, 10], seed=9)
    tokens = tmp_path / "prompts.txt"
    tokens.write_text("\n".join(" ".join(map(str, p)) for p in ps) + "\n")
    cmd = [sys.executable, os.path.join(ROOT, "bin", "sb-gen"), "-m", folders[name], "--tokens", str(tokens), "-n", "6",
           "--dtype", "fp32", "--stop", ""]
    out = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr
    got = [[int(t) for t in line.split()] for line in out.stdout.strip().splitlines()]
    assert got == [R.greedy(CONFIGS[name], _PLAIN[name], p, 6) for p in ps]
    cfg_file = tmp_path / "config.json"
    cfg_file.write_text(json.dumps(CONFIGS["L"]))
    cmd = [sys.executable, os.path.join(ROOT, "bin", "sb-gen"), "--random", str(cfg_file), "--seed", "3",
           "--tokens", str(tokens), "-n", "5", "--temperature", "0.8", "--sample-seed", "11", "--top-k", "20"]
    one = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    two = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert one.returncode == 0 and one.stdout == two.stdout and len(one.stdout.split()) == 10, one.stderr
    # replay
    a, b = prompts(name, [75, 12], seed=10)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:70], "want": [0, 69]}, {"id": "b", "tokens": b[:9], "want": [8]}], "end": []}]
    for k in range(3):
        steps.append({"step": k + 1, "entries": [{"id": "a", "tokens": [a[70 + k]], "want": [0]},
                                                 {"id": "b", "tokens": [b[9 + k]], "want": [] if k == 1 else [0]}],
                      "end": ["b"] if k == 2 else []})
    steps.append({"step": 4, "entries": [{"id": "a", "tokens": a[73:75], "want": [1]}], "end": ["a"]})
    outdir = tmp_path / "out"
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folders[name], "--dtype", "float32",
                          "--out", str(outdir), "--max-tokens", "256"], input="\n".join(json.dumps(x) for x in steps) + "\n",
                         capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr
    assert [ln for ln in run.stdout.splitlines() if ln.startswith("done")] == [f"done {i}" for i in range(5)]
    wa, wb = want_logits(name, a), want_logits(name, b)
    vocab = CONFIGS[name]["vocab"]
    read = lambda i: np.fromfile(outdir / f"{i}.f32", dtype="<f4").reshape(-1, vocab)
    close(read(0), np.stack([wa[0], wa[69], wb[8]]), "float32", "replay, prompts")
    close(read(1), np.stack([wa[70], wb[9]]), "float32", "replay, first single tokens")
    close(read(2), wa[71:72], "float32", "replay, a step where one request wants nothing")
    close(read(3), np.stack([wa[72], wb[11]]), "float32", "replay, last step of the short request")
    close(read(4), wa[74:75], "float32", "replay, two more tokens alone")
    # many short requests at once, with no more --max-tokens than the tokens they hold: every one of them
    # takes a page of its own in the cache, which the program makes room for
    shorts = prompts(name, [3] * 14, seed=12)
    steps = [{"step": 0, "entries": [{"id": f"s{i}", "tokens": p[:2], "want": [1]} for i, p in enumerate(shorts)], "end": []},
             {"step": 1, "entries": [{"id": f"s{i}", "tokens": p[2:], "want": [0]} for i, p in enumerate(shorts)],
              "end": [f"s{i}" for i in range(14)]}]
    outdir2 = tmp_path / "out2"
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folders[name], "--dtype", "bfloat16",
                          "--out", str(outdir2), "--max-tokens", str(3 * 14)], input="\n".join(json.dumps(x) for x in steps) + "\n",
                         capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr
    got = np.fromfile(outdir2 / "1.f32", dtype="<f4").reshape(-1, vocab)
    close(got, np.stack([want_logits(name, p)[2] for p in shorts]), "bfloat16", "replay, fourteen short requests")


# ---- mechanisms alone ---------------------------------------------------------------------------
def runtime(dtype):
    from sonicboom_amd.parts import Runtime
    return Runtime(torch.device(DEV), TORCH_DT[dtype], True)


def rand(*shape, scale=1.0, seed=0):
    g = torch.Generator().manual_seed(1000 * seed + sum(shape) + len(shape))
    return torch.randn(*shape, generator=g) * scale


def part_tensors(spec, dtype, seed=0, scale=0.3):
    dev, ref = {}, {}
    for i, t in enumerate(spec.all_tensors()):
        a = (rand(*t.shape, scale=scale, seed=seed + i) + t.init[0]).to(TORCH_DT[dtype])
        dev[t.name], ref[t.name] = a.to(DEV), a.float().numpy().astype(np.float64)
    return dev, ref


def part_close(got, want, dtype, what):
    got, want = got.detach().float().cpu().numpy().astype(np.float64), np.asarray(want, dtype=np.float64)
    scale = max(float(np.abs(want).max()), 1e-30)
    err = np.abs(got - want).max() / scale
    assert got.shape == want.shape and err <= (2e-5 if dtype == "float32" else 2.5e-2), f"{what}: off by {err:.3g} of the largest value"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width, groups", [(96, 1), (96, 2), (60, 3), (520, 4), (4096, 2), (66, 6), (35, 5)])
def test_grouped_norm_alone(dtype, width, groups):
    from sonicboom_amd.parts import build_part
    from sonicboom_amd.parts.norm import rmsnorm_spec
    spec = rmsnorm_spec("n", width, 2e-3, groups)
    dev, ref = part_tensors(spec, dtype)
    norm = build_part(spec, dev, runtime(dtype))
    x = rand(7, width, scale=3.0)
    x[:, : width // groups] *= 20.0                 # one group much larger than the others: a norm over the whole row shows
    part_close(norm.forward(x.to(DEV), TORCH_DT[dtype]), R.grouped_rms_norm(x.numpy(), ref["n"], 2e-3, groups), dtype, "norm")
    rows = torch.tensor([5, 0, 5], dtype=torch.int32, device=DEV)
    part_close(norm.forward(x.to(DEV), TORCH_DT[dtype], rows=rows),
               R.grouped_rms_norm(x.numpy()[[5, 0, 5]], ref["n"], 2e-3, groups), dtype, "norm of picked rows")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows", [3, 70, 300])
def test_dense_feed_forward_alone(dtype, rows):
    from sonicboom_amd.parts import build_part
    from sonicboom_amd.parts.ffn import dense_ffn_spec
    from sonicboom_amd.parts.norm import rmsnorm_spec
    spec = dense_ffn_spec("up", "down", 72, 200, "xielu", act_name="act", out_scale=0.7)
    dev, ref = part_tensors(spec, dtype)
    ffn = build_part(spec, dev, runtime(dtype))
    nspec = rmsnorm_spec("n", 72, 1e-5, 3)
    ndev, nref = part_tensors(nspec, dtype, seed=9)
    norm = build_part(nspec, ndev, runtime(dtype))
    h, x = rand(rows, 72, scale=2.0).to(TORCH_DT[dtype]), rand(rows, 72, seed=5)
    xd = x.to(DEV)
    normed = ffn.forward(h.to(DEV), xd, None, then_norm=norm)
    w = {"m.up": ref["up"], "m.down": ref["down"], "m.act": ref["act"]}
    want = x.numpy() + 0.7 * R.dense_ff(h.float().numpy(), w, "m.")
    part_close(xd, want, dtype, "feed-forward")
    if normed is not None:                          # the last pass applied the next norm as well
        part_close(normed, R.grouped_rms_norm(xd.cpu().numpy(), nref["n"], 1e-5, 3), dtype, "norm in the last pass")
    z = np.linspace(-6, 6, 25)
    assert np.allclose(R.xielu(z, 0.3, -0.2)[z > 0], np.log1p(np.exp(0.3)) * z[z > 0] ** 2 + z[z > 0] / 2)


def mixer_harness(mixer, rt, n_tokens_cap=64 * 16):
    """A cache for one mixer alone, and a function that feeds rows of one sequence in cuts."""
    from sonicboom_amd.cache import PagedCache, group_entries
    from sonicboom_amd.engine.model import LayerBinding
    from sonicboom_amd.engine.step import StepContext, StepEntry
    cs, ss = mixer.cache_spec(), mixer.state_spec()
    groups = group_entries({0: cs.key()}) if cs is not None else []
    cache = PagedCache(groups, n_tokens_cap, rt.cache_dtype, rt.device,
                       {0: (tuple(ss.shape), ss.dtype)} if ss is not None else None, max_slots=4)
    tiles = getattr(mixer, "row_tile", None) or ()
    tiles = (tiles,) if isinstance(tiles, int) else tuple(tiles)

    def feed(h_rows, cuts, width):
        k = v = g = None
        if cs is not None:
            k, v, g = cache.entry_views(0)
        binding = LayerBinding(0, g, k, v, cs is not None, cache.state.get(0))
        slot = cache.alloc_slot()
        outs, at = [], 0
        try:
            for n in cuts:
                cache.reserve([slot], [n])
                ctx = StepContext(cache, [StepEntry(slot, [0] * n, ())], rt.device, tiles)
                x = torch.zeros((n, width), dtype=F32, device=DEV)
                mixer.forward(h_rows[at:at + n].to(DEV).contiguous(), x, ctx, binding)
                cache.advance([slot], [n])
                outs.append(x)
                at += n
        finally:
            cache.free_slot(slot)
        return torch.cat(outs)
    return feed


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width, inner", [(48, 80), (40, 300), (64, 24)])
def test_mingru_alone(dtype, width, inner):
    """Whole, in portions longer and shorter than a chunk of the parallel form, and token by token."""
    from sonicboom_amd.parts import build_part
    from sonicboom_amd.parts.recurrent import mingru_spec
    spec = mingru_spec("m.", width, inner, out_scale=1.0)
    dev, ref = part_tensors(spec, dtype, scale=0.6)
    rt = runtime(dtype)
    feed = mixer_harness(build_part(spec, dev, rt), rt)
    n = 300
    h = rand(n, width, scale=1.5).to(TORCH_DT[dtype])
    want = R.mingru_mixer(h.float().numpy(), ref, "m.")
    for cuts in ([n], [2, 2, 130, 65, 64, 1, 36], [1] * 20 + [280]):
        part_close(feed(h, cuts, width), want, dtype, f"mingru cuts {cuts[:3]}")
    # the candidate's two branches, and a state that starts from what the last step left
    z, cand = R.mingru_gates(h.float().numpy(), ref, "m.")
    assert (cand[cand >= 0.5] >= 0.5).all() and (cand > 0).all()
    s = R.mingru_scan(z, cand)
    assert np.allclose(R.mingru_scan(z[100:], cand[100:], start=s[99]), s[100:])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, dim, rot_dim, dims, vdim, rank, window", [
    (3, 16, 8, 8, 24, 32, 50), (1, 8, 16, 6, 8, 72, 0), (5, 24, 4, 4, 40, 16, 64), (2, 6, 2, 2, 10, 20, 1)])
def test_latent_attention_alone(dtype, heads, dim, rot_dim, dims, vdim, rank, window):
    from sonicboom_amd.parts import build_part
    from sonicboom_amd.parts.latent_attention import latent_attention_spec
    from sonicboom_amd.parts.position import rope_interleaved_spec
    width, n = 56, 200
    spec = latent_attention_spec("a.", width, heads, dim, rot_dim, vdim, rank, 0.3, rope_interleaved_spec(dims, 300.0),
                                 window=window, eps=1e-4)
    dev, ref = part_tensors(spec, dtype, scale=0.5)
    rt = runtime(dtype)
    feed = mixer_harness(build_part(spec, dev, rt), rt)
    h = rand(n, width).to(TORCH_DT[dtype])
    mx = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank, "scale": 0.3,
          "rot": {"base": 300.0, "dims": dims}, "mask": {"size": window}}
    pos = np.arange(n)
    want = R.latent_attention_mixer(h.float().numpy(), pos, ref, "a.", mx, 1e-4,
                                    R.latent_kv(h.float().numpy(), pos, ref, "a.", mx, 1e-4))
    for cuts in ([n], [70, 2, 60] + [1] * 68):
        part_close(feed(h, cuts, width), want, dtype, f"latent attention cuts {cuts[:3]}")


def planted_mixer(dtype, window, heads=2, dim=8, rot_dim=4, vdim=12, rank=16, width=32, gain=14.0):
    """A latent-attention mixer whose weights are set by hand: the latent reads the input's first
    `rank` numbers, the plain query part the `dim` numbers behind them, and W_uk picks the latent's
    first `dim` again.  A row whose input has number `rank` set then asks for keys whose input has
    number 0 set, and scores nothing on rows without it; rotated parts are zero; values, gate and
    output are random."""
    from sonicboom_amd.parts import build_part
    from sonicboom_amd.parts.latent_attention import latent_attention_spec
    from sonicboom_amd.parts.position import rope_interleaved_spec
    spec = latent_attention_spec("a.", width, heads, dim, rot_dim, vdim, rank, 1.0, rope_interleaved_spec(rot_dim, 100.0),
                                 window=window, eps=1e-6)
    t = {s.name: torch.zeros(s.shape) for s in spec.all_tensors()}
    for a in range(heads):
        for d in range(dim):
            t["a.q"][a * (dim + rot_dim) + d, rank + d] = 1.0
            t["a.uk"][a * dim + d, d] = 1.0
    t["a.q"] *= gain / np.sqrt(rank)
    for i in range(rank):
        t["a.dkv"][i, i] = 1.0
    t["a.dkv.norm"][:] = 1.0
    t["a.uv"], t["a.g"], t["a.o"] = rand(heads * vdim, rank, seed=1), rand(heads * vdim, width, seed=2), rand(width, heads * vdim, scale=0.3, seed=3)
    rt = runtime(dtype)
    dev = {k: v.to(TORCH_DT[dtype]).to(DEV) for k, v in t.items()}
    ref = {k: v.to(TORCH_DT[dtype]).float().numpy().astype(np.float64) for k, v in t.items()}
    mx = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank, "scale": 1.0,
          "rot": {"base": 100.0, "dims": rot_dim}, "mask": {"size": window}}
    return build_part(spec, dev, rt), rt, ref, mx, width


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [0, 100, 64, 129])
def test_one_key_stands_out(dtype, window):
    """A prompt of 700 rows in which the last row asks and one row answers (see planted_mixer): the
    query's whole weight falls on that key when it sees it, and spreads evenly when it does not.
    The key is planted far back, at both sides of page borders, and just inside and just outside the
    window; the query runs as the last row of a prompt and as a single decoded row.  The result with
    the key seen and with it hidden differ by far more than any bound here."""
    mixer, rt, ref, mx, width = planted_mixer(dtype, window)
    feed = mixer_harness(mixer, rt)
    n = 700
    t = n - 1
    back = [1, 2, 63, 64, 65, 127, 128, 129, 500, 699]
    if window:
        back += [window - 2, window - 1, window, window + 1]
    seen_differs = 0
    for b in sorted(set(back)):
        j = t - b
        if j < 0:
            continue
        h = rand(n, width, seed=b)
        h[:, 0] = 0.0                 # no key answers ...
        h[:, 16:24] = 0.0             # ... and no row asks,
        h[j, 0], h[t, 16] = 8.0, 2.0  # but for these two
        h = h.to(TORCH_DT[dtype])
        hn = h.float().numpy()
        pos = np.arange(n)
        kv = R.latent_kv(hn, pos, ref, "a.", mx, 1e-6)
        want = R.latent_attention_mixer(hn, pos, ref, "a.", mx, 1e-6, kv)
        for cuts in ([n], [n - 1, 1], [300, 336, 63, 1]):
            got = feed(h, cuts, width)
            part_close(got[t:], want[t:], dtype, f"window {window}, key {b} back, cuts {cuts}")
        # what the row would be if the planted key were hidden (or seen) the other way round
        flipped = dict(mx, mask={"size": b if (window == 0 or b < window) else b + 1})
        other = R.latent_attention_mixer(hn, pos, ref, "a.", flipped, 1e-6, kv)
        if np.abs(other[t] - want[t]).max() > 0.2 * np.abs(want[t]).max():
            seen_differs += 1
    assert seen_differs >= len(set(back)) - 3, "the planted key does not decide the result: the test shows nothing"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows, heads, n_in, n_out", [(37, 3, 20, 45), (100, 2, 24, 72), (5, 17, 128, 40), (300, 1, 8, 200)])
def test_head_products_and_activation_alone(dtype, rows, heads, n_in, n_out):
    """The per-head products, plain and (bfloat16, inner sizes in eights) on the matrix cores: into a
    wider output of which only a head's own numbers may be written, with and without the gate."""
    from sonicboom_amd import ops
    dt = TORCH_DT[dtype]
    x, w = rand(rows, heads, n_in).to(dt), rand(heads, n_out, n_in, scale=0.3).to(dt)
    gate = rand(rows, heads * n_out + 16, seed=4).to(DEV)
    want = np.einsum("tai,aoi->tao", x.float().numpy().astype(np.float64), w.float().numpy().astype(np.float64))
    for g in (None, gate[:, 8:8 + heads * n_out]):
        out = torch.zeros((rows, heads, n_out + 8), dtype=dt, device=DEV)
        ops.head_product(x.to(DEV), w.to(DEV), out, gate=g)
        ref = want if g is None else want * R.sigmoid(g.cpu().numpy().reshape(rows, heads, n_out))
        part_close(out[:, :, :n_out], ref, dtype, "head product")
        assert float(out[:, :, n_out:].abs().max()) == 0.0        # only a head's own numbers are written
    z = torch.linspace(-9, 9, 400)
    p = torch.tensor([0.4, -0.3]).to(dt)
    got = ops.activate(z.to(DEV), dt, "xielu", p.to(DEV))
    part_close(got, R.xielu(z.numpy(), float(p[0]), float(p[1])), dtype, "xielu")


@pytest.mark.parametrize("heads, dim, rot_dim, vdim, rank, window", [
    (4, 32, 16, 24, 64, 0), (20, 16, 8, 16, 40, 100), (3, 64, 32, 40, 256, 70), (2, 128, 64, 128, 512, 130)])
def test_matrix_core_latent_attention_equals_the_plain_kernel(heads, dim, rot_dim, vdim, rank, window):
    """bfloat16, the sizes of each compiled shape of the matrix-core kernel: a prompt, portions, and
    single rows (where a wave takes 16 heads of a row) against the kernel of one wave per (row, head)."""
    from sonicboom_amd.parts import build_part
    from sonicboom_amd.parts.latent_attention import latent_attention_spec
    from sonicboom_amd.parts.position import rope_interleaved_spec
    from sonicboom_amd.parts import Runtime
    width, n = 64, 330
    spec = latent_attention_spec("a.", width, heads, dim, rot_dim, vdim, rank, 0.5, rope_interleaved_spec(rot_dim, 1e4),
                                 window=window, eps=1e-5)
    dev, ref = part_tensors(spec, "bfloat16", scale=0.5)
    h = rand(n, width).to(BF16)
    outs = {}
    for fast in (True, False):
        rt = Runtime(torch.device(DEV), BF16, fast)
        mixer = build_part(spec, dict(dev), rt)
        assert (getattr(mixer, "row_tile", None) is not None) == fast
        feed = mixer_harness(mixer, rt)
        outs[fast] = [feed(h, cuts, width) for cuts in ([n], [200, 66] + [1] * 64)]
    for a, b in zip(outs[True], outs[False]):
        part_close(a, b.float().cpu().numpy(), "bfloat16", "matrix-core against plain")
    part_close(outs[True][1], outs[True][0].float().cpu().numpy(), "bfloat16", "portions and single rows against whole")


@pytest.mark.parametrize("rows, n_out, n_in", [(300, 96, 64), (1000, 520, 256), (129, 40, 72)])
def test_tiled_product_adds_into_the_stream_with_a_multiplier(rows, n_out, n_in):
    """resid += scale * (x W^T + b) in the tiled product's epilogue, against the product followed by the scaled add."""
    from sonicboom_amd import ops
    x, w, b = rand(rows, n_in).to(BF16), rand(n_out, n_in, scale=0.2, seed=1).to(BF16), rand(n_out, seed=2)
    resid = rand(rows, n_out, seed=3)
    got = resid.to(DEV)
    assert ops.gemm_bf16_add_scaled(x.to(DEV), ops.pack_weight(w.to(DEV)), b.to(DEV), got, 0.3, (n_out, n_in))
    want = resid.numpy().astype(np.float64) + 0.3 * (x.float().numpy().astype(np.float64) @ w.float().numpy().astype(np.float64).T + b.numpy())
    assert np.abs(got.cpu().numpy() - want).max() <= 1e-4 * max(1.0, np.abs(want).max())
    # a multiplier of one gives the bits of the product's plain residual form
    one, plain = resid.to(DEV), resid.to(DEV)
    assert ops.gemm_bf16_add_scaled(x.to(DEV), ops.pack_weight(w.to(DEV)), b.to(DEV), one, 1.0, (n_out, n_in))
    ops.gemm_bf16(x.to(DEV), ops.pack_weight(w.to(DEV)), b.to(DEV), plain, F32, plain, packed_shape=(n_out, n_in))
    assert torch.equal(one, plain)
