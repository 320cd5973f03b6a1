"""Putulorn through the engine (checkpoint loader, registry, slots, paged cache, replay and generation entry points)
against the plain float64 oracle in putulorn_oracle.py.  Every test runs on the CPU (reference ops: model, cache,
state and scheduler logic) and, marked gpu, on the HIP kernels.  Small own configurations, random weights."""

import copy

import pytest
import torch

import putulorn_oracle as oracle
from k8s_llm_scheduler_amd.engine import SamplingParams, build_engine
from k8s_llm_scheduler_amd.models import load_config, model_class
from k8s_llm_scheduler_amd.models.putulorn import (PutulornModel, config_from_json, config_to_json, random_tensors,
                                                   save_checkpoint)

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
TOL = {"float32": 3e-4, "bfloat16": 6e-2}


def latent(heads=3, dim=12, rot_dim=8, vdim=10, kv_rank=20, window=6, dims=None, base=5000.0, scale=0.31):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank,
         "rot": {"dims": rot_dim if dims is None else dims, "base": base}, "scale": scale}
    if window:
        m["mask"] = {"size": window}
    return {"type": "latent_attention", "mixer": m, "mlp": None}


def wkv(heads=2, dim=20):
    return {"type": "wkv", "mixer": {"heads": heads, "dim": dim}, "mlp": None}


def dense(ff=40):
    return {"kind": "dense", "ff": ff}


def moe(experts=6, top=3, ff=12, scale=1.7, limit=0.8, shared=True, shared_limit=1.3):
    d = {"kind": "moe", "router": {"experts": experts, "top": top, "scale": scale},
         "expert": {"ff": ff, **({"limit": limit} if limit else {})}}
    if shared:
        d["shared"] = {"ff": ff + 4, **({"limit": shared_limit} if shared_limit else {})}
    return d


def with_mlp(layer, mlp):
    layer = copy.deepcopy(layer)
    layer["mlp"] = mlp
    return layer


def config(layers, width=48, vocab=90, loop=None, mult=0.6, eps=1e-5):
    c = {"architecture": "Putulorn", "vocab": vocab, "width": width, "layers": layers, "norm": {"eps": eps},
         "residual_mult": mult}
    if loop:
        c["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return c


FULL = config([with_mlp(latent(), dense()), with_mlp(wkv(), moe()), with_mlp(latent(window=9, dims=4), moe(top=1, shared=False, limit=0)),
               wkv(heads=3, dim=16)], loop=(1, 3, 3))


# bfloat16 comparisons: no top-1 routing, where one close call of a router in bf16 replaces a row's whole feed-forward
SOFT = config([with_mlp(latent(), dense()), with_mlp(wkv(), moe()), with_mlp(latent(window=9, dims=4), dense(20)),
               wkv(heads=3, dim=16)], loop=(1, 3, 2))


def model_for(dtype):
    return FULL if dtype == "float32" else SOFT


def make(tmp_path, cfg, device, dtype, seed=0, max_tokens=256, slots=4, graphs=False, scale_embed=None):
    pc = config_from_json(cfg, "case")
    tensors = random_tensors(pc, seed)
    if scale_embed:
        for tok, f in scale_embed.items():
            tensors["embed"][tok] *= f
    save_checkpoint(pc, tensors, tmp_path / "ckpt")
    eng = build_engine(weights=str(tmp_path / "ckpt"), device=device, dtype=dtype, max_batch=slots, block_size=16,
                       num_blocks=max_tokens // 16, max_model_len=max_tokens, cuda_graphs=graphs, capture=graphs)
    assert isinstance(eng.model, PutulornModel)
    return eng, tensors


def row_errs(got, want):
    """Per row: rms of the difference (its mean taken off) over the rms of the centred expected row."""
    got, want = got.double(), want.double()
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    w = want - want.mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / w.pow(2).mean(-1).sqrt().clamp_min(1e-9)


def rel_err(got, want):
    return row_errs(got, want).max().item()


def close(got, want, dtype):
    """float32: every row within rounding.  bfloat16: rows are within bf16 rounding of a few layers, except that a
    router's close call may pick another expert for a row in bf16 -- nine rows in ten must be tight, none far off."""
    e = row_errs(got, want)
    if dtype == "float32":
        return e.max().item() < TOL[dtype]
    return e.quantile(0.9).item() < TOL[dtype] and e.max().item() < 0.3


def tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def whole(eng, key, toks):
    return eng.replay_step([(key, toks, list(range(len(toks))))], [key])


# ----------------------------------------------------------------------------- registry, configuration, loader
def test_registry_and_config_roundtrip(tmp_path):
    pc = config_from_json(FULL, "x")
    assert config_to_json(pc) == {**FULL, "layers": config_to_json(pc)["layers"]}
    assert config_from_json(config_to_json(pc), "x") == pc
    save_checkpoint(pc, random_tensors(pc, 1), tmp_path / "m")
    got = load_config(str(tmp_path / "m"))
    assert model_class(got) is PutulornModel and got.runs() == pc.runs()
    assert [r for r in pc.runs()] == [(0, None), (1, 0), (2, None), (1, 1), (2, None), (1, 2), (2, None), (3, None)]
    assert model_class(load_config("tiny")).__name__ == "LlamaModel"
    assert model_class(load_config("putulorn-tiny")) is PutulornModel


# ----------------------------------------------------------------------------- each mechanism alone
MECHANISMS = {
    "wkv": config([wkv()]),
    "wkv_wide_heads": config([wkv(heads=1, dim=48)]),                       # heads * dim == width, one head
    "latent_window": config([latent()]),
    "latent_no_window": config([latent(window=0)]),
    "latent_partial_rotation": config([latent(dims=4, window=5)]),          # rot.dims < rot_dim: the rest passes
    "latent_no_rotation": config([latent(rot_dim=0, dims=0, window=4)]),
    "latent_one_head": config([latent(heads=1, dim=16, vdim=16, kv_rank=16, window=3)]),
    "dense_ff": config([with_mlp(wkv(), dense())]),
    "moe_shared": config([with_mlp(wkv(), moe())]),
    "moe_top1_unclamped_no_shared": config([with_mlp(latent(), moe(top=1, limit=0, shared=False, scale=1.0))]),
    "moe_all_experts": config([with_mlp(wkv(), moe(experts=3, top=3))]),
    "loop_whole_model": config([with_mlp(wkv(), dense()), latent()], loop=(0, 2, 2), mult=1.0),
    "loop_once": config([latent(), wkv()], loop=(1, 2, 1)),
}


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", sorted(MECHANISMS))
def test_mechanism_alone(tmp_path, device, name):
    cfg = MECHANISMS[name]
    eng, tensors = make(tmp_path, cfg, device, "float32")
    toks = tokens(37, cfg["vocab"], 3)
    assert rel_err(whole(eng, "a", toks), oracle.forward(cfg, tensors, toks)) < TOL["float32"]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_full_model_and_layer_streams(tmp_path, device, dtype):
    cfg = model_for(dtype)
    eng, tensors = make(tmp_path, cfg, device, dtype)
    toks = tokens(45, cfg["vocab"], 4)
    streams = []
    want = oracle.forward(cfg, tensors, toks, streams)
    assert close(whole(eng, "a", toks), want, dtype)
    # the residual stream after every layer run (a looped layer counts each time)
    m, dev = eng.model, eng.device
    T = len(toks)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)
    b = m.batch_meta(i32(list(range(T))), i32(list(range(T))), i32([0, T]), i32([list(range(16))]), i32([0]))
    got = m.residual_after_runs(i32(toks), b)
    assert len(got) == len(streams) == len(oracle.layer_order(cfg))
    for g, w in zip(got, streams):
        assert close(g.cpu(), w, dtype)


# ----------------------------------------------------------------------------- cutting, batching, reuse
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_prefill_against_token_by_token(tmp_path, device, dtype):
    cfg = model_for(dtype)
    eng, tensors = make(tmp_path, cfg, device, dtype)
    toks = tokens(40, cfg["vocab"], 5)
    want = oracle.forward(cfg, tensors, toks)
    rows = [eng.replay_step([("s", [t], [0])], ["s"] if i == len(toks) - 1 else []) for i, t in enumerate(toks)]
    assert close(torch.cat(rows), want, dtype)
    assert len(eng.free_slots) == eng.max_batch and eng.allocator.num_free == eng.num_blocks


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("sizes", [[2, 2, 2, 3, 1, 1, 29], [17, 16, 1, 6], [1, 15, 16, 8], [39, 1], [5] * 8])
def test_portions(tmp_path, device, sizes):
    eng, tensors = make(tmp_path, FULL, device, "float32")
    toks = tokens(sum(sizes), FULL["vocab"], 6)
    want = oracle.forward(FULL, tensors, toks)
    rows, at = [], 0
    for n in sizes:
        rows.append(eng.replay_step([("p", toks[at:at + n], list(range(n)))]))
        at += n
    assert rel_err(torch.cat(rows), want) < TOL["float32"]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_unequal_batch_against_each_alone_with_reuse(tmp_path, device, dtype):
    """Four slots and 96 cache tokens for six requests of unequal length: portions of some beside single tokens of
    others, requests left out of steps, slots and blocks taken again by later requests."""
    cfg = model_for(dtype)
    eng, tensors = make(tmp_path, cfg, device, dtype, max_tokens=96, slots=4)
    V = cfg["vocab"]
    seqs = {k: tokens(n, V, 10 + i) for i, (k, n) in enumerate([("a", 30), ("b", 7), ("c", 18), ("d", 1), ("e", 33),
                                                                 ("f", 20)])}
    want = {k: oracle.forward(cfg, tensors, v) for k, v in seqs.items()}
    plan = [  # (key, count) per step
        [("a", 11), ("b", 3)],
        [("a", 1), ("b", 2), ("c", 9), ("d", 1)],            # d ends: its slot is free again
        [("a", 1), ("c", 2)],                                 # b left out
        [("a", 1), ("b", 1), ("c", 1), ("e", 5)],             # e takes d's slot
        [("a", 16), ("b", 1), ("c", 6), ("e", 2)],            # a, b, c end
        [("e", 1), ("f", 20)],                                # f in a freed slot and freed blocks
        [("e", 25)],
    ]
    at = {k: 0 for k in seqs}
    got = {k: [] for k in seqs}
    for step in plan:
        entries, end = [], []
        for k, n in step:
            entries.append((k, seqs[k][at[k]:at[k] + n], list(range(n))))
            at[k] += n
            if at[k] == len(seqs[k]):
                end.append(k)
        rows = eng.replay_step(entries, end)
        o = 0
        for k, n in step:
            got[k].append(rows[o:o + n])
            o += n
    assert at == {k: len(v) for k, v in seqs.items()}
    for k in seqs:
        assert close(torch.cat(got[k]), want[k], dtype), k
    assert len(eng.free_slots) == 4 and eng.allocator.num_free == eng.num_blocks


@pytest.mark.parametrize("device", DEVICES)
def test_reused_slot_starts_from_zero_state(tmp_path, device):
    """One slot, one request after another: the second must not see the first's recurrent state, shifted token or
    cached rows."""
    cfg = config([wkv(), latent(window=0)])
    eng, tensors = make(tmp_path, cfg, device, "float32", max_tokens=32, slots=1)
    a, b = tokens(30, cfg["vocab"], 1), tokens(25, cfg["vocab"], 2)
    whole(eng, "a", a)
    got = [eng.replay_step([("b", b[:9], list(range(9)))]), eng.replay_step([("b", b[9:], list(range(16)))], ["b"])]
    assert rel_err(torch.cat(got), oracle.forward(cfg, tensors, b)) < TOL["float32"]


# ----------------------------------------------------------------------------- windows, far keys, first tokens
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("window", [1, 2, 16, 17])
def test_window_edges_in_prompt_and_decoding(tmp_path, device, window):
    """A loud token (its embedding scaled, so its rotated key dominates the scores it takes part in) placed so that
    it is the oldest key inside the window of one query and just outside the next one's, in a prompt portion and
    among tokens decoded one by one, across block borders (block 16)."""
    cfg = config([latent(window=window, heads=2), with_mlp(latent(window=window + 3, heads=2), dense())], vocab=60)
    loud = 7
    eng, tensors = make(tmp_path, cfg, device, "float32", scale_embed={loud: 6.0})
    toks = [t if t != loud else 8 for t in tokens(70, 60, 8)]
    for p in (3, 14, 31, 40, 52):
        toks[p] = loud
    want = oracle.forward(cfg, tensors, toks)
    quiet = oracle.forward(cfg, tensors, [8 if t == loud else t for t in toks])
    assert rel_err(quiet, want) > 0.05                     # the loud token matters
    rows = [eng.replay_step([("w", toks[:36], list(range(36)))])]
    rows += [eng.replay_step([("w", [t], [0])]) for t in toks[36:]]
    got = torch.cat(rows)
    assert rel_err(got, want) < TOL["float32"]
    for p in (31, 40, 52):                                  # the rows around each edge, one by one
        for i in (p + window - 1, p + window):
            if i < len(toks):
                assert rel_err(got[i:i + 1], want[i:i + 1]) < TOL["float32"], (p, i)


@pytest.mark.parametrize("device", DEVICES)
def test_far_keys_and_long_decoding(tmp_path, device):
    """No window and a recurrent state: position 200+ still depends on the first tokens (checked on the oracle), over
    many block borders, with 90 tokens decoded one by one."""
    cfg = config([latent(window=0, heads=2), wkv(heads=2, dim=12), with_mlp(latent(window=150, heads=2), dense(24))],
                 width=32, vocab=50)
    eng, tensors = make(tmp_path, cfg, device, "float32", max_tokens=256, scale_embed={5: 5.0})
    toks = [t if t != 5 else 6 for t in tokens(215, 50, 9)]
    toks[1] = toks[64] = 5
    want = oracle.forward(cfg, tensors, toks)
    other = oracle.forward(cfg, tensors, [toks[0], 6] + toks[2:])
    assert rel_err(other[-1:], want[-1:]) > 1e-3            # the end sees position 1
    rows = [eng.replay_step([("f", toks[:100], list(range(100)))]), eng.replay_step([("f", toks[100:125], list(range(25)))])]
    rows += [eng.replay_step([("f", [t], [0])]) for t in toks[125:]]
    assert rel_err(torch.cat(rows), want) < TOL["float32"]


@pytest.mark.parametrize("device", DEVICES)
def test_first_tokens(tmp_path, device):
    eng, tensors = make(tmp_path, FULL, device, "float32")
    for n in (1, 2, 3):
        toks = tokens(n, FULL["vocab"], 20 + n)
        assert rel_err(whole(eng, f"s{n}", toks), oracle.forward(FULL, tensors, toks)) < TOL["float32"]
    toks = tokens(4, FULL["vocab"], 30)
    got = [eng.replay_step([("x", toks[:1], [0])]), eng.replay_step([("x", toks[1:2], [0])]),
           eng.replay_step([("x", toks[2:], [0, 1])], ["x"])]
    assert rel_err(torch.cat(got), oracle.forward(FULL, tensors, toks)) < TOL["float32"]


# ----------------------------------------------------------------------------- other sizes
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("case", range(3))
def test_other_sizes(tmp_path, device, case):
    cfg = [
        # wide latent (two accumulator columns per lane), many heads (more than the waves of a workgroup), big window
        config([with_mlp(latent(heads=10, dim=8, rot_dim=6, vdim=5, kv_rank=70, window=40, dims=6, scale=0.2), dense(33)),
                with_mlp(wkv(heads=5, dim=8), moe(experts=70, top=4, ff=6, scale=0.5, limit=2.5))], width=40, vocab=77,
               mult=1.0, eps=1e-6),
        # head dimension above one wave, experts without limits, a loop over the last layers
        config([wkv(heads=1, dim=72), with_mlp(latent(heads=2, dim=32, rot_dim=16, vdim=32, kv_rank=32, window=64, scale=1.0),
                                                moe(experts=2, top=2, ff=20, limit=0, shared_limit=0))],
               width=64, vocab=40, loop=(0, 2, 2), mult=0.25),
        # odd sizes everywhere
        config([with_mlp(latent(heads=5, dim=7, rot_dim=10, vdim=9, kv_rank=13, window=11, dims=6, base=100.0), moe(experts=5, top=2, ff=7)),
                with_mlp(wkv(heads=3, dim=11), dense(19))], width=37, vocab=53, loop=(1, 2, 2), mult=0.9),
    ][case]
    eng, tensors = make(tmp_path, cfg, device, "float32")
    toks = tokens(50, cfg["vocab"], 40 + case)
    want = oracle.forward(cfg, tensors, toks)
    rows = [eng.replay_step([("o", toks[:33], list(range(33)))])] + [eng.replay_step([("o", [t], [0])]) for t in toks[33:]]
    assert rel_err(torch.cat(rows), want) < TOL["float32"]


@pytest.mark.parametrize("device", DEVICES)
def test_bfloat16_aligned_sizes_long_context(tmp_path, device):
    """Sizes whose rows are 16-byte aligned (on the GPU: the matrix-core attention and GEMM kernels) in bfloat16:
    a prompt in portions, then 70 tokens one by one across 32-key steps, with and without a window."""
    cfg = config([with_mlp(latent(heads=4, dim=16, rot_dim=16, vdim=16, kv_rank=32, window=0, scale=0.18), dense(64)),
                  with_mlp(wkv(heads=2, dim=32), moe(experts=4, top=2, ff=16)),
                  latent(heads=20, dim=8, rot_dim=8, vdim=8, kv_rank=48, window=37, scale=0.25)], width=64, vocab=80)
    eng, tensors = make(tmp_path, cfg, device, "bfloat16", max_tokens=256)
    toks = tokens(190, 80, 12)
    want = oracle.forward(cfg, tensors, toks)
    rows = [eng.replay_step([("m", toks[:90], list(range(90)))]), eng.replay_step([("m", toks[90:120], list(range(30)))])]
    rows += [eng.replay_step([("m", [t], [0])]) for t in toks[120:]]
    assert close(torch.cat(rows), want, "bfloat16")


# ----------------------------------------------------------------------------- generation entry point
@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_through_the_scheduler(tmp_path, device):
    """engine.generate: admission, chunked prefill, mixed steps and (on the GPU) the captured decode graphs; three
    prompts of unequal length on two slots, so the third waits for a slot and reuses it."""
    eng, tensors = make(tmp_path, FULL, device, "float32", max_tokens=192, slots=2, graphs=device == "cuda", seed=3)
    prompts = [tokens(n, FULL["vocab"], 50 + n) for n in (21, 5, 34)]
    sp = SamplingParams(max_tokens=12, temperature=0.0, ignore_eos=True, stop_on_json_close=False)
    outs = eng.generate(prompts, sp)
    for p, o in zip(prompts, outs):
        assert o.finish_reason == "length" and o.token_ids == oracle.greedy(FULL, tensors, p, 12)
    if device == "cuda":
        assert eng.stats["graph_replays"] > 0
    assert len(eng.free_slots) == 2 and eng.allocator.num_free == eng.num_blocks


# ----------------------------------------------------------------------------- command line
def test_replay_and_generate_command_line(tmp_path):
    """The replay runner as a user starts it: steps on standard input, one logits file per step that wants rows,
    `done <step>` after every step; and `generate` on token ids."""
    import json
    import subprocess
    import sys
    from pathlib import Path

    import numpy as np

    root = Path(__file__).resolve().parent.parent
    cfg = config([with_mlp(latent(), dense()), with_mlp(wkv(), moe())], loop=(0, 2, 2))
    pc = config_from_json(cfg, "cli")
    tensors = random_tensors(pc, 5)
    save_checkpoint(pc, tensors, tmp_path / "ckpt")
    a, b = tokens(21, cfg["vocab"], 70), tokens(9, cfg["vocab"], 71)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:17], "want": [0, 16]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[17:18], "want": []}, {"id": "b", "tokens": b, "want": [8]}],
              "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": a[18:], "want": [2]}], "end": ["a"]}]
    out = tmp_path / "out"
    r = subprocess.run([str(root / "bin" / "trace_run"), "--model", str(tmp_path / "ckpt"), "--dtype", "float32", "--out",
                        str(out), "--max-tokens", "64", "--device", "cpu"], input="\n".join(map(json.dumps, steps)) + "\n",
                       capture_output=True, text=True, timeout=300, cwd=str(root))
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    assert sorted(p.name for p in out.iterdir()) == ["0.f32", "1.f32", "2.f32"]
    wa, wb = oracle.forward(cfg, tensors, a), oracle.forward(cfg, tensors, b)
    V = cfg["vocab"]
    got = {i: torch.from_numpy(np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, V)) for i in range(3)}
    assert rel_err(got[0], wa[[0, 16]]) < TOL["float32"]
    assert rel_err(got[1], wb[[8]]) < TOL["float32"]
    assert rel_err(got[2], wa[[20]]) < TOL["float32"]
    g = subprocess.run([sys.executable, "-m", "k8s_llm_scheduler_amd", "generate", "--model", str(tmp_path / "ckpt"),
                        "--dtype", "float32", "--prompt", " ".join(map(str, b)), "--max-new", "5", "--device", "cpu",
                        "--no-graphs"], capture_output=True, text=True, timeout=300, cwd=str(root))
    assert g.returncode == 0, g.stderr[-2000:]
    line = json.loads([l for l in g.stdout.splitlines() if l.startswith("{")][-1])
    assert line["token_ids"] == oracle.greedy(cfg, tensors, b, 5)


# ----------------------------------------------------------------------------- random configurations
def random_config(seed):
    """A random small model: 2-5 layers of either mixer in any order, any feed-forward (or none), sizes that are and
    are not multiples of 8 / 16, windows from 1 to beyond the sequence, an optional loop over any span."""
    import random

    rng = random.Random(seed)
    aligned = rng.random() < 0.5
    pick = lambda xs: rng.choice(xs)
    width = pick([32, 64, 96]) if aligned else pick([24, 37, 50, 72])
    layers = []
    for _ in range(rng.randint(2, 5)):
        if rng.random() < 0.5:
            heads = pick([1, 2, 3, 4])
            layer = wkv(heads=heads, dim=pick([8, 16, 32]) if aligned else pick([5, 12, 20, 33]))
        else:
            rd = pick([0, 8, 16]) if aligned else pick([0, 2, 6, 10])
            layer = latent(heads=pick([1, 2, 5, 17]), dim=pick([8, 16, 24]) if aligned else pick([3, 10, 12]),
                           rot_dim=rd, vdim=pick([8, 16]) if aligned else pick([5, 9]),
                           kv_rank=pick([16, 32, 48]) if aligned else pick([7, 20, 36]),
                           window=pick([0, 1, 2, 7, 31, 32, 33, 50, 500]), dims=pick([rd, rd // 2 * 2 // 2 * 2, rd]),
                           base=pick([100.0, 10000.0, 1e6]), scale=pick([0.1, 0.25, 0.5]))
        r = rng.random()
        if r < 0.35:
            layer = with_mlp(layer, dense(pick([16, 40, 64]) if aligned else pick([10, 27])))
        elif r < 0.8:
            e = pick([2, 3, 8, 20])
            layer = with_mlp(layer, moe(experts=e, top=rng.randint(1, min(e, 4)), ff=pick([8, 16]) if aligned else pick([5, 12]),
                                        scale=pick([0.5, 1.0, 2.5]), limit=pick([0, 0.7, 3.0]), shared=rng.random() < 0.6,
                                        shared_limit=pick([0, 1.5])))
        layers.append(layer)
    loop = None
    if rng.random() < 0.6:
        a = rng.randrange(len(layers))
        loop = (a, rng.randint(a + 1, len(layers)), rng.randint(1, 3))
    return config(layers, width=width, vocab=pick([40, 64, 101]), loop=loop, mult=pick([0.3, 0.7, 1.0]),
                  eps=pick([1e-6, 1e-5]))


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("seed", range(8))
def test_random_configurations(tmp_path, device, seed):
    """A prompt in two portions, a second request beside its decoded tokens, then tokens one by one."""
    cfg = random_config(seed)
    eng, tensors = make(tmp_path, cfg, device, "float32", seed=seed, max_tokens=160, slots=2)
    V = cfg["vocab"]
    a, b = tokens(75, V, 100 + seed), tokens(28, V, 200 + seed)
    wa, wb = oracle.forward(cfg, tensors, a), oracle.forward(cfg, tensors, b)
    ga = [eng.replay_step([("a", a[:40], list(range(40)))]), eng.replay_step([("a", a[40:43], [0, 1, 2])])]
    gb = []
    for i in range(43, 75):
        if i == 50:
            rows = eng.replay_step([("a", [a[i]], [0]), ("b", b[:20], list(range(20)))])
            gb.append(rows[1:])
        elif 50 < i <= 58:
            rows = eng.replay_step([("a", [a[i]], [0]), ("b", [b[20 + i - 51]], [0])], ["b"] if i == 58 else [])
            gb.append(rows[1:])
        else:
            rows = eng.replay_step([("a", [a[i]], [0])])
        ga.append(rows[:1])
    assert rel_err(torch.cat(ga), wa) < TOL["float32"], cfg
    assert rel_err(torch.cat(gb), wb) < TOL["float32"], cfg
