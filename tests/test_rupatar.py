"""Rupatar through the engine (checkpoint loader, registry, slots, paged cache with pooled blocks, recurrent state,
replay and generation entry points) against the plain float64 oracle in rupatar_oracle.py.  Every test runs on the CPU
(reference ops: model, cache, state and scheduler logic) and, marked gpu, on the HIP kernels.  Small own
configurations, random weights; where random weights would hide a fault the weights are shaped so that it shows."""

import copy
import math

import pytest
import torch

import rupatar_oracle as oracle
from k8s_llm_scheduler_amd.engine import SamplingParams, build_engine
from k8s_llm_scheduler_amd.models import load_config, model_class
from k8s_llm_scheduler_amd.models.rupatar import (RupatarModel, config_from_json, config_to_json, random_tensors,
                                                  save_checkpoint)

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
TOL = {"float32": 3e-4, "bfloat16": 6e-2}


def attn(heads=4, kv_heads=2, dim=12, vdim=10, window=7, pool=3, dims=8, base=5000.0, factor=2.0, scale=0.4, v_mix=True):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "v_mix": v_mix}
    if dims:
        m["rot"] = {"dims": dims, "base": base, "scaling": {"factor": factor}}
    if window:
        m["mask"] = {"size": window, **({"pool": pool} if pool else {})}
    return {"type": "attention", "mixer": m, "mlp": None}


def hgrn2(heads=3, dim=8, vdim=12):
    return {"type": "hgrn2", "mixer": {"heads": heads, "dim": dim, "vdim": vdim}, "mlp": None}


def mlstm(heads=2, dim=12, vdim=20, cap=9.0):
    return {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}, "mlp": None}


def moe(experts=6, top=3, ff=12, shared=16):
    return {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff},
            "shared": {"ff": shared} if shared else None}


def with_mlp(layer, mlp):
    layer = copy.deepcopy(layer)
    layer["mlp"] = mlp
    return layer


def config(layers, width=48, vocab=90, groups=3, eps=1e-5, embed_scale=2.5):
    return {"architecture": "Rupatar", "vocab": vocab, "width": width, "layers": layers,
            "norm": {"eps": eps, "groups": groups}, "embedding": {"scale": embed_scale}}


FULL = config([with_mlp(attn(), moe()), with_mlp(hgrn2(), moe(top=1, shared=0)), with_mlp(attn(window=9, pool=4, dims=4), moe()),
               mlstm(), with_mlp(attn(v_mix=False, window=5, pool=0, heads=2, kv_heads=2), moe(experts=3, top=3))])

# bfloat16 comparisons: no top-1 routing, where one close call of a router in bf16 replaces a row's whole feed-forward
SOFT = config([with_mlp(attn(), moe()), with_mlp(hgrn2(), moe(top=4)), with_mlp(attn(window=9, pool=4, dims=4), moe()),
               mlstm(), with_mlp(attn(v_mix=False, window=5, pool=0, heads=2, kv_heads=2), moe(experts=3, top=3))])


def model_for(dtype):
    return FULL if dtype == "float32" else SOFT


def make(tmp_path, cfg, device, dtype, seed=0, max_tokens=256, slots=4, graphs=False, edit=None):
    pc = config_from_json(cfg, "case")
    tensors = random_tensors(pc, seed)
    if edit:
        edit(tensors)
    save_checkpoint(pc, tensors, tmp_path / "ckpt")
    eng = build_engine(weights=str(tmp_path / "ckpt"), device=device, dtype=dtype, max_batch=slots, block_size=16,
                       num_blocks=max_tokens // 16, max_model_len=max_tokens, cuda_graphs=graphs, capture=graphs)
    assert isinstance(eng.model, RupatarModel)
    return eng, tensors


def expect(cfg, tensors, toks, streams=False):
    logits, after = oracle.forward(toks, tensors, cfg)
    return (logits, after) if streams else logits


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


def tokens(n, vocab, seed, avoid=()):
    g = torch.Generator().manual_seed(seed)
    out = torch.randint(0, vocab, (n,), generator=g).tolist()
    return [t if t not in avoid else (t + 1) % vocab for t in out]


def whole(eng, key, toks):
    return eng.replay_step([(key, toks, list(range(len(toks))))], [key])


def stepwise(eng, key, toks, first):
    """The first ``first`` tokens as one portion, the rest one by one."""
    rows = [eng.replay_step([(key, toks[:first], list(range(first)))])] if first else []
    rows += [eng.replay_step([(key, [t], [0])]) for t in toks[first:]]
    return torch.cat(rows)


# ----------------------------------------------------------------------------- registry, configuration, loader
def test_registry_and_config_roundtrip(tmp_path):
    pc = config_from_json(FULL, "x")
    assert config_from_json(config_to_json(pc), "x") == pc
    save_checkpoint(pc, random_tensors(pc, 1), tmp_path / "m")
    got = load_config(str(tmp_path / "m"))
    assert model_class(got) is RupatarModel and got.layers == pc.layers
    assert (got.norm_groups, got.embed_scale, got.rms_eps) == (3, 2.5, 1e-5)
    a = got.layers[2].mixer
    assert (a.window, a.pool, a.rot_dims, a.rot_factor, a.kv_heads, a.v_mix) == (9, 4, 4, 2.0, 2, True)
    assert model_class(load_config("rupatar-tiny")) is RupatarModel
    assert model_class(load_config("putulorn-tiny")).__name__ == "PutulornModel"
    assert model_class(load_config("tiny")).__name__ == "LlamaModel"


# ----------------------------------------------------------------------------- each mechanism alone
MECHANISMS = {
    "attention_window_pool": config([attn()]),
    "attention_no_window": config([attn(window=0)]),
    "attention_window_no_pool": config([attn(pool=0)]),
    "attention_pool_of_one": config([attn(window=4, pool=1)]),
    "attention_pool_beyond_a_page": config([attn(window=3, pool=19)]),
    "attention_full_rotation": config([attn(dims=12, factor=1.0)]),
    "attention_no_rotation": config([attn(dims=0)]),
    "attention_one_kv_head": config([attn(heads=3, kv_heads=1)]),
    "attention_all_kv_heads": config([attn(heads=3, kv_heads=3)]),
    "value_mixing": config([attn(), attn(v_mix=False), attn(window=11, pool=2), hgrn2(), attn(window=0)]),
    "value_mixing_starts_late": config([attn(v_mix=False), attn(), attn()]),
    "hgrn2": config([hgrn2()]),
    "hgrn2_one_head": config([hgrn2(heads=1, dim=20, vdim=7)]),
    "mlstm": config([mlstm()]),
    "mlstm_tight_cap": config([mlstm(heads=3, dim=6, vdim=6, cap=0.7)]),
    "moe_shared": config([with_mlp(hgrn2(), moe())]),
    "moe_top1_no_shared": config([with_mlp(hgrn2(), moe(top=1, shared=0))]),
    "moe_all_experts": config([with_mlp(mlstm(), moe(experts=3, top=3))]),
    "one_norm_group_unit_embedding": config([with_mlp(attn(), moe())], groups=1, embed_scale=1.0),
    "many_norm_groups": config([with_mlp(hgrn2(), moe()), mlstm()], groups=12),
}


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", sorted(MECHANISMS))
def test_mechanism_alone(tmp_path, device, name):
    cfg = MECHANISMS[name]
    eng, tensors = make(tmp_path, cfg, device, "float32")
    toks = tokens(45, cfg["vocab"], 3)
    assert rel_err(whole(eng, "a", toks), expect(cfg, tensors, toks)) < TOL["float32"]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_full_model_and_layer_streams(tmp_path, device, dtype):
    cfg = model_for(dtype)
    eng, tensors = make(tmp_path, cfg, device, dtype)
    toks = tokens(45, cfg["vocab"], 4)
    want, streams = expect(cfg, tensors, toks, streams=True)
    assert close(whole(eng, "a", toks), want, dtype)
    m, dev = eng.model, eng.device
    T = len(toks)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)
    b = m.batch_meta(i32(list(range(T))), i32(list(range(T))), i32([0, T]), i32([list(range(16))]), i32([0]))
    got = m.residual_after_runs(i32(toks), b)
    assert len(got) == len(streams) == len(cfg["layers"])
    for g, w in zip(got, streams):
        assert close(g.cpu(), w, dtype)


# ----------------------------------------------------------------------------- cutting, batching, reuse
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_prefill_against_token_by_token(tmp_path, device, dtype):
    cfg = model_for(dtype)
    eng, tensors = make(tmp_path, cfg, device, dtype)
    toks = tokens(40, cfg["vocab"], 5)
    want = expect(cfg, tensors, toks)
    rows = [eng.replay_step([("s", [t], [0])], ["s"] if i == len(toks) - 1 else []) for i, t in enumerate(toks)]
    assert close(torch.cat(rows), want, dtype)
    assert len(eng.free_slots) == eng.max_batch and eng.allocator.num_free == eng.num_blocks


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("sizes", [[2, 2, 2, 3, 1, 1, 29], [17, 16, 1, 6], [1, 15, 16, 8], [39, 1], [5] * 8])
def test_portions(tmp_path, device, sizes):
    eng, tensors = make(tmp_path, FULL, device, "float32")
    toks = tokens(sum(sizes), FULL["vocab"], 6)
    want = expect(FULL, tensors, toks)
    rows, at = [], 0
    for n in sizes:
        rows.append(eng.replay_step([("p", toks[at:at + n], list(range(n)))]))
        at += n
    assert rel_err(torch.cat(rows), want) < TOL["float32"]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_unequal_batch_against_each_alone_with_reuse(tmp_path, device, dtype):
    """Four slots and 96 cache tokens for six requests of unequal length: portions of some beside single tokens of
    others, requests left out of steps, slots and blocks (with their pooled entries) taken again by later requests."""
    cfg = model_for(dtype)
    eng, tensors = make(tmp_path, cfg, device, dtype, max_tokens=96, slots=4)
    V = cfg["vocab"]
    seqs = {k: tokens(n, V, 10 + i) for i, (k, n) in enumerate([("a", 30), ("b", 7), ("c", 18), ("d", 1), ("e", 33),
                                                                 ("f", 20)])}
    want = {k: expect(cfg, tensors, v) for k, v in seqs.items()}
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
def test_reused_slot_and_pages_start_clean(tmp_path, device):
    """One slot, one request after another: the second must not see the first's recurrent state, running maximum,
    cached rows or pooled blocks."""
    cfg = config([hgrn2(), mlstm(), attn(window=4, pool=2), attn(window=0)])
    eng, tensors = make(tmp_path, cfg, device, "float32", max_tokens=32, slots=1)
    a, b = tokens(30, cfg["vocab"], 1), tokens(25, cfg["vocab"], 2)
    whole(eng, "a", a)
    got = [eng.replay_step([("b", b[:9], list(range(9)))]), eng.replay_step([("b", b[9:], list(range(16)))], ["b"])]
    assert rel_err(torch.cat(got), expect(cfg, tensors, b)) < TOL["float32"]


# ----------------------------------------------------------------------------- windows, pooled blocks, far keys
LOUD, DIM_U = 7, 10


def loud_weights(cfg):
    """Queries and keys are unit vectors, so a token is made loud through the weights: width coordinate 0 is set for the
    loud token only, every key head maps it onto the unrotated head dimension DIM_U, and every query carries a bias
    there.  The loud token's key then dominates every softmax it is part of, alone or inside a pooled block."""
    def edit(t):
        t["embed"][:, 0] = 0
        t["embed"][LOUD] = 0
        t["embed"][LOUD, 0] = 8.0
        for i, L in enumerate(cfg["layers"]):
            if L["type"] != "attention":
                continue
            m = L["mixer"]
            D = m["dim"]
            for g in range(m["kv_heads"]):
                t[f"l{i}.mix.k"][g * D + DIM_U, 0] = 4.0
            for h in range(m["heads"]):
                t[f"l{i}.mix.q.b"][h * D + DIM_U] = 3.0
    return edit


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("window,pool", [(1, 1), (2, 3), (16, 4), (17, 16), (5, 0), (9, 21)])
def test_window_and_pool_edges_in_prompt_and_decoding(tmp_path, device, window, pool):
    """The loud token is the oldest key inside the window of one query, outside the next one's (seen by nobody until
    its block is whole and wholly before the window), then part of a pooled block: in a prompt portion and among tokens
    decoded one by one, across page borders (pages of 16)."""
    cfg = config([attn(window=window, pool=pool, dim=16, dims=6, scale=1.0, heads=2, kv_heads=1),
                  with_mlp(attn(window=window + 3, pool=pool, dim=16, dims=6, scale=1.0, heads=2, kv_heads=2, v_mix=False), moe())],
                 vocab=60)
    eng, tensors = make(tmp_path, cfg, device, "float32", edit=loud_weights(cfg))
    toks = tokens(90, 60, 8, avoid=(LOUD,))
    places = (3, 14, 31, 40, 52, 63)
    for p in places:
        toks[p] = LOUD
    want = expect(cfg, tensors, toks)
    quiet = expect(cfg, tensors, [8 if t == LOUD else t for t in toks])
    assert rel_err(quiet, want) > 0.05                     # the loud token matters
    got = stepwise(eng, "w", toks, 36)
    assert rel_err(got, want) < TOL["float32"]
    for p in places:                                        # the rows around each edge, one by one
        edges = [p + window - 1, p + window]
        if pool:
            seen = (p // pool) * pool + pool - 1 + window   # the first query that sees the loud token's block
            edges += [seen - 1, seen]
        for i in edges:
            if i < len(toks):
                assert rel_err(got[i:i + 1], want[i:i + 1]) < TOL["float32"], (p, i)


@pytest.mark.parametrize("device", DEVICES)
def test_edges_move_the_output(tmp_path, device):
    """The premise of the edge test, on the oracle: one position more or less of window, or one block more or less,
    changes the rows at the edges by far more than the tolerance."""
    if device != "cpu":
        pytest.skip("a property of the oracle")
    cfg = config([attn(window=6, pool=4, dim=16, dims=6, scale=1.0, heads=2, kv_heads=1)], vocab=60)
    pc = config_from_json(cfg, "case")
    tensors = random_tensors(pc, 0)
    loud_weights(cfg)(tensors)
    toks = tokens(40, 60, 8, avoid=(LOUD,))
    toks[9] = LOUD
    want = expect(cfg, tensors, toks)
    for size, pool in ((5, 4), (7, 4), (6, 3), (6, 5)):
        other = copy.deepcopy(cfg)
        other["layers"][0]["mixer"]["mask"] = {"size": size, "pool": pool}
        assert rel_err(expect(other, tensors, toks), want) > 0.02, (size, pool)


@pytest.mark.parametrize("device", DEVICES)
def test_far_keys_and_long_decoding(tmp_path, device):
    """Pooled blocks, an unwindowed layer and both recurrences: position 200+ still depends on the first tokens (checked
    on the oracle), over many page borders, with 90 tokens decoded one by one."""
    cfg = config([attn(window=12, pool=5, dim=16, dims=6, scale=1.0, heads=2, kv_heads=1), hgrn2(heads=2, dim=12, vdim=8),
                  with_mlp(attn(window=0, dim=16, dims=4, heads=2, kv_heads=2, v_mix=False), moe(experts=4, top=2, ff=8, shared=8)),
                  mlstm(heads=2, dim=8, vdim=8)], width=32, vocab=50, groups=2)
    eng, tensors = make(tmp_path, cfg, device, "float32", max_tokens=256, edit=loud_weights(cfg))
    toks = tokens(215, 50, 9, avoid=(LOUD,))
    toks[1] = toks[64] = LOUD
    want = expect(cfg, tensors, toks)
    other = expect(cfg, tensors, [toks[0], 8] + toks[2:])
    assert rel_err(other[-1:], want[-1:]) > 1e-3            # the end sees position 1
    rows = [eng.replay_step([("f", toks[:100], list(range(100)))]), eng.replay_step([("f", toks[100:125], list(range(25)))])]
    rows += [eng.replay_step([("f", [t], [0])]) for t in toks[125:]]
    assert rel_err(torch.cat(rows), want) < TOL["float32"]


@pytest.mark.parametrize("device", DEVICES)
def test_far_block_among_hundreds(tmp_path, device):
    """One attention layer: the loud token lies in one pooled block among dozens, hundreds of positions back; the last
    rows change by far more than the tolerance when it is silenced, and the engine follows the oracle."""
    cfg = config([attn(window=8, pool=6, dim=16, dims=6, scale=1.0, heads=2, kv_heads=1)], width=32, vocab=50, groups=1)
    eng, tensors = make(tmp_path, cfg, device, "float32", max_tokens=320, edit=loud_weights(cfg))
    toks = tokens(300, 50, 11, avoid=(LOUD,))
    toks[20] = LOUD
    want = expect(cfg, tensors, toks)
    other = expect(cfg, tensors, toks[:20] + [8] + toks[21:])
    assert rel_err(other[-3:], want[-3:]) > 0.005
    got = torch.cat([eng.replay_step([("g", toks[:250], list(range(250)))]), stepwise(eng, "g", toks[250:], 0)])
    assert rel_err(got, want) < TOL["float32"]


@pytest.mark.parametrize("device", DEVICES)
def test_first_tokens(tmp_path, device):
    eng, tensors = make(tmp_path, FULL, device, "float32")
    for n in (1, 2, 3):
        toks = tokens(n, FULL["vocab"], 20 + n)
        assert rel_err(whole(eng, f"s{n}", toks), expect(FULL, tensors, toks)) < TOL["float32"]
    toks = tokens(4, FULL["vocab"], 30)
    got = [eng.replay_step([("x", toks[:1], [0])]), eng.replay_step([("x", toks[1:2], [0])]),
           eng.replay_step([("x", toks[2:], [0, 1])], ["x"])]
    assert rel_err(torch.cat(got), expect(FULL, tensors, toks)) < TOL["float32"]


# ----------------------------------------------------------------------------- other sizes
OTHER_SIZES = [
    # head sizes above one wave, many query heads per key head (more than the waves of a workgroup), big window
    config([with_mlp(attn(heads=20, kv_heads=2, dim=72, vdim=80, window=40, pool=7, dims=70, scale=0.11), moe(experts=70, top=4, ff=6)),
            with_mlp(hgrn2(heads=2, dim=72, vdim=96), moe(experts=2, top=2, ff=20, shared=0)),
            mlstm(heads=1, dim=100, vdim=70, cap=30.0)], width=40, vocab=77, groups=5, eps=1e-6, embed_scale=1.0),
    # odd sizes everywhere
    config([with_mlp(attn(heads=5, kv_heads=5, dim=7, vdim=9, window=11, pool=3, dims=6, base=100.0, factor=1.5, scale=0.6),
                     moe(experts=5, top=2, ff=7, shared=3)),
            with_mlp(hgrn2(heads=3, dim=11, vdim=5), moe(experts=3, top=1, ff=9)),
            mlstm(heads=3, dim=5, vdim=13, cap=4.5),
            attn(heads=5, kv_heads=5, dim=7, vdim=9, window=2, pool=2, dims=2, scale=0.3)], width=37, vocab=53, groups=1),
    # one of everything: one head, one expert, value size one, a pool longer than the window
    config([with_mlp(attn(heads=1, kv_heads=1, dim=4, vdim=1, window=3, pool=8, dims=4, scale=1.0), moe(experts=1, top=1, ff=4, shared=1)),
            hgrn2(heads=1, dim=4, vdim=1), mlstm(heads=1, dim=2, vdim=1, cap=1.0)], width=8, vocab=11, groups=8),
    # recurrent heads wider than two waves: key channels in groups of 32 and 64
    config([hgrn2(heads=1, dim=40, vdim=200), with_mlp(mlstm(heads=1, dim=144, vdim=136, cap=20.0), moe(experts=3, top=2, ff=8, shared=0)),
            hgrn2(heads=2, dim=250, vdim=24)], width=48, vocab=31, groups=2),
    # aligned sizes with mixers of different widths in one model
    config([with_mlp(attn(heads=8, kv_heads=4, dim=32, vdim=16, window=33, pool=16, dims=32, scale=0.18), moe(experts=4, top=2, ff=32, shared=64)),
            hgrn2(heads=4, dim=16, vdim=32), mlstm(heads=2, dim=64, vdim=64, cap=11.0),
            with_mlp(attn(heads=8, kv_heads=4, dim=64, vdim=16, window=64, pool=32, dims=16, scale=0.125), moe(experts=8, top=8, ff=16, shared=0))],
           width=64, vocab=80, groups=4),
]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("case", range(len(OTHER_SIZES)))
def test_other_sizes(tmp_path, device, case):
    cfg = OTHER_SIZES[case]
    eng, tensors = make(tmp_path, cfg, device, "float32")
    toks = tokens(70, cfg["vocab"], 40 + case)
    assert rel_err(stepwise(eng, "o", toks, 45), expect(cfg, tensors, toks)) < TOL["float32"]


@pytest.mark.parametrize("device", DEVICES)
def test_bfloat16_aligned_sizes_long_context(tmp_path, device):
    """Sizes whose rows are 16-byte aligned (on the GPU: the matrix-core kernels) in bfloat16: a prompt in portions,
    then 70 tokens one by one, windows and pooled blocks across many pages."""
    cfg = config([with_mlp(attn(heads=4, kv_heads=2, dim=16, vdim=16, window=0, dims=8, scale=0.25), moe(experts=4, top=2, ff=16)),
                  with_mlp(hgrn2(heads=2, dim=32, vdim=32), moe(experts=4, top=3, ff=16)),
                  attn(heads=16, kv_heads=2, dim=32, vdim=16, window=37, pool=8, dims=16, scale=0.18), mlstm(heads=2, dim=32, vdim=32)],
                 width=64, vocab=80, groups=2)
    eng, tensors = make(tmp_path, cfg, device, "bfloat16", max_tokens=256)
    toks = tokens(190, 80, 12)
    want = expect(cfg, tensors, toks)
    rows = [eng.replay_step([("m", toks[:90], list(range(90)))]), eng.replay_step([("m", toks[90:120], list(range(30)))])]
    rows += [eng.replay_step([("m", [t], [0])]) for t in toks[120:]]
    assert close(torch.cat(rows), want, "bfloat16")


@pytest.mark.parametrize("device", DEVICES)
def test_cache_rounding_is_the_only_difference_in_bfloat16(tmp_path, device):
    """A pooled block is the mean of the keys and values as the cache holds them: in bfloat16 the engine follows an
    oracle that rounds what it caches, more closely than one that does not."""
    cfg = config([attn(window=4, pool=4, heads=2, kv_heads=1, dim=16, vdim=16, dims=8, scale=1.0)], width=32, vocab=40, groups=1)
    eng, tensors = make(tmp_path, cfg, device, "bfloat16")
    toks = tokens(60, 40, 13)
    got = whole(eng, "r", toks)
    rounded, _ = oracle.forward(toks, tensors, cfg, round_cache=lambda x: x.to(torch.bfloat16).to(torch.float64))
    assert rel_err(got, rounded) < TOL["bfloat16"]


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
        assert o.finish_reason == "length" and o.token_ids == oracle.greedy(p, tensors, FULL, 12)
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
    cfg = config([with_mlp(attn(), moe()), with_mlp(hgrn2(), moe()), mlstm()])
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
    wa, wb = expect(cfg, tensors, a), expect(cfg, tensors, b)
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
    assert line["token_ids"] == oracle.greedy(b, tensors, cfg, 5)


# ----------------------------------------------------------------------------- random configurations
def random_config(seed):
    """A random small model: 2-5 layers of any mixer in any order, experts or no feed-forward, sizes that are and are
    not multiples of 8 / 16, windows from 1 to beyond the sequence, pools from 1 to beyond a page."""
    import random

    rng = random.Random(seed)
    aligned = rng.random() < 0.5
    pick = lambda xs: rng.choice(xs)
    groups = pick([1, 2, 4])
    width = pick([32, 64, 96]) if aligned else pick([24, 36, 52, 72])
    layers = []
    gv = None                     # the mixing layers share the size of their values
    for _ in range(rng.randint(2, 5)):
        r = rng.random()
        if r < 0.3:
            layer = hgrn2(heads=pick([1, 2, 3, 4]), dim=pick([8, 16, 32]) if aligned else pick([5, 12, 20, 33]),
                          vdim=pick([8, 16, 64]) if aligned else pick([3, 17, 40]))
        elif r < 0.55:
            layer = mlstm(heads=pick([1, 2, 3]), dim=pick([8, 16, 32]) if aligned else pick([5, 12, 33]),
                          vdim=pick([8, 32]) if aligned else pick([6, 21]), cap=pick([2.0, 10.0, 15.0]))
        else:
            kv = pick([1, 2, 3])
            dim = pick([8, 16, 24]) if aligned else pick([6, 10, 12])
            vdim = pick([8, 16]) if aligned else pick([5, 9])
            mix = rng.random() < 0.7
            if mix:
                if gv is None:
                    gv = (kv, vdim)
                kv, vdim = gv
            window = pick([0, 1, 2, 7, 31, 32, 33, 50, 500])
            layer = attn(heads=kv * pick([1, 2, 5]), kv_heads=kv, dim=dim, vdim=vdim, window=window,
                         pool=pick([0, 1, 2, 5, 16, 23]), dims=pick([0, 2, dim // 2 * 2, dim // 4 * 2]),
                         base=pick([100.0, 10000.0, 1e6]), factor=pick([1.0, 4.0, 8.0]), scale=pick([0.1, 0.25, 0.5]), v_mix=mix)
        if rng.random() < 0.7:
            e = pick([2, 3, 8, 20])
            layer = with_mlp(layer, moe(experts=e, top=rng.randint(1, min(e, 4)), ff=pick([8, 16]) if aligned else pick([5, 12]),
                                        shared=pick([0, 8, 24]) if aligned else pick([0, 7])))
        layers.append(layer)
    return config(layers, width=width, vocab=pick([40, 64, 101]), groups=groups, eps=pick([1e-6, 1e-5]),
                  embed_scale=pick([1.0, math.sqrt(width)]))


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("seed", range(8))
def test_random_configurations(tmp_path, device, seed):
    """A prompt in two portions, a second request beside its decoded tokens, then tokens one by one."""
    cfg = random_config(seed)
    eng, tensors = make(tmp_path, cfg, device, "float32", seed=seed, max_tokens=160, slots=2)
    V = cfg["vocab"]
    a, b = tokens(75, V, 100 + seed), tokens(28, V, 200 + seed)
    wa, wb = expect(cfg, tensors, a), expect(cfg, tensors, b)
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
