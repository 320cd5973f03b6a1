"""Rupatar: a decoder with an fp32 residual stream, pre-norm blocks ``x += mixer(norm(x)); x += moe(norm(x))`` whose
norms divide each of ``norm.groups`` consecutive parts of the vector by its own root mean square, and three mixers in
any order the config lists:

* ``attention``: grouped-query attention with biased projections, interleaved-pair rotary positions on the first
  ``rot.dims`` dimensions (frequencies ``base^(-2i / dims) / factor``), unit-RMS queries and keys, a sliding window of
  ``mask.size`` tokens beside which every block of ``mask.pool`` tokens that lies wholly before the window is seen as
  one key / value (the block's mean as cached), one softmax over both with a sink (``p_j = e^s_j / (1 + sum e^s)``),
  values mixed with the first mixing layer's (``v <- (1 - lam) v + lam v_first``, cached after mixing), and a sigmoid
  output gate on the concatenated heads;
* ``hgrn2``: per head ``S <- diag(f) S + (1 - f) v^T``, ``o = S^T silu(W_q h)`` with the forget gate bounded below,
  ``f = low + (1 - low) sigmoid(W_f h + b)``; each head's output RMS-normed with a weight shared by the heads;
* ``mlstm``: per head ``S <- e^(f + m - m') S + e^(i - m') k v^T`` (and ``n`` likewise with ``k``) under the running
  maximum ``m' = max(f + m, i)`` (``m`` starts at 0), soft-capped log gates ``i = cap tanh(z_i / cap)``,
  ``f = logsigmoid(cap tanh(z_f / cap))``, ``o = S^T q / (max(|n . q|, e^(-m')) + 1e-6)`` with ``q`` scaled by
  ``dim^(-1/2)``; unit RMS per head, a norm weight over all heads and a sigmoid gate.

The feed-forward is a mixture of experts with a sigmoid router: the ``top`` largest scores choose the experts, the
scores (not renormalised) scale the experts' *inputs*, experts are ``W_down gelu(W_up x)`` with the exact gelu, and a
shared expert of the same form runs for every token.  The embedding is scaled by ``embedding.scale``.

The model presents the engine's interface through :class:`~.stream.StreamModel`; caches: per attention layer a paged
K / V cache plus the pooled blocks' fp32 entries (kept with the page of a block's first token), per recurrent layer one
fp32 state record per (request slot, head).  Every op is a kernel of :mod:`..ops.seqmix`; ``dtype=float32`` runs
everything in true fp32.  Single rank (TP = 1).
"""

from __future__ import annotations

import math
from dataclasses import dataclass, field
from pathlib import Path
from typing import Dict, List, Optional

import torch

from ..ops import reference as ref
from ..ops import seqmix as sm
from ..parallel import TPGroup
from . import stream
from .stream import StreamModel

ARCHITECTURE = "Rupatar"
MIXERS = ("attention", "hgrn2", "mlstm")
F32 = torch.float32


# ----------------------------------------------------------------------------- configuration
@dataclass
class MixerConfig:
    type: str
    heads: int
    dim: int
    vdim: int
    # attention
    kv_heads: int = 0
    window: int = 0          # 0: every earlier token is seen, no pooled blocks
    pool: int = 0            # 0: nothing is seen before the window
    rot_dims: int = 0
    rot_base: float = 10000.0
    rot_factor: float = 1.0
    scale: float = 1.0
    v_mix: bool = False
    # mlstm
    gate_cap: float = 0.0


@dataclass
class MlpConfig:
    experts: int
    top: int
    ff: int
    shared_ff: int = 0       # 0: no shared expert


@dataclass
class LayerConfig:
    mixer: MixerConfig
    mlp: Optional[MlpConfig]


@dataclass
class RupatarConfig:
    name: str
    vocab: int
    hidden: int
    layers: List[LayerConfig]
    rms_eps: float = 1e-6
    norm_groups: int = 1
    embed_scale: float = 1.0
    max_position: int = 1 << 20
    bos_id: int = 0
    eos_ids: tuple = ()
    extra: dict = field(default_factory=dict)
    token_ids_only = True    # checkpoints of this design ship no tokenizer: requests are token ids

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    def validate_tp(self, tp: int) -> None:
        if tp != 1:
            raise ValueError(f"{self.name}: this design runs on one rank (tp={tp})")


def _mixer_from(d: dict, kind: str) -> MixerConfig:
    if kind not in MIXERS:
        raise ValueError(f"unknown mixer type {kind!r}")
    heads, dim, vdim = int(d["heads"]), int(d["dim"]), int(d["vdim"])
    if kind == "hgrn2":
        return MixerConfig(kind, heads, dim, vdim)
    if kind == "mlstm":
        return MixerConfig(kind, heads, dim, vdim, gate_cap=float(d["gate_cap"]))
    rot, mask = d.get("rot") or {}, d.get("mask") or {}
    window = int(mask.get("size") or 0)
    return MixerConfig(kind, heads, dim, vdim, kv_heads=int(d.get("kv_heads") or heads), window=window,
                       pool=int(mask.get("pool") or 0) if window else 0, rot_dims=int(rot.get("dims") or 0),
                       rot_base=float(rot.get("base", 10000.0)),
                       rot_factor=float((rot.get("scaling") or {}).get("factor", 1.0)),
                       scale=float(d.get("scale", 1.0 / math.sqrt(dim))), v_mix=bool(d.get("v_mix", False)))


def _mlp_from(d: Optional[dict]) -> Optional[MlpConfig]:
    if d is None:
        return None
    if d.get("kind", "moe") != "moe":
        raise ValueError(f"unknown mlp kind {d['kind']!r}")
    r, s = d["router"], d.get("shared")
    return MlpConfig(int(r["experts"]), int(r["top"]), int(d["expert"]["ff"]), int(s["ff"]) if s else 0)


def config_from_json(c: dict, name: str = "rupatar") -> RupatarConfig:
    layers = [LayerConfig(_mixer_from(l["mixer"], l["type"]), _mlp_from(l.get("mlp"))) for l in c["layers"]]
    norm = c.get("norm") or {}
    return RupatarConfig(name=name, vocab=int(c["vocab"]), hidden=int(c["width"]), layers=layers,
                         rms_eps=float(norm.get("eps", 1e-6)), norm_groups=int(norm.get("groups", 1)),
                         embed_scale=float((c.get("embedding") or {}).get("scale", 1.0)))


def config_to_json(cfg: RupatarConfig) -> dict:
    layers = []
    for L in cfg.layers:
        m = L.mixer
        mixer: dict = {"heads": m.heads, "dim": m.dim, "vdim": m.vdim}
        if m.type == "mlstm":
            mixer["gate_cap"] = m.gate_cap
        elif m.type == "attention":
            mixer.update({"kv_heads": m.kv_heads, "scale": m.scale, "v_mix": m.v_mix})
            if m.rot_dims:
                mixer["rot"] = {"dims": m.rot_dims, "base": m.rot_base, "scaling": {"factor": m.rot_factor}}
            if m.window:
                mixer["mask"] = {"size": m.window, **({"pool": m.pool} if m.pool else {})}
        f = L.mlp
        mlp = None
        if f is not None:
            mlp = {"kind": "moe", "router": {"experts": f.experts, "top": f.top}, "expert": {"ff": f.ff},
                   "shared": {"ff": f.shared_ff} if f.shared_ff else None}
        layers.append({"type": m.type, "mixer": mixer, "mlp": mlp})
    return {"architecture": ARCHITECTURE, "vocab": cfg.vocab, "width": cfg.hidden, "layers": layers,
            "norm": {"eps": cfg.rms_eps, "groups": cfg.norm_groups}, "embedding": {"scale": cfg.embed_scale}}


def tensor_shapes(cfg: RupatarConfig) -> Dict[str, tuple]:
    """Checkpoint tensor names and shapes of a configuration."""
    W = cfg.hidden
    t: Dict[str, tuple] = {"embed": (cfg.vocab, W), "final.norm": (W,), "head": (cfg.vocab, W)}
    for i, L in enumerate(cfg.layers):
        p, m = f"l{i}.", L.mixer
        H, D, V = m.heads, m.dim, m.vdim
        t[p + "norm1"] = (W,)
        if m.type == "attention":
            G = m.kv_heads
            t.update({p + "mix.q": (H * D, W), p + "mix.q.b": (H * D,), p + "mix.k": (G * D, W),
                      p + "mix.k.b": (G * D,), p + "mix.v": (G * V, W), p + "mix.v.b": (G * V,), p + "mix.vmix": (),
                      p + "mix.g": (H * V, W), p + "mix.o": (W, H * V), p + "mix.o.b": (W,)})
        elif m.type == "hgrn2":
            t.update({p + "mix.q": (H * D, W), p + "mix.f": (H * D, W), p + "mix.f.b": (H * D,),
                      p + "mix.lower": (H * D,), p + "mix.v": (H * V, W), p + "mix.norm": (V,), p + "mix.o": (W, H * V)})
        else:
            t.update({p + "mix.q": (H * D, W), p + "mix.k": (H * D, W), p + "mix.v": (H * V, W), p + "mix.i": (H, W),
                      p + "mix.i.b": (H,), p + "mix.f": (H, W), p + "mix.f.b": (H,), p + "mix.g": (H * V, W),
                      p + "mix.norm": (H * V,), p + "mix.o": (W, H * V)})
        f = L.mlp
        if f is None:
            continue
        t[p + "norm2"] = (W,)
        for e in range(f.experts):
            t.update({f"{p}mlp.e{e}.up": (f.ff, W), f"{p}mlp.e{e}.down": (W, f.ff)})
        t[p + "mlp.router"] = (f.experts, W)
        if f.shared_ff:
            t.update({p + "mlp.shared.up": (f.shared_ff, W), p + "mlp.shared.down": (W, f.shared_ff)})
    return t


def random_tensors(cfg: RupatarConfig, seed: int = 0, device="cpu") -> Dict[str, torch.Tensor]:
    """Random bf16 weights of a configuration (benchmarks and tests): projections ~ N(0, 1 / fan_in), norm weights
    around one, biases and gate offsets of order one, lower bounds and mixing factors in (0, 1)."""
    g = torch.Generator(device=device).manual_seed(seed)
    out: Dict[str, torch.Tensor] = {}
    rand = lambda shape: torch.rand(shape, generator=g, device=device)
    randn = lambda shape: torch.randn(shape, generator=g, device=device)
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.rsplit(".", 1)[-1]
        if leaf in ("norm", "norm1", "norm2"):
            t = 1.0 + randn(shape) * 0.1
        elif leaf == "lower":
            t = rand(shape) * 0.9
        elif leaf == "vmix":
            t = 0.2 + rand(shape) * 0.5
        elif leaf == "b":
            t = randn(shape) * (1.0 if name.endswith(("mix.f.b", "mix.i.b")) else 0.2)
        elif leaf == "embed":
            t = randn(shape) / math.sqrt(max(cfg.embed_scale, 1.0))
        else:
            t = randn(shape) / math.sqrt(shape[-1])
        out[name] = t.to(torch.bfloat16)
    return out


def save_checkpoint(cfg: RupatarConfig, tensors: Dict[str, torch.Tensor], path: Path) -> None:
    stream.save_checkpoint(config_to_json(cfg), tensors, path)


def preset(name: str, width: int, vocab: int, repeats: int, *, heads: int, kv_heads: int, dim: int, vdim: int,
           window: int, pool: int, rot_dims: int, scan_heads: int, scan_dim: int, scan_vdim: int, experts: int, top: int,
           expert_ff: int, shared_ff: int, groups: int = 4, order=("attention", "hgrn2", "attention", "mlstm")
           ) -> RupatarConfig:
    """``repeats`` x ``order``, every layer with a mixture of experts."""
    layers = []
    for _ in range(repeats):
        for kind in order:
            if kind == "attention":
                mixer = MixerConfig(kind, heads, dim, vdim, kv_heads=kv_heads, window=window, pool=pool,
                                    rot_dims=rot_dims, rot_base=10000.0, rot_factor=2.0, scale=1.0 / math.sqrt(dim),
                                    v_mix=True)
            else:
                mixer = MixerConfig(kind, scan_heads, scan_dim, scan_vdim, gate_cap=15.0 if kind == "mlstm" else 0.0)
            layers.append(LayerConfig(mixer, MlpConfig(experts, top, expert_ff, shared_ff)))
    return RupatarConfig(name, vocab, width, layers, norm_groups=groups, embed_scale=math.sqrt(width))


PRESETS = {
    # runs on the CPU in tests: every mixer, experts with a shared expert, pooled blocks behind a short window
    "rupatar-tiny": preset("rupatar-tiny", 96, 320, 1, heads=6, kv_heads=3, dim=16, vdim=24, window=20, pool=5,
                           rot_dims=8, scan_heads=3, scan_dim=16, scan_vdim=32, experts=6, top=2, expert_ff=48,
                           shared_ff=80, groups=3),
    # layer shapes of a ~1B-class model (benchmarks, random weights)
    "rupatar-1b": preset("rupatar-1b", 2048, 32768, 4, heads=16, kv_heads=4, dim=128, vdim=128, window=1024, pool=16,
                         rot_dims=64, scan_heads=16, scan_dim=64, scan_vdim=128, experts=16, top=2, expert_ff=2048,
                         shared_ff=2048),
}


# ----------------------------------------------------------------------------- weights
@dataclass
class _Attention:
    cfg: MixerConfig
    w_in: torch.Tensor                  # [H D + G D + G V + H V, W]: q | k | v | gate
    qb: torch.Tensor
    kb: torch.Tensor
    vb: torch.Tensor
    o: torch.Tensor                     # [W, H V]
    ob: torch.Tensor                    # [W]
    lam: float
    cos_sin: Optional[torch.Tensor]     # [positions, rot_dims] fp32
    koff: int = 0
    voff: int = 0
    goff: int = 0


@dataclass
class _Scan:
    cfg: MixerConfig
    kind: int
    w_in: torch.Tensor                  # hgrn2: q | f | v;  mlstm: q | k | v | i | f | g
    cols: Dict[str, int]
    norm: torch.Tensor
    o: torch.Tensor
    fb: Optional[torch.Tensor] = None
    ib: Optional[torch.Tensor] = None
    lower: Optional[torch.Tensor] = None


@dataclass
class _Moe:
    cfg: MlpConfig
    up: torch.Tensor                    # [E, F, W]
    down: torch.Tensor                  # [E, W, F]
    router: torch.Tensor                # [E, W]
    s_up: Optional[torch.Tensor] = None
    s_down: Optional[torch.Tensor] = None


@dataclass
class _Layer:
    n1: torch.Tensor
    mixer: object
    n2: Optional[torch.Tensor]
    mlp: Optional[_Moe]
    cache: int = -1                     # index into kv_cache (attention) or states (recurrences)


def _columns(parts) -> Dict[str, int]:
    cols, at = {}, 0
    for key, n in parts:
        cols[key] = at
        at += n
    return cols


class RupatarModel(StreamModel):
    def __init__(self, cfg: RupatarConfig, tp: Optional[TPGroup] = None, device="cpu", dtype=torch.bfloat16,
                 seed: int = 0, weights: Optional[str] = None, tensors: Optional[Dict[str, torch.Tensor]] = None,
                 max_model_len: int = 8192, weight_dtype: str = "bf16"):
        super().__init__(cfg, tp, device, dtype, seed, max_model_len, weight_dtype)
        self._rope: Dict[tuple, torch.Tensor] = {}
        if tensors is None:
            tensors = self._open(Path(weights)) if weights else random_tensors(cfg, seed, self.device)
        get = tensors if callable(tensors) else tensors.__getitem__
        self._build(get)

    # ------------------------------------------------------------------ weights
    def _rope_table(self, m: MixerConfig) -> Optional[torch.Tensor]:
        if not m.rot_dims:
            return None
        key = (m.rot_dims, m.rot_base, m.rot_factor)
        if key not in self._rope:
            self._rope[key] = ref.rope_table(m.rot_dims, self.max_model_len, m.rot_base,
                                             {"type": "linear", "factor": m.rot_factor}).to(self.device).contiguous()
        return self._rope[key]

    def _build(self, get) -> None:
        c, t = self.cfg, self._t
        W = c.hidden
        if W % c.norm_groups:
            raise ValueError(f"{c.name}: {c.norm_groups} norm groups do not divide the width {W}")
        self.embed = t(get("embed"))
        self.final_norm = t(get("final.norm"))
        self.lm_head = t(get("head"))
        self.layers: List[_Layer] = []
        n_att = n_scan = 0
        for i, L in enumerate(c.layers):
            p, m = f"l{i}.mix.", L.mixer
            H, D, V = m.heads, m.dim, m.vdim
            if m.type == "attention":
                G = m.kv_heads
                if H % G:
                    raise ValueError(f"layer {i}: {H} query heads over {G} key / value heads")
                if m.rot_dims > D or m.rot_dims % 2:
                    raise ValueError(f"layer {i}: rot.dims {m.rot_dims} must be even and at most dim {D}")
                cols = _columns((("q", H * D), ("k", G * D), ("v", G * V), ("g", H * V)))
                mixer = _Attention(m, t(torch.cat([get(p + s) for s in ("q", "k", "v", "g")])), t(get(p + "q.b")),
                                   t(get(p + "k.b")), t(get(p + "v.b")), t(get(p + "o")), t(get(p + "o.b")),
                                   float(get(p + "vmix").float()) if m.v_mix else 0.0, self._rope_table(m),
                                   cols["k"], cols["v"], cols["g"])
                cache, n_att = n_att, n_att + 1
            else:
                if max(D, V) > sm.gated_scan_max_dim():
                    raise ValueError(f"layer {i}: head sizes {D} x {V} exceed {sm.gated_scan_max_dim()}")
                if m.type == "hgrn2":
                    cols = _columns((("q", H * D), ("f", H * D), ("v", H * V)))
                    mixer = _Scan(m, sm.SCAN_HGRN2, t(torch.cat([get(p + s) for s in ("q", "f", "v")])), cols,
                                  t(get(p + "norm")), t(get(p + "o")), fb=t(get(p + "f.b")), lower=t(get(p + "lower")))
                else:
                    cols = _columns((("q", H * D), ("k", H * D), ("v", H * V), ("i", H), ("f", H), ("g", H * V)))
                    mixer = _Scan(m, sm.SCAN_MLSTM, t(torch.cat([get(p + s) for s in ("q", "k", "v", "i", "f", "g")])),
                                  cols, t(get(p + "norm")), t(get(p + "o")), fb=t(get(p + "f.b")), ib=t(get(p + "i.b")))
                cache, n_scan = n_scan, n_scan + 1
            f, mlp, n2 = L.mlp, None, None
            if f is not None:
                q = f"l{i}.mlp."
                n2 = t(get(f"l{i}.norm2"))
                mlp = _Moe(f, t(torch.stack([get(f"{q}e{e}.up") for e in range(f.experts)])),
                           t(torch.stack([get(f"{q}e{e}.down") for e in range(f.experts)])), t(get(q + "router")))
                if f.shared_ff:
                    mlp.s_up, mlp.s_down = t(get(q + "shared.up")), t(get(q + "shared.down"))
            self.layers.append(_Layer(t(get(f"l{i}.norm1")), mixer, n2, mlp, cache))

    def _weight_roots(self) -> tuple:
        return (self.embed, self.final_norm, self.lm_head, *self.layers)

    # ------------------------------------------------------------------ cache and state
    def _attention_layers(self) -> List[_Attention]:
        return [L.mixer for L in self.layers if isinstance(L.mixer, _Attention)]

    def _scan_layers(self) -> List[_Scan]:
        return [L.mixer for L in self.layers if isinstance(L.mixer, _Scan)]

    def _needs_state(self) -> bool:
        return bool(self._scan_layers())

    def allocate_kv(self, num_blocks: int, block_size: int):
        """Per attention layer: paged keys [slots, G, D] and values [slots, G, V], and (pooled blocks) their fp32 means
        [pages * ceil(block_size / pool), G, D or V], a block's entry kept with the page of its first token."""
        self.block_size = block_size
        self.kv_cache = []
        for a in self._attention_layers():
            m, n = a.cfg, num_blocks * block_size
            kc = torch.zeros(n, m.kv_heads, m.dim, dtype=self.dtype, device=self.device)
            vc = torch.zeros(n, m.kv_heads, m.vdim, dtype=self.dtype, device=self.device)
            kp = vp = None
            if m.pool:
                e = num_blocks * sm.pool_entries_per_page(block_size, m.pool)
                kp = torch.zeros(e, m.kv_heads, m.dim, dtype=F32, device=self.device)
                vp = torch.zeros(e, m.kv_heads, m.vdim, dtype=F32, device=self.device)
            self.kv_cache.append((kc, vc, kp, vp))
        return self.kv_cache

    def kv_bytes_per_block(self, block_size: int) -> int:
        eb = torch.finfo(self.dtype).bits // 8
        n = 0
        for a in self._attention_layers():
            m = a.cfg
            row = m.kv_heads * (m.dim + m.vdim)
            n += block_size * row * eb + sm.pool_entries_per_page(block_size, m.pool) * row * 4
        return max(1, n)

    def allocate_state(self, slots: int) -> None:
        """Per recurrent layer and request slot: the heads' fp32 state records."""
        self.state_slots = slots
        self.states = [torch.zeros(slots, s.cfg.heads, sm.gated_scan_record(s.kind, s.cfg.dim, s.cfg.vdim), dtype=F32,
                                   device=self.device) for s in self._scan_layers()]

    def state_bytes_per_slot(self) -> int:
        return sum(s.cfg.heads * sm.gated_scan_record(s.kind, s.cfg.dim, s.cfg.vdim) * 4 for s in self._scan_layers())

    # ------------------------------------------------------------------ layers
    def _attention(self, w: _Attention, L: _Layer, h, b):
        m = w.cfg
        H, G, D, V = m.heads, m.kv_heads, m.dim, m.vdim
        kc, vc, kp, vp = self.kv_cache[L.cache]
        proj = sm.linear(h, w.w_in)                                        # [T, q | k | v | gate]
        v_in = v_out = None
        if m.v_mix:
            if b.get("v_first") is None:
                v_out = b["v_first"] = torch.empty(h.shape[0], G * V, dtype=F32, device=h.device)
            else:
                v_in = b["v_first"]
                if v_in.shape[1] != G * V:
                    raise ValueError("value mixing needs equal value sizes in the mixing layers")
        sm.window_kv_write(kc, vc, proj, w.koff, w.voff, w.qb, w.kb, w.vb, w.cos_sin, b["positions"], b["slot_mapping"],
                           H, G, D, V, m.rot_dims, self.cfg.rms_eps, True, vfirst_in=v_in, vfirst_out=v_out, lam=w.lam)
        if m.pool:
            sm.window_pool(kp, vp, kc, vc, b["block_tables"], b["tok_seq"], b["positions"], m.pool, self.block_size)
        a = sm.window_attention(proj, proj[:, w.goff:w.goff + H * V], kc, vc, kp, vp, b["block_tables"], b["tok_seq"],
                                b["positions"], H, m.window, m.pool, m.scale, True, self.block_size, b["cu_q"],
                                b.get("max_qlen", 0), b.get("max_keys", 0))
        return sm.linear(a, w.o), w.ob

    def _scan(self, w: _Scan, L: _Layer, h, b):
        m = w.cfg
        proj = sm.linear(h, w.w_in, out_dtype=F32)                         # gates and decays stay fp32
        y = sm.gated_scan(proj, w.kind, w.cols, w.norm, self.states[L.cache], b["cu_q"], b["seq_slots"], b["positions"],
                          m.heads, m.dim, m.vdim, self.cfg.rms_eps, self.dtype, fbias=w.fb, ibias=w.ib, lower=w.lower,
                          cap=m.gate_cap)
        return sm.linear(y, w.o), None

    def _moe(self, w: _Moe, h) -> torch.Tensor:
        f = w.cfg
        T = h.shape[0]
        logits = sm.linear(h, w.router, out_dtype=F32)                     # router in fp32
        idx, wts = sm.moe_route(logits, f.experts, f.top, 1.0, score="sigmoid")
        sorted_tok, pos, seg, tiles = sm.moe_align(idx, f.experts)
        P = T * f.top
        u = sm.gemm(h, w.up, a_rows=sorted_tok, tiles=tiles, rows=P, seg=seg)             # [P, F]
        # the router weight scales the expert's input: W_up (s x) = s (W_up x), applied before the activation
        a = sm.act(u, sm.ACT_GELU_ERF, row_scale=wts.view(-1), row_map=pos)
        d = sm.gemm(a, w.down, tiles=tiles, rows=P, seg=seg)
        shared = None
        if w.s_up is not None:
            shared = sm.linear(sm.act(sm.linear(h, w.s_up), sm.ACT_GELU_ERF), w.s_down)
        return sm.moe_combine(d, pos, None, shared, None, -1, top=f.top)

    def _blocks(self, ids, b, after=None):
        """The residual stream before the last pending branch is added: (x, pending branch, pending bias)."""
        c, dt = self.cfg, self.dtype
        kw = dict(out_dtype=dt, groups=c.norm_groups)
        x = sm.embed_rows(ids, self.embed, c.embed_scale)
        b["v_first"] = None
        pend = bias = None                # the branch output not yet added: the next norm adds it in fp32
        for L in self.layers:
            h = sm.resnorm(x, L.n1, c.rms_eps, branch=pend, rowvec=bias, **kw)
            run = self._attention if isinstance(L.mixer, _Attention) else self._scan
            pend, bias = run(L.mixer, L, h, b)
            if L.mlp is not None:
                h = sm.resnorm(x, L.n2, c.rms_eps, branch=pend, rowvec=bias, **kw)
                pend, bias = self._moe(L.mlp, h), None
            if after is not None:
                sm.resnorm(x, None, c.rms_eps, branch=pend, rowvec=bias, **kw)
                pend = bias = None
                after.append(x.clone())
        return x, pend, bias

    def _forward(self, ids, b, rows) -> torch.Tensor:
        c = self.cfg
        x, pend, bias = self._blocks(ids, b)
        xs = x.index_select(0, rows)
        hf = sm.resnorm(xs, self.final_norm, c.rms_eps, branch=pend.index_select(0, rows) if pend is not None else None,
                        rowvec=bias, out_dtype=self.dtype, groups=c.norm_groups)
        return sm.linear(hf, self.lm_head, out_dtype=F32).unsqueeze(0)                    # [1, S, vocab]

    def residual_after_runs(self, ids, b) -> List[torch.Tensor]:
        """(debugging / tests) the fp32 residual stream after every layer."""
        after: List[torch.Tensor] = []
        self._blocks(ids, b, after)
        return after
