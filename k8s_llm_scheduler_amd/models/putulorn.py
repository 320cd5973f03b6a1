"""Putulorn: a decoder with an fp32 residual stream whose layers alternate, in any order the config lists, between

* ``wkv``: a recurrent mixer (token shift with learned per-channel mixes, a data-dependent per-channel decay
  ``w = exp(-exp(W2 tanh(W1 x) + w0))``, a matrix state ``S <- diag(w) S + k v^T`` per head read with a current-token
  bonus ``(S + diag(u) k v^T)^T r``, per-head unit norm, silu output gate), and
* ``latent_attention``: sliding-window softmax attention whose keys and values are up-projections of one cached
  low-rank row per token (RMS-normed latent + one rotary key part shared by the heads); queries are absorbed into the
  latent space (``q W_uk``), so the cache is attended as it is stored and ``W_uv`` is applied after the softmax;

each followed by a dense gated feed-forward (tanh-gelu) or a mixture of experts (softmax router, top-k renormalised and
scaled, clamped ``g sigmoid(1.702 g) (u + 1)`` experts, an optional sigmoid-gated shared expert) or nothing.  A span of
layers may run several times in a row with shared weights (``loop``): every pass has its own cache / state and adds
its own learned vector to the stream before its first layer.  Pre-norm blocks ``x += m * f(norm(x))`` with norm weights
stored around zero (``1 + w``).

The model presents the interface the engine drives (``forward_prefill`` over varlen batches, ``forward_decode`` over
the slot rows, ``allocate_kv``) plus ``allocate_state``: per-slot recurrent state next to the paged cache.  Every op
is a kernel of :mod:`..ops.seqmix` (fitting bf16 products go to the framework's tuned GEMMs); ``dtype=float32`` runs
everything in true fp32.  Single rank (TP = 1).
"""

from __future__ import annotations

import json
import math
from dataclasses import dataclass, field
from pathlib import Path
from typing import Callable, Dict, List, Optional

import torch

from ..ops import reference as ref
from ..ops import seqmix as sm
from ..parallel import TPGroup
from . import stream
from .stream import StreamModel

ARCHITECTURE = "Putulorn"
SWISH_ALPHA = 1.702          # the experts' sigmoid slope
MU_ORDER = ("r", "k", "v", "g", "w")


# ----------------------------------------------------------------------------- configuration
@dataclass
class MixerConfig:
    type: str
    heads: int
    dim: int
    # latent attention only
    rot_dim: int = 0
    vdim: int = 0
    kv_rank: int = 0
    window: int = 0          # 0: no window
    rot_dims: int = 0
    rot_base: float = 10000.0
    scale: float = 1.0
    decay_rank: int = 0      # wkv: rank of the decay's low-rank projection when weights are generated (0: H D / 16)


@dataclass
class MlpConfig:
    kind: str                # "dense" | "moe"
    ff: int = 0
    experts: int = 0
    top: int = 0
    router_scale: float = 1.0
    limit: float = 0.0       # 0: no clamp
    shared_ff: int = 0       # 0: no shared expert
    shared_limit: float = 0.0


@dataclass
class LayerConfig:
    mixer: MixerConfig
    mlp: Optional[MlpConfig]


@dataclass
class PutulornConfig:
    name: str
    vocab: int
    hidden: int
    layers: List[LayerConfig]
    rms_eps: float = 1e-6
    residual_mult: float = 1.0
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1
    max_position: int = 1 << 20
    bos_id: int = 0
    eos_ids: tuple = ()
    extra: dict = field(default_factory=dict)
    token_ids_only = True    # checkpoints of this design ship no tokenizer: requests are token ids

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    def runs(self) -> List[tuple]:
        """(layer, pass) in execution order; pass is the loop pass number at the pass's first layer, else None."""
        n = len(self.layers)
        if self.loop_times <= 1 and self.loop_stop <= self.loop_start:
            return [(i, None) for i in range(n)]
        out = [(i, None) for i in range(self.loop_start)]
        for t in range(self.loop_times):
            out += [(i, t if i == self.loop_start else None) for i in range(self.loop_start, self.loop_stop)]
        return out + [(i, None) for i in range(self.loop_stop, n)]

    def validate_tp(self, tp: int) -> None:
        if tp != 1:
            raise ValueError(f"{self.name}: this design runs on one rank (tp={tp})")


def _mixer_from(d: dict, kind: str) -> MixerConfig:
    if kind == "wkv":
        return MixerConfig("wkv", int(d["heads"]), int(d["dim"]))
    if kind != "latent_attention":
        raise ValueError(f"unknown mixer type {kind!r}")
    rot = d.get("rot") or {}
    rot_dim = int(d.get("rot_dim", 0))
    mask = d.get("mask") or {}
    dim = int(d["dim"])
    return MixerConfig("latent_attention", int(d["heads"]), dim, rot_dim=rot_dim, vdim=int(d["vdim"]),
                       kv_rank=int(d["kv_rank"]), window=int(mask.get("size") or 0),
                       rot_dims=int(rot.get("dims", rot_dim)), rot_base=float(rot.get("base", 10000.0)),
                       scale=float(d.get("scale", 1.0 / math.sqrt(dim + rot_dim))))


def _mlp_from(d: Optional[dict]) -> Optional[MlpConfig]:
    if d is None:
        return None
    if d["kind"] == "dense":
        return MlpConfig("dense", ff=int(d["ff"]))
    if d["kind"] != "moe":
        raise ValueError(f"unknown mlp kind {d['kind']!r}")
    r, e, s = d["router"], d["expert"], d.get("shared")
    return MlpConfig("moe", ff=int(e["ff"]), experts=int(r["experts"]), top=int(r["top"]),
                     router_scale=float(r.get("scale", 1.0)), limit=float(e.get("limit") or 0.0),
                     shared_ff=int(s["ff"]) if s else 0, shared_limit=float(s.get("limit") or 0.0) if s else 0.0)


def config_from_json(c: dict, name: str = "putulorn") -> PutulornConfig:
    layers = [LayerConfig(_mixer_from(l["mixer"], l["type"]), _mlp_from(l.get("mlp"))) for l in c["layers"]]
    loop = c.get("loop") or {}
    return PutulornConfig(name=name, vocab=int(c["vocab"]), hidden=int(c["width"]), layers=layers,
                          rms_eps=float((c.get("norm") or {}).get("eps", 1e-6)),
                          residual_mult=float(c.get("residual_mult", 1.0)), loop_start=int(loop.get("start", 0)),
                          loop_stop=int(loop.get("stop", 0)), loop_times=int(loop.get("times", 1)))


def config_to_json(cfg: PutulornConfig) -> dict:
    layers = []
    for L in cfg.layers:
        m = L.mixer
        if m.type == "wkv":
            mixer = {"heads": m.heads, "dim": m.dim}
        else:
            mixer = {"heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "vdim": m.vdim, "kv_rank": m.kv_rank,
                     "rot": {"dims": m.rot_dims, "base": m.rot_base}, "scale": m.scale}
            if m.window:
                mixer["mask"] = {"size": m.window}
        p = L.mlp
        if p is None:
            mlp = None
        elif p.kind == "dense":
            mlp = {"kind": "dense", "ff": p.ff}
        else:
            mlp = {"kind": "moe", "router": {"experts": p.experts, "top": p.top, "scale": p.router_scale},
                   "expert": {"ff": p.ff, **({"limit": p.limit} if p.limit else {})}}
            if p.shared_ff:
                mlp["shared"] = {"ff": p.shared_ff, **({"limit": p.shared_limit} if p.shared_limit else {})}
        layers.append({"type": m.type, "mixer": mixer, "mlp": mlp})
    out = {"architecture": ARCHITECTURE, "vocab": cfg.vocab, "width": cfg.hidden, "layers": layers,
           "norm": {"eps": cfg.rms_eps}, "residual_mult": cfg.residual_mult}
    if cfg.loop_stop > cfg.loop_start:
        out["loop"] = {"start": cfg.loop_start, "stop": cfg.loop_stop, "times": cfg.loop_times}
    return out


def tensor_shapes(cfg: PutulornConfig) -> Dict[str, tuple]:
    """Checkpoint tensor names and shapes of a configuration."""
    W = cfg.hidden
    t: Dict[str, tuple] = {"embed": (cfg.vocab, W), "final.norm": (W,), "head": (cfg.vocab, W)}
    if cfg.loop_stop > cfg.loop_start:
        t["loop.step"] = (cfg.loop_times, W)
    for i, L in enumerate(cfg.layers):
        p, m = f"l{i}.", L.mixer
        t[p + "norm1"] = (W,)
        if m.type == "wkv":
            HD = m.heads * m.dim
            lora = m.decay_rank or max(8, HD // 16)
            for s in MU_ORDER:
                t[p + "mix.mu." + s] = (W,)
            for s in ("r", "k", "v", "g"):
                t[p + "mix." + s] = (HD, W)
            t.update({p + "mix.w1": (lora, W), p + "mix.w2": (HD, lora), p + "mix.w0": (HD,),
                      p + "mix.u": (m.heads, m.dim), p + "mix.norm": (HD,), p + "mix.o": (W, HD)})
        else:
            t.update({p + "mix.q": (m.heads * (m.dim + m.rot_dim), W), p + "mix.dkv": (m.kv_rank + m.rot_dim, W),
                      p + "mix.dkv.norm": (m.kv_rank,), p + "mix.uk": (m.heads * m.dim, m.kv_rank),
                      p + "mix.uv": (m.heads * m.vdim, m.kv_rank), p + "mix.o": (W, m.heads * m.vdim)})
        f = L.mlp
        if f is None:
            continue
        t[p + "norm2"] = (W,)
        if f.kind == "dense":
            t.update({p + "mlp.gate": (f.ff, W), p + "mlp.up": (f.ff, W), p + "mlp.down": (W, f.ff)})
        else:
            for e in range(f.experts):
                t.update({f"{p}mlp.e{e}.gate": (f.ff, W), f"{p}mlp.e{e}.up": (f.ff, W), f"{p}mlp.e{e}.down": (W, f.ff)})
            t[p + "mlp.router"] = (f.experts, W)
            if f.shared_ff:
                t.update({p + "mlp.shared.gate": (f.shared_ff, W), p + "mlp.shared.up": (f.shared_ff, W),
                          p + "mlp.shared.down": (W, f.shared_ff), p + "mlp.shared.sg": (1, W)})
    return t


def random_tensors(cfg: PutulornConfig, seed: int = 0, device="cpu") -> Dict[str, torch.Tensor]:
    """Random bf16 weights of a configuration (benchmarks and tests): projections ~ N(0, 1 / fan_in), norm weights and
    token-shift mixes small, decay offsets spread so that the heads forget at different rates."""
    g = torch.Generator(device=device).manual_seed(seed)
    out: Dict[str, torch.Tensor] = {}
    rand = lambda shape, generator: torch.rand(shape, generator=generator, device=device)
    randn = lambda shape, generator: torch.randn(shape, generator=generator, device=device)
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.rsplit(".", 1)[-1]
        if ".mu." in name:
            t = rand(shape, g)
        elif leaf in ("norm", "norm1", "norm2") and len(shape) == 1:
            t = randn(shape, g) * 0.1 + (1.0 if name.endswith("dkv.norm") or ".mix.norm" in name else 0.0)
        elif leaf == "w0":
            t = rand(shape, g) * 4.0 - 3.0
        elif leaf == "u":
            t = randn(shape, g) * 0.5
        elif leaf == "step":
            t = randn(shape, g) * 0.1
        elif leaf == "embed":
            t = randn(shape, g)
        else:
            t = randn(shape, g) / math.sqrt(shape[-1])
        out[name] = t.to(torch.bfloat16)
    return out


def save_checkpoint(cfg: PutulornConfig, tensors: Dict[str, torch.Tensor], path: Path) -> None:
    stream.save_checkpoint(config_to_json(cfg), tensors, path)


def preset(name: str, width: int, vocab: int, pairs: int, *, heads: int, wkv_dim: int, dim: int, rot_dim: int, vdim: int,
           kv_rank: int, window: int, ff: int, experts: int = 0, top: int = 0, expert_ff: int = 0,
           loop: tuple = ()) -> PutulornConfig:
    """``pairs`` x (latent attention + dense feed-forward, wkv + mixture of experts or dense)."""
    layers = []
    for _ in range(pairs):
        layers.append(LayerConfig(MixerConfig("latent_attention", heads, dim, rot_dim=rot_dim, vdim=vdim,
                                              kv_rank=kv_rank, window=window, rot_dims=rot_dim, rot_base=10000.0,
                                              scale=1.0 / math.sqrt(dim + rot_dim)), MlpConfig("dense", ff=ff)))
        mlp = MlpConfig("moe", ff=expert_ff, experts=experts, top=top, router_scale=1.0, limit=7.0,
                        shared_ff=expert_ff, shared_limit=7.0) if experts else MlpConfig("dense", ff=ff)
        layers.append(LayerConfig(MixerConfig("wkv", width // wkv_dim, wkv_dim), mlp))
    lp = loop or (0, 0, 1)
    return PutulornConfig(name, vocab, width, layers, residual_mult=1.0, loop_start=lp[0], loop_stop=lp[1],
                          loop_times=lp[2])


PRESETS = {
    # runs on the CPU in tests: every branch (both mixers, dense + experts + shared expert, a looped span)
    "putulorn-tiny": preset("putulorn-tiny", 128, 512, 2, heads=4, wkv_dim=32, dim=32, rot_dim=16, vdim=32, kv_rank=64,
                            window=24, ff=256, experts=8, top=2, expert_ff=64, loop=(1, 3, 2)),
    # layer shapes of a ~1B-class model (benchmarks, random weights)
    "putulorn-1b": preset("putulorn-1b", 2048, 32768, 8, heads=16, wkv_dim=64, dim=128, rot_dim=64, vdim=128,
                          kv_rank=512, window=1024, ff=8192, experts=16, top=2, expert_ff=2048),
    # the same width with dense feed-forwards only: beside a Llama of equal width and depth
    "putulorn-1b-dense": preset("putulorn-1b-dense", 2048, 32768, 8, heads=16, wkv_dim=64, dim=128, rot_dim=64,
                                vdim=128, kv_rank=512, window=1024, ff=8192),
}


# ----------------------------------------------------------------------------- weights
@dataclass
class _Wkv:
    cfg: MixerConfig
    mu: torch.Tensor        # [5, W]: r, k, v, g, w
    w_rkvg: torch.Tensor    # [4, H D, W]
    w1: torch.Tensor        # [lora, W]
    w2: torch.Tensor        # [H D, lora]
    w0: torch.Tensor        # [H D]
    u: torch.Tensor         # [H D]
    lnw: torch.Tensor       # [H D]
    o: torch.Tensor         # [W, H D]


@dataclass
class _Latent:
    cfg: MixerConfig
    q: torch.Tensor         # [H (Dn + R), W]
    dkv: torch.Tensor       # [C + R, W]
    dkv_norm: torch.Tensor  # [C]
    uk_t: torch.Tensor      # [H, C, Dn]: per head W_uk^T (absorbs the query into the latent space)
    uv: torch.Tensor        # [H, V, C]
    o: torch.Tensor         # [W, H V]
    cos_sin: torch.Tensor   # [positions, rot_dims] fp32


@dataclass
class _Mlp:
    cfg: MlpConfig
    wgu: Optional[torch.Tensor] = None      # dense: [2 F, W]; moe: [E, 2 F, W]
    down: Optional[torch.Tensor] = None     # dense: [W, F];   moe: [E, W, F]
    router: Optional[torch.Tensor] = None   # [E (+ 1), W]: the shared expert's gate row appended
    s_wgu: Optional[torch.Tensor] = None
    s_down: Optional[torch.Tensor] = None
    sg_col: int = -1


@dataclass
class _Layer:
    n1: torch.Tensor
    mixer: object
    n2: Optional[torch.Tensor]
    mlp: Optional[_Mlp]


@dataclass
class _Run:
    layer: int
    step: Optional[int]     # loop pass whose vector is added before this run
    cache: int = -1         # index into kv_caches (latent attention) or states (wkv)


class PutulornModel(StreamModel):
    def __init__(self, cfg: PutulornConfig, tp: Optional[TPGroup] = None, device="cpu", dtype=torch.bfloat16,
                 seed: int = 0, weights: Optional[str] = None, tensors: Optional[Dict[str, torch.Tensor]] = None,
                 max_model_len: int = 8192, weight_dtype: str = "bf16"):
        super().__init__(cfg, tp, device, dtype, seed, max_model_len, weight_dtype)
        self._rope: Dict[tuple, torch.Tensor] = {}
        if tensors is None:
            tensors = self._open(Path(weights)) if weights else random_tensors(cfg, seed, self.device)
        get = tensors if callable(tensors) else tensors.__getitem__
        self._build(get)
        self.runs: List[_Run] = []
        n_lat = n_wkv = 0
        for li, step in cfg.runs():
            if cfg.layers[li].mixer.type == "wkv":
                self.runs.append(_Run(li, step, n_wkv))
                n_wkv += 1
            else:
                self.runs.append(_Run(li, step, n_lat))
                n_lat += 1

    # ------------------------------------------------------------------ weights
    def _rope_table(self, dims: int, base: float) -> torch.Tensor:
        key = (dims, base)
        if key not in self._rope:
            self._rope[key] = ref.rope_table(dims, self.max_model_len, base).to(self.device).contiguous() if dims \
                else torch.zeros(self.max_model_len, 0, device=self.device)
        return self._rope[key]

    def _build(self, get) -> None:
        c, t = self.cfg, self._t
        W = c.hidden
        self.embed = t(get("embed"))
        self.final_norm = t(get("final.norm"))
        self.lm_head = t(get("head"))
        self.loop_step = t(get("loop.step")) if c.loop_stop > c.loop_start else None
        self.layers: List[_Layer] = []
        for i, L in enumerate(c.layers):
            p, m = f"l{i}.mix.", L.mixer
            if m.type == "wkv":
                mixer = _Wkv(m, t(torch.stack([get(p + "mu." + s) for s in MU_ORDER])),
                             t(torch.stack([get(p + s) for s in ("r", "k", "v", "g")])), t(get(p + "w1")),
                             t(get(p + "w2")), t(get(p + "w0")), t(get(p + "u").reshape(-1)), t(get(p + "norm")),
                             t(get(p + "o")))
                if m.dim > sm.wkv_max_dim():
                    raise ValueError(f"layer {i}: wkv head dimension {m.dim} exceeds {sm.wkv_max_dim()}")
            else:
                H, Dn, C, V = m.heads, m.dim, m.kv_rank, m.vdim
                if m.rot_dims > m.rot_dim or m.rot_dims % 2:
                    raise ValueError(f"layer {i}: rot.dims {m.rot_dims} must be even and at most rot_dim {m.rot_dim}")
                mixer = _Latent(m, t(get(p + "q")), t(get(p + "dkv")), t(get(p + "dkv.norm")),
                                t(get(p + "uk").reshape(H, Dn, C).transpose(1, 2)), t(get(p + "uv").reshape(H, V, C)),
                                t(get(p + "o")), self._rope_table(m.rot_dims, m.rot_base))
            f, mlp, n2 = L.mlp, None, None
            if f is not None:
                q = f"l{i}.mlp."
                n2 = t(get(f"l{i}.norm2"))
                if f.kind == "dense":
                    mlp = _Mlp(f, t(torch.cat([get(q + "gate"), get(q + "up")])), t(get(q + "down")))
                else:
                    wgu = torch.stack([torch.cat([get(f"{q}e{e}.gate"), get(f"{q}e{e}.up")]) for e in range(f.experts)])
                    down = torch.stack([get(f"{q}e{e}.down") for e in range(f.experts)])
                    mlp = _Mlp(f, t(wgu), t(down))
                    router = get(q + "router")
                    if f.shared_ff:
                        mlp.s_wgu = t(torch.cat([get(q + "shared.gate"), get(q + "shared.up")]))
                        mlp.s_down = t(get(q + "shared.down"))
                        try:
                            router = torch.cat([router, get(q + "shared.sg").reshape(1, W)])
                            mlp.sg_col = f.experts
                        except KeyError:
                            pass
                    mlp.router = t(router)
            self.layers.append(_Layer(t(get(f"l{i}.norm1")), mixer, n2, mlp))

    def _weight_roots(self) -> tuple:
        return (self.embed, self.final_norm, self.lm_head, self.loop_step, *self.layers)

    # ------------------------------------------------------------------ cache and state
    def _latent_runs(self):
        return [(r, self.layers[r.layer].mixer) for r in self.runs if isinstance(self.layers[r.layer].mixer, _Latent)]

    def _wkv_runs(self):
        return [(r, self.layers[r.layer].mixer) for r in self.runs if isinstance(self.layers[r.layer].mixer, _Wkv)]

    def allocate_kv(self, num_blocks: int, block_size: int):
        """One paged cache per latent-attention run (a looped layer has one per pass): [slots, kv_rank + rot_dim]."""
        self.block_size = block_size
        self.kv_cache = [torch.zeros(num_blocks * block_size, m.cfg.kv_rank + m.cfg.rot_dim, dtype=self.dtype,
                                     device=self.device) for _, m in self._latent_runs()]
        return self.kv_cache

    def kv_bytes_per_block(self, block_size: int) -> int:
        eb = torch.finfo(self.dtype).bits // 8
        return max(1, sum(block_size * (m.cfg.kv_rank + m.cfg.rot_dim) * eb for _, m in self._latent_runs()))

    def allocate_state(self, slots: int) -> None:
        """Per recurrent run and sequence slot: the heads' matrix state (fp32) and the previous token's mixer input."""
        self.state_slots = slots
        self.states = [(torch.zeros(slots, m.cfg.heads, m.cfg.dim, m.cfg.dim, dtype=torch.float32, device=self.device),
                        torch.zeros(slots, self.cfg.hidden, dtype=self.dtype, device=self.device))
                       for _, m in self._wkv_runs()]

    def state_bytes_per_slot(self) -> int:
        eb = torch.finfo(self.dtype).bits // 8
        return sum(m.cfg.heads * m.cfg.dim * m.cfg.dim * 4 + self.cfg.hidden * eb for _, m in self._wkv_runs())

    # ------------------------------------------------------------------ layers
    def _wkv(self, w: _Wkv, run: _Run, h, b) -> torch.Tensor:
        m = w.cfg
        S, shift = self.states[run.cache]
        mix = sm.token_shift(h, w.mu, shift, b["cu_q"], b["tok_seq"], b["seq_slots"], b["positions"])   # [5, T, W]
        sm.shift_save(shift, h, b["cu_q"], b["seq_slots"], b["positions"])
        if sm.FAST_GEMM and h.is_cuda and sm._route_fast(mix[0], w.w_rkvg[0], self.dtype):
            r, k, v, g = (sm.linear(mix[i], w.w_rkvg[i]) for i in range(4))
        else:
            r, k, v, g = sm.gemm(mix[:4], w.w_rkvg).unbind(0)
        lo = sm.act(sm.linear(mix[4], w.w1), sm.ACT_TANH)
        z = sm.linear(lo, w.w2, out_dtype=torch.float32)                  # decay logits stay fp32
        y = sm.wkv_scan(r, k, v, g, z, w.w0, w.u, w.lnw, S, b["cu_q"], b["seq_slots"], b["positions"], m.heads, m.dim,
                        self.cfg.rms_eps)
        return sm.linear(y, w.o)

    def _latent(self, w: _Latent, run: _Run, h, b) -> torch.Tensor:
        m = w.cfg
        T = h.shape[0]
        H, Dn, R, C, V = m.heads, m.dim, m.rot_dim, m.kv_rank, m.vdim
        cache = self.kv_cache[run.cache]
        q = sm.linear(h, w.q)                                              # [T, H (Dn + R)]
        dkv = sm.linear(h, w.dkv)                                          # [T, C + R]
        sm.latent_kv_write(cache, dkv, w.dkv_norm, q, w.cos_sin, b["positions"], b["slot_mapping"], C, R, H, Dn,
                           m.rot_dims, self.cfg.rms_eps)
        q_abs = torch.empty(T, H, C, dtype=self.dtype, device=h.device)
        sm.gemm(q.view(T, H, Dn + R)[:, :, :Dn].permute(1, 0, 2), w.uk_t, out=q_abs.permute(1, 0, 2))
        lat = sm.latent_attention(q_abs, q, cache, b["block_tables"], b["tok_seq"], b["positions"], C, R, H, Dn,
                                  m.window, m.scale, self.block_size, b.get("max_keys", 0), b["cu_q"],
                                  b.get("max_qlen", 0))                   # [T, H, C]
        a = torch.empty(T, H, V, dtype=self.dtype, device=h.device)
        sm.gemm(lat.permute(1, 0, 2), w.uv, out=a.permute(1, 0, 2))
        return sm.linear(a.view(T, H * V), w.o)

    def _mlp(self, w: _Mlp, h) -> torch.Tensor:
        f = w.cfg
        if f.kind == "dense":
            return sm.linear(sm.act(sm.linear(h, w.wgu), sm.ACT_GELU_TANH), w.down)
        T = h.shape[0]
        logits = sm.linear(h, w.router, out_dtype=torch.float32)          # router (and shared gate) in fp32
        idx, wts = sm.moe_route(logits, f.experts, f.top, f.router_scale)
        sorted_tok, pos, seg, tiles = sm.moe_align(idx, f.experts)
        P = T * f.top
        gu = sm.gemm(h, w.wgu, a_rows=sorted_tok, tiles=tiles, rows=P, seg=seg)          # [P, 2 F]
        D = sm.gemm(sm.act(gu, sm.ACT_SWISH_CLAMP, f.limit, SWISH_ALPHA), w.down, tiles=tiles, rows=P, seg=seg)
        shared = None
        if w.s_wgu is not None:
            shared = sm.linear(sm.act(sm.linear(h, w.s_wgu), sm.ACT_SWISH_CLAMP, f.shared_limit, SWISH_ALPHA), w.s_down)
        return sm.moe_combine(D, pos, wts, shared, logits, w.sg_col)

    def _forward(self, ids, b, rows) -> torch.Tensor:
        c, dt = self.cfg, self.dtype
        eps, mult = c.rms_eps, c.residual_mult
        x = sm.embed_rows(ids, self.embed)
        pend = None                       # the branch output not yet added: the next norm adds it in fp32
        for run in self.runs:
            L = self.layers[run.layer]
            step = self.loop_step[run.step] if run.step is not None else None
            h = sm.resnorm(x, L.n1, eps, branch=pend, mult=mult, rowvec=step, offset=1.0, out_dtype=dt)
            y = self._wkv(L.mixer, run, h, b) if isinstance(L.mixer, _Wkv) else self._latent(L.mixer, run, h, b)
            if L.mlp is not None:
                h = sm.resnorm(x, L.n2, eps, branch=y, mult=mult, offset=1.0, out_dtype=dt)
                pend = self._mlp(L.mlp, h)
            else:
                pend = y
        xs = x.index_select(0, rows)
        hf = sm.resnorm(xs, self.final_norm, eps, branch=pend.index_select(0, rows) if pend is not None else None,
                        mult=mult, offset=1.0, out_dtype=dt)
        return sm.linear(hf, self.lm_head, out_dtype=torch.float32).unsqueeze(0)      # [1, S, vocab]

    def residual_after_runs(self, ids, b) -> List[torch.Tensor]:
        """(debugging / tests) the fp32 residual stream after every layer run."""
        outs = []
        c, dt = self.cfg, self.dtype
        x = sm.embed_rows(ids, self.embed)
        for run in self.runs:
            L = self.layers[run.layer]
            step = self.loop_step[run.step] if run.step is not None else None
            h = sm.resnorm(x, L.n1, c.rms_eps, rowvec=step, offset=1.0, out_dtype=dt)
            y = self._wkv(L.mixer, run, h, b) if isinstance(L.mixer, _Wkv) else self._latent(L.mixer, run, h, b)
            if L.mlp is not None:
                h = sm.resnorm(x, L.n2, c.rms_eps, branch=y, mult=c.residual_mult, offset=1.0, out_dtype=dt)
                y = self._mlp(L.mlp, h)
            sm.resnorm(x, None, c.rms_eps, branch=y, mult=c.residual_mult, out_dtype=dt)
            outs.append(x.clone())
        return outs

    def _needs_state(self) -> bool:
        return bool(self._wkv_runs())
