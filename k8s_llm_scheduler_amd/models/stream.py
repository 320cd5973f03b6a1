"""What the models with an fp32 residual stream and per-slot recurrent state share: checkpoint access, the engine
interface (``forward_prefill`` over varlen batches, ``forward_decode`` over the slot rows) and checkpoint writing.

A subclass builds its weights (``_build``), owns its caches and states (``allocate_kv``, ``allocate_state``,
``kv_bytes_per_block``, ``state_bytes_per_slot``) and runs a batch (``_forward(ids, b, rows)`` with the batch
description ``b`` made here)."""

from __future__ import annotations

import json
from pathlib import Path
from typing import Callable, Dict, Optional

import torch

from ..parallel import TPGroup


def save_checkpoint(config_json: dict, tensors: Dict[str, torch.Tensor], path: Path) -> None:
    """config.json + model.safetensors in ``path``."""
    from safetensors.torch import save_file

    path = Path(path)
    path.mkdir(parents=True, exist_ok=True)
    save_file({k: v.detach().cpu().contiguous() for k, v in tensors.items()}, str(path / "model.safetensors"))
    (path / "config.json").write_text(json.dumps(config_json))


class StreamModel:
    stateful = True          # per-slot recurrent state: the engine passes each sequence's slot, keeps prefix caching,
    prefill_graphs = False   # speculative decoding and padded prefill graphs off
    gather_logits = True
    prefill_overlap = False
    prefill_overlap_min = 1 << 30
    fused_decode = True

    def __init__(self, cfg, tp: Optional[TPGroup], device, dtype, seed: int, max_model_len: int, weight_dtype: str):
        self.cfg = cfg
        self.tp = tp or TPGroup()
        cfg.validate_tp(self.tp.world)
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("dtype must be bfloat16 or float32")
        if weight_dtype != "bf16":
            raise ValueError(f"{cfg.name}: weight_dtype {weight_dtype!r} is not supported")
        self.device = torch.device(device)
        self.dtype = dtype
        self.seed = seed
        self.max_model_len = min(max_model_len, cfg.max_position)
        self.block_size = 16
        self.kv_cache = None
        self.states: list = []
        self.state_slots = 0

    # ------------------------------------------------------------------ weights
    @staticmethod
    def _open(path: Path) -> Callable[[str], torch.Tensor]:
        from safetensors import safe_open

        files = sorted(path.glob("*.safetensors")) if path.is_dir() else [path]
        if not files:
            raise FileNotFoundError(f"no *.safetensors in {path}")
        index: Dict[str, object] = {}
        for f in files:
            h = safe_open(str(f), framework="pt")
            for k in h.keys():
                index[k] = h
        return lambda name: index[name].get_tensor(name)

    def _t(self, t: torch.Tensor) -> torch.Tensor:
        return t.to(self.dtype).to(self.device).contiguous()

    def _weight_roots(self) -> tuple:
        raise NotImplementedError

    def weight_bytes(self) -> int:
        n = 0
        seen = set()

        def add(o):
            nonlocal n
            if isinstance(o, torch.Tensor):
                if o.data_ptr() not in seen:
                    seen.add(o.data_ptr())
                    n += o.numel() * o.element_size()
            elif hasattr(o, "__dict__"):
                for v in vars(o).values():
                    add(v)

        for o in self._weight_roots():
            add(o)
        return n

    # ------------------------------------------------------------------ engine interface
    def _needs_state(self) -> bool:
        raise NotImplementedError

    def _check_ready(self) -> None:
        if self.kv_cache is None or (self._needs_state() and not self.states):
            raise RuntimeError("allocate_kv / allocate_state first")

    def batch_meta(self, positions, slot_mapping, cu_q, block_tables, seq_slots) -> dict:
        T = positions.shape[0]
        tok = torch.arange(T, dtype=torch.int32, device=positions.device)
        tok_seq = torch.searchsorted(cu_q[1:].contiguous(), tok, right=True).to(torch.int32)
        return {"positions": positions.contiguous(), "slot_mapping": slot_mapping.contiguous(),
                "cu_q": cu_q.contiguous(), "tok_seq": tok_seq, "block_tables": block_tables.contiguous(),
                "seq_slots": seq_slots.to(torch.int32).contiguous()}

    def forward_prefill(self, ids, positions, slot_mapping, cu_q, context_lens, block_tables, max_qlen, last_idx,
                        split=None, seq_slots=None) -> torch.Tensor:
        """Varlen batch: portions of several sequences (a running decode is a 1-token portion).  ``seq_slots``: the
        state slot of every sequence.  Returns fp32 logits [1, len(last_idx), vocab]."""
        self._check_ready()
        if seq_slots is None:
            raise ValueError("a stateful model needs the sequences' state slots")
        b = self.batch_meta(positions, slot_mapping, cu_q, block_tables, seq_slots)
        b["max_qlen"] = int(max_qlen)
        return self._forward(ids, b, last_idx.long())

    def forward_decode(self, tokens, context_lens, block_tables, max_context, cascade=None) -> torch.Tensor:
        """One token for each of the B slot rows (row i = state slot i); rows with context length 0 are idle and
        touch neither cache nor state."""
        self._check_ready()
        B = tokens.shape[0]
        dev = tokens.device
        bs = self.block_size
        pos = (context_lens - 1).clamp(min=0).long()
        blk = block_tables.long().gather(1, (pos // bs).unsqueeze(1)).squeeze(1)
        slots = torch.where(context_lens > 0, blk * bs + pos % bs, torch.full_like(blk, -1)).to(torch.int32)
        ar = torch.arange(B + 1, dtype=torch.int32, device=dev)
        b = {"positions": (context_lens - 1).to(torch.int32), "slot_mapping": slots.contiguous(), "cu_q": ar,
             "tok_seq": ar[:B], "block_tables": block_tables.contiguous(), "seq_slots": ar[:B],
             "max_keys": int(max_context)}
        return self._forward(tokens, b, ar[:B].long())

    def warm(self) -> None:
        pass
