"""What the flat-row models share (``kazolorn_hip.KazolornHIP``, ``dibizen_hip.DibizenHIP``): requests live on slots of a
``SlotArena``, a step is ``forward_rows(arena, slots, tokens, want)`` over the new tokens of all its requests one after another,
and the adapters' ``model(input_ids, past_key_values=...)`` convention is served on top of that."""
from __future__ import annotations

from typing import List, Optional

import torch

from .kv_arena import SlotArena
from .llama_hip import CausalLMOutput


class SlotKV:
    """``past_key_values`` of this model: the arena and the slots of the batch rows, in order."""

    def __init__(self, arena: SlotArena, slots: List[int]):
        self.arena, self.slots = arena, list(slots)

    def __len__(self):
        return len(self.arena.planes)

    def __del__(self):
        try:
            for s in self.slots:
                if s in self.arena._live:
                    self.arena.free(s)
        except Exception:
            pass


class SlotModel:
    """Mixin of the flat-row models.  The subclass provides ``device``, ``dtype``, ``V`` (vocabulary), ``decode_headroom``,
    ``default_arena``, ``_buf`` (scratch by name), ``new_arena(slots, cap)`` and ``forward_rows``; one that replays its one-token
    steps from captured graphs (``_decode_graphed``) also ``_graphs``, ``max_graphs`` and ``_run``."""

    # ---- scratch -----------------------------------------------------------------------------------------------------------
    def _scratch(self, name: str, numel: int, dtype) -> torch.Tensor:
        """A named scratch buffer of at least ``numel`` elements (grown by doubling, never shrunk)."""
        t = self._buf.get(name)
        if t is None or t.numel() < numel or t.dtype != dtype:
            n = max(numel, 2 * t.numel() if t is not None and t.dtype == dtype else 0, 1024)
            t = torch.empty(n, dtype=dtype, device=self.device)
            self._buf[name] = t
        return t

    def _mat(self, name: str, rows: int, cols: int, dtype) -> torch.Tensor:
        return self._scratch(name, max(rows, 1) * cols, dtype)[:max(rows, 1) * cols].view(max(rows, 1), cols)

    # ---- one-token steps as captured graphs (models whose step is ``_run(arena, device tables, dims, logits)``) ------------------
    def _decode_graphed(self, arena, blob, d):
        """A step of T requests with one token each, replayed from a hipGraph captured per (T, arena planes).  What changes
        between steps -- tokens, slots, positions -- lives in the step's tables, which the graph reads from a device block that
        one copy from pinned memory refreshes; no launch dimension depends on the requests' lengths."""
        T = d["T"]
        key = (T, arena.serial, arena.generation)
        ent = self._graphs.pop(key, None)
        if ent is None:
            for k in [k for k in self._graphs if k[1] == arena.serial and k[2] != arena.generation]:
                del self._graphs[k]                               # graphs over planes that have moved
            while len(self._graphs) >= self.max_graphs:
                self._graphs.pop(next(iter(self._graphs)))
            ent = dict(graph=None, bufs={}, host=torch.empty(blob.size, dtype=torch.uint8, pin_memory=True),
                       dev=torch.empty(blob.size, dtype=torch.uint8, device=self.device),
                       logits=torch.empty((T, self.V), dtype=torch.float32, device=self.device), copied=torch.cuda.Event())
        self._graphs[key] = ent                                   # (re-inserted at the young end)
        ent["copied"].synchronize()                               # the previous step's upload has left the pinned block
        ent["host"].numpy()[:] = blob
        ent["dev"].copy_(ent["host"], non_blocking=True)
        ent["copied"].record()
        if ent["graph"] is None:
            from .llama_hip import prime_graph_capture
            saved, self._buf = self._buf, ent["bufs"]             # the graph owns its scratch
            try:
                self._run(arena, ent["dev"], d, ent["logits"])    # eager first: sizes every scratch buffer, and is this step's result
                torch.cuda.synchronize()
                # (capture records the launches without executing them: the recurrent states advance once, by the eager run)
                prime_graph_capture(self.device)
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g):
                    self._run(arena, ent["dev"], d, ent["logits"])
                ent["graph"] = g
            finally:
                self._buf = saved
            return ent["logits"].clone()
        ent["graph"].replay()
        return ent["logits"].clone()

    # ---- the adapters' calling convention --------------------------------------------------------------------------------------
    @torch.inference_mode()
    def __call__(self, input_ids: torch.Tensor, position_ids: Optional[torch.Tensor] = None, past_key_values=None,
                 attention_mask: Optional[torch.Tensor] = None, use_cache: bool = True, last_token_only: bool = False,
                 num_layers: Optional[int] = None, **_unused) -> CausalLMOutput:
        """``input_ids`` [B, q]; right padding is described by ``attention_mask`` [B, q] (1 = token).  Positions count from 0 in
        each sequence and enter only as distances, so ``position_ids`` are not needed (they are accepted and ignored).
        Logits come back as [B, q, vocab] (padded places hold zeros), or [B, 1, vocab] with ``last_token_only``."""
        ids = input_ids.detach().to("cpu").reshape(input_ids.shape[0], -1)
        Bn, q_len = ids.shape
        if attention_mask is not None:
            am = attention_mask.detach().to("cpu").reshape(Bn, -1)[:, -q_len:]
            if bool((am[:, 1:] > am[:, :-1]).any()):
                raise NotImplementedError("left / interior padding masks are not supported")
            counts = [int(c) for c in am.sum(dim=1)]
        else:
            counts = [q_len] * Bn
        if past_key_values is None:
            arena = self.default_arena
            if arena is None:
                arena = self.default_arena = self.new_arena(Bn, q_len + self.decode_headroom)
            past_key_values = SlotKV(arena, [arena.alloc() for _ in range(Bn)])
        elif not isinstance(past_key_values, SlotKV) or len(past_key_values.slots) != Bn:
            raise ValueError("past_key_values must be what an earlier call of this model returned, for the same batch")
        arena, slots = past_key_values.arena, past_key_values.slots
        toks = [ids[b, :counts[b]].tolist() for b in range(Bn)]
        want = [[c - 1] for c in counts] if last_token_only else [list(range(c)) for c in counts]
        flat = self.forward_rows(arena, slots, toks, want, num_layers=num_layers)
        if last_token_only:
            logits = flat.view(Bn, 1, self.V)
        elif all(c == q_len for c in counts):
            logits = flat.view(Bn, q_len, self.V)
        else:
            logits = torch.zeros((Bn, q_len, self.V), dtype=torch.float32, device=self.device)
            at = 0
            for b, c in enumerate(counts):
                logits[b, :c] = flat[at:at + c]
                at += c
        return CausalLMOutput(logits=logits, past_key_values=past_key_values if use_cache else None)
