"""Kazolorn forward pass on MI355X (``config.KazolornShape`` says what the design is).

Unlike the fp16 split-plane stacks of ``llama_hip.py`` this model keeps plain row-major tensors in ONE element type --
bfloat16 (the serving mode: matrix products on the bf16 matrix cores with fp32 accumulation) or float32 (everything in true
32-bit) -- and an fp32 residual stream; its kernels are the building blocks of ``libpromptcache_blocks.so`` (``_blocks.py``).

A step works on FLAT rows: the new tokens of all requests of the step one after another, each request appending behind the
positions its slot of the ``SlotArena`` already holds.  No padding exists anywhere, so a request's rows see the same
arithmetic whatever else is in the step; what a row reads from other rows is its own slot's keys and nothing else.

Per layer i (x = the layer's input, X_j = earlier results, X_0 = the embedding rows):

    x        = sum_j dwa_(i-1)[j] X_j              (i > 0; fused with the two norms: pcb_mix_norm)
    h1, h2   = rms(x) g1, rms(x) g2
    q | k    = Wqk h1 + b                          (one projection; the k part lands in the slot's cache rows)
    a        = attention(q, cached k; values = keys, distance bias, head mixing, window, sink)      (pcb_attn_talk)
    X_(i+1)  = x + ls1 * (Wo a + bo)               (projection epilogue)
    X_(i+1) += ls2 * ff(h2)                        (dense: up -> polynorm -> down's epilogue;
                                                    sparse: router -> bucket by expert -> gated units on w*h2 -> combine)

and the logits are ``head . rms(sum_j dwa_last[j] X_j) g`` for the rows that were asked for.
"""
from __future__ import annotations

import os
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch

from .. import _blocks as B
from .config import KazolornShape
from .kv_arena import SlotArena
from .slot_model import SlotKV, SlotModel  # noqa: F401  (SlotKV is re-exported)

ATTN_SCRATCH_FLOATS = 1 << 28          # the score band of one attention call is kept below 1 GiB (more rows: several calls)


def distance_slopes(heads: int) -> torch.Tensor:
    """slope_h = 2 ** (-8 (h + 1) / H), h = 0 .. H - 1, any head count."""
    return torch.tensor([2.0 ** (-8.0 * (h + 1) / heads) for h in range(heads)], dtype=torch.float32)


class KazolornHIP(SlotModel):
    def __init__(self, shape: KazolornShape, weights: Dict[str, torch.Tensor], device="cuda:0", dtype=torch.bfloat16,
                 decode_headroom: int = 256):
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Kazolorn runs in bfloat16 or float32")
        B.load()                                   # fail loudly (or build once) before anything else
        self.config = shape
        self.device = torch.device(device)
        self.dtype = dtype
        self.decode_headroom = decode_headroom
        self.L = len(shape.layers)
        self.W, self.V = shape.hidden_size, shape.vocab_size
        dev = self.device

        def e(name):                               # element-type tensor (projections, biases, tables)
            return weights[name].to(device=dev, dtype=dtype).contiguous()

        def f(name):                               # fp32 tensor (gains, scales, coefficients, routers)
            return weights[name].to(device=dev, dtype=torch.float32).contiguous()

        self.embed = e("embed")
        self.final_norm = f("final.norm")
        self.head = e("head")
        self.layers = []
        for i, l in enumerate(shape.layers):
            p = f"l{i}."
            ent = dict(cfg=l, g1=f(p + "norm1"), ls1=f(p + "ls1"), dwa=f(p + "dwa"),
                       wqk=torch.cat([e(p + "mix.q"), e(p + "mix.k")], dim=0).contiguous(),
                       bqk=torch.cat([e(p + "mix.q.b"), e(p + "mix.k.b")], dim=0).contiguous(),
                       talk=f(p + "mix.talk"), wo=e(p + "mix.o"), bo=e(p + "mix.o.b"),
                       slopes=distance_slopes(l.heads).to(dev))
            if ent["dwa"].numel() < i + 2:
                raise ValueError(f"{p}dwa has {ent['dwa'].numel()} weights, layer {i} sums {i + 2} streams")
            ent["dwa"] = ent["dwa"].reshape(-1)[:i + 2].contiguous()
            if l.heads > 32 or l.dim > 256:
                raise ValueError(f"layer {i}: the attention kernels take up to 32 heads of up to 256 columns (got {l.heads} x {l.dim})")
            if l.mlp_kind:
                ent.update(g2=f(p + "norm2"), ls2=f(p + "ls2"))
            if l.mlp_kind == "dense":
                ent.update(up=e(p + "mlp.up"), down=e(p + "mlp.down"), act=f(p + "mlp.act"))
            elif l.mlp_kind == "moe":
                ent.update(router=e(p + "mlp.router"),
                           gate=torch.stack([e(p + f"mlp.e{j}.gate") for j in range(l.experts)]).contiguous(),
                           up=torch.stack([e(p + f"mlp.e{j}.up") for j in range(l.experts)]).contiguous(),
                           down=torch.stack([e(p + f"mlp.e{j}.down") for j in range(l.experts)]).contiguous())
            self.layers.append(ent)
        self._buf = {}
        self.default_arena: Optional[SlotArena] = None
        self.use_graphs = os.environ.get("PC_KZ_GRAPHS", "1") != "0"      # one-token steps replay a captured hipGraph
        self._graphs = {}
        self.max_graphs = 16

    # ---- cache -------------------------------------------------------------------------------------------------------------
    def new_arena(self, slots: int, cap: int) -> SlotArena:
        return SlotArena([(l.kv_heads, l.dim) for l in self.config.layers], slots, cap, self.device, self.dtype)

    def kv_bytes_per_token(self) -> int:
        return sum(l.kv_heads * l.dim for l in self.config.layers) * (2 if self.dtype == torch.bfloat16 else 4)

    # ---- one step ------------------------------------------------------------------------------------------------------------
    @torch.inference_mode()
    def forward_rows(self, arena: SlotArena, slots: Sequence[int], tokens: Sequence[Sequence[int]],
                     want: Optional[Sequence[Sequence[int]]] = None, num_layers: Optional[int] = None,
                     return_streams: bool = False):
        """Append ``tokens[b]`` behind slot ``slots[b]`` for every b, and return fp32 logits ``[n_wanted, vocab]`` for the places
        ``want[b]`` (indices into ``tokens[b]``; default: each request's last token), in request order.
        ``return_streams``: also the layer inputs that follow each layer, fp32 ``[layers, rows, width]`` (for tests)."""
        dev, E, f32 = self.device, self.dtype, torch.float32
        counts = [len(t) for t in tokens]
        if len(set(slots)) != len(slots) or len(slots) != len(tokens):
            raise ValueError("one distinct slot per request")
        if not counts:
            return torch.empty((0, self.V), dtype=f32, device=dev)
        if min(counts, default=1) < 1:
            raise ValueError("every request of a step brings at least one token")
        T = sum(counts)
        if want is None:
            want = [[c - 1] for c in counts]
        for s, c in zip(slots, counts):
            arena.room_for(s, c)
        starts = [arena.lengths[s] for s in slots]
        max_kv = max(st + c for st, c in zip(starts, counts))
        W, V = self.W, self.V

        # host-side tables of the step, one upload
        ids = np.fromiter((t for req in tokens for t in req), dtype=np.int32, count=T)
        if ids.size and (ids.min() < 0 or ids.max() >= V):
            raise ValueError("token id outside the vocabulary")
        row_slot = np.repeat(np.asarray(slots, dtype=np.int64), counts)
        row_pos = np.concatenate([np.arange(st, st + c, dtype=np.int64) for st, c in zip(starts, counts)])
        row0 = np.concatenate([[0], np.cumsum(counts)])
        tiles = []
        for b, (s, st, c) in enumerate(zip(slots, starts, counts)):
            for q in range(0, c, 16):
                tiles.append((s, st + q, min(16, c - q), int(row0[b]) + q))
        tiles = np.asarray(tiles, dtype=np.int32).reshape(-1, 4)
        tiles64 = np.asarray([(s, st + q, min(64, c - q), int(row0[b]) + q) for b, (s, st, c) in enumerate(zip(slots, starts, counts))
                              for q in range(0, c, 64)], dtype=np.int32).reshape(-1, 4)
        for b, ws in enumerate(want):
            if any(not 0 <= int(w) < counts[b] for w in ws):
                raise ValueError("a wanted place lies outside its request's tokens")
        # one-token steps run as a captured graph whose launches have fixed sizes: logits of every row, picked from afterwards
        graphed = (self.use_graphs and T <= self.GRAPH_MAX_ROWS and all(c == 1 for c in counts) and num_layers is None
                   and not return_streams)
        picked = None
        if graphed and any(len(ws) != 1 for ws in want):
            picked = [b for b, ws in enumerate(want) for _ in ws]
        want_rows = np.arange(T, dtype=np.int32) if graphed else \
            np.asarray([int(row0[b]) + int(w) for b, ws in enumerate(want) for w in ws], dtype=np.int32)
        sigs = sorted({(l.kv_heads, l.dim) for l in self.config.layers})
        offs = np.stack([row_slot * (g * arena.cap * d) + row_pos * d for g, d in sigs]) if T else np.zeros((len(sigs), 0), np.int64)
        n32 = T + tiles.size + want_rows.size + tiles64.size
        blob = np.empty(n32 * 4 + offs.size * 8 + 8, dtype=np.uint8)
        o64 = (n32 * 4 + 7) // 8 * 8
        blob[:n32 * 4].view(np.int32)[:] = np.concatenate([ids, tiles.reshape(-1), want_rows, tiles64.reshape(-1)])
        blob[o64:o64 + offs.size * 8].view(np.int64)[:] = offs.reshape(-1)
        n_want = int(want_rows.size)
        res = self._decode_graphed(arena, T, blob, n32, o64, sigs) if graphed else None
        if res is None:
            dblob = torch.from_numpy(blob).to(dev)
            logits = torch.empty((n_want, V), dtype=f32, device=dev)
            res = self._run(arena, T, dblob, n32, o64, sigs, tiles, tiles.shape[0], tiles64.shape[0], n_want, max_kv, logits,
                            num_layers, return_streams)
        for s_, c in zip(slots, counts):
            arena.lengths[s_] += c
        if picked is not None:
            res = res[torch.as_tensor(picked, dtype=torch.long, device=dev)] if picked else res[:0]
        return res

    def _run(self, arena, T, dblob, n32, o64, sigs, tiles, n_tiles, n64, n_want, max_kv, logits, num_layers=None,
             return_streams=False):
        """The device side of a step: every launch of the forward, reading the step's tables from ``dblob`` (token ids, the two
        tile tables, wanted rows as int32, then the cache offsets of every row as int64)."""
        dev, E, f32 = self.device, self.dtype, torch.float32
        W, V = self.W, self.V
        d32 = dblob[:n32 * 4].view(torch.int32)
        ids_d, tiles_d = d32[:T], d32[T:T + 4 * n_tiles]
        want_d = d32[T + 4 * n_tiles:T + 4 * n_tiles + n_want]
        tiles64_d = d32[T + 4 * n_tiles + n_want:T + 4 * n_tiles + n_want + 4 * n64]
        offs_d = dblob[o64:o64 + len(sigs) * T * 8].view(torch.int64).view(len(sigs), T)
        layers = self.layers if num_layers is None else self.layers[:num_layers]
        L = len(layers)
        hist = self._scratch("hist", (L + 1) * T * W, f32)[:(L + 1) * T * W].view(L + 1, T, W)
        x = self._mat("x", T, W, f32)
        h1, h2 = self._mat("h1", T, W, E), self._mat("h2", T, W, E)
        streams = torch.empty((L, T, W), dtype=f32, device=dev) if return_streams else None
        B.embed_rows(self.embed, ids_d, hist[0])
        eps = self.config.norm_eps

        for i, lw in enumerate(layers):
            l = lw["cfg"]
            has_ff = l.mlp_kind is not None
            if i == 0:
                B.mix_norm(hist, 1, None, lw["g1"], h1, lw.get("g2"), h2 if has_ff else None, eps=eps, n_rows=T)
                base = hist[0]
            else:
                B.mix_norm(hist, i + 1, layers[i - 1]["dwa"], lw["g1"], h1, lw.get("g2"), h2 if has_ff else None, x_out=x,
                           eps=eps, n_rows=T)
                base = x
                if streams is not None:
                    streams[i - 1].copy_(x)
            HD, GD = l.heads * l.dim, l.kv_heads * l.dim
            q = self._mat("q", T, HD, E)
            plane = arena.planes[i]
            B.linear(h1, lw["wqk"], q, M=T, bias=lw["bqk"], split_n=HD, y2=plane, row_off2=offs_d[sigs.index((l.kv_heads, l.dim))],
                     head_dim2=l.dim, head_stride2=arena.head_stride(i))
            att = self._mat("att", T, HD, E)
            self._attention(q, att, tiles, n_tiles, tiles_d, tiles64_d, n64, plane, arena, i, l, lw, max_kv,
                            max_rows=1 if n_tiles == T else (int(tiles[:, 2].max()) if tiles is not None and n64 == n_tiles else 0))
            B.linear(att, lw["wo"], hist[i + 1], M=T, epilogue=B.EPI_SCALE_ADD, bias=lw["bo"], base=base, col_scale=lw["ls1"])
            if l.mlp_kind == "dense":
                z = self._mat("z", T, l.ff, f32)
                B.linear(h2, lw["up"], z, M=T)
                act = self._mat("act", T, l.ff, E)
                B.polynorm(z, lw["act"], act, eps, T)
                B.linear(act, lw["down"], hist[i + 1], M=T, epilogue=B.EPI_SCALE_ADD, col_scale=lw["ls2"])
            elif l.mlp_kind == "moe":
                P = T * l.top
                ex = self._scratch("moe_i", 3 * P + l.experts + 1, torch.int32)
                sc = self._scratch("moe_f", 2 * P, f32)
                expert, row_src, row_dst, goff = ex[:P], ex[P:2 * P], ex[2 * P:3 * P], ex[3 * P:3 * P + l.experts + 1]
                weight, row_scale = sc[:P], sc[P:2 * P]
                rl = self._mat("router", T, l.experts, f32)
                B.linear(h2, lw["router"], rl, M=T)                  # fp32 accumulation of exact products: 32-bit logits
                B.router_topk(rl, l.top, expert, weight, T)
                B.moe_plan(expert, weight, P, l.top, l.experts, goff, row_src, row_dst, row_scale)
                gact = self._mat("gact", P, l.ff, E)
                B.linear(h2, lw["gate"], gact, M=P, epilogue=B.EPI_SILU_MUL, w2=lw["up"], row_src=row_src, row_scale=row_scale,
                         group_off=goff, n_groups=l.experts)
                pair = self._mat("pair", P, W, f32)
                B.linear(gact, lw["down"], pair, M=P, row_dst=row_dst, group_off=goff, n_groups=l.experts)
                B.moe_combine(pair, lw["ls2"], hist[i + 1], T, l.top)

        if streams is not None:
            B.mix_norm(hist, L + 1, layers[-1]["dwa"], None, None, x_out=x, eps=eps, n_rows=T)
            streams[L - 1].copy_(x)
        if n_want:
            hn = self._mat("hn", n_want, W, E)
            B.mix_norm(hist, L + 1, layers[-1]["dwa"], self.final_norm, hn, rows=want_d, eps=eps, n_rows=n_want)
            B.linear(hn, self.head, logits, M=n_want)
        return (logits, streams) if return_streams else logits

    # ---- decode steps as captured graphs -----------------------------------------------------------------------------------------
    GRAPH_MAX_ROWS = 64

    def _decode_graphed(self, arena, T, blob, n32, o64, sigs):
        """A step of T requests with one token each, replayed from a hipGraph captured per (T, arena planes).  What changes between
        steps -- tokens, slots, positions -- lives in the step's tables, which the graph reads from a device block that one copy
        from pinned memory refreshes; every launch dimension is sized for the arena's row capacity instead of the current
        lengths.  Returns None when the score band of such a launch would be too large (the caller then runs eagerly)."""
        cap = arena.cap
        worst = max(16 * T * l.heads * B.attn_talk_band(l.window, cap) for l in self.config.layers)
        if worst > ATTN_SCRATCH_FLOATS // 4:
            return None
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
            saved, self._buf = self._buf, ent["bufs"]             # the graph owns its scratch: later, larger steps may regrow the shared one
            try:
                args = (arena, T, ent["dev"], n32, o64, sigs, None, T, T, T, cap, ent["logits"])
                self._run(*args)                                  # eager first: sizes every scratch buffer, and is this step's result
                torch.cuda.synchronize()
                prime_graph_capture(self.device)
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g):
                    self._run(*args)
                ent["graph"] = g
            finally:
                self._buf = saved
            # (the eager run already appended this step's keys and produced its logits; the capture itself launches nothing)
            return ent["logits"].clone()
        ent["graph"].replay()
        return ent["logits"].clone()

    def _attention(self, q, att, tiles, n_tiles, tiles_d, tiles64_d, n64, plane, arena, i, l, lw, max_kv, max_rows=0):
        band = B.attn_talk_band(l.window, max_kv)
        per_tile = 16 * l.heads * band
        chunk = max(1, ATTN_SCRATCH_FLOATS // per_tile)
        if n_tiles <= chunk:
            scratch = self._scratch("band", n_tiles * per_tile, torch.float32)
            B.attn_talk(q, tiles_d, n_tiles, plane, arena.slot_stride(i), arena.head_stride(i), l.heads, l.kv_heads, l.dim, l.scale,
                        l.window, max_kv, lw["slopes"], lw["talk"], True, scratch, att, tiles64=tiles64_d, n_tiles64=n64,
                        max_tile_rows=max_rows)
            return
        # too many rows for one score band: several calls, each over a run of tiles with rows counted from the run's first
        scratch = self._scratch("band", chunk * per_tile, torch.float32)
        for lo in range(0, n_tiles, chunk):
            part = tiles[lo:lo + chunk].copy()
            r0 = int(part[0, 3])
            part[:, 3] -= r0
            part_d = torch.from_numpy(part.reshape(-1)).to(self.device)
            B.attn_talk(q[r0:], part_d, part.shape[0], plane, arena.slot_stride(i), arena.head_stride(i), l.heads, l.kv_heads, l.dim,
                        l.scale, l.window, max_kv, lw["slopes"], lw["talk"], True, scratch, att[r0:])
