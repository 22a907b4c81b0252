"""Dibizen forward pass on MI355X (``config.DibizenShape`` says what the design is).

Like ``kazolorn_hip.KazolornHIP`` this model keeps plain row-major tensors in one element type E -- bfloat16 (serving: matrix
products on the bf16 matrix cores, fp32 accumulation) or float32 (everything in true 32-bit) -- runs on the building blocks of
``libpromptcache_blocks.so`` (``_blocks.py``) and steps over FLAT rows: the new tokens of all requests of a step one after
another, each request continuing from what its slot of the ``SlotArena`` holds.  Nothing is padded, and a row reads nothing but
its own slot, so a request's numbers do not depend on the rest of the step.

What a slot holds differs by layer: an attention layer keeps keys (row by row) and values (column by column, so that the matrix
cores' value operand -- eight positions of one column -- is read with wide loads; a layer that borrows another layer's keys and
values keeps nothing), a lightning layer one fp32 matrix per head, a
mamba layer its fp32 scan state and the last inputs of its convolution.

There are S residual streams X_1..X_S (fp32, all equal to the embedding rows at first).  Sublayer by sublayer (f = mixer or
feed-forward, with its own in / mix / out weights and Dynamic-Tanh norm):

    u   = sum_s in[s] X_s                       h = tanh(alpha u) w + b              (pcb_hyper_norm, read half)
    y   = f(h)                                  fp32 rows
    X_t <- sum_s mix[s][t] X_s + out[t] y       (pcb_hyper_norm, write half -- fused with the next sublayer's read half)

    lightning   q | k | v | g = silu, silu, silu, sigmoid of ONE projection; per head S <- decay S + k v^T, o = S^T q
                (pcb_decay_attn); y = Wo (rms(o) gain * g)                           (pcb_gated_norm)
    attention   q | g | k | v of ONE projection whose k and v columns land in the slot's cache; softmax(temp(pos) scale q.k) v,
                times sigmoid(g) in the attention kernel's store (pcb_attn_softmax); y = Wo (.)
    mamba1      x | z = Win h; x = silu(conv(x)) (pcb_causal_conv); dt_low | B | C = Wx x; dt = softplus(Wdt dt_low + b);
                S <- exp(dt A) S + dt x B, y = (S C + D x) silu(z) (pcb_selective_scan); y = Wo (.)
    experts     router logits (fp32) -> softmax, corrected choice scores, best groups, top-k, weights renormalised
                (pcb_router_select); pairs bucketed by expert (pcb_moe_plan); relu(Wup h)^2 and Wdown per bucket (grouped
                pcb_linear); y = sum_k w_k (expert result, or h itself for an identity expert)   (pcb_moe_mix)

and the logits are ``cap tanh(head . dyt(sum_s X_s) / cap)`` for the rows that were asked for.
"""
from __future__ import annotations

import math
import os
from typing import Dict, Optional, Sequence

import numpy as np
import torch

from .. import _blocks as B
from .config import DibizenShape
from .kv_arena import SlotArena
from .slot_model import SlotKV, SlotModel  # noqa: F401


class DibizenHIP(SlotModel):
    GRAPH_MAX_ROWS = 64
    SEGMENT = int(os.environ.get("PC_DZ_SEGMENT", "128"))   # a step that brings a request more tokens than this runs its recurrent mixers segment-parallel
    MAX_SEGMENTS = 64       # (segments grow beyond SEGMENT tokens rather than exceed this many per request)

    def __init__(self, shape: DibizenShape, weights: Dict[str, torch.Tensor], device="cuda:0", dtype=torch.bfloat16,
                 decode_headroom: int = 256):
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Dibizen runs in bfloat16 or float32")
        B.load()                                   # fail loudly (or build once) before anything else
        self.config = shape
        self.device = torch.device(device)
        self.dtype = dtype
        self.decode_headroom = decode_headroom
        self.L = len(shape.layers)
        self.W, self.V, self.S = shape.hidden_size, shape.vocab_size, shape.streams
        if not 1 <= self.S <= 8:
            raise ValueError(f"1 to 8 residual streams (got {self.S})")
        dev = self.device

        def e(name):                               # element-type tensor (projections, tables, biases of projections)
            return weights[name].to(device=dev, dtype=dtype).contiguous()

        def f(name):                               # fp32 tensor (norms, stream weights, decays, router corrections)
            return weights[name].to(device=dev, dtype=torch.float32).contiguous()

        def norm(name):
            return dict(gain=f(name), bias=f(name + ".b"), alpha=f(name + ".alpha").reshape(1))

        def hyper(name):
            return dict(in_w=f(name + ".in"), out_w=f(name + ".out"), mix=f(name + ".mix"))

        self.embed, self.pos = e("embed"), e("pos")
        self.max_positions = self.pos.shape[0]
        self.final_norm = norm("final.norm")
        self.head = e("head")
        self.layers = []
        for i, l in enumerate(shape.layers):
            p, m = f"l{i}.", f"l{i}.mix."
            ent = dict(cfg=l, norm1=norm(p + "norm1"), hc1=hyper(p + "hc1"))
            if l.kind == "lightning":
                if l.dim > 256:
                    raise ValueError(f"layer {i}: lightning heads take up to 256 key columns (got {l.dim})")
                ent.update(w_in=torch.cat([e(m + "q"), e(m + "k"), e(m + "v"), e(m + "g")], dim=0).contiguous(), wo=e(m + "o"),
                           gain=f(m + "norm"), decay=torch.tensor(l.decay, dtype=torch.float32, device=dev))
                # ln(decay) per state element: the factor a state takes over a segment of n tokens is exp(n ln(decay))
                lnd = torch.tensor([math.log(d) if d > 0 else -math.inf for d in l.decay], dtype=torch.float32, device=dev)
                ent["ln_decay"] = lnd.view(-1, 1).expand(l.heads, l.dim * l.vdim).reshape(-1).contiguous()
            elif l.kind == "attention":
                if max(l.dim, l.vdim) > 256:
                    raise ValueError(f"layer {i}: attention heads take up to 256 columns (got {l.dim} / {l.vdim})")
                parts = [e(m + "q"), e(m + "g")] + ([e(m + "k"), e(m + "v")] if l.kv_from < 0 else [])
                ent.update(w_in=torch.cat(parts, dim=0).contiguous(), wo=e(m + "o"))
            else:
                if l.state > 256 or l.conv > 16:
                    raise ValueError(f"layer {i}: up to 256 states per channel and 16 taps (got {l.state}, {l.conv})")
                wx = e(m + "x")
                ent.update(w_in=e(m + "in"), conv=e(m + "conv"), conv_b=e(m + "conv.b"), wx_dt=wx[:l.dt_rank].contiguous(),
                           wx_bc=wx[l.dt_rank:].contiguous(), wdt=e(m + "dt"), dt_b=e(m + "dt.b"),
                           A=(-torch.exp(f(m + "A_log"))).contiguous(), D=f(m + "D"), wo=e(m + "o"))
            if l.experts + l.identity:
                if l.experts + l.identity > 2048 or l.groups > 64 or l.top > 64:
                    raise ValueError(f"layer {i}: up to 2048 router outputs in up to 64 groups, top <= 64")
                ent.update(norm2=norm(p + "norm2"), hc2=hyper(p + "hc2"), router=e(p + "mlp.router"), correction=f(p + "mlp.correction"))
                if l.experts:
                    ent.update(up=torch.stack([e(p + f"mlp.e{j}.up") for j in range(l.experts)]).contiguous(),
                               down=torch.stack([e(p + f"mlp.e{j}.down") for j in range(l.experts)]).contiguous())
            self.layers.append(ent)
        self._buf = {}
        self.default_arena: Optional[SlotArena] = None
        self.use_graphs = os.environ.get("PC_DZ_GRAPHS", "1") != "0"      # one-token steps replay a captured hipGraph
        self._graphs = {}
        self.max_graphs = 16
        # which (coef, every) pairs the attention layers' query temperatures use: one fp32 factor per row and pair
        self._temps = sorted({(l.qt_coef, l.qt_every) for l in shape.layers if l.kind == "attention" and l.qt_every})
        # cache offsets of a row, one table per distinct (heads, columns) of the key planes and of the value planes
        self._sigs = sorted({(l.kv_heads, l.dim) for l in shape.layers if l.kind == "attention" and l.kv_from < 0})
        self._vsigs = sorted({(l.kv_heads, l.vdim) for l in shape.layers if l.kind == "attention" and l.kv_from < 0})

    # ---- cache and state -------------------------------------------------------------------------------------------------------
    def new_arena(self, slots: int, cap: int) -> SlotArena:
        dims, cols, states = [], [], []
        f32 = torch.float32
        for l in self.config.layers:
            own = l.kind == "attention" and l.kv_from < 0
            dims.append((l.kv_heads, l.dim) if own else (0, 0))          # keys row by row
            cols.append((l.kv_heads, l.vdim) if own else (0, 0))         # values column by column
            if l.kind == "lightning":
                states.append([((l.heads, l.dim, l.vdim), f32)])
            elif l.kind == "mamba1":
                states.append([((l.inner, l.state), f32), ((l.conv - 1, l.inner), self.dtype)])
            else:
                states.append([])
        return SlotArena(dims, slots, cap, self.device, self.dtype, states=states, col_dims=cols)

    def kv_bytes_per_token(self) -> int:
        es = 2 if self.dtype == torch.bfloat16 else 4
        return sum(l.kv_heads * (l.dim + l.vdim) for l in self.config.layers if l.kind == "attention" and l.kv_from < 0) * es

    # ---- one step ------------------------------------------------------------------------------------------------------------
    @torch.inference_mode()
    def forward_rows(self, arena: SlotArena, slots: Sequence[int], tokens: Sequence[Sequence[int]],
                     want: Optional[Sequence[Sequence[int]]] = None, num_layers: Optional[int] = None,
                     return_streams: bool = False):
        """Append ``tokens[b]`` behind slot ``slots[b]`` for every b, and return fp32 logits ``[n_wanted, vocab]`` for the places
        ``want[b]`` (indices into ``tokens[b]``; default: each request's last token), in request order.
        ``return_streams``: also the sum of the residual streams after each layer, fp32 ``[layers, rows, width]`` (for tests)."""
        dev, f32 = self.device, torch.float32
        counts = [len(t) for t in tokens]
        if len(set(slots)) != len(slots) or len(slots) != len(tokens):
            raise ValueError("one distinct slot per request")
        if not counts:
            return torch.empty((0, self.V), dtype=f32, device=dev)
        if min(counts) < 1:
            raise ValueError("every request of a step brings at least one token")
        T, R = sum(counts), len(counts)
        if want is None:
            want = [[c - 1] for c in counts]
        for s, c in zip(slots, counts):
            arena.room_for(s, c)
        starts = [arena.lengths[s] for s in slots]
        if max(st + c for st, c in zip(starts, counts)) > self.max_positions:
            raise ValueError(f"a request would pass position {self.max_positions - 1}, the last one the position table has")
        V = self.V

        ids = np.fromiter((t for req in tokens for t in req), dtype=np.int32, count=T)
        if ids.min() < 0 or ids.max() >= V:
            raise ValueError("token id outside the vocabulary")
        for b, ws in enumerate(want):
            if any(not 0 <= int(w) < counts[b] for w in ws):
                raise ValueError("a wanted place lies outside its request's tokens")
        row0 = np.concatenate([[0], np.cumsum(counts)]).astype(np.int64)
        row_slot = np.repeat(np.asarray(slots, dtype=np.int64), counts)
        row_idx = np.concatenate([np.arange(c, dtype=np.int64) for c in counts])
        row_pos = row_idx + np.repeat(np.asarray(starts, dtype=np.int64), counts)
        meta = np.stack([row_slot, row_pos, row_idx, np.zeros_like(row_idx)], axis=1).astype(np.int32)
        reqs = np.asarray([(s, st, c, int(row0[b])) for b, (s, st, c) in enumerate(zip(slots, starts, counts))], dtype=np.int32)
        tiles = np.asarray([(s, st + q, min(16, c - q), int(row0[b]) + q) for b, (s, st, c) in enumerate(zip(slots, starts, counts))
                            for q in range(0, c, 16)], dtype=np.int32).reshape(-1, 4)
        graphed = (self.use_graphs and T <= self.GRAPH_MAX_ROWS and all(c == 1 for c in counts) and num_layers is None
                   and not return_streams)
        picked = None
        if graphed and any(len(ws) != 1 for ws in want):
            picked = [b for b, ws in enumerate(want) for _ in ws]
        want_rows = np.arange(T, dtype=np.int32) if graphed else \
            np.asarray([int(row0[b]) + int(w) for b, ws in enumerate(want) for w in ws], dtype=np.int32)
        # segments of the recurrent mixers' prefill (only when some request brings more than SEGMENT tokens)
        seg_a = seg_c = chains = np.zeros((0, 4), np.int32)
        seg_n = np.zeros(0, np.float32)
        if max(counts) > self.SEGMENT and any(l.kind != "attention" for l in self.config.layers):
            seg = max(self.SEGMENT, -(-max(counts) // self.MAX_SEGMENTS))
            seg = -(-seg // 16) * 16
            sa, ch = [], []
            for b, (s, st, c) in enumerate(zip(slots, starts, counts)):
                ch.append((s, st, len(sa), -(-c // seg)))
                sa += [(len(sa) + k, 0, min(seg, c - q), int(row0[b]) + q) for k, q in enumerate(range(0, c, seg))]
            seg_a = np.asarray(sa, dtype=np.int32)
            seg_c = seg_a.copy()
            seg_c[:, 1] = 1                                 # the second pass starts every segment from a state that was put there
            chains = np.asarray(ch, dtype=np.int32)
            seg_n = seg_a[:, 2].astype(np.float32)
        temps = np.stack([1.0 + coef * np.log(np.floor((row_pos + 1) / every) + 1.0) for coef, every in self._temps]).astype(np.float32) \
            if self._temps else np.zeros((0, T), np.float32)
        offs = np.stack([row_slot * (g * arena.cap * d) + row_pos * d for g, d in self._sigs] +
                        [row_slot * (g * d * arena.cap) + row_pos for g, d in self._vsigs]) if self._sigs else np.zeros((0, T), np.int64)
        # one block: int32 tables, then fp32 temperatures, then int64 cache offsets
        parts32 = [ids, row_pos.astype(np.int32), meta.reshape(-1), reqs.reshape(-1), tiles.reshape(-1), want_rows, seg_a.reshape(-1),
                   seg_c.reshape(-1), chains.reshape(-1)]
        n32 = sum(p.size for p in parts32)
        nf = temps.size + seg_n.size
        o64 = ((n32 + nf) * 4 + 7) // 8 * 8
        blob = np.empty(o64 + offs.size * 8 + 8, dtype=np.uint8)
        blob[:n32 * 4].view(np.int32)[:] = np.concatenate(parts32)
        blob[n32 * 4:(n32 + nf) * 4].view(np.float32)[:] = np.concatenate([temps.reshape(-1), seg_n])
        blob[o64:o64 + offs.size * 8].view(np.int64)[:] = offs.reshape(-1)
        dims = dict(T=T, R=R, n_tiles=tiles.shape[0], n_want=int(want_rows.size), n32=n32, o64=o64, n_seg=seg_a.shape[0],
                    n_chains=chains.shape[0])
        res = self._decode_graphed(arena, blob, dims) if graphed else None
        if res is None:
            dblob = torch.from_numpy(blob).to(dev)
            logits = torch.empty((dims["n_want"], V), dtype=f32, device=dev)
            res = self._run(arena, dblob, dims, logits, num_layers, return_streams)
        for s_, c in zip(slots, counts):
            arena.lengths[s_] += c
        if picked is not None:
            res = res[torch.as_tensor(picked, dtype=torch.long, device=dev)] if picked else res[:0]
        return res

    def _tables(self, dblob, d):
        T, R, nt, nw, ns = d["T"], d["R"], d["n_tiles"], d["n_want"], d["n_seg"]
        i32 = dblob[:d["n32"] * 4].view(torch.int32)
        at, out = 0, {}
        for name, n in (("ids", T), ("pos", T), ("meta", 4 * T), ("reqs", 4 * R), ("tiles", 4 * nt), ("want", nw), ("seg_a", 4 * ns),
                        ("seg_c", 4 * ns), ("chains", 4 * d["n_chains"])):
            out[name] = i32[at:at + n]
            at += n
        nf = len(self._temps) * T
        f32 = dblob[d["n32"] * 4:(d["n32"] + nf + ns) * 4].view(torch.float32)
        out["temps"] = f32[:nf].view(len(self._temps), T)
        out["seg_n"] = f32[nf:nf + ns]
        out["n_seg"], out["n_chains"] = ns, d["n_chains"]
        no = len(self._sigs) + len(self._vsigs)
        out["offs"] = dblob[d["o64"]:d["o64"] + no * T * 8].view(torch.int64).view(no, T)
        return out

    def _run(self, arena, dblob, d, logits, num_layers=None, return_streams=False):
        """The device side of a step: every launch of the forward, reading the step's tables from ``dblob``."""
        dev, E, f32 = self.device, self.dtype, torch.float32
        W, S, T, R = self.W, self.S, d["T"], d["R"]
        tb = self._tables(dblob, d)
        layers = self.layers if num_layers is None else self.layers[:num_layers]
        eps = self.config.norm_eps
        xs = self._scratch("streams", S * T * W, f32)[:S * T * W].view(S, T, W)
        y = self._mat("y", T, W, f32)
        h = self._mat("h", T, W, E)
        sums = torch.empty((len(layers), T, W), dtype=f32, device=dev) if return_streams else None
        B.embed_pos_rows(self.embed, self.pos, tb["ids"], tb["pos"], xs)
        pending = None                             # the hyper-connection whose write half is still to be applied to y

        def read(hc, nm):
            nonlocal pending
            w = pending or {}
            B.hyper_norm(xs, y=y if pending else None, mix=w.get("mix"), out_w=w.get("out_w"), in_w=hc["in_w"], norm=B.NORM_DYT,
                         gain=nm["gain"], bias=nm["bias"], alpha=nm["alpha"], eps=eps, out=h, n_rows=T)
            pending = None

        for i, lw in enumerate(layers):
            l = lw["cfg"]
            read(lw["hc1"], lw["norm1"])
            if l.kind == "lightning":
                self._lightning(arena, i, l, lw, h, y, tb, T, R)
            elif l.kind == "attention":
                self._attention(arena, i, l, lw, h, y, tb, T, d["n_tiles"])
            else:
                self._mamba(arena, i, l, lw, h, y, tb, T, R)
            pending = lw["hc1"]
            if l.experts + l.identity:
                read(lw["hc2"], lw["norm2"])
                self._experts(l, lw, h, y, T)
                pending = lw["hc2"]
            if sums is not None:
                B.hyper_norm(xs, y=y, mix=pending["mix"], out_w=pending["out_w"], x_out=sums[i], n_rows=T)
                pending = None
        if d["n_want"]:
            nw = d["n_want"]
            hn = self._mat("hn", nw, W, E)
            w = pending or {}
            fn = self.final_norm
            B.hyper_norm(xs, y=y if pending else None, mix=w.get("mix"), out_w=w.get("out_w"), norm=B.NORM_DYT, gain=fn["gain"],
                         bias=fn["bias"], alpha=fn["alpha"], eps=eps, out=hn, rows=tb["want"], n_rows=nw)
            cap = self.config.logit_softcap
            B.linear(hn, self.head, logits, M=nw, act=B.ACT_SOFTCAP if cap > 0 else B.ACT_NONE, act_param=cap)
        return (logits, sums) if return_streams else logits

    # ---- mixers ----------------------------------------------------------------------------------------------------------------
    def _lightning(self, arena, i, l, lw, h, y, tb, T, R):
        HD, HV = l.heads * l.dim, l.heads * l.vdim
        N = 2 * HD + 2 * HV
        qkvg = self._mat("mix_in", T, N, self.dtype)
        B.linear(h, lw["w_in"], qkvg, M=T, act=B.ACT_SILU, act_split=2 * HD + HV, act2=B.ACT_SIGMOID)
        o = self._mat("mix_o32", T, HV, torch.float32)
        state, ns = arena.states[i][0], tb["n_seg"]
        q, k, v = qkvg, qkvg[:, HD:], qkvg[:, 2 * HD:]
        if ns:
            # every segment from a zero state (only the states move), the segments chained, then every segment from its start state
            elems = l.heads * l.dim * l.vdim
            local = self._scratch("seg_local", ns * elems, torch.float32)[:ns * elems].view(ns, l.heads, l.dim, l.vdim)
            start = self._scratch("seg_start", ns * elems, torch.float32)[:ns * elems].view(ns, l.heads, l.dim, l.vdim)
            B.decay_attn(q, k, v, N, tb["seg_a"], ns, local, lw["decay"], l.heads, l.dim, l.vdim, None)
            B.state_chain(local, start, state, tb["chains"], tb["n_chains"], lw["ln_decay"], tb["seg_n"], elems)
            B.decay_attn(q, k, v, N, tb["seg_c"], ns, start, lw["decay"], l.heads, l.dim, l.vdim, o)
        else:
            B.decay_attn(q, k, v, N, tb["reqs"], R, state, lw["decay"], l.heads, l.dim, l.vdim, o)
        on = self._mat("mix_out", T, HV, self.dtype)
        B.gated_norm(o, lw["gain"], qkvg[:, 2 * HD + HV:], N, on, self.config.norm_eps, T)
        B.linear(on, lw["wo"], y, M=T)

    def _attention(self, arena, i, l, lw, h, y, tb, T, n_tiles):
        HD, HV, GD = l.heads * l.dim, l.heads * l.vdim, l.kv_heads * l.dim
        src = i if l.kv_from < 0 else l.kv_from
        plane, vplane = arena.planes[src], arena.col_planes[src]
        qg = self._mat("mix_in", T, HD + HV, self.dtype)
        if l.kv_from < 0:
            # one projection: q | g stay rows, the k columns go to the slot's key rows, the v columns to its value columns
            B.linear(h, lw["w_in"], qg, M=T, act_split=HD, act2=B.ACT_SIGMOID, split_n=HD + HV, y2=plane,
                     row_off2=tb["offs"][self._sigs.index((l.kv_heads, l.dim))], head_dim2=l.dim, head_stride2=arena.head_stride(src),
                     split_n3=HD + HV + GD, y3=vplane, row_off3=tb["offs"][len(self._sigs) + self._vsigs.index((l.kv_heads, l.vdim))],
                     col_stride3=arena.cap)
        else:
            B.linear(h, lw["w_in"], qg, M=T, act_split=HD, act2=B.ACT_SIGMOID)
        att = self._mat("mix_out", T, HV, self.dtype)
        temp = tb["temps"][self._temps.index((l.qt_coef, l.qt_every))] if l.qt_every else None
        # few (tile, head) pairs cannot fill the chip: each is cut into runs of its keys (steps of few rows over long caches)
        splits = 1 if n_tiles * l.heads >= 512 or arena.cap <= 256 else max(1, min(16, 1024 // (n_tiles * l.heads), arena.cap // 128))
        part = self._scratch("attn_part", B.attn_softmax_part(T, l.heads, splits, l.vdim), torch.float32) if splits > 1 else None
        B.attn_softmax(qg, HD + HV, tb["tiles"], n_tiles, plane, (arena.slot_stride(src), arena.head_stride(src), l.dim), vplane, 0,
                       (arena.col_slot_stride(src), arena.col_head_stride(src), arena.cap), True, l.heads, l.kv_heads, l.dim, l.vdim,
                       l.scale, att, q_scale=temp, gate=qg[:, HD:], ldg=HD + HV, n_splits=splits, part=part)
        B.linear(att, lw["wo"], y, M=T)

    def _mamba(self, arena, i, l, lw, h, y, tb, T, R):
        C, N, E = l.inner, l.state, self.dtype
        state, conv_state = arena.states[i]
        xz = self._mat("mix_in", T, 2 * C, E)
        B.linear(h, lw["w_in"], xz, M=T)
        xc = self._mat("mix_out", T, C, E)
        B.causal_conv(xz, 2 * C, lw["conv"], lw["conv_b"], True, tb["meta"], conv_state, xc, T)
        B.conv_state_update(xz, 2 * C, tb["reqs"], R, conv_state)
        low = self._mat("scan_low", T, l.dt_rank, E)
        B.linear(xc, lw["wx_dt"], low, M=T)
        bc = self._mat("scan_bc", T, 2 * N, torch.float32)
        B.linear(xc, lw["wx_bc"], bc, M=T)
        dt = self._mat("scan_dt", T, C, torch.float32)
        B.linear(low, lw["wdt"], dt, M=T, bias=lw["dt_b"], act=B.ACT_SOFTPLUS)
        ys = self._mat("scan_y", T, C, E)
        ns = tb["n_seg"]
        if ns:
            local = self._scratch("seg_local", ns * C * N, torch.float32)[:ns * C * N].view(ns, C, N)
            start = self._scratch("seg_start", ns * C * N, torch.float32)[:ns * C * N].view(ns, C, N)
            dsum = self._mat("seg_dt", ns, C, torch.float32)
            B.selective_scan(xc, dt, bc, None, 0, lw["A"], None, tb["seg_a"], ns, local, None, dt_sum=dsum)
            B.state_chain(local, start, state, tb["chains"], tb["n_chains"], lw["A"].view(-1), dsum, N)
            B.selective_scan(xc, dt, bc, xz[:, C:], 2 * C, lw["A"], lw["D"], tb["seg_c"], ns, start, ys)
        else:
            B.selective_scan(xc, dt, bc, xz[:, C:], 2 * C, lw["A"], lw["D"], tb["reqs"], R, state, ys)
        B.linear(ys, lw["wo"], y, M=T)

    def _experts(self, l, lw, h, y, T):
        n_out, P, W = l.experts + l.identity, T * l.top, self.W
        ex = self._scratch("moe_i", 3 * P + n_out + 1, torch.int32)
        sc = self._scratch("moe_f", 2 * P, torch.float32)
        expert, row_src, row_dst, goff = ex[:P], ex[P:2 * P], ex[2 * P:3 * P], ex[3 * P:3 * P + n_out + 1]
        weight, row_scale = sc[:P], sc[P:2 * P]
        rl = self._mat("router", T, n_out, torch.float32)
        B.linear(h, lw["router"], rl, M=T)                     # fp32 accumulation of exact products: 32-bit logits
        B.router_select(rl, l.top, expert, weight, T, score_fn=B.SCORE_SOFTMAX, correction=lw["correction"], groups=l.groups,
                        groups_keep=l.groups_keep, renorm=True)
        pair = self._mat("pair", P, W, torch.float32)
        if l.experts:
            B.moe_plan(expert, weight, P, l.top, n_out, goff, row_src, row_dst, row_scale)
            act = self._mat("moe_act", P, l.ff, self.dtype)
            B.linear(h, lw["up"], act, M=P, row_src=row_src, group_off=goff[:l.experts + 1], n_groups=l.experts, act=B.ACT_RELU2)
            B.linear(act, lw["down"], pair, M=P, row_dst=row_dst, group_off=goff[:l.experts + 1], n_groups=l.experts)
        B.moe_mix(pair, expert, weight, h, l.experts, y, T, l.top)
