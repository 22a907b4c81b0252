"""Fivesun forward pass on MI355X (``config.FivesunShape`` says what the design is).

Like ``dibizen_hip.DibizenHIP`` this model keeps plain row-major tensors in one element type E -- bfloat16 (serving: matrix
products on the bf16 matrix cores, fp32 accumulation) or float32 (everything in true 32-bit) -- runs on the building blocks of
``libpromptcache_blocks.so`` (``_blocks.py``) and steps over FLAT rows: the new tokens of all requests of a step one after
another, each request continuing from what its slot of the ``SlotArena`` holds.  Nothing is padded, and a row reads nothing but
its own slot, so a request's numbers do not depend on the rest of the step.

What a slot holds differs by layer: an attention layer keeps keys (row by row, normed and rotated) and values (column by column,
normed and blended), a latent-attention layer ONE row per token -- the normed latent followed by the rotated shared key part --,
an mLSTM layer its fp32 matrix memory, normaliser and running maximum.

The residual x is fp32.  Sublayer by sublayer (f = mixer or feed-forward, each between a norm before and a norm after it):

    h = rms(x) g_before                          t = f(h) * sigmoid(W_r h + b_r)          x <- x + rms(t) g_after

``pcb_post_norm`` applies a finished sublayer's t and takes the next sublayer's norm in one launch; the sigmoid gate rides in the
same projection as the mixer's inputs (or is one projection beside the feed-forward's).

    attention   q | k | v | g | r = ONE projection (sigmoid on g | r); pcb_head_prep: per-head RMS norms, rotary pairs (angles as
                float64 products), value blend with the first blending layer's values, keys / values into the slot's cache;
                pcb_attn_softmax: keys of the query's own block of positions only, exp(sink_h) in the denominator, one gate per head
    latent      q | down | g | r = ONE projection; pcb_head_prep: the latent normed, the shared key part and the queries' rotated
                parts turned (YaRN frequencies), latent | key part into the slot's row.  The keys' and values' up-projections are
                folded into the query and the output: q'_h = W_uk,h^T q_h (grouped pcb_linear), attention of [q'_h | q_rot,h] over
                the cached rows with the latent itself as value (pcb_attn_softmax, one key head, sliding window), o_h = W_uv,h (.)
                (grouped pcb_linear), times sigmoid(g)
    mlstm       q | k | v | i | f | g | r = ONE projection; pcb_mlstm: the gated matrix memory token by token; per-head unit RMS,
                gain, sigmoid(g) (pcb_gated_norm)
    dense ff    act(W_gate h + b) * (W_up h + b) in one projection's epilogue, then W_down (.) + b

and the logits are ``head . rms(x) g`` for the rows that were asked for.
"""
from __future__ import annotations

import math
import os
from typing import Dict, Optional, Sequence

import numpy as np
import torch

from .. import _blocks as B
from .config import FivesunShape
from .kv_arena import SlotArena
from .slot_model import SlotKV, SlotModel  # noqa: F401

ACTS = {"relu": B.ACT_RELU, "silu": B.ACT_SILU, "gelu_tanh": B.ACT_GELU_TANH}


def rotary_frequencies(base: float, dims: int, factor: float = 1.0, original: float = 0.0, fast: float = 32.0, slow: float = 1.0):
    """float64 frequencies of the ``dims / 2`` rotated column pairs and the factor on cos and sin.  Plain: base^(-2i/dims) / factor.
    With ``original`` > 0 (YaRN): pairs that complete more than ``fast`` turns over ``original`` positions keep their frequency,
    those with fewer than ``slow`` turns are divided by ``factor``, a linear ramp over the pair index between them; the rotated
    vector grows by 0.1 ln(factor) + 1."""
    f = np.asarray([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=np.float64)
    if original <= 0:
        return f / factor, 1.0

    def pair_of(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo, hi = max(math.floor(pair_of(fast)), 0), min(math.ceil(pair_of(slow)), dims - 1)
    ramp = np.clip((np.arange(dims // 2, dtype=np.float64) - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


class FivesunHIP(SlotModel):
    GRAPH_MAX_ROWS = 64
    SEGMENT = int(os.environ.get("PC_FS_SEGMENT", "64"))    # a step that brings a request more tokens than this runs its mLSTM layers segment-parallel
    MAX_SEGMENTS = 128      # (segments grow beyond SEGMENT tokens rather than exceed this many per request)

    def __init__(self, shape: FivesunShape, weights: Dict[str, torch.Tensor], device="cuda:0", dtype=torch.bfloat16,
                 decode_headroom: int = 256):
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Fivesun runs in bfloat16 or float32")
        B.load()                                   # fail loudly (or build once) before anything else
        shape.check()
        self.config = shape
        self.device = torch.device(device)
        self.dtype = dtype
        self.decode_headroom = decode_headroom
        self.L = len(shape.layers)
        self.W, self.V = shape.hidden_size, shape.vocab_size
        if self.W > 16384:
            raise ValueError(f"width up to 16384 (got {self.W})")
        dev, W = self.device, self.W

        def e(name):                               # element-type tensor (projections and their biases)
            return weights[name].to(device=dev, dtype=dtype).contiguous()

        def f(name):                               # fp32 tensor (norm gains, sinks, blend weights)
            return weights[name].to(device=dev, dtype=torch.float32).contiguous()

        def zeros(n):
            return torch.zeros(n, dtype=dtype, device=dev)

        self.embed, self.final_norm, self.head = e("embed"), f("final.norm"), e("head")
        self.first_v_mix = shape.first_v_mix
        self.layers = []
        for i, l in enumerate(shape.layers):
            p, m = f"l{i}.", f"l{i}.mix."
            ent = dict(cfg=l, norm1=f(p + "norm1"), norm1b=f(p + "norm1b"))
            rg, rgb = e(p + "rg1"), e(p + "rg1.b")
            if l.kind == "attention":
                if l.dim > 384 or l.vdim > 256:
                    raise ValueError(f"layer {i}: attention heads take up to 384 key and 256 value columns (got {l.dim} / {l.vdim})")
                HD, GD, GV = l.heads * l.dim, l.kv_heads * l.dim, l.kv_heads * l.vdim
                fr, mag = rotary_frequencies(l.rot_base, l.rot_dims, l.rot_factor) if l.rot_dims else (np.zeros(0), 1.0)
                ent.update(w_in=torch.cat([e(m + "q"), e(m + "k"), e(m + "v"), e(m + "g"), rg], dim=0).contiguous(),
                           b_in=torch.cat([zeros(HD + GD + GV + l.heads), rgb]).contiguous(), act_from=HD + GD + GV,
                           q_gain=f(m + "q.norm"), k_gain=f(m + "k.norm"), sink=f(m + "sink"), wo=e(m + "o"),
                           blend=f(m + "vmix").reshape(1) if (l.v_mix and i != self.first_v_mix) else None,
                           freqs=torch.from_numpy(fr).to(dev) if l.rot_dims else None, rot_mag=mag)
            elif l.kind == "latent_attention":
                C, R = l.kv_rank, l.rot_dim
                if C + R > 384 or C > 256:
                    raise ValueError(f"layer {i}: a latent of up to 256 columns plus a rotated part within 384 together (got {C} + {R})")
                HQ, HV = l.heads * (l.dim + R), l.heads * l.vdim
                fr, mag = rotary_frequencies(l.rot_base, R, l.rot_factor, l.yarn_original, l.yarn_fast, l.yarn_slow) if R else (np.zeros(0), 1.0)
                ent.update(w_in=torch.cat([e(m + "q"), e(m + "dkv"), e(m + "g"), rg], dim=0).contiguous(),
                           b_in=torch.cat([zeros(HQ + C + R + HV), rgb]).contiguous(), act_from=HQ + C + R,
                           c_gain=f(m + "dkv.norm"), wo=e(m + "o"),
                           # per head: the key up-projection transposed ([C, dim]: it maps a query to the latent's columns) and the
                           # value up-projection as stored ([vdim, C])
                           w_abs=e(m + "uk").view(l.heads, l.dim, C).transpose(1, 2).contiguous(),
                           w_uv=e(m + "uv").view(l.heads, l.vdim, C).contiguous(),
                           freqs=torch.from_numpy(fr).to(dev) if R else None, rot_mag=mag)
            else:
                if l.dim > 256:
                    raise ValueError(f"layer {i}: mLSTM heads take up to 256 key columns (got {l.dim})")
                HD, HV, H = l.heads * l.dim, l.heads * l.vdim, l.heads
                ent.update(w_in=torch.cat([e(m + "q"), e(m + "k"), e(m + "v"), e(m + "i"), e(m + "f"), e(m + "g"), rg], dim=0).contiguous(),
                           b_in=torch.cat([zeros(2 * HD + HV), e(m + "i.b"), e(m + "f.b"), zeros(HV), rgb]).contiguous(),
                           act_from=2 * HD + HV + 2 * H, gain=f(m + "norm"), wo=e(m + "o"))
            if l.ff:
                if l.act not in ACTS:
                    raise ValueError(f"layer {i}: unknown activation {l.act!r}")
                q = p + "mlp."
                ent.update(norm2=f(p + "norm2"), norm2b=f(p + "norm2b"), rg2=e(p + "rg2"), rg2b=e(p + "rg2.b"),
                           w_gate=e(q + "gate"), b_gate=e(q + "gate.b"), w_up=e(q + "up"), b_up=e(q + "up.b"),
                           w_down=e(q + "down"), b_down=e(q + "down.b"))
            self.layers.append(ent)
        self._buf = {}
        self.default_arena: Optional[SlotArena] = None
        self.use_graphs = os.environ.get("PC_FS_GRAPHS", "1") != "0"      # one-token steps replay a captured hipGraph
        self._graphs = {}
        self.max_graphs = 16
        # cache offsets of a row, one table per distinct (heads, columns) of the row-wise planes and of the column-wise planes
        att = [l for l in shape.layers if l.kind == "attention"]
        self._sigs = sorted({(l.kv_heads, l.dim) for l in att} | {(1, l.kv_rank + l.rot_dim) for l in shape.layers if l.kind == "latent_attention"})
        self._vsigs = sorted({(l.kv_heads, l.vdim) for l in att})
        # (token, head) row orders of the per-head projections around the latent attention, one table per distinct head count
        self._perm_heads = sorted({l.heads for l in shape.layers if l.kind == "latent_attention"})

    # ---- cache and state -------------------------------------------------------------------------------------------------------
    def new_arena(self, slots: int, cap: int) -> SlotArena:
        dims, cols, states = [], [], []
        for l in self.config.layers:
            if l.kind == "attention":
                dims.append((l.kv_heads, l.dim)); cols.append((l.kv_heads, l.vdim)); states.append([])
            elif l.kind == "latent_attention":
                dims.append((1, l.kv_rank + l.rot_dim)); cols.append((0, 0)); states.append([])
            else:
                dims.append((0, 0)); cols.append((0, 0))
                states.append([((B.mlstm_state_floats(l.heads, l.dim, l.vdim),), torch.float32)])
        return SlotArena(dims, slots, cap, self.device, self.dtype, states=states, col_dims=cols)

    def kv_bytes_per_token(self) -> int:
        es = 2 if self.dtype == torch.bfloat16 else 4
        return sum(l.kv_heads * (l.dim + l.vdim) if l.kind == "attention" else (l.kv_rank + l.rot_dim if l.kind == "latent_attention" else 0)
                   for l in self.config.layers) * es

    # ---- one step ------------------------------------------------------------------------------------------------------------
    @torch.inference_mode()
    def forward_rows(self, arena: SlotArena, slots: Sequence[int], tokens: Sequence[Sequence[int]],
                     want: Optional[Sequence[Sequence[int]]] = None, num_layers: Optional[int] = None,
                     return_streams: bool = False):
        """Append ``tokens[b]`` behind slot ``slots[b]`` for every b, and return fp32 logits ``[n_wanted, vocab]`` for the places
        ``want[b]`` (indices into ``tokens[b]``; default: each request's last token), in request order.
        ``return_streams``: also the residual stream after each layer, fp32 ``[layers, rows, width]`` (for tests)."""
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
        V = self.V

        ids = np.fromiter((t for req in tokens for t in req), dtype=np.int32, count=T)
        if ids.min() < 0 or ids.max() >= V:
            raise ValueError("token id outside the vocabulary")
        for b, ws in enumerate(want):
            if any(not 0 <= int(w) < counts[b] for w in ws):
                raise ValueError("a wanted place lies outside its request's tokens")
        row0 = np.concatenate([[0], np.cumsum(counts)]).astype(np.int64)
        row_slot = np.repeat(np.asarray(slots, dtype=np.int64), counts)
        row_pos = np.concatenate([np.arange(c, dtype=np.int64) for c in counts]) + np.repeat(np.asarray(starts, dtype=np.int64), counts)
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
        # rows of the per-head projections: bucket h holds (token, head h) for every token; perm[h * T + t] = t * H + h
        perms = [np.concatenate([(np.arange(T, dtype=np.int32) * H + h) for h in range(H)] + [np.arange(H + 1, dtype=np.int32) * T])
                 for H in self._perm_heads]
        # segments of the matrix memories' prefill (only when some request brings more than SEGMENT tokens)
        seg_a = seg_c = chains = np.zeros((0, 4), np.int32)
        seg_end = np.zeros(0, np.int32)
        if max(counts) > self.SEGMENT and any(l.kind == "mlstm" for l in self.config.layers):
            seg = max(self.SEGMENT, -(-max(counts) // self.MAX_SEGMENTS))
            sa, ch = [], []
            for b, (s, st, c) in enumerate(zip(slots, starts, counts)):
                ch.append((s, st, len(sa), -(-c // seg)))
                sa += [(len(sa) + k, 0, min(seg, c - q), int(row0[b]) + q) for k, q in enumerate(range(0, c, seg))]
            seg_a = np.asarray(sa, dtype=np.int32)
            seg_c = seg_a.copy()
            seg_c[:, 1] = 1                                 # the second pass starts every segment from a state that was put there
            chains = np.asarray(ch, dtype=np.int32)
            seg_end = np.full(len(sa), -1, dtype=np.int32)  # a request's last segment leaves the slot's new state
            seg_end[chains[:, 2] + chains[:, 3] - 1] = chains[:, 0]
        offs = np.stack([row_slot * (g * arena.cap * d) + row_pos * d for g, d in self._sigs] +
                        [row_slot * (g * d * arena.cap) + row_pos for g, d in self._vsigs]) if self._sigs else np.zeros((0, T), np.int64)
        # one block: int32 tables, then int64 cache offsets
        parts32 = [ids, row_pos.astype(np.int32), reqs.reshape(-1), tiles.reshape(-1), want_rows, seg_a.reshape(-1), seg_c.reshape(-1),
                   chains.reshape(-1), seg_end] + perms
        n32 = sum(p.size for p in parts32)
        o64 = (n32 * 4 + 7) // 8 * 8
        blob = np.empty(o64 + offs.size * 8 + 8, dtype=np.uint8)
        blob[:n32 * 4].view(np.int32)[:] = np.concatenate(parts32)
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
        T, R, nt, nw = d["T"], d["R"], d["n_tiles"], d["n_want"]
        i32 = dblob[:d["n32"] * 4].view(torch.int32)
        at, out = 0, {}
        ns = d["n_seg"]
        out["n_seg"], out["n_chains"] = ns, d["n_chains"]
        for name, n in [("ids", T), ("pos", T), ("reqs", 4 * R), ("tiles", 4 * nt), ("want", nw), ("seg_a", 4 * ns), ("seg_c", 4 * ns),
                        ("chains", 4 * d["n_chains"]), ("seg_end", ns)] + \
                       [(("perm", H), T * H + H + 1) for H in self._perm_heads]:
            out[name] = i32[at:at + n]
            at += n
        no = len(self._sigs) + len(self._vsigs)
        out["offs"] = dblob[d["o64"]:d["o64"] + no * T * 8].view(torch.int64).view(no, T)
        return out

    def _run(self, arena, dblob, d, logits, num_layers=None, return_streams=False):
        """The device side of a step: every launch of the forward, reading the step's tables from ``dblob``."""
        dev, E, f32 = self.device, self.dtype, torch.float32
        W, T, R = self.W, d["T"], d["R"]
        tb = self._tables(dblob, d)
        layers = self.layers if num_layers is None else self.layers[:num_layers]
        eps = self.config.norm_eps
        x = self._mat("x", T, W, f32)
        h = self._mat("h", T, W, E)
        y1, y2 = self._mat("y1", T, W, f32), self._mat("y2", T, W, f32)
        streams = torch.empty((len(layers), T, W), dtype=f32, device=dev) if return_streams else None
        B.embed_scaled_rows(self.embed, tb["ids"], self.config.embed_scale, x)
        pending = {}                               # the sublayer result that is still to be gated, normed and added to x

        def step(gain, out, **kw):
            nonlocal pending
            B.post_norm(x, gain=gain, out=out, eps=eps, n_rows=kw.pop("n_rows", T), **pending, **kw)
            pending = {}

        for i, lw in enumerate(layers):
            l = lw["cfg"]
            step(lw["norm1"], h)
            gate, ldg = getattr(self, "_" + l.kind)(arena, i, l, lw, h, y1, tb, T, R, d["n_tiles"])
            pending = dict(y=y1, gate=gate, ldg=ldg, post_gain=lw["norm1b"])
            if l.ff:
                step(lw["norm2"], h)
                rg = self._mat("ff_gate", T, W, E)
                B.linear(h, lw["rg2"], rg, M=T, bias=lw["rg2b"], act=B.ACT_SIGMOID)
                mid = self._mat("ff_mid", T, l.ff, E)
                B.linear(h, lw["w_gate"], mid, M=T, epilogue=B.EPI_SILU_MUL, w2=lw["w_up"], bias=lw["b_gate"], bias2=lw["b_up"],
                         act=ACTS[l.act])
                B.linear(mid, lw["w_down"], y2, M=T, bias=lw["b_down"])
                pending = dict(y=y2, gate=rg, ldg=W, post_gain=lw["norm2b"])
            if streams is not None:
                B.post_norm(x, eps=eps, n_rows=T, x_out=streams[i], **pending)
                pending = {}
        if d["n_want"]:
            nw = d["n_want"]
            hn = self._mat("hn", nw, W, E)
            step(self.final_norm, hn, rows=tb["want"], n_rows=nw)
            B.linear(hn, self.head, logits, M=nw)
        return (logits, streams) if return_streams else logits

    # ---- mixers (each leaves its result in y, fp32 [T, W], and returns where the residual gate's sigmoid lies) --------------------
    def _project_in(self, lw, h, T):
        N = lw["w_in"].shape[0]
        P = self._mat("mix_in", T, N, self.dtype)
        B.linear(h, lw["w_in"], P, M=T, bias=lw["b_in"], act_split=lw["act_from"], act2=B.ACT_SIGMOID)
        return P, N

    def _splits(self, arena, n_tiles, heads):
        # few (tile, head) pairs cannot fill the chip: each is cut into runs of its keys (steps of few rows over long caches)
        return 1 if n_tiles * heads >= 512 or arena.cap <= 256 else max(1, min(16, 1024 // (n_tiles * heads), arena.cap // 128))

    def _attention(self, arena, i, l, lw, h, y, tb, T, R, n_tiles):
        E = self.dtype
        H, G, D, Dv = l.heads, l.kv_heads, l.dim, l.vdim
        HD, GD, GV = H * D, G * D, G * Dv
        P, N = self._project_in(lw, h, T)
        plane, vplane = arena.planes[i], arena.col_planes[i]
        q = self._mat("q_rows", T, HD, E)
        vf = self._mat("v_first", T, GV, torch.float32) if l.v_mix else None
        segs = [B.head_seg(P, N, H, D, q, norm=True, gain=lw["q_gain"], rot_dims=l.rot_dims, ld_dst=HD),
                B.head_seg(P[:, HD:], N, G, D, plane, norm=True, gain=lw["k_gain"], rot_dims=l.rot_dims,
                           row_off=tb["offs"][self._sigs.index((G, D))], head_stride=arena.head_stride(i)),
                B.head_seg(P[:, HD + GD:], N, G, Dv, vplane, norm=True, blend=lw["blend"], other=vf if lw["blend"] is not None else None,
                           keep=vf if i == self.first_v_mix else None,
                           row_off=tb["offs"][len(self._sigs) + self._vsigs.index((G, Dv))], head_stride=arena.col_head_stride(i),
                           col_stride=arena.cap)]
        B.head_prep(segs, T, E, pos=tb["pos"], freqs=lw["freqs"], rot_mag=lw["rot_mag"], eps=self.config.norm_eps)
        att = self._mat("mix_out", T, H * Dv, E)
        splits = self._splits(arena, n_tiles, H)
        part = self._scratch("attn_part", B.attn_softmax_part(T, H, splits, Dv), torch.float32) if splits > 1 else None
        B.attn_softmax(q, HD, tb["tiles"], n_tiles, plane, (arena.slot_stride(i), arena.head_stride(i), D), vplane, 0,
                       (arena.col_slot_stride(i), arena.col_head_stride(i), arena.cap), True, H, G, D, Dv, l.scale, att,
                       block=l.mask, sink=lw["sink"], gate=P[:, HD + GD + GV:], ldg=N, gate_per_head=True, n_splits=splits, part=part)
        B.linear(att, lw["wo"], y, M=T)
        return P[:, HD + GD + GV + H:], N

    def _latent_attention(self, arena, i, l, lw, h, y, tb, T, R, n_tiles):
        E = self.dtype
        H, D, Rd, Dv, C = l.heads, l.dim, l.rot_dim, l.vdim, l.kv_rank
        HQ, HV, CR = H * (D + Rd), H * Dv, C + Rd
        P, N = self._project_in(lw, h, T)
        plane = arena.planes[i]
        off = tb["offs"][self._sigs.index((1, CR))]
        qn = self._mat("q_rows", T, H * D, E)                 # the queries' unrotated parts, head by head
        qa = self._mat("q_latent", T, H * CR, E)              # per head [W_uk^T q | rotated part]: a query over the cached rows
        segs = [B.head_seg(P, N, H, D, qn, src_head_stride=D + Rd, ld_dst=H * D),
                B.head_seg(P[:, HQ:], N, 1, C, plane, norm=True, gain=lw["c_gain"], row_off=off)]
        if Rd:
            segs += [B.head_seg(P[:, D:], N, H, Rd, qa, src_head_stride=D + Rd, rot_dims=Rd, ld_dst=H * CR, head_stride=CR, dst_offset=C),
                     B.head_seg(P[:, HQ + C:], N, 1, Rd, plane, rot_dims=Rd, row_off=off, dst_offset=C)]
        B.head_prep(segs, T, E, pos=tb["pos"], freqs=lw["freqs"], rot_mag=lw["rot_mag"], eps=self.config.norm_eps)
        perm = tb[("perm", H)]
        rows, goff = perm[:T * H], perm[T * H:]
        B.linear(qn.view(T * H, D), lw["w_abs"], qa.view(T * H, CR), M=T * H, row_src=rows, row_dst=rows, group_off=goff, n_groups=H,
                 ldy=CR)
        ol = self._mat("mix_out", T, H * C, E)
        one_each = T == R                                    # one token per request: 16 heads share a pass over the slot's rows
        splits = self._splits(arena, n_tiles, -(-H // 16) if one_each else H)
        part = self._scratch("attn_part", B.attn_softmax_part(T, H, splits, C), torch.float32) if splits > 1 else None
        B.attn_softmax(qa, H * CR, tb["tiles"], n_tiles, plane, (arena.slot_stride(i), 0, CR), plane, 0, (arena.slot_stride(i), 0, CR),
                       False, H, 1, CR, C, l.scale, ol, window=l.mask, n_splits=splits, part=part, head_rows=one_each)
        ov = self._mat("mix_o32", T, HV, torch.float32)
        B.linear(ol.view(T * H, C), lw["w_uv"], ov.view(T * H, Dv), M=T * H, row_src=rows, row_dst=rows, group_off=goff, n_groups=H)
        og = self._mat("mix_gated", T, HV, E)
        B.gated_norm(ov, None, P[:, HQ + CR:], N, og, self.config.norm_eps, T)
        B.linear(og, lw["wo"], y, M=T)
        return P[:, HQ + CR + HV:], N

    def _mlstm(self, arena, i, l, lw, h, y, tb, T, R, n_tiles):
        H, D, Dv = l.heads, l.dim, l.vdim
        HD, HV = H * D, H * Dv
        P, N = self._project_in(lw, h, T)
        o = self._mat("mix_o32", T, HV, torch.float32)
        cols = (P, P[:, HD:], P[:, 2 * HD:], P[:, 2 * HD + HV:], P[:, 2 * HD + HV + H:], N)
        state, ns = arena.states[i][0], tb["n_seg"]
        if ns:
            # every segment from nothing (only the states move), the segments chained, then every segment from its start state
            rec = B.mlstm_state_floats(H, D, Dv)
            local, start = self._mat("seg_local", ns, rec, torch.float32), self._mat("seg_start", ns, rec, torch.float32)
            fsum = self._mat("seg_logf", ns, H, torch.float32)
            B.mlstm(*cols, tb["seg_a"], ns, local, H, D, Dv, D ** -0.5, l.gate_cap, None, from_nothing=True, log_f_sum=fsum)
            B.mlstm_chain(local, fsum, start, state, tb["chains"], tb["n_chains"], H, D, Dv)
            B.mlstm(*cols, tb["seg_c"], ns, start, H, D, Dv, D ** -0.5, l.gate_cap, o, end_slots=tb["seg_end"], end_state=state)
        else:
            B.mlstm(*cols, tb["reqs"], R, state, H, D, Dv, D ** -0.5, l.gate_cap, o)
        on = self._mat("mix_gated", T, HV, self.dtype)
        B.gated_norm(o, lw["gain"], P[:, 2 * HD + HV + 2 * H:], N, on, self.config.norm_eps, T, group=Dv)
        B.linear(on, lw["wo"], y, M=T)
        return P[:, 2 * HD + 2 * HV + 2 * H:], N
