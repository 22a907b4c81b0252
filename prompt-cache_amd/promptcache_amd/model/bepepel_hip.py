"""Bepepel forward pass on MI355X (``config.BepepelShape`` says what the design is).

Like ``dibizen_hip.DibizenHIP`` and ``fivesun_hip.FivesunHIP`` this model keeps plain row-major tensors in one element type E --
bfloat16 (serving: matrix products on the bf16 matrix cores, fp32 accumulation) or float32 (everything in true 32-bit) -- runs on
the building blocks of ``libpromptcache_blocks.so`` (``_blocks.py``) and steps over FLAT rows: the new tokens of all requests of a
step one after another, each request continuing from what its slot of the ``SlotArena`` holds.  Nothing is padded, and a row
reads nothing but its own slot, so a request's numbers do not depend on the rest of the step.

What a slot holds differs by layer: a gla layer one fp32 matrix per head; a parallel layer keys (row by row) and values (column by
column) of its attention half, the fp32 matrix state of its state-space half, and the last inputs of both halves' short
convolutions.

With the residual x in fp32, m = ``residual_mult`` and ln(.) a layer norm with weight and bias, sublayer by sublayer:

    h = ln(x);  y = f(h) (fp32 rows);  x <- x + m y          (pcb_post_norm: one launch adds a finished y and norms for the next f)

    gla         q | k | v | a | g of ONE projection (SiLU on g's columns); log decay = logsigmoid(W_a2 a + b) / tau, fp32, in the second
                projection's epilogue; per head S <- diag(decay) S + k v^T, o = S^T q / sqrt(dim) (pcb_gla); y = Wo (rms(o) gain * g)
    parallel    left:  q | k | v of ONE projection with biases -> causal convolution (pcb_causal_conv) -> per head unit RMS and rotary
                       pairs; k rows and v columns land in the slot's cache (pcb_head_prep); softmax over a sliding window that keeps
                       the first positions (pcb_attn_softmax); y = Wo (.)
                right: z | x | B | C of ONE projection (SiLU on z), dt = softplus(W_dt h + b) in fp32; x | B | C through a causal
                       convolution and SiLU; per head S <- exp(-e^A_log dt) S + dt B x^T, y = S^T C (pcb_gla with one decay per head);
                       rms_parts((y + D x) silu(z)) gain (pcb_gated_norm, the gate first); y += right_scale / left_scale * Wo (.),
                       and the residual step multiplies y by left_scale
    dense       Wdown (gelu_tanh(Wgate h) * Wup h), the product in the first projection's epilogue
    experts     router logits (fp32, with bias) -> the top logits and the softmax over them (pcb_router_select); pairs bucketed by
                expert (pcb_moe_plan); silu(Wgate h) * Wup h and Wdown per bucket (grouped pcb_linear); y = sum_k w_k (expert result)
                (pcb_moe_mix); the shared expert's result is added in its down projection's epilogue

and the logits are ``logit_scale * head . ln(x)`` for the rows that were asked for.
"""
from __future__ import annotations

import math
import os
from typing import Dict, Optional, Sequence

import numpy as np
import torch

from .. import _blocks as B
from .config import BepepelShape
from .kv_arena import SlotArena
from .slot_model import SlotKV, SlotModel  # noqa: F401


def scaled_rotary_frequencies(base: float, dims: int, scaling=None) -> np.ndarray:
    """float64 frequencies of the ``dims / 2`` rotated column pairs: base^(-2i/dims), and with ``scaling`` = (factor, low, high,
    original) the wavelength-dependent form: a pair whose wavelength 2 pi / f is shorter than original / high keeps f, one longer
    than original / low turns at f / factor, and between the two f / factor and f are blended linearly in original / wavelength."""
    f = np.asarray([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=np.float64)
    if not scaling:
        return f
    factor, low, high, original = scaling
    wl = 2.0 * math.pi / f
    s = np.clip((original / wl - low) / (high - low), 0.0, 1.0) if high != low else np.ones_like(f)
    mid = (1.0 - s) * f / factor + s * f
    return np.where(wl < original / high, f, np.where(wl > original / low, f / factor, mid))


class BepepelHIP(SlotModel):
    GRAPH_MAX_ROWS = 64
    SEGMENT = int(os.environ.get("PC_BP_SEGMENT", "64"))    # a step that brings a request more tokens than this runs its recurrences segment-parallel
    MAX_SEGMENTS = 128      # (segments grow beyond SEGMENT tokens rather than exceed this many per request)

    def __init__(self, shape: BepepelShape, weights: Dict[str, torch.Tensor], device="cuda:0", dtype=torch.bfloat16,
                 decode_headroom: int = 256):
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Bepepel runs in bfloat16 or float32")
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

        def e(name):                               # element-type tensor (projections, their biases, convolution taps)
            return weights[name].to(device=dev, dtype=dtype).contiguous()

        def f(name):                               # fp32 tensor (norms, decay rates, skip weights)
            return weights[name].to(device=dev, dtype=torch.float32).contiguous()

        def const(n, v):
            return torch.full((n,), float(v), dtype=torch.float32, device=dev)

        def unit(pre):
            return dict(gate=e(pre + "gate"), up=e(pre + "up"), down=e(pre + "down"))

        self.embed, self.head = e("embed"), e("head")
        self.final_norm = (f("final.norm"), f("final.norm.b"))
        self.ones_w = const(W, 1.0)
        self.layers = []
        for i, l in enumerate(shape.layers):
            p, m = f"l{i}.", f"l{i}.mix."
            ent = dict(cfg=l, norm1=(f(p + "norm1"), f(p + "norm1.b")))
            if l.kind == "gla":
                if l.dim > 256:
                    raise ValueError(f"layer {i}: gla heads take up to 256 key columns (got {l.dim})")
                a1 = e(m + "a1")
                if l.a_rank and a1.shape[0] != l.a_rank:
                    raise ValueError(f"layer {i}: the decay projection has rank {a1.shape[0]}, the configuration says {l.a_rank}")
                ent.update(w_in=torch.cat([e(m + "q"), e(m + "k"), e(m + "v"), a1, e(m + "g")], dim=0).contiguous(), rank=a1.shape[0],
                           a2=e(m + "a2"), a2b=e(m + "a2.b"), gain=f(m + "norm").repeat(l.heads).contiguous(), wo=e(m + "o"),
                           chain_coef=const(l.heads * l.dim * l.vdim, 1.0))
            else:
                a, b = l.left, l.right
                if a.dim > 384 or a.vdim > 256:
                    raise ValueError(f"layer {i}: attention heads take up to 384 key and 256 value columns (got {a.dim} / {a.vdim})")
                if b.state > 256 or max(a.conv, b.conv) > 16:
                    raise ValueError(f"layer {i}: up to 256 states per head and 16 taps (got {b.state}, {a.conv}, {b.conv})")
                lp, rp = m + "left.", m + "right."
                w_in = e(rp + "in")
                nm = b.in_columns - b.heads                 # z | x | B | C; the step sizes' rows are a projection of their own
                ent.update(
                    l_in=torch.cat([e(lp + "q"), e(lp + "k"), e(lp + "v")], dim=0).contiguous(),
                    l_in_b=torch.cat([e(lp + "q.b"), e(lp + "k.b"), e(lp + "v.b")]).contiguous(),
                    l_conv=torch.cat([e(lp + "q.conv"), e(lp + "k.conv"), e(lp + "v.conv")], dim=0).contiguous() if a.conv else None,
                    l_wo=e(lp + "o"), l_scale=float(l.left_scale),
                    freqs=torch.from_numpy(scaled_rotary_frequencies(a.rot_base, a.rot_dims, a.rot_scaling)).to(dev) if a.rot_dims else None,
                    r_in=w_in[:nm].contiguous(), r_dt=w_in[nm:].contiguous(), r_dt_b=e(rp + "dt_bias"),
                    r_conv=e(rp + "conv") if b.conv else None, r_conv_b=e(rp + "conv.b") if b.conv else None,
                    r_rate=(-torch.exp(f(rp + "A_log"))).contiguous(), r_D=f(rp + "D"), r_gain=f(rp + "norm"), r_wo=e(rp + "o"),
                    r_scale=const(W, l.right_scale / l.left_scale if l.left_scale != 0.0 else l.right_scale), chain_coef=const(b.heads * b.state * b.vdim, 1.0))
            if l.ff_kind:
                q = p + "mlp."
                ent.update(norm2=(f(p + "norm2"), f(p + "norm2.b")))
                if l.ff_kind == "dense":
                    ent.update(ff=unit(q))
                else:
                    if l.experts > 2048 or l.top > 64:
                        raise ValueError(f"layer {i}: up to 2048 experts, top <= 64")
                    us = [unit(q + f"e{j}.") for j in range(l.experts)]
                    ent.update(router=e(q + "router"), router_b=e(q + "router.b"),
                               e_gate=torch.stack([u["gate"] for u in us]).contiguous(), e_up=torch.stack([u["up"] for u in us]).contiguous(),
                               e_down=torch.stack([u["down"] for u in us]).contiguous(), shared=unit(q + "shared.") if l.shared_ff else None)
            self.layers.append(ent)
        self._buf = {}
        self.default_arena: Optional[SlotArena] = None
        self.use_graphs = os.environ.get("PC_BP_GRAPHS", "1") != "0"      # one-token steps replay a captured hipGraph
        self._graphs = {}
        self.max_graphs = 16
        # cache offsets of a row, one table per distinct (heads, columns) of the key planes and of the value planes
        att = [l.left for l in shape.layers if l.kind == "parallel"]
        self._sigs = sorted({(a.kv_heads, a.dim) for a in att})
        self._vsigs = sorted({(a.kv_heads, a.vdim) for a in att})
        self._recurrent = True                     # every layer of this design carries a matrix state

    # ---- cache and state -------------------------------------------------------------------------------------------------------
    def new_arena(self, slots: int, cap: int) -> SlotArena:
        dims, cols, states = [], [], []
        f32 = torch.float32
        for l in self.config.layers:
            if l.kind == "gla":
                dims.append((0, 0)); cols.append((0, 0))
                states.append([((l.heads, l.dim, l.vdim), f32)])
            else:
                a, b = l.left, l.right
                dims.append((a.kv_heads, a.dim)); cols.append((a.kv_heads, a.vdim))
                # the matrix state, then the last inputs of the right and of the left convolution (a single tap keeps nothing)
                st = [((b.heads, b.state, b.vdim), f32)]
                if b.conv > 1:
                    st.append(((b.conv - 1, b.conv_channels), self.dtype))
                if a.conv > 1:
                    st.append(((a.conv - 1, (a.heads + a.kv_heads) * a.dim + a.kv_heads * a.vdim), self.dtype))
                states.append(st)
        return SlotArena(dims, slots, cap, self.device, self.dtype, states=states, col_dims=cols)

    def _no_state(self, channels: int) -> torch.Tensor:
        """What a convolution of a single tap keeps between steps: nothing, in the shape the kernel's binding checks."""
        key = ("no_state", channels)
        if key not in self._buf:
            self._buf[key] = torch.empty((1, 0, channels), dtype=self.dtype, device=self.device)
        return self._buf[key]

    def kv_bytes_per_token(self) -> int:
        es = 2 if self.dtype == torch.bfloat16 else 4
        return sum(l.left.kv_heads * (l.left.dim + l.left.vdim) for l in self.config.layers if l.kind == "parallel") * es

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
        # segments of the recurrences' prefill (only when some request brings more than SEGMENT tokens)
        seg_a = seg_c = chains = np.zeros((0, 4), np.int32)
        if max(counts) > self.SEGMENT:
            seg = max(self.SEGMENT, -(-max(counts) // self.MAX_SEGMENTS))
            sa, ch = [], []
            for b, (s, st, c) in enumerate(zip(slots, starts, counts)):
                ch.append((s, st, len(sa), -(-c // seg)))
                sa += [(len(sa) + k, 0, min(seg, c - q), int(row0[b]) + q) for k, q in enumerate(range(0, c, seg))]
            seg_a = np.asarray(sa, dtype=np.int32)
            seg_c = seg_a.copy()
            seg_c[:, 1] = 1                                 # the second pass starts every segment from a state that was put there
            chains = np.asarray(ch, dtype=np.int32)
        offs = np.stack([row_slot * (g * arena.cap * d) + row_pos * d for g, d in self._sigs] +
                        [row_slot * (g * d * arena.cap) + row_pos for g, d in self._vsigs]) if self._sigs else np.zeros((0, T), np.int64)
        # one block: int32 tables, then int64 cache offsets
        parts32 = [ids, row_pos.astype(np.int32), meta.reshape(-1), reqs.reshape(-1), tiles.reshape(-1), want_rows, seg_a.reshape(-1),
                   seg_c.reshape(-1), chains.reshape(-1)]
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
        T, R, nt, nw, ns = d["T"], d["R"], d["n_tiles"], d["n_want"], d["n_seg"]
        i32 = dblob[:d["n32"] * 4].view(torch.int32)
        at, out = 0, {"n_seg": ns, "n_chains": d["n_chains"]}
        for name, n in (("ids", T), ("pos", T), ("meta", 4 * T), ("reqs", 4 * R), ("tiles", 4 * nt), ("want", nw), ("seg_a", 4 * ns),
                        ("seg_c", 4 * ns), ("chains", 4 * d["n_chains"])):
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
        eps, mult = self.config.norm_eps, self.config.residual_mult
        x = self._mat("x", T, W, f32)
        h = self._mat("h", T, W, E)
        y1, y2 = self._mat("y1", T, W, f32), self._mat("y2", T, W, f32)
        streams = torch.empty((len(layers), T, W), dtype=f32, device=dev) if return_streams else None
        B.embed_rows(self.embed, tb["ids"], x)
        pending = {}                               # the sublayer result that is still to be added to x

        def step(norm, out, **kw):
            nonlocal pending
            B.post_norm(x, gain=norm[0], bias=norm[1], layer_norm=True, out=out, eps=eps, n_rows=kw.pop("n_rows", T),
                        **{"y_scale": mult, **pending}, **kw)
            pending = {}

        for i, lw in enumerate(layers):
            l = lw["cfg"]
            step(lw["norm1"], h)
            if l.kind == "gla":
                self._gla(arena, i, l, lw, h, y1, tb, T, R)
                pending = dict(y=y1)
            else:
                pending = dict(y=y1, y_scale=mult * self._parallel(arena, i, l, lw, h, y1, tb, T, R, d["n_tiles"]))
            if l.ff_kind:
                step(lw["norm2"], h)
                if l.ff_kind == "dense":
                    self._unit(lw["ff"], h, y2, T, B.ACT_GELU_TANH)
                else:
                    self._experts(l, lw, h, y2, T)
                pending = dict(y=y2)
            if streams is not None:
                B.post_norm(x, eps=eps, n_rows=T, x_out=streams[i], **{"y_scale": mult, **pending})
                pending = {}
        if d["n_want"]:
            nw = d["n_want"]
            hn = self._mat("hn", nw, W, E)
            step(self.final_norm, hn, rows=tb["want"], n_rows=nw)
            B.linear(hn, self.head, logits, M=nw, act=B.ACT_SCALE, act_param=self.config.logit_scale)
        return (logits, streams) if return_streams else logits

    # ---- the matrix-state recurrence, whole or in segments -------------------------------------------------------------------------
    def _recurrence(self, state, coef, tb, R, q, k, v, ld, lds_, dcols, H, Hk, D, Dv, q_scale, o, **kw):
        ns = tb["n_seg"]
        if not ns:
            B.gla(q, k, v, ld, lds_, dcols, tb["reqs"], R, state, H, Hk, D, Dv, q_scale, o, **kw)
            return
        # every segment from a zero state (only the states move), the segments chained, then every segment from its start state
        elems = H * D * Dv
        local = self._scratch("seg_local", ns * elems, torch.float32)[:ns * elems].view(ns, H, D, Dv)
        start = self._scratch("seg_start", ns * elems, torch.float32)[:ns * elems].view(ns, H, D, Dv)
        lsum = self._mat("seg_ld", ns, H * dcols, torch.float32)
        B.gla(q, k, v, ld, lds_, dcols, tb["seg_a"], ns, local, H, Hk, D, Dv, q_scale, None, ld_sum=lsum, **kw)
        B.state_chain(local.view(ns, elems), start.view(ns, elems), state, tb["chains"], tb["n_chains"], coef, lsum,
                      Dv if dcols > 1 else D * Dv)
        B.gla(q, k, v, ld, lds_, dcols, tb["seg_c"], ns, start, H, Hk, D, Dv, q_scale, o, **kw)

    # ---- mixers (each leaves its result in y, fp32 [T, W]) ---------------------------------------------------------------------------
    def _gla(self, arena, i, l, lw, h, y, tb, T, R):
        E, f32 = self.dtype, torch.float32
        H, D, Dv, r = l.heads, l.dim, l.vdim, lw["rank"]
        HD, HV = H * D, H * Dv
        N = 2 * HD + HV + r + HV
        P = self._mat("mix_in", T, N, E)
        B.linear(h, lw["w_in"], P, M=T, act_split=2 * HD + HV + r, act2=B.ACT_SILU)
        ld = self._mat("mix_ld", T, HD, f32)
        B.linear(P[:, 2 * HD + HV:], lw["a2"], ld, M=T, bias=lw["a2b"], act=B.ACT_LOGSIGMOID, act_param=1.0 / l.tau, ldx=N)
        o = self._mat("mix_o32", T, HV, f32)
        self._recurrence(arena.states[i][0], lw["chain_coef"], tb, R, P, P[:, HD:], P[:, 2 * HD:], ld, (N, N, N, HD), D, H, H, D, Dv,
                         D ** -0.5, o)
        on = self._mat("mix_out", T, HV, E)
        B.gated_norm(o, lw["gain"], P[:, 2 * HD + HV + r:], N, on, self.config.norm_eps, T, group=Dv)
        B.linear(on, lw["wo"], y, M=T)

    def _splits(self, arena, n_tiles, heads):
        # few (tile, head) pairs cannot fill the chip: each is cut into runs of its keys (steps of few rows over long caches)
        return 1 if n_tiles * heads >= 512 or arena.cap <= 256 else max(1, min(16, 1024 // (n_tiles * heads), arena.cap // 128))

    def _parallel(self, arena, i, l, lw, h, y, tb, T, R, n_tiles):
        """Leaves left + (right_scale / left_scale) right in y and returns left_scale, the factor that is still to come (the
        residual step multiplies by it together with the residual factor): the plain store of the left projection is the faster
        epilogue.  A left_scale of 0 is applied in the projection itself."""
        E, f32, eps = self.dtype, torch.float32, self.config.norm_eps
        a, b = l.left, l.right
        states = list(arena.states[i])
        ssd_state = states.pop(0)
        r_conv_state = states.pop(0) if b.conv > 1 else None
        l_conv_state = states.pop(0) if a.conv > 1 else None
        # ---- left: softmax attention behind a short convolution
        H, G, D, Dv = a.heads, a.kv_heads, a.dim, a.vdim
        HD, GD, GV = H * D, G * D, G * Dv
        NL = HD + GD + GV
        P = self._mat("mix_in", T, NL, E)
        B.linear(h, lw["l_in"], P, M=T, bias=lw["l_in_b"])
        if a.conv:
            Pc = self._mat("mix_conv", T, NL, E)
            st = l_conv_state if l_conv_state is not None else self._no_state(NL)
            B.causal_conv(P, NL, lw["l_conv"], None, False, tb["meta"], st, Pc, T)
            if l_conv_state is not None:
                B.conv_state_update(P, NL, tb["reqs"], R, l_conv_state)
            P = Pc
        plane, vplane = arena.planes[i], arena.col_planes[i]
        q = self._mat("q_rows", T, HD, E)
        # (a rotation leaves a head's mean square as it is, so the unit-RMS step commutes with it: the kernel norms, then turns)
        segs = [B.head_seg(P, NL, H, D, q, norm=True, rot_dims=a.rot_dims, ld_dst=HD),
                B.head_seg(P[:, HD:], NL, G, D, plane, norm=True, rot_dims=a.rot_dims, row_off=tb["offs"][self._sigs.index((G, D))],
                           head_stride=arena.head_stride(i)),
                B.head_seg(P[:, HD + GD:], NL, G, Dv, vplane, row_off=tb["offs"][len(self._sigs) + self._vsigs.index((G, Dv))],
                           head_stride=arena.col_head_stride(i), col_stride=arena.cap)]
        B.head_prep(segs, T, E, pos=tb["pos"], freqs=lw["freqs"], eps=eps)
        att = self._mat("mix_out", T, H * Dv, E)
        splits = self._splits(arena, n_tiles, H)
        part = self._scratch("attn_part", B.attn_softmax_part(T, H, splits, Dv), f32) if splits > 1 else None
        B.attn_softmax(q, HD, tb["tiles"], n_tiles, plane, (arena.slot_stride(i), arena.head_stride(i), D), vplane, 0,
                       (arena.col_slot_stride(i), arena.col_head_stride(i), arena.cap), True, H, G, D, Dv, a.scale, att,
                       window=a.window, keep_first=a.keep_first, n_splits=splits, part=part)
        if lw["l_scale"] != 0.0:
            B.linear(att, lw["l_wo"], y, M=T)
        else:
            B.linear(att, lw["l_wo"], y, M=T, act=B.ACT_SCALE, act_param=0.0)
        # ---- right: the state-space half
        Hs, Pv, N, Gs = b.heads, b.vdim, b.state, b.groups
        inner, CC = b.inner, b.conv_channels
        NR = inner + CC
        Z = self._mat("ssd_in", T, NR, E)
        # z takes its SiLU here; without a convolution x | B | C take theirs here as well
        B.linear(h, lw["r_in"], Z, M=T, act=B.ACT_SILU, act_split=0 if not b.conv else inner, act2=B.ACT_NONE)
        dt = self._mat("ssd_dt", T, Hs, f32)
        B.linear(h, lw["r_dt"], dt, M=T, bias=lw["r_dt_b"], act=B.ACT_SOFTPLUS)
        if b.conv:
            xbc = self._mat("ssd_xbc", T, CC, E)
            st = r_conv_state if r_conv_state is not None else self._no_state(CC)
            B.causal_conv(Z[:, inner:], NR, lw["r_conv"], lw["r_conv_b"], True, tb["meta"], st, xbc, T)
            if r_conv_state is not None:
                B.conv_state_update(Z[:, inner:], NR, tb["reqs"], R, r_conv_state)
            ldx = CC
        else:
            xbc, ldx = Z[:, inner:], NR
        ys = self._mat("ssd_y32", T, inner, f32)
        self._recurrence(ssd_state, lw["chain_coef"], tb, R, xbc[:, inner + Gs * N:], xbc[:, inner:], xbc, dt, (ldx, ldx, ldx, Hs), 1,
                         Hs, Gs, N, Pv, 1.0, ys, ld_coef=lw["r_rate"], v_scale=dt, ldvs=Hs)
        yn = self._mat("ssd_out", T, inner, E)
        B.gated_norm(ys, lw["r_gain"], Z, NR, yn, eps, T, group=inner // b.norm_groups, gate_first=True, skip=xbc, lds=ldx,
                     skip_w=lw["r_D"], skip_group=Pv)
        B.linear(yn, lw["r_wo"], y, M=T, epilogue=B.EPI_SCALE_ADD, col_scale=lw["r_scale"])
        return lw["l_scale"] if lw["l_scale"] != 0.0 else 1.0

    # ---- feed-forwards -----------------------------------------------------------------------------------------------------------------
    def _unit(self, u, h, y, T, act, add=False):
        mid = self._mat("ff_mid", T, u["gate"].shape[0], self.dtype)
        B.linear(h, u["gate"], mid, M=T, epilogue=B.EPI_SILU_MUL, w2=u["up"], act=act)
        if add:
            B.linear(mid, u["down"], y, M=T, epilogue=B.EPI_SCALE_ADD, col_scale=self.ones_w)
        else:
            B.linear(mid, u["down"], y, M=T)

    def _experts(self, l, lw, h, y, T):
        n_out, P, W = l.experts, T * l.top, self.W
        ex = self._scratch("moe_i", 3 * P + n_out + 1, torch.int32)
        sc = self._scratch("moe_f", 2 * P, torch.float32)
        expert, row_src, row_dst, goff = ex[:P], ex[P:2 * P], ex[2 * P:3 * P], ex[3 * P:3 * P + n_out + 1]
        weight, row_scale = sc[:P], sc[P:2 * P]
        rl = self._mat("router", T, n_out, torch.float32)
        B.linear(h, lw["router"], rl, M=T, bias=lw["router_b"])     # fp32 accumulation of exact products: 32-bit logits
        # the softmax over all logits, renormalised over the chosen ones, IS the softmax over the chosen logits alone
        B.router_select(rl, l.top, expert, weight, T, score_fn=B.SCORE_SOFTMAX, renorm=True)
        pair = self._mat("pair", P, W, torch.float32)
        B.moe_plan(expert, weight, P, l.top, n_out, goff, row_src, row_dst, row_scale)
        act = self._mat("moe_act", P, l.expert_ff, self.dtype)
        B.linear(h, lw["e_gate"], act, M=P, epilogue=B.EPI_SILU_MUL, w2=lw["e_up"], act=B.ACT_SILU, row_src=row_src, group_off=goff,
                 n_groups=n_out)
        B.linear(act, lw["e_down"], pair, M=P, row_dst=row_dst, group_off=goff, n_groups=n_out)
        B.moe_mix(pair, expert, weight, h, n_out, y, T, l.top)
        if lw["shared"] is not None:
            self._unit(lw["shared"], h, y, T, B.ACT_SILU, add=True)
