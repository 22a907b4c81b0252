"""Bepepel on the GPU against the plain float64 oracle (``oracle/bepepel_oracle.py``): every new or extended building-block kernel
alone -- with inputs built so that a window's edge, a kept first key or a far key decides the result --, then the model through its
arena: prompts, token-by-token decoding, portions down to two tokens, unequal batches, reused slots and states, long decoding
through captured graphs, and greedy generation through the batch engine and the trace runner.  float32 runs are held to float32
accuracy; bfloat16 runs to what bf16 operands allow."""
import json
import os
import subprocess

import pytest
import torch

from oracle import bepepel_oracle as O
from promptcache_amd.model import weights as W
from promptcache_amd.model.config import BepepelAttention, BepepelLayer, BepepelSSD, BepepelShape

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEV = "cuda:0"
F64 = torch.float64
DTYPES = [torch.float32, torch.bfloat16]


def rel(got, want):
    got, want = got.detach().to("cpu", F64), want.detach().to("cpu", F64)
    return float((got - want).pow(2).mean().sqrt() / want.pow(2).mean().sqrt().clamp_min(1e-30))


def tol(dtype, f32=2e-5, bf16=2e-2):
    return f32 if dtype == torch.float32 else bf16


def close(got, want, dtype, f32=3e-5, bf16=3e-2):
    """Logits row by row.  float32: every row within float32 accuracy.  bfloat16: where two router logits of the float64 oracle lie
    closer than bf16 operands resolve, a token may take another expert than the oracle's and leave a trace in the states behind it,
    so rows are judged together: the median row within ``bf16``, at most one row in ten (or one) beyond three times that."""
    got, want = got.detach().to("cpu", F64), want.detach().to("cpu", F64)
    err = (got - want).pow(2).mean(dim=-1).sqrt() / want.pow(2).mean(dim=-1).sqrt().clamp_min(1e-30)
    if dtype == torch.float32:
        return bool(err.max() < f32)
    return bool(err.median() <= bf16) and int((err > 3 * bf16).sum()) <= max(1, err.numel() // 10)


def B():
    from promptcache_amd import _blocks
    return _blocks


def rnd(*shape, dtype=torch.float32, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (scale * torch.randn(*shape, generator=g)).to(dtype).to(DEV)


def f64(t):
    return t.detach().to("cpu", F64)


def dev_i32(rows):
    return torch.tensor(rows, dtype=torch.int32, device=DEV).reshape(-1)


def gla(heads, dim, vdim, tau=6.0, rank=5, **ff):
    return BepepelLayer("gla", heads=heads, dim=dim, vdim=vdim, tau=tau, a_rank=rank, **ff)


def par(H, G, D, Dv, window, keep, sh, sp, sn, sg=1, parts=1, convl=3, convr=4, rot=None, scaling=(4.0, 1.0, 4.0, 64.0), scale=None,
        ls=1.25, rs=0.8, base=5000.0, **ff):
    left = BepepelAttention(heads=H, kv_heads=G, dim=D, vdim=Dv, scale=scale or 2.0 * D ** -0.5, conv=convl, window=window, keep_first=keep,
                            rot_base=base, rot_dims=D if rot is None else rot, rot_scaling=scaling)
    right = BepepelSSD(heads=sh, vdim=sp, state=sn, groups=sg, norm_groups=parts, conv=convr)
    return BepepelLayer("parallel", left=left, right=right, left_scale=ls, right_scale=rs, **ff)


MOE = dict(ff_kind="moe", experts=6, top=2, expert_ff=24, shared_ff=20)
DENSE = dict(ff_kind="dense", ff=56)


# ---- shapes: layers differ from one another, come in different orders, and no size is a round one -------------------------------
def shape_mixed():
    return BepepelShape(vocab_size=150, hidden_size=96, norm_eps=1e-5, residual_mult=0.4, logit_scale=1.5, layers=[
        par(6, 3, 24, 40, 21, 3, 5, 24, 20, sg=1, parts=3, rot=16, **MOE),
        gla(3, 20, 24, tau=4.0, **DENSE),
        gla(2, 40, 16, tau=12.0, rank=7, **MOE),
        par(4, 2, 40, 24, 33, 0, 6, 16, 12, sg=3, parts=1, convl=2, convr=2, scaling=None, **DENSE),
        par(2, 2, 16, 24, 0, 0, 4, 8, 40, sg=2, parts=2, rot=0),
    ])


def shape_odd():
    """Sizes that are no multiple of a 16-byte chunk in either element type; one head, one expert of which one is used, a window of
    one position, more kept tokens than the window is long, single-tap and absent convolutions, tau 1, factors of 1."""
    return BepepelShape(vocab_size=75, hidden_size=50, norm_eps=1e-6, residual_mult=1.0, logit_scale=1.0, layers=[
        gla(1, 6, 10, tau=1.0, rank=1, ff_kind="moe", experts=1, top=1, expert_ff=14, shared_ff=0),
        par(3, 3, 10, 6, 1, 0, 1, 10, 7, convl=1, convr=1, rot=6, scaling=None, ls=1.0, rs=1.0),
        par(1, 1, 6, 10, 3, 5, 3, 5, 1, sg=3, parts=3, convl=0, convr=0, rot=0, ff_kind="moe", experts=3, top=3, expert_ff=10, shared_ff=6),
        gla(2, 7, 5, tau=30.0, rank=3, ff_kind="dense", ff=10),
    ])


def shape_wide():
    """Enough heads and columns to reach the wider kernel instantiations; windows longer than a key block, many kept tokens."""
    return BepepelShape(vocab_size=320, hidden_size=128, norm_eps=1e-6, residual_mult=0.35, logit_scale=2.5, layers=[
        gla(2, 200, 136, tau=16.0, rank=16, **DENSE),
        par(8, 2, 128, 72, 64, 40, 4, 64, 128, sg=2, parts=2, rot=64, **MOE),
        gla(4, 64, 64, tau=8.0, rank=8),
        par(4, 4, 272, 72, 100, 4, 10, 40, 100, sg=5, parts=5, convl=4, convr=3, rot=32, scaling=(6.0, 1.0, 4.0, 400.0), **DENSE),
    ])


SHAPES = {"mixed": shape_mixed, "odd": shape_odd, "wide": shape_wide}
_models = {}


def model(name, dtype, seed=11):
    from promptcache_amd.model.bepepel_hip import BepepelHIP
    key = (name, dtype, seed)
    if key not in _models:
        s = SHAPES[name]()
        w = W.make_bepepel_weights(s, seed=seed)
        _models[key] = (s, w, BepepelHIP(s, w, device=DEV, dtype=dtype))
    return _models[key]


def toks(n, vocab, seed=0):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def run_alone(m, tokens, cuts=None):
    """One request on a fresh arena, its tokens cut into the given portions; logits of every token."""
    ar = m.new_arena(1, 8)
    s = ar.alloc()
    cuts = cuts or [len(tokens)]
    assert sum(cuts) == len(tokens)
    out, at = [], 0
    for c in cuts:
        out.append(m.forward_rows(ar, [s], [tokens[at:at + c]], [list(range(c))]))
        at += c
    return torch.cat(out)


_oracle = {}


def oracle_logits(s, w, tokens, key=None):
    if key is not None and key in _oracle:
        return _oracle[key]
    out = O.forward(s, O.to_f64(w), tokens, return_streams=True)
    if key is not None:
        _oracle[key] = out
    return out


# =====================================================================================================================================
# building blocks alone
# =====================================================================================================================================
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("W_", [50, 192, 2048])
def test_layer_norm_and_the_residual_factor(dtype, W_):
    T = 9
    x0, y = rnd(T, W_, seed=1, scale=3.0) + 2.0, rnd(T, W_, seed=2)
    gain, bias = rnd(W_, seed=3) + 1.0, rnd(W_, seed=4)
    x, out = x0.clone(), torch.empty(T, W_, dtype=dtype, device=DEV)
    B().post_norm(x, y=y, gain=gain, bias=bias, layer_norm=True, out=out, eps=1e-5, y_scale=0.3)
    xs = f64(x0) + 0.3 * f64(y)
    assert rel(x, xs) < 1e-6 and rel(out, O.layer_norm(xs, f64(gain), f64(bias), 1e-5)) < tol(dtype, 1e-5, 4e-3)
    rows = dev_i32([7, 0, 7])                                # chosen rows: normed, not written back
    x, out = x0.clone(), torch.empty(3, W_, dtype=dtype, device=DEV)
    B().post_norm(x, y=y, gain=gain, bias=bias, layer_norm=True, out=out, eps=1e-5, y_scale=-2.0, rows=rows, n_rows=3)
    assert torch.equal(x, x0)
    assert rel(out, O.layer_norm((f64(x0) - 2.0 * f64(y))[[7, 0, 7]], f64(gain), f64(bias), 1e-5)) < tol(dtype, 1e-5, 4e-3)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("cols,group,sg", [(48, 16, 6), (60, 60, 10), (384, 192, 48), (10, 5, 1)])
def test_gate_before_the_norm_with_a_skip_path(dtype, cols, group, sg):
    T = 7
    x, gate, skip = rnd(T, cols, seed=1), rnd(T, cols + 9, dtype=dtype, seed=2), rnd(T, cols + 4, dtype=dtype, seed=3)
    gain, sw = rnd(cols, seed=4) + 1.0, rnd(cols // sg, seed=5)
    out = torch.empty(T, cols, dtype=dtype, device=DEV)
    B().gated_norm(x, gain, gate[:, 9:], cols + 9, out, 1e-6, T, group=group, gate_first=True, skip=skip[:, 4:], lds=cols + 4, skip_w=sw,
                   skip_group=sg)
    v = (f64(x) + f64(sw).repeat_interleave(sg) * f64(skip[:, 4:])) * f64(gate[:, 9:])
    want = O.unit_rms(v.view(T, cols // group, group), 1e-6).reshape(T, cols) * f64(gain)
    assert rel(out, want) < tol(dtype, 1e-5, 4e-3)
    # the old order (norm, then gate) still holds, also with a skip path
    B().gated_norm(x, gain, gate[:, 9:], cols + 9, out, 1e-6, T, group=group, skip=skip[:, 4:], lds=cols + 4, skip_w=sw, skip_group=sg)
    v = f64(x) + f64(sw).repeat_interleave(sg) * f64(skip[:, 4:])
    want = O.unit_rms(v.view(T, cols // group, group), 1e-6).reshape(T, cols) * f64(gain) * f64(gate[:, 9:])
    assert rel(out, want) < tol(dtype, 1e-5, 4e-3)


@pytest.mark.parametrize("dtype", DTYPES)
def test_log_decay_and_scaled_epilogues(dtype):
    M, K, N = 37, 24, 50
    x, w, b = rnd(M, K + 3, dtype=dtype, seed=1, scale=2.0), rnd(N, K, dtype=dtype, seed=2), rnd(N, dtype=dtype, seed=3, scale=4.0)
    y = torch.empty(M, N, dtype=torch.float32, device=DEV)
    B().linear(x[:, 3:], w, y, M=M, bias=b, act=B().ACT_LOGSIGMOID, act_param=1.0 / 7.0, ldx=K + 3)
    z = f64(x[:, 3:]) @ f64(w).T + f64(b)
    assert rel(y, torch.log(torch.sigmoid(z)) / 7.0) < 1e-5 and float(y.max()) <= 0.0
    B().linear(x[:, 3:], w, y, M=M, act=B().ACT_SCALE, act_param=-2.5, ldx=K + 3)
    assert rel(y, -2.5 * (f64(x[:, 3:]) @ f64(w).T)) < 1e-5


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("taps,bias,act", [(3, False, False), (4, True, True), (2, False, True), (1, False, False), (1, True, True), (7, True, False)])
def test_short_convolution_over_steps_and_reused_slots(dtype, taps, bias, act):
    """Two sequences on two slots, fed in portions of unequal sizes (also of one token, also shorter than the taps reach back); a
    slot that held another sequence starts from zeros when its new sequence starts at position 0."""
    Cn, ld = 37, 45
    w = rnd(Cn, taps, dtype=dtype, seed=1)
    b = rnd(Cn, dtype=dtype, seed=2) if bias else None
    state = torch.full((2, taps - 1, Cn), 9.0, dtype=dtype, device=DEV)               # (what a slot held before must not matter)
    seqs = {0: rnd(23, ld, dtype=dtype, seed=3), 1: rnd(11, ld, dtype=dtype, seed=4)}
    plan = [{0: 1, 1: 4}, {0: 2, 1: 1}, {0: 9}, {1: 6, 0: 11}]                         # tokens per slot and step
    at, got = {0: 0, 1: 0}, {0: [], 1: []}
    for step in plan:
        rows, meta, reqs = [], [], []
        for slot, n in step.items():
            reqs.append((slot, at[slot], n, len(meta)))
            meta += [(slot, at[slot] + i, i, 0) for i in range(n)]
            rows.append(seqs[slot][at[slot]:at[slot] + n])
        x = torch.cat(rows).contiguous()
        out = torch.empty(len(meta), Cn, dtype=dtype, device=DEV)
        B().causal_conv(x[:, 5:], ld, w, b, act, dev_i32(meta), state, out, len(meta))
        if taps > 1:
            B().conv_state_update(x[:, 5:], ld, dev_i32(reqs), len(reqs), state)
        r = 0
        for slot, n in step.items():
            got[slot].append(out[r:r + n])
            at[slot] += n
            r += n
    for slot in (0, 1):
        want, _ = O.short_conv(f64(seqs[slot][:, 5:5 + Cn]), f64(w), f64(b) if bias else None, torch.zeros(taps - 1, Cn, dtype=F64))
        if act:
            want = O.silu(want)
        assert rel(torch.cat(got[slot]), want) < tol(dtype, 1e-6, 6e-3)
    # slot 1 goes to a new sequence: position 0 again
    x = rnd(5, ld, dtype=dtype, seed=8)
    out = torch.empty(5, Cn, dtype=dtype, device=DEV)
    B().causal_conv(x[:, 5:], ld, w, b, act, dev_i32([(1, i, i, 0) for i in range(5)]), state, out, 5)
    want, _ = O.short_conv(f64(x[:, 5:5 + Cn]), f64(w), f64(b) if bias else None, torch.zeros(taps - 1, Cn, dtype=F64))
    assert rel(out, O.silu(want) if act else want) < tol(dtype, 1e-6, 6e-3)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("D,rot,scaling", [(24, 16, (8.0, 1.0, 4.0, 64.0)), (10, 10, None), (64, 2, (4.0, 0.5, 2.0, 16.0)), (6, 0, None)])
def test_rotation_then_unit_norm_per_head(dtype, D, rot, scaling):
    """The design rotates the leading pairs and THEN divides each head by its root mean square; the kernel divides first.  Both are
    checked against the oracle's order, at positions from 0 to the thousands, with plain and wavelength-scaled frequencies."""
    from promptcache_amd.model.bepepel_hip import scaled_rotary_frequencies
    H, n = 3, 40
    x = rnd(n, H * D + 7, dtype=dtype, seed=1, scale=3.0)
    pos = torch.tensor([0, 1, 2, 3, 63, 64, 65, 511, 512, 1000] + list(range(2000, 2030)), dtype=torch.int32, device=DEV)
    out = torch.empty(n, H * D, dtype=dtype, device=DEV)
    freqs = torch.from_numpy(scaled_rotary_frequencies(777.0, rot, scaling)).to(DEV) if rot else None
    B().head_prep([B().head_seg(x[:, 7:], H * D + 7, H, D, out, norm=True, rot_dims=rot, ld_dst=H * D)], n, dtype, pos=pos, freqs=freqs, eps=1e-5)
    fr = O.rotary_frequencies(777.0, rot, scaling) if rot else torch.zeros(0, dtype=F64)
    want = O.unit_rms(O.rotate_pairs(f64(x[:, 7:]).view(n, H, D), pos.cpu(), fr), 1e-5).reshape(n, H * D)
    assert rel(out, want) < tol(dtype, 2e-6, 4e-3)


@pytest.mark.parametrize("n_exp,top", [(16, 4), (5, 5), (1, 1), (9, 1), (64, 8)])
def test_router_takes_the_top_logits_and_the_softmax_over_them(n_exp, top):
    T, K = 50, 24
    h, wr, br = rnd(T, K, seed=1), rnd(n_exp, K, seed=2), rnd(n_exp, seed=3, scale=2.0)
    logits = torch.empty(T, n_exp, dtype=torch.float32, device=DEV)
    B().linear(h, wr, logits, M=T, bias=br)
    expert = torch.empty(T * top, dtype=torch.int32, device=DEV)
    weight = torch.empty(T * top, dtype=torch.float32, device=DEV)
    B().router_select(logits, top, expert, weight, T, score_fn=B().SCORE_SOFTMAX, renorm=True)
    idx, w = O.route(f64(h), {"r.router": f64(wr), "r.router.b": f64(br)}, "r.", top)
    assert torch.equal(expert.view(T, top).cpu().long(), idx) and rel(weight.view(T, top), w) < 1e-5
    assert float((weight.view(T, top).sum(dim=1) - 1.0).abs().max()) < 1e-5


def _recurrence_inputs(dtype, n, H, Hk, D, Dv, dcols, seed):
    q, k, v = rnd(n, Hk * D + 3, dtype=dtype, seed=seed), rnd(n, Hk * D + 5, dtype=dtype, seed=seed + 1), rnd(n, H * Dv, dtype=dtype, seed=seed + 2)
    ld = torch.rand(n, H * dcols, generator=torch.Generator().manual_seed(seed + 3)).to(DEV) * 0.5     # (times a negative rate: a log decay)
    step = torch.rand(n, H + 2, generator=torch.Generator().manual_seed(seed + 4)).to(DEV) + 0.1
    rate = -torch.rand(H, generator=torch.Generator().manual_seed(seed + 5)).to(DEV) - 0.5
    return q, k, v, ld, step, rate


def _recurrence_oracle(q, k, v, ld, step, rate, H, Hk, D, Dv, dcols, q_scale, S0=None):
    n = q.shape[0]
    out, S = torch.zeros(n, H, Dv, dtype=F64), torch.zeros(H, D, Dv, dtype=F64) if S0 is None else S0.clone()
    for h in range(H):
        g = h // (H // Hk)
        decay = torch.exp(f64(rate)[h] * f64(ld)[:, h * dcols:(h + 1) * dcols])
        out[:, h], S[h] = O.matrix_state_steps(f64(q)[:, g * D:(g + 1) * D] * q_scale, f64(k)[:, g * D:(g + 1) * D],
                                               f64(step)[:, h:h + 1] * f64(v)[:, h * Dv:(h + 1) * Dv], decay, S[h])
    return out.reshape(n, H * Dv), S


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,Hk,D,Dv,per_channel", [(3, 3, 20, 24, True), (4, 2, 7, 70, False), (2, 2, 130, 33, True), (6, 1, 48, 48, False),
                                                   (1, 1, 256, 8, True), (2, 1, 1, 5, False)])
def test_matrix_state_recurrence_alone(dtype, H, Hk, D, Dv, per_channel):
    """Two requests of unequal length in one launch, one of them continuing on a state that an earlier launch left; decays per key
    channel or per head, step sizes on the values, fewer key heads than value heads."""
    dcols = D if per_channel else 1
    na, nb = 21, 9
    q, k, v, ld, step, rate = _recurrence_inputs(dtype, na + nb, H, Hk, D, Dv, dcols, seed=5)
    state = torch.full((3, H, D, Dv), 7.0, dtype=torch.float32, device=DEV)       # (what a slot held before position 0 must not matter)
    out = torch.empty(na + nb, H * Dv, dtype=torch.float32, device=DEV)
    lds_ = (Hk * D + 3, Hk * D + 5, H * Dv, H * dcols)
    kw = dict(ld_coef=rate, v_scale=step, ldvs=H + 2)
    # request a: 13 tokens on slot 2, then its other 8 next to request b's 9 on slot 0
    B().gla(q, k, v, ld, lds_, dcols, dev_i32([(2, 0, 13, 0)]), 1, state, H, Hk, D, Dv, 0.5, out, **kw)
    B().gla(q, k, v, ld, lds_, dcols, dev_i32([(0, 0, nb, na), (2, 13, 8, 13)]), 2, state, H, Hk, D, Dv, 0.5, out, **kw)
    wa, Sa = _recurrence_oracle(q[:na], k[:na], v[:na], ld[:na], step[:na], rate, H, Hk, D, Dv, dcols, 0.5)
    wb, Sb = _recurrence_oracle(q[na:], k[na:], v[na:], ld[na:], step[na:], rate, H, Hk, D, Dv, dcols, 0.5)
    t = tol(dtype, 1e-5, 1e-5)                               # (bf16 operands widen exactly: the arithmetic is fp32 either way)
    assert rel(out[:na], wa) < t and rel(out[na:], wb) < t
    assert rel(state[2], Sa) < t and rel(state[0], Sb) < t and float((state[1] - 7.0).abs().max()) == 0.0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,Hk,D,Dv,per_channel", [(3, 3, 20, 24, True), (4, 2, 40, 70, False)])
def test_recurrence_in_segments_equals_token_by_token(dtype, H, Hk, D, Dv, per_channel):
    """A first pass from zero states with the sums of the log decays, the chain over the segments, a second pass from the start
    states: the outputs and the slot's final state are those of one pass over all tokens; a request that continues an older state
    keeps it through the chain."""
    dcols = D if per_channel else 1
    n0, n = 10, 75
    q, k, v, ld, step, rate = _recurrence_inputs(dtype, n0 + n, H, Hk, D, Dv, dcols, seed=9)
    lds_ = (Hk * D + 3, Hk * D + 5, H * Dv, H * dcols)
    kw = dict(ld_coef=rate, v_scale=step, ldvs=H + 2)
    state = torch.zeros(2, H, D, Dv, dtype=torch.float32, device=DEV)
    out = torch.empty(n0 + n, H * Dv, dtype=torch.float32, device=DEV)
    B().gla(q, k, v, ld, lds_, dcols, dev_i32([(1, 0, n0, 0)]), 1, state, H, Hk, D, Dv, 1.0, out, **kw)
    segs = [(g, 0, min(16, n - c), n0 + c) for g, c in enumerate(range(0, n, 16))]
    ns, elems = len(segs), H * D * Dv
    local, start = torch.zeros(ns, H, D, Dv, device=DEV), torch.zeros(ns, H, D, Dv, device=DEV)
    lsum = torch.zeros(ns, H * dcols, device=DEV)
    B().gla(q, k, v, ld, lds_, dcols, dev_i32(segs), ns, local, H, Hk, D, Dv, 1.0, None, ld_sum=lsum, **kw)
    B().state_chain(local.view(ns, elems), start.view(ns, elems), state, dev_i32([(1, n0, 0, ns)]), 1, torch.ones(elems, device=DEV), lsum,
                    Dv if per_channel else D * Dv)
    B().gla(q, k, v, ld, lds_, dcols, dev_i32([(g, 1, c, r) for g, _, c, r in segs]), ns, start, H, Hk, D, Dv, 1.0, out, **kw)
    want, S = _recurrence_oracle(q, k, v, ld, step, rate, H, Hk, D, Dv, dcols, 1.0)
    assert rel(out, want) < 2e-5 and rel(state[1], S) < 2e-5 and float(state[0].abs().max()) == 0.0


def _attend(dtype, q, keys, vals, qpos, H, G, scale, *, window=0, keep_first=0, splits=1):
    """q [n, H, D] at positions qpos of ONE sequence whose keys [m, G, D] / values [m, G, Dv] sit at positions 0 .. m-1 of slot 1."""
    n, m, D, Dv = q.shape[0], keys.shape[0], q.shape[2], vals.shape[2]
    cap = -(-m // 32) * 32
    kplane = torch.zeros(2, G, cap, D, dtype=dtype, device=DEV)
    kplane[1, :, :m] = keys.transpose(0, 1)
    vplane = torch.full((2, G, Dv, cap), float("nan"), dtype=dtype, device=DEV)       # (what lies past the keys need not be numbers)
    vplane[1, :, :, :m] = vals.permute(1, 2, 0)
    tiles, at = [], 0
    while at < n:                                            # tiles of up to 16 consecutive positions
        run = 1
        while at + run < n and run < 16 and qpos[at + run] == qpos[at] + run:
            run += 1
        tiles.append((1, qpos[at], run, at))
        at += run
    out = torch.empty(n, H * Dv, dtype=dtype, device=DEV)
    part = torch.empty(B().attn_softmax_part(n, H, splits, Dv), dtype=torch.float32, device=DEV) if splits > 1 else None
    B().attn_softmax(q.reshape(n, H * D).contiguous(), H * D, dev_i32(tiles), len(tiles), kplane, (G * cap * D, cap * D, D), vplane, 0,
                     (G * Dv * cap, Dv * cap, cap), True, H, G, D, Dv, scale, out, window=window, keep_first=keep_first, n_splits=splits, part=part)
    return out.view(n, H, Dv)


def _attend_oracle(q, keys, vals, qpos, H, G, scale, window, keep_first):
    out = torch.zeros(q.shape[0], H, vals.shape[2], dtype=F64)
    for h in range(H):
        g = h // (H // G)
        out[:, h] = O.softmax_over_seen(f64(q[:, h]), f64(keys[:, g]), f64(vals[:, g]), qpos, window, keep_first, scale)
    return out


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("splits", [1, 3])
@pytest.mark.parametrize("window,keep", [(40, 4), (40, 0), (70, 33), (5, 64), (1, 1), (200, 7), (0, 9)])
def test_attention_behind_a_window_that_keeps_the_first_keys(dtype, splits, window, keep):
    H, G, D, Dv, m = 4, 2, 24, 40, 310
    keys, vals = rnd(m, G, D, dtype=dtype, seed=1), rnd(m, G, Dv, dtype=dtype, seed=2)
    qpos = list(range(0, 12)) + list(range(28, 110)) + [150, 151, 255, 256, 257, 309]      # prompt rows from the start, then single rows
    q = rnd(len(qpos), H, D, dtype=dtype, seed=3)
    got = _attend(dtype, q, keys, vals, qpos, H, G, 0.3, window=window, keep_first=keep, splits=splits)
    want = _attend_oracle(q, keys, vals, qpos, H, G, 0.3, window, keep)
    assert rel(got, want) < tol(dtype, 1e-5, 1e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window,keep,loud", [(40, 4, 130), (40, 4, 3), (40, 4, 4), (33, 32, 31), (33, 32, 32), (1, 0, 200), (64, 0, 63), (64, 70, 69), (64, 70, 70)])
def test_one_loud_key_at_the_windows_edge_and_among_the_kept_first(dtype, window, keep, loud):
    """Every key is quiet but one, whose score towers over the rest.  A query that sees it returns its value; one that does not must
    not, whatever the hundreds of other keys say: just inside and just outside the window, the last kept position and the one
    after it, far away, as rows of a prompt tile and as single decoded rows, whole and in runs of the keys."""
    H, G, D, Dv, m = 2, 1, 16, 8, 300
    keys, vals = 0.05 * rnd(m, G, D, dtype=dtype, seed=1), rnd(m, G, Dv, dtype=dtype, seed=2)
    keys[loud] = 0.0
    keys[loud, 0, 3] = 30.0
    vals[loud] = 5.0
    q = 0.05 * rnd(m, H, D, dtype=dtype, seed=3)
    q[:, :, 3] = 2.0
    inside, outside = loud + window - 1, loud + window
    for pos in (list(range(inside - 5, outside + 5)), [inside, outside], [outside + 60, 299]):
        pos = [p for p in pos if p < m]
        for splits in (1, 4):
            got = _attend(dtype, q[pos], keys, vals, pos, H, G, 1.0, window=window, keep_first=keep, splits=splits)
            assert rel(got, _attend_oracle(q[pos], keys, vals, pos, H, G, 1.0, window, keep)) < tol(dtype, 1e-5, 1e-2)
            for x, p in enumerate(pos):
                hit = float((got[x].float() - 5.0).abs().max()) < 0.05
                assert hit == O.sees(p, loud, window, keep), (p, loud)


# =====================================================================================================================================
# the model through its arena
# =====================================================================================================================================
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(SHAPES))
def test_whole_prompt_against_the_oracle_layer_by_layer(name, dtype):
    s, w, m = model(name, dtype)
    t = toks(150, s.vocab_size, 1)                           # (longer than a segment of the recurrences' prefill)
    want, streams = oracle_logits(s, w, t, key=(name, 150))
    ar = m.new_arena(1, 8)
    got, gs = m.forward_rows(ar, [ar.alloc()], [t], [list(range(150))], return_streams=True)
    for i in range(len(s.layers)):
        assert close(gs[i], streams[i], dtype, 2e-5), (i, s.layers[i].kind)
    assert close(got, want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(SHAPES))
def test_prompt_equals_token_by_token_decoding_and_any_portions(name, dtype):
    s, w, m = model(name, dtype)
    t = toks(150, s.vocab_size, 1)
    want = oracle_logits(s, w, t, key=(name, 150))[0]
    whole = run_alone(m, t)
    for cuts in ([1] * 150, [2] * 75, [3, 2, 64, 1, 65, 15], [149, 1], [70, 80]):
        got = run_alone(m, t, cuts)
        assert close(got, want, dtype), cuts
        # how a prompt is cut changes summation order only (bf16: and with it now and then the rounding of an operand)
        assert close(got, whole, dtype, 5e-6, 1e-2), cuts


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("graphs", [True, False])
def test_unequal_batches_reused_slots_and_states(dtype, graphs):
    """Three requests of unequal length prefilled together, decoded together (the shortest ends first and its slot -- keys, values,
    convolution inputs and matrix states -- goes to a newcomer that starts from position 0), each against itself alone."""
    s, w, m = model("mixed", dtype)
    m.use_graphs = graphs
    try:
        V = s.vocab_size
        a, b_, c, d = toks(90, V, 1), toks(5, V, 2), toks(40, V, 3), toks(30, V, 4)
        wa, wb, wc, wd = (oracle_logits(s, w, x, key=("mixed", "batch", i))[0] for i, x in enumerate((a, b_, c, d)))
        ar = m.new_arena(3, 32)
        sa, sb, sc = ar.alloc(), ar.alloc(), ar.alloc()
        got = [m.forward_rows(ar, [sa, sb, sc], [a[:70], b_[:3], c[:20]], [[69], [0, 2], list(range(20))])]
        want = [wa[69:70], wb[[0, 2]], wc[:20]]
        for k in range(2):
            got.append(m.forward_rows(ar, [sa, sb, sc], [[a[70 + k]], [b_[3 + k]], [c[20 + k]]]))
            want += [wa[70 + k:71 + k], wb[3 + k:4 + k], wc[20 + k:21 + k]]
        ar.free(sb)
        sd = ar.alloc()
        assert sd == sb                                      # the freed slot comes back, with everything the old request left in it
        got.append(m.forward_rows(ar, [sd, sa, sc], [d[:17], a[72:90], c[22:30]], [[16], [17], [7]]))
        want += [wd[16:17], wa[89:90], wc[29:30]]
        for k in range(10):
            got.append(m.forward_rows(ar, [sc, sd], [[c[30 + k]], [d[17 + k]]]))
            want += [wc[30 + k:31 + k], wd[17 + k:18 + k]]
        assert close(torch.cat(got), torch.cat(want), dtype)
        if dtype == torch.bfloat16:                          # and in bf16 every row is what the request gets alone, flips and all
            alone = torch.cat([run_alone(m, d)[17:27], run_alone(m, c)[30:40]])
            mine = torch.cat([torch.stack([g[1] for g in got[-10:]]), torch.stack([g[0] for g in got[-10:]])])
            assert close(mine, alone, dtype, bf16=1e-2)
    finally:
        m.use_graphs = True


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding_through_graphs_across_every_edge_and_a_growing_arena(dtype):
    s, w, m = model("mixed", dtype)
    t = toks(200, s.vocab_size, 7)
    want = oracle_logits(s, w, t, key=("mixed", 200))[0]
    ar = m.new_arena(1, 8)                                   # (the arena grows under the captured steps)
    sl = ar.alloc()
    got = [m.forward_rows(ar, [sl], [t[:2]], [[0, 1]])] + [m.forward_rows(ar, [sl], [[x]]) for x in t[2:]]
    assert close(torch.cat(got), want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_far_positions_in_a_long_prompt_and_after_it(dtype):
    """A prompt of many segments and key blocks, then decoding behind it: the kept first keys are hundreds of positions away."""
    s, w, m = model("wide", dtype)
    t = toks(700, s.vocab_size, 9)
    want = oracle_logits(s, w, t, key=("wide", 700))[0]
    ar = m.new_arena(1, 8)
    sl = ar.alloc()
    places = [0, 1, 39, 40, 63, 64, 99, 100, 139, 140, 400, 679]
    got = [m.forward_rows(ar, [sl], [t[:680]], [places])] + [m.forward_rows(ar, [sl], [[x]]) for x in t[680:]]
    assert close(got[0], want[places], dtype) and close(torch.cat(got[1:]), want[680:], dtype)


def test_same_rows_same_values_whatever_the_company():
    """float32: a request's logits next to other requests, and on another slot, agree with those it gets alone to summation order."""
    s, w, m = model("wide", torch.float32)
    a, b_, c = toks(50, s.vocab_size, 1), toks(9, s.vocab_size, 2), toks(23, s.vocab_size, 3)
    alone = run_alone(m, a)
    ar = m.new_arena(3, 64)
    s0, s1, s2 = ar.alloc(), ar.alloc(), ar.alloc()
    out = m.forward_rows(ar, [s0, s2, s1], [b_, a, c], [[0], list(range(50)), []])
    assert rel(out[1:], alone) < 2e-6


@pytest.mark.parametrize("dtype", DTYPES)
def test_greedy_generation_through_the_batch_engine(dtype):
    from promptcache_amd import BatchEngine, GenerationParameters
    from promptcache_amd.model import Bepepel
    s = shape_mixed()
    w = W.make_bepepel_weights(s, seed=11)
    lm = Bepepel(shape=s, weights=w, device=DEV, dtype=dtype)
    prompts = [toks(n, s.vocab_size, seed=40 + n) for n in (12, 3, 30)]
    eng = BatchEngine(lm, max_tokens=80)                      # (a budget that does not hold all three at once)
    params = GenerationParameters(temperature=0.0, max_new_tokens=12, stop_token_ids=[])
    got = eng.generate(prompts, params)
    p6 = O.to_f64(w)
    for prompt, out in zip(prompts, got):
        assert len(out) == 12
        seq = list(prompt)
        for k, tok in enumerate(out):                         # every generated token is the oracle's choice given the same history,
            logits = O.forward(s, p6, seq)[-1]                # unless the oracle's two best are closer than the format resolves
            best = int(logits.argmax())
            if tok != best:
                assert float(logits[best] - logits[tok]) < (1e-4 if dtype == torch.float32 else 0.15), (k, tok, best)
            seq.append(tok)


def random_shape(rng):
    """Sizes, layer order, windows, kept tokens, rotated parts, taps, groups and constants drawn at random."""
    width = rng.choice([64, 72, 96, 160, 200, 256])
    layers = []
    for _ in range(rng.randrange(2, 6)):
        ff = rng.choice([{}, dict(ff_kind="dense", ff=rng.choice([32, 56, width])),
                         dict(ff_kind="moe", experts=rng.choice([2, 5, 8, 16]), top=rng.choice([1, 2]), expert_ff=rng.choice([16, 40, 96]),
                              shared_ff=rng.choice([0, 24, 64]))])
        if rng.random() < 0.5:
            layers.append(gla(rng.choice([1, 2, 4, 6]), rng.choice([8, 16, 32, 48, 100]), rng.choice([8, 16, 32, 48, 130]), tau=rng.choice([1.0, 4.0, 16.0]),
                              rank=rng.choice([2, 8, 16]), **ff))
        else:
            G, sg, D = rng.choice([1, 2, 4]), rng.choice([1, 2, 4]), rng.choice([16, 24, 48, 64, 96, 160])
            sh = sg * rng.choice([1, 2, 3])
            sp = rng.choice([8, 16, 48, 64])
            parts = rng.choice([p for p in (1, 2, sh) if (sh * sp) % p == 0])
            layers.append(par(G * rng.choice([1, 2, 3]), G, D, rng.choice([16, 40, 64, 128]), rng.choice([0, 1, 7, 32, 50, 100]), rng.choice([0, 1, 4, 40]),
                              sh, sp, rng.choice([4, 16, 48, 128]), sg=sg, parts=parts, convl=rng.choice([0, 2, 3, 4]), convr=rng.choice([0, 2, 4]),
                              rot=rng.choice([D, D // 4 * 2, 0]), scaling=rng.choice([None, (8.0, 1.0, 4.0, 128.0), (2.0, 0.5, 8.0, 32.0)]),
                              scale=rng.choice([0.125, 0.5, 1.0]), ls=rng.choice([1.0, 1.3]), rs=rng.choice([1.0, 0.7]),
                              base=rng.choice([300000.0, 1000.0]), **ff))
    return BepepelShape(vocab_size=rng.randrange(50, 900), hidden_size=width, norm_eps=rng.choice([1e-5, 1e-6]),
                        residual_mult=rng.choice([1.0, 0.45]), logit_scale=rng.choice([1.0, 1.75]), layers=layers)


@pytest.mark.parametrize("seed", range(8))
def test_random_configurations_whole_decoded_and_in_company(seed):
    import random
    from promptcache_amd.model.bepepel_hip import BepepelHIP
    rng = random.Random(2000 + seed)
    s = BepepelShape.from_config(json.loads(json.dumps(random_shape(rng).to_config())))
    for l in s.layers:                                       # (the decay projection's rank is a tensor's shape, not a configuration key)
        assert l.kind != "gla" or l.a_rank > 0
    w = W.make_bepepel_weights(s, seed=seed)
    n = rng.randrange(90, 260)
    a, b_ = toks(n, s.vocab_size, seed), toks(rng.randrange(1, 70), s.vocab_size, seed + 1)
    want_a, want_b = oracle_logits(s, w, a)[0], oracle_logits(s, w, b_)[0]
    for dtype in DTYPES:
        m = BepepelHIP(s, w, device=DEV, dtype=dtype)
        assert close(run_alone(m, a), want_a, dtype, 5e-5, 4e-2), s.to_config()
        ar = m.new_arena(1, 16)
        sa, sb = ar.alloc(), ar.alloc()
        cut = n - 20
        out = [m.forward_rows(ar, [sb, sa], [b_, a[:cut]], [list(range(len(b_))), list(range(cut))])]
        out += [m.forward_rows(ar, [sa], [[t_]], [[0]]) for t_ in a[cut:]]
        got = torch.cat(out)
        assert close(got[len(b_):], want_a, dtype, 5e-5, 4e-2) and close(got[:len(b_)], want_b, dtype, 5e-5, 4e-2), s.to_config()


def test_single_request_engine_and_the_adapters_call():
    """GenerationEngine drives the model through the adapters' ``model(input_ids, past_key_values)`` call; a padded batch through
    that call gives each row its own logits."""
    from promptcache_amd import BatchEngine, GenerationEngine, GenerationParameters
    from promptcache_amd.model import Bepepel
    s = shape_mixed()
    w = W.make_bepepel_weights(s, seed=21)
    lm = Bepepel(shape=s, weights=w, device=DEV, dtype=torch.float32)
    prompts = [toks(13, s.vocab_size, 30), toks(5, s.vocab_size, 31)]
    params = GenerationParameters(temperature=0.0, max_new_tokens=6, stop_token_ids=[])
    want = BatchEngine(lm).generate(prompts, params)
    out = None
    for out in GenerationEngine(lm).generate(prompts[0], list(range(13)), params):
        pass
    assert out is not None and lm.decode(want[0]) == out.new_text
    ids, mask = torch.zeros((2, 13), dtype=torch.long), torch.zeros((2, 13), dtype=torch.long)
    ids[0, :13], mask[0, :13] = torch.tensor(prompts[0]), 1
    ids[1, :5], mask[1, :5] = torch.tensor(prompts[1]), 1
    res = lm(input_ids=ids, attention_mask=mask, past_key_values=None, use_cache=True)
    p6 = O.to_f64(w)
    assert rel(res.logits[0], O.forward(s, p6, prompts[0])) < 3e-5 and rel(res.logits[1, :5], O.forward(s, p6, prompts[1])) < 3e-5
    assert int(res.logits[0, 12].argmax()) == want[0][0] and int(res.logits[1, 4].argmax()) == want[1][0]


def test_checkpoint_directory_command_line_and_trace_runner(tmp_path):
    """config.json + model.safetensors written from a shape, found by the registry, and replayed by bin/trace_run in both formats."""
    from safetensors.torch import save_file
    from promptcache_amd.model import load_language_model
    s = shape_odd()
    w = W.make_bepepel_weights(s, seed=3)
    d = tmp_path / "ckpt"
    d.mkdir()
    cfg = s.to_config()
    for lc in cfg["layers"]:
        lc["mixer"].pop("a_rank", None)                      # as a checkpoint's configuration comes: the rank is the tensor's shape
    (d / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in w.items()}, str(d / "model.safetensors"))
    lm = load_language_model(str(d), dtype=torch.float32)
    assert type(lm).__name__ == "Bepepel" and lm.hf_model.config.to_config() == s.to_config()
    a, b_ = toks(21, s.vocab_size, 1), toks(6, s.vocab_size, 2)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:15], "want": [0, 14]}, {"id": "b", "tokens": b_[:5], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[15:16], "want": [0]}, {"id": "b", "tokens": b_[5:], "want": [0]}], "end": ["b"]}] + \
            [{"step": 2 + k, "entries": [{"id": "a", "tokens": [a[16 + k]], "want": [0] if k % 2 else []}], "end": ["a"] if k == 4 else []}
             for k in range(5)]
    wa, wb = oracle_logits(s, w, a)[0], oracle_logits(s, w, b_)[0]
    want = {0: wa[[0, 14]], 1: torch.stack([wa[15], wb[5]]), 3: wa[17:18], 5: wa[19:20]}
    env = dict(os.environ, PYTHONPATH=os.pathsep.join([ROOT, os.path.join(ROOT, "prompt-cache_amd")]))
    for fmt, t in (("float32", 3e-5), ("bfloat16", 8e-2)):
        out = tmp_path / fmt
        r = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", str(d), "--dtype", fmt, "--out", str(out), "--max-tokens", "40"],
                           input="\n".join(json.dumps(x) for x in steps) + "\n", capture_output=True, text=True, env=env, timeout=600)
        assert r.returncode == 0, r.stderr[-2000:]
        assert [ln for ln in r.stdout.splitlines() if ln.startswith("done")] == [f"done {k}" for k in range(7)]
        assert sorted(os.listdir(out)) == ["0.f32", "1.f32", "3.f32", "5.f32"]
        for k, wv in want.items():
            import numpy as np
            got = torch.from_numpy(np.fromfile(out / f"{k}.f32", dtype="<f4").reshape(-1, s.vocab_size))
            assert rel(got, wv) < t, (fmt, k)
