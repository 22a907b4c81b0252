"""Fivesun on the GPU against the plain float64 oracle (``oracle/fivesun_oracle.py``): every new building-block kernel alone --
with inputs built so that a window's or block's edge, a sink or a far key decides the result --, then the model through its
arena: prompts, token-by-token decoding, portions, unequal batches, reused slots and states, long decoding through captured
graphs, and greedy generation through the batch engine and the trace runner.  float32 runs are held to float32 accuracy; bfloat16
runs to what bf16 operands allow (every sublayer's result is normed to unit size before it joins the residual, so a few percent of
operand rounding in a narrow random model arrive in the stream undiminished)."""
import json
import math
import os
import subprocess

import pytest
import torch

from oracle import fivesun_oracle as O
from promptcache_amd.model import weights as W
from promptcache_amd.model.config import FivesunLayer, FivesunShape

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


def B():
    from promptcache_amd import _blocks
    return _blocks


def rnd(*shape, dtype=torch.float32, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (scale * torch.randn(*shape, generator=g)).to(dtype).to(DEV)


def dev_i32(rows):
    return torch.tensor(rows, dtype=torch.int32, device=DEV).reshape(-1)


def att(heads, kv, dim, vdim, mask, rot_dims=None, v_mix=False, ff=0, scale=None, factor=3.0, base=30000.0):
    return FivesunLayer("attention", heads=heads, kv_heads=kv, dim=dim, vdim=vdim, scale=scale or dim ** -0.5, mask=mask, rot_base=base,
                        rot_dims=dim if rot_dims is None else rot_dims, rot_factor=factor, v_mix=v_mix, ff=ff)


def lat(heads, dim, rot, vdim, rank, mask, ff=0, original=64.0, factor=4.0, fast=8.0, slow=1.0, base=10000.0):
    return FivesunLayer("latent_attention", heads=heads, kv_heads=1, dim=dim, vdim=vdim, kv_rank=rank, rot_dim=rot, rot_dims=rot,
                        scale=(dim + rot) ** -0.5, mask=mask, rot_base=base, rot_factor=factor, yarn_original=original, yarn_fast=fast,
                        yarn_slow=slow, ff=ff)


def mls(heads, dim, vdim, cap=9.0, ff=0):
    return FivesunLayer("mlstm", heads=heads, kv_heads=heads, dim=dim, vdim=vdim, gate_cap=cap, ff=ff)


# ---- shapes: layers differ from one another, come in different orders, and no size is a round one -------------------------------
def shape_mixed():
    return FivesunShape(vocab_size=150, hidden_size=96, norm_eps=1e-5, embed_scale=7.5, layers=[
        mls(3, 20, 24, cap=6.0, ff=40),
        att(6, 3, 24, 40, mask=21, rot_dims=16, v_mix=False, ff=56),
        att(4, 2, 40, 24, mask=33, v_mix=True, ff=0),
        lat(5, 24, 8, 20, 40, mask=17, ff=72),
        att(4, 2, 16, 24, mask=50, rot_dims=0, v_mix=True, ff=48, factor=1.0),
        att(2, 2, 32, 24, mask=0, v_mix=True, ff=24),
    ])


def shape_odd():
    """Sizes that are no multiple of a 16-byte chunk in either element type; one head, equal key and query heads, a window and a
    block of one position, no rotation, plain (unscaled) frequencies, an uncapped mLSTM, layers without a feed-forward."""
    return FivesunShape(vocab_size=75, hidden_size=50, norm_eps=1e-6, embed_scale=1.0, layers=[
        lat(1, 10, 0, 6, 14, mask=0, ff=14),
        att(3, 3, 10, 6, mask=1, rot_dims=6, ff=0, factor=1.0),
        mls(1, 6, 10, cap=0.0, ff=10),
        lat(3, 6, 4, 10, 22, mask=1, ff=0, original=0.0, factor=1.0),
        mls(2, 7, 5, cap=2.5, ff=0),
    ])


def shape_wide():
    """Enough heads and columns to reach the wider kernel instantiations (keys beyond 256 columns, 200-column mLSTM heads)."""
    return FivesunShape(vocab_size=320, hidden_size=128, norm_eps=1e-6, embed_scale=11.3, layers=[
        att(8, 2, 128, 72, mask=64, v_mix=True, ff=96),
        lat(4, 48, 32, 40, 256, mask=40, ff=64, original=128.0),
        mls(2, 200, 136, ff=64),
        att(4, 2, 272, 72, mask=100, rot_dims=64, v_mix=True, ff=0),
    ])


SHAPES = {"mixed": shape_mixed, "odd": shape_odd, "wide": shape_wide}
_models = {}


def model(name, dtype, seed=11):
    from promptcache_amd.model.fivesun_hip import FivesunHIP
    key = (name, dtype, seed)
    if key not in _models:
        s = SHAPES[name]()
        w = W.make_fivesun_weights(s, seed=seed)
        _models[key] = (s, w, FivesunHIP(s, w, device=DEV, dtype=dtype))
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


# =====================================================================================================================================
# building blocks alone
# =====================================================================================================================================
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M", [3, 40, 150])
@pytest.mark.parametrize("act", ["relu", "silu", "gelu_tanh"])
def test_gated_unit_with_biases(dtype, M, act):
    K, N = 50, 70
    x, wg, wu = rnd(M, K, dtype=dtype, seed=1), rnd(N, K, dtype=dtype, seed=2, scale=0.3), rnd(N, K, dtype=dtype, seed=3, scale=0.3)
    bg, bu = rnd(N, dtype=dtype, seed=4), rnd(N, dtype=dtype, seed=5)
    y = torch.empty(M, N, dtype=dtype, device=DEV)
    from promptcache_amd.model.fivesun_hip import ACTS
    B().linear(x, wg, y, M=M, epilogue=B().EPI_SILU_MUL, w2=wu, bias=bg, bias2=bu, act=ACTS[act])
    x6, f = x.to("cpu", F64), lambda t: t.to("cpu", F64)
    want = O.activation(act)(x6 @ f(wg).T + f(bg)) * (x6 @ f(wu).T + f(bu))
    assert rel(y, want) < tol(dtype, 1e-5, 1e-2)
    # the epilogue without an activation named is the SiLU unit without biases, as before
    B().linear(x, wg, y, M=M, epilogue=B().EPI_SILU_MUL, w2=wu)
    assert rel(y, O.activation("silu")(x6 @ f(wg).T) * (x6 @ f(wu).T)) < tol(dtype, 1e-5, 1e-2)


def test_embedding_rows_times_a_constant():
    table, ids = rnd(9, 37, dtype=torch.bfloat16, seed=1), dev_i32([8, 0, 3, 3])
    out = torch.empty(4, 37, dtype=torch.float32, device=DEV)
    B().embed_scaled_rows(table, ids, 17.25, out)
    assert torch.equal(out, table.float()[ids.long()] * 17.25)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("W_", [50, 1500])
def test_post_norm_halves(dtype, W_):
    T, eps = 7, 1e-5
    x0, y = rnd(T, W_, seed=1, scale=3.0), rnd(T, W_, seed=2)
    gate = rnd(T, W_ + 9, dtype=dtype, seed=3).sigmoid()
    pg, g = 1 + 0.1 * rnd(W_, seed=4), 1 + 0.1 * rnd(W_, seed=5)
    f = lambda t: t.to("cpu", F64)
    t = f(y) * f(gate)[:, 4:4 + W_]
    x_new = f(x0) + O.unit_rms(t, eps) * f(pg)
    # both halves at once
    x, out, xo = x0.clone(), torch.empty(T, W_, dtype=dtype, device=DEV), torch.empty(T, W_, dtype=torch.float32, device=DEV)
    B().post_norm(x, y=y, gate=gate[:, 4:], ldg=W_ + 9, post_gain=pg, gain=g, out=out, x_out=xo, eps=eps)
    assert rel(x, x_new) < 1e-6 and torch.equal(x, xo) and rel(out, O.unit_rms(x_new, eps) * f(g)) < tol(dtype, 1e-6, 5e-3)
    # a subset of the rows: the sum is used, not written back
    rows = dev_i32([5, 0, 5])
    x, out3 = x0.clone(), torch.empty(3, W_, dtype=dtype, device=DEV)
    B().post_norm(x, y=y, gate=gate[:, 4:], ldg=W_ + 9, post_gain=pg, gain=g, out=out3, rows=rows, eps=eps)
    assert torch.equal(x, x0) and torch.equal(out3, out[rows.long()])
    # no gate, no norm after the sublayer: a plain residual sum; and the read half alone
    x = x0.clone()
    B().post_norm(x, y=y, eps=eps)
    assert rel(x, f(x0) + f(y)) < 1e-7
    B().post_norm(x0, gain=g, out=out, eps=eps)
    assert rel(out, O.unit_rms(f(x0), eps) * f(g)) < tol(dtype, 1e-6, 5e-3)


@pytest.mark.parametrize("dtype", DTYPES)
def test_norm_per_head_with_gate(dtype):
    T, H, Dv = 5, 3, 10
    x, gain, gate = rnd(T, H * Dv, seed=1, scale=4.0), 1 + 0.2 * rnd(H * Dv, seed=2), rnd(T, 2 * H * Dv, dtype=dtype, seed=3).sigmoid()
    out = torch.empty(T, H * Dv, dtype=dtype, device=DEV)
    B().gated_norm(x, gain, gate[:, H * Dv:], 2 * H * Dv, out, 1e-5, T, group=Dv)
    f = lambda t: t.to("cpu", F64)
    want = O.unit_rms(f(x).view(T, H, Dv), 1e-5).reshape(T, -1) * f(gain) * f(gate)[:, H * Dv:]
    assert rel(out, want) < tol(dtype, 1e-6, 5e-3)
    # one group = the whole row: the old form
    B().gated_norm(x, gain, None, 0, out, 1e-5, T, group=H * Dv)
    assert rel(out, O.unit_rms(f(x), 1e-5) * f(gain)) < tol(dtype, 1e-6, 5e-3)


@pytest.mark.parametrize("dtype", DTYPES)
def test_head_preparation_norm_blend_rotation_and_destinations(dtype):
    """Queries into rows, keys into a cache kept row by row, values (blended) into one kept column by column; positions in the
    hundreds of thousands, where an angle taken in 32-bit would have lost its low bits."""
    T, H, G, D, Dv, cap, eps = 6, 3, 2, 14, 6, 32, 1e-5
    N = H * D + G * D + G * Dv + 5
    P = rnd(T, N, dtype=dtype, seed=1)
    pos = [0, 1, 31, 250001, 7, 999983]
    slot_of = [0, 0, 0, 1, 1, 1]
    place = [0, 1, 31, 5, 7, 30]                           # where the row lands in its slot (the test's own choice)
    qg, kg = 1 + 0.1 * rnd(D, seed=2), 1 + 0.1 * rnd(D, seed=3)
    other, lam = rnd(T, G * Dv, seed=4), torch.tensor([0.3], device=DEV)
    fr, mag = O.yarn_frequencies(10000.0, 8, 4.0, 64.0, 8.0, 1.0)
    q = torch.zeros(T, H * D, dtype=dtype, device=DEV)
    kplane = torch.zeros(2, G, cap, D, dtype=dtype, device=DEV)
    vplane = torch.zeros(2, G, Dv, cap, dtype=dtype, device=DEV)
    keep = torch.zeros(T, G * Dv, dtype=torch.float32, device=DEV)
    koff = torch.tensor([s * G * cap * D + p * D for s, p in zip(slot_of, place)], dtype=torch.int64, device=DEV)
    voff = torch.tensor([s * G * Dv * cap + p for s, p in zip(slot_of, place)], dtype=torch.int64, device=DEV)
    b = B()
    segs = [b.head_seg(P, N, H, D, q, norm=True, gain=qg, rot_off=4, rot_dims=8, ld_dst=H * D),
            b.head_seg(P[:, H * D:], N, G, D, kplane, norm=True, gain=kg, rot_off=4, rot_dims=8, row_off=koff, head_stride=cap * D),
            b.head_seg(P[:, H * D + G * D:], N, G, Dv, vplane, norm=True, blend=lam, other=other, keep=keep, row_off=voff,
                       head_stride=Dv * cap, col_stride=cap)]
    b.head_prep(segs, T, dtype, pos=dev_i32(pos), freqs=fr.to(DEV), rot_mag=mag, eps=eps)
    f = lambda t: t.to("cpu", F64)
    P6, p6 = f(P), torch.tensor(pos)

    def turned(x):
        x = x.clone()
        x[..., 4:12] = O.rotate_pairs(x[..., 4:12], p6, fr, mag)
        return x
    want_q = turned(O.unit_rms(P6[:, :H * D].view(T, H, D), eps) * f(qg))
    want_k = turned(O.unit_rms(P6[:, H * D:H * D + G * D].view(T, G, D), eps) * f(kg))
    want_v = 0.7 * O.unit_rms(P6[:, H * D + G * D:H * D + G * D + G * Dv].view(T, G, Dv), eps) + 0.3 * f(other).view(T, G, Dv)
    t = tol(dtype, 2e-6, 5e-3)
    assert rel(q, want_q.reshape(T, -1)) < t and rel(keep, want_v.reshape(T, -1)) < 1e-6
    got_k = torch.stack([kplane[s, :, p] for s, p in zip(slot_of, place)])
    got_v = torch.stack([vplane[s, :, :, p] for s, p in zip(slot_of, place)])
    assert rel(got_k, want_k) < t and rel(got_v, want_v) < t
    untouched = torch.ones(2, cap, dtype=torch.bool)
    for s, p in zip(slot_of, place):
        untouched[s, p] = False
    assert float(kplane.float().abs().sum(dim=(1, 3)).cpu()[untouched].sum()) == 0.0


def _attend(dtype, q, keys, vals, qpos, H, G, scale, *, window=0, block=0, sink=None, gate=None, splits=1, cols=True, head_rows=False):
    """q [n, H, D] at positions qpos of ONE sequence whose keys [m, G, D] / values [m, G, Dv] sit at positions 0 .. m-1."""
    n, m, D, Dv = q.shape[0], keys.shape[0], q.shape[2], vals.shape[2]
    cap = -(-m // 32) * 32
    kplane = torch.zeros(2, G, cap, D, dtype=dtype, device=DEV)
    kplane[1, :, :m] = keys.transpose(0, 1)
    if cols:
        vplane = torch.full((2, G, Dv, cap), float("nan"), dtype=dtype, device=DEV)       # (what lies past the keys need not be numbers)
        vplane[1, :, :, :m] = vals.permute(1, 2, 0)
        vstr = (G * Dv * cap, Dv * cap, cap)
    else:
        vplane = torch.zeros(2, G, cap, Dv, dtype=dtype, device=DEV)
        vplane[1, :, :m] = vals.transpose(0, 1)
        vstr = (G * cap * Dv, cap * Dv, Dv)
    # tiles of up to 16 consecutive positions
    tiles, at = [], 0
    while at < n:
        run = 1
        while at + run < n and run < 16 and qpos[at + run] == qpos[at] + run and not head_rows:
            run += 1
        tiles.append((1, qpos[at], run, at))
        at += run
    out = torch.empty(n, H * Dv, dtype=dtype, device=DEV)
    part = torch.empty(B().attn_softmax_part(n, H, splits, Dv), dtype=torch.float32, device=DEV) if splits > 1 else None
    B().attn_softmax(q.reshape(n, H * D).contiguous(), H * D, dev_i32(tiles), len(tiles), kplane, (G * cap * D, cap * D, D), vplane, 0, vstr, cols,
                     H, G, D, Dv, scale, out, window=window, block=block, sink=sink, gate=gate, ldg=H if gate is not None else 0,
                     gate_per_head=gate is not None, n_splits=splits, part=part, head_rows=head_rows)
    return out.view(n, H, Dv)


def _attend_oracle(q, keys, vals, qpos, H, G, scale, sees, sink=None, gate=None):
    f = lambda t: t.to("cpu", F64)
    out = torch.zeros(q.shape[0], H, vals.shape[2], dtype=F64)
    for h in range(H):
        g = h // (H // G)
        out[:, h] = O.softmax_attention(f(q[:, h]), f(keys[:, g]), f(vals[:, g]), qpos, sees, scale, sink=f(sink)[h] if sink is not None else None)
        if gate is not None:
            out[:, h] *= f(gate)[:, h:h + 1]
    return out


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("splits", [1, 3])
@pytest.mark.parametrize("D,Dv,cols", [(24, 40, True), (72, 24, False), (272, 40, True)])
def test_attention_blocks_sinks_and_head_gates(dtype, splits, D, Dv, cols):
    H, G, m, block = 4, 2, 150, 37
    keys, vals = rnd(m, G, D, dtype=dtype, seed=1), rnd(m, G, Dv, dtype=dtype, seed=2)
    qpos = list(range(30, 80)) + [110, 111, 147, 148, 149]          # prompt rows across two block edges, then single rows
    q = rnd(len(qpos), H, D, dtype=dtype, seed=3)
    sink, gate = rnd(H, seed=4, scale=2.0), rnd(len(qpos), H, dtype=dtype, seed=5).sigmoid()
    got = _attend(dtype, q, keys, vals, qpos, H, G, 0.3, block=block, sink=sink, gate=gate, splits=splits, cols=cols)
    want = _attend_oracle(q, keys, vals, qpos, H, G, 0.3, lambda i, j: O.sees_block(i, j, block), sink, gate)
    assert rel(got, want) < tol(dtype, 1e-5, 1e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("splits", [1, 4])
@pytest.mark.parametrize("H", [20, 3])
def test_sixteen_heads_of_one_token_share_a_pass_over_one_key_head(dtype, splits, H):
    """Single decoded rows over ONE key head whose values are the first columns of the key rows themselves (a shared latent):
    heads as the rows of a tile, a full block of 16 and a partial one, with a window."""
    D, Dv, m, window = 40, 24, 200, 90
    keys = rnd(m, 1, D, dtype=dtype, seed=1)
    vals = keys[:, :, :Dv].contiguous()
    qpos = [0, 5, 89, 90, 91, 150, 199]
    q = rnd(len(qpos), H, D, dtype=dtype, seed=3)
    sink = rnd(H, seed=4)
    got = _attend(dtype, q, keys, vals, qpos, H, 1, 0.2, window=window, sink=sink, splits=splits, cols=False, head_rows=True)
    want = _attend_oracle(q, keys, vals, qpos, H, 1, 0.2, lambda i, j: O.sees_window(i, j, window), sink)
    assert rel(got, want) < tol(dtype, 1e-5, 1e-2)
    same = _attend(dtype, q, keys, vals, qpos, H, 1, 0.2, window=window, sink=sink, splits=splits, cols=False)
    assert rel(got, same) < tol(dtype, 1e-6, 1e-6)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind,size", [("window", 40), ("block", 40), ("window", 1), ("block", 1), ("block", 64)])
def test_one_loud_key_just_inside_and_just_outside_the_edge(dtype, kind, size):
    """Every key is quiet but one, whose score towers over the rest: a query that sees it returns its value, a query one position
    further -- or in the next block -- must not, whatever the hundreds of other keys say."""
    H, G, D, Dv, m = 2, 1, 16, 8, 300
    keys, vals = 0.05 * rnd(m, G, D, dtype=dtype, seed=1), rnd(m, G, Dv, dtype=dtype, seed=2)
    loud = 130
    if kind == "block":
        loud = (loud // size) * size + size - 1               # the last position of its block
    keys[loud] = 0.0
    keys[loud, 0, 3] = 30.0
    vals[loud] = 5.0
    q = 0.05 * rnd(m, H, D, dtype=dtype, seed=3)
    q[:, :, 3] = 2.0
    if kind == "window":
        inside, outside = loud + size - 1, loud + size
        sees = lambda i, j: O.sees_window(i, j, size)
    else:
        inside, outside = loud, loud + 1
        sees = lambda i, j: O.sees_block(i, j, size)
    qpos = [inside, outside]
    for prompt in (True, False):                              # as rows of a prompt tile, and as single decoded rows
        pos = list(range(inside - 5, outside + 5)) if prompt else qpos
        got = _attend(dtype, q[pos], keys, vals, pos, H, G, 1.0, window=size if kind == "window" else 0, block=size if kind == "block" else 0)
        want = _attend_oracle(q[pos], keys, vals, pos, H, G, 1.0, sees)
        assert rel(got, want) < tol(dtype, 1e-5, 1e-2)
        a, b = got[pos.index(inside)].float(), got[pos.index(outside)].float()
        assert float((a - 5.0).abs().max()) < 0.05 and float((b - 5.0).abs().min()) > 1.0


@pytest.mark.parametrize("dtype", DTYPES)
def test_far_key_among_hundreds_and_a_sink_that_takes_it_all(dtype):
    H, G, D, Dv, m = 2, 2, 32, 16, 900
    keys, vals = 0.05 * rnd(m, G, D, dtype=dtype, seed=1), rnd(m, G, Dv, dtype=dtype, seed=2)
    keys[3, :, 5], vals[3] = 25.0, -4.0
    q = 0.05 * rnd(2, H, D, dtype=dtype, seed=3)
    q[:, :, 5] = 2.0
    for splits in (1, 7):
        got = _attend(dtype, q, keys, vals, [898, 899], H, G, 1.0, splits=splits)
        assert float((got.float() + 4.0).abs().max()) < 0.05
        sink = torch.tensor([80.0, -80.0], device=DEV)        # head 0: the sink outweighs even the loud key; head 1: it is nothing
        got = _attend(dtype, q, keys, vals, [898, 899], H, G, 1.0, sink=sink, splits=splits)
        assert float(got[:, 0].float().abs().max()) < 1e-3 and float((got[:, 1].float() + 4.0).abs().max()) < 0.05


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,D,Dv,cap_", [(2, 16, 24, 12.0), (1, 40, 130, 0.0), (3, 100, 10, 4.0), (2, 200, 70, 7.0)])
def test_matrix_memory_alone(dtype, H, D, Dv, cap_):
    """Two requests of different lengths in one launch, then both continued from their states (one token, then several), on slots
    that held other states before."""
    b = B()
    n = [37, 5]
    T = sum(n) + 1 + 6
    N = 2 * H * D + H * Dv + 2 * H
    P = rnd(T, N, dtype=dtype, seed=1)
    P[:, 2 * H * D + H * Dv + H:] += 3.0                       # forget gates that keep most of the memory
    state = rnd(4, b.mlstm_state_floats(H, D, Dv), seed=2)   # (junk: a request that starts at position 0 starts from zero)
    out = torch.empty(T, H * Dv, dtype=torch.float32, device=DEV)

    def launch(reqs):
        b.mlstm(P, P[:, H * D:], P[:, 2 * H * D:], P[:, 2 * H * D + H * Dv:], P[:, 2 * H * D + H * Dv + H:], N, dev_i32(reqs), len(reqs), state,
                H, D, Dv, D ** -0.5, cap_, out)
    launch([(3, 0, n[0], 0), (1, 0, n[1], n[0])])
    launch([(1, n[1], 1, n[0] + n[1])])
    launch([(3, n[0], 6, n[0] + n[1] + 1)])
    f = lambda t: t.to("cpu", F64)
    P6 = f(P)

    def oracle(rows, st=None):
        x = P6[rows]
        k = len(rows)
        q, kk, v = x[:, :H * D].view(k, H, D) * D ** -0.5, x[:, H * D:2 * H * D].view(k, H, D), x[:, 2 * H * D:2 * H * D + H * Dv].view(k, H, Dv)
        gi, gf = x[:, 2 * H * D + H * Dv:2 * H * D + H * Dv + H], x[:, 2 * H * D + H * Dv + H:]
        return O.matrix_memory(q, kk, v, O.soft_cap(gi, cap_), torch.nn.functional.logsigmoid(O.soft_cap(gf, cap_)), st)
    a0, st0 = oracle(list(range(0, n[0])))
    a1, st1 = oracle(list(range(n[0], n[0] + n[1])))
    a2, _ = oracle([n[0] + n[1]], st1)
    a3, st3 = oracle(list(range(n[0] + n[1] + 1, T)), st0)
    want = torch.cat([a0, a1, a2, a3]).reshape(T, -1)
    assert rel(out, want) < tol(dtype, 2e-5, 2e-5)            # (the recurrence is 32-bit in both; the inputs are exact either way)
    S = state[3].view(H, -1)
    assert rel(S[:, :D * Dv].reshape(H, D, Dv), st3[0]) < 2e-5 and rel(S[:, D * Dv:D * Dv + D], st3[1]) < 2e-5
    assert rel(S[:, -1], st3[2]) < 1e-6


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,D,Dv", [(2, 16, 24), (1, 100, 70), (3, 200, 10)])
def test_matrix_memory_in_segments_equals_token_by_token(dtype, H, D, Dv):
    """Two requests -- one continues from a state, one starts at position 0 on a slot that holds junk -- cut into segments of
    unequal lengths that start from nothing, are chained and run again from their start states: outputs and final states equal
    those of one pass over each request."""
    b = B()
    n, cap_ = [75, 41], 5.0
    T = sum(n)
    N = 2 * H * D + H * Dv + 2 * H
    P = rnd(T, N, dtype=dtype, seed=1)
    P[:, 2 * H * D + H * Dv + H:] += 2.0
    rec = b.mlstm_state_floats(H, D, Dv)
    state0 = rnd(3, rec, seed=2)
    state0.view(3, H, -1)[:, :, -1] = 0.7                      # (a running maximum the first request resumes from)
    cols = (P, P[:, H * D:], P[:, 2 * H * D:], P[:, 2 * H * D + H * Dv:], P[:, 2 * H * D + H * Dv + H:], N)
    reqs = [(2, 9, n[0], 0), (0, 0, n[1], n[0])]
    plain, seg = state0.clone(), state0.clone()
    want = torch.empty(T, H * Dv, dtype=torch.float32, device=DEV)
    b.mlstm(*cols, dev_i32(reqs), 2, plain, H, D, Dv, D ** -0.5, cap_, want)
    cuts = [[16, 1, 30, 28], [40, 1]]
    sa, chains, at = [], [], 0
    for (slot, pos, cnt, row), cs in zip(reqs, cuts):
        chains.append((slot, pos, len(sa), len(cs)))
        for c in cs:
            sa.append((len(sa), 0, c, at))
            at += c
    ns = len(sa)
    sc = [(g, 1, c, r) for g, _, c, r in sa]
    local, start = torch.zeros(ns, rec, device=DEV), torch.zeros(ns, rec, device=DEV)
    fsum = torch.zeros(ns, H, device=DEV)
    got = torch.empty_like(want)
    b.mlstm(*cols, dev_i32(sa), ns, local, H, D, Dv, D ** -0.5, cap_, None, from_nothing=True, log_f_sum=fsum)
    b.mlstm_chain(local, fsum, start, seg, dev_i32(chains), 2, H, D, Dv)
    ends = [-1] * ns
    for slot, _, first, count in chains:
        ends[first + count - 1] = slot
    b.mlstm(*cols, dev_i32(sc), ns, start, H, D, Dv, D ** -0.5, cap_, got, end_slots=dev_i32(ends), end_state=seg)
    assert rel(got, want) < 3e-6
    assert rel(seg[2], plain[2]) < 3e-6 and rel(seg[0], plain[0]) < 3e-6 and torch.equal(seg[1], state0[1])


# =====================================================================================================================================
# the model through its arena
# =====================================================================================================================================
def oracle_logits(s, w, tokens):
    logits, streams, _ = O.forward(s, O.to_f64(w), tokens)
    return logits, streams


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(SHAPES))
def test_whole_prompt_against_the_oracle_layer_by_layer(name, dtype):
    s, w, m = model(name, dtype)
    tokens = toks(75, s.vocab_size, seed=3)
    ar = m.new_arena(1, 80)
    logits, streams = m.forward_rows(ar, [ar.alloc()], [tokens], [list(range(len(tokens)))], return_streams=True)
    want, want_streams = oracle_logits(s, w, tokens)
    for i in range(len(s.layers)):
        assert rel(streams[i], want_streams[i]) < tol(dtype, 2e-5, 0.15), f"layer {i} ({s.layers[i].kind})"
    assert rel(logits, want) < tol(dtype, 3e-5, 0.15)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(SHAPES))
def test_prompt_equals_token_by_token_decoding_and_any_portions(name, dtype):
    s, w, m = model(name, dtype)
    n = 70
    tokens = toks(n, s.vocab_size, seed=5)
    whole = run_alone(m, tokens)
    t = tol(dtype, 1e-5, 8e-2)
    for cuts in ([1] * n, [2] * (n // 2), [33, 2, 2, 17, 16], [16, 16, 16, 22], [1, 69], [40] + [1] * 30):
        assert rel(run_alone(m, tokens, cuts), whole) < t, cuts
    if dtype == torch.float32:
        assert rel(whole, oracle_logits(s, w, tokens)[0]) < 3e-5


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("graphs", [True, False])
def test_unequal_batches_reused_slots_and_states(dtype, graphs):
    """Requests of different lengths step together, some end, newcomers take their slots (keys, values, latents and matrix memories
    of the previous owner still lie there), the rest go on: every request's logits equal those it gets alone."""
    s, w, m = model("mixed", dtype)
    m.use_graphs = graphs
    try:
        prompts = {k: toks(n, s.vocab_size, seed=20 + k) for k, n in enumerate([41, 3, 18, 1, 27])}
        alone = {k: run_alone(m, p) for k, p in prompts.items()}
        ar = m.new_arena(2, 16)
        got = {k: [] for k in prompts}
        slots, at = {}, {k: 0 for k in prompts}

        def step(parts):
            for k in parts:
                if k not in slots:
                    slots[k] = ar.alloc()
            ks = list(parts)
            out = m.forward_rows(ar, [slots[k] for k in ks], [prompts[k][at[k]:at[k] + parts[k]] for k in ks], [list(range(parts[k])) for k in ks])
            o = 0
            for k in ks:
                got[k].append(out[o:o + parts[k]])
                o += parts[k]
                at[k] += parts[k]
                if at[k] == len(prompts[k]):
                    ar.free(slots.pop(k))
        step({0: 30, 1: 2, 2: 10})
        for _ in range(1):
            step({0: 1, 1: 1, 2: 1})                          # request 1 ends here
        step({0: 1, 2: 1, 3: 1})                              # 3 arrives on 1's slot and ends at once
        step({2: 6, 4: 20, 0: 1})                             # 4 arrives on that slot again; 2 ends
        while any(at[k] < len(prompts[k]) for k in (0, 4)):
            step({k: 1 for k in (0, 4) if at[k] < len(prompts[k])})
        t = tol(dtype, 1e-5, 8e-2)
        for k in prompts:
            assert rel(torch.cat(got[k]), alone[k]) < t, k
    finally:
        m.use_graphs = True


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding_through_graphs_across_every_edge_and_a_growing_arena(dtype):
    """A short prompt, then 150 tokens one by one on an arena that starts too small: the decoded positions pass several block and
    window edges, and the planes move (captured steps are recaptured)."""
    s, w, m = model("mixed", dtype)
    tokens = toks(160, s.vocab_size, seed=9)
    want = oracle_logits(s, w, tokens)[0]
    ar = m.new_arena(1, 24)
    slot = ar.alloc()
    out = [m.forward_rows(ar, [slot], [tokens[:10]], [list(range(10))])]
    for t_ in tokens[10:]:
        out.append(m.forward_rows(ar, [slot], [[t_]], [[0]]))
    assert ar.cap >= 160
    assert rel(torch.cat(out), want) < tol(dtype, 3e-5, 8e-2)


@pytest.mark.parametrize("dtype", DTYPES)
def test_far_positions_in_a_long_prompt_and_after_it(dtype):
    """600 tokens through layers whose blocks and windows are wider than the usual test prompt: a prompt tile deep in the sequence
    and decoded tokens after it, against the oracle at those places."""
    s = FivesunShape(vocab_size=90, hidden_size=48, norm_eps=1e-6, embed_scale=6.9, layers=[
        att(4, 2, 16, 8, mask=256, v_mix=True, ff=32), lat(2, 16, 8, 16, 24, mask=300, ff=0, original=256.0), mls(2, 16, 16, ff=0),
        att(4, 2, 16, 8, mask=0, v_mix=True, ff=0)])
    from promptcache_amd.model.fivesun_hip import FivesunHIP
    w = W.make_fivesun_weights(s, seed=4)
    m = FivesunHIP(s, w, device=DEV, dtype=dtype)
    tokens = toks(600, s.vocab_size, seed=2)
    places = [0, 1, 255, 256, 257, 299, 300, 301, 511, 512, 590]
    ar = m.new_arena(1, 640)
    slot = ar.alloc()
    got = [m.forward_rows(ar, [slot], [tokens[:592]], [places])]
    for t_ in tokens[592:]:
        got.append(m.forward_rows(ar, [slot], [[t_]], [[0]]))
    want = oracle_logits(s, w, tokens)[0][places + list(range(592, 600))]
    assert rel(torch.cat(got), want) < tol(dtype, 5e-5, 8e-2)


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
    from promptcache_amd.model import Fivesun
    s = shape_mixed()
    w = W.make_fivesun_weights(s, seed=11)
    lm = Fivesun(shape=s, weights=w, device=DEV, dtype=dtype)
    prompts = [toks(n, s.vocab_size, seed=40 + n) for n in (12, 3, 30)]
    eng = BatchEngine(lm, max_tokens=80)                      # (a budget that does not hold all three at once)
    params = GenerationParameters(temperature=0.0, max_new_tokens=12, stop_token_ids=[])
    got = eng.generate(prompts, params)
    p6 = O.to_f64(w)
    for prompt, out in zip(prompts, got):
        assert len(out) == 12
        seq = list(prompt)
        for k, tok in enumerate(out):                         # every generated token is the oracle's choice given the same history,
            logits = O.forward(s, p6, seq)[0][-1]             # unless the oracle's two best are closer than the format resolves
            best = int(logits.argmax())
            if tok != best:
                assert float(logits[best] - logits[tok]) < (1e-4 if dtype == torch.float32 else 0.15), (k, tok, best)
            seq.append(tok)


def random_shape(rng):
    """Sizes, layer order, masks, rotated parts and constants drawn at random (blended values share one shape, as they must)."""
    width = rng.choice([64, 72, 96, 160, 200, 256])
    G, Dv = rng.choice([1, 2, 3, 4]), rng.choice([16, 24, 40, 64, 72])
    layers = []
    for _ in range(rng.randrange(2, 6)):
        kind, ff = rng.choice(["attention", "latent_attention", "mlstm"]), rng.choice([0, 32, 56, width, 2 * width])
        if kind == "attention":
            vm = rng.random() < 0.6
            g = G if vm else rng.choice([1, 2, 4])
            dim = rng.choice([16, 24, 48, 64, 96, 160])
            layers.append(att(g * rng.choice([1, 2, 3, 4]), g, dim, Dv if vm else rng.choice([16, 40, 128]), mask=rng.choice([0, 1, 7, 32, 50, 100]),
                              rot_dims=rng.choice([dim, dim // 4 * 2, 0]), v_mix=vm, ff=ff, factor=rng.choice([1.0, 2.5]), scale=0.7 * dim ** -0.5))
        elif kind == "latent_attention":
            layers.append(lat(rng.choice([1, 2, 6, 12, 20]), rng.choice([16, 32, 48, 96]), rng.choice([0, 4, 8, 32, 64]), rng.choice([16, 32, 80]),
                              rng.choice([16, 40, 96, 200, 256]), mask=rng.choice([0, 1, 5, 33, 96]), ff=ff, original=rng.choice([0.0, 64.0, 1000.0]),
                              factor=rng.choice([2.0, 8.0]), fast=rng.choice([32.0, 8.0]), slow=rng.choice([1.0, 2.0])))
        else:
            layers.append(mls(rng.choice([1, 2, 4, 8]), rng.choice([8, 16, 48, 100, 192]), rng.choice([8, 16, 48, 130]), cap=rng.choice([0.0, 5.0, 11.0]), ff=ff))
    return FivesunShape(vocab_size=rng.randrange(50, 900), hidden_size=width, norm_eps=rng.choice([1e-5, 1e-6]),
                        embed_scale=rng.choice([1.0, width ** 0.5]), layers=layers)


@pytest.mark.parametrize("seed", range(8))
def test_random_configurations_whole_decoded_and_in_company(seed):
    import random
    from promptcache_amd.model.fivesun_hip import FivesunHIP
    rng = random.Random(1000 + seed)
    s = FivesunShape.from_config(json.loads(json.dumps(random_shape(rng).to_config())))
    w = W.make_fivesun_weights(s, seed=seed)
    n = rng.randrange(90, 260)
    a, b_ = toks(n, s.vocab_size, seed), toks(rng.randrange(1, 70), s.vocab_size, seed + 1)
    want_a, want_b = oracle_logits(s, w, a)[0], oracle_logits(s, w, b_)[0]
    for dtype in DTYPES:
        m = FivesunHIP(s, w, device=DEV, dtype=dtype)
        t = tol(dtype, 5e-5, 0.15)
        assert rel(run_alone(m, a), want_a) < t, s.to_config()
        ar = m.new_arena(1, 16)
        sa, sb = ar.alloc(), ar.alloc()
        cut = n - 20
        out = [m.forward_rows(ar, [sb, sa], [b_, a[:cut]], [list(range(len(b_))), list(range(cut))])]
        out += [m.forward_rows(ar, [sa], [[t_]], [[0]]) for t_ in a[cut:]]
        got = torch.cat(out)
        assert rel(got[len(b_):], want_a) < t and rel(got[:len(b_)], want_b) < t, s.to_config()


def test_single_request_engine_and_the_adapters_call():
    """GenerationEngine drives the model through the adapters' ``model(input_ids, past_key_values)`` call; a padded batch through
    that call gives each row its own logits."""
    from promptcache_amd import BatchEngine, GenerationEngine, GenerationParameters
    from promptcache_amd.model import Fivesun
    s = shape_mixed()
    w = W.make_fivesun_weights(s, seed=21)
    lm = Fivesun(shape=s, weights=w, device=DEV, dtype=torch.float32)
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
    assert rel(res.logits[0], O.forward(s, p6, prompts[0])[0]) < 3e-5 and rel(res.logits[1, :5], O.forward(s, p6, prompts[1])[0]) < 3e-5
    assert int(res.logits[0, 12].argmax()) == want[0][0] and int(res.logits[1, 4].argmax()) == want[1][0]


def test_checkpoint_directory_command_line_and_trace_runner(tmp_path):
    """config.json + model.safetensors written from a shape, found by the registry, and replayed by bin/trace_run in both formats."""
    from safetensors.torch import save_file
    from promptcache_amd.model import load_language_model
    s = shape_odd()
    w = W.make_fivesun_weights(s, seed=3)
    d = tmp_path / "ckpt"
    d.mkdir()
    (d / "config.json").write_text(json.dumps(s.to_config()))
    save_file({k: v.contiguous() for k, v in w.items()}, str(d / "model.safetensors"))
    lm = load_language_model(str(d), dtype=torch.float32)
    assert type(lm).__name__ == "Fivesun" and lm.hf_model.config.to_config() == s.to_config()
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
