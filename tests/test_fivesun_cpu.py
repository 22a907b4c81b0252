"""CPU-side checks of the Fivesun integration: configuration reader, tensor naming, checkpoint directories, the arena's planes and
states for this design, the blocks library's new argument structures, the frequency tables the model hands to its kernels, and
properties of the plain oracle itself (each mechanism made visible by inputs built for it)."""
import ctypes
import json
import math
import os
import subprocess

import pytest
import torch

from oracle import fivesun_oracle as O
from promptcache_amd.model import weights as W
from promptcache_amd.model.config import FivesunLayer, FivesunShape, architecture_of

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
F = torch.float64


def small_shape():
    return FivesunShape(vocab_size=60, hidden_size=24, norm_eps=1e-5, embed_scale=3.5, layers=[
        FivesunLayer("mlstm", heads=2, kv_heads=2, dim=6, vdim=8, gate_cap=4.0, ff=16),
        FivesunLayer("attention", heads=4, kv_heads=2, dim=8, vdim=6, scale=0.3, mask=5, rot_base=100.0, rot_dims=4, rot_factor=2.0, v_mix=True),
        FivesunLayer("latent_attention", heads=3, kv_heads=1, dim=6, vdim=4, kv_rank=10, rot_dim=4, rot_dims=4, scale=0.25, mask=4,
                     rot_base=50.0, rot_factor=4.0, yarn_original=16.0, yarn_fast=4.0, yarn_slow=1.0, ff=12),
        FivesunLayer("attention", heads=2, kv_heads=2, dim=8, vdim=6, scale=0.4, mask=0, rot_base=100.0, rot_dims=8, rot_factor=1.0, v_mix=True, ff=8),
    ])


def rnd(*shape, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=F)


# ---- configuration and tensors -------------------------------------------------------------------------------------------------
def test_config_round_trip_and_every_branch(tmp_path):
    s = small_shape()
    c = s.to_config()
    assert c["architecture"] == "Fivesun" and c["layers"][1]["mlp"] is None and c["layers"][3]["mixer"].get("mask") is None
    assert c["layers"][2]["mixer"]["rot"]["scaling"]["original"] == 16.0 and c["embedding"]["scale"] == 3.5
    back = FivesunShape.from_config(json.loads(json.dumps(c)))
    assert back.to_config() == c and back.first_v_mix == 1 and [l.kind for l in back.layers] == [l.kind for l in s.layers]
    (tmp_path / "config.json").write_text(json.dumps(c))
    assert architecture_of(str(tmp_path)) == "fivesun"
    # what a configuration leaves out does not exist: no mask, no scaling, key heads = query heads, value size = key size
    lean = {"architecture": "Fivesun", "vocab": 9, "width": 8, "layers": [
        {"type": "attention", "mixer": {"heads": 2, "dim": 4, "rot": {"base": 10.0, "dims": 2}}, "mlp": None}]}
    l = FivesunShape.from_config(lean).layers[0]
    assert (l.kv_heads, l.vdim, l.mask, l.rot_factor, l.v_mix, l.ff, l.rot_dims) == (2, 4, 0, 1.0, False, 0, 2)
    for bad in ({"type": "conv"}, {"type": "attention", "mixer": {"heads": 3, "kv_heads": 2, "dim": 4}},
                {"type": "attention", "mixer": {"heads": 2, "dim": 4, "rot": {"dims": 3}}},
                {"type": "latent_attention", "mixer": {"heads": 2, "dim": 4, "kv_rank": 4, "rot_dim": 2, "rot": {"dims": 4}}},
                {"type": "mlstm", "mixer": {"heads": 2, "dim": 4}, "mlp": {"kind": "moe", "ff": 4}}):
        with pytest.raises(ValueError):
            FivesunShape.from_config(dict(lean, layers=[bad]))
    # blended values must have the first blending layer's shape
    two = [{"type": "attention", "mixer": {"heads": 2, "dim": 4, "v_mix": True}}, {"type": "attention", "mixer": {"heads": 2, "dim": 4, "vdim": 6, "v_mix": True}}]
    with pytest.raises(ValueError):
        FivesunShape.from_config(dict(lean, layers=two))


def test_tensor_names_and_checkpoint_directory(tmp_path):
    from safetensors.torch import save_file
    s = small_shape()
    shapes = W.fivesun_weight_shapes(s)
    assert shapes["l1.mix.sink"] == (4,) and shapes["l1.mix.g"] == (4, 24) and shapes["l1.mix.vmix"] == () and "l1.norm2" not in shapes
    assert shapes["l2.mix.dkv"] == (14, 24) and shapes["l2.mix.uk"] == (18, 10) and shapes["l2.mix.q"] == (30, 24)
    assert shapes["l0.mix.i"] == (2, 24) and shapes["l0.mix.norm"] == (16,) and shapes["l0.mlp.down.b"] == (24,) and shapes["l0.rg2"] == (24, 24)
    w = W.make_fivesun_weights(s, seed=2)
    assert set(w) == set(shapes) and all(tuple(w[k].shape) == tuple(v) and w[k].dtype == torch.bfloat16 for k, v in shapes.items())
    assert 0.0 < float(w["l3.mix.vmix"]) < 1.0 and float(w["l1.mix.sink"].float().abs().min()) > 0.0
    (tmp_path / "config.json").write_text(json.dumps(s.to_config()))
    save_file({k: v.contiguous() for k, v in w.items()}, str(tmp_path / "model.safetensors"))
    back = W.load_fivesun_safetensors(str(tmp_path), FivesunShape.from_dir(str(tmp_path)))
    assert all(torch.equal(back[k], w[k]) for k in w)
    w2 = dict(w)
    w2["l2.mix.uv"] = w["l2.mix.uv"][:, :-1].contiguous()
    save_file({k: v.contiguous() for k, v in w2.items()}, str(tmp_path / "model.safetensors"))
    with pytest.raises(ValueError):
        W.load_fivesun_safetensors(str(tmp_path), s)
    del w2["l2.mix.uv"]
    save_file({k: v.contiguous() for k, v in w2.items()}, str(tmp_path / "model.safetensors"))
    with pytest.raises(KeyError):
        W.load_fivesun_safetensors(str(tmp_path), s)


def test_arena_serial_numbers_never_repeat():
    from promptcache_amd.model.kv_arena import SlotArena
    seen = set()
    for _ in range(5):
        ar = SlotArena([(1, 4)], 1, 4, "cpu", torch.float32)
        assert ar.serial not in seen
        seen.add(ar.serial)
        del ar


def test_frequency_tables_follow_the_oracle():
    from promptcache_amd.model.fivesun_hip import rotary_frequencies
    fr, mag = rotary_frequencies(30000.0, 12, 3.0)
    want, wm = O.plain_frequencies(30000.0, 12, 3.0)
    assert mag == wm == 1.0 and torch.allclose(torch.from_numpy(fr), want, rtol=1e-14)
    for args in ((70000.0, 32, 3.0, 1024.0, 16.0, 2.0), (10000.0, 8, 4.0, 64.0, 8.0, 1.0), (100.0, 4, 8.0, 16.0, 2.0, 0.5)):
        fr, mag = rotary_frequencies(*args)
        want, wm = O.yarn_frequencies(*args)
        assert abs(mag - wm) < 1e-15 and torch.allclose(torch.from_numpy(fr), want, rtol=1e-14)


# ---- the blocks library's argument structures --------------------------------------------------------------------------------------
def test_blocks_struct_layouts_match_the_header(tmp_path):
    from promptcache_amd import _blocks
    structs = (("pcb_post_norm_args", _blocks.PostNormArgs), ("pcb_head_prep_seg", _blocks.HeadPrepSeg), ("pcb_head_prep_args", _blocks.HeadPrepArgs),
               ("pcb_mlstm_args", _blocks.MlstmArgs), ("pcb_attn_softmax_args", _blocks.AttnSoftmaxArgs), ("pcb_linear_args", _blocks.LinearArgs))
    body = ['#include <stdio.h>', '#include <stddef.h>', f'#include "{ROOT}/include/promptcache_blocks.h"', 'int main(void) {']
    for st, cls in structs:
        body.append(f'  printf("{st} %zu\\n", sizeof({st}));')
        for f, _ in cls._fields_:
            body.append(f'  printf("{st}.{f} %zu\\n", offsetof({st}, {f}));')
    body += ['  return 0;', '}']
    src = tmp_path / "layout.c"
    src.write_text("\n".join(body))
    exe = tmp_path / "layout"
    subprocess.check_call(["gcc", "-std=c99", "-Wall", "-Werror", str(src), "-o", str(exe)])
    got = dict(line.rsplit(" ", 1) for line in subprocess.check_output([str(exe)], text=True).strip().splitlines())
    for st, cls in structs:
        assert int(got[st]) == ctypes.sizeof(cls), st
        for name, _ in cls._fields_:
            assert int(got[f"{st}.{name}"]) == getattr(cls, name).offset, (st, name)


def test_blocks_reject_bad_arguments_on_the_host():
    from promptcache_amd import _blocks
    assert os.path.exists(_blocks.lib_path()), "run __graft_entry__.build() first"
    lb = _blocks.load(build_missing=False)
    a = _blocks.PostNormArgs(ctypes.sizeof(_blocks.PostNormArgs), 0, None, None, None, 0, None, None, None, None, None, 1e-6, 2, 20000)
    assert lb.pcb_post_norm(ctypes.byref(a), None) == -2001 and b"width" in lb.pcb_last_error_string()
    a.width = 8
    assert lb.pcb_post_norm(ctypes.byref(a), None) == -2001 and b"null pointer" in lb.pcb_last_error_string()
    a.struct_bytes -= 4
    assert lb.pcb_post_norm(ctypes.byref(a), None) == -2001 and b"struct size" in lb.pcb_last_error_string()
    m = _blocks.MlstmArgs(ctypes.sizeof(_blocks.MlstmArgs), 0, None, None, None, None, None, 600, 600, 16, 2, 2, None, 1, None, 10 ** 6, 2, 300, 8,
                          1.0, 0.0, None, 16)
    assert lb.pcb_mlstm(ctypes.byref(m), None) == -2001 and b"256 key columns" in lb.pcb_last_error_string()
    h = _blocks.HeadPrepArgs(ctypes.sizeof(_blocks.HeadPrepArgs), 0, 0, 1, None, None, 1.0, 1e-6)
    h.seg[0] = _blocks.HeadPrepSeg(None, 8, 8, 1, 8, 0, None, None, None, 0, None, 0, 3, 4, None, 8, None, 8, 1)
    assert lb.pcb_head_prep(ctypes.byref(h), None) == -2001 and b"pairs" in lb.pcb_last_error_string()      # an odd first rotated column
    assert lb.pcb_gated_norm(None, 12, None, None, 0, None, 12, 0, 1e-6, 2, 12, 5, 0, None, 0, None, 0, None) == -2001 and b"divide" in lb.pcb_last_error_string()
    assert lb.pcb_embed_scaled_rows(None, 0, None, 2.0, None, 3, 8, 10, None) == -2001 and b"null pointer" in lb.pcb_last_error_string()


# ---- the oracle's own properties ---------------------------------------------------------------------------------------------------
def test_oracle_forward_does_not_look_ahead_carries_its_state_and_layers_matter():
    s = small_shape()
    p = O.to_f64(W.make_fivesun_weights(s, seed=5))
    t = torch.randint(0, s.vocab_size, (19,), generator=torch.Generator().manual_seed(1)).tolist()
    full, streams, _ = O.forward(s, p, t)
    assert torch.allclose(O.forward(s, p, t[:9])[0], full[:9], atol=1e-10) and streams.shape == (4, 19, 24)
    a, _, carry = O.forward(s, p, t[:11])
    b, _, carry = O.forward(s, p, t[11:12], pos0=11, carry=carry)
    c, _, _ = O.forward(s, p, t[12:], pos0=12, carry=carry)
    assert torch.allclose(torch.cat([a, b, c]), full, atol=1e-9)
    for i in range(1, 4):
        assert float((streams[i] - streams[i - 1]).abs().max()) > 1e-3
    # the blend reaches layer 3 from layer 1: another blend weight changes the result, and so do layer 1's own values
    p2 = dict(p)
    p2["l3.mix.vmix"] = p["l3.mix.vmix"] + 0.2
    assert float((O.forward(s, p2, t)[0] - full).abs().max()) > 1e-4
    p2 = dict(p)
    p2["l1.mix.vmix"] = p["l1.mix.vmix"] + 0.2              # (the first blending layer's own weight is not used)
    assert torch.equal(O.forward(s, p2, t)[0], full)


def test_oracle_rotation_depends_on_distance_only_and_leaves_the_rest():
    fr, mag = O.plain_frequencies(100.0, 4, 2.0)
    assert torch.allclose(fr, torch.tensor([0.5, 0.05], dtype=F))
    q, k = rnd(1, 6, seed=1), rnd(1, 6, seed=2)
    def score(i, j):
        return float(O.rotate_pairs(q, torch.tensor([i]), fr) @ O.rotate_pairs(k, torch.tensor([j]), fr).T)
    assert abs(score(9, 4) - score(105, 100)) < 1e-12 and abs(score(9, 4) - score(9, 5)) > 1e-6
    r = O.rotate_pairs(q, torch.tensor([3]), fr, 1.5)
    assert torch.equal(r[:, 4:], q[:, 4:])                                                       # columns past the rotated ones
    a = 3 * 0.5
    assert abs(float(r[0, 0]) - 1.5 * (float(q[0, 0]) * math.cos(a) - float(q[0, 1]) * math.sin(a))) < 1e-12    # neighbours pair up
    assert abs(float(r[0, 1]) - 1.5 * (float(q[0, 1]) * math.cos(a) + float(q[0, 0]) * math.sin(a))) < 1e-12


def test_oracle_yarn_keeps_fast_pairs_and_slows_the_slow_ones():
    base, dims, factor, original = 10000.0, 16, 4.0, 256.0
    fr, mag = O.yarn_frequencies(base, dims, factor, original, 32.0, 1.0)
    plain, _ = O.plain_frequencies(base, dims)
    turns = original * plain / (2 * math.pi)
    assert abs(mag - (0.1 * math.log(4.0) + 1.0)) < 1e-15
    assert float(turns[0]) > 32 and fr[0] == plain[0]                                           # turns often: untouched
    assert float(turns[-1]) < 1 and abs(float(fr[-1]) - float(plain[-1]) / 4.0) < 1e-18         # hardly turns: divided by the factor
    mid = [i for i in range(8) if plain[i] / 4.0 < fr[i] < plain[i]]
    assert mid and all(fr[i] > fr[i + 1] for i in range(7))


def test_oracle_masks_sinks_and_grouped_heads():
    assert [j for j in range(12) if O.sees_block(9, j, 4)] == [8, 9] and [j for j in range(12) if O.sees_block(8, j, 4)] == [8]
    assert [j for j in range(12) if O.sees_window(9, j, 4)] == [6, 7, 8, 9] and [j for j in range(5) if O.sees_block(3, j, 0)] == [0, 1, 2, 3]
    m, D, Dv = 7, 5, 3
    q, k, v = rnd(m, D, seed=1), rnd(m, D, seed=2), rnd(m, Dv, seed=3)
    plain = O.softmax_attention(q, k, v, list(range(m)), lambda i, j: j <= i, 0.4)
    assert torch.allclose(plain[0], v[0], atol=1e-12)
    sunk = O.softmax_attention(q, k, v, list(range(m)), lambda i, j: j <= i, 0.4, sink=torch.tensor(0.7, dtype=F))
    s0 = float(q[0] @ k[0]) * 0.4
    assert torch.allclose(sunk[0], v[0] * math.exp(s0) / (math.exp(s0) + math.exp(0.7)), atol=1e-12)     # the sink is not scaled, counts once
    far = O.softmax_attention(q, k, v, list(range(m)), lambda i, j: j <= i, 0.4, sink=torch.tensor(-50.0, dtype=F))
    assert torch.allclose(far, plain, atol=1e-12)


def test_oracle_latent_attention_equals_its_folded_form():
    """Keys and values rebuilt from the latent per head (how the oracle writes it) against up-projections folded into the query
    and the output (how the product computes it)."""
    lay = small_shape().layers[2]
    H, D, R, Dv, C = lay.heads, lay.dim, lay.rot_dim, lay.vdim, lay.kv_rank
    Wd = 24
    p = {"m.q": rnd(H * (D + R), Wd, seed=1), "m.dkv": rnd(C + R, Wd, seed=2), "m.dkv.norm": 1 + 0.1 * rnd(C, seed=3), "m.uk": rnd(H * D, C, seed=4),
         "m.uv": rnd(H * Dv, C, seed=5), "m.g": rnd(H * Dv, Wd, seed=6), "m.o": rnd(Wd, H * Dv, seed=7)}
    h = rnd(9, Wd, seed=8)
    y, (c, kr) = O.latent_mixer(h, p, "m.", lay, 1e-5, 0, None)
    fr, mag = O.yarn_frequencies(lay.rot_base, R, lay.rot_factor, lay.yarn_original, lay.yarn_fast, lay.yarn_slow)
    pos = torch.arange(9)
    q = (h @ p["m.q"].T).view(9, H, D + R)
    out = torch.zeros(9, H, Dv, dtype=F)
    for hd in range(H):
        uk, uv = p["m.uk"][hd * D:(hd + 1) * D], p["m.uv"][hd * Dv:(hd + 1) * Dv]
        qq = torch.cat([q[:, hd, :D] @ uk, O.rotate_pairs(q[:, hd, D:], pos, fr, mag)], dim=1)
        o = O.softmax_attention(qq, torch.cat([c, kr], dim=1), c, pos.tolist(), lambda i, j: O.sees_window(i, j, lay.mask), lay.scale)
        out[:, hd] = o @ uv.T
    folded = (out.reshape(9, -1) * torch.sigmoid(h @ p["m.g"].T)) @ p["m.o"].T
    assert torch.allclose(folded, y, atol=1e-10)


def test_oracle_matrix_memory_in_closed_form():
    """With the running maximum taken out, token t's numerator is sum_j exp(F_t - F_j + i_j) (q_t . k_j) v_j, F the running sum of
    the log forget gates; the maximum only rescales numerator and denominator alike, except through the floor exp(-m)."""
    n, H, D, Dv = 8, 1, 3, 2
    q, k, v = rnd(n, H, D, seed=1), rnd(n, H, D, seed=2), rnd(n, H, Dv, seed=3)
    li, lf = rnd(n, H, seed=4), -rnd(n, H, seed=5).abs()
    out, (S, nv, m) = O.matrix_memory(q, k, v, li, lf)
    Fs = torch.cumsum(lf[:, 0], 0)
    for t in (0, 3, 7):
        wts = torch.stack([torch.exp(Fs[t] - Fs[j] + li[j, 0]) * (q[t, 0] @ k[j, 0]) for j in range(t + 1)])
        num = (wts.unsqueeze(1) * v[:t + 1, 0]).sum(0)
        mt = 0.0                                              # the running maximum, starting from 0
        for j in range(t + 1):
            mt = max(float(lf[j, 0]) + mt, float(li[j, 0]))
        den = max(abs(float(wts.sum())), 1.0) * math.exp(-mt) + 1e-6    # (both sides of the max carry exp(-m): |n.q| e^-m vs e^-m)
        assert torch.allclose(out[t, 0], num * math.exp(-mt) / den, atol=1e-10), t
    a, st = O.matrix_memory(q[:5], k[:5], v[:5], li[:5], lf[:5])
    b, st2 = O.matrix_memory(q[5:], k[5:], v[5:], li[5:], lf[5:], st)
    assert torch.allclose(torch.cat([a, b]), out, atol=1e-12) and torch.allclose(st2[0], S, atol=1e-12) and torch.allclose(st2[2], m, atol=1e-12)
    assert O.soft_cap(torch.tensor(100.0, dtype=F), 9.0) < 9.0 and O.soft_cap(torch.tensor(3.0, dtype=F), 0.0) == 3.0


def test_oracle_gated_sublayer_and_feed_forward():
    Wd, ff = 6, 5
    p = {"l.norm2": 1 + 0.1 * rnd(Wd, seed=1), "l.norm2b": 1 + 0.1 * rnd(Wd, seed=2), "l.rg2": rnd(Wd, Wd, seed=3), "l.rg2.b": rnd(Wd, seed=4),
         "m.gate": rnd(ff, Wd, seed=5), "m.gate.b": rnd(ff, seed=6), "m.up": rnd(ff, Wd, seed=7), "m.up.b": rnd(ff, seed=8),
         "m.down": rnd(Wd, ff, seed=9), "m.down.b": rnd(Wd, seed=10)}
    x = rnd(4, Wd, seed=11)
    h = O.unit_rms(x, 1e-5) * p["l.norm2"]
    y = (torch.relu(h @ p["m.gate"].T + p["m.gate.b"]) * (h @ p["m.up"].T + p["m.up.b"])) @ p["m.down"].T + p["m.down.b"]
    assert torch.allclose(O.dense_ff(h, p, "m."), y, atol=1e-12)
    t = y * torch.sigmoid(h @ p["l.rg2"].T + p["l.rg2.b"])
    want = x + t / torch.sqrt(t.pow(2).mean(-1, keepdim=True) + 1e-5) * p["l.norm2b"]
    assert torch.allclose(O.gated_sublayer(x, lambda hh: O.dense_ff(hh, p, "m."), p, "l.", "2", 1e-5), want, atol=1e-12)
    z = torch.tensor([-1.0, 0.5, 2.0], dtype=F)
    assert torch.allclose(O.activation("gelu_tanh")(z), 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3))))
