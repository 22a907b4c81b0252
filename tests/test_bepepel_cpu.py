"""Bepepel without a GPU: the configuration reader and writer, the checkpoint reader, the registry, the host-side frequency table
against the oracle's, and the float64 oracle (``oracle/bepepel_oracle.py``) against itself -- a prompt at once, token by token,
and in portions must agree, which pins how it carries keys, convolution inputs and matrix states from step to step."""
import ctypes
import json
import math
import os

import pytest
import torch

from oracle import bepepel_oracle as O
from promptcache_amd.model import weights as W
from promptcache_amd.model.config import BepepelAttention, BepepelLayer, BepepelSSD, BepepelShape, architecture_of

F64 = torch.float64


def small_shape():
    left = BepepelAttention(heads=4, kv_heads=2, dim=12, vdim=10, scale=0.3, conv=3, window=9, keep_first=2, rot_base=900.0, rot_dims=8,
                            rot_scaling=(4.0, 1.0, 3.0, 40.0))
    right = BepepelSSD(heads=4, vdim=6, state=5, groups=2, norm_groups=3, conv=4)
    return BepepelShape(vocab_size=61, hidden_size=40, norm_eps=1e-5, residual_mult=0.4, logit_scale=1.7, layers=[
        BepepelLayer("gla", heads=3, dim=6, vdim=10, tau=5.0, a_rank=4, ff_kind="moe", experts=5, top=2, expert_ff=12, shared_ff=9),
        BepepelLayer("parallel", left=left, right=right, left_scale=1.3, right_scale=0.6, ff_kind="dense", ff=24),
        BepepelLayer("gla", heads=2, dim=8, vdim=4, tau=1.0, a_rank=3),
    ])


def toks(n, vocab, seed=0):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def test_configuration_round_trip_and_what_is_left_out():
    s = small_shape()
    c = json.loads(json.dumps(s.to_config()))
    assert BepepelShape.from_config(c).to_config() == c
    # what a configuration leaves out does not exist: no window, no kept tokens, no rotation, no convolution, no feed-forward
    c["layers"][1]["mixer"]["left"] = {"heads": 2, "dim": 8, "scale": 0.5}
    c["layers"][1]["mlp"] = None
    t = BepepelShape.from_config(c).layers[1]
    a = t.left
    assert (a.kv_heads, a.vdim, a.window, a.keep_first, a.rot_dims, a.conv, a.rot_scaling, t.ff_kind) == (2, 8, 0, 0, 0, 0, None, "")
    with pytest.raises(ValueError):
        BepepelShape.from_config(dict(c, architecture="Other"))
    c["layers"][0]["type"] = "unknown"
    with pytest.raises(ValueError):
        BepepelShape.from_config(c)


def test_checkpoint_directory_reader_and_registry(tmp_path):
    from safetensors.torch import save_file
    s = small_shape()
    w = W.make_bepepel_weights(s, seed=1)
    assert set(w) == set(W.bepepel_weight_shapes(s)) and all(tuple(w[k].shape) == tuple(v) for k, v in W.bepepel_weight_shapes(s).items())
    (tmp_path / "config.json").write_text(json.dumps(s.to_config()))
    save_file({k: v.contiguous() for k, v in w.items()}, str(tmp_path / "model.safetensors"))
    assert architecture_of(str(tmp_path)) == "bepepel"
    s2 = BepepelShape.from_dir(str(tmp_path))
    for l in s2.layers:
        l.a_rank = 0                                         # the rank of the decay projection is read off the tensor
    got = W.load_bepepel_safetensors(str(tmp_path), s2)
    assert [l.a_rank for l in s2.layers] == [4, 0, 3] and all(torch.equal(got[k], w[k]) for k in w)
    bad = dict(w)
    bad["l1.mix.right.in"] = bad["l1.mix.right.in"][:-1]
    save_file({k: v.contiguous() for k, v in bad.items()}, str(tmp_path / "model.safetensors"))
    with pytest.raises(ValueError):
        W.load_bepepel_safetensors(str(tmp_path), s2)


@pytest.mark.parametrize("scaling", [None, (8.0, 1.0, 4.0, 64.0), (2.0, 2.0, 16.0, 1000.0), (4.0, 1.0, 4.0, 1e9)])
@pytest.mark.parametrize("base,dims", [(10000.0, 32), (250.0, 6), (1e6, 64)])
def test_frequency_table_of_the_model_is_the_oracles(scaling, base, dims):
    from promptcache_amd.model.bepepel_hip import scaled_rotary_frequencies
    got = torch.from_numpy(scaled_rotary_frequencies(base, dims, scaling))
    want = O.rotary_frequencies(base, dims, scaling)
    assert got.dtype == F64 and float(((got - want) / want).abs().max()) < 1e-14
    if scaling and scaling[3] < 1e8:
        plain = O.rotary_frequencies(base, dims)
        assert float((want / plain).min()) >= 1.0 / scaling[0] - 1e-12 and float((want / plain).max()) <= 1.0 + 1e-12


def test_visibility_rule():
    assert O.sees(50, 50, 8, 2) and O.sees(50, 43, 8, 2) and not O.sees(50, 42, 8, 2)
    assert O.sees(50, 1, 8, 2) and not O.sees(50, 2, 8, 2) and not O.sees(3, 4, 8, 2)
    assert O.sees(1000, 0, 0, 0) and all(O.sees(5, j, 100, 0) for j in range(6))


def test_short_convolution_carries_its_last_inputs():
    g = torch.Generator().manual_seed(3)
    u, w, b = torch.randn(11, 5, generator=g, dtype=F64), torch.randn(5, 4, generator=g, dtype=F64), torch.randn(5, generator=g, dtype=F64)
    whole, last = O.short_conv(u, w, b, torch.zeros(3, 5, dtype=F64))
    assert torch.allclose(whole[0], w[:, 3] * u[0] + b) and torch.allclose(whole[2], w[:, 1] * u[0] + w[:, 2] * u[1] + w[:, 3] * u[2] + b)
    before, parts = torch.zeros(3, 5, dtype=F64), []
    for lo, hi in ((0, 1), (1, 2), (2, 7), (7, 11)):
        o, before = O.short_conv(u[lo:hi], w, b, before)
        parts.append(o)
    assert torch.allclose(torch.cat(parts), whole) and torch.equal(before, last) and torch.equal(last, u[8:])


def test_router_takes_the_largest_logits_and_their_softmax():
    g = torch.Generator().manual_seed(5)
    h = torch.randn(7, 6, generator=g, dtype=F64)
    p = {"r.router": torch.randn(9, 6, generator=g, dtype=F64), "r.router.b": torch.randn(9, generator=g, dtype=F64)}
    idx, w = O.route(h, p, "r.", 3)
    z = h @ p["r.router"].T + p["r.router.b"]
    for t in range(7):
        order = sorted(range(9), key=lambda e: -float(z[t, e]))[:3]
        assert idx[t].tolist() == order
        e = torch.exp(z[t, order])
        assert torch.allclose(w[t], e / e.sum())


def test_matrix_state_steps_unrolled():
    g = torch.Generator().manual_seed(7)
    q, k, v = (torch.randn(4, 3, generator=g, dtype=F64) for _ in range(3))
    v = v[:, :2]
    a = torch.rand(4, 3, generator=g, dtype=F64)
    out, S = O.matrix_state_steps(q, k, v, a, torch.zeros(3, 2, dtype=F64))
    # o_2 = sum_j (q_2 * prod_{j < i <= 2} a_i * k_j) v_j
    want = sum(((q[2] * a[j + 1:3].prod(dim=0) * k[j]).sum()) * v[j] for j in range(3))
    assert torch.allclose(out[2], want)
    again, S2 = O.matrix_state_steps(q[2:], k[2:], v[2:], a[2:], O.matrix_state_steps(q[:2], k[:2], v[:2], a[:2], torch.zeros(3, 2, dtype=F64))[1])
    assert torch.allclose(again, out[2:]) and torch.allclose(S2, S)


@pytest.mark.parametrize("seed", [0, 1])
def test_oracle_prompt_equals_token_by_token_and_portions(seed):
    s = small_shape()
    p = O.to_f64(W.make_bepepel_weights(s, seed=seed))
    t = toks(27, s.vocab_size, seed)
    whole = O.forward(s, p, t)
    assert whole.shape == (27, s.vocab_size) and bool(torch.isfinite(whole).all())
    for cuts in ([1] * 27, [2, 2, 5, 1, 17], [26, 1]):
        assert float((O.forward_in_portions(s, p, t, cuts) - whole).abs().max()) < 1e-10
    # the window matters, and so do the kept first tokens and the residual factor
    import copy
    for change in ("window", "keep_first"):
        s2 = copy.deepcopy(s)
        setattr(s2.layers[1].left, change, 0)
        assert float((O.forward(s2, p, t)[-1] - whole[-1]).abs().max()) > 1e-6
    s2 = copy.deepcopy(s)
    s2.residual_mult = 0.5
    assert float((O.forward(s2, p, t)[-1] - whole[-1]).abs().max()) > 1e-4
    assert math.isclose(float(whole[3, 5] / s.logit_scale * 2.0), float(O.forward(dataclass_with(s, logit_scale=2.0), p, t)[3, 5]), rel_tol=1e-12)


def dataclass_with(s, **kw):
    import copy
    s2 = copy.deepcopy(s)
    for k, v in kw.items():
        setattr(s2, k, v)
    return s2


def test_blocks_reject_bad_arguments_on_the_host():
    """The library checks its arguments before it launches anything, so these calls need no GPU."""
    from promptcache_amd import _blocks
    assert os.path.exists(_blocks.lib_path()), "run __graft_entry__.build() first"
    lb = _blocks.load(build_missing=False)
    g = _blocks.GlaArgs(ctypes.sizeof(_blocks.GlaArgs), 0, None, None, None, 600, 600, 16, None, 600, 300, None, None, 0, None, 1, None, 10 ** 6,
                        2, 2, 300, 8, 1.0, None, 16, None)
    assert lb.pcb_gla(ctypes.byref(g), None) == -2001 and b"256 key columns" in lb.pcb_last_error_string()
    g.dim, g.dcols = 64, 3                                    # a decay per key column, or one per head: nothing between
    assert lb.pcb_gla(ctypes.byref(g), None) == -2001 and b"bad sizes" in lb.pcb_last_error_string()
    g.dcols, g.Hk = 64, 3                                     # value heads must divide over the key heads
    assert lb.pcb_gla(ctypes.byref(g), None) == -2001
    g.Hk = 1
    assert lb.pcb_gla(ctypes.byref(g), None) == -2001 and b"null pointer" in lb.pcb_last_error_string()
    g.struct_bytes -= 8
    assert lb.pcb_gla(ctypes.byref(g), None) == -2001 and b"struct size" in lb.pcb_last_error_string()
    # a skip path without its weights
    assert lb.pcb_gated_norm(None, 12, None, None, 0, None, 12, 0, 1e-6, 2, 12, 4, 1, 1, 12, None, 4, None) == -2001 and \
        b"skip" in lb.pcb_last_error_string()
