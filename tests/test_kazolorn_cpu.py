"""CPU-side checks of the Kazolorn integration: configuration reader, tensor naming, the slot arena's bookkeeping, the batch
engine's scheduling (on a recording stand-in model), the blocks library's ABI, and properties of the plain oracle itself."""
import ctypes
import os
import re
import subprocess

import pytest
import torch

from oracle import kazolorn_oracle as O
from promptcache_amd.model import weights as W
from promptcache_amd.model.config import KazolornLayer, KazolornShape
from promptcache_amd.model.kv_arena import SlotArena

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def mixed_shape():
    return KazolornShape(vocab_size=96, hidden_size=48, norm_eps=1e-5, layers=[
        KazolornLayer(heads=4, kv_heads=4, dim=12, scale=0.3, window=7, mlp_kind="dense", ff=40),
        KazolornLayer(heads=6, kv_heads=2, dim=8, scale=0.4, window=0, mlp_kind="moe", ff=24, experts=5, top=2),
        KazolornLayer(heads=2, kv_heads=1, dim=16, scale=0.25, window=3, mlp_kind=None),
    ])


# ---- configuration and tensors -------------------------------------------------------------------------------------------------
def test_config_round_trip_and_every_branch():
    s = mixed_shape()
    c = s.to_config()
    assert c["layers"][2]["mlp"] is None and "mask" not in c["layers"][1]["mixer"]
    back = KazolornShape.from_config(c)
    assert back.layers == s.layers and back.vocab_size == 96 and back.hidden_size == 48 and back.norm_eps == 1e-5


@pytest.mark.parametrize("edit, msg", [
    (lambda c: c.update(architecture="Other"), "not Kazolorn"),
    (lambda c: c["layers"][0].update(type="conv"), "unknown mixer"),
    (lambda c: c["layers"][0]["mixer"].update(vdim=5), "vdim"),
    (lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "divide"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=9), "top"),
    (lambda c: c["layers"][0]["mlp"].update(kind="other"), "unknown feed-forward"),
])
def test_config_errors_are_loud(edit, msg):
    c = mixed_shape().to_config()
    edit(c)
    with pytest.raises(ValueError, match=msg):
        KazolornShape.from_config(c)


def test_weight_names_follow_the_layers():
    s = mixed_shape()
    shp = W.kazolorn_weight_shapes(s)
    assert shp["l0.mix.k"] == (48, 48) and shp["l1.mix.k"] == (16, 48) and shp["l1.mix.talk"] == (6, 6)
    assert shp["l1.mlp.e4.down"] == (48, 24) and shp["l1.mlp.router"] == (5, 48) and "l1.mlp.e5.gate" not in shp
    assert shp["l0.mlp.act"] == (4,) and shp["l2.dwa"] == (4,) and "l2.norm2" not in shp and "l2.ls2" not in shp
    w = W.make_kazolorn_weights(s, seed=3)
    assert set(w) == set(shp) and all(tuple(w[k].shape) == shp[k] and w[k].dtype == torch.bfloat16 for k in shp)
    w2 = W.make_kazolorn_weights(s, seed=3)
    assert all(torch.equal(w[k], w2[k]) for k in w)


def test_checkpoint_directory_round_trip(tmp_path):
    import json
    from safetensors.torch import save_file
    from promptcache_amd.model.config import architecture_of
    s = mixed_shape()
    w = W.make_kazolorn_weights(s, seed=1)
    save_file(w, str(tmp_path / "model.safetensors"))
    (tmp_path / "config.json").write_text(json.dumps(s.to_config()))
    assert architecture_of(str(tmp_path)) == "kazolorn"
    s2 = KazolornShape.from_dir(str(tmp_path))
    got = W.load_kazolorn_safetensors(str(tmp_path), s2)
    assert all(torch.equal(got[k], w[k]) for k in w)
    bad = dict(w)
    bad["l0.mix.q"] = bad["l0.mix.q"][:, :-1].contiguous()
    save_file(bad, str(tmp_path / "model.safetensors"))
    with pytest.raises(ValueError, match="l0.mix.q"):
        W.load_kazolorn_safetensors(str(tmp_path), s2)


# ---- slot arena ------------------------------------------------------------------------------------------------------------------
def test_slot_arena_alloc_free_reuse_and_growth():
    a = SlotArena([(2, 4), (1, 8)], slots=2, cap=8, device="cpu", dtype=torch.float32)
    s0, s1 = a.alloc(), a.alloc()
    assert (s0, s1) == (0, 1) and a.slot_stride(0) == 2 * 8 * 4 and a.head_stride(1) == 8 * 8
    a.planes[0][s1, :, :3] = 7.0
    a.lengths[s1] = 3
    gen = a.generation
    s2 = a.alloc()                                  # no free slot: the planes grow and keep the live rows
    assert s2 == 2 and a.slots >= 3 and a.generation > gen
    assert torch.all(a.planes[0][s1, :, :3] == 7.0)
    a.room_for(s1, 20)                              # longer rows
    assert a.cap >= 23 and torch.all(a.planes[0][s1, :, :3] == 7.0) and a.keys(0, s1).shape == (2, 3, 4)
    a.free(s0)
    assert a.alloc() == s0 and a.lengths[s0] == 0   # the lowest free slot comes back first, empty
    with pytest.raises(KeyError):
        a.free(17)
    assert a.live == [0, 1, 2]


# ---- batch engine on a recording model --------------------------------------------------------------------------------------------
class _Recorder:
    """Stands in for the model: logs every step and answers with logits that make request r's next token r's own counter."""
    decode_headroom = 4

    def __init__(self, vocab=50):
        self.V, self.steps, self.arena = vocab, [], None

    def new_arena(self, slots, cap):
        self.arena = SlotArena([(1, 2)], slots, cap, "cpu", torch.float32)
        return self.arena

    def forward_rows(self, arena, slots, tokens, want):
        self.steps.append([(s, len(t), arena.lengths[s]) for s, t in zip(slots, tokens)])
        rows = []
        for s, t, w in zip(slots, tokens, want):
            arena.room_for(s, len(t))
            arena.lengths[s] += len(t)
            for _ in w:
                r = torch.zeros(self.V)
                r[(arena.lengths[s] * 3) % self.V] = 5.0
                rows.append(r)
        return torch.stack(rows) if rows else torch.zeros((0, self.V))


def test_batch_engine_steps_and_slot_reuse():
    from promptcache_amd import BatchEngine
    m = _Recorder()
    e = BatchEngine(m, max_tokens=64)
    out = e.step([("a", [1, 2, 3], [0, 2]), ("b", [4], [])])
    assert out.shape == (2, 50) and e.held_tokens() == 4
    e.step([("a", [5], [0]), ("b", [6], [0])], end=["b"])
    assert m.steps[1] == [(0, 1, 3), (1, 1, 1)] and "b" not in e.slots
    e.step([("c", [7, 8], [1])])                     # the freed slot is used again, from position 0
    assert m.steps[2] == [(1, 2, 0)]
    with pytest.raises(ValueError):
        e.step([("a", [1], []), ("a", [2], [])])
    assert e.step([], end=["a", "c"]) is None and e.held_tokens() == 0


def test_batch_engine_generate_admits_within_the_budget_and_retires():
    from promptcache_amd import BatchEngine, GenerationParameters
    m = _Recorder()
    e = BatchEngine(m, max_tokens=20)
    params = GenerationParameters(temperature=0.0, max_new_tokens=3, stop_token_ids=[])
    prompts = [[1, 2, 3, 4], [5, 6], [7, 8, 9, 10, 11]]            # needs 7 + 5 + 8 = 20 tokens: all fit at once
    out = e.generate(prompts, params)
    assert [len(o) for o in out] == [3, 3, 3]
    assert out[0] == [(4 * 3) % 50, (5 * 3) % 50, (6 * 3) % 50]
    assert len(m.steps[0]) == 3 and e.held_tokens() == 0
    m2 = _Recorder()
    e2 = BatchEngine(m2, max_tokens=12)                             # 7 + 5 fit, the third waits for room
    out2 = e2.generate(prompts, params)
    assert out2 == out and len(m2.steps[0]) == 2 and any(len(s) == 1 and s[0][1] == 5 for s in m2.steps)


# ---- the blocks library's ABI ----------------------------------------------------------------------------------------------------
def _declared_blocks():
    src = re.sub(r"/\*.*?\*/", "", open(os.path.join(ROOT, "include", "promptcache_blocks.h")).read(), flags=re.S)
    out = {}
    for m in re.finditer(r"\b(pcb_[a-z0-9_]+)\s*\(([^;{]*?)\)\s*;", src, flags=re.S):
        params = m.group(2).strip()
        out[m.group(1)] = 0 if params in ("", "void") else params.count(",") + 1
    return out


def test_blocks_library_exports_what_the_header_declares():
    from promptcache_amd import _blocks
    assert os.path.exists(_blocks.lib_path()), "run __graft_entry__.build() first"
    lib = ctypes.CDLL(_blocks.lib_path())
    decl = _declared_blocks()
    assert sorted(decl) == sorted(_blocks.SIGNATURES)
    for name, arity in decl.items():
        assert hasattr(lib, name), name
        assert len(_blocks.SIGNATURES[name][1]) == arity, name
    lb = _blocks.load(build_missing=False)
    assert lb.pcb_version() == _blocks.ABI_VERSION == 4
    assert lb.pcb_embed_rows(None, 0, None, None, 3, 8, 10, None) == -2001 and b"null pointer" in lb.pcb_last_error_string()
    assert lb.pcb_attn_talk_band(5, 100) == 32 and lb.pcb_attn_talk_band(0, 100) == 128 and lb.pcb_attn_talk_band(500, 100) == 128


def test_blocks_struct_layouts_match_the_header(tmp_path):
    from promptcache_amd import _blocks
    structs = (("pcb_mix_norm_args", _blocks.MixNormArgs), ("pcb_linear_args", _blocks.LinearArgs),
               ("pcb_attn_talk_args", _blocks.AttnTalkArgs))
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


# ---- the oracle's own properties ---------------------------------------------------------------------------------------------------
def test_oracle_is_causal_windowed_and_has_a_sink():
    torch.manual_seed(0)
    H, G, D, n = 4, 2, 6, 12
    q, k = torch.randn(n, H, D, dtype=torch.float64), torch.randn(n, G, D, dtype=torch.float64)
    talk = torch.eye(H, dtype=torch.float64) + 0.1 * torch.randn(H, H, dtype=torch.float64)
    full = O.talking_attention(q, k, 0.4, 5, talk)
    # a later key changes no earlier row; a key one step outside the window changes nothing, one step inside does
    k2 = k.clone(); k2[9] += 3.0
    assert torch.equal(O.talking_attention(q, k2, 0.4, 5, talk)[:9], full[:9])
    k3 = k.clone(); k3[2] += 3.0
    out3 = O.talking_attention(q, k3, 0.4, 5, talk)
    assert torch.equal(out3[7], full[7]) and not torch.allclose(out3[6], full[6])
    # decode form: the last row alone, from its position, equals the row of the whole
    assert torch.allclose(O.talking_attention(q[-1:], k, 0.4, 5, talk, first_pos=n - 1)[0], full[-1])
    # the sink takes weight: with huge negative scores the output vanishes instead of averaging the keys
    w = O.sink_softmax(torch.full((1, 4), -30.0, dtype=torch.float64), torch.ones(1, 4, dtype=torch.bool))
    assert float(w.sum()) < 1e-10
    w = O.sink_softmax(torch.zeros(1, 4, dtype=torch.float64), torch.ones(1, 4, dtype=torch.bool))
    assert abs(float(w.sum()) - 0.8) < 1e-12
    assert abs(float(O.head_slopes(4)[0]) - 0.25) < 1e-15 and abs(float(O.head_slopes(4)[3]) - 2.0 ** -8) < 1e-18


def test_oracle_forward_does_not_look_ahead():
    s = mixed_shape()
    w = W.make_kazolorn_weights(s, seed=5)
    toks = [3, 17, 40, 8, 91, 2, 55, 13, 60]
    a = O.forward(s, w, toks)
    b = O.forward(s, w, toks[:6])
    assert torch.allclose(a[:6], b, atol=1e-10)
    assert O.route(torch.randn(3, 48, dtype=torch.float64), torch.randn(5, 48, dtype=torch.float64), 2)[0].shape == (3, 2)
