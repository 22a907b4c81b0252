"""Plain, slow statement of the Bepepel design in float64 torch on the CPU: one function per mechanism, written from the
equations and sharing nothing with the product path (``promptcache_amd/model/bepepel_hip.py`` and its kernels).

Notation: n tokens of one sequence at positions pos0 .. pos0 + n - 1; ``p`` a dict of float64 tensors keyed like the checkpoint;
``lay`` a ``config.BepepelLayer``.  Attention is written over explicit lists of visible keys, recurrences and convolutions as
literal loops over the tokens.  ``carry`` is what a sequence leaves behind for its next tokens: per layer a dict with the keys /
values so far, the last inputs of the short convolutions and the matrix states.
"""
from __future__ import annotations

import math

import torch

F = torch.float64


def silu(z):
    return z * torch.sigmoid(z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def unit_rms(x, eps):
    return x / torch.sqrt(x.pow(2).mean(dim=-1, keepdim=True) + eps)


def layer_norm(x, w, b, eps):
    mu = x.mean(dim=-1, keepdim=True)
    var = (x - mu).pow(2).mean(dim=-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w + b


# ---- short causal convolution ---------------------------------------------------------------------------------------------------------
def short_conv(u, w, bias, before):
    """u [n, C] the step's inputs, w [C, taps] (the last column is the current token's), ``before`` [taps - 1, C] the inputs just
    ahead of the step (zeros before the sequence's start).  Returns the outputs [n, C] and the new ``before``."""
    taps = w.shape[1]
    full = torch.cat([before, u], dim=0)
    out = torch.zeros_like(u)
    for t in range(u.shape[0]):
        for j in range(taps):
            out[t] += w[:, j] * full[t + j]            # full[t + taps - 1] is token t itself
    if bias is not None:
        out = out + bias
    return out, full[full.shape[0] - (taps - 1):] if taps > 1 else before


# ---- rotary positions -------------------------------------------------------------------------------------------------------------------
def rotary_frequencies(base, dims, scaling=None):
    """f_i = base^(-2i/dims); with ``scaling`` (factor, low, high, original) a frequency whose wavelength is shorter than
    original / high stays, one longer than original / low is divided by factor, and between the two the blend
    (1 - s) f / factor + s f with s = (original / wavelength - low) / (high - low)."""
    out = []
    for i in range(dims // 2):
        f = base ** (-2.0 * i / dims)
        if scaling:
            factor, low, high, orig = scaling
            wl = 2.0 * math.pi / f
            if wl < orig / high:
                pass
            elif wl > orig / low:
                f = f / factor
            else:
                s = (orig / wl - low) / (high - low)
                f = (1.0 - s) * f / factor + s * f
        out.append(f)
    return torch.tensor(out, dtype=F)


def rotate_pairs(x, positions, freqs):
    """x [n, heads, dim]: neighbours (2i, 2i + 1), i < len(freqs), turn by positions * freqs[i]; other columns pass unchanged."""
    m = freqs.numel()
    if m == 0:
        return x
    out = x.clone()
    ang = positions.to(F).view(-1, 1, 1) * freqs
    c, s = torch.cos(ang), torch.sin(ang)
    u, v = x[..., 0:2 * m:2], x[..., 1:2 * m:2]
    out[..., 0:2 * m:2] = u * c - v * s
    out[..., 1:2 * m:2] = v * c + u * s
    return out


# ---- attention over explicit lists of visible keys ---------------------------------------------------------------------------------------
def sees(i, j, window, keep_first):
    """Does the query at position i see the key at position j?"""
    return j <= i and (window <= 0 or i - j < window or j < keep_first)


def softmax_over_seen(q, keys, vals, qpos, window, keep_first, scale):
    """q [n, D] at positions qpos; keys [m, D] and vals [m, Dv] at positions 0 .. m - 1.  Returns [n, Dv]."""
    out = torch.zeros(q.shape[0], vals.shape[1], dtype=F)
    for t, i in enumerate(qpos):
        seen = [j for j in range(keys.shape[0]) if sees(i, j, window, keep_first)]
        w = torch.softmax((keys[seen] @ q[t]) * scale, dim=0)
        out[t] = w @ vals[seen]
    return out


# ---- a matrix state with a decay per token -------------------------------------------------------------------------------------------------
def matrix_state_steps(q, k, v, decay, S):
    """S_t = diag(decay_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t, token by token.  q, k [n, D]; v [n, Dv]; decay [n, D] (or [n, 1]: one
    decay for all rows); S [D, Dv].  Returns the outputs [n, Dv] and the last state."""
    out = torch.zeros(q.shape[0], v.shape[1], dtype=F)
    for t in range(q.shape[0]):
        S = decay[t].reshape(-1, 1) * S + k[t].reshape(-1, 1) * v[t].reshape(1, -1)
        out[t] = S.T @ q[t]
    return out, S


def to_f64(weights):
    return {k: v.to("cpu", F) for k, v in weights.items()}


# ---- the mixers ----------------------------------------------------------------------------------------------------------------------
def gla_mixer(h, p, pre, lay, eps, carry):
    """Gated linear attention with one decay per key channel and token."""
    n = h.shape[0]
    H, D, Dv = lay.heads, lay.dim, lay.vdim
    q = (h @ p[pre + "q"].T).view(n, H, D) * D ** -0.5
    k = (h @ p[pre + "k"].T).view(n, H, D)
    v = (h @ p[pre + "v"].T).view(n, H, Dv)
    z = (h @ p[pre + "a1"].T) @ p[pre + "a2"].T + p[pre + "a2.b"]
    alpha = torch.sigmoid(z).pow(1.0 / lay.tau).view(n, H, D)
    S = carry.get("S")
    if S is None:
        S = torch.zeros(H, D, Dv, dtype=F)
    o = torch.zeros(n, H, Dv, dtype=F)
    S = S.clone()
    for hh in range(H):
        o[:, hh], S[hh] = matrix_state_steps(q[:, hh], k[:, hh], v[:, hh], alpha[:, hh], S[hh])
    carry["S"] = S
    o = unit_rms(o, eps) * p[pre + "norm"]
    return (o.reshape(n, H * Dv) * silu(h @ p[pre + "g"].T)) @ p[pre + "o"].T


def window_attention(h, p, pre, a, eps, pos0, carry):
    """Softmax attention behind short convolutions: grouped key heads, rotated and unit-RMS queries and keys, a sliding window that
    keeps the sequence's first tokens.  ``a`` holds the sub-mixer's sizes and constants."""
    n = h.shape[0]
    H, G, D, Dv = a.heads, a.kv_heads, a.dim, a.vdim
    proj = {}
    for name in ("q", "k", "v"):
        u = h @ p[pre + name].T + p[pre + name + ".b"]
        if a.conv:
            before = carry.get("conv_" + name)
            if before is None:
                before = torch.zeros(a.conv - 1, u.shape[1], dtype=F)
            u, carry["conv_" + name] = short_conv(u, p[pre + name + ".conv"], None, before)
        proj[name] = u
    pos = torch.arange(pos0, pos0 + n)
    freqs = rotary_frequencies(a.rot_base, a.rot_dims, a.rot_scaling) if a.rot_dims else torch.zeros(0, dtype=F)
    q = unit_rms(rotate_pairs(proj["q"].view(n, H, D), pos, freqs), eps)
    k = unit_rms(rotate_pairs(proj["k"].view(n, G, D), pos, freqs), eps)
    v = proj["v"].view(n, G, Dv)
    keys = k if "k" not in carry else torch.cat([carry["k"], k], dim=0)
    vals = v if "v" not in carry else torch.cat([carry["v"], v], dim=0)
    carry["k"], carry["v"] = keys, vals
    out = torch.zeros(n, H, Dv, dtype=F)
    for hh in range(H):
        g = hh // (H // G)
        out[:, hh] = softmax_over_seen(q[:, hh], keys[:, g], vals[:, g], list(range(pos0, pos0 + n)), a.window, a.keep_first, a.scale)
    return out.reshape(n, H * Dv) @ p[pre + "o"].T


def ssd_mixer(h, p, pre, b, eps, carry):
    """Mamba-2: per head one scalar decay per token and a state of ``state`` x ``vdim`` numbers."""
    n = h.shape[0]
    H, P, N, G = b.heads, b.vdim, b.state, b.groups
    inner = H * P
    proj = h @ p[pre + "in"].T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    if b.conv:
        before = carry.get("conv")
        if before is None:
            before = torch.zeros(b.conv - 1, xbc.shape[1], dtype=F)
        xbc, carry["conv"] = short_conv(xbc, p[pre + "conv"], p[pre + "conv.b"], before)
    xbc = silu(xbc)
    x = xbc[:, :inner].view(n, H, P)
    Bm = xbc[:, inner:inner + G * N].view(n, G, N)
    Cm = xbc[:, inner + G * N:].view(n, G, N)
    dt = torch.nn.functional.softplus(dt + p[pre + "dt_bias"], threshold=1e9)
    A = torch.exp(p[pre + "A_log"])
    S = carry.get("S")
    if S is None:
        S = torch.zeros(H, N, P, dtype=F)
    y = torch.zeros(n, H, P, dtype=F)
    S = S.clone()
    for hh in range(H):
        g = hh // (H // G)
        y[:, hh], S[hh] = matrix_state_steps(Cm[:, g], Bm[:, g], dt[:, hh:hh + 1] * x[:, hh], torch.exp(-A[hh] * dt[:, hh:hh + 1]), S[hh])
        y[:, hh] += p[pre + "D"][hh] * x[:, hh]
    carry["S"] = S
    y = y.reshape(n, inner) * silu(z)
    parts = b.norm_groups
    y = unit_rms(y.view(n, parts, inner // parts), eps).reshape(n, inner) * p[pre + "norm"]
    return y @ p[pre + "o"].T


def parallel_mixer(h, p, pre, lay, eps, pos0, carry):
    left = window_attention(h, p, pre + "left.", lay.left, eps, pos0, carry.setdefault("left", {}))
    right = ssd_mixer(h, p, pre + "right.", lay.right, eps, carry.setdefault("right", {}))
    return lay.left_scale * left + lay.right_scale * right


# ---- feed-forwards ------------------------------------------------------------------------------------------------------------------------
def gated_unit(h, p, pre, act):
    return (act(h @ p[pre + "gate"].T) * (h @ p[pre + "up"].T)) @ p[pre + "down"].T


def route(h, p, pre, top):
    """Per token the ``top`` experts with the largest router logits and the softmax over those logits alone."""
    z = h @ p[pre + "router"].T + p[pre + "router.b"]
    val, idx = torch.sort(z, dim=-1, descending=True, stable=True)
    return idx[:, :top], torch.softmax(val[:, :top], dim=-1)


def feed_forward(h, p, pre, lay):
    if lay.ff_kind == "dense":
        return gated_unit(h, p, pre, gelu_tanh)
    idx, w = route(h, p, pre, lay.top)
    out = torch.zeros(h.shape[0], p[pre + "e0.down"].shape[0], dtype=F)
    for t in range(h.shape[0]):
        for k in range(lay.top):
            out[t] += w[t, k] * gated_unit(h[t:t + 1], p, pre + f"e{int(idx[t, k])}.", silu)[0]
    if lay.shared_ff:
        out = out + gated_unit(h, p, pre + "shared.", silu)
    return out


# ---- the stack ----------------------------------------------------------------------------------------------------------------------------
def forward(cfg, p, tokens, pos0=0, carry=None, return_streams=False):
    """Logits [n, vocab] of ``tokens`` at positions pos0 .. ; ``carry`` (a list of per-layer dicts, updated in place) holds what
    earlier calls left.  ``return_streams``: also the residual stream after every layer [layers, n, width]."""
    if carry is None:
        carry = [{} for _ in cfg.layers]
    eps, m = cfg.norm_eps, cfg.residual_mult
    x = p["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    streams = []
    for i, lay in enumerate(cfg.layers):
        pre = f"l{i}."
        h = layer_norm(x, p[pre + "norm1"], p[pre + "norm1.b"], eps)
        if lay.kind == "gla":
            y = gla_mixer(h, p, pre + "mix.", lay, eps, carry[i])
        else:
            y = parallel_mixer(h, p, pre + "mix.", lay, eps, pos0, carry[i])
        x = x + m * y
        if lay.ff_kind:
            h = layer_norm(x, p[pre + "norm2"], p[pre + "norm2.b"], eps)
            x = x + m * feed_forward(h, p, pre + "mlp.", lay)
        streams.append(x)
    logits = layer_norm(x, p["final.norm"], p["final.norm.b"], eps) @ p["head"].T * cfg.logit_scale
    return (logits, torch.stack(streams)) if return_streams else logits


def forward_in_portions(cfg, p, tokens, cuts):
    """The same sequence fed in portions of the given sizes, each continuing from what the ones before left."""
    carry = [{} for _ in cfg.layers]
    out, at = [], 0
    for c in cuts:
        out.append(forward(cfg, p, tokens[at:at + c], pos0=at, carry=carry))
        at += c
    return torch.cat(out)
