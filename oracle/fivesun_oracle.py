"""Plain, slow statement of the Fivesun design in float64 torch on the CPU: one function per mechanism, written from the
equations and sharing nothing with the product path (``promptcache_amd/model/fivesun_hip.py`` and its kernels).

Notation: n tokens of one sequence at positions pos0 .. pos0 + n - 1; ``p`` a dict of float64 tensors keyed like the checkpoint;
``lay`` a ``config.FivesunLayer``.  Attention is written over explicit lists of visible keys, recurrences as literal loops over
the tokens.  ``carry`` is what a sequence leaves behind for its next tokens: per layer the keys / values / latents so far, or the
mLSTM's (S, n, m).
"""
from __future__ import annotations

import math

import torch

F = torch.float64


def unit_rms(x, eps):
    return x / torch.sqrt(x.pow(2).mean(dim=-1, keepdim=True) + eps)


def activation(name):
    if name == "relu":
        return torch.relu
    if name == "silu":
        return lambda z: z * torch.sigmoid(z)
    if name == "gelu_tanh":
        return lambda z: 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))
    raise ValueError(name)


# ---- rotary positions ---------------------------------------------------------------------------------------------------------------
def plain_frequencies(base, dims, factor=1.0):
    """f_i = base^(-2i/dims) / factor, i = 0 .. dims/2 - 1; magnitude 1."""
    return torch.tensor([base ** (-2.0 * i / dims) / factor for i in range(dims // 2)], dtype=F), 1.0


def yarn_frequencies(base, dims, factor, original, fast, slow):
    """Frequencies that turn fast keep their value, those that turn slowly are divided by ``factor``, with a linear ramp between;
    the rotated vector also grows by 0.1 ln(factor) + 1."""
    def column_of(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(column_of(fast)), 0)
    hi = min(math.ceil(column_of(slow)), dims - 1)
    out = []
    for i in range(dims // 2):
        f = base ** (-2.0 * i / dims)
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f / factor * ramp + f * (1.0 - ramp))
    return torch.tensor(out, dtype=F), 0.1 * math.log(factor) + 1.0


def rotate_pairs(x, positions, freqs, magnitude=1.0):
    """x [n, ..., 2m]: neighbours (2i, 2i + 1) turn by positions * freqs[i]; columns past 2 len(freqs) pass unchanged."""
    m = freqs.numel()
    out = x.clone()
    ang = positions.to(F).view(-1, *([1] * (x.dim() - 2)), 1) * freqs
    c, s = torch.cos(ang) * magnitude, torch.sin(ang) * magnitude
    u, v = x[..., 0:2 * m:2], x[..., 1:2 * m:2]
    out[..., 0:2 * m:2] = u * c - v * s
    out[..., 1:2 * m:2] = v * c + u * s
    return out


# ---- which keys a query sees --------------------------------------------------------------------------------------------------------
def sees_block(i, j, size):
    """Blocks of ``size`` positions counted from 0: a key is seen inside the query's own block only (size 0: every earlier key)."""
    return j <= i and (size <= 0 or i // size == j // size)


def sees_window(i, j, size):
    return j <= i and (size <= 0 or i - j < size)


def softmax_attention(q, k, v, qpos, sees, scale, sink=None):
    """q [n, D] at positions qpos; k [m, D], v [m, Dv] at positions 0 .. m-1.  ``sink``: one more exp(sink) in the denominator."""
    out = torch.zeros(q.shape[0], v.shape[1], dtype=F)
    for r, i in enumerate(qpos):
        js = [j for j in range(k.shape[0]) if sees(i, j)]
        s = (k[js] @ q[r]) * scale
        top = s.max() if sink is None else torch.maximum(s.max(), sink)
        e = torch.exp(s - top)
        den = e.sum() + (torch.exp(sink - top) if sink is not None else 0.0)
        out[r] = (e / den) @ v[js]
    return out


# ---- mixers -------------------------------------------------------------------------------------------------------------------------
def attention_mixer(h, p, pre, lay, eps, pos0, past, v_first, lam):
    """-> (result [n, W], (keys, values) so far, this layer's values of the new tokens).  ``v_first``: the first blending layer's
    values of the same tokens (None: this layer does not blend, or is that layer)."""
    n = h.shape[0]
    H, G, D, Dv = lay.heads, lay.kv_heads, lay.dim, lay.vdim
    pos = torch.arange(pos0, pos0 + n)
    q = unit_rms((h @ p[pre + "q"].T).view(n, H, D), eps) * p[pre + "q.norm"]
    k = unit_rms((h @ p[pre + "k"].T).view(n, G, D), eps) * p[pre + "k.norm"]
    v = unit_rms((h @ p[pre + "v"].T).view(n, G, Dv), eps)
    if lay.rot_dims:
        fr, mag = plain_frequencies(lay.rot_base, lay.rot_dims, lay.rot_factor)
        q, k = rotate_pairs(q, pos, fr, mag), rotate_pairs(k, pos, fr, mag)
    if v_first is not None:
        v = (1.0 - lam) * v + lam * v_first
    if past is not None:
        k, v_all = torch.cat([past[0], k]), torch.cat([past[1], v])
    else:
        v_all = v
    gate = torch.sigmoid(h @ p[pre + "g"].T)                      # [n, H]
    out = torch.zeros(n, H, Dv, dtype=F)
    for hd in range(H):
        g = hd // (H // G)
        out[:, hd] = softmax_attention(q[:, hd], k[:, g], v_all[:, g], pos.tolist(), lambda i, j: sees_block(i, j, lay.mask), lay.scale,
                                       sink=p[pre + "sink"][hd]) * gate[:, hd:hd + 1]
    return out.reshape(n, H * Dv) @ p[pre + "o"].T, (k, v_all), v


def latent_mixer(h, p, pre, lay, eps, pos0, past):
    """-> (result, (latents, rotated key parts) so far).  Keys and values of every head are rebuilt from the latents."""
    n = h.shape[0]
    H, D, R, Dv, C = lay.heads, lay.dim, lay.rot_dim, lay.vdim, lay.kv_rank
    pos = torch.arange(pos0, pos0 + n)
    if lay.yarn_original:
        fr, mag = yarn_frequencies(lay.rot_base, R, lay.rot_factor, lay.yarn_original, lay.yarn_fast, lay.yarn_slow)
    else:
        fr, mag = plain_frequencies(lay.rot_base, R, lay.rot_factor)
    q = (h @ p[pre + "q"].T).view(n, H, D + R)
    q_plain, q_rot = q[..., :D], rotate_pairs(q[..., D:], pos, fr, mag)
    down = h @ p[pre + "dkv"].T
    c = unit_rms(down[:, :C], eps) * p[pre + "dkv.norm"]
    k_rot = rotate_pairs(down[:, C:], pos, fr, mag)
    if past is not None:
        c, k_rot = torch.cat([past[0], c]), torch.cat([past[1], k_rot])
    k_plain = (c @ p[pre + "uk"].T).view(-1, H, D)
    v = (c @ p[pre + "uv"].T).view(-1, H, Dv)
    out = torch.zeros(n, H, Dv, dtype=F)
    for hd in range(H):
        qq = torch.cat([q_plain[:, hd], q_rot[:, hd]], dim=1)
        kk = torch.cat([k_plain[:, hd], k_rot], dim=1)
        out[:, hd] = softmax_attention(qq, kk, v[:, hd], pos.tolist(), lambda i, j: sees_window(i, j, lay.mask), lay.scale)
    out = out.reshape(n, H * Dv) * torch.sigmoid(h @ p[pre + "g"].T)
    return out @ p[pre + "o"].T, (c, k_rot)


def soft_cap(z, cap):
    return cap * torch.tanh(z / cap) if cap > 0 else z


def matrix_memory(q, k, v, log_i, log_f, state=None):
    """q, k [n, H, D], v [n, H, Dv], log_i, log_f [n, H]; per head, token by token, with a running maximum m (0 at the start):
        m' = max(log_f + m, log_i);  S' = exp(log_f + m - m') S + exp(log_i - m') k v^T;  n' likewise with k alone;
        o = S'^T q / (max(|n' . q|, exp(-m')) + 1e-6).
    -> (o [n, H, Dv], (S, n, m))."""
    T, H, D = q.shape
    Dv = v.shape[-1]
    if state is None:
        S, nv, m = torch.zeros(H, D, Dv, dtype=F), torch.zeros(H, D, dtype=F), torch.zeros(H, dtype=F)
    else:
        S, nv, m = (t.clone() for t in state)
    out = torch.zeros(T, H, Dv, dtype=F)
    for t in range(T):
        for hd in range(H):
            m_new = torch.maximum(log_f[t, hd] + m[hd], log_i[t, hd])
            keep, take = torch.exp(log_f[t, hd] + m[hd] - m_new), torch.exp(log_i[t, hd] - m_new)
            S[hd] = keep * S[hd] + take * torch.outer(k[t, hd], v[t, hd])
            nv[hd] = keep * nv[hd] + take * k[t, hd]
            m[hd] = m_new
            den = torch.maximum((nv[hd] @ q[t, hd]).abs(), torch.exp(-m_new)) + 1e-6
            out[t, hd] = (S[hd].T @ q[t, hd]) / den
    return out, (S, nv, m)


def mlstm_mixer(h, p, pre, lay, eps, past):
    n = h.shape[0]
    H, D, Dv = lay.heads, lay.dim, lay.vdim
    q = (h @ p[pre + "q"].T).view(n, H, D) * D ** -0.5
    k = (h @ p[pre + "k"].T).view(n, H, D)
    v = (h @ p[pre + "v"].T).view(n, H, Dv)
    log_i = soft_cap(h @ p[pre + "i"].T + p[pre + "i.b"], lay.gate_cap)
    log_f = torch.nn.functional.logsigmoid(soft_cap(h @ p[pre + "f"].T + p[pre + "f.b"], lay.gate_cap))
    o, state = matrix_memory(q, k, v, log_i, log_f, past)
    o = unit_rms(o, eps).reshape(n, H * Dv) * p[pre + "norm"] * torch.sigmoid(h @ p[pre + "g"].T)
    return o @ p[pre + "o"].T, state


def dense_ff(h, p, pre, act="relu"):
    a = activation(act)(h @ p[pre + "gate"].T + p[pre + "gate.b"])
    return (a * (h @ p[pre + "up"].T + p[pre + "up.b"])) @ p[pre + "down"].T + p[pre + "down.b"]


def gated_sublayer(x, f, p, pre, which, eps):
    """x + norm_after(sigmoid(W h + b) * f(h)), h = norm_before(x); ``which`` = "1" (mixer) or "2" (feed-forward)."""
    h = unit_rms(x, eps) * p[pre + "norm" + which]
    y = f(h) * torch.sigmoid(h @ p[pre + "rg" + which].T + p[pre + "rg" + which + ".b"])
    return x + unit_rms(y, eps) * p[pre + "norm" + which + "b"]


# ---- the stack ----------------------------------------------------------------------------------------------------------------------
def forward(cfg, p, tokens, pos0=0, carry=None, num_layers=None):
    """-> (logits [n, V], residual stream after every layer [L, n, W], carry for the sequence's next tokens)."""
    eps = cfg.norm_eps
    x = p["embed"][torch.as_tensor(tokens, dtype=torch.long)] * cfg.embed_scale
    layers = cfg.layers if num_layers is None else cfg.layers[:num_layers]
    carry = list(carry) if carry is not None else [None] * len(cfg.layers)
    first, v_first, streams = cfg.first_v_mix, None, []
    for i, lay in enumerate(layers):
        pre = f"l{i}."
        box = {}

        def mixer(h, i=i, lay=lay, pre=pre, box=box):
            nonlocal v_first
            if lay.kind == "attention":
                blend = lay.v_mix and i != first
                y, box["carry"], v = attention_mixer(h, p, pre + "mix.", lay, eps, pos0, carry[i], v_first if blend else None,
                                                     p[pre + "mix.vmix"] if blend else None)
                if i == first:
                    v_first = v
            elif lay.kind == "latent_attention":
                y, box["carry"] = latent_mixer(h, p, pre + "mix.", lay, eps, pos0, carry[i])
            else:
                y, box["carry"] = mlstm_mixer(h, p, pre + "mix.", lay, eps, carry[i])
            return y

        x = gated_sublayer(x, mixer, p, pre, "1", eps)
        carry[i] = box["carry"]
        if lay.ff:
            x = gated_sublayer(x, lambda h, pre=pre, lay=lay: dense_ff(h, p, pre + "mlp.", lay.act), p, pre, "2", eps)
        streams.append(x)
    logits = (unit_rms(x, eps) * p["final.norm"]) @ p["head"].T
    return logits, torch.stack(streams) if streams else torch.zeros(0, *x.shape, dtype=F), carry


def to_f64(weights):
    return {k: v.to(F) for k, v in weights.items()}
