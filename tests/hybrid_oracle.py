"""Plain, slow restatement of the hybrid decoder family (parallel-residual layers whose token mixer is sink-softmax chunked
attention with rotated values, an HGRN2 recurrence or a gated-linear-attention recurrence): one function per mechanism, straight
from the equations, token by token where the mechanism is recurrent.  Pure torch on the CPU; shares nothing with the package.

Notation: x [T, W] residual stream of ONE sequence at positions 0..T-1, weights as a dict name -> tensor with linear weights
stored [out, in].  Everything runs in the dtype of the tensors handed in (float32 or float64)."""
import math

import torch


def rms_unit(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def offset_norm(x, w, eps):
    """RMS norm whose stored weight is an offset from one."""
    return rms_unit(x, eps) * (1.0 + w)


def plain_norm(x, w, eps):
    return rms_unit(x, eps) * w


def pair_angles(positions, n_pairs, span, base):
    """angle[p, i] = p * base^(-2 i / span), i < n_pairs."""
    i = torch.arange(n_pairs, dtype=torch.float64)
    f = (float(base) ** (-2.0 * i / span))
    return positions.to(torch.float64)[:, None] * f[None, :]


def rotate_interleaved(t, positions, dims, base, sign=1.0):
    """Rotate channel pairs (2i, 2i+1), i < dims/2, of t [T, heads, d] by sign * position * base^(-2i/dims); channels >= dims pass."""
    if dims == 0:
        return t
    a = (sign * pair_angles(positions, dims // 2, dims, base)).to(t.dtype)
    c, s = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    u, v = t[..., 0:dims:2], t[..., 1:dims:2]
    out = t.clone()
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def rotate_halves(t, positions, dims, base, sign=1.0):
    """Same turn, pair m = (m, m + dims/2)."""
    a = (sign * pair_angles(positions, dims // 2, dims, base)).to(t.dtype)
    c, s = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    h = dims // 2
    u, v = t[..., :h], t[..., h:dims]
    out = t.clone()
    out[..., :h] = u * c - v * s
    out[..., h:dims] = v * c + u * s
    return out


def attention_keys_values(h, wts, pre, mx, eps):
    """What an attention layer caches for positions 0..T-1: rotated keys [T, G, dim] and unit-normed, rotated values [T, G, vdim]."""
    T = h.shape[0]
    G, d, dv = mx.get("kv_heads", mx["heads"]), mx["dim"], mx["vdim"]
    pos = torch.arange(T)
    rot = mx.get("rot") or {"dims": 0, "base": 1.0}
    k = (h @ wts[pre + "k"].T).view(T, G, d)
    v = (h @ wts[pre + "v"].T).view(T, G, dv)
    k = rotate_interleaved(k, pos, rot["dims"], rot["base"])
    v = rms_unit(v, eps)
    if rot["dims"]:
        v = rotate_interleaved(v, pos, dv, rot["base"])
    return k, v


def attention_mixer(h, wts, pre, mx, eps, kv):
    """kv: (keys, values) as cached by the layer that owns them (this layer or the one named by kv_from)."""
    T = h.shape[0]
    H, G, d, dv = mx["heads"], mx.get("kv_heads", mx["heads"]), mx["dim"], mx["vdim"]
    rot = mx.get("rot") or {"dims": 0, "base": 1.0}
    pos = torch.arange(T)
    q = rotate_interleaved((h @ wts[pre + "q"].T).view(T, H, d), pos, rot["dims"], rot["base"])
    k, v = kv
    size = (mx.get("mask") or {}).get("size")
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for i in range(T):
        lo = 0 if size is None else (i // size) * size
        for hh in range(H):
            g = hh // (H // G)
            s = (k[lo:i + 1, g] @ q[i, hh]) * mx["scale"]
            e = torch.exp(s)
            p = e / (1.0 + e.sum())                      # denominator carries an extra exp(0): an always-present null key
            out[i, hh] = p @ v[lo:i + 1, g]
    if rot["dims"]:
        out = rotate_interleaved(out, pos, dv, rot["base"], sign=-1.0)
    return out.reshape(T, H * dv) @ wts[pre + "o"].T


def gated_scan(q, k, v, a):
    """S_t = diag(a_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t for one head.  q, k, a [T, d], v [T, dv]."""
    T, d = q.shape
    S = torch.zeros(d, v.shape[1], dtype=q.dtype)
    o = []
    for t in range(T):
        S = a[t][:, None] * S + k[t][:, None] * v[t][None, :]
        o.append(S.T @ q[t])
    return torch.stack(o)


def hgrn2_mixer(h, wts, pre, mx, eps):
    T = h.shape[0]
    H, d, dv = mx["heads"], mx["dim"], mx["vdim"]
    q = torch.nn.functional.silu(h @ wts[pre + "q"].T).view(T, H, d)
    v = (h @ wts[pre + "v"].T).view(T, H, dv)
    low = wts[pre + "lower"].view(H, d)
    f = low + (1.0 - low) * torch.sigmoid(h @ wts[pre + "f"].T + wts[pre + "f.b"]).view(T, H, d)
    o = torch.stack([gated_scan(q[:, i], 1.0 - f[:, i], v[:, i], f[:, i]) for i in range(H)], 1)
    o = plain_norm(o, wts[pre + "norm"], eps)
    return o.reshape(T, H * dv) @ wts[pre + "o"].T


def gla_mixer(h, wts, pre, mx, eps):
    T = h.shape[0]
    H, d, dv = mx["heads"], mx["dim"], mx["vdim"]
    q = (h @ wts[pre + "q"].T).view(T, H, d) * d ** -0.5
    k = (h @ wts[pre + "k"].T).view(T, H, d)
    v = (h @ wts[pre + "v"].T).view(T, H, dv)
    z = (h @ wts[pre + "a1"].T) @ wts[pre + "a2"].T + wts[pre + "a2.b"]
    alpha = torch.exp(torch.nn.functional.logsigmoid(z) / mx["tau"]).view(T, H, d)
    o = torch.stack([gated_scan(q[:, i], k[:, i], v[:, i], alpha[:, i]) for i in range(H)], 1)
    o = plain_norm(o, wts[pre + "norm"], eps).reshape(T, H * dv)
    return (o * torch.nn.functional.silu(h @ wts[pre + "g"].T)) @ wts[pre + "o"].T


def dense_mlp(h, wts, pre):
    return (torch.relu(h @ wts[pre + "gate"].T) * (h @ wts[pre + "up"].T)) @ wts[pre + "down"].T


def forward(cfg, wts, tokens, collect=None):
    """Logits [T, vocab] of one sequence run whole.  collect: a list that receives the residual stream after every layer."""
    eps, m = cfg["norm"]["eps"], cfg["residual_mult"]
    x = wts["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    kv = {}
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        h1 = offset_norm(x, wts[p + "norm1"], eps)
        mx = L["mixer"]
        if L["type"] == "attention":
            src = mx.get("kv_from")
            if src is None:
                kv[i] = attention_keys_values(h1, wts, p + "mix.", mx, eps)
                src = i
            y = attention_mixer(h1, wts, p + "mix.", mx, eps, kv[src])
        elif L["type"] == "hgrn2":
            y = hgrn2_mixer(h1, wts, p + "mix.", mx, eps)
        elif L["type"] == "gla":
            y = gla_mixer(h1, wts, p + "mix.", mx, eps)
        else:
            raise ValueError(L["type"])
        if L.get("mlp") is not None:
            y = y + dense_mlp(offset_norm(x, wts[p + "norm2"], eps), wts, p + "mlp.")
        x = x + m * y
        if collect is not None:
            collect.append(x.clone())
    logits = offset_norm(x, wts["final.norm"], eps) @ wts["head"].T
    cap = cfg.get("logit_softcap")
    return cap * torch.tanh(logits / cap) if cap else logits
