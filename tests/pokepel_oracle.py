"""Plain, slow restatement of the Pokepel decoder: single-norm parallel layers with sigmoid-gated branches, whose token mixer is
low-rank latent attention (a shared compressed key/value vector per token, a per-head learned softmax sink, a sigmoid output gate) or
retention (a fixed-decay linear recurrence), and whose feed-forward is a PolyNorm MLP or a group-limited mixture of experts with a shared
expert.  One function per mechanism, token by token where it is recurrent.  Pure torch on the CPU; shares nothing with the package.

Notation: h [T, W] normed activations of ONE sequence at positions 0..T-1, weights as a dict name -> tensor ([out, in] for linears).
Everything runs in the dtype of the tensors handed in."""
import math

import torch


def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rotary_table(rot):
    """(angular step per pair [dims / 2] in float64, magnitude applied to cos and sin) of a rotary description {base, dims, scaling?}.
    scaling {factor, original, fast, slow}: pairs whose wavelength is long against the original context are slowed by `factor`, with a
    linear ramp between the pair indices that turn `fast` and `slow` times over that context."""
    dims, base = int(rot["dims"]), float(rot["base"])
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = base ** (-2.0 * i / dims)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    idx = lambda turns: dims * math.log(sc["original"] / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(idx(sc["fast"])), 0)
    hi = min(math.ceil(idx(sc["slow"])), dims - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return f / sc["factor"] * ramp + f * (1.0 - ramp), 0.1 * math.log(sc["factor"]) + 1.0


def rotate(t, positions, rot, layout):
    """Turn the first rot.dims channels of t [T, heads, d] by position * step; pairs are (2i, 2i+1) ("interleaved") or (i, i + dims/2)
    ("halves")."""
    dims = int(rot["dims"])
    if dims == 0:
        return t
    f, mag = rotary_table(rot)
    a = (positions.to(torch.float64)[:, None] * f[None, :]).to(t.dtype)
    c, s = (torch.cos(a) * mag)[:, None, :], (torch.sin(a) * mag)[:, None, :]
    out = t.clone()
    if layout == "interleaved":
        u, v = t[..., 0:dims:2], t[..., 1:dims:2]
        out[..., 0:dims:2] = u * c - v * s
        out[..., 1:dims:2] = v * c + u * s
    else:
        hf = dims // 2
        u, v = t[..., :hf], t[..., hf:dims]
        out[..., :hf] = u * c - v * s
        out[..., hf:dims] = v * c + u * s
    return out


def latent_attention(h, wts, pre, mx, eps):
    """Keys and values of every head are linear images of one latent vector c_t per token; one rotated key part is shared by the heads.
    Computed the long way round: keys and values are materialised per head."""
    T = h.shape[0]
    H, d, dr, dv, R = mx["heads"], mx["dim"], mx["rot_dim"], mx["vdim"], mx["kv_rank"]
    pos = torch.arange(T)
    q = (h @ wts[pre + "q"].T).view(T, H, d + dr)
    rot = mx.get("rot") or {"dims": 0}
    q_plain, q_rot = q[..., :d], rotate(q[..., d:], pos, rot, "interleaved")
    down = h @ wts[pre + "dkv"].T
    c = rms_unit(down[:, :R], eps) * wts[pre + "dkv.norm"]
    k_rot = rotate(down[:, None, R:], pos, rot, "interleaved")[:, 0]           # [T, dr], one for all heads
    k_plain = (c @ wts[pre + "uk"].T).view(T, H, d)
    v = (c @ wts[pre + "uv"].T).view(T, H, dv)
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for i in range(T):
        for hh in range(H):
            s = (k_plain[:i + 1, hh] @ q_plain[i, hh] + k_rot[:i + 1] @ q_rot[i, hh]) * mx["scale"]
            sink = wts[pre + "sink"][hh]
            m = torch.maximum(s.max(), sink)
            e = torch.exp(s - m)
            out[i, hh] = (e / (e.sum() + torch.exp(sink - m))) @ v[:i + 1, hh]
    out = out.reshape(T, H * dv) * torch.sigmoid(h @ wts[pre + "g"].T)
    return out @ wts[pre + "o"].T


def retention(h, wts, pre, mx, eps):
    """S_t = decay_h S_(t-1) + k_t v_t^T, o_t = S_t^T q_t with rotated q and k, k shrunk by sqrt(dim) after the turn; every head's o is
    brought to unit RMS, gated by silu and projected."""
    T = h.shape[0]
    H, d, dv = mx["heads"], mx["dim"], mx["vdim"]
    pos = torch.arange(T)
    rot = mx.get("rot") or {"dims": 0}
    q = rotate((h @ wts[pre + "q"].T).view(T, H, d), pos, rot, "halves")
    k = rotate((h @ wts[pre + "k"].T).view(T, H, d), pos, rot, "halves") * d ** -0.5
    v = (h @ wts[pre + "v"].T).view(T, H, dv)
    o = torch.zeros(T, H, dv, dtype=h.dtype)
    for hh in range(H):
        S = torch.zeros(d, dv, dtype=h.dtype)
        for t in range(T):
            S = mx["decay"][hh] * S + k[t, hh][:, None] * v[t, hh][None, :]
            o[t, hh] = S.T @ q[t, hh]
    o = rms_unit(o, eps).reshape(T, H * dv) * torch.nn.functional.silu(h @ wts[pre + "g"].T)
    return o @ wts[pre + "o"].T


def polynorm_mlp(h, wts, pre, eps):
    """down(a N(z) + b N(z^2) + c N(z^3) + e), z = up h, N = unit RMS over the hidden channels of a token."""
    z = h @ wts[pre + "up"].T
    a, b, c, e = [float(t) for t in wts[pre + "act"]]
    return (a * rms_unit(z, eps) + b * rms_unit(z * z, eps) + c * rms_unit(z * z * z, eps) + e) @ wts[pre + "down"].T


def silu_expert(h, wts, pre):
    return (torch.nn.functional.silu(h @ wts[pre + "gate"].T) * (h @ wts[pre + "up"].T)) @ wts[pre + "down"].T


def route(h, wts, pre, router):
    """-> (expert ids [T, top], weights [T, top]): softmax scores; experts outside the `keep` groups with the largest best score are
    barred; the weights are the raw scores of the chosen experts."""
    E, top = router["experts"], router["top"]
    s = torch.softmax(h @ wts[pre + "router"].T, -1)
    allowed = torch.ones_like(s, dtype=torch.bool)
    grp = router.get("groups")
    if grp:
        per = E // grp["count"]
        best = s.view(-1, grp["count"], per).max(-1).values
        keep = best.topk(grp["keep"], -1).indices
        ok = torch.zeros_like(best, dtype=torch.bool).scatter_(1, keep, True)
        allowed = ok[:, :, None].expand(-1, -1, per).reshape(-1, E)
    ids = s.masked_fill(~allowed, -1.0).topk(top, -1).indices
    return ids, s.gather(1, ids)


def moe(h, wts, pre, mlp):
    ids, wgt = route(h, wts, pre, mlp["router"])
    out = torch.zeros(h.shape[0], wts[pre + "e0.down"].shape[0], dtype=h.dtype)
    for t in range(h.shape[0]):
        for j in range(ids.shape[1]):
            out[t] += wgt[t, j] * silu_expert(h[t:t + 1], wts, f"{pre}e{int(ids[t, j])}.")[0]
    if mlp.get("shared"):
        out = out + silu_expert(h, wts, pre + "shared.")
    return out


def forward(cfg, wts, tokens, collect=None):
    """Logits [T, vocab] of one sequence run whole.  collect: receives the residual stream after every layer."""
    eps = cfg["norm"]["eps"]
    x = wts["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = rms_unit(x, eps) * wts[p + "norm1"]
        mixer = {"latent_attention": latent_attention, "retention": retention}[L["type"]]
        y = mixer(h, wts, p + "mix.", L["mixer"], eps) * torch.sigmoid(h @ wts[p + "rg1"].T + wts[p + "rg1.b"])
        mlp = L.get("mlp")
        if mlp is not None:
            f = polynorm_mlp(h, wts, p + "mlp.", eps) if mlp["kind"] == "dense" else moe(h, wts, p + "mlp.", mlp)
            y = y + f * torch.sigmoid(h @ wts[p + "rg2"].T + wts[p + "rg2.b"])
        x = x + y
        if collect is not None:
            collect.append(x.clone())
    return (rms_unit(x, eps) * wts["final.norm"]) @ wts["head"].T
