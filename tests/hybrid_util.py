"""Small random configurations and checkpoints of the hybrid decoder family for the tests (config.json dicts + name -> tensor)."""
import torch


def attention_layer(heads=4, kv_heads=2, dim=16, vdim=24, rot_dims=None, base=10000.0, chunk=32, ff=64, kv_from=None, scale=None):
    mx = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim ** -0.5 if scale is None else scale}
    if chunk:
        mx["mask"] = {"size": chunk}
    if rot_dims != 0:
        mx["rot"] = {"base": base, "dims": dim if rot_dims is None else rot_dims}
    if kv_from is not None:
        mx["kv_from"] = kv_from
    return {"type": "attention", "mixer": mx, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def hgrn2_layer(heads=2, dim=24, vdim=32, ff=64):
    return {"type": "hgrn2", "mixer": {"heads": heads, "dim": dim, "vdim": vdim}, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def gla_layer(heads=2, dim=16, vdim=32, tau=8.0, ff=64, rank=8):
    return {"type": "gla", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau, "_rank": rank},
            "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def make_config(layers, vocab=96, width=64, eps=1e-5, residual_mult=0.5, softcap=20.0):
    return {"architecture": "Nufalorn", "layers": layers, "vocab": vocab, "width": width, "norm": {"eps": eps},
            "residual_mult": residual_mult, "logit_softcap": softcap}


def make_weights(cfg, seed=0):
    """Random float32 tensors under the family's checkpoint names (values exactly representable in bfloat16)."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]
    rn = lambda *s, k=1.0: (torch.randn(*s, generator=g) * k).bfloat16().float()
    lin = lambda o, i: rn(o, i, k=i ** -0.5)
    w = {"embed": rn(cfg["vocab"], W), "head": lin(cfg["vocab"], W), "final.norm": rn(W, k=0.1)}
    for i, L in enumerate(cfg["layers"]):
        p, mx = f"l{i}.", L["mixer"]
        w[p + "norm1"] = rn(W, k=0.1)
        H, d, dv = mx["heads"], mx["dim"], mx["vdim"]
        if L["type"] == "attention":
            G = mx.get("kv_heads", H)
            w[p + "mix.q"], w[p + "mix.o"] = lin(H * d, W), lin(W, H * dv)
            if mx.get("kv_from") is None:
                w[p + "mix.k"], w[p + "mix.v"] = lin(G * d, W), lin(G * dv, W)
        elif L["type"] == "hgrn2":
            w[p + "mix.q"], w[p + "mix.f"], w[p + "mix.v"], w[p + "mix.o"] = lin(H * d, W), lin(H * d, W), lin(H * dv, W), lin(W, H * dv)
            w[p + "mix.f.b"] = rn(H * d, k=0.5)
            w[p + "mix.lower"] = torch.sigmoid(torch.randn(H * d, generator=g)).bfloat16().float()
            w[p + "mix.norm"] = (1.0 + rn(dv, k=0.1)).bfloat16().float()
        else:
            r = mx.get("_rank", 8)
            for n, o in (("q", H * d), ("k", H * d), ("v", H * dv), ("g", H * dv), ("a1", r)):
                w[p + "mix." + n] = lin(o, W)
            w[p + "mix.a2"], w[p + "mix.a2.b"] = lin(H * d, r), rn(H * d, k=1.0) + 2.0
            w[p + "mix.a2.b"] = w[p + "mix.a2.b"].bfloat16().float()
            w[p + "mix.norm"] = (1.0 + rn(dv, k=0.1)).bfloat16().float()
            w[p + "mix.o"] = lin(W, H * dv)
        if L.get("mlp") is not None:
            ff = L["mlp"]["ff"]
            w[p + "norm2"] = rn(W, k=0.1)
            w[p + "mlp.gate"], w[p + "mlp.up"], w[p + "mlp.down"] = lin(ff, W), lin(ff, W), lin(W, ff)
    return w


def oracle_logits(cfg, w, tokens, collect=None):
    """float64 logits [T, vocab] of the plain implementation."""
    import hybrid_oracle
    return hybrid_oracle.forward(cfg, {k: v.double() for k, v in w.items()}, tokens, collect)
