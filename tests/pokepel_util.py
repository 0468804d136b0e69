"""Small random configurations and checkpoints of the Pokepel decoder for the tests (config.json dicts + name -> tensor)."""
import torch

YARN = {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}


def latent_layer(heads=3, dim=16, rot_dim=8, vdim=24, kv_rank=40, base=10000.0, scaling=None, scale=None, mlp=None):
    rot = {"base": base, "dims": rot_dim}
    if scaling:
        rot["scaling"] = dict(scaling)
    mx = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "rot": rot,
          "scale": (dim + rot_dim) ** -0.5 if scale is None else scale}
    return {"type": "latent_attention", "mixer": mx, "mlp": mlp}


def retention_layer(heads=2, dim=16, vdim=24, decay=None, rot_dims=None, base=10000.0, scaling=None, mlp=None):
    mx = {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay) if decay is not None else [1.0 - 2.0 ** -(3 + i) for i in range(heads)]}
    if rot_dims != 0:
        mx["rot"] = {"base": base, "dims": dim if rot_dims is None else rot_dims}
        if scaling:
            mx["rot"]["scaling"] = dict(scaling)
    return {"type": "retention", "mixer": mx, "mlp": mlp}


def dense(ff=48):
    return {"kind": "dense", "ff": ff}


def moe(experts=8, top=2, groups=4, keep=2, ff=32, shared=40):
    m = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if groups:
        m["router"]["groups"] = {"count": groups, "keep": keep}
    if shared:
        m["shared"] = {"ff": shared}
    return m


def make_config(layers, vocab=96, width=64, eps=1e-5):
    return {"architecture": "Pokepel", "layers": layers, "vocab": vocab, "width": width, "norm": {"eps": eps}}


def make_weights(cfg, seed=0, router_gain=4.0):
    """Random float32 tensors under the checkpoint names (values exactly representable in bfloat16).  The router is scaled up so that the
    chosen experts are well apart from the next ones."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]
    rn = lambda *s, k=1.0: (torch.randn(*s, generator=g) * k).bfloat16().float()
    lin = lambda o, i: rn(o, i, k=i ** -0.5)
    w = {"embed": rn(cfg["vocab"], W), "head": lin(cfg["vocab"], W), "final.norm": (1.0 + rn(W, k=0.1)).bfloat16().float()}
    for i, L in enumerate(cfg["layers"]):
        p, mx, mlp = f"l{i}.", L["mixer"], L.get("mlp")
        w[p + "norm1"] = (1.0 + rn(W, k=0.1)).bfloat16().float()
        H, d, dv = mx["heads"], mx["dim"], mx["vdim"]
        if L["type"] == "latent_attention":
            dr, R = mx["rot_dim"], mx["kv_rank"]
            w[p + "mix.q"], w[p + "mix.dkv"] = lin(H * (d + dr), W), lin(R + dr, W)
            w[p + "mix.dkv.norm"] = (1.0 + rn(R, k=0.1)).bfloat16().float()
            w[p + "mix.uk"], w[p + "mix.uv"] = lin(H * d, R), lin(H * dv, R)
            w[p + "mix.sink"] = rn(H, k=1.0)
            w[p + "mix.g"], w[p + "mix.o"] = lin(H * dv, W), lin(W, H * dv)
        else:
            w[p + "mix.q"], w[p + "mix.k"], w[p + "mix.v"] = lin(H * d, W), lin(H * d, W), lin(H * dv, W)
            w[p + "mix.g"], w[p + "mix.o"] = lin(H * dv, W), lin(W, H * dv)
        w[p + "rg1"], w[p + "rg1.b"] = lin(W, W), rn(W, k=0.5)
        if mlp is None:
            continue
        w[p + "rg2"], w[p + "rg2.b"] = lin(W, W), rn(W, k=0.5)
        if mlp["kind"] == "dense":
            w[p + "mlp.up"], w[p + "mlp.down"] = lin(mlp["ff"], W), lin(W, mlp["ff"])
            w[p + "mlp.act"] = torch.tensor([0.75, 0.5, -0.25, 0.125])
        else:
            ff = mlp["expert"]["ff"]
            w[p + "mlp.router"] = (lin(mlp["router"]["experts"], W) * router_gain).bfloat16().float()
            names = [f"e{j}" for j in range(mlp["router"]["experts"])] + (["shared"] if mlp.get("shared") else [])
            for n in names:
                f = mlp["shared"]["ff"] if n == "shared" else ff
                w[p + f"mlp.{n}.gate"], w[p + f"mlp.{n}.up"], w[p + f"mlp.{n}.down"] = lin(f, W), lin(f, W), lin(W, f)
    return w


def oracle_logits(cfg, w, tokens, collect=None):
    """float64 logits [T, vocab] of the plain implementation."""
    import pokepel_oracle
    return pokepel_oracle.forward(cfg, {k: v.double() for k, v in w.items()}, tokens, collect)
