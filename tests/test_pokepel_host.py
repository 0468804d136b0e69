"""Host-side pieces of the Pokepel member of the hybrid family, on the CPU: reading its config.json, the registry, the rotary tables, and the
plain implementation's own consistency against closed forms."""
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import pokepel_oracle as O  # noqa: E402
import pokepel_util as U  # noqa: E402


def test_config_reading_and_registry():
    from rtp_llm_amd import registry
    from rtp_llm_amd.hybrid import HybridConfig
    from rtp_llm_amd.mixers import LatentAttentionSpec, RetentionSpec
    assert "pokepel" in registry.families()
    cfg = U.make_config([U.retention_layer(heads=3, rot_dims=4, mlp=U.dense(ff=72)), U.latent_layer(scaling=U.YARN, mlp=U.moe(experts=12, top=3, groups=3, keep=2, ff=24, shared=56)),
                         U.latent_layer(mlp=U.moe(groups=None, shared=None)), U.retention_layer(rot_dims=0)], vocab=70, width=40, eps=3e-6)
    c = HybridConfig.from_json(cfg)
    assert (c.name, c.vocab, c.width, c.eps) == ("Pokepel", 70, 40, 3e-6)
    assert c.shared_norm and c.branch_gates and c.norm_offset == 0.0 and c.residual_mult == 1.0 and c.logit_softcap == 0.0
    r, a, b, n = c.layers
    assert isinstance(r.mixer, RetentionSpec) and r.mixer.decay == tuple(cfg["layers"][0]["mixer"]["decay"]) and r.mixer.rot.dims == 4 and r.mixer.rot.layout == "halves"
    assert (r.mlp_kind, r.ff) == ("polynorm", 72)
    assert isinstance(a.mixer, LatentAttentionSpec) and a.mixer.rot.layout == "interleaved" and a.mixer.rot.scaling.factor == U.YARN["factor"]
    assert (a.mlp_kind, a.ff, a.shared_ff, a.router.experts, a.router.top, a.router.groups, a.router.keep) == ("experts", 24, 56, 12, 3, 3, 2)
    assert (b.router.groups, b.router.keep, b.shared_ff) == (1, 1, None) and b.mixer.rot.scaling is None
    assert n.ff is None and n.mixer.rot is None
    bad = U.make_config([U.retention_layer(heads=2, decay=[0.5])])
    with pytest.raises(ValueError):
        HybridConfig.from_json(bad)
    with pytest.raises(NotImplementedError):
        HybridConfig.from_json({**cfg, "layers": [{"type": "conv", "mixer": {}, "mlp": None}]})
    with pytest.raises(NotImplementedError):
        HybridConfig.from_json({**cfg, "architecture": "Unknown"})


def test_rotary_steps_with_frequency_scaling():
    from rtp_llm_amd.mixers import RotarySpec, rotary_table
    for rot in ({"base": 1e4, "dims": 16}, {"base": 5e5, "dims": 32, "scaling": U.YARN}, {"base": 100.0, "dims": 8, "scaling": {"factor": 16.0, "original": 4096, "fast": 64.0, "slow": 2.0}}):
        f, mag = rotary_table(RotarySpec.from_json(rot, "halves"), "cpu")
        rf, rmag = O.rotary_table(rot)
        assert abs(mag - rmag) < 1e-12 and float((f.double() - rf).abs().max() / rf.max()) < 1e-7
    sc = O.rotary_table({"base": 5e5, "dims": 32, "scaling": U.YARN})[0] / O.rotary_table({"base": 5e5, "dims": 32})[0]
    assert float(sc[0]) == 1.0 and abs(float(sc[-1]) - 0.25) < 1e-12 and 0.25 < float(sc[2]) < float(sc[1]) < 1.0   # fast pairs keep their step, slow ones are divided




def test_oracle_retention_equals_the_explicit_decayed_sum():
    cfg = U.make_config([U.retention_layer(heads=2, dim=8, vdim=6, rot_dims=4, decay=[0.75, 1.0])], width=16)
    w = {k: v.double() for k, v in U.make_weights(cfg, seed=1).items()}
    mx = cfg["layers"][0]["mixer"]
    h = torch.randn(12, 16, dtype=torch.float64, generator=torch.Generator().manual_seed(2))
    pos = torch.arange(12)
    q = O.rotate((h @ w["l0.mix.q"].T).view(12, 2, 8), pos, mx["rot"], "halves")
    k = O.rotate((h @ w["l0.mix.k"].T).view(12, 2, 8), pos, mx["rot"], "halves") * 8 ** -0.5
    v = (h @ w["l0.mix.v"].T).view(12, 2, 6)
    o = torch.zeros(12, 2, 6, dtype=torch.float64)
    for t in range(12):
        for j in range(t + 1):
            for hh in range(2):
                o[t, hh] += mx["decay"][hh] ** (t - j) * (q[t, hh] @ k[j, hh]) * v[j, hh]
    ref = (O.rms_unit(o, 1e-5).reshape(12, 12) * torch.nn.functional.silu(h @ w["l0.mix.g"].T)) @ w["l0.mix.o"].T
    assert float((O.retention(h, w, "l0.mix.", mx, 1e-5) - ref).abs().max()) < 1e-10


def test_oracle_rotation_depends_on_distance_only_and_pairs_are_where_they_should_be():
    rot = {"base": 50.0, "dims": 4}
    x = torch.randn(1, 1, 6, dtype=torch.float64, generator=torch.Generator().manual_seed(3))
    y = torch.randn(1, 1, 6, dtype=torch.float64, generator=torch.Generator().manual_seed(4))
    for layout in ("interleaved", "halves"):
        d = [float((O.rotate(x, torch.tensor([p]), rot, layout) * O.rotate(y, torch.tensor([p - 3]), rot, layout)).sum()) for p in (3, 10, 200)]
        assert max(d) - min(d) < 1e-9
        assert torch.equal(O.rotate(x, torch.tensor([7]), rot, layout)[..., 4:], x[..., 4:])          # channels past the span pass
    one = torch.zeros(1, 1, 6, dtype=torch.float64); one[..., 0] = 1.0
    assert float(O.rotate(one, torch.tensor([1]), rot, "interleaved")[0, 0, 1]) > 0.5                # partner of 0 is 1 ...
    assert float(O.rotate(one, torch.tensor([1]), rot, "halves")[0, 0, 2]) > 0.5                     # ... or 2 = 0 + dims / 2


def test_oracle_routing_respects_groups():
    z = torch.tensor([[5.0, 0.0, 0.0, 4.9, 4.8, 0.0]], dtype=torch.float64)
    eye = {"r.router": torch.eye(6, dtype=torch.float64)}
    ids, wts = O.route(z, eye, "r.", {"experts": 6, "top": 2})
    assert ids.tolist() == [[0, 3]]
    ids, wts = O.route(z, eye, "r.", {"experts": 6, "top": 2, "groups": {"count": 3, "keep": 1}})    # groups {0,1} {2,3} {4,5}: only the first stays
    assert ids.tolist() == [[0, 1]] and abs(float(wts.sum()) - float(torch.softmax(z, -1)[0, :2].sum())) < 1e-12
    ids, _ = O.route(z, eye, "r.", {"experts": 6, "top": 2, "groups": {"count": 2, "keep": 1}})      # groups {0,1,2} {3,4,5}
    assert ids.tolist() == [[0, 1]] or ids.tolist() == [[0, 2]]
