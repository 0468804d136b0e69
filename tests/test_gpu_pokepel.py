"""The Pokepel member of the hybrid family on the GPU against the plain implementation in pokepel_oracle (float64, CPU): every mechanism
alone, whole prompts against token-by-token decoding, portions, unequal batches, reused pages and slots, far keys and page edges with
weights built so that one key dominates, the softmax sink, long decoding, other sizes, graph replay, and greedy generation through the
scheduler and the command line."""
import json
import os
import subprocess
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import pokepel_oracle as O  # noqa: E402
import pokepel_util as U  # noqa: E402

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def engine(cfg, w, dtype=torch.float32, max_tokens=1024, max_seqs=4, **kw):
    from rtp_llm_amd.hybrid import HybridConfig, HybridModel
    from rtp_llm_amd.scheduler import ServingEngine
    return ServingEngine(HybridModel(HybridConfig.from_json(cfg), w, dtype, DEV), max_tokens=max_tokens, max_seqs=max_seqs, **kw)


def toks(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def close(got, ref, tol):
    err = float((got.double().cpu() - ref).abs().max())
    assert err <= tol, f"max |error| {err} > {tol}"


def whole(eng, t, sid="s"):
    out = eng.run_step([(sid, t, range(len(t)))])
    eng.release(sid)
    return out


FULL = [U.retention_layer(mlp=U.dense()), U.latent_layer(scaling=U.YARN, mlp=U.moe()), U.retention_layer(heads=3, dim=8, vdim=40, rot_dims=4, mlp=U.moe(shared=None)),
        U.latent_layer(heads=2, dim=24, rot_dim=4, vdim=8, kv_rank=28, mlp=U.dense(ff=40)), U.latent_layer(mlp=None)]


# ------------------------------------------------------------------------------------------------ single operations
def test_grouped_linear_heads_and_sorted_rows():
    from rtp_llm_amd import hybrid_ops as hops
    g = torch.Generator(device=DEV).manual_seed(1)
    for dt, tol in ((torch.float32, 2e-5), (torch.bfloat16, 2e-5)):
        for M, G, N, K in [(1, 3, 40, 16), (5, 2, 24, 8), (70, 5, 130, 72), (200, 1, 64, 40), (17, 4, 96, 20)]:
            x = torch.randn(M, G * K + 8, device=DEV, generator=g).to(dt)
            w = (torch.randn(G, N, K, device=DEV, generator=g) * K ** -0.5).to(dt)
            y = hops.dense_grouped(x, w, x_step=K, y_step=N + 3, out_dtype=torch.float32)
            for j in range(G):
                close(y[:, j * (N + 3):j * (N + 3) + N], (x[:, j * K:(j + 1) * K].double() @ w[j].double().T).cpu(), tol)
            gate = torch.randn(M, G * N + 5, device=DEV, generator=g)                # outputs times the sigmoid of a slice of a wider buffer
            y = hops.dense_grouped(x, w, x_step=K, y_step=N, out_dtype=torch.float32, mul_sigmoid=gate[:, 2:2 + G * N])
            ref = torch.cat([x[:, j * K:(j + 1) * K].double() @ w[j].double().T for j in range(G)], 1) * torch.sigmoid(gate[:, 2:2 + G * N].double())
            close(y, ref.cpu(), tol)
        # rows sorted by group with a gather on the input, empty groups, groups larger than a tile; gated epilogue
        E, K, ff, T = 6, 40, 32, 90
        for counts in ([0, 75, 1, 0, 130, 3], [0, 2, 1, 0, 5, 3], [0, 0, 0, 1, 0, 0]):      # prompt-sized, and the few rows of a decode step
            n = sum(counts)
            offs = torch.tensor([0] + list(torch.tensor(counts).cumsum(0)), dtype=torch.int32, device=DEV)
            src = torch.randint(0, T, (n,), generator=torch.Generator().manual_seed(2)).to(torch.int32).to(DEV)
            x = torch.randn(T, K, device=DEV, generator=g).to(dt)
            gt, up = [(torch.randn(E, ff, K, device=DEV, generator=g) * 0.2).to(dt) for _ in range(2)]
            wgu = torch.stack([hops.group_gate_up(gt[e], up[e]) for e in range(E)]).contiguous()
            a = hops.dense_grouped(x, wgu, offs=offs, gather=src, rows=n, gated=True, act=hops.ACT_SILU, out_dtype=torch.float32)
            wd = (torch.randn(E, 24, ff, device=DEV, generator=g) * 0.2).to(dt)
            xs = torch.randn(n, ff, device=DEV, generator=g).to(dt)
            y = hops.dense_grouped(xs, wd, offs=offs, rows=n, out_dtype=torch.float32)
            tl = [(e, m) for e in range(E) for m in range(int(offs[e]), int(offs[e + 1]), 64)]
            tiles = torch.tensor([len(tl)] + [v for pr in tl for v in pr] + [0, 0], dtype=torch.int32, device=DEV)      # the same through a tile list
            assert torch.equal(y, hops.dense_grouped(xs, wd, offs=offs, tiles=tiles, rows=n, out_dtype=torch.float32))
            at = 0
            for e, c in enumerate(counts):
                if not c:
                    continue
                xe = x[src[at:at + c].long()].double()
                close(a[at:at + c], (torch.nn.functional.silu(xe @ gt[e].double().T) * (xe @ up[e].double().T)).cpu(), tol)
                close(y[at:at + c], (xs[at:at + c].double() @ wd[e].double().T).cpu(), tol)
                at += c


def test_gated_branches_join_the_stream():
    from rtp_llm_amd import hybrid_ops as hops
    g = torch.Generator().manual_seed(3)
    for W in (8, 50, 64, 1000):
        x, a, b = [torch.randn(7, W, generator=g) for _ in range(3)]
        gate = torch.randn(7, 2 * W + 4, generator=g) * 2
        w1 = 1.0 + torch.randn(W, generator=g) * 0.2
        xd = x.to(DEV)
        h1, none = hops.residual_norm(xd, a.to(DEV), b.to(DEV), 1.0, w1.to(DEV), None, 1e-6, gate=gate.to(DEV))
        xn = x.double() + torch.sigmoid(gate[:, :W].double()) * a.double() + torch.sigmoid(gate[:, W:2 * W].double()) * b.double()
        close(xd, xn, 1e-5)
        close(h1, O.rms_unit(xn, 1e-6) * w1.double(), 1e-4)
        xd = x.to(DEV)                                          # the mixer's branch alone
        hops.residual_norm(xd, a.to(DEV), None, 1.0, w1.to(DEV), None, 1e-6, gate=gate.to(DEV))
        close(xd, x.double() + torch.sigmoid(gate[:, :W].double()) * a.double(), 1e-5)
        # the second branch as a mixture's weighted sum formed inside the kernel (with and without a shared expert's output), also under a row gather
        y, wts = torch.randn(21, W, generator=g), torch.rand(7, 3, generator=g)
        place = torch.randperm(21, generator=g).to(torch.int32).view(7, 3)
        mix = (wts.double()[:, :, None] * y.double()[place.long()]).sum(1)
        for extra in (b, None):
            ms = hops.MoeSum(y.to(DEV), place.to(DEV), wts.to(DEV), None if extra is None else extra.to(DEV))
            want = mix + (0 if extra is None else extra.double())
            close(hops.moe_combine(ms), want, 1e-5)
            xd = x.to(DEV)
            h1, _ = hops.residual_norm(xd, a.to(DEV), ms, 1.0, w1.to(DEV), None, 1e-6, gate=gate.to(DEV))
            xn = x.double() + torch.sigmoid(gate[:, :W].double()) * a.double() + torch.sigmoid(gate[:, W:2 * W].double()) * want
            close(xd, xn, 1e-5)
            close(h1, O.rms_unit(xn, 1e-6) * w1.double(), 1e-4)
            xd = x.to(DEV)
            rows = torch.tensor([6, 2], dtype=torch.int32, device=DEV)
            h3, _ = hops.residual_norm(xd, a.to(DEV), ms, 1.0, w1.to(DEV), None, 1e-6, gate=gate.to(DEV), rows=rows)
            close(h3, (O.rms_unit(xn, 1e-6) * w1.double())[[6, 2]], 1e-4)
            close(xd, x.double(), 0.0)


def test_polynorm_activation():
    from rtp_llm_amd import hybrid_ops as hops
    g = torch.Generator().manual_seed(4)
    for n in (5, 64, 300, 1111):
        z = torch.randn(9, n, generator=g) * 1.5
        coef = (0.7, -0.4, 0.2, 0.05)
        ref = sum(c * O.rms_unit(z.double() ** (k + 1), 1e-5) for k, c in enumerate(coef[:3])) + coef[3]
        close(hops.polynorm(z.to(DEV), coef, 1e-5, torch.float32), ref, 1e-5)


@pytest.mark.parametrize("E,groups,keep,top", [(8, 4, 2, 2), (12, 3, 1, 3), (6, 1, 1, 1), (64, 8, 4, 6), (130, 2, 2, 5), (9, 9, 3, 3)])
def test_router_choices_and_weights(E, groups, keep, top):
    from rtp_llm_amd import hybrid_ops as hops
    z = torch.randn(100, E, generator=torch.Generator().manual_seed(E)) * 3
    ids, wts = hops.moe_route(z.to(DEV), groups, keep, top)
    router = {"experts": E, "top": top, "groups": {"count": groups, "keep": keep}}
    want_ids, want_w = O.route(z.double(), {"r.router": torch.eye(E, dtype=torch.float64)}, "r.", router)       # identity router: logits = z
    assert torch.equal(ids.cpu().long(), want_ids)
    close(wts, want_w, 1e-6)
    def check_sort(ids, offs, src, place, tiles):
        offs, src, place, tiles = offs.cpu(), src.cpu(), place.cpu(), tiles.cpu().tolist()
        want_tiles = [(e, m) for e in range(E) for m in range(int(offs[e]), int(offs[e + 1]), 64)]
        assert tiles[0] == len(want_tiles) and list(zip(tiles[1:1 + 2 * tiles[0]:2], tiles[2:2 + 2 * tiles[0]:2])) == want_tiles
        flat = ids.cpu().flatten()
        assert offs[0] == 0 and offs[-1] == flat.numel() and sorted(place.tolist()) == list(range(flat.numel()))
        for i, e in enumerate(flat.tolist()):
            assert offs[e] <= place[i] < offs[e + 1] and src[place[i]] == i // top

    check_sort(ids, *hops.moe_align(ids, E))
    for T in (1, 17, 50, 100):                                   # up to 64 tokens: routing and sorting in one launch; more: the two launches
        got = hops.moe_route_sorted(z[:T].to(DEV), E, groups, keep, top)
        assert torch.equal(got[0].cpu().long(), want_ids[:T])
        close(got[1], want_w[:T], 1e-6)
        check_sort(got[0], *got[2:])


# ------------------------------------------------------------------------------------------------ mechanisms alone
ALONE = {
    "latent": U.latent_layer(),
    "latent_scaled_rotary": U.latent_layer(scaling=U.YARN, base=300.0),
    "latent_one_head_rank_not_of_8": U.latent_layer(heads=1, dim=12, rot_dim=6, vdim=10, kv_rank=22),
    "latent_row_fills_its_padding": U.latent_layer(heads=4, dim=8, rot_dim=16, vdim=72, kv_rank=48),
    "latent_wide_rank": U.latent_layer(heads=2, dim=40, rot_dim=32, vdim=16, kv_rank=200),
    "latent_rank_over_256": U.latent_layer(heads=2, dim=16, rot_dim=16, vdim=16, kv_rank=336),
    "latent_odd_rank": U.latent_layer(heads=3, dim=8, rot_dim=8, vdim=12, kv_rank=27),
    "latent_no_rotated_part_scaled": U.latent_layer(heads=5, dim=16, rot_dim=2, vdim=16, kv_rank=16, scale=0.5),
    "retention": U.retention_layer(),
    "retention_partial_rotary": U.retention_layer(heads=3, dim=24, vdim=16, rot_dims=8),
    "retention_no_rotary_one_head": U.retention_layer(heads=1, dim=40, vdim=72, rot_dims=0, decay=[0.9]),
    "retention_scaled_rotary_long_keys": U.retention_layer(heads=2, dim=160, vdim=8, scaling=U.YARN, decay=[0.5, 1.0]),
    "polynorm_mlp": U.retention_layer(heads=1, dim=8, vdim=8, mlp=U.dense(ff=100)),
    "experts_grouped": U.retention_layer(heads=1, dim=8, vdim=8, mlp=U.moe()),
    "experts_plain_top1_no_shared": U.retention_layer(heads=1, dim=8, vdim=8, mlp=U.moe(experts=5, top=1, groups=None, shared=None, ff=24)),
    "experts_top3_of_one_group": U.latent_layer(mlp=U.moe(experts=12, top=3, groups=3, keep=1, ff=40, shared=8)),
    "experts_all_groups_kept": U.latent_layer(mlp=U.moe(experts=6, top=4, groups=3, keep=3, ff=64, shared=64)),
}


@pytest.mark.parametrize("name", sorted(ALONE))
def test_one_layer_models(name):
    cfg = U.make_config([ALONE[name]], vocab=80, width=48)
    w = U.make_weights(cfg, seed=3)
    t = toks(70, 80, 4)
    col, ocol = [], []
    ref = U.oracle_logits(cfg, w, t, ocol)
    eng = engine(cfg, w)
    got = eng.run_step([("x", t, range(len(t)))], collect=col)
    close(col[0], ocol[0], 2e-4)
    close(got, ref, 2e-4)
    eng.release("x")
    one = torch.cat([eng.run_step([("d", [tk], [0])]) for tk in t[:20]])       # and token by token from the first token on
    close(one, ref[:20], 2e-4)


def test_all_mechanisms_together_residual_stream_and_bf16():
    cfg = U.make_config(FULL)
    w = U.make_weights(cfg, seed=5)
    t = toks(90, cfg["vocab"], 6)
    ocol = []
    ref = U.oracle_logits(cfg, w, t, ocol)
    col = []
    got = engine(cfg, w).run_step([("x", t, range(len(t)))], collect=col)
    assert len(col) == len(FULL)
    for a, b in zip(col, ocol):
        close(a, b, 3e-4)
    close(got, ref, 3e-4)
    scale = float(ref.pow(2).mean().sqrt())
    for tiles in (True, False):                                    # prompt attention on the matrix cores and on the row kernel
        eng = engine(cfg, w, torch.bfloat16)
        for _, mixer, *_ in eng.model.layers:
            mixer.use_tiles = tiles
        d = whole(eng, t).double().cpu() - ref
        assert float(d.pow(2).mean().sqrt()) < 0.05 * scale, "bf16 step is off by more than rounding"


# ------------------------------------------------------------------------------------------------ schedules
def test_prefill_against_token_by_token_and_first_tokens():
    cfg = U.make_config(FULL)
    w = U.make_weights(cfg, seed=9)
    t = toks(75, cfg["vocab"], 10)
    ref = U.oracle_logits(cfg, w, t)
    eng = engine(cfg, w)
    close(whole(eng, t), ref, 3e-4)
    one = torch.cat([eng.run_step([("d", [tk], [0])]) for tk in t])
    eng.release("d")
    close(one, ref, 3e-4)
    for n in (1, 2, 3):                                            # the shortest sequences
        close(whole(eng, t[:n]), ref[:n], 3e-4)


@pytest.mark.parametrize("sizes", [[2] * 30, [33, 2, 31, 5, 64, 1, 1, 2, 60], [63, 1, 64, 65, 6], [1, 198]])
def test_portions(sizes):
    cfg = U.make_config(FULL)
    w = U.make_weights(cfg, seed=11)
    n = sum(sizes)
    t = toks(n, cfg["vocab"], 12)
    ref = U.oracle_logits(cfg, w, t)
    eng = engine(cfg, w)
    at, outs = 0, []
    for s in sizes:
        outs.append(eng.run_step([("p", t[at:at + s], range(s))]))
        at += s
    close(torch.cat(outs), ref, 3e-4)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 3e-4), (torch.bfloat16, None)])
def test_unequal_batches_reused_pages_and_slots(dtype, tol):
    cfg = U.make_config(FULL)
    w = U.make_weights(cfg, seed=13)
    lens = {"a": 150, "b": 9, "c": 70, "d": 131, "e": 64, "f": 40}
    seqs = {k: toks(n, cfg["vocab"], 20 + i) for i, (k, n) in enumerate(lens.items())}
    ref = {k: U.oracle_logits(cfg, w, v) for k, v in seqs.items()}
    # pool: 7 pages of 64 and 3 slots -- less than the requests need together, so pages and slots come back and go out again
    eng = engine(cfg, w, dtype, max_tokens=7 * 64, max_seqs=3)
    plan = [
        [("a", 100), ("b", 4)],
        [("a", 1), ("b", 1), ("c", 30)],
        [("b", 4), ("c", 40), ("a", 49)],            # a, b, c complete -> released
        [("d", 2), ("e", 64)],
        [("d", 129), ("f", 3)],                      # d, e complete
        [("f", 1)], [("f", 36)],
    ]
    at = {k: 0 for k in seqs}
    got = {k: [] for k in seqs}
    for step in plan:
        entries = [(k, seqs[k][at[k]:at[k] + n], range(n)) for k, n in step]
        out = eng.run_step(entries)
        o = 0
        for k, n in step:
            got[k].append(out[o:o + n]); o += n; at[k] += n
            if at[k] == lens[k]:
                eng.release(k)
    assert eng.cache.pages.free == 7 and eng.cache.slots.free == 3
    for k in seqs:
        if tol is not None:
            close(torch.cat(got[k]), ref[k], tol)
        else:
            d = torch.cat(got[k]).double().cpu() - ref[k]
            assert float(d.pow(2).mean().sqrt()) < 0.05 * float(ref[k].pow(2).mean().sqrt())
    with pytest.raises(MemoryError):
        eng.run_step([("big", toks(8 * 64, cfg["vocab"], 1), [])])


# ------------------------------------------------------------------------------------------------ far keys and page edges, with one key that dominates
def _beacon_model(sink=-30.0, heads=2, dim=16, rot_dim=8, vdim=16, kv_rank=24, width=32, vocab=40):
    """One latent-attention layer in which token 1 (the beacon) caches a latent that the query of token 2 (the asker) scores about 25 above
    every other key, through an un-rotated channel; the beacon's value is far from the others'.  Seeing or not seeing the beacon moves the
    asker's logits by a lot.  The sinks are far below every score unless asked otherwise."""
    cfg = U.make_config([U.latent_layer(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=kv_rank, scale=1.0)], vocab=vocab, width=width)
    w = U.make_weights(cfg, seed=17)
    w["l0.mix.q"] *= 0.05
    w["l0.mix.dkv"] *= 0.05
    w["l0.norm1"].fill_(1.0)
    w["l0.mix.dkv.norm"].fill_(1.0)
    w["l0.mix.sink"].fill_(sink)
    w["l0.mix.g"].zero_()                               # output gate one half everywhere
    w["l0.rg1"].zero_(); w["l0.rg1.b"].fill_(4.0)
    e = torch.randn(vocab, width, generator=torch.Generator().manual_seed(18)) * 0.05
    e[:, :2] = 0.0                                      # only the beacon and the asker live on the first two axes
    e[1], e[2] = 0.0, 0.0
    e[1, 0], e[2, 1] = 1.0, 1.0                         # after the norm: sqrt(width) on that axis
    w["embed"] = e.bfloat16().float()
    # the beacon's latent is (nearly) one-hot on channel 0 -> after its norm sqrt(kv_rank) there; head h's key reads it into channel 0
    w["l0.mix.dkv"][0] = 0.0
    w["l0.mix.dkv"][0, 0] = 4.0
    w["l0.mix.uk"].mul_(0.2)
    for h in range(heads):
        w["l0.mix.uk"][h * dim] = 0.0
        w["l0.mix.uk"][h * dim, 0] = 1.0
        w["l0.mix.q"][h * (dim + rot_dim), 1] = 25.0 / (width ** 0.5 * kv_rank ** 0.5)
    w["l0.mix.uv"][:, 0] = 3.0
    return cfg, {k: v.bfloat16().float() for k, v in w.items()}


@pytest.mark.parametrize("beacon,asker", [(0, 250), (3, 299), (63, 290), (64, 290), (127, 128), (128, 191), (190, 191), (1, 2)])
def test_dominant_key_far_back_and_at_page_edges_prompt_and_decoded(beacon, asker):
    cfg, w = _beacon_model()
    t = [3 + (i % 30) for i in range(asker + 1)]
    t[beacon], t[asker] = 1, 2
    ref = U.oracle_logits(cfg, w, t)
    t2 = list(t); t2[beacon] = 5
    assert float((U.oracle_logits(cfg, w, t2)[asker] - ref[asker]).abs().max()) > 0.05, "the beacon must move the asker's logits"
    for dtype, tol in ((torch.float32, 3e-4), (torch.bfloat16, 0.05 * float(ref[asker].abs().max()) + 0.05)):
        eng = engine(cfg, w, dtype)
        close(eng.run_step([("w", t, [asker])]), ref[asker:asker + 1], tol)              # in a prompt
        eng.release("w")
        eng.run_step([("d", t[:asker], [])])
        close(eng.run_step([("d", [t[asker]], [0])]), ref[asker:asker + 1], tol)         # decoded alone
        eng.release("d")
        cut = max(1, beacon)                                                              # a portion that starts at the beacon
        eng.run_step([("p", t[:cut], [])])
        close(eng.run_step([("p", t[cut:], [asker - cut])]), ref[asker:asker + 1], tol)


def test_sink_takes_its_share_of_the_softmax():
    """With one head's sink far above its scores that head's output vanishes; far below, it is a plain softmax: both must match, and differ."""
    outs = []
    for sinks in ((12.0, -30.0), (-30.0, 12.0), (0.5, -0.5)):
        cfg, w = _beacon_model()
        w["l0.mix.sink"] = torch.tensor(sinks)
        t = [3 + (i % 30) for i in range(100)]
        ref = U.oracle_logits(cfg, w, t)
        outs.append(ref)
        eng = engine(cfg, w)
        close(whole(eng, t), ref, 3e-4)
        eng.run_step([("d", t[:70], [])])
        close(torch.cat([eng.run_step([("d", [tk], [0])]) for tk in t[70:]]), ref[70:], 3e-4)
        close(whole(engine(cfg, w, torch.bfloat16), t), ref, 0.05 * float(ref.abs().max()) + 0.05)
    assert float((outs[0] - outs[1]).abs().max()) > 0.05 and float((outs[0] - outs[2]).abs().max()) > 0.05


def test_retention_state_carries_a_far_token():
    """A beacon at position 2 whose key the asker's query meets through an un-rotated channel (every other key has a zero there) must still
    steer the asker hundreds of tokens later through the slow head's state; the fast head has forgotten it."""
    W, d = 32, 16
    cfg = U.make_config([U.retention_layer(heads=2, dim=d, vdim=16, rot_dims=8, decay=[1.0 - 2.0 ** -10, 0.5])], vocab=40, width=W)
    w = U.make_weights(cfg, seed=19)
    w["l0.norm1"].fill_(1.0)
    e = torch.randn(40, W, generator=torch.Generator().manual_seed(20)) * 0.05
    e[:, :2] = 0.0
    e[1], e[2] = 0.0, 0.0
    e[1, 0], e[2, 1] = 1.0, 1.0
    w["embed"] = e
    for hh in range(2):
        w["l0.mix.k"][hh * d + d - 1] = 0.0
        w["l0.mix.q"][hh * d + d - 1] = 0.0
        w["l0.mix.k"][hh * d + d - 1, 0] = 2.0
        w["l0.mix.q"][hh * d + d - 1, 1] = 2.0
    w = {k: v.bfloat16().float() for k, v in w.items()}
    t = [3 + (i % 30) for i in range(400)]
    t[2], t[399] = 1, 2
    ref = U.oracle_logits(cfg, w, t)
    t2 = list(t); t2[2] = 7
    assert float((U.oracle_logits(cfg, w, t2)[-1] - ref[-1]).abs().max()) > 0.05
    eng = engine(cfg, w)
    close(whole(eng, t)[-1:], ref[-1:], 3e-4)
    eng.run_step([("d", t[:350], [])])
    out = torch.cat([eng.run_step([("d", [tk], [0])]) for tk in t[350:]])
    close(out, ref[350:], 3e-4)
    eng.release("d")
    eng.run_step([("p", t[:2], [])])                                    # a portion that starts at the beacon, then two-token portions
    eng.run_step([("p", t[2:395], [])])
    out = torch.cat([eng.run_step([("p", t[395:397], [0, 1])]), eng.run_step([("p", t[397:399], [0, 1])]), eng.run_step([("p", t[399:], [0])])])
    close(out, ref[395:], 3e-4)


def test_long_decoding():
    cfg = U.make_config([U.latent_layer(scaling=U.YARN, mlp=U.moe()), U.retention_layer(mlp=U.dense()), U.latent_layer(heads=2, kv_rank=56, mlp=U.moe(top=1))])
    w = U.make_weights(cfg, seed=23)
    t = toks(330, cfg["vocab"], 24)
    ref = U.oracle_logits(cfg, w, t)
    eng = engine(cfg, w)
    eng.run_step([("d", t[:10], [])])
    out = torch.cat([eng.run_step([("d", [tk], [0])]) for tk in t[10:]])
    close(out, ref[10:], 5e-4)


# ------------------------------------------------------------------------------------------------ generation
def _oracle_greedy(cfg, w, prompt, n):
    seq, margins = list(prompt), []
    for _ in range(n):
        lg = U.oracle_logits(cfg, w, seq)[-1]
        top = lg.topk(2).values
        margins.append(float(top[0] - top[1]))
        seq.append(int(lg.argmax()))
    return seq[len(prompt):], margins


def test_greedy_generation_through_the_scheduler():
    cfg = U.make_config([U.retention_layer(mlp=U.dense()), U.latent_layer(mlp=U.moe()), U.retention_layer(mlp=U.moe(top=1, shared=None))], vocab=64, width=48)
    w = U.make_weights(cfg, seed=29)
    prompts = [toks(n, 64, 30 + n) for n in (5, 40, 1, 70, 18, 33)]            # six requests over three slots: some wait their turn
    eng = engine(cfg, w, max_tokens=5 * 64, max_seqs=3, max_step_tokens=48)     # prompts are cut into portions of the step budget
    outs = eng.generate(prompts, 12)
    assert eng.cache.pages.free == 5 and eng.cache.slots.free == 3 and not eng.running and not eng.waiting
    for p, o in zip(prompts, outs):
        ref, margins = _oracle_greedy(cfg, w, p, 12)
        for i, (a, b) in enumerate(zip(o, ref)):
            if a != b:
                assert margins[i] < 1e-3, f"token {i}: {a} != {b} with a top-2 margin of {margins[i]}"
                break
    eng.use_graphs = True                                                        # decode-only steps as replayed graphs give the same tokens
    assert eng.generate(prompts[:3], 12) == outs[:3]
    sampled = eng.generate(prompts[:2], 6, top_k=5, top_p=0.9, temperature=0.8, seed=3)
    assert sampled == eng.generate(prompts[:2], 6, top_k=5, top_p=0.9, temperature=0.8, seed=3)
    assert all(len(o) == 6 and all(0 <= x < 64 for x in o) for o in sampled)


def test_command_line_generate_and_trace(tmp_path):
    from safetensors.torch import save_file
    cfg = U.make_config([U.latent_layer(mlp=U.moe()), U.retention_layer(mlp=U.dense())], vocab=64, width=48)
    w = U.make_weights(cfg, seed=31)
    d = tmp_path / "model"
    d.mkdir()
    (d / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.bfloat16().contiguous() for k, v in w.items()}, str(d / "model.safetensors"))
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    p = toks(21, 64, 32)
    r = subprocess.run([sys.executable, "-m", "rtp_llm_amd.cli", "generate", "--model", str(d), "--dtype", "float32", "--max-new-tokens", "5",
                        "--prompt-ids", ",".join(map(str, p))], cwd=root, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    gen = json.loads(r.stdout.strip().splitlines()[-1])["generated"]
    ref, margins = _oracle_greedy(cfg, w, p, 5)
    assert gen == ref or min(margins) < 1e-3
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": p[:9], "want": [8]}, {"id": "b", "tokens": p[:2], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": p[9:], "want": [0, 11]}], "end": ["a", "b"]}]
    out = tmp_path / "out"
    r = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", str(d), "--dtype", "float32", "--out", str(out), "--max-tokens", "128"],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", cwd=root, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "done 0" in r.stdout and "done 1" in r.stdout, r.stderr[-2000:]
    import numpy as np
    full = U.oracle_logits(cfg, w, p)
    close(torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4").reshape(1, -1)), full[8:9], 3e-4)
    close(torch.from_numpy(np.fromfile(out / "1.f32", dtype="<f4").reshape(2, -1)), full[[9, 20]], 3e-4)


def test_graph_replayed_decode_steps_match_eager_and_oracle():
    """Decode steps through the captured graph (routing, sorting by expert and the grouped linears replay without the host), with eager
    prompt portions and eager decode steps between the replays."""
    cfg = U.make_config(FULL)
    w = U.make_weights(cfg, seed=37)
    seqs = {k: toks(n, cfg["vocab"], 40 + i) for i, (k, n) in enumerate({"a": 90, "b": 61, "c": 75}.items())}
    ref = {k: U.oracle_logits(cfg, w, v) for k, v in seqs.items()}
    eng = engine(cfg, w)
    eng.run_step([("a", seqs["a"][:50], []), ("b", seqs["b"][:30], [])])
    at = {"a": 50, "b": 30, "c": 0}
    for i in range(30):
        eng.use_graphs = i % 3 != 2                                   # every third decode step runs eagerly
        out = eng.run_step([(k, [seqs[k][at[k]]], [0]) for k in ("a", "b")])
        for j, k in enumerate(("a", "b")):
            close(out[j:j + 1], ref[k][at[k]:at[k] + 1], 3e-4)
            at[k] += 1
        if i == 10:                                                   # an eager prefill step between replays
            eng.use_graphs = True
            eng.run_step([("c", seqs["c"][:70], [])]); at["c"] = 70
    eng.use_graphs = True
    out = eng.run_step([(k, [seqs[k][at[k]]], [0]) for k in ("a", "b", "c")])     # another shape: a second graph
    for j, k in enumerate(("a", "b", "c")):
        close(out[j:j + 1], ref[k][at[k]:at[k] + 1], 3e-4)
    assert len(eng._graphs) == 2
