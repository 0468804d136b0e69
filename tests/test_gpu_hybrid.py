"""The hybrid decoder family on the GPU against the plain implementation in hybrid_oracle (float64, CPU): every mechanism alone, whole
prompts against token-by-token decoding, portions, unequal batches, reused pages and slots, mask / page edges with weights built so
that one key dominates, long decoding, other sizes, and greedy generation through the scheduler and the command line."""
import json
import os
import subprocess
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import hybrid_util as U  # noqa: E402

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
    assert err <= tol, f"max |logit error| {err} > {tol}"


def whole(eng, t, sid="s"):
    out = eng.run_step([(sid, t, range(len(t)))])
    eng.release(sid)
    return out


FULL = [U.gla_layer(), U.attention_layer(), U.hgrn2_layer(), U.attention_layer(kv_from=1), U.gla_layer(heads=1, dim=40, vdim=72, ff=None)]


# ------------------------------------------------------------------------------------------------ mechanisms alone
def test_dense_linear_shapes_and_epilogues():
    from rtp_llm_amd import hybrid_ops as hops
    g = torch.Generator(device=DEV).manual_seed(1)
    for dt, tol in ((torch.float32, 2e-5), (torch.bfloat16, 2e-5)):
        for M, N, K in [(1, 40, 64), (3, 72, 200), (9, 64, 16), (17, 130, 72), (70, 96, 20), (150, 264, 328), (16, 8, 12)]:
            x = torch.randn(M, K, device=DEV, generator=g).to(dt)
            w = (torch.randn(N, K, device=DEV, generator=g) * K ** -0.5).to(dt)
            b = torch.randn(N, device=DEV, generator=g).to(dt)
            ref = x.double() @ w.double().T + b.double()
            close(hops.dense_linear(x, w, b, out_dtype=torch.float32), ref.cpu(), tol)
            close(hops.dense_linear(x, w, None, out_dtype=torch.float32, softcap=3.0), (3.0 * torch.tanh((x.double() @ w.double().T) / 3.0)).cpu(), tol)
        for M, ff in [(2, 32), (11, 96), (80, 160)]:
            x = torch.randn(M, 72, device=DEV, generator=g).to(dt)
            gt, up = [(torch.randn(ff, 72, device=DEV, generator=g) * 0.1).to(dt) for _ in range(2)]
            for act, fn in ((hops.ACT_RELU, torch.relu), (hops.ACT_SILU, torch.nn.functional.silu)):
                ref = fn(x.double() @ gt.double().T) * (x.double() @ up.double().T)
                close(hops.dense_linear(x, hops.group_gate_up(gt, up), gated=True, act=act, out_dtype=torch.float32), ref.cpu(), tol)
    # a column slice of a wider buffer as input, a 16-bit output
    x = torch.randn(20, 96, device=DEV, generator=g).bfloat16()
    w = (torch.randn(24, 32, device=DEV, generator=g) * 0.2).bfloat16()
    y = hops.dense_linear(x[:, 64:], w)
    assert y.dtype == torch.bfloat16
    close(y.float(), (x[:, 64:].double() @ w.double().T).cpu(), 3e-2)


def test_residual_and_offset_norms():
    import hybrid_oracle as O
    from rtp_llm_amd import hybrid_ops as hops
    g = torch.Generator().manual_seed(2)
    for W in (8, 50, 64, 1000):
        x, a, b = [torch.randn(7, W, generator=g) for _ in range(3)]
        w1, w2 = torch.randn(W, generator=g) * 0.2, torch.randn(W, generator=g) * 0.2
        xd = x.to(DEV)
        h1, h2 = hops.residual_norm(xd, a.to(DEV), b.to(DEV), 0.3, w1.to(DEV), w2.to(DEV), 1e-5, weight_offset=1.0)
        xn = x.double() + 0.3 * (a.double() + b.double())
        close(xd, xn, 1e-5)
        close(h1, O.offset_norm(xn, w1.double(), 1e-5), 1e-4)
        close(h2, O.offset_norm(xn, w2.double(), 1e-5), 1e-4)
        rows = torch.tensor([5, 0, 5], dtype=torch.int32, device=DEV)
        h3, none = hops.residual_norm(xd, None, a.to(DEV), 2.0, w1.to(DEV), None, 1e-5, weight_offset=0.0, rows=rows)
        assert none is None
        close(h3, O.plain_norm(xn + 2.0 * a.double(), w1.double(), 1e-5)[[5, 0, 5]], 1e-4)
        close(xd, xn, 1e-5)                                   # a gathering call leaves the stream alone


ALONE = {
    "attention_gqa": U.attention_layer(heads=4, kv_heads=2, dim=16, vdim=24, chunk=16, ff=None),
    "attention_mha_partial_rotary": U.attention_layer(heads=3, kv_heads=3, dim=24, vdim=16, rot_dims=8, chunk=7, ff=None),
    "attention_one_kv_head_plain_causal": U.attention_layer(heads=4, kv_heads=1, dim=8, vdim=40, chunk=0, ff=None),
    "attention_chunk_of_one": U.attention_layer(heads=2, kv_heads=2, dim=16, vdim=16, chunk=1, ff=None),
    "attention_odd_head_size": U.attention_layer(heads=2, kv_heads=1, dim=12, vdim=10, rot_dims=6, chunk=20, ff=None),
    "attention_wide_values": U.attention_layer(heads=2, kv_heads=1, dim=32, vdim=200, chunk=50, ff=None),
    "hgrn2": U.hgrn2_layer(ff=None),
    "hgrn2_long_keys": U.hgrn2_layer(heads=1, dim=72, vdim=16, ff=None),
    "hgrn2_wide_values": U.hgrn2_layer(heads=3, dim=8, vdim=136, ff=None),
    "gla": U.gla_layer(ff=None),
    "gla_tau_one_rank_four": U.gla_layer(heads=3, dim=40, vdim=24, tau=1.0, ff=None, rank=4),
    "mlp_unaligned_channels": U.hgrn2_layer(heads=1, dim=8, vdim=8, ff=40),
    "gla_key_size_160": U.gla_layer(heads=2, dim=160, vdim=16, ff=None),
    "hgrn2_key_size_320": U.hgrn2_layer(heads=1, dim=320, vdim=72, ff=None),
    "attention_key_size_264": U.attention_layer(heads=2, kv_heads=1, dim=264, vdim=8, rot_dims=64, chunk=30, ff=None),
}


@pytest.mark.parametrize("name", sorted(ALONE))
def test_one_layer_models(name):
    cfg = U.make_config([ALONE[name]], vocab=80, width=48, residual_mult=0.7, softcap=15.0)
    w = U.make_weights(cfg, seed=3)
    t = toks(70, 80, 4)
    col, ocol = [], []
    ref = U.oracle_logits(cfg, w, t, ocol)
    eng = engine(cfg, w)
    got = eng.run_step([("x", t, range(len(t)))], collect=col)
    close(col[0], ocol[0], 2e-4)
    close(got, ref, 2e-4)


def test_all_mixers_together_residual_stream_and_bf16():
    cfg = U.make_config(FULL)
    w = U.make_weights(cfg, seed=5)
    t = toks(90, cfg["vocab"], 6)
    ocol = []
    ref = U.oracle_logits(cfg, w, t, ocol)
    col = []
    got = engine(cfg, w).run_step([("x", t, range(len(t)))], collect=col)
    for a, b in zip(col, ocol):
        close(a, b, 3e-4)
    close(got, ref, 3e-4)
    got16 = whole(engine(cfg, w, torch.bfloat16), t)
    d = got16.double().cpu() - ref
    assert float(d.pow(2).mean().sqrt()) < 0.05 * float(ref.pow(2).mean().sqrt()), "bf16 step is off by more than rounding"


def test_no_softcap_unit_multiplier_first_layer_attention():
    cfg = U.make_config([U.attention_layer(chunk=9), U.gla_layer(), U.attention_layer(kv_from=0, chunk=9)], residual_mult=1.0, softcap=None)
    w = U.make_weights(cfg, seed=7)
    t = toks(40, cfg["vocab"], 8)
    close(whole(engine(cfg, w), t), U.oracle_logits(cfg, w, t), 5e-4)


# ------------------------------------------------------------------------------------------------ schedules
def test_prefill_against_token_by_token_and_first_tokens():
    cfg = U.make_config(FULL)
    w = U.make_weights(cfg, seed=9)
    t = toks(75, cfg["vocab"], 10)
    ref = U.oracle_logits(cfg, w, t)
    eng = engine(cfg, w)
    close(whole(eng, t), ref, 3e-4)
    one = torch.cat([eng.run_step([("d", [tk], [0])]) for tk in t])       # decoding from the very first token on
    eng.release("d")
    close(one, ref, 3e-4)
    for n in (1, 2, 3):                                                    # the shortest sequences
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


def test_unequal_batches_reused_pages_and_slots():
    cfg = U.make_config(FULL)
    w = U.make_weights(cfg, seed=13)
    lens = {"a": 150, "b": 9, "c": 70, "d": 131, "e": 64, "f": 40}
    seqs = {k: toks(n, cfg["vocab"], 20 + i) for i, (k, n) in enumerate(lens.items())}
    ref = {k: U.oracle_logits(cfg, w, v) for k, v in seqs.items()}
    # pool: 7 pages of 64 and 3 slots -- less than the requests need together, so pages and slots come back and go out again
    eng = engine(cfg, w, max_tokens=7 * 64, max_seqs=3)
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
        close(torch.cat(got[k]), ref[k], 3e-4)
    with pytest.raises(MemoryError):
        eng.run_step([("big", toks(8 * 64, cfg["vocab"], 1), [])])


# ------------------------------------------------------------------------------------------------ edges, with one key that dominates
def _beacon_model(chunk, dim=16, rot=8, vdim=16, heads=2, kv_heads=1, width=32, vocab=40):
    """One attention layer in which token 1 (the beacon) writes a key that the query of token 2 (the asker) scores about 25 above every
    other key, through a channel outside the rotary span; the beacon's value is far from the others'.  Seeing or not seeing the beacon
    moves the asker's logits by a lot."""
    cfg = U.make_config([U.attention_layer(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, rot_dims=rot, chunk=chunk, ff=None, scale=1.0)],
                        vocab=vocab, width=width, residual_mult=1.0, softcap=None)
    w = U.make_weights(cfg, seed=17)
    for k in ("l0.mix.q", "l0.mix.k"):
        w[k] *= 0.05
    w["l0.norm1"].zero_()
    e = torch.randn(vocab, width, generator=torch.Generator().manual_seed(18)) * 0.05
    e[:, :2] = 0.0                                    # only the beacon and the asker live on the first two axes
    e[1], e[2] = 0.0, 0.0
    e[1, 0], e[2, 1] = 1.0, 1.0                       # after the norm: sqrt(width) on that axis
    w["embed"] = e.bfloat16().float()
    c = dim - 1                                       # a channel that is not rotated
    w["l0.mix.k"][c, 0] = 5.0 / width ** 0.5
    for h in range(heads):
        w["l0.mix.q"][h * dim + c, 1] = 5.0 / width ** 0.5
    w["l0.mix.v"][:, 0] = 3.0
    return cfg, {k: v.bfloat16().float() for k, v in w.items()}


@pytest.mark.parametrize("chunk,beacon,asker", [
    (48, 48, 95), (48, 47, 95),        # first position of the asker's block / last of the block before
    (48, 96, 96 + 47), (48, 95, 96),   # whole block apart / one apart across the edge
    (300, 63, 290), (300, 64, 290), (300, 3, 299),   # either side of a page border, and far back
    (0, 0, 250),                        # no blocks: the first token stays visible
    (64, 128, 191), (64, 127, 191),    # mask edge on a page edge
])
def test_dominant_key_at_edges_prompt_and_decoded(chunk, beacon, asker):
    cfg, w = _beacon_model(chunk)
    t = [3 + (i % 30) for i in range(asker + 1)]
    t[beacon], t[asker] = 1, 2
    ref = U.oracle_logits(cfg, w, t)
    t2 = list(t); t2[beacon] = 5
    visible = (chunk == 0 or beacon // chunk == asker // chunk)
    moved = float((U.oracle_logits(cfg, w, t2)[asker] - ref[asker]).abs().max())
    assert (moved > 0.05) == visible, f"the beacon moves the asker's logits by {moved}"
    eng = engine(cfg, w)
    close(eng.run_step([("w", t, [asker])]), ref[asker:asker + 1], 3e-4)              # in a prompt
    eng.release("w")
    eng.run_step([("d", t[:asker], [])])
    close(eng.run_step([("d", [t[asker]], [0])]), ref[asker:asker + 1], 3e-4)         # decoded alone
    eng.release("d")
    cut = max(1, beacon)                                                                # a portion that starts at the beacon
    eng.run_step([("p", t[:cut], [])])
    close(eng.run_step([("p", t[cut:], [asker - cut])]), ref[asker:asker + 1], 3e-4)


def test_recurrent_state_carries_a_far_token():
    """A token at position 2 must still be felt hundreds of tokens later through the recurrent state (slow decay)."""
    cfg = U.make_config([U.gla_layer(tau=64.0, ff=None), U.hgrn2_layer(ff=None)], residual_mult=1.0)
    w = U.make_weights(cfg, seed=19)
    w["l0.mix.a2.b"] += 4.0
    w["l1.mix.lower"] = (0.99 + 0.01 * w["l1.mix.lower"]).bfloat16().float()
    t = toks(400, cfg["vocab"], 21)
    ref = U.oracle_logits(cfg, w, t)
    t2 = list(t); t2[2] = (t[2] + 1) % cfg["vocab"]
    assert float((U.oracle_logits(cfg, w, t2)[-1] - ref[-1]).abs().max()) > 1e-2
    eng = engine(cfg, w)
    close(whole(eng, t)[-1:], ref[-1:], 3e-4)
    eng.run_step([("d", t[:350], [])])
    out = torch.cat([eng.run_step([("d", [tk], [0])]) for tk in t[350:]])
    close(out, ref[350:], 3e-4)


def test_long_decoding():
    cfg = U.make_config([U.attention_layer(chunk=100), U.hgrn2_layer(), U.gla_layer(), U.attention_layer(kv_from=0, chunk=100)])
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
    cfg = U.make_config([U.gla_layer(), U.attention_layer(chunk=24), U.hgrn2_layer()], vocab=64, width=48)
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
    sampled = eng.generate(prompts[:2], 6, top_k=5, top_p=0.9, temperature=0.8, seed=3)
    assert sampled == eng.generate(prompts[:2], 6, top_k=5, top_p=0.9, temperature=0.8, seed=3)
    assert all(len(o) == 6 and all(0 <= x < 64 for x in o) for o in sampled)


def test_command_line_generate_and_trace(tmp_path):
    from safetensors.torch import save_file
    cfg = U.make_config([U.hgrn2_layer(), U.attention_layer(chunk=16)], vocab=64, width=48)
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
    """Decode steps through the captured graph, with eager prompt portions and eager decode steps between the replays."""
    cfg = U.make_config([U.gla_layer(), U.attention_layer(chunk=40), U.hgrn2_layer(), U.attention_layer(kv_from=1, chunk=40)])
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


@pytest.mark.parametrize("dim,vdim,heads,kv_heads,chunk,layout", [(32, 16, 2, 1, 40, "interleaved"), (64, 48, 4, 2, 0, "interleaved"),
                                                                   (128, 128, 4, 1, 100, "interleaved"), (96, 64, 3, 3, 33, "halves"),
                                                                   (256, 256, 2, 2, 64, "interleaved")])
def test_matrix_core_attention_for_portions_equals_row_kernel(dim, vdim, heads, kv_heads, chunk, layout):
    """Both attention kernels over the same bf16 pages: ragged portions of three sequences that start inside pages and mask blocks, with
    tiles of every fill (1 .. 16 rows), scattered pages, a sink and rotated values."""
    from rtp_llm_amd import hybrid_ops as hops
    from rtp_llm_amd.mixers import rotary_steps
    g = torch.Generator(device=DEV).manual_seed(dim + vdim)
    page, num_pages, width = 64, 24, 8
    starts, counts = [0, 70, 250], [45, 130, 17]                       # first position and row count of each sequence's portion
    tables = torch.randperm(num_pages, generator=torch.Generator().manual_seed(1), dtype=torch.int32)[:3 * width].reshape(3, width)
    pos, seq, t0, tn, row = [], [], [], [], 0
    for s_, (a, n) in enumerate(zip(starts, counts)):
        pos += list(range(a, a + n)); seq += [s_] * n
        t0 += list(range(row, row + n, 16)); tn += [min(16, n - r) for r in range(0, n, 16)]
        row += n
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    kc = torch.randn(num_pages, kv_heads, page, dim, device=DEV, generator=g).bfloat16()
    vc = torch.randn(num_pages, kv_heads, page, vdim, device=DEV, generator=g).bfloat16()
    q = torch.randn(row, heads * dim, device=DEV, generator=g)
    geom = hops.attn_geometry(heads, kv_heads, dim, vdim, dim, 0, hops.LAYOUTS[layout], page, width, num_pages)
    vf = rotary_steps(vdim // 2, vdim, 1e4, DEV)
    assert hops.attn_tiles_supported(torch.bfloat16, dim, vdim, True, hops.LAYOUTS[layout])
    for sink, vfreq in ((torch.zeros(heads, device=DEV), vf), (None, None)):
        a = hops.attn_rows(q, dim ** -0.5, geom, chunk, sink, vfreq, i32(pos), i32(seq), tables.to(DEV), kc, vc, heads, vdim)
        b = hops.attn_tiles(q, dim ** -0.5, geom, chunk, sink, vfreq, i32(pos), i32(seq), tables.to(DEV), i32(t0), i32(tn), kc, vc, heads, vdim)
        err = (a.float() - b.float()).abs()
        assert float(err.max()) <= 2e-2 and float(err.mean()) < 1e-3, f"kernels differ: max {float(err.max())} mean {float(err.mean())}"


def test_bf16_dominant_key_through_matrix_core_attention():
    """The mask edges again in bfloat16, where prompt portions run on the matrix cores: the asker's logits with the beacon just inside and just
    outside its block must each match the plain implementation (they differ from one another by far more than bf16 rounding)."""
    for beacon, asker in ((64, 127), (63, 127), (127, 127 + 64), (0, 60)):
        cfg, w = _beacon_model(64, dim=32, rot=16, vdim=32)
        t = [3 + (i % 30) for i in range(asker + 1)]
        t[beacon], t[asker] = 1, 2
        ref = U.oracle_logits(cfg, w, t)[asker]
        eng = engine(cfg, w, torch.bfloat16)
        got = eng.run_step([("w", t, [asker])])[0].double().cpu()
        assert float((got - ref).abs().max()) < 0.05 * float(ref.abs().max()) + 0.05
