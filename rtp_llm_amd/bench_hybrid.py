"""`bench.py --hybrid`: prefill and decode throughput of the hybrid decoder family at layer sizes of real models (random weights), beside
the Qwen2 / Llama engine at equal width, depth, head geometry, FFN width and vocabulary (bf16, 16-bit weights), and the kernels of both
against their rooflines (HBM 8 TB/s, dense bf16 MFMA 2.5 PFLOP/s, fp32 vector FMA 157 TFLOP/s).

Output: one JSON line {"hybrid_bench": {size: {"hybrid": {...}, "qwen2": {...}, "kernels": [...]}}}."""
import json
import math
import sys
import time

import torch

HBM, MFMA_BF16, VALU_F32 = 8.0e12, 2.5e15, 157.0e12

SIZES = {
    "w1024": dict(width=1024, layers=8, heads=8, kv=2, hd=128, ff=2816, vocab=32000),
    "w2048": dict(width=2048, layers=16, heads=16, kv=4, hd=128, ff=5632, vocab=32000),
    "w4096": dict(width=4096, layers=8, heads=32, kv=8, hd=128, ff=11008, vocab=32000),
}
PATTERN = ["gla", "attention", "hgrn2", "gla", "gla", "shared", "hgrn2", "gla"]


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def hybrid_config(s, chunk=1024):
    layers, owner = [], None
    for i in range(s["layers"]):
        kind = PATTERN[i % len(PATTERN)]
        mlp = {"kind": "dense", "ff": s["ff"]}
        if kind in ("attention", "shared"):
            mx = {"heads": s["heads"], "kv_heads": s["kv"], "dim": s["hd"], "vdim": s["hd"], "scale": s["hd"] ** -0.5, "mask": {"size": chunk},
                  "rot": {"base": 1e6, "dims": s["hd"]}}
            if kind == "shared":
                mx["kv_from"] = owner
            else:
                owner = i
            layers.append({"type": "attention", "mixer": mx, "mlp": mlp})
        elif kind == "gla":
            layers.append({"type": "gla", "mixer": {"heads": s["heads"], "dim": s["hd"] // 2, "vdim": s["hd"], "tau": 16.0}, "mlp": mlp})
        else:
            layers.append({"type": "hgrn2", "mixer": {"heads": s["heads"], "dim": s["hd"] // 2, "vdim": s["hd"]}, "mlp": mlp})
    return {"architecture": "Nufalorn", "layers": layers, "vocab": s["vocab"], "width": s["width"], "norm": {"eps": 1e-5},
            "residual_mult": 0.3, "logit_softcap": 30.0}


def hybrid_weights(cfg, dev, seed=0):
    g = torch.Generator(device=dev).manual_seed(seed)
    W = cfg["width"]
    lin = lambda o, i: (torch.randn(o, i, device=dev, generator=g) * i ** -0.5).bfloat16()
    vec = lambda n, k=0.1, off=0.0: (torch.randn(n, device=dev, generator=g) * k + off).bfloat16()
    w = {"embed": (torch.randn(cfg["vocab"], W, device=dev, generator=g)).bfloat16(), "head": lin(cfg["vocab"], W), "final.norm": vec(W)}
    for i, L in enumerate(cfg["layers"]):
        p, mx = f"l{i}.", L["mixer"]
        H, d, dv = mx["heads"], mx["dim"], mx["vdim"]
        w[p + "norm1"], w[p + "norm2"] = vec(W), vec(W)
        if L["type"] == "attention":
            w[p + "mix.q"], w[p + "mix.o"] = lin(H * d, W), lin(W, H * dv)
            if "kv_from" not in mx:
                w[p + "mix.k"], w[p + "mix.v"] = lin(mx["kv_heads"] * d, W), lin(mx["kv_heads"] * dv, W)
        elif L["type"] == "hgrn2":
            for n, o in (("q", H * d), ("f", H * d), ("v", H * dv)):
                w[p + "mix." + n] = lin(o, W)
            w[p + "mix.f.b"], w[p + "mix.lower"], w[p + "mix.norm"] = vec(H * d, 0.5), torch.sigmoid(vec(H * d, 1.0).float()).bfloat16(), vec(dv, 0.1, 1.0)
            w[p + "mix.o"] = lin(W, H * dv)
        else:
            for n, o in (("q", H * d), ("k", H * d), ("v", H * dv), ("g", H * dv), ("a1", 16)):
                w[p + "mix." + n] = lin(o, W)
            w[p + "mix.a2"], w[p + "mix.a2.b"], w[p + "mix.norm"], w[p + "mix.o"] = lin(H * d, 16), vec(H * d, 1.0, 2.0), vec(dv, 0.1, 1.0), lin(W, H * dv)
        ff = L["mlp"]["ff"]
        w[p + "mlp.gate"], w[p + "mlp.up"], w[p + "mlp.down"] = lin(ff, W), lin(ff, W), lin(W, ff)
    return w


def timed(fn, reps=5, warm=2, graph=False):
    """Seconds per call.  graph: the calls are captured into one HIP graph and the replay is timed, so the figure is the kernels' own
    time and not the host's launch path (what a graph-replayed step pays)."""
    for _ in range(warm):
        fn()
    if graph:
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for _ in range(reps):
                fn()
        inner, fn, reps = reps, g.replay, 3
        g.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / (reps * inner) * 1e-3
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / reps * 1e-3


def bench_hybrid_engine(s, dev, prompt, batch, steps):
    from .hybrid import HybridConfig, HybridModel
    from .scheduler import ServingEngine
    cfg = hybrid_config(s)
    model = HybridModel(HybridConfig.from_json(cfg), hybrid_weights(cfg, dev), torch.bfloat16, dev)
    eng = ServingEngine(model, max_tokens=batch * (prompt + 8 * (steps + 3) + 128), max_seqs=batch, max_step_tokens=1 << 20)
    g = torch.Generator().manual_seed(1)
    toks = lambda n: torch.randint(0, s["vocab"], (n,), generator=g).tolist()
    out = {}
    # prefill: one sequence of `prompt` tokens per step (released afterwards), then `batch` sequences in one step
    def one():
        eng.run_step([("p", toks(prompt), [prompt - 1])]); eng.release("p")
    t = timed(one, reps=3, warm=1)
    out["prefill_1x%d_tok_s" % prompt] = round(prompt / t)
    ids = [f"s{i}" for i in range(batch)]
    torch.cuda.synchronize(); t0 = time.time()
    eng.run_step([(i, toks(prompt), [prompt - 1]) for i in ids])
    torch.cuda.synchronize()
    out["prefill_%dx%d_tok_s" % (batch, prompt)] = round(batch * prompt / (time.time() - t0))
    # decode: `batch` live sequences, one token each per step
    for b in sorted({1, min(8, batch), batch}):
        step = lambda: eng.run_step([(i, [7], [0]) for i in ids[:b]])
        for graph in (False, True):
            eng.use_graphs = graph
            t = timed(step, reps=steps, warm=3)
            out["decode_b%d_%s_tok_s" % (b, "graph" if graph else "eager")] = round(b / t)
            out["decode_b%d_%s_ms" % (b, "graph" if graph else "eager")] = round(t * 1e3, 3)
    for i in ids:
        eng.release(i)
    return out, model, eng


def bench_qwen2_engine(s, dev, prompt, batch, steps):
    from . import model as M
    cfg = M.ModelConfig("qwen2-like", s["layers"], s["width"], s["heads"], s["kv"], s["hd"], s["ff"], s["vocab"], max_pos=prompt + 8 * steps + 256)
    w = M.synth_model(cfg, "fp16", dev, seed=0)
    page = 64
    per = (prompt + 8 * steps + 128 + page - 1) // page
    eng = M.DecoderEngine(cfg, w, kv_int8=False, page=page, num_blocks=per * batch, max_batch=max(batch, 1), max_seq_len=per * page, device=dev,
                          dtype=torch.bfloat16)
    g = torch.Generator().manual_seed(1)
    toks = lambda n: torch.randint(0, s["vocab"], (n,), generator=g).tolist()
    bt = torch.arange(per * batch, dtype=torch.int32).reshape(batch, per)
    out = {}
    t = timed(lambda: eng.prefill([toks(prompt)], bt[:1], chunk=512), reps=3, warm=1)
    out["prefill_1x%d_tok_s" % prompt] = round(prompt / t)
    torch.cuda.synchronize(); t0 = time.time()
    eng.prefill([toks(prompt) for _ in range(batch)], bt, chunk=512)
    torch.cuda.synchronize()
    out["prefill_%dx%d_tok_s" % (batch, prompt)] = round(batch * prompt / (time.time() - t0))
    for b in sorted({1, min(8, batch), batch}):
        eng.set_inputs([7] * b, [prompt] * b, bt[:b])
        eng.capture(b)
        t = timed(lambda: eng.replay(b, 1), reps=steps, warm=3)
        out["decode_b%d_graph_tok_s" % b] = round(b / t)
        out["decode_b%d_graph_ms" % b] = round(t * 1e3, 3)
    return out, eng


def kernel_table(s, dev, prompt):
    """Time the kernels of both families at this size; roofline time = max(bytes / HBM, flops / peak of the unit that does them)."""
    from . import hybrid_ops as hops, ops, quant
    rows = []
    timed_k = lambda fn: timed(fn, reps=10, warm=2, graph=True)
    g = torch.Generator(device=dev).manual_seed(3)
    bf = lambda *sh: torch.randn(*sh, device=dev, generator=g).bfloat16()
    W, H, G, hd, ff = s["width"], s["heads"], s["kv"], s["hd"], s["ff"]

    def add(family, name, shape, t, nbytes, flops, peak):
        roof = max(nbytes / HBM, flops / peak)
        rows.append({"family": family, "kernel": name, "shape": shape, "us": round(t * 1e6, 1), "roofline_us": round(roof * 1e6, 2),
                     "x_roofline": round(t / roof, 1)})

    # linears: the FFN up projection (N = 2 ff gated) and the attention output projection
    for M_ in (prompt, 8, 1):
        x = bf(M_, W)
        wgu = hops.group_gate_up(bf(ff, W), bf(ff, W))
        t = timed_k(lambda: hops.dense_linear(x, wgu, gated=True, act=hops.ACT_RELU))
        add("hybrid", "dense_linear gated", f"M={M_} N={2 * ff} K={W}", t, 2 * ff * W * 2 + M_ * (W + ff) * 2, 2.0 * M_ * 2 * ff * W, MFMA_BF16)
        pw = quant.pack_fp16(quant.interleave_gate_up(bf(W, 2 * ff), -1))
        t = timed_k(lambda: ops.linear(x, pw, None, epilogue=1))
        add("qwen2", "linear W16 silu_mul", f"M={M_} N={2 * ff} K={W}", t, 2 * ff * W * 2 + M_ * (W + ff) * 2, 2.0 * M_ * 2 * ff * W, MFMA_BF16)
        xo, wo = bf(M_, H * hd), bf(W, H * hd)
        t = timed_k(lambda: hops.dense_linear(xo, wo, out_dtype=torch.float32))
        add("hybrid", "dense_linear", f"M={M_} N={W} K={H * hd}", t, W * H * hd * 2 + M_ * (H * hd * 2 + W * 4), 2.0 * M_ * W * H * hd, MFMA_BF16)
        pwo = quant.pack_fp16(bf(H * hd, W))
        t = timed_k(lambda: ops.linear(xo, pwo))
        add("qwen2", "linear W16", f"M={M_} N={W} K={H * hd}", t, W * H * hd * 2 + M_ * (H * hd + W) * 2, 2.0 * M_ * W * H * hd, MFMA_BF16)
    # norms
    for M_ in (prompt, 8):
        x, a, b = [torch.randn(M_, W, device=dev, generator=g) for _ in range(3)]
        w1, w2 = bf(W), bf(W)
        t = timed_k(lambda: hops.residual_norm(x, a, b, 0.3, w1, w2, 1e-5, weight_offset=1.0))
        add("hybrid", "residual + 2 norms (fp32 stream)", f"M={M_} W={W}", t, M_ * W * (4 * 4 + 2 * 2), 0, VALU_F32)
        xh, rh, wh = bf(M_, W).to(torch.bfloat16), bf(M_, W), bf(W)
        t = timed_k(lambda: ops.add_rmsnorm(xh, rh, wh, 1e-6))
        add("qwen2", "add + rmsnorm (16-bit stream)", f"M={M_} W={W}", t, M_ * W * 2 * 4, 0, VALU_F32)
    # attention: prefill rows over a chunk-local mask vs plain causal rows; decode at a context of `prompt`
    page, chunk = 64, 1024
    nblk = (prompt + page - 1) // page + 1
    geom = hops.attn_geometry(H, G, hd, hd, hd, 0, 0, page, nblk, nblk)
    kc, vc = bf(nblk, G, page, hd), bf(nblk, G, page, hd)
    bt = torch.arange(nblk, dtype=torch.int32, device=dev).reshape(1, nblk)
    vf = torch.ones(hd // 2, device=dev) * 1e-3
    for T_, name in ((prompt, "prefill"), (1, "decode")):
        pos = (torch.arange(T_, dtype=torch.int32, device=dev) if T_ > 1 else torch.tensor([prompt - 1], dtype=torch.int32, device=dev))
        seq = torch.zeros(T_, dtype=torch.int32, device=dev)
        q = torch.randn(T_, H * hd, device=dev, generator=g)
        t = timed_k(lambda: hops.attn_rows(q, hd ** -0.5, geom, chunk, True, vf, pos, seq, bt, kc, vc, H, hd))
        keys = float(sum(min(int(p) % chunk + 1, chunk) for p in pos.tolist()))
        add("hybrid", f"attn_rows {name} (chunk {chunk})", f"T={T_} H={H} G={G} hd={hd} ctx={prompt}", t,
            min(prompt, chunk if T_ == 1 else prompt) * G * hd * 2 * 2 + T_ * H * hd * 6, 4.0 * keys * H * hd, MFMA_BF16)
        if T_ > 1:
            t0 = torch.arange(0, T_, 16, dtype=torch.int32, device=dev)
            tn = torch.full_like(t0, 16)
            t = timed_k(lambda: hops.attn_tiles(q, hd ** -0.5, geom, chunk, True, vf, pos, seq, bt, t0, tn, kc, vc, H, hd))
            add("hybrid", f"attn_tiles {name} (chunk {chunk}, MFMA)", f"T={T_} H={H} G={G} hd={hd} ctx={prompt}", t,
                prompt * G * hd * 2 * 2 + T_ * H * hd * 6, 4.0 * keys * H * hd, MFMA_BF16)
        kvb = torch.randn(nblk, 2, G, page, hd, device=dev, generator=g).bfloat16()
        qh = bf(T_, H, hd)
        if T_ > 1:
            q_len = 512
            posr = torch.arange(q_len, dtype=torch.int32, device=dev) + (prompt - q_len)
            qh = bf(q_len, H, hd)
            t = timed_k(lambda: ops.paged_attention_rows(qh, kvb, None, bt, posr, G, page, q_len, nblk * page))
            keysq = float(sum(int(p) + 1 for p in posr.tolist()))
            add("qwen2", "paged_attn_rows prefill (last 512 rows, causal)", f"T={q_len} H={H} G={G} hd={hd} ctx={prompt}", t,
                prompt * G * hd * 2 * 2 + q_len * H * hd * 4, 4.0 * keysq * H * hd, MFMA_BF16)
        else:
            sl = torch.tensor([prompt], dtype=torch.int32, device=dev)
            t = timed_k(lambda: ops.paged_decode_attention(qh, kvb, None, bt, sl, G, page, nblk * page))
            add("qwen2", "paged_decode_attn", f"B=1 H={H} G={G} hd={hd} ctx={prompt}", t, prompt * G * hd * 2 * 2, 4.0 * prompt * H * hd, MFMA_BF16)
    # recurrence: no counterpart in the Qwen2 family
    d = hd // 2
    for T_, name in ((prompt, "prefill"), (8, "decode b=8")):
        nseq = 1 if T_ > 8 else 8
        proj = torch.randn(T_, 2 * H * d + 2 * H * hd, device=dev, generator=g)
        z = torch.randn(T_, H * d, device=dev, generator=g)
        rs = torch.arange(0, T_ + 1, T_ // nseq, dtype=torch.int32, device=dev)
        slot = torch.arange(nseq, dtype=torch.int32, device=dev)
        fp = torch.ones(nseq, dtype=torch.int32, device=dev)
        state = torch.zeros(nseq, H, d, hd, device=dev)
        t = timed_k(lambda: hops.scan(hops.SCAN_GLA, proj, 0, H * d, 2 * H * d, z, None, None, 16.0, d ** -0.5, H, d, hd, rs, slot, fp, state, torch.bfloat16))
        add("hybrid", f"scan GLA {name}", f"T={T_} H={H} dim={d} vdim={hd}", t, T_ * (3 * H * d + 2 * H * hd) * 4 + 2 * nseq * H * d * hd * 4,
            4.0 * T_ * H * d * hd, VALU_F32)
    return rows


def run(args):
    from . import _C
    _C.lib(); _C.hybrid_lib()
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    sizes = [x for x in (args.hybrid_sizes.split(",") if args.hybrid_sizes else SIZES)]
    prompt, batch, steps = args.hybrid_prompt, args.hybrid_batch, args.steps
    out = {}
    for name in sizes:
        s = SIZES[name]
        log(f"[hybrid bench] {name}: {s}")
        rec = {"config": s, "prompt": prompt, "batch": batch}
        rec["hybrid"], model, eng = bench_hybrid_engine(s, dev, prompt, batch, steps)
        del model, eng
        torch.cuda.empty_cache()
        log(f"[hybrid bench] {name} hybrid: {rec['hybrid']}")
        rec["qwen2"], q = bench_qwen2_engine(s, dev, prompt, batch, steps)
        del q
        torch.cuda.empty_cache()
        log(f"[hybrid bench] {name} qwen2 : {rec['qwen2']}")
        rec["kernels"] = kernel_table(s, dev, prompt)
        for r in rec["kernels"]:
            log(f"    {r['family']:7s} {r['kernel']:48s} {r['shape']:44s} {r['us']:10.1f} us  roofline {r['roofline_us']:9.2f} us  x{r['x_roofline']}")
        out[name] = rec
    print(json.dumps({"hybrid_bench": out, "dtype": "bf16", "data": "synthetic (random weights and tokens)"}))
    return 0
