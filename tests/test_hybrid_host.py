"""Host-side pieces of the hybrid family and its serving engine, on the CPU: pools, cache manager, step builder, configuration and
registry, and the plain implementation's own consistency."""
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import hybrid_oracle as O  # noqa: E402
import hybrid_util as U  # noqa: E402
from rtp_llm_amd.kvcache import CacheManager, PagePool  # noqa: E402


def test_hybrid_library_builds_and_exports_every_declared_symbol():
    import ctypes
    import re
    from rtp_llm_amd import _C
    from rtp_llm_amd.build import build_hybrid
    lib = ctypes.CDLL(build_hybrid(verbose=False))              # hipcc cross-compiles gfx950 without a GPU
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    src = re.sub(r"/\*.*?\*/", "", open(os.path.join(root, "include", "mi355_hybrid.h")).read(), flags=re.S)
    declared = set(re.findall(r"\b(mi355_[a-z0-9_]+)\s*\(", src))
    assert declared and declared | {"mi355_abi_version", "mi355_last_error"} == set(_C.HYBRID_SIGNATURES)
    for name in _C.HYBRID_SIGNATURES:
        assert hasattr(lib, name), f"{name} is not exported"
    l = _C.hybrid_lib()
    assert l.mi355_abi_version() == _C.ABI_VERSION
    assert l.mi355_dense_linear(None, 0, 1, None, 8, 8, None, None, 8, 0, 0, 0, 0.0, _C.ACT_BF16, None) == _C.ERR_ARG   # argument errors need no GPU
    assert b"dense_linear" in l.mi355_last_error()


def test_page_pool_reuses_what_came_back():
    p = PagePool(4)
    assert p.take(3) == [0, 1, 2]
    p.give([1])
    assert p.take(2) == [1, 3] and p.free == 0
    with pytest.raises(MemoryError):
        p.take(1)
    p.give([0, 2])
    with pytest.raises(ValueError):
        p.give([2])
    with pytest.raises(ValueError):
        p.give([9])


def test_cache_manager_growth_promises_and_release():
    cm = CacheManager(num_pages=6, page=8, num_slots=2)
    assert cm.can_admit(48) and not cm.can_admit(49)
    a = cm.admit("a", reserve_tokens=20)                 # 3 pages promised
    assert cm.can_admit(24) and not cm.can_admit(25)
    cm.grow("a", 9); cm.advance("a", 9)
    assert len(a.pages) == 2 and a.length == 9 and cm.pages.free == 4
    assert cm.can_admit(24) and not cm.can_admit(25)     # one page of the promise is still out
    cm.grow("a", 7); cm.advance("a", 7)                  # 16 tokens: still 2 pages
    assert len(a.pages) == 2
    b = cm.admit("b")
    assert b.slot != a.slot and not cm.can_admit(1)      # no slot left
    with pytest.raises(MemoryError):
        cm.admit("c")
    with pytest.raises(KeyError):
        cm.admit("a")
    cm.grow("b", 32)
    assert cm.pages.free == 0
    with pytest.raises(MemoryError):
        cm.grow("a", 1)
    cm.release("b")
    assert cm.pages.free == 4 and cm.slots.free == 1
    cm.grow("a", 1)
    assert len(a.pages) == 3
    cm.release("a")
    assert cm.pages.free == 6 and cm.slots.free == 2 and not cm.live


class _FakeModel:
    """Records the batches it is given; logits row = (token, position, slot)."""
    page, device = 4, torch.device("cpu")

    def __init__(self):
        self.batches = []

    def alloc_cache(self, num_pages, num_slots):
        return []

    def forward(self, batch, caches, collect=None):
        self.batches.append(batch)
        w = batch.want.long()
        seq = batch.seq.long()[w]
        return torch.stack([batch.tokens[w].float(), batch.pos[w].float(), batch.slot.long()[seq].float()], 1)


def test_step_builder_positions_tables_and_slots():
    from rtp_llm_amd.scheduler import ServingEngine
    m = _FakeModel()
    eng = ServingEngine(m, max_tokens=24, max_seqs=2)
    out = eng.run_step([("a", [7, 8, 9, 10, 11], [4]), ("b", [1], [0])])
    assert out.tolist() == [[11.0, 4.0, 0.0], [1.0, 0.0, 1.0]]
    b = m.batches[-1]
    assert b.pos.tolist() == [0, 1, 2, 3, 4, 0] and b.seq.tolist() == [0, 0, 0, 0, 0, 1] and b.row_start.tolist() == [0, 5, 6]
    assert b.first_pos.tolist() == [0, 0] and b.block_table[0, :2].tolist() == [0, 1] and b.block_table[1, 0].item() == 2
    assert eng.run_step([("b", [2, 3], [])]) is None                 # a sequence may sit out a step; nothing wanted
    out = eng.run_step([("b", [4], [0]), ("a", [12], [0])])
    assert out.tolist() == [[4.0, 3.0, 1.0], [12.0, 5.0, 0.0]]
    assert m.batches[-1].first_pos.tolist() == [3, 5]
    eng.release("a")
    out = eng.run_step([("c", [5, 5, 5, 5, 5], [0])])                # takes a's slot and pages
    assert out.tolist() == [[5.0, 0.0, 0.0]] and m.batches[-1].block_table[0, :2].tolist() == [1, 0]
    with pytest.raises(ValueError):
        eng.run_step([("c", [1], [0]), ("c", [2], [0])])
    with pytest.raises(MemoryError):
        eng.run_step([("d", [1], [0])])                              # both slots are taken
    live = dict(eng.cache.live)
    with pytest.raises(MemoryError):
        eng.run_step([("b", [1] * 40, [])])                          # more pages than the pool has
    assert dict(eng.cache.live) == live


def test_config_reading_and_registry():
    from rtp_llm_amd import registry
    from rtp_llm_amd.hybrid import HybridConfig
    cfg = U.make_config([U.attention_layer(rot_dims=8, chunk=0), U.gla_layer(), U.attention_layer(rot_dims=8, chunk=5, kv_from=0), U.hgrn2_layer(ff=None)],
                        softcap=None)
    hc = HybridConfig.from_json(cfg)
    a, g, a2, h = [L.mixer for L in hc.layers]
    assert a.chunk == 0 and a.rot.dims == 8 and a.sink and a.value_norm and a.value_rot and a.kv_from is None
    assert a2.kv_from == 0 and a2.chunk == 5 and g.tau == 8.0 and h.kind == "hgrn2" and hc.layers[3].ff is None
    assert hc.logit_softcap == 0.0 and hc.norm_offset == 1.0
    assert registry.architecture_of(cfg) == "Nufalorn" and "nufalorn" in registry.families()
    assert registry.architecture_of({"architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2"}) == "Qwen2ForCausalLM"
    bad = U.make_config([U.gla_layer(), U.attention_layer(kv_from=0)])
    with pytest.raises(ValueError):
        HybridConfig.from_json(bad)
    bad = U.make_config([U.attention_layer(), U.attention_layer(kv_from=0, dim=32)])
    with pytest.raises(ValueError):
        HybridConfig.from_json(bad)
    bad = U.make_config([{"type": "conv", "mixer": {}, "mlp": None}])
    with pytest.raises(NotImplementedError):
        HybridConfig.from_json(bad)


def test_plain_implementation_is_consistent_with_itself():
    g = torch.Generator().manual_seed(0)
    T, d, dv = 9, 5, 4
    q, k, a = [torch.rand(T, d, generator=g, dtype=torch.float64) for _ in range(3)]
    v = torch.randn(T, dv, generator=g, dtype=torch.float64)
    o = O.gated_scan(q, k, v, a)
    # closed form: o_t = sum_{j<=t} (q_t * prod_{j<i<=t} a_i * k_j) . v_j
    for t in range(T):
        ref = torch.zeros(dv, dtype=torch.float64)
        for j in range(t + 1):
            ref += ((q[t] * a[j + 1:t + 1].prod(0) * k[j]).sum()) * v[j]
        assert torch.allclose(o[t], ref, atol=1e-12)
    x = torch.randn(6, 3, 8, generator=g, dtype=torch.float64)
    pos = torch.arange(6)
    for rot in (O.rotate_interleaved, O.rotate_halves):
        y = rot(x, pos, 8, 100.0)
        assert torch.allclose(rot(y, pos, 8, 100.0, sign=-1.0), x, atol=1e-12) and torch.allclose(y[0], x[0])
        assert torch.allclose(y.norm(dim=-1), x.norm(dim=-1))
    # the logits of a position do not depend on what follows it
    cfg = U.make_config([U.gla_layer(), U.attention_layer(chunk=4), U.hgrn2_layer()])
    w = U.make_weights(cfg)
    t = list(range(20))
    full = U.oracle_logits(cfg, w, t)
    assert torch.allclose(U.oracle_logits(cfg, w, t[:11]), full[:11], atol=1e-10)
