"""Token mixers of the hybrid decoder family, each a mechanism with its constants as parameters:

  * ``PagedChunkAttention`` -- grouped-query attention over the paged cache with a partial rotary embedding of either pair layout, a
    mask that is causal inside blocks of `chunk` positions (0: plain causal), an optional softmax sink (one added to the denominator),
    optional unit-normed values and optional value rotation (values are turned by their own position when cached and the head output
    is turned back by the query's position, so a value enters the sum turned by the distance).  A layer may read the cache that an
    earlier layer with the same geometry wrote (`kv_from`) and then has no key / value projections.
  * ``GatedLinearRecurrence`` -- S_t = diag(a_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t per head with the state in an fp32 slot, in the
    HGRN2 parametrisation (a = f, k = 1 - f with a lower-bounded forget gate f, q = silu) or the gated-linear-attention one
    (a = sigmoid(low-rank z)^(1/tau), q scaled by dim^-1/2, output gate silu(g)); per-head RMS norm of o, then the output projection.

Both take the normed activations of a ragged batch (``StepBatch``) and return the fp32 branch output [T, width]."""
import math
from dataclasses import dataclass
from typing import Dict, Optional

import torch

from . import hybrid_ops as hops


@dataclass
class RotarySpec:
    dims: int
    base: float
    layout: str = "interleaved"          # "interleaved": pairs (2i, 2i+1); "halves": (i, i + dims / 2)


@dataclass
class AttentionSpec:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: Optional[RotarySpec] = None
    chunk: int = 0                       # 0: every earlier position is visible
    sink: bool = False
    value_norm: bool = False
    value_rot: bool = False
    value_layout: str = "interleaved"
    kv_from: Optional[int] = None


@dataclass
class RecurrenceSpec:
    kind: str                            # "hgrn2" | "gla"
    heads: int
    dim: int
    vdim: int
    tau: float = 1.0


@dataclass
class StepBatch:
    """One ragged step on the device.  Row r is a token at position pos[r] of sequence seq[r]; sequence s owns rows
    row_start[s] .. row_start[s + 1] - 1 (in position order), the block-table row s and state slot slot[s]; first_pos[s] is the
    position of its first row in this step (0: the sequence starts here and recurrent states start from zero)."""
    tokens: torch.Tensor
    pos: torch.Tensor
    seq: torch.Tensor
    row_start: torch.Tensor
    slot: torch.Tensor
    first_pos: torch.Tensor
    block_table: torch.Tensor
    want: torch.Tensor                   # rows whose logits are computed
    tile_row0: Optional[torch.Tensor] = None   # tiles of at most 16 consecutive rows of one sequence covering every row: first row ...
    tile_n: Optional[torch.Tensor] = None      # ... and row count (the matrix-core attention for prompt portions works on them)
    host: Optional[torch.Tensor] = None        # the pinned buffer all index fields were uploaded from (one copy per step)


def rotary_steps(n_pairs: int, span: int, base: float, device) -> torch.Tensor:
    """fp32 angular step of pair i: base^(-2 i / span), evaluated in float64 and rounded once."""
    i = torch.arange(n_pairs, dtype=torch.float64)
    return torch.pow(torch.tensor(float(base), dtype=torch.float64), -2.0 * i / span).to(torch.float32).to(device)


class PagedChunkAttention:
    def __init__(self, spec: AttentionSpec, weights: Dict[str, torch.Tensor], eps: float, page: int, device):
        s = self.spec = spec
        self.eps, self.page = eps, page
        if s.heads % s.kv_heads:
            raise ValueError(f"attention: {s.heads} query heads over {s.kv_heads} key/value heads")
        self.owns_cache = s.kv_from is None
        parts = [weights["q"]] + ([weights["k"], weights["v"]] if self.owns_cache else [])
        self.w_in = torch.cat(parts, 0).contiguous()
        self.w_o = weights["o"].contiguous()
        self.koff, self.voff = s.heads * s.dim, (s.heads + s.kv_heads) * s.dim
        rot = s.rot
        self.kfreq = rotary_steps(rot.dims // 2, rot.dims, rot.base, device) if rot and rot.dims else None
        self.vfreq = rotary_steps(s.vdim // 2, s.vdim, rot.base, device) if s.value_rot and rot else None
        self._geom = None
        self.use_tiles = True

    def cache_shapes(self):
        """(K page tensor shape, V page tensor shape) without the leading page count."""
        s = self.spec
        return (s.kv_heads, self.page, s.dim), (s.kv_heads, self.page, s.vdim)

    def geometry(self, max_blocks: int, num_pages: int):
        s = self.spec
        key = (max_blocks, num_pages)
        if self._geom is None or self._geom[0] != key:
            rot = s.rot
            self._geom = (key, hops.attn_geometry(s.heads, s.kv_heads, s.dim, s.vdim, rot.dims if rot else 0,
                                                  hops.LAYOUTS[rot.layout] if rot else 0, hops.LAYOUTS[s.value_layout], self.page, max_blocks,
                                                  num_pages))
        return self._geom[1]

    def forward(self, h: torch.Tensor, batch: StepBatch, kcache: torch.Tensor, vcache: torch.Tensor) -> torch.Tensor:
        s = self.spec
        geom = self.geometry(batch.block_table.shape[1], kcache.shape[0])
        qkv = hops.dense_linear(h, self.w_in, out_dtype=torch.float32)
        write = self.owns_cache
        hops.attn_prep(qkv, self.koff, self.voff, geom, self.kfreq, self.vfreq, s.value_norm, self.eps, batch.pos, batch.seq, batch.block_table,
                       kcache if write else None, vcache if write else None)
        T = qkv.shape[0]
        # prompt portions (tiles mostly full) go to the matrix-core kernel, decode rows to the one that spreads a row's keys over four waves
        if (self.use_tiles and batch.tile_row0 is not None and batch.tile_row0.numel() * 4 <= T
                and hops.attn_tiles_supported(kcache.dtype, s.dim, s.vdim, self.vfreq is not None, hops.LAYOUTS[s.value_layout])):
            o = hops.attn_tiles(qkv, s.scale, geom, s.chunk, s.sink, self.vfreq, batch.pos, batch.seq, batch.block_table, batch.tile_row0, batch.tile_n,
                                kcache, vcache, s.heads, s.vdim)
        else:
            o = hops.attn_rows(qkv, s.scale, geom, s.chunk, s.sink, self.vfreq, batch.pos, batch.seq, batch.block_table, kcache, vcache, s.heads, s.vdim)
        return hops.dense_linear(o, self.w_o, out_dtype=torch.float32)


class GatedLinearRecurrence:
    def __init__(self, spec: RecurrenceSpec, weights: Dict[str, torch.Tensor], eps: float):
        s = self.spec = spec
        self.eps = eps
        hd = s.heads * s.dim
        if s.kind == "hgrn2":
            self.w_in = torch.cat([weights["q"], weights["f"], weights["v"]], 0).contiguous()
            self.lower, self.fbias = weights["lower"].contiguous(), weights["f.b"].contiguous()
            self.qo, self.ko, self.vo, self.go = 0, hd, 2 * hd, None
            self.mode = hops.SCAN_HGRN2
        elif s.kind == "gla":
            self.w_in = torch.cat([weights["q"], weights["k"], weights["v"], weights["g"]], 0).contiguous()
            self.w_a1, self.w_a2, self.b_a2 = weights["a1"].contiguous(), weights["a2"].contiguous(), weights["a2.b"].contiguous()
            self.qo, self.ko, self.vo, self.go = 0, hd, 2 * hd, 2 * hd + s.heads * s.vdim
            self.lower = self.fbias = None
            self.mode = hops.SCAN_GLA
        else:
            raise ValueError(f"recurrence kind {s.kind!r}")
        self.norm, self.w_o = weights["norm"].contiguous(), weights["o"].contiguous()
        self.act = self.w_o.dtype

    def state_shape(self):
        s = self.spec
        return (s.heads, s.dim, s.vdim)

    def forward(self, h: torch.Tensor, batch: StepBatch, state: torch.Tensor) -> torch.Tensor:
        s = self.spec
        proj = hops.dense_linear(h, self.w_in, out_dtype=torch.float32)
        z = None
        if self.mode == hops.SCAN_GLA:
            z = hops.dense_linear(hops.dense_linear(h, self.w_a1), self.w_a2, self.b_a2, out_dtype=torch.float32)
        o = hops.scan(self.mode, proj, self.qo, self.ko, self.vo, z, self.lower, self.fbias, s.tau, 1.0 / math.sqrt(s.dim), s.heads, s.dim, s.vdim,
                      batch.row_start, batch.slot, batch.first_pos, state, self.act)
        o = hops.head_norm(o, s.heads, s.vdim, self.norm, self.eps, proj if self.go is not None else None, self.go or 0)
        return hops.dense_linear(o, self.w_o, out_dtype=torch.float32)


class GatedMLP:
    """down(act(gate h) * up h) with the gate and up weights grouped for the fused epilogue of the dense linear.  Channel counts that are
    not a multiple of 32 are padded with zero channels (zero gate and up rows, zero down columns)."""

    def __init__(self, gate: torch.Tensor, up: torch.Tensor, down: torch.Tensor, act: str = "relu"):
        ff, K = gate.shape
        pad = (-ff) % 32
        if pad:
            z = torch.zeros(pad, K, dtype=gate.dtype, device=gate.device)
            gate, up = torch.cat([gate, z]), torch.cat([up, z])
            down = torch.cat([down, torch.zeros(down.shape[0], pad, dtype=down.dtype, device=down.device)], 1)
        self.w_gate_up = hops.group_gate_up(gate, up)
        self.w_down = down.contiguous()
        self.act = hops.ACTIVATIONS[act]

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return hops.dense_linear(hops.dense_linear(h, self.w_gate_up, gated=True, act=self.act), self.w_down, out_dtype=torch.float32)
