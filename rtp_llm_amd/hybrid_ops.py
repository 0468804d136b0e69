"""Tensor-level wrappers over libmi355_hybrid.so: dense linears on checkpoint-layout weights and the kernels of the hybrid decoder
family (csrc/gemm_dense.hip, csrc/hybrid_ops.hip).  As in ``ops``: PyTorch supplies device memory and the current stream, every
function enqueues hand-written HIP kernels and never falls back.  Activations and weights are bfloat16 or float32 (`act`); what the
family keeps in 32-bit (residual stream, projections that feed gates and rotations, recurrent state, logits) is float32 in both."""
import ctypes as C
from typing import Optional

import torch

from . import _C

ACT_NONE, ACT_RELU, ACT_SILU = 0, 1, 2
ACTIVATIONS = {"none": ACT_NONE, "relu": ACT_RELU, "silu": ACT_SILU}
SCAN_HGRN2, SCAN_GLA = 0, 1
LAYOUTS = {"interleaved": 0, "halves": 1}


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _p(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def act_code(dtype: torch.dtype) -> int:
    if dtype == torch.bfloat16:
        return _C.ACT_BF16
    if dtype == torch.float32:
        return _C.ACT_F32
    raise _C.Mi355Error(f"hybrid ops run in bfloat16 or float32, not {dtype}")


def _dev(t: torch.Tensor, dtype, name: str):
    if not t.is_cuda:
        raise _C.Mi355Error(f"{name}: tensor must live on the GPU (no CPU path exists)")
    if t.dtype != dtype:
        raise _C.Mi355Error(f"{name}: expected {dtype}, got {t.dtype}")


def _rows(t: torch.Tensor, name: str) -> int:
    """Leading dimension of a 2-D tensor whose rows are contiguous (a column slice of a wider buffer is fine)."""
    if t.dim() != 2 or t.stride(1) != 1:
        raise _C.Mi355Error(f"{name}: expected a 2-D tensor with contiguous rows, got shape {tuple(t.shape)} strides {t.stride()}")
    return t.stride(0)


def dense_linear(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None, *, out_dtype: Optional[torch.dtype] = None,
                 gated: bool = False, act: int = ACT_NONE, softcap: float = 0.0, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """y = x @ w.T (+ bias) for w [N, K] in checkpoint layout.  gated: w holds groups of 32 gate rows followed by the 32 up rows of the
    same channels and y [M, N / 2] = act(gate) * up.  out_dtype float32 keeps the accumulator; softcap > 0 applies cap * tanh(y / cap)."""
    _dev(x, w.dtype, "dense_linear.x"); _dev(w, w.dtype, "dense_linear.w")
    ldx = _rows(x, "dense_linear.x")
    M, K = x.shape
    N = w.shape[0]
    if w.dim() != 2 or w.shape[1] != K or not w.is_contiguous():
        raise _C.Mi355Error(f"dense_linear: x {tuple(x.shape)} against w {tuple(w.shape)}")
    if bias is not None:
        _dev(bias, w.dtype, "dense_linear.bias")
        if bias.numel() != N or not bias.is_contiguous():
            raise _C.Mi355Error(f"dense_linear: bias {tuple(bias.shape)} for N={N}")
    if gated and N % 64:
        raise _C.Mi355Error(f"dense_linear: a gated weight has whole groups of 64 rows, N={N}")
    od = out_dtype or w.dtype
    if w.dtype == torch.float32:
        od = torch.float32
    if od not in (torch.float32, w.dtype):
        raise _C.Mi355Error(f"dense_linear: output {od} from {w.dtype} operands")
    n_out = N // 2 if gated else N
    if out is None:
        out = torch.empty(M, n_out, dtype=od, device=x.device)
    else:
        _dev(out, od, "dense_linear.out")
        if out.shape != (M, n_out):
            raise _C.Mi355Error(f"dense_linear: out {tuple(out.shape)} for [{M}, {n_out}]")
    ldy = _rows(out, "dense_linear.out")
    if M == 0:
        return out
    _C.check_hybrid(_C.hybrid_lib().mi355_dense_linear(x.data_ptr(), ldx, M, w.data_ptr(), N, K, _p(bias), out.data_ptr(), ldy,
                                                       1 if od == torch.float32 else 0, 1 if gated else 0, act, float(softcap),
                                                       act_code(w.dtype), _stream()), "dense_linear")
    return out


def group_gate_up(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """[ff, K] gate and up weights -> the [2 ff, K] weight of a gated dense_linear: per 32 channels, 32 gate rows then 32 up rows
    (ff % 32 == 0)."""
    ff, K = gate.shape
    if ff % 32 or up.shape != gate.shape:
        raise ValueError(f"group_gate_up: gate {tuple(gate.shape)} up {tuple(up.shape)} (channels in whole groups of 32)")
    return torch.stack([gate.view(ff // 32, 32, K), up.view(ff // 32, 32, K)], dim=1).reshape(2 * ff, K).contiguous()


def embed(ids: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
    """fp32 stream rows [T, W] of the token ids."""
    _dev(ids, torch.int32, "embed.ids")
    T = ids.numel()
    out = torch.empty(T, table.shape[1], dtype=torch.float32, device=table.device)
    if T:
        _C.check_hybrid(_C.hybrid_lib().mi355_hy_embed(ids.data_ptr(), T, table.data_ptr(), table.shape[1], table.shape[0], out.data_ptr(),
                                                       act_code(table.dtype), _stream()), "hy_embed")
    return out


def residual_norm(x: torch.Tensor, a: Optional[torch.Tensor], b: Optional[torch.Tensor], mult: float, w1: torch.Tensor,
                  w2: Optional[torch.Tensor], eps: float, *, weight_offset: float = 0.0, rows: Optional[torch.Tensor] = None):
    """x <- x + mult * (a + b) on the fp32 stream (in place; skipped for absent branches, and x is only read when `rows` gathers), then
    RMS norms of the new rows under w1 and w2 (stored weight + weight_offset).  -> (h1, h2) in the weights' dtype."""
    _dev(x, torch.float32, "residual_norm.x")
    W = x.shape[1]
    n = x.shape[0] if rows is None else rows.numel()
    for t, nm in ((a, "a"), (b, "b")):
        if t is not None:
            _dev(t, torch.float32, "residual_norm." + nm)
            if t.shape != x.shape or not t.is_contiguous():
                raise _C.Mi355Error(f"residual_norm.{nm}: {tuple(t.shape)} against the stream {tuple(x.shape)}")
    if rows is not None:
        _dev(rows, torch.int32, "residual_norm.rows")
    if not x.is_contiguous() or w1.numel() != W or (w2 is not None and (w2.numel() != W or w2.dtype != w1.dtype)):
        raise _C.Mi355Error("residual_norm: stream must be contiguous and the weights [W] of one dtype")
    h1 = torch.empty(n, W, dtype=w1.dtype, device=x.device)
    h2 = torch.empty(n, W, dtype=w1.dtype, device=x.device) if w2 is not None else None
    if n:
        _C.check_hybrid(_C.hybrid_lib().mi355_hy_residual_norm(x.data_ptr(), _p(a), _p(b), float(mult), _p(rows), n, W, w1.data_ptr(), _p(w2),
                                                               float(weight_offset), float(eps), h1.data_ptr(), _p(h2), act_code(w1.dtype),
                                                               _stream()), "hy_residual_norm")
    return h1, h2


def attn_geometry(heads, kv_heads, dim, vdim, rot_dims, rot_layout, v_layout, page, max_blocks, num_pages):
    return (C.c_int32 * 10)(heads, kv_heads, dim, vdim, rot_dims, rot_layout, v_layout, page, max_blocks, num_pages)


def attn_prep(qkv: torch.Tensor, koff: int, voff: int, geom, kfreq, vfreq, v_norm: bool, eps: float, pos, seq, block_table,
              kcache: Optional[torch.Tensor], vcache: Optional[torch.Tensor]):
    """Rotate the query heads of qkv (fp32 [T, ld], in place); with caches: rotate the keys, unit-norm and rotate the values, and write both
    to their pages."""
    _dev(qkv, torch.float32, "attn_prep.qkv")
    ld = _rows(qkv, "attn_prep.qkv")
    T = qkv.shape[0]
    if not T:
        return
    dt = kcache.dtype if kcache is not None else torch.float32
    _C.check_hybrid(_C.hybrid_lib().mi355_hy_attn_prep(qkv.data_ptr(), ld, koff, voff, geom, _p(kfreq), _p(vfreq), 1 if v_norm else 0, float(eps),
                                                       pos.data_ptr(), seq.data_ptr(), _p(block_table), T, _p(kcache), _p(vcache), act_code(dt),
                                                       _stream()), "hy_attn_prep")


def attn_rows(q: torch.Tensor, scale: float, geom, chunk: int, sink: bool, vfreq, pos, seq, block_table, kcache, vcache, heads: int, vdim: int):
    """Attention of every row over its sequence's pages -> [T, heads * vdim] in the cache dtype."""
    _dev(q, torch.float32, "attn_rows.q")
    T = q.shape[0]
    out = torch.empty(T, heads * vdim, dtype=kcache.dtype, device=q.device)
    if T:
        _C.check_hybrid(_C.hybrid_lib().mi355_hy_attn_rows(q.data_ptr(), _rows(q, "attn_rows.q"), float(scale), geom, int(chunk), 1 if sink else 0, _p(vfreq),
                                                           pos.data_ptr(), seq.data_ptr(), block_table.data_ptr(), T, kcache.data_ptr(), vcache.data_ptr(),
                                                           out.data_ptr(), act_code(kcache.dtype), _stream()), "hy_attn_rows")
    return out


def attn_tiles_supported(dtype: torch.dtype, dim: int, vdim: int, value_rot: bool, v_layout: int) -> bool:
    """Shapes the MFMA kernel for prompt portions takes (attn_rows serves every other)."""
    return dtype == torch.bfloat16 and dim % 32 == 0 and dim <= 256 and vdim % 16 == 0 and vdim <= 256 and not (value_rot and v_layout and vdim % 32)


def attn_tiles(q: torch.Tensor, scale: float, geom, chunk: int, sink: bool, vfreq, pos, seq, block_table, tile_row0, tile_n, kcache, vcache,
               heads: int, vdim: int):
    """attn_rows for prompt portions on the matrix cores: tile t = rows tile_row0[t] .. + tile_n[t] - 1 (at most 16 consecutive rows of one
    sequence); every row of the batch must lie in exactly one tile."""
    _dev(q, torch.float32, "attn_tiles.q"); _dev(tile_row0, torch.int32, "attn_tiles.tile_row0"); _dev(tile_n, torch.int32, "attn_tiles.tile_n")
    T = q.shape[0]
    out = torch.empty(T, heads * vdim, dtype=kcache.dtype, device=q.device)
    if T:
        _C.check_hybrid(_C.hybrid_lib().mi355_hy_attn_tiles(q.data_ptr(), _rows(q, "attn_tiles.q"), float(scale), geom, int(chunk), 1 if sink else 0, _p(vfreq),
                                                            pos.data_ptr(), seq.data_ptr(), block_table.data_ptr(), tile_row0.data_ptr(), tile_n.data_ptr(),
                                                            tile_row0.numel(), kcache.data_ptr(), vcache.data_ptr(), out.data_ptr(),
                                                            act_code(kcache.dtype), _stream()), "hy_attn_tiles")
    return out


def scan(mode: int, proj: torch.Tensor, qo: int, ko: int, vo: int, z: Optional[torch.Tensor], lower, fbias, tau: float, qscale: float,
         heads: int, dim: int, vdim: int, row_start, slot, first_pos, state: torch.Tensor, act: torch.dtype) -> torch.Tensor:
    """Gated linear recurrence over the rows of every sequence, continuing (and leaving) the fp32 state of its slot -> fp32 [T, heads * vdim]."""
    _dev(proj, torch.float32, "scan.proj"); _dev(state, torch.float32, "scan.state")
    T = proj.shape[0]
    out = torch.empty(T, heads * vdim, dtype=torch.float32, device=proj.device)
    nseq = slot.numel()
    if T and nseq:
        _C.check_hybrid(_C.hybrid_lib().mi355_hy_scan(mode, proj.data_ptr(), _rows(proj, "scan.proj"), qo, ko, vo, _p(z), 0 if z is None else _rows(z, "scan.z"),
                                                      _p(lower), _p(fbias), float(tau), float(qscale), heads, dim, vdim, row_start.data_ptr(),
                                                      slot.data_ptr(), first_pos.data_ptr(), nseq, state.data_ptr(), out.data_ptr(), act_code(act),
                                                      _stream()), "hy_scan")
    return out


def head_norm(o: torch.Tensor, heads: int, vdim: int, w: torch.Tensor, eps: float, gate: Optional[torch.Tensor] = None, goff: int = 0) -> torch.Tensor:
    """Per-head RMS norm of o (fp32 [T, heads * vdim]) under the shared weight w [vdim], times silu(gate[:, goff:]) when a gate is given."""
    _dev(o, torch.float32, "head_norm.o")
    T = o.shape[0]
    out = torch.empty(T, heads * vdim, dtype=w.dtype, device=o.device)
    if T:
        _C.check_hybrid(_C.hybrid_lib().mi355_hy_head_norm(o.data_ptr(), T, heads, vdim, w.data_ptr(), float(eps), _p(gate),
                                                           0 if gate is None else _rows(gate, "head_norm.gate"), goff, out.data_ptr(),
                                                           act_code(w.dtype), _stream()), "hy_head_norm")
    return out
