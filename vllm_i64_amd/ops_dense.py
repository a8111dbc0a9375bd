"""Torch-facing wrappers over libi64hip_dense.so (include/i64h_dense.h): memory and stream plumbing only, no torch math and no
CPU path.  Activations are fp32 tensors, weights bf16 tensors [out, in]."""
from __future__ import annotations

import ctypes
from typing import Optional

import torch

from . import _lib
from ._lib import call_dense, ptr
from .ops import _chk, _stream

EPI_STORE, EPI_GELU_MUL, EPI_MUL_SIGMOID, EPI_SOFTCAP = 0, 1, 2, 3
CACHE_DTYPE_CODE = {torch.float32: 0, torch.bfloat16: 2}


def _ref(s):
    return ctypes.addressof(s)


def linear(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, *, m: Optional[int] = None, n: Optional[int] = None, k: Optional[int] = None,
           a_off: int = 0, lda: Optional[int] = None, a_rows: Optional[torch.Tensor] = None, c_off: int = 0, ldc: Optional[int] = None,
           batch: int = 1, a_batch: int = 0, w_batch: int = 0, c_batch: int = 0, exact: bool = False, epilogue: int = EPI_STORE,
           e: Optional[torch.Tensor] = None, e_off: int = 0, lde: int = 0, e_batch: int = 0, softcap: float = 0.0) -> torch.Tensor:
    """out[b][:, c_off + b * c_batch : + n] = epilogue(a[b][rows, a_off + b * a_batch : + k] @ w[b]^T): see i64h_linear.  a, out and e are
    fp32 matrices addressed by (column offset, row stride); w is bf16 [n, k] (EPI_GELU_MUL: [2n, k], gate rows first), or a stack
    [batch, n, k] with w_batch = n * k."""
    _chk(a, torch.float32, "a"), _chk(w, torch.bfloat16, "w"), _chk(out, torch.float32, "out")
    if a_rows is not None:
        _chk(a_rows, torch.int32, "a_rows")
    N = int(n if n is not None else w.shape[-2] // (2 if epilogue == EPI_GELU_MUL else 1))
    K = int(k if k is not None else w.shape[-1])
    M = int(m if m is not None else (a_rows.numel() if a_rows is not None else a.shape[0]))
    lda = int(lda if lda is not None else a.shape[-1])
    ldc = int(ldc if ldc is not None else out.shape[-1])
    if w.shape[-1] != K or a_off + (batch - 1) * a_batch + K > lda or c_off + (batch - 1) * c_batch + N > ldc:
        raise _lib.I64HError(f"linear: K {K} / N {N} do not fit a (row stride {lda}), w {tuple(w.shape)} or out (row stride {ldc})")
    if out.numel() < (M - 1) * ldc + c_off + (batch - 1) * c_batch + N or (a_rows is None and a.numel() < (M - 1) * lda + a_off + (batch - 1) * a_batch + K):
        raise _lib.I64HError("linear: operand smaller than the launch reads or writes")
    if w.numel() < (batch - 1) * w_batch + N * K * (2 if epilogue == EPI_GELU_MUL else 1):
        raise _lib.I64HError("linear: weight smaller than the launch reads")
    if e is not None:
        _chk(e, torch.float32, "e")
        if e.numel() < (M - 1) * lde + e_off + (batch - 1) * e_batch + N:
            raise _lib.I64HError("linear: gate operand smaller than the launch reads")
    d = _lib.Linear(A=ptr(a) + 4 * a_off, lda=lda, a_rows=ptr(a_rows), W=ptr(w), C=ptr(out) + 4 * c_off, ldc=ldc, M=M, N=N, K=K, batch=batch,
                    a_batch=a_batch, w_batch=w_batch, c_batch=c_batch, exact=int(exact), epilogue=epilogue,
                    E=(ptr(e) + 4 * e_off) if e is not None else 0, lde=lde, e_batch=e_batch, softcap=float(softcap))
    call_dense("i64h_linear_run", _ref(d), _stream())
    return out


def embed_scaled(ids: torch.Tensor, table: torch.Tensor, scale: float, out: torch.Tensor) -> torch.Tensor:
    _chk(ids, torch.int64, "ids"), _chk(table, torch.bfloat16, "table"), _chk(out, torch.float32, "out")
    V, W = table.shape
    assert out.numel() >= ids.numel() * W
    call_dense("i64h_embed_scaled", ptr(ids), ptr(table), float(scale), ptr(out), ids.numel(), W, V, _stream())
    return out


def gated_postnorm(x: torch.Tensor, norm_w: torch.Tensor, groups: int, eps: float, *, n: Optional[int] = None, alpha: float = 1.0,
                   y: Optional[torch.Tensor] = None, ldy: Optional[int] = None, gate_pre: Optional[torch.Tensor] = None, gate_off: int = 0,
                   ldg: int = 0, gate_bias: Optional[torch.Tensor] = None, x_rows: Optional[torch.Tensor] = None,
                   out: Optional[torch.Tensor] = None, hist: Optional[torch.Tensor] = None, hist_index: int = 0,
                   mix_w: Optional[torch.Tensor] = None, mix_out: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """See i64h_postnorm.  x fp32 [*, W]; n rows (default: x_rows' count, else x's); hist fp32 [layers + 1, n, W]."""
    _chk(x, torch.float32, "x"), _chk(norm_w, torch.float32, "norm_w")
    W = norm_w.numel()
    rows = int(n if n is not None else (x_rows.numel() if x_rows is not None else x.numel() // W))
    for t, name in ((y, "y"), (gate_pre, "gate_pre"), (gate_bias, "gate_bias"), (out, "out"), (hist, "hist"), (mix_w, "mix_w"), (mix_out, "mix_out")):
        if t is not None:
            _chk(t, torch.float32, name)
    if x_rows is not None:
        _chk(x_rows, torch.int32, "x_rows")
    if mix_w is not None:
        if hist is None or mix_out is None or mix_w.numel() < hist_index + 1 or hist.numel() < (hist_index + 1) * rows * W or hist.shape[-2] != rows:
            raise _lib.I64HError("gated_postnorm: the depth mix needs hist [>= hist_index + 1, n, W], mix_out and hist_index + 1 weights")
    d = _lib.PostNorm(x=ptr(x), x_rows=ptr(x_rows), y=ptr(y), ldy=int(ldy if ldy is not None else W), gate_pre=(ptr(gate_pre) + 4 * gate_off) if gate_pre is not None else 0,
                      ldg=int(ldg), gate_bias=ptr(gate_bias), alpha=float(alpha), norm_w=ptr(norm_w), groups=int(groups), eps=float(eps),
                      out=ptr(out), hist=ptr(hist), hist_index=int(hist_index), mix_w=ptr(mix_w), mix_out=ptr(mix_out), n=rows, W=W)
    call_dense("i64h_gated_postnorm", _ref(d), _stream())
    return out if out is not None else mix_out


def latent_prep(p: torch.Tensor, *, q_off: int, dkv_off: int, heads: int, dim: int, rot_dim: int, kv_rank: int, rot_dims: int,
                c_norm_w: torch.Tensor, eps: float, inv_freq: Optional[torch.Tensor], positions: torch.Tensor, slot_ids: torch.Tensor,
                block_table: torch.Tensor, block_size: int, cache: torch.Tensor, q: torch.Tensor, n: Optional[int] = None) -> None:
    _chk(p, torch.float32, "p"), _chk(c_norm_w, torch.float32, "c_norm_w"), _chk(q, torch.float32, "q")
    _chk(positions, torch.int32, "positions"), _chk(slot_ids, torch.int32, "slot_ids"), _chk(block_table, torch.int32, "block_table")
    _chk(cache, None, "cache")
    rows = int(n if n is not None else positions.numel())
    D = kv_rank + rot_dim
    if cache.shape[-1] != D or cache.shape[-2] != block_size or q.numel() < rows * heads * D or positions.numel() < rows or slot_ids.numel() < rows:
        raise _lib.I64HError("latent_prep: cache / query / position shapes do not fit the sizes")
    if q_off + heads * (dim + rot_dim) > p.shape[-1] or dkv_off + D > p.shape[-1] or c_norm_w.numel() != kv_rank:
        raise _lib.I64HError("latent_prep: projection columns outside the projection rows")
    if rot_dims:
        _chk(inv_freq, torch.float32, "inv_freq")
        assert inv_freq.numel() >= rot_dims // 2
    d = _lib.LatentPrep(P=ptr(p), ldp=p.shape[-1], q_off=q_off, dkv_off=dkv_off, heads=heads, dim=dim, rot_dim=rot_dim, kv_rank=kv_rank,
                        rot_dims=rot_dims, c_norm_w=ptr(c_norm_w), eps=float(eps), inv_freq=ptr(inv_freq) if rot_dims else 0,
                        positions=ptr(positions), slot_ids=ptr(slot_ids), block_table=ptr(block_table), max_blocks_per_seq=block_table.shape[1],
                        block_size=block_size, cache=ptr(cache), cache_dtype=CACHE_DTYPE_CODE[cache.dtype], Q=ptr(q), n=rows)
    call_dense("i64h_latent_prep", _ref(d), _stream())


def latent_attn(q: torch.Tensor, cache: torch.Tensor, block_table: torch.Tensor, slot_ids: torch.Tensor, positions: torch.Tensor, *,
                window: int, scale: float, heads: int, kv_rank: int, rot_dim: int, out: torch.Tensor, n: Optional[int] = None,
                mode: int = 0, splits: int = 1, workspace: Optional[torch.Tensor] = None) -> torch.Tensor:
    _chk(q, torch.float32, "q"), _chk(out, torch.float32, "out"), _chk(cache, None, "cache")
    _chk(positions, torch.int32, "positions"), _chk(slot_ids, torch.int32, "slot_ids"), _chk(block_table, torch.int32, "block_table")
    rows = int(n if n is not None else positions.numel())
    D = kv_rank + rot_dim
    if cache.shape[-1] != D or q.numel() < rows * heads * D or out.numel() < rows * heads * kv_rank:
        raise _lib.I64HError("latent_attn: cache / query / output shapes do not fit the sizes")
    if splits > 1:
        need = latent_attn_workspace_floats(rows, heads, kv_rank, splits)
        if workspace is None:
            workspace = torch.empty(need, dtype=torch.float32, device=q.device)
        _chk(workspace, torch.float32, "workspace")
        if workspace.numel() < need:
            raise _lib.I64HError(f"latent_attn: workspace of {workspace.numel()} floats, {need} needed")
    d = _lib.LatentAttn(Q=ptr(q), cache=ptr(cache), cache_dtype=CACHE_DTYPE_CODE[cache.dtype], block_table=ptr(block_table),
                        max_blocks_per_seq=block_table.shape[1], block_size=cache.shape[-2], slot_ids=ptr(slot_ids), positions=ptr(positions),
                        window=int(window), scale=float(scale), out=ptr(out), n=rows, heads=heads, kv_rank=kv_rank, rot_dim=rot_dim, mode=mode,
                        splits=int(splits) if splits > 1 else 1, workspace=ptr(workspace) if splits > 1 else 0)
    call_dense("i64h_latent_attn", _ref(d), _stream())
    return out


def latent_attn_workspace_floats(n: int, heads: int, kv_rank: int, splits: int) -> int:
    return int(_lib.load_dense().i64h_latent_attn_workspace_floats(n, heads, kv_rank, splits))


def sample_rows(logits: torch.Tensor, out: Optional[torch.Tensor] = None, temperature: Optional[torch.Tensor] = None,
                top_k: Optional[torch.Tensor] = None, top_p: Optional[torch.Tensor] = None, u: Optional[torch.Tensor] = None) -> torch.Tensor:
    """One token per row (see i64h_sample_rows); with no temperature tensor every row is greedy."""
    _chk(logits, torch.float32, "logits")
    rows, V = logits.shape
    if out is None:
        out = torch.empty(rows, dtype=torch.int64, device=logits.device)
    for t, dt, name in ((temperature, torch.float32, "temperature"), (top_k, torch.int32, "top_k"), (top_p, torch.float32, "top_p"), (u, torch.float32, "u")):
        if t is not None:
            _chk(t, dt, name)
            assert t.numel() == rows
    call_dense("i64h_sample_rows", ptr(logits), ptr(out), rows, V, ptr(temperature), ptr(top_k), ptr(top_p), ptr(u), _stream())
    return out
