"""Runner of the Morilorn design on one MI355X: a post-norm decoder whose sublayer results pass a learned sigmoid gate, whose
norms are RMS norms over consecutive groups of the width, whose layer inputs are learned mixes of ALL earlier layer outputs, and
whose attention caches one low-rank latent row per token (latent attention with a sliding window).

    x_0 = embed[token] * s
    layer i on its input x:   a = norm1(alpha x + sigmoid(R1 x + b1) * mixer(x))
                              X_{i+1} = norm2(alpha a + sigmoid(R2 a + b2) * ff(a))          (ff: W_down(gelu_tanh(W_gate a) * W_up a))
                              next input = sum_{j <= i+1} dwa_i[j] X_j
    logits = cap * tanh(head . norm(x) / cap)

The residual stream, norms, gates, rotary angles, scores, softmax and the cache arithmetic are fp32; "bfloat16" rounds the inputs of
the matrix products to bf16 (fp32 sums on the matrix cores), "float32" keeps them in 32 bits.  Per layer and step: one Linear for
everything that reads the layer input (queries, latent, output gate, residual gate), the latent kernels of ops_dense, batched
per-head Linears that carry the query into latent space and the summed latents into value space, and the fused gated post-norm.
torch holds memory and streams; every arithmetic step is a libi64hip_dense.so kernel.  The step interface is I64MoEModel's, so
the same engine, scheduler and decoders drive both."""
from __future__ import annotations

import os
from typing import Dict, List, Optional

import torch

from . import ops_dense as D
from .config import MorilornConfig
from .model import attention_segments
from .paged_cache import LatentCache


def inverse_frequencies(base: float, dims: int) -> torch.Tensor:
    """f_i = base^(-2i / dims), i < dims / 2: evaluated in 64 bits, rounded once to fp32."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    return torch.pow(torch.tensor(float(base), dtype=torch.float64), -2.0 * i / max(dims, 1)).to(torch.float32)


class _StepBuffers:
    def __init__(self, model: "MorilornModel", n: int, m: int):
        f32 = dict(dtype=torch.float32, device=model.device)
        W = model.cfg.width
        self.hist = torch.empty(model.cfg.num_layers + 1, n, W, **f32)     # X_0 .. X_L of this step's rows
        self.x = torch.empty(n, W, **f32)                                  # the mixed input of the next layer
        self.a = torch.empty(n, W, **f32)
        self.y = torch.empty(n, W, **f32)
        self.p = torch.empty(n * model.max_proj, **f32)
        self.p2 = torch.empty(n, W, **f32)
        self.q = torch.empty(n * model.max_q, **f32)
        self.olat = torch.empty(n * model.max_olat, **f32)
        self.og = torch.empty(n * model.max_og, **f32)
        self.act = torch.empty(n * max(model.max_ff, 1), **f32)
        self.xf = torch.empty(m, W, **f32)
        self.logits = torch.empty(m, model.cfg.vocab, **f32)
        self.attn_ws: Dict[tuple, torch.Tensor] = {}   # partial results of split attention launches by (rows, heads, rank, splits)


class MorilornModel:
    MAX_BUFFER_SETS = int(os.environ.get("I64H_MAX_BUFFER_SETS", "8"))
    ATTN_MAX_SEGMENTS = 4     # more runs than this in one step (finely interleaved kinds) collapse into one launch
    ATTN_WAVES = 1024         # waves a decode-sized attention launch aims at (256 CUs, four SIMDs each)

    def __init__(self, cfg: MorilornConfig, weights: Dict[str, torch.Tensor], device="cuda:0", dtype: str = "bfloat16", max_seqs: int = 4,
                 num_kv_blocks: int = 256, kv_block: int = 16, cache_dtype: Optional[torch.dtype] = None):
        if dtype not in ("bfloat16", "float32"):
            raise ValueError(f"dtype {dtype}: bfloat16 or float32")
        self.cfg, self.device, self.dtype = cfg, torch.device(device), dtype
        self.exact = dtype == "float32"
        dev = self.device
        bf = lambda t: t.to(device=dev, dtype=torch.bfloat16).contiguous()
        f = lambda t: t.to(device=dev, dtype=torch.float32).contiguous()
        W = cfg.width
        self.embed, self.head, self.final_norm = bf(weights["embed"]), bf(weights["head"]), f(weights["final.norm"])
        if tuple(self.embed.shape) != (cfg.vocab, W) or tuple(self.head.shape) != (cfg.vocab, W):
            raise ValueError(f"embed {tuple(self.embed.shape)} / head {tuple(self.head.shape)} do not fit vocab {cfg.vocab} x width {W}")
        self.layers: List[dict] = []
        for i, L in enumerate(cfg.layers):
            p, m = f"l{i}.", L.mixer
            H, r, rd = m.heads, m.kv_rank, m.rot_dim
            want = {"mix.q": (m.q_width, W), "mix.dkv": (r + rd, W), "mix.dkv.norm": (r,), "mix.uk": (H * m.dim, r), "mix.uv": (H * m.vdim, r),
                    "mix.g": (H * m.vdim, W), "mix.o": (W, H * m.vdim), "rg1": (W, W), "rg1.b": (W,), "norm1": (W,), "dwa": (i + 2,)}
            if L.mlp is not None:
                want.update({"mlp.gate": (L.mlp.ff, W), "mlp.up": (L.mlp.ff, W), "mlp.down": (W, L.mlp.ff), "rg2": (W, W), "rg2.b": (W,), "norm2": (W,)})
            for k, shp in want.items():
                if p + k not in weights:
                    raise KeyError(f"tensor '{p + k}' is missing")
                if tuple(weights[p + k].shape) != shp:
                    raise ValueError(f"'{p + k}': shape {tuple(weights[p + k].shape)}, config says {shp}")
            d = dict(cfg=L, m=m)
            # everything that reads the layer input, one weight: [queries | latent + shared key | output gate | residual gate]
            d["w_in"] = bf(torch.cat([weights[p + "mix.q"], weights[p + "mix.dkv"], weights[p + "mix.g"], weights[p + "rg1"]], 0))
            d["q_off"], d["dkv_off"], d["g_off"] = 0, m.q_width, m.q_width + r + rd
            d["rg_off"] = d["g_off"] + H * m.vdim
            d["n_in"] = d["rg_off"] + W
            # a head's score against a cached latent c is q_h . (U_h c) = (U_h^T q_h) . c: the key projection transposed per head
            d["uk_t"] = bf(weights[p + "mix.uk"].reshape(H, m.dim, r).transpose(1, 2))       # [H, r, dim]
            d["uv"] = bf(weights[p + "mix.uv"].reshape(H, m.vdim, r))                        # [H, vdim, r]
            d["o"] = bf(weights[p + "mix.o"])
            d["c_norm"], d["rg1_b"], d["norm1"], d["dwa"] = f(weights[p + "mix.dkv.norm"]), f(weights[p + "rg1.b"]), f(weights[p + "norm1"]), f(weights[p + "dwa"])
            d["inv_freq"] = inverse_frequencies(m.rot_base, m.rot_dims).to(dev) if m.rot_dims else None
            if L.mlp is not None:
                d["gate_up"] = bf(torch.cat([weights[p + "mlp.gate"], weights[p + "mlp.up"]], 0))
                d["rg2"], d["down"] = bf(weights[p + "rg2"]), bf(weights[p + "mlp.down"])
                d["rg2_b"], d["norm2"] = f(weights[p + "rg2.b"]), f(weights[p + "norm2"])
            self.layers.append(d)
        mix = [l.mixer for l in cfg.layers]
        self.max_proj = max(d["n_in"] for d in self.layers)
        self.max_q = max(m.heads * m.cache_width for m in mix)
        self.max_olat = max(m.heads * m.kv_rank for m in mix)
        self.max_og = max(m.heads * m.vdim for m in mix)
        self.max_ff = max([l.mlp.ff for l in cfg.layers if l.mlp is not None] or [0])
        if cache_dtype is None:
            cache_dtype = torch.float32 if self.exact else torch.bfloat16
        self.kv = LatentCache([m.cache_width for m in mix], num_kv_blocks, max_seqs, dev, dtype=cache_dtype, block=kv_block)
        self._bufs: Dict[tuple, _StepBuffers] = {}
        self._pinned: set = set()

    # ---- step buffers (same policy as I64MoEModel: the most recent row counts are kept, pinned sets stay for captured graphs) ----
    def buffers(self, n: int, m: int) -> _StepBuffers:
        key = (n, m)
        B = self._bufs.pop(key, None)
        if B is None:
            B = _StepBuffers(self, n, m)
        self._bufs[key] = B
        loose = [k for k in self._bufs if k not in self._pinned and k != key]
        for k in loose[:max(0, len(loose) + 1 - self.MAX_BUFFER_SETS)]:
            del self._bufs[k]
        return B

    def pin_buffers(self, n: int, m: int) -> None:
        self.buffers(n, m)
        self._pinned.add((n, m))

    def check_sync(self, force: bool = True):
        """No launch of this runner waits on a grid barrier: nothing to read back."""

    # ---- mechanisms ----
    def _mixer(self, B: _StepBuffers, d: dict, l: int, n: int, x: torch.Tensor, positions, slot_ids, kvc, runs, ctx_hint: int) -> None:
        """latent attention of layer l on the rows x; the result (before the output projection's gate of the residual) lands in B.y."""
        m, ex = d["m"], self.exact
        H, r, rd, D_ = m.heads, m.kv_rank, m.rot_dim, m.cache_width
        N1 = d["n_in"]
        P = B.p[: n * N1].view(n, N1)
        D.linear(x, d["w_in"], P, exact=ex)
        cache = kvc.rows[l]
        D.latent_prep(P, q_off=d["q_off"], dkv_off=d["dkv_off"], heads=H, dim=m.dim, rot_dim=rd, kv_rank=r, rot_dims=m.rot_dims, c_norm_w=d["c_norm"],
                      eps=self.cfg.norm_eps, inv_freq=d["inv_freq"], positions=positions, slot_ids=slot_ids, block_table=kvc.block_table,
                      block_size=kvc.block, cache=cache, q=B.q, n=n)
        # queries into latent space, per head: Q[:, h, :r] = q_unrotated[:, h, :] @ U_h
        D.linear(P, d["uk_t"], B.q, m=n, n=r, k=m.dim, a_off=d["q_off"], lda=N1, ldc=H * D_, batch=H, a_batch=m.dim + rd, w_batch=r * m.dim,
                 c_batch=D_, exact=ex)
        # runs of rows that are one per sequence (decode rows: a wave takes a token's heads) and runs of prompt portions (a wave takes 16
        # consecutive rows of one head), each one launch
        for a, b, one_per_seq in runs:
            splits, ws = 1, None
            if one_per_seq:
                # few rows with long contexts: a token's keys are dealt to several waves, about four waves per CU in the launch, a wave
                # keeping at least two tiles of 32 keys
                keys = min(m.window, ctx_hint) if m.window > 0 else ctx_hint
                splits = max(1, min(self.ATTN_WAVES // max(1, (b - a) * ((H + 15) // 16)), keys // 64, 64))
                if splits > 1:
                    key = (b - a, H, r, splits)
                    ws = B.attn_ws.get(key)
                    if ws is None:
                        ws = B.attn_ws[key] = torch.empty(max(1, D.latent_attn_workspace_floats(b - a, H, r, splits)), dtype=torch.float32, device=self.device)
            D.latent_attn(B.q[a * H * D_: b * H * D_], cache, kvc.block_table, slot_ids[a:b], positions[a:b], window=m.window, scale=m.scale, heads=H,
                          kv_rank=r, rot_dim=rd, out=B.olat[a * H * r: b * H * r], n=b - a, mode=2 if one_per_seq else 3, splits=splits, workspace=ws)
        # summed latents into value space, per head, times the output gate sigmoid(W_g x)
        D.linear(B.olat, d["uv"], B.og, m=n, n=m.vdim, k=r, lda=H * r, ldc=H * m.vdim, batch=H, a_batch=r, w_batch=m.vdim * r, c_batch=m.vdim,
                 exact=ex, epilogue=D.EPI_MUL_SIGMOID, e=P, e_off=d["g_off"], lde=N1, e_batch=m.vdim)
        D.linear(B.og, d["o"], B.y, m=n, k=H * m.vdim, lda=H * m.vdim, exact=ex)

    @torch.no_grad()
    def forward(self, token_ids: torch.Tensor, positions: torch.Tensor, slot_ids: torch.Tensor, ctx_len: Optional[torch.Tensor] = None,
                logit_rows: Optional[torch.Tensor] = None, max_ctx_hint: int = 0, record: Optional[dict] = None, kv=None,
                rows_are_slots: bool = False, tokens_per_seq: Optional[List[int]] = None) -> torch.Tensor:
        """token_ids int64 [N]; positions / slot_ids int32 [N] (a row sees the cached positions of its sequence up to its own, within
        the layer's window); logit_rows int32 [M] selects the rows whose logits are wanted (None = all).  Returns fp32 logits [M, V].
        record: dict filled with the stream after every layer ("l<i>.out": the mixed input of the next layer, "l<i>.x": the layer's own
        output).  kv: a LatentCache other than the runner's own.  ctx_len, max_ctx_hint, rows_are_slots and tokens_per_seq belong to
        the shared step interface; tokens_per_seq (or rows_are_slots) only picks the attention launch forms."""
        cfg = self.cfg
        kvc = kv if kv is not None else self.kv
        n = token_ids.numel()
        M = logit_rows.numel() if logit_rows is not None else n
        B = self.buffers(n, M)
        if n == 0:
            return B.logits
        W, al, G, eps = cfg.width, cfg.postln_alpha, cfg.norm_groups, cfg.norm_eps
        D.embed_scaled(token_ids, self.embed, cfg.embedding_scale, B.hist[0])
        x = B.hist[0]
        if tokens_per_seq is not None:
            runs = attention_segments(tokens_per_seq, n, self.ATTN_MAX_SEGMENTS)
        else:
            runs = [(0, n, bool(rows_are_slots))]
        for l, d in enumerate(self.layers):
            self._mixer(B, d, l, n, x, positions, slot_ids, kvc, runs, int(max_ctx_hint))
            mixk = dict(hist=B.hist, hist_index=l + 1, mix_w=d["dwa"], mix_out=B.x)
            gate1 = dict(y=B.y, gate_pre=B.p, gate_off=d["rg_off"], ldg=d["n_in"], gate_bias=d["rg1_b"], alpha=al, n=n)
            if d["cfg"].mlp is None:
                D.gated_postnorm(x, d["norm1"], G, eps, **gate1, **mixk)
            else:
                ff = d["cfg"].mlp.ff
                D.gated_postnorm(x, d["norm1"], G, eps, out=B.a, **gate1)
                act = B.act[: n * ff].view(n, ff)
                D.linear(B.a, d["gate_up"], act, exact=self.exact, epilogue=D.EPI_GELU_MUL)
                D.linear(B.a, d["rg2"], B.p2, exact=self.exact)
                D.linear(act, d["down"], B.y, exact=self.exact)
                D.gated_postnorm(B.a, d["norm2"], G, eps, y=B.y, gate_pre=B.p2, ldg=W, gate_bias=d["rg2_b"], alpha=al, n=n, **mixk)
            x = B.x
            if record is not None:
                record[f"l{l}.x"] = B.hist[l + 1].clone()
                record[f"l{l}.out"] = B.x.clone()
        D.gated_postnorm(x, self.final_norm, G, eps, x_rows=logit_rows, out=B.xf, n=M)
        cap = cfg.logit_softcap
        D.linear(B.xf, self.head, B.logits, exact=self.exact, epilogue=D.EPI_SOFTCAP if cap > 0 else D.EPI_STORE, softcap=cap)
        return B.logits
