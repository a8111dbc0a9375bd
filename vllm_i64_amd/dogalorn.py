"""Runner of the Dogalorn design on one MI355X: a pre-norm decoder whose residual is a set of streams (every sublayer reads a
learned combination of them and writes back through a learned mixing matrix), whose norms carry one number as weight, whose
embedding adds a row chosen by a hash of the previous and the current token, and whose layers (some of which borrow another layer's
tensors) have one of two mixers:

  mamba2    in-projection -> causal convolution + silu over (x, B, C) -> per head S <- exp(-exp(A) dt) S + dt B x^T, y = S^T C + D x
            -> y * silu(z) -> RMS norm in groups -> out-projection
  parallel  attention over the query's chunk of positions whose values are the un-normed keys (whole-row query / key norms, per-head
            temperature, bias by bucketed distance, one added to the softmax denominator) side by side with a gated recurrence
            S <- (1 - z) S + z c(u); the mean of the two separately normed results

  sublayer q of a layer:   u = sum_s in_q[s] x_s;  y = f_q(rms(u) * g_q);  x_t <- sum_s mix_q[s, t] x_s + out_q[t] y
  logits = head . (rms(sum_s x_s) * g) * logit_scale

The streams, norms, recurrences with their decays and gates, scores and softmax are fp32 in both modes; "bfloat16" rounds the inputs
of the matrix products to bf16 (fp32 sums on the matrix cores) and keeps the cached keys in bf16, "float32" keeps everything in 32 bits.
Per layer: one Linear for everything that reads the sublayer input, the recurrent / attention kernels of ops_dense, the output
projections, the feed-forward's two Linears (bias and activation in their epilogues), and one multi-stream launch per sublayer that
writes the streams and prepares the next sublayer's normed input.  torch holds memory and streams; every arithmetic step is a
libi64hip_dense.so kernel.  The step interface is I64MoEModel's, so the same engine, scheduler and decoders drive it."""
from __future__ import annotations

import math
import os
from typing import Dict, List, Optional

import torch

from . import ops_dense as D
from .config import DogalornConfig
from .model import attention_segments
from .paged_cache import HybridCache


def distance_bias_table(rel: torch.Tensor, far: float) -> torch.Tensor:
    """rel [R, heads] -> bias by distance [max(far, R // 2) + 1, heads]: distances below R // 2 take their own row, the rest share the
    upper rows on a logarithmic scale that reaches the last row at `far`; every distance from `far` on takes the last row, so the
    table's last row stands for all of them."""
    R = rel.shape[0]
    half = R // 2
    top = max(int(math.ceil(far)), half) + 1
    bucket = []
    for n in range(top):
        if n < half:
            bucket.append(n)
        elif half > 0 and far > half:
            bucket.append(min(R - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (R - half)))))
        else:
            bucket.append(R - 1)
    return rel.to(torch.float32)[torch.tensor(bucket, dtype=torch.int64)].contiguous()


class _StepBuffers:
    def __init__(self, model: "DogalornModel", n: int, m: int):
        f32 = dict(dtype=torch.float32, device=model.device)
        W = model.cfg.width
        self.streams = torch.empty(model.S, n, W, **f32)
        self.h = torch.empty(n, W, **f32)                       # the normed input of the current sublayer
        self.y = torch.empty(n, W, **f32)
        self.y2 = torch.empty(n, W, **f32)
        self.p = torch.empty(n * model.max_proj, **f32)         # everything projected from the sublayer input
        self.a = torch.empty(n * model.max_a, **f32)            # convolution output / queries
        self.b = torch.empty(n * model.max_b, **f32)            # recurrence / attention output
        self.c = torch.empty(n * model.max_b, **f32)
        self.act = torch.empty(n * max(model.max_ff, 1), **f32)
        self.xf = torch.empty(m, W, **f32)
        self.logits = torch.empty(m, model.cfg.vocab, **f32)
        self.attn_ws: Dict[tuple, torch.Tensor] = {}   # partial results of split attention launches by (rows, heads, key heads, dim, splits)


class DogalornModel:
    MAX_BUFFER_SETS = int(os.environ.get("I64H_MAX_BUFFER_SETS", "8"))
    ATTN_MAX_SEGMENTS = 4     # more runs than this in one step (finely interleaved kinds) collapse into one launch
    ATTN_WAVES = {64: 3072, 128: 2048, 256: 1024}     # waves a decode-sized attention launch aims at, by head size: 1024 SIMDs, and the
                                                      # kernel's instance for narrow rows leaves registers for three waves on each

    def __init__(self, cfg: DogalornConfig, weights: Dict[str, torch.Tensor], device="cuda:0", dtype: str = "bfloat16", max_seqs: int = 4,
                 num_kv_blocks: int = 256, kv_block: int = 16, cache_dtype: Optional[torch.dtype] = None):
        if dtype not in ("bfloat16", "float32"):
            raise ValueError(f"dtype {dtype}: bfloat16 or float32")
        self.cfg, self.device, self.dtype = cfg, torch.device(device), dtype
        self.exact = dtype == "float32"
        dev = self.device
        bf = lambda t: t.to(device=dev, dtype=torch.bfloat16).contiguous()
        f = lambda t: t.to(device=dev, dtype=torch.float32).contiguous()
        W = cfg.width
        self.S = max(1, cfg.streams)

        def need(name, shape):
            if name not in weights:
                raise KeyError(f"tensor '{name}' is missing")
            if tuple(weights[name].shape) != tuple(shape) and not (tuple(shape) == () and weights[name].numel() == 1):     # (a single number, however it is stored)
                raise ValueError(f"'{name}': shape {tuple(weights[name].shape)}, config says {tuple(shape)}")
            return weights[name]

        self.embed, self.head = bf(need("embed", (cfg.vocab, W))), bf(need("head", (cfg.vocab, W)))
        self.final_norm = f(need("final.norm", ()).reshape(1))
        self.bigram = bf(need("bigram", (cfg.bigram.buckets + 1, W))) if cfg.bigram is not None else None
        own = {i: self._load_layer(i, L, weights, need, bf, f) for i, L in enumerate(cfg.layers) if L.weights_of is None}
        self.layers: List[dict] = []
        specs = []
        for i, L in enumerate(cfg.layers):
            self.layers.append(own[i if L.weights_of is None else L.weights_of])     # a borrowed layer: the same tensors, its own cache and state
            if L.type == "mamba2":
                m = L.mixer
                specs.append({"state": {"conv": (max(m.conv - 1, 0), m.conv_channels), "ssm": (m.heads, m.vdim, m.state)}})
            else:
                specs.append({"rows": L.mixer.left.kv_heads * L.mixer.left.dim, "state": {"gru": (L.mixer.right.width,)}})
        self.max_proj = max(d["n_in"] for d in self.layers)
        self.max_a = max(d["n_a"] for d in self.layers)
        self.max_b = max(d["n_b"] for d in self.layers)
        self.max_ff = max([l.mlp.ff for l in cfg.layers if l.mlp is not None] or [0])
        if cache_dtype is None:
            cache_dtype = torch.float32 if self.exact else torch.bfloat16
        self.kv = HybridCache(specs, num_kv_blocks, max_seqs, dev, dtype=cache_dtype, block=kv_block,
                              seq_state={"prev_token": ((), torch.int64)} if cfg.bigram is not None else None)
        self._bufs: Dict[tuple, _StepBuffers] = {}
        self._pinned: set = set()
        self._arange: Dict[int, torch.Tensor] = {}

    # ---- load-time layout work: one weight for everything that reads the sublayer input; small vectors in fp32 ----
    def _load_layer(self, i: int, L, weights, need, bf, f) -> dict:
        cfg, W, S, p = self.cfg, self.cfg.width, self.S, f"l{i}."
        d = dict(type=L.type, m=L.mixer, mlp=L.mlp)
        subs = (1, 2) if L.mlp is not None else (1,)
        for q in subs:
            d[f"norm{q}"] = f(need(f"{p}norm{q}", ()).reshape(1))
            if cfg.streams:
                d[f"hc{q}"] = dict(in_w=f(need(f"{p}hc{q}.in", (S,))), out_w=f(need(f"{p}hc{q}.out", (S,))), mix=f(need(f"{p}hc{q}.mix", (S, S))))
            else:   # the ordinary residual: one stream, read as it is, written back as x + y
                d[f"hc{q}"] = dict(in_w=None, out_w=torch.ones(1, dtype=torch.float32, device=self.device), mix=None)
        if L.type == "mamba2":
            m = L.mixer
            d["w_in"] = bf(need(p + "mix.in", (m.in_width, W)))
            d["b_in"] = None
            d["conv_w"] = f(need(p + "mix.conv", (m.conv_channels, m.conv)))
            d["conv_b"] = f(need(p + "mix.conv.b", (m.conv_channels,)))
            d["dt_bias"], d["A_log"], d["D"] = f(need(p + "mix.dt_bias", (m.heads,))), f(need(p + "mix.A_log", (m.heads,))), f(need(p + "mix.D", (m.heads,)))
            d["norm"], d["o"] = f(need(p + "mix.norm", (m.inner,))), bf(need(p + "mix.o", (W, m.inner)))
            d["n_in"], d["n_a"], d["n_b"] = m.in_width, m.conv_channels, m.inner
        else:
            a, g = L.mixer.left, L.mixer.right
            nq, nk, R = a.heads * a.dim, a.kv_heads * a.dim, g.width
            lp, rp = p + "mix.left.", p + "mix.right."
            # [queries | keys | recurrence gate | recurrence candidate | output gate]
            d["w_in"] = bf(torch.cat([need(lp + "q", (nq, W)), need(lp + "k", (nk, W)), need(rp + "z", (R, W)), need(rp + "x", (R, W)), need(rp + "g", (R, W))], 0))
            d["b_in"] = f(torch.cat([torch.zeros(nq + nk), need(rp + "z.b", (R,)).float(), need(rp + "x.b", (R,)).float(), torch.zeros(R)]))
            d["q_off"], d["k_off"], d["z_off"], d["x_off"], d["g_off"] = 0, nq, nq + nk, nq + nk + R, nq + nk + 2 * R
            d["q_norm"], d["k_norm"] = f(need(lp + "q.norm", (nq,))), f(need(lp + "k.norm", (nk,)))
            d["temp"] = f(need(lp + "temp", (a.heads,)))
            if lp + "rel" not in weights or weights[lp + "rel"].dim() != 2:
                raise KeyError(f"tensor '{lp}rel' is missing or is no table")
            rel = need(lp + "rel", (weights[lp + "rel"].shape[0], a.heads))      # the number of distance buckets is the table's height
            d["bias"] = distance_bias_table(rel.float(), a.bias_max).to(self.device)
            d["o_left"], d["o_right"] = bf(need(lp + "o", (W, a.heads * a.vdim))), bf(need(rp + "o", (W, R)))
            d["out_left"], d["out_right"] = f(need(p + "mix.left.out", (W,))), f(need(p + "mix.right.out", (W,)))
            d["n_in"], d["n_a"], d["n_b"] = nq + nk + 3 * R, nq, max(nq, R)
        if L.mlp is not None:
            ff = L.mlp.ff
            d["up"], d["up_b"] = bf(need(p + "mlp.up", (ff, W))), f(need(p + "mlp.up.b", (ff,)))
            d["down"], d["down_b"] = bf(need(p + "mlp.down", (W, ff))), f(need(p + "mlp.down.b", (W,)))
        return d

    # ---- step buffers (same policy as the other runners: the most recent row counts are kept, pinned sets stay for captured graphs) ----
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

    def snapshot_state(self):
        """The per-sequence recurrent state, for a caller that runs a step which must not count (a warm-up before a graph capture)."""
        return self.kv.snapshot()

    def restore_state(self, held) -> None:
        self.kv.restore(held)

    def _runs(self, n: int, slot_ids: torch.Tensor, tokens_per_seq, rows_are_slots: bool):
        """First rows of the runs of consecutive rows of one sequence, int32 [runs + 1] on the device, and their number."""
        if rows_are_slots:
            t = self._arange.get(n)
            if t is None:
                t = self._arange[n] = torch.arange(n + 1, dtype=torch.int32, device=self.device)
            return t, n
        if tokens_per_seq is None:      # (a caller that does not say how its rows are grouped: read it off the slot ids)
            s = slot_ids.tolist()
            tokens_per_seq, k = [], 0
            for j in range(1, n + 1):
                if j == n or s[j] != s[j - 1]:
                    tokens_per_seq.append(j - k)
                    k = j
        starts = [0]
        for t in tokens_per_seq:
            if int(t) > 0:
                starts.append(starts[-1] + int(t))
        if starts[-1] != n:
            raise ValueError(f"tokens_per_seq adds up to {starts[-1]} rows, the step has {n}")
        return torch.tensor(starts, dtype=torch.int32).to(self.device), len(starts) - 1

    # ---- mixers: the sublayer input is B.h; the result lands in B.y (and B.y2 for the second of two side-by-side mixers) ----
    def _mamba2(self, B, d, l, n, positions, slot_ids, kvc, seg, nseg) -> None:
        m, ex = d["m"], self.exact
        P = B.p[: n * m.in_width].view(n, m.in_width)
        D.linear(B.h, d["w_in"], P, exact=ex)
        xbc = B.a[: n * m.conv_channels].view(n, m.conv_channels)
        st = kvc.state[l]
        D.causal_conv(P, off=m.inner, channels=m.conv_channels, w=d["conv_w"], bias=d["conv_b"], positions=positions, slot_ids=slot_ids,
                      state=st["conv"], out=xbc, n=n)
        y = B.b[: n * m.inner].view(n, m.inner)
        D.ssm_scan(xbc, P, dt_off=m.inner + m.conv_channels, lddt=m.in_width, dt_bias=d["dt_bias"], a_log=d["A_log"], d_skip=d["D"], heads=m.heads,
                   vdim=m.vdim, state=m.state, groups=m.groups, seg_start=seg, nseg=nseg, positions=positions, slot_ids=slot_ids, ssm_state=st["ssm"],
                   y=y, n=n)
        g = B.c[: n * m.inner].view(n, m.inner)
        D.gate_norm(y, d["norm"], g, groups=m.norm_groups, eps=self.cfg.norm_eps, z=P, z_off=0, ldz=m.in_width, n=n)
        D.linear(g, d["o"], B.y, exact=ex)

    def _parallel(self, B, d, l, n, positions, slot_ids, kvc, seg, nseg, runs, ctx_hint) -> None:
        a, g, ex = d["m"].left, d["m"].right, self.exact
        N1 = d["n_in"]
        P = B.p[: n * N1].view(n, N1)
        D.linear(B.h, d["w_in"], P, exact=ex, bias=d["b_in"], epilogue=D.EPI_STORE)
        nq = a.heads * a.dim
        Q = B.a[: n * nq].view(n, nq)
        D.kattn_prep(P, q_off=d["q_off"], k_off=d["k_off"], heads=a.heads, kv_heads=a.kv_heads, dim=a.dim, q_norm_w=d["q_norm"], k_norm_w=d["k_norm"],
                     temp=d["temp"], scale=a.scale, eps=self.cfg.norm_eps, positions=positions, slot_ids=slot_ids, block_table=kvc.block_table,
                     cache=kvc.rows[l], kscale=kvc.kscale[l], q=Q, n=n)
        O = B.b[: n * nq].view(n, nq)
        # runs of rows that are one per sequence (a wave takes a token's query heads of one key head, the keys dealt to several waves) and
        # runs of prompt portions (a wave takes 16 consecutive rows of one head), each one launch
        for r0, r1, one_per_seq in runs:
            splits, ws = 1, None
            if one_per_seq and not ex:
                keys = min(a.chunk, ctx_hint) if a.chunk > 0 else ctx_hint
                tasks = (r1 - r0) * a.kv_heads * ((a.heads // a.kv_heads + 15) // 16)
                waves = self.ATTN_WAVES[64 if a.dim <= 64 else (128 if a.dim <= 128 else 256)]
                splits = max(1, min(waves // max(1, tasks), keys // 64, 64))
                if splits > 1:
                    key = (r1 - r0, a.heads, a.kv_heads, a.dim, splits)
                    ws = B.attn_ws.get(key)
                    if ws is None:
                        ws = B.attn_ws[key] = torch.empty(max(1, D.kattn_workspace_floats(r1 - r0, a.heads, a.kv_heads, a.dim, splits)), dtype=torch.float32,
                                                          device=self.device)
            D.kattn(Q[r0:r1], kvc.rows[l], kvc.kscale[l], kvc.block_table, slot_ids[r0:r1], positions[r0:r1], chunk=a.chunk, bias=d["bias"], sink=True,
                    heads=a.heads, kv_heads=a.kv_heads, dim=a.dim, out=O[r0:r1], n=r1 - r0, mode=2 if one_per_seq else 3, splits=splits, workspace=ws)
        D.linear(O, d["o_left"], B.y, exact=ex)
        R = B.c[: n * g.width].view(n, g.width)
        D.mingru_scan(P, z_off=d["z_off"], x_off=d["x_off"], g_off=d["g_off"], width=g.width, seg_start=seg, nseg=nseg, positions=positions,
                      slot_ids=slot_ids, state=kvc.state[l]["gru"], out=R, n=n)
        D.linear(R, d["o_right"], B.y2, exact=ex)

    @torch.no_grad()
    def forward(self, token_ids: torch.Tensor, positions: torch.Tensor, slot_ids: torch.Tensor, ctx_len: Optional[torch.Tensor] = None,
                logit_rows: Optional[torch.Tensor] = None, max_ctx_hint: int = 0, record: Optional[dict] = None, kv=None,
                rows_are_slots: bool = False, tokens_per_seq: Optional[List[int]] = None) -> torch.Tensor:
        """token_ids int64 [N]; positions / slot_ids int32 [N], rows in sequence order (the rows of a sequence consecutive, positions
        consecutive, continuing what the sequence's slot and pages hold; position 0 starts a sequence afresh); logit_rows int32 [M]
        selects the rows whose logits are wanted (None = all).  Returns fp32 logits [M, V].  record: dict filled with the summed streams
        after every layer ("l<i>.x").  kv: a HybridCache other than the runner's own.  tokens_per_seq (rows per sequence, in order) or
        rows_are_slots (every row a sequence of its own) say how the rows are grouped; without them the slot ids are read back.
        ctx_len and max_ctx_hint belong to the shared step interface."""
        cfg = self.cfg
        kvc = kv if kv is not None else self.kv
        n = token_ids.numel()
        M = logit_rows.numel() if logit_rows is not None else n
        B = self.buffers(n, M)
        if n == 0:
            return B.logits
        eps = cfg.norm_eps
        seg, nseg = self._runs(n, slot_ids, tokens_per_seq, rows_are_slots)
        if tokens_per_seq is not None:
            runs = attention_segments(tokens_per_seq, n, self.ATTN_MAX_SEGMENTS)
        else:
            runs = [(0, n, bool(rows_are_slots))]
        bg = cfg.bigram
        D.embed_bigram(token_ids, positions, slot_ids, self.embed, B.streams, bigram=self.bigram, buckets=bg.buckets if bg else 0,
                       mul_prev=bg.mul_prev if bg else 0, mul_cur=bg.mul_cur if bg else 0, prev_token=kvc.seq_state.get("prev_token"))
        # every multi-stream launch writes the result of the sublayer before it and reads for the sublayer after it
        first = self.layers[0]
        D.streams_step(B.streams, in_w=first["hc1"]["in_w"], norm_w=first["norm1"], eps=eps, h=B.h)
        subs = [(l, q) for l, d in enumerate(self.layers) for q in ((1, 2) if d["mlp"] is not None else (1,))]
        for i, (l, q) in enumerate(subs):
            d = self.layers[l]
            two = False
            if q == 1:
                if d["type"] == "mamba2":
                    self._mamba2(B, d, l, n, positions, slot_ids, kvc, seg, nseg)
                else:
                    self._parallel(B, d, l, n, positions, slot_ids, kvc, seg, nseg, runs, int(max_ctx_hint))
                    two = True
            else:
                ff = d["mlp"].ff
                act = B.act[: n * ff].view(n, ff)
                D.linear(B.h, d["up"], act, exact=self.exact, bias=d["up_b"], epilogue=D.EPI_GELU_ERF)
                D.linear(act, d["down"], B.y, exact=self.exact, bias=d["down_b"])
            hc = d[f"hc{q}"]
            write = dict(y=B.y, mix=hc["mix"], out_w=hc["out_w"])
            if two:
                write.update(y2=B.y2, yn_w=d["out_left"], y2n_w=d["out_right"], y_eps=eps)
            if i + 1 < len(subs):
                nl, nq_ = subs[i + 1]
                nd = self.layers[nl]
                D.streams_step(B.streams, **write, in_w=nd[f"hc{nq_}"]["in_w"], norm_w=nd[f"norm{nq_}"], eps=eps, h=B.h)
            else:
                D.streams_step(B.streams, **write)
            if record is not None and (i + 1 == len(subs) or subs[i + 1][0] != l):
                record[f"l{l}.x"] = B.streams.sum(0)
        rows = logit_rows if logit_rows is not None else None
        D.streams_step(B.streams, norm_w=self.final_norm, eps=eps, h=B.xf, rows=rows)
        D.linear(B.xf, self.head, B.logits, exact=self.exact, epilogue=D.EPI_SCALE, scale=cfg.logit_scale)
        return B.logits

