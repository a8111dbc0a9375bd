"""CPU oracle (TEST INFRASTRUCTURE ONLY) of the Dogalorn design: a plain, slow restatement of its equations in 64-bit torch, one
function per mechanism, one whole sequence at a time, token-by-token loops for everything recurrent, no cache, no state object and
no code shared with vllm_i64_amd/.  However the product path cuts, batches, pages and slots a sequence, its logits at a position
must agree with this file's.

Notation: T tokens, width w; weights `W[name]` as stored ([out, in] matrices); `m` a layer's 'mixer' entry of the config.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

F64 = torch.float64


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def gelu_erf(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.logaddexp(z, torch.zeros_like(z))


# ---- embedding -----------------------------------------------------------------------------------------------------------------
def embedding(W: Dict[str, torch.Tensor], cfg: dict, tokens: List[int]) -> torch.Tensor:
    """embed[token] plus, when the config has a bigram table, its row hash(previous, current); the first token takes the extra last row."""
    x = W["embed"][tokens].clone()
    bg = (cfg.get("embedding") or {}).get("bigram")
    if bg:
        n, a, b = int(bg["buckets"]), int(bg["mul_prev"]), int(bg["mul_cur"])
        rows = [n] + [(tokens[t - 1] * a + tokens[t] * b) % n for t in range(1, len(tokens))]
        x = x + W["bigram"][rows]
    return x


# ---- distance bias ---------------------------------------------------------------------------------------------------------------
def distance_bucket(n: int, rows: int, far: float) -> int:
    """Distances below rows // 2 have a row each; the rest share the upper rows on a logarithmic scale that ends at `far`."""
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half))))


# ---- the two side-by-side mixers -------------------------------------------------------------------------------------------------
def chunked_bias_attention(W: Dict[str, torch.Tensor], p: str, m: dict, eps: float, h: torch.Tensor) -> torch.Tensor:
    """Attention whose values are the unnormalised keys, with a learned distance bias, a sink in the softmax and visibility limited
    to the query's own chunk of positions.  h [T, w] -> [T, w]."""
    T = h.shape[0]
    H, G, d = int(m["heads"]), int(m["kv_heads"]), int(m["dim"])
    size = int((m.get("mask") or {}).get("size", 0))
    q = h @ W[p + "q"].T
    k = h @ W[p + "k"].T
    v = k.reshape(T, G, d)
    qn = (rms(q, eps) * W[p + "q.norm"]).reshape(T, H, d)
    kn = (rms(k, eps) * W[p + "k.norm"]).reshape(T, G, d)
    rel, temp = W[p + "rel"], W[p + "temp"]
    R = rel.shape[0]
    out = torch.zeros(T, H, d, dtype=F64)
    for i in range(T):
        lo = (i // size) * size if size > 0 else 0
        rows = [distance_bucket(i - j, R, float(m["bias_max"])) for j in range(lo, i + 1)]
        for a in range(H):
            g = a // (H // G)
            s = (kn[lo:i + 1, g] @ qn[i, a]) * float(m["scale"]) * temp[a] + rel[rows, a]
            mx = torch.clamp(s.max(), min=0.0)
            e = torch.exp(s - mx)
            wgt = e / (torch.exp(-mx) + e.sum())          # the sink: a score of zero that carries no value
            out[i, a] = wgt @ v[lo:i + 1, g]
    return out.reshape(T, -1) @ W[p + "o"].T


def min_gru(W: Dict[str, torch.Tensor], p: str, h: torch.Tensor) -> torch.Tensor:
    """A gated recurrence whose gate and candidate depend on the current token only."""
    T = h.shape[0]
    z = torch.sigmoid(h @ W[p + "z"].T + W[p + "z.b"])
    u = h @ W[p + "x"].T + W[p + "x.b"]
    cand = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    gate = silu(h @ W[p + "g"].T)
    S = torch.zeros(z.shape[1], dtype=F64)
    rows = []
    for t in range(T):
        S = (1.0 - z[t]) * S + z[t] * cand[t]
        rows.append(S * gate[t])
    return torch.stack(rows) @ W[p + "o"].T


def parallel_mixer(W: Dict[str, torch.Tensor], p: str, m: dict, eps: float, h: torch.Tensor) -> torch.Tensor:
    a = chunked_bias_attention(W, p + "left.", m["left"], eps, h)
    b = min_gru(W, p + "right.", h)
    return 0.5 * (rms(a, eps) * W[p + "left.out"] + rms(b, eps) * W[p + "right.out"])


# ---- state-space mixer -----------------------------------------------------------------------------------------------------------
def mamba2(W: Dict[str, torch.Tensor], p: str, m: dict, eps: float, h: torch.Tensor) -> torch.Tensor:
    T = h.shape[0]
    Hh, P, N, G, taps = int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m["groups"]), int(m["conv"])
    inner = Hh * P
    proj = h @ W[p + "in"].T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    # causal per-channel convolution: the last column of the kernel meets the current token
    cw, cb = W[p + "conv"], W[p + "conv.b"]
    padded = torch.cat([torch.zeros(taps - 1, xbc.shape[1], dtype=F64), xbc], 0)
    conv = torch.stack([(padded[t:t + taps] * cw.T).sum(0) for t in range(T)]) + cb
    act = silu(conv)
    x = act[:, :inner].reshape(T, Hh, P)
    Bm = act[:, inner:inner + G * N].reshape(T, G, N)
    Cm = act[:, inner + G * N:].reshape(T, G, N)
    dt = softplus(dt + W[p + "dt_bias"])
    decay = torch.exp(-torch.exp(W[p + "A_log"]) * dt)               # [T, heads]
    y = torch.zeros(T, Hh, P, dtype=F64)
    for a in range(Hh):
        g = a // (Hh // G)
        S = torch.zeros(N, P, dtype=F64)
        for t in range(T):
            S = decay[t, a] * S + dt[t, a] * torch.outer(Bm[t, g], x[t, a])
            y[t, a] = S.T @ Cm[t, g] + W[p + "D"][a] * x[t, a]
    y = y.reshape(T, inner) * silu(z)
    parts = int(m.get("norm_groups", 1))
    y = rms(y.reshape(T, parts, inner // parts), eps).reshape(T, inner) * W[p + "norm"]
    return y @ W[p + "o"].T


MIXERS = {"parallel": parallel_mixer, "mamba2": mamba2}


# ---- feed-forward ----------------------------------------------------------------------------------------------------------------
def dense_mlp(W: Dict[str, torch.Tensor], p: str, h: torch.Tensor) -> torch.Tensor:
    return gelu_erf(h @ W[p + "up"].T + W[p + "up.b"]) @ W[p + "down"].T + W[p + "down.b"]


# ---- multi-stream residual -------------------------------------------------------------------------------------------------------
def stream_read(W: Dict[str, torch.Tensor], p: str, xs: torch.Tensor) -> torch.Tensor:
    """xs [S, T, w] -> the sublayer's input before its norm: the streams weighted by '<p>in'."""
    return torch.einsum("s,stw->tw", W[p + "in"], xs)


def stream_write(W: Dict[str, torch.Tensor], p: str, xs: torch.Tensor, y: torch.Tensor) -> torch.Tensor:
    """new stream t = sum_s mix[s, t] * old stream s + out[t] * y."""
    return torch.einsum("st,sTw->tTw", W[p + "mix"], xs) + W[p + "out"][:, None, None] * y[None]


# ---- the model -------------------------------------------------------------------------------------------------------------------
def forward(weights: Dict[str, torch.Tensor], cfg: dict, tokens: List[int], layer_outputs: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence.  layer_outputs (a list) receives the summed streams after every layer."""
    W = {k: v.to(F64) for k, v in weights.items()}
    eps = float(cfg["norm"]["eps"])
    S = int(cfg.get("streams", 0))
    x0 = embedding(W, cfg, tokens)
    xs = x0[None].repeat(max(S, 1), 1, 1)
    for i, L in enumerate(cfg["layers"]):
        p = f"l{L.get('weights_of', i)}."
        subs = [(1, lambda h: MIXERS[L["type"]](W, p + "mix.", L["mixer"], eps, h))]
        if L.get("mlp"):
            subs.append((2, lambda h: dense_mlp(W, p + "mlp.", h)))
        for q, fn in subs:
            if S:
                u = stream_read(W, f"{p}hc{q}.", xs)
                xs = stream_write(W, f"{p}hc{q}.", xs, fn(rms(u, eps) * W[f"{p}norm{q}"]))
            else:
                xs = xs + fn(rms(xs[0], eps) * W[f"{p}norm{q}"])[None]
        if layer_outputs is not None:
            layer_outputs.append(xs.sum(0))
    x = xs.sum(0)
    return (rms(x, eps) * W["final.norm"]) @ W["head"].T * float(cfg.get("logit_scale", 1.0))
