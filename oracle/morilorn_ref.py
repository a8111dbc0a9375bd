"""CPU oracle (TEST INFRASTRUCTURE ONLY) of the Morilorn design: a plain, slow restatement of its equations in 64-bit torch, one
function per mechanism, whole sequences at once, keys and values of every head written out in full (no latent-space shortcut).
It shares no code with vllm_i64_amd/ and has no cache: whatever way the product path cuts, batches and pages a sequence, its
logits at a position must agree with this file's.

Notation: T tokens, width w, H heads; per head d unrotated and e rotated query/key dimensions, v value dimensions; latent rank r.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

F64 = torch.float64


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float, groups: int = 1) -> torch.Tensor:
    """The last axis in `groups` equal consecutive parts, each divided by sqrt(mean(part^2) + eps); then * weight."""
    shape = x.shape
    parts = x.reshape(*shape[:-1], groups, shape[-1] // groups)
    parts = parts / torch.sqrt(parts.pow(2).mean(-1, keepdim=True) + eps)
    return parts.reshape(shape) * weight


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z.pow(3))))


def rotate_pairs(x: torch.Tensor, positions: torch.Tensor, base: float, dims: int) -> torch.Tensor:
    """x [T, ..., n]: dimensions 2i and 2i+1 (i < dims/2) of the last axis turn by positions[t] * base^(-2i/dims); the rest stay."""
    out = x.clone()
    T = x.shape[0]
    for i in range(dims // 2):
        ang = positions.to(F64) * (float(base) ** (-2.0 * i / dims))
        c = torch.cos(ang).reshape(T, *([1] * (x.dim() - 2)))
        s = torch.sin(ang).reshape(T, *([1] * (x.dim() - 2)))
        a, b = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = a * c - b * s
        out[..., 2 * i + 1] = b * c + a * s
    return out


def visible(T: int, window: int) -> torch.Tensor:
    """[T, T] bool: query i sees key j iff 0 <= i - j (< window when window > 0)."""
    i = torch.arange(T).reshape(T, 1)
    j = torch.arange(T).reshape(1, T)
    ok = (i - j) >= 0
    if window > 0:
        ok = ok & ((i - j) < window)
    return ok


def latent_attention(w: Dict[str, torch.Tensor], p: str, m: dict, eps: float, h: torch.Tensor) -> torch.Tensor:
    """The mixer on the rows h [T, w] of one sequence (positions 0 .. T-1).  m: the layer's 'mixer' entry of the config."""
    T = h.shape[0]
    H, d, e, v, r = m["heads"], m["dim"], m.get("rot_dim", 0), m["vdim"], m["kv_rank"]
    rot = m.get("rot") or {}
    base, rdims = rot.get("base", 10000.0), rot.get("dims", e)
    window = (m.get("mask") or {}).get("size", 0)
    pos = torch.arange(T)
    q = (h @ w[p + "mix.q"].T).reshape(T, H, d + e)
    down = h @ w[p + "mix.dkv"].T
    latent = rms_norm(down[:, :r], w[p + "mix.dkv.norm"], eps)
    k_rot = rotate_pairs(down[:, r:], pos, base, rdims) if e else down[:, r:]
    q_plain, q_rot = q[..., :d], q[..., d:]
    if e:
        q_rot = rotate_pairs(q_rot, pos, base, rdims)
    k_plain = (latent @ w[p + "mix.uk"].T).reshape(T, H, d)
    val = (latent @ w[p + "mix.uv"].T).reshape(T, H, v)
    see = visible(T, window)
    heads = []
    for a in range(H):
        s = (q_plain[:, a] @ k_plain[:, a].T + q_rot[:, a] @ k_rot.T) * m["scale"]
        s = s.masked_fill(~see, float("-inf"))
        heads.append(torch.softmax(s, dim=-1) @ val[:, a])
    o = torch.cat(heads, dim=-1) * torch.sigmoid(h @ w[p + "mix.g"].T)
    return o @ w[p + "mix.o"].T


def dense_ff(w: Dict[str, torch.Tensor], p: str, h: torch.Tensor) -> torch.Tensor:
    return (gelu_tanh(h @ w[p + "mlp.gate"].T) * (h @ w[p + "mlp.up"].T)) @ w[p + "mlp.down"].T


def gated_postnorm(x: torch.Tensor, sub: torch.Tensor, gate_w: torch.Tensor, gate_b: torch.Tensor, alpha: float, norm_w: torch.Tensor,
                   eps: float, groups: int) -> torch.Tensor:
    """norm(alpha x + sigmoid(gate_w x + gate_b) * sub)."""
    return rms_norm(alpha * x + torch.sigmoid(x @ gate_w.T + gate_b) * sub, norm_w, eps, groups)


def forward(cfg: dict, weights: Dict[str, torch.Tensor], tokens: List[int], streams: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence.  streams (a list) receives the input of the next layer after every layer."""
    w = {k: t.to(F64) for k, t in weights.items()}
    norm = cfg.get("norm") or {}
    eps, groups, alpha = norm.get("eps", 1e-6), norm.get("groups", 1), cfg.get("postln_alpha", 1.0)
    x = w["embed"][torch.tensor(tokens)] * (cfg.get("embedding") or {}).get("scale", 1.0)
    outs = [x]
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        assert layer["type"] == "latent_attention"
        x = gated_postnorm(x, latent_attention(w, p, layer["mixer"], eps, x), w[p + "rg1"], w[p + "rg1.b"], alpha, w[p + "norm1"], eps, groups)
        if layer.get("mlp"):
            x = gated_postnorm(x, dense_ff(w, p, x), w[p + "rg2"], w[p + "rg2.b"], alpha, w[p + "norm2"], eps, groups)
        outs.append(x)
        x = sum(w[p + "dwa"][j] * outs[j] for j in range(i + 2))
        if streams is not None:
            streams.append(x)
    logits = rms_norm(x, w["final.norm"], eps, groups) @ w["head"].T
    cap = cfg.get("logit_softcap") or 0.0
    return cap * torch.tanh(logits / cap) if cap > 0 else logits


def greedy(cfg: dict, weights: Dict[str, torch.Tensor], prompt: List[int], steps: int) -> List[int]:
    """Greedy continuation, the whole sequence run again for every token."""
    toks, out = list(prompt), []
    for _ in range(steps):
        nxt = int(forward(cfg, weights, toks)[-1].argmax())
        out.append(nxt)
        toks.append(nxt)
    return out


def make_config(*, vocab=96, width=48, layers=2, heads=3, dim=8, rot_dim=4, vdim=12, kv_rank=20, window=7, ff=40, groups=3, scale=0.31,
                alpha=1.7, embed_scale=3.0, softcap=9.0, rot_base=500.0, rot_dims=None, eps=1e-5, per_layer: Optional[list] = None) -> dict:
    """A small configuration in the checkpoint's config.json form; per_layer: a list of dicts overriding the mixer keys
    (and 'ff', None for a layer without feed-forward, 'window') layer by layer."""
    out = []
    for i in range(layers):
        o = dict(per_layer[i]) if per_layer else {}
        e = o.get("rot_dim", rot_dim)
        mixer = {"heads": o.get("heads", heads), "dim": o.get("dim", dim), "rot_dim": e, "vdim": o.get("vdim", vdim), "kv_rank": o.get("kv_rank", kv_rank),
                 "scale": o.get("scale", scale), "rot": {"base": o.get("rot_base", rot_base), "dims": o.get("rot_dims", rot_dims if rot_dims is not None else e)}}
        win = o.get("window", window)
        if win:
            mixer["mask"] = {"size": win}
        f = o.get("ff", ff)
        out.append({"type": "latent_attention", "mixer": mixer, "mlp": {"kind": "dense", "ff": f} if f else None})
    return {"architecture": "Morilorn", "vocab": vocab, "width": width, "layers": out, "embedding": {"scale": embed_scale}, "postln_alpha": alpha,
            "norm": {"eps": eps, "groups": groups}, "logit_softcap": softcap}


def make_weights(cfg: dict, seed: int = 0) -> Dict[str, torch.Tensor]:
    """Random bf16 weights of the checkpoint's names and shapes; scales chosen so that gates, scores and logits stay in a range
    where every mechanism matters (no saturated sigmoid, no one-hot softmax)."""
    g = torch.Generator().manual_seed(seed)
    w_, V = cfg["width"], cfg["vocab"]

    def mat(n, k, gain=1.0):
        return (torch.randn(n, k, generator=g) * (gain / math.sqrt(k))).to(torch.bfloat16)

    def vec(n, mean=1.0, std=0.1):
        return (mean + std * torch.randn(n, generator=g)).to(torch.bfloat16)

    out = {"embed": (torch.randn(V, w_, generator=g) * 0.5).to(torch.bfloat16), "head": mat(V, w_, 2.0), "final.norm": vec(w_)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        H, d, e, v, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
        out.update({p + "mix.q": mat(H * (d + e), w_, 2.0), p + "mix.dkv": mat(r + e, w_, 2.0), p + "mix.dkv.norm": vec(r), p + "mix.uk": mat(H * d, r, 2.0),
                    p + "mix.uv": mat(H * v, r, 2.0), p + "mix.g": mat(H * v, w_), p + "mix.o": mat(w_, H * v, 2.0), p + "rg1": mat(w_, w_), p + "rg1.b": vec(w_, 0.3, 0.3),
                    p + "norm1": vec(w_), p + "dwa": (torch.randn(i + 2, generator=g) * 0.4 + 0.5).to(torch.bfloat16)})
        if layer.get("mlp"):
            f = layer["mlp"]["ff"]
            out.update({p + "mlp.gate": mat(f, w_, 2.0), p + "mlp.up": mat(f, w_, 2.0), p + "mlp.down": mat(w_, f, 2.0), p + "rg2": mat(w_, w_),
                        p + "rg2.b": vec(w_, 0.3, 0.3), p + "norm2": vec(w_)})
    return out
