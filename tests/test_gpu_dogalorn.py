"""The Dogalorn design on the GPU against the CPU oracle (oracle/dogalorn_ref.py): every mechanism alone, then whole models of
several small shapes under every way of cutting, batching, paging and slotting their sequences, through the engine and the command
line.  Weights are random and bf16-representable; where random weights would hide a fault (a far key among many, the edge of a
chunk) the inputs are made so that one score stands out."""
import json
import math
import os
import subprocess
import sys

import pytest
import torch

from oracle import dogalorn_ref as R

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
# rms over the vocabulary of the logit difference / rms of the logits, worst position.  bfloat16: rows of 32 to 128 values average little
# of the 2^-9 input rounding of every matrix product out, and a recurrence carries it on: 1.5 % at the mean position and up to 8 % at the
# worst of 150, the same to seven digits whether a prompt runs whole or token by token; a wrong mechanism gives 50 % and more
TOL = {"float32": 3e-5, "bfloat16": 1.5e-1}


@pytest.fixture(scope="module")
def dev():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


def rel_err(got, want):
    got, want = torch.as_tensor(got, dtype=torch.float64).cpu(), torch.as_tensor(want, dtype=torch.float64).cpu()
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    return float((d.pow(2).mean(-1).sqrt() / want.pow(2).mean(-1).sqrt().clamp_min(1e-9)).max())


def close(got, want, tol=2e-5):
    got, want = torch.as_tensor(got, dtype=torch.float64).cpu(), torch.as_tensor(want, dtype=torch.float64).cpu()
    return float((got - want).abs().max() / want.abs().max().clamp_min(1e-9)) <= tol


# ---- configurations: nothing equal and nothing a power of two / the branches that a config may leave out / wider vectors ----
def mamba(heads, vdim, state, groups=1, conv=4, norm_groups=1):
    return {"type": "mamba2", "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv, "norm_groups": norm_groups}}


def par(heads, kv_heads, dim, chunk, width, scale=None, bias_max=20, rel_rows=8):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale if scale is not None else dim ** -0.5, "bias_max": bias_max}
    if chunk:
        left["mask"] = {"size": chunk}
    return {"type": "parallel", "mixer": {"left": left, "right": {"width": width}}, "_rel_rows": rel_rows}


def layer(mix, ff, weights_of=None):
    d = dict(mix)
    d["mlp"] = {"kind": "dense", "ff": ff} if ff else None
    if weights_of is not None:
        d["weights_of"] = weights_of
    return d


SHAPES = {
    "odd": {"architecture": "Dogalorn", "vocab": 83, "width": 40, "streams": 3, "logit_scale": 1.7, "norm": {"eps": 1e-5},
            "embedding": {"bigram": {"buckets": 13, "mul_prev": 5, "mul_cur": 3}},
            "layers": [layer(par(6, 2, 10, 7, 24, rel_rows=9, bias_max=11), 36), layer(mamba(6, 10, 6, groups=3, conv=3, norm_groups=2), None),
                       layer(par(6, 2, 10, 7, 24, rel_rows=9, bias_max=11), 36, weights_of=0), layer(mamba(2, 14, 5, conv=6), 28),
                       layer(mamba(6, 10, 6, groups=3, conv=3, norm_groups=2), None, weights_of=1)]},
    "plain": {"architecture": "Dogalorn", "vocab": 64, "width": 32, "norm": {"eps": 1e-6},
              "layers": [layer(mamba(2, 8, 4, conv=1), 48), layer(par(1, 1, 16, 0, 8, bias_max=40, rel_rows=6), 48), layer(par(4, 4, 4, 16, 40, rel_rows=4, bias_max=9), None)]},
    "wide": {"architecture": "Dogalorn", "vocab": 200, "width": 128, "streams": 1, "logit_scale": 0.5, "norm": {"eps": 1e-6},
             "embedding": {"bigram": {"buckets": 64, "mul_prev": 1, "mul_cur": 1}},
             "layers": [layer(mamba(4, 64, 16, groups=2, conv=5, norm_groups=4), 160), layer(par(2, 1, 64, 33, 128, rel_rows=32, bias_max=48), 160),
                        layer(par(3, 3, 32, 5, 100, rel_rows=2, bias_max=3), 96)]},
}


def config_of(name):
    cfg = json.loads(json.dumps(SHAPES[name]))
    for l in cfg["layers"]:
        l.pop("_rel_rows", None)
    return cfg


def make_weights(name, seed=0):
    shape = SHAPES[name]
    g = torch.Generator().manual_seed(seed)
    W, S = shape["width"], shape.get("streams", 0)
    rn = lambda *s, std=1.0: (torch.randn(*s, generator=g) * std).to(torch.bfloat16)
    un = lambda lo, hi, *s: (torch.rand(tuple(s), generator=g) * (hi - lo) + lo).to(torch.bfloat16)
    lin = lambda o, i: rn(o, i, std=i ** -0.5)
    w = {"embed": rn(shape["vocab"], W), "head": lin(shape["vocab"], W), "final.norm": un(0.5, 1.5)}
    bg = (shape.get("embedding") or {}).get("bigram")
    if bg:
        w["bigram"] = rn(bg["buckets"] + 1, W, std=0.7)
    for i, L in enumerate(shape["layers"]):
        if "weights_of" in L:
            continue
        p, m = f"l{i}.", L["mixer"]
        for q in (1, 2) if L["mlp"] else (1,):
            w[f"{p}norm{q}"] = un(0.5, 1.5)
            if S:
                w[f"{p}hc{q}.in"] = un(0.2, 1.0, S)
                w[f"{p}hc{q}.out"] = un(0.5, 1.5, S)
                w[f"{p}hc{q}.mix"] = (torch.eye(S) * 0.8 + torch.randn(S, S, generator=g) * 0.2).to(torch.bfloat16)
        if L["type"] == "mamba2":
            inner, ch = m["heads"] * m["vdim"], m["heads"] * m["vdim"] + 2 * m["groups"] * m["state"]
            w.update({p + "mix.in": lin(inner + ch + m["heads"], W), p + "mix.conv": rn(ch, m["conv"], std=0.5), p + "mix.conv.b": rn(ch, std=0.2),
                      p + "mix.dt_bias": un(-2.0, 1.0, m["heads"]), p + "mix.A_log": un(-1.5, 1.0, m["heads"]), p + "mix.D": un(0.5, 1.5, m["heads"]),
                      p + "mix.norm": un(0.5, 1.5, inner), p + "mix.o": lin(W, inner)})
        else:
            a, r = m["left"], m["right"]["width"]
            nq, nk = a["heads"] * a["dim"], a["kv_heads"] * a["dim"]
            w.update({p + "mix.left.q": lin(nq, W), p + "mix.left.k": lin(nk, W), p + "mix.left.q.norm": un(0.5, 1.5, nq), p + "mix.left.k.norm": un(0.5, 1.5, nk),
                      p + "mix.left.rel": rn(L["_rel_rows"], a["heads"]), p + "mix.left.temp": un(0.5, 2.0, a["heads"]), p + "mix.left.o": lin(W, nq),
                      p + "mix.right.z": lin(r, W), p + "mix.right.z.b": rn(r, std=0.5), p + "mix.right.x": lin(r, W), p + "mix.right.x.b": rn(r, std=0.5),
                      p + "mix.right.g": lin(r, W), p + "mix.right.o": lin(W, r), p + "mix.left.out": un(0.5, 1.5, W), p + "mix.right.out": un(0.5, 1.5, W)})
        if L["mlp"]:
            ff = L["mlp"]["ff"]
            w.update({p + "mlp.up": lin(ff, W), p + "mlp.up.b": rn(ff, std=0.3), p + "mlp.down": lin(W, ff), p + "mlp.down.b": rn(W, std=0.3)})
    return w


def make_model(name, dtype, dev, max_tokens=512, max_seqs=4, seed=0, block=16):
    from vllm_i64_amd.config import DogalornConfig
    from vllm_i64_amd.dogalorn import DogalornModel
    return DogalornModel(DogalornConfig.from_dict(config_of(name)), make_weights(name, seed), device=dev, dtype=dtype, max_seqs=max_seqs,
                         num_kv_blocks=(max_tokens + block - 1) // block, kv_block=block)


def tokens(name, n, seed):
    return torch.randint(0, SHAPES[name]["vocab"], (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def oracle_logits(name, toks, seed=0, layers=None):
    return R.forward(make_weights(name, seed), config_of(name), toks, layers)


def replay(engine, requests, schedule):
    """schedule: steps of [(id, count)]; every position's logits are asked for.  Returns id -> [T, V] (CPU)."""
    at = {i: 0 for i in requests}
    got = {i: [] for i in requests}
    for step in schedule:
        entries, end = [], []
        for i, count in step:
            lo, hi = at[i], at[i] + count
            entries.append((i, requests[i][lo:hi], list(range(count))))
            at[i] = hi
            if hi == len(requests[i]):
                end.append(i)
        lg = engine.step(entries, end=end).cpu()
        row = 0
        for i, count in step:
            got[i].append(lg[row:row + count].clone())
            row += count
    return {i: torch.cat(v) for i, v in got.items() if v}


# =================================================== mechanisms alone =============================================================
class Rows:
    """Rows of a step for op-level calls: sequences of (slot, first position, count) laid out one after the other."""

    def __init__(self, dev, runs):
        self.slots = torch.tensor([s for s, p, c in runs for _ in range(c)], dtype=torch.int32, device=dev)
        self.pos = torch.tensor([p + j for s, p, c in runs for j in range(c)], dtype=torch.int32, device=dev)
        st = [0]
        for s, p, c in runs:
            st.append(st[-1] + c)
        self.seg = torch.tensor(st, dtype=torch.int32, device=dev)
        self.nseg, self.n = len(runs), st[-1]


def cuts_of(T, sizes):
    out, at, i = [], 0, 0
    while at < T:
        c = min(sizes[i % len(sizes)], T - at)
        out.append((at, c))
        at += c
        i += 1
    return out


@pytest.mark.parametrize("epi", ["bias", "gelu_erf", "scale"])
@pytest.mark.parametrize("M", [1, 5, 40, 150])
@pytest.mark.parametrize("exact", [False, True])
def test_linear_bias_epilogues(dev, epi, M, exact):
    from vllm_i64_amd import ops_dense as D
    g = torch.Generator().manual_seed(M)
    N, K = 72, 104
    a = torch.randn(M, K, generator=g)
    w = (torch.randn(N, K, generator=g) * K ** -0.5).to(torch.bfloat16)
    b = torch.randn(N, generator=g)
    out = torch.empty(M, N, device=dev)
    ar = a.to(torch.bfloat16).double() if not exact else a.double()
    z = ar @ w.double().T + b.double()
    if epi == "bias":
        D.linear(a.to(dev), w.to(dev), out, exact=exact, bias=b.to(dev))
        want = z
    elif epi == "gelu_erf":
        D.linear(a.to(dev), w.to(dev), out, exact=exact, bias=b.to(dev), epilogue=D.EPI_GELU_ERF)
        want = R.gelu_erf(z)
    else:
        D.linear(a.to(dev), w.to(dev), out, exact=exact, bias=b.to(dev), epilogue=D.EPI_SCALE, scale=2.5)
        want = z * 2.5
    assert close(out, want, 1e-5)


def test_bigram_embedding_keeps_the_previous_token_per_slot(dev):
    from vllm_i64_amd import ops_dense as D
    g = torch.Generator().manual_seed(1)
    V, W, nb = 50, 24, 7
    cfg = {"embedding": {"bigram": {"buckets": nb, "mul_prev": 11, "mul_cur": 4}}}
    w = {"embed": torch.randn(V, W, generator=g).to(torch.bfloat16), "bigram": torch.randn(nb + 1, W, generator=g).to(torch.bfloat16)}
    seqs = {0: torch.randint(0, V, (9,), generator=g).tolist(), 2: torch.randint(0, V, (6,), generator=g).tolist()}
    want = {s: R.embedding({k: v.double() for k, v in w.items()}, cfg, t) for s, t in seqs.items()}
    prev = torch.full((4,), 33, dtype=torch.int64, device=dev)      # stale values: a slot that was used before
    emb, big = w["embed"].to(dev), w["bigram"].to(dev)
    # step 1: 4 tokens of slot 0 and 1 of slot 2; step 2: 1 and 3; step 3: the rest
    at = {0: 0, 2: 0}
    for counts in ({0: 4, 2: 1}, {0: 1, 2: 3}, {2: 2, 0: 4}):
        runs = [(s, at[s], c) for s, c in counts.items()]
        r = Rows(dev, runs)
        ids = torch.tensor([t for s, p, c in runs for t in seqs[s][p:p + c]], dtype=torch.int64, device=dev)
        out = torch.empty(2, r.n, W, device=dev)
        D.embed_bigram(ids, r.pos, r.slots, emb, out, bigram=big, buckets=nb, mul_prev=11, mul_cur=4, prev_token=prev)
        row = 0
        for s, p, c in runs:
            for copy in range(2):
                assert close(out[copy, row:row + c], want[s][p:p + c], 1e-6)
            row += c
            at[s] += c
    assert prev[0].item() == seqs[0][-1] and prev[2].item() == seqs[2][-1]


@pytest.mark.parametrize("S,W", [(1, 24), (2, 300), (3, 40), (8, 64)])
def test_streams_write_and_read(dev, S, W):
    from vllm_i64_amd import ops_dense as D
    g = torch.Generator().manual_seed(S)
    n, eps = 5, 1e-5
    xs, y, y2 = torch.randn(S, n, W, generator=g), torch.randn(n, W, generator=g), torch.randn(n, W, generator=g) * 3
    w = {"a.mix": torch.randn(S, S, generator=g), "a.out": torch.randn(S, generator=g), "b.in": torch.randn(S, generator=g)}
    wd = {k: v.double() for k, v in w.items()}
    nw, lw, rw = torch.rand(1, generator=g) + 0.5, torch.rand(W, generator=g) + 0.5, torch.rand(W, generator=g) + 0.5
    for two in (False, True):
        v = 0.5 * (R.rms(y.double(), eps) * lw.double() + R.rms(y2.double(), eps) * rw.double()) if two else y.double()
        new = R.stream_write(wd, "a.", xs.double(), v)
        want_h = R.rms(R.stream_read(wd, "b.", new), eps) * nw.double()
        st, h = xs.clone().to(dev), torch.empty(n, W, device=dev)
        kw = dict(y2=y2.to(dev), yn_w=lw.to(dev), y2n_w=rw.to(dev), y_eps=eps) if two else {}
        D.streams_step(st, y=y.to(dev), mix=w["a.mix"].to(dev), out_w=w["a.out"].to(dev), in_w=w["b.in"].to(dev), norm_w=nw.to(dev), eps=eps, h=h, **kw)
        assert close(st, new, 1e-5) and close(h, want_h, 1e-5)
    # read only, gathered rows, the plain sum of the streams, a norm weight per column
    rows = torch.tensor([4, 0, 2], dtype=torch.int32, device=dev)
    h = torch.empty(3, W, device=dev)
    D.streams_step(xs.to(dev), norm_w=lw.to(dev), eps=eps, h=h, rows=rows)
    assert close(h, (R.rms(xs.double().sum(0), eps) * lw.double())[[4, 0, 2]], 1e-5)
    # the ordinary residual: one stream, no mixing matrix
    if S == 1:
        st = xs.clone().to(dev)
        D.streams_step(st, y=y.to(dev), out_w=torch.ones(1, device=dev))
        assert close(st, xs + y, 1e-6)


def _mamba_case(dev, heads, vdim, state, groups, conv, norm_groups, cut_sizes, seed, lens=None):
    """The state-space mixer from its in-projection's output on: convolution, recurrence, gate and norm; two sequences in slots 3 and 1,
    cut into portions, against the oracle (whose out-projection is the identity here)."""
    from vllm_i64_amd import ops_dense as D
    g = torch.Generator().manual_seed(seed)
    inner, ch = heads * vdim, heads * vdim + 2 * groups * state
    nin = inner + ch + heads
    m = {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv, "norm_groups": norm_groups}
    w = {"in": torch.eye(nin), "conv": torch.randn(ch, conv, generator=g) * 0.5, "conv.b": torch.randn(ch, generator=g) * 0.2,
         "dt_bias": torch.rand(heads, generator=g) * 3 - 2, "A_log": torch.rand(heads, generator=g) * 2.5 - 1.5, "D": torch.rand(heads, generator=g) + 0.5,
         "norm": torch.rand(inner, generator=g) + 0.5, "o": torch.eye(inner)}
    eps = 1e-5
    lens = lens or {3: 150, 1: 70}
    proj = {s: torch.randn(T, nin, generator=g) for s, T in lens.items()}
    want = {s: R.mamba2({k: v.double() for k, v in w.items()}, "", m, eps, proj[s].double()) for s in lens}
    cw, cb = w["conv"].to(dev), w["conv.b"].to(dev)
    conv_state = torch.full((4, max(conv - 1, 0), ch), 7.0, device=dev)       # stale contents: position 0 has to ignore them
    ssm_state = torch.full((4, heads, vdim, state), -3.0, device=dev)
    cuts = {s: cuts_of(T, cut_sizes) for s, T in lens.items()}
    got = {s: [] for s in lens}
    for k in range(max(len(c) for c in cuts.values())):
        runs = [(s, *cuts[s][k]) for s in lens if k < len(cuts[s])]
        r = Rows(dev, runs)
        P = torch.cat([proj[s][p:p + c] for s, p, c in runs]).to(dev).contiguous()
        xbc, y, o = torch.empty(r.n, ch, device=dev), torch.empty(r.n, inner, device=dev), torch.empty(r.n, inner, device=dev)
        D.causal_conv(P, off=inner, channels=ch, w=cw, bias=cb, positions=r.pos, slot_ids=r.slots, state=conv_state, out=xbc, n=r.n)
        D.ssm_scan(xbc, P, dt_off=inner + ch, lddt=nin, dt_bias=w["dt_bias"].to(dev), a_log=w["A_log"].to(dev), d_skip=w["D"].to(dev), heads=heads, vdim=vdim,
                   state=state, groups=groups, seg_start=r.seg, nseg=r.nseg, positions=r.pos, slot_ids=r.slots, ssm_state=ssm_state, y=y, n=r.n)
        D.gate_norm(y, w["norm"].to(dev), o, groups=norm_groups, eps=eps, z=P, z_off=0, ldz=nin, n=r.n)
        row = 0
        for s, p, c in runs:
            got[s].append(o[row:row + c].cpu())
            row += c
    for s in lens:
        assert close(torch.cat(got[s]), want[s], 3e-5), (s, cut_sizes)


@pytest.mark.parametrize("cut_sizes", [[64], [200], [1], [2, 5, 1, 3, 90], [7, 2]])
def test_mamba2_mechanism_under_cuts(dev, cut_sizes):
    _mamba_case(dev, heads=6, vdim=10, state=6, groups=3, conv=3, norm_groups=2, cut_sizes=cut_sizes, seed=1)
    _mamba_case(dev, heads=2, vdim=64, state=16, groups=1, conv=5, norm_groups=1, cut_sizes=cut_sizes, seed=2)
    _mamba_case(dev, heads=1, vdim=3, state=130, groups=1, conv=1, norm_groups=3, cut_sizes=cut_sizes, seed=3)
    _mamba_case(dev, heads=2, vdim=20, state=32, groups=2, conv=8, norm_groups=1, cut_sizes=cut_sizes, seed=4)
    _mamba_case(dev, heads=1, vdim=17, state=7, groups=1, conv=11, norm_groups=1, cut_sizes=cut_sizes, seed=5)


@pytest.mark.parametrize("conv", [2, 4, 7, 8])
def test_mamba2_mechanism_long_launches(dev, conv):
    """Launches of 512 rows and more (the convolution then walks 16 rows per thread), runs that start and end inside a walk."""
    for cut_sizes in ([700], [523, 1, 40]):
        _mamba_case(dev, heads=2, vdim=5, state=4, groups=1, conv=conv, norm_groups=1, cut_sizes=cut_sizes, seed=conv, lens={3: 571, 1: 90, 0: 7})


@pytest.mark.parametrize("cut_sizes", [[200], [1], [2, 9, 1, 30]])
@pytest.mark.parametrize("width", [5, 300])
def test_mingru_mechanism_under_cuts(dev, cut_sizes, width):
    from vllm_i64_amd import ops_dense as D
    g = torch.Generator().manual_seed(width)
    w = {"z": torch.eye(width), "x": torch.eye(width), "g": torch.eye(width), "o": torch.eye(width), "z.b": torch.zeros(width), "x.b": torch.zeros(width)}
    wd = {k: v.double() for k, v in w.items()}
    lens = {0: 200, 2: 9}
    # the oracle projects one input three times; here the three projections are separate columns, so the oracle runs on a mechanism
    # of three equal projections and the product on three copies of the same columns
    h = {s: torch.randn(T, width, generator=g) * 2 for s, T in lens.items()}
    want = {s: R.min_gru(wd, "", h[s].double()) for s in lens}
    state = torch.full((4, width), 9.0, device=dev)
    cuts = {s: cuts_of(T, cut_sizes) for s, T in lens.items()}
    got = {s: [] for s in lens}
    for k in range(max(len(c) for c in cuts.values())):
        runs = [(s, *cuts[s][k]) for s in lens if k < len(cuts[s])]
        r = Rows(dev, runs)
        x = torch.cat([h[s][p:p + c] for s, p, c in runs])
        P = torch.cat([x, x, x], 1).to(dev).contiguous()
        out = torch.empty(r.n, width, device=dev)
        D.mingru_scan(P, z_off=0, x_off=width, g_off=2 * width, width=width, seg_start=r.seg, nseg=r.nseg, positions=r.pos, slot_ids=r.slots, state=state, out=out, n=r.n)
        row = 0
        for s, p, c in runs:
            got[s].append(out[row:row + c].cpu())
            row += c
    for s in lens:
        assert close(torch.cat(got[s]), want[s], 2e-5)


class KeyPages:
    """A hand-made paged key cache for one sequence in slot 1 whose pages are scattered and in no order."""

    def __init__(self, dev, T, width, block, dtype):
        nb = (T + block - 1) // block
        self.rows = torch.zeros(2 * nb + 3, block, width, dtype=dtype, device=dev)
        self.kscale = torch.zeros(2 * nb + 3, block, device=dev)
        perm = torch.randperm(2 * nb + 3, generator=torch.Generator().manual_seed(T))[:nb]
        bt = torch.full((3, nb), -1, dtype=torch.int32)
        bt[1] = perm.to(torch.int32)
        self.bt = bt.to(dev)


def _kattn_run(dev, h, m, w, eps, cut_sizes, block, dtype=torch.float32, form="row"):
    """Query / key projections are the identity: the rows h are both; returns the attention output per position [T, heads * dim].
    form: "row" the one-wave-per-(row, head) kernel; "mfma" the matrix-core kernel (bf16 cache), 16 rows of a head per wave for
    portions and the heads of one token per wave, its keys dealt to three waves, for single rows."""
    from vllm_i64_amd import ops_dense as D
    from vllm_i64_amd.dogalorn import distance_bias_table
    T, nq = h.shape
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    pages = KeyPages(dev, T, G * d, block, dtype)
    bias = distance_bias_table(w["rel"], float(m["bias_max"])).to(dev)
    outs = []
    for p, c in cuts_of(T, cut_sizes):
        r = Rows(dev, [(1, p, c)])
        P = h[p:p + c].to(dev).contiguous()
        Q, O = torch.empty(c, nq, device=dev), torch.empty(c, nq, device=dev)
        D.kattn_prep(P, q_off=0, k_off=0, heads=H, kv_heads=G, dim=d, q_norm_w=w["q.norm"].to(dev), k_norm_w=w["k.norm"].to(dev), temp=w["temp"].to(dev),
                     scale=m["scale"], eps=eps, positions=r.pos, slot_ids=r.slots, block_table=pages.bt, cache=pages.rows, kscale=pages.kscale, q=Q, n=c)
        mode, splits = (1, 1) if form == "row" else ((2, 3) if c == 1 else (3, 1))
        D.kattn(Q, pages.rows, pages.kscale, pages.bt, r.slots, r.pos, chunk=(m.get("mask") or {}).get("size", 0), bias=bias, sink=True, heads=H, kv_heads=G,
                dim=d, out=O, n=c, mode=mode, splits=splits)
        outs.append(O.cpu())
    return torch.cat(outs)


def _kattn_weights(H, d, rel_rows, g):
    n = H * d
    return {"q": torch.eye(n), "k": torch.eye(n), "o": torch.eye(n), "q.norm": torch.rand(n, generator=g) + 0.5, "k.norm": torch.rand(n, generator=g) + 0.5,
            "rel": torch.randn(rel_rows, H, generator=g), "temp": torch.rand(H, generator=g) + 0.5}


@pytest.mark.parametrize("chunk,block", [(7, 16), (16, 16), (33, 4), (0, 8), (1, 16), (96, 16)])
@pytest.mark.parametrize("cut_sizes", [[500], [1], [2, 11, 1, 64]])
def test_key_attention_random_rows(dev, chunk, block, cut_sizes):
    g = torch.Generator().manual_seed(chunk + block)
    H, d, T, eps = 3, 12, 120, 1e-5
    m = {"heads": H, "kv_heads": H, "dim": d, "scale": 0.4, "bias_max": 30, "mask": {"size": chunk} if chunk else None}
    w = _kattn_weights(H, d, 10, g)
    h = torch.randn(T, H * d, generator=g)
    want = R.chunked_bias_attention({k: v.double() for k, v in w.items()}, "", m, eps, h.double())
    assert close(_kattn_run(dev, h, m, w, eps, cut_sizes, block), want, 2e-5)


@pytest.mark.parametrize("H,G,d", [(3, 3, 16), (8, 2, 48), (34, 2, 32), (2, 1, 256)])
@pytest.mark.parametrize("chunk,block", [(7, 16), (33, 4), (0, 16), (96, 16)])
@pytest.mark.parametrize("cut_sizes", [[500], [1], [2, 11, 1, 40]])
def test_key_attention_matrix_core_form(dev, H, G, d, chunk, block, cut_sizes):
    """bf16 cache and bf16-representable keys: the cache holds them exactly, what is left is the two-term split of query and weights."""
    g = torch.Generator().manual_seed(H + chunk)
    T, eps = 90, 1e-5
    m = {"heads": H, "kv_heads": G, "dim": d, "scale": 0.4, "bias_max": 30, "mask": {"size": chunk} if chunk else None}
    w = {"q": torch.randn(H * d, G * d, generator=g) * (G * d) ** -0.5, "k": torch.eye(G * d), "o": torch.eye(H * d), "q.norm": torch.rand(H * d, generator=g) + 0.5,
         "k.norm": torch.rand(G * d, generator=g) + 0.5, "rel": torch.randn(10, H, generator=g), "temp": torch.rand(H, generator=g) + 0.5}
    h = torch.randn(T, G * d, generator=g).to(torch.bfloat16).float()
    want = R.chunked_bias_attention({k: v.double() for k, v in w.items()}, "", m, eps, h.double())
    from vllm_i64_amd import ops_dense as D
    from vllm_i64_amd.dogalorn import distance_bias_table
    bias = distance_bias_table(w["rel"], 30.0).to(dev)
    # single rows: the kernel that requests its tiles ahead (1), and the general kernel with a token's heads per wave (0)
    for single_row_form in ((1, 0) if 1 in cut_sizes else (1,)):
        D.call_dense("i64h_set_latent_attn_decode_form", single_row_form)
        try:
            pages = KeyPages(dev, T, G * d, block, torch.bfloat16)
            outs = []
            for p, c in cuts_of(T, cut_sizes):
                r = Rows(dev, [(1, p, c)])
                P = torch.cat([h[p:p + c] @ w["q"].T, h[p:p + c]], 1).to(dev).contiguous()
                Q, O = torch.empty(c, H * d, device=dev), torch.empty(c, H * d, device=dev)
                D.kattn_prep(P, q_off=0, k_off=H * d, heads=H, kv_heads=G, dim=d, q_norm_w=w["q.norm"].to(dev), k_norm_w=w["k.norm"].to(dev),
                             temp=w["temp"].to(dev), scale=0.4, eps=eps, positions=r.pos, slot_ids=r.slots, block_table=pages.bt, cache=pages.rows,
                             kscale=pages.kscale, q=Q, n=c)
                mode, splits = (2, 3) if c == 1 else (3, 1)
                D.kattn(Q, pages.rows, pages.kscale, pages.bt, r.slots, r.pos, chunk=chunk, bias=bias, sink=True, heads=H, kv_heads=G, dim=d, out=O, n=c,
                        mode=mode, splits=splits)
                outs.append(O.cpu())
        finally:
            D.call_dense("i64h_set_latent_attn_decode_form", 1)
        assert close(torch.cat(outs), want, 1e-4), single_row_form


def test_key_attention_matrix_core_form_batches_of_unequal_rows(dev):
    """One launch over portions of three sequences whose borders fall inside a tile of 16 rows, and one over single rows of three
    sequences at different positions, against each sequence alone on the row kernel."""
    from vllm_i64_amd import ops_dense as D
    from vllm_i64_amd.dogalorn import distance_bias_table
    g = torch.Generator().manual_seed(11)
    H, G, d, chunk, block = 4, 2, 32, 24, 16
    lens = [37, 5, 60]
    nb = sum((T + 1 + block - 1) // block for T in lens)
    rows = torch.zeros(nb + 2, block, G * d, dtype=torch.bfloat16, device=dev)
    ksc = torch.zeros(nb + 2, block, device=dev)
    bt = torch.full((3, 8), -1, dtype=torch.int32)
    perm = torch.randperm(nb + 2, generator=g).tolist()
    for s, T in enumerate(lens):
        for b in range((T + 1 + block - 1) // block):
            bt[s, b] = perm.pop()
    bt = bt.to(dev)
    qn, kn, temp = torch.rand(H * d, generator=g) + 0.5, torch.rand(G * d, generator=g) + 0.5, torch.rand(H, generator=g) + 0.5
    bias = distance_bias_table(torch.randn(6, H, generator=g), 20.0).to(dev)
    P = {s: torch.randn(T + 1, (H + G) * d, generator=g) for s, T in enumerate(lens)}

    def run(runs, mode, splits=1):
        r = Rows(dev, runs)
        X = torch.cat([P[s][p:p + c] for s, p, c in runs]).to(dev).contiguous()
        Q, O = torch.empty(r.n, H * d, device=dev), torch.empty(r.n, H * d, device=dev)
        D.kattn_prep(X, q_off=0, k_off=H * d, heads=H, kv_heads=G, dim=d, q_norm_w=qn.to(dev), k_norm_w=kn.to(dev), temp=temp.to(dev), scale=0.3, eps=1e-6,
                     positions=r.pos, slot_ids=r.slots, block_table=bt, cache=rows, kscale=ksc, q=Q, n=r.n)
        D.kattn(Q, rows, ksc, bt, r.slots, r.pos, chunk=chunk, bias=bias, sink=True, heads=H, kv_heads=G, dim=d, out=O, n=r.n, mode=mode, splits=splits)
        return O.cpu()

    together = run([(s, 0, T) for s, T in enumerate(lens)], 3)
    alone = torch.cat([run([(s, 0, T)], 1) for s, T in enumerate(lens)])
    assert close(together, alone, 1e-4)
    together = run([(s, T, 1) for s, T in enumerate(lens)], 2, splits=2)
    alone = torch.cat([run([(s, T, 1)], 1) for s, T in enumerate(lens)])
    assert close(together, alone, 1e-4)


@pytest.mark.parametrize("mode", ["prompt", "decode"])
@pytest.mark.parametrize("chunk,block,T", [(48, 16, 200), (50, 16, 230), (0, 16, 300), (129, 8, 400)])
def test_key_attention_one_key_stands_out(dev, mode, chunk, block, T):
    """The query row and ONE other row are the same direction (that row three times as long: same normed key, three times the
    value): where the chunk lets the query see it, the output doubles - placed at the far end of the chunk, at page borders, at the
    chunk's first position (just inside) and the position before it (just outside)."""
    g = torch.Generator().manual_seed(T)
    H, d, eps = 2, 16, 1e-6
    m = {"heads": H, "kv_heads": H, "dim": d, "scale": 1.5, "bias_max": 64, "mask": {"size": chunk} if chunk else None}
    w = _kattn_weights(H, d, 6, g)
    w["q.norm"].fill_(1.0), w["k.norm"].fill_(1.0), w["temp"].fill_(1.0), w["rel"].mul_(0.05)
    wd = {k: v.double() for k, v in w.items()}
    i = T - 1
    lo = (i // chunk) * chunk if chunk else 0
    for j in sorted({lo, lo - 1, lo + 1, (lo // block) * block + block, (lo // block) * block + block - 1, i - 1, 0} - {i}):
        if j < 0 or j >= i:
            continue
        h = torch.randn(T, H * d, generator=g).double()
        for b in range(H):       # every other row is orthogonal to the query's, head by head: their scores are the bias alone
            v = h[i, b * d:(b + 1) * d].clone()
            blk = h[:, b * d:(b + 1) * d]
            blk -= (blk @ v)[:, None] / (v @ v) * v
            blk[i] = v
        h = h.float()
        h[j] = 3.0 * h[i]
        want = R.chunked_bias_attention(wd, "", m, eps, h.double())
        seen = j >= lo
        ratio = float(want[i].norm() / h[i].double().norm())
        assert (ratio > 1.8) == seen, (j, lo, ratio)       # the oracle itself shows the difference between seen and unseen
        got = _kattn_run(dev, h, m, w, eps, [T] if mode == "prompt" else [T - 1, 1], block)
        assert close(got[i], want[i], 2e-5), (j, lo)
        hb = h.to(torch.bfloat16).float()
        got = _kattn_run(dev, hb, m, w, eps, [T] if mode == "prompt" else [T - 1, 1], block, dtype=torch.bfloat16, form="mfma")
        assert close(got[i], R.chunked_bias_attention(wd, "", m, eps, hb.double())[i], 2e-4), (j, lo, "matrix cores")


def test_key_attention_sink_and_grouped_heads(dev):
    """Two query heads per key head; all scores far below zero: the sink takes nearly all the weight and the output shrinks."""
    g = torch.Generator().manual_seed(5)
    H, G, d, T, eps = 4, 2, 6, 40, 1e-6
    m = {"heads": H, "kv_heads": G, "dim": d, "scale": 0.5, "bias_max": 16, "mask": {"size": 16}}
    w = {"q": torch.randn(H * d, G * d, generator=g), "k": torch.eye(G * d), "o": torch.eye(H * d), "q.norm": torch.rand(H * d, generator=g) + 0.5,
         "k.norm": torch.rand(G * d, generator=g) + 0.5, "rel": torch.randn(4, H, generator=g) - 12.0, "temp": torch.rand(H, generator=g) + 0.5}
    h = torch.randn(T, G * d, generator=g)
    want = R.chunked_bias_attention({k: v.double() for k, v in w.items()}, "", m, eps, h.double())
    assert float(want.abs().max()) < 5e-2
    from vllm_i64_amd import ops_dense as D
    from vllm_i64_amd.dogalorn import distance_bias_table
    pages = KeyPages(dev, T, G * d, 16, torch.float32)
    r = Rows(dev, [(1, 0, T)])
    P = torch.cat([h @ w["q"].T, h], 1).to(dev).contiguous()
    Q, O = torch.empty(T, H * d, device=dev), torch.empty(T, H * d, device=dev)
    D.kattn_prep(P, q_off=0, k_off=H * d, heads=H, kv_heads=G, dim=d, q_norm_w=w["q.norm"].to(dev), k_norm_w=w["k.norm"].to(dev), temp=w["temp"].to(dev),
                 scale=0.5, eps=eps, positions=r.pos, slot_ids=r.slots, block_table=pages.bt, cache=pages.rows, kscale=pages.kscale, q=Q, n=T)
    D.kattn(Q, pages.rows, pages.kscale, pages.bt, r.slots, r.pos, chunk=16, bias=distance_bias_table(w["rel"], 16.0).to(dev), sink=True, heads=H, kv_heads=G,
            dim=d, out=O, n=T)
    assert close(O, want, 2e-5)


# ===================================================== whole models ===============================================================
@pytest.mark.parametrize("name", list(SHAPES))
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_prompt_and_layer_streams(dev, name, dtype):
    model = make_model(name, dtype, dev)
    toks = tokens(name, 140, 1)
    layers = []
    want = oracle_logits(name, toks, layers=layers)
    model.kv.reserve(2, len(toks))
    rec = {}
    got = model.forward(torch.tensor(toks, dtype=torch.int64, device=dev), torch.arange(len(toks), dtype=torch.int32, device=dev),
                        torch.full((len(toks),), 2, dtype=torch.int32, device=dev), record=rec, tokens_per_seq=[len(toks)])
    for i, x in enumerate(layers):
        assert rel_err(rec[f"l{i}.x"], x) < TOL[dtype], f"stream after layer {i}"
    assert rel_err(got, want) < TOL[dtype]


@pytest.mark.parametrize("name", list(SHAPES))
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_cuts_batches_and_reuse(dev, name, dtype):
    """Token by token from the first token; portions of changing size down to two tokens; four live requests of unequal length in a
    pool that only fits with page reuse, more requests than slots over the run; a request left out of steps."""
    from vllm_i64_amd.engine import Engine
    model = make_model(name, dtype, dev, max_tokens=4 * 64, max_seqs=4)
    reqs = {"a": tokens(name, 61, 2), "b": tokens(name, 38, 3), "c": tokens(name, 1, 4), "d": tokens(name, 50, 5), "e": tokens(name, 33, 6), "f": tokens(name, 64, 7)}
    want = {i: oracle_logits(name, t) for i, t in reqs.items()}
    eng = Engine(model)
    got = replay(eng, {"b": reqs["b"]}, [[("b", 1)] for _ in range(38)])
    assert rel_err(got["b"], want["b"]) < TOL[dtype]
    got = replay(eng, {"a": reqs["a"]}, [[("a", c)] for _, c in cuts_of(61, [2, 17, 1, 3, 16, 2, 5])])
    assert rel_err(got["a"], want["a"]) < TOL[dtype]
    sched = [[("a", 30), ("b", 2)], [("a", 1), ("b", 20), ("c", 1), ("d", 7)], [("b", 1), ("d", 2), ("e", 16)], [("a", 28), ("b", 1), ("d", 1), ("e", 1)],
             [("a", 2), ("b", 14), ("d", 40), ("e", 2)], [("e", 14), ("f", 33)], [("f", 1)], [("f", 30)]]
    got = replay(eng, reqs, sched)
    for i in reqs:
        assert rel_err(got[i], want[i]) < TOL[dtype], i
    assert model.kv.free_blocks == model.kv.num_blocks and not eng.seqs


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_past_chunks_and_pages(dev, dtype):
    from vllm_i64_amd.engine import Engine
    name = "odd"
    toks = tokens(name, 150, 8)
    want = oracle_logits(name, toks)
    eng = Engine(make_model(name, dtype, dev, max_tokens=160, max_seqs=1))
    got = replay(eng, {"x": toks}, [[("x", 9)]] + [[("x", 1)] for _ in range(141)])
    assert rel_err(got["x"], want) < TOL[dtype]


@pytest.mark.parametrize("name", ["odd", "plain"])
def test_greedy_generation_through_the_engine(dev, name):
    """More prompts than slots; the engine's own scheduler, batching and sampling; against the oracle's greedy continuation."""
    from vllm_i64_amd.engine import Engine, SamplingParams
    model = make_model(name, "float32", dev, max_tokens=3 * 64, max_seqs=2)
    prompts = [tokens(name, n, 20 + n) for n in (5, 19, 1, 12)]
    new = 6
    want = []
    for p in prompts:
        t = list(p)
        for _ in range(new):
            t.append(int(oracle_logits(name, t)[-1].argmax()))
        want.append(t[len(p):])
    eng = Engine(model, max_batch_tokens=16)
    assert eng.generate(prompts, SamplingParams(max_new_tokens=new)) == want


def test_graph_decoder_steps_match_the_oracle(dev):
    """The batch decoder (a captured HIP graph replayed per step) from the first token on: the recurrent state, the previous token and
    the key pages advance inside the graph."""
    from vllm_i64_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("the batch decoder takes its argmax from the first library, which is not built")
    from vllm_i64_amd.model import GreedyDecoder
    name = "odd"
    model = make_model(name, "float32", dev, max_tokens=256, max_seqs=3)
    prompts = [tokens(name, n, 40 + n) for n in (4, 11, 7)]
    dec = GreedyDecoder(model, 3, use_graph=True)
    dec.prefill([torch.tensor(p) for p in prompts], reserve_extra=8)
    seqs = [list(p) + [int(t)] for p, t in zip(prompts, dec.tokens.tolist())]
    for _ in range(5):
        dec.step()
        torch.cuda.synchronize()
        for s, t in zip(seqs, dec.tokens.tolist()):
            s.append(int(t))
    for p, s in zip(prompts, seqs):
        t = list(p)
        for _ in range(6):
            t.append(int(oracle_logits(name, t)[-1].argmax()))
        assert s == t


def test_trace_command_on_a_checkpoint_folder(dev, tmp_path):
    from safetensors.torch import save_file
    name = "plain"
    ck = tmp_path / "ck"
    ck.mkdir()
    (ck / "config.json").write_text(json.dumps(config_of(name)))
    save_file(make_weights(name), str(ck / "model.safetensors"))
    toks = tokens(name, 21, 9)
    steps = [{"step": 0, "entries": [{"id": "q", "tokens": toks[:10], "want": [0, 9]}], "end": []},
             {"step": 1, "entries": [{"id": "q", "tokens": toks[10:12], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "q", "tokens": toks[12:], "want": [8]}, {"id": "r", "tokens": toks[:3], "want": [2]}], "end": ["q", "r"]}]
    out = tmp_path / "out"
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", str(ck), "--dtype", "float32", "--out", str(out), "--max-tokens", "128"],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    import numpy as np
    want = oracle_logits(name, toks)
    V = SHAPES[name]["vocab"]
    a = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4").reshape(-1, V))
    c = torch.from_numpy(np.fromfile(out / "2.f32", dtype="<f4").reshape(-1, V))
    assert not (out / "1.f32").exists()
    assert rel_err(a, want[[0, 9]]) < TOL["float32"] and rel_err(c, torch.stack([want[20], want[2]])) < TOL["float32"]
