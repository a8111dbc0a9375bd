"""The Morilorn design on the GPU against the CPU oracle (oracle/morilorn_ref.py): every mechanism alone, then whole models of
several small shapes under every way of cutting, batching and paging their sequences, through the engine and the command line."""
import json
import math
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from oracle import morilorn_ref as R

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
# rms over the vocabulary of the logit difference / rms of the logits.  bfloat16: the inputs of every matrix product are rounded to 8
# bits of mantissa (2^-9 relative each); with rows of only 48 to 128 values little of that averages out over a product, and it
# passes through two or three layers - a few percent at the worst position of a sequence, where a wrong mechanism gives 50 % and more
TOL = {"float32": 3e-5, "bfloat16": 6e-2}


@pytest.fixture(scope="module")
def dev():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


def bf16(t):
    return t.to(torch.bfloat16)


def rel_err(got, want):
    got, want = torch.as_tensor(got, dtype=torch.float64), torch.as_tensor(want, dtype=torch.float64)
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    return float((d.pow(2).mean(-1).sqrt() / want.pow(2).mean(-1).sqrt().clamp_min(1e-9)).max())


def make_model(cfg, w, dtype, dev, max_tokens=512, max_seqs=4):
    from vllm_i64_amd.config import MorilornConfig
    from vllm_i64_amd.morilorn import MorilornModel
    return MorilornModel(MorilornConfig.from_dict(cfg), w, device=dev, dtype=dtype, max_seqs=max_seqs, num_kv_blocks=(max_tokens + 15) // 16)


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


def tokens(cfg, n, seed):
    return torch.randint(0, cfg["vocab"], (n,), generator=torch.Generator().manual_seed(seed)).tolist()


# a shape with nothing equal and nothing a power of two; one with single head / single group / no window and wide vectors; one whose
# layers differ from each other (sizes, windows, a layer without feed-forward, a part of the rotated dimensions left unrotated)
SHAPES = {
    "odd": dict(vocab=97, width=48, layers=2, heads=3, dim=10, rot_dim=6, vdim=14, kv_rank=20, window=7, ff=44, groups=3),
    "wide": dict(vocab=160, width=128, layers=2, heads=1, dim=32, rot_dim=16, vdim=32, kv_rank=80, window=0, ff=96, groups=1, alpha=1.0, embed_scale=1.0, softcap=0.0),
    "mixed_layers": dict(vocab=120, width=64, layers=3, groups=2, per_layer=[
        dict(heads=2, dim=16, rot_dim=8, vdim=16, kv_rank=32, window=5, ff=80),
        dict(heads=5, dim=4, rot_dim=12, vdim=6, kv_rank=24, window=33, ff=None, rot_dims=8, scale=0.2),
        dict(heads=4, dim=8, rot_dim=8, vdim=8, kv_rank=144, window=1, ff=24, rot_base=77.0)]),
}


# ---- mechanisms alone ------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("exact", [False, True])
@pytest.mark.parametrize("M,N,K", [(1, 5, 3), (7, 33, 20), (8, 72, 64), (70, 65, 100), (130, 200, 64), (3, 130, 256), (64, 40, 168), (33, 16, 1024)])
def test_linear_plain_and_epilogues(dev, exact, M, N, K):
    from vllm_i64_amd import ops_dense as D
    g = torch.Generator().manual_seed(M * 1000 + N + K)
    a = torch.randn(M, K + 5, generator=g)
    w = bf16(torch.randn(2 * N, K, generator=g) / math.sqrt(K))
    e = torch.randn(M, N + 3, generator=g)
    ad, wd, ed = a.to(dev), w.to(dev), e.to(dev)
    A = a[:, 2:2 + K].double() if exact else bf16(a[:, 2:2 + K]).double()
    tol = 1e-5 if exact else 2e-5   # both forms sum exact products in fp32
    for skinny in (7, 1, 0):     # every kernel where it applies; rows <= 8 on their own kernel only; everything on the 64 x 64 tile kernel
        D.call_dense("i64h_set_linear_skinny", skinny)
        out = torch.full((M, N + 4), 7.0, device=dev)
        D.linear(ad, wd, out, n=N, k=K, a_off=2, lda=K + 5, c_off=1, ldc=N + 4, exact=exact)
        ref = A @ w[:N].double().T
        assert torch.allclose(out[:, 1:1 + N].cpu().double(), ref, atol=tol * K ** 0.5, rtol=tol)
        assert bool((out[:, 0] == 7).all()) and bool((out[:, N + 1:] == 7).all())
        out2 = torch.empty(M, N, device=dev)
        D.linear(ad, wd, out2, n=N, k=K, a_off=2, lda=K + 5, exact=exact, epilogue=D.EPI_GELU_MUL)
        ref2 = R.gelu_tanh(ref) * (A @ w[N:].double().T)
        assert torch.allclose(out2.cpu().double(), ref2, atol=1e-4, rtol=1e-4)
        D.linear(ad, wd, out2, n=N, k=K, a_off=2, lda=K + 5, exact=exact, epilogue=D.EPI_MUL_SIGMOID, e=ed, e_off=3, lde=N + 3)
        assert torch.allclose(out2.cpu().double(), ref * torch.sigmoid(e[:, 3:].double()), atol=1e-4, rtol=1e-4)
        D.linear(ad, wd, out2, n=N, k=K, a_off=2, lda=K + 5, exact=exact, epilogue=D.EPI_SOFTCAP, softcap=0.7)
        assert torch.allclose(out2.cpu().double(), 0.7 * torch.tanh(ref / 0.7), atol=1e-4, rtol=1e-4)
    D.call_dense("i64h_set_linear_skinny", 3)


@pytest.mark.parametrize("exact", [False, True])
@pytest.mark.parametrize("M,heads,n,k", [(5, 3, 20, 10), (40, 2, 24, 16), (2, 4, 8, 136)])
def test_linear_batched_over_heads_and_gathered_rows(dev, exact, M, heads, n, k):
    """Per-head weights on column blocks of wider matrices (how the query enters and the values leave latent space), and a_rows."""
    from vllm_i64_amd import ops_dense as D
    g = torch.Generator().manual_seed(11)
    a = torch.randn(M, 3 + heads * (k + 2), generator=g)
    w = bf16(torch.randn(heads, n, k, generator=g))
    out = torch.zeros(M, heads * (n + 1), device=dev)
    D.linear(a.to(dev), w.to(dev), out, m=M, n=n, k=k, a_off=3, lda=a.shape[1], ldc=out.shape[1], batch=heads, a_batch=k + 2, w_batch=n * k, c_batch=n + 1, exact=exact)
    for h in range(heads):
        A = a[:, 3 + h * (k + 2): 3 + h * (k + 2) + k]
        A = A.double() if exact else bf16(A).double()
        assert torch.allclose(out[:, h * (n + 1): h * (n + 1) + n].cpu().double(), A @ w[h].double().T, atol=1e-4, rtol=1e-4)
    rows = torch.tensor([M - 1, 0, M - 1], dtype=torch.int32)
    out = torch.empty(3, n, device=dev)
    D.linear(a.to(dev), w[0].contiguous().to(dev), out, n=n, k=k, lda=a.shape[1], a_rows=rows.to(dev), exact=exact)
    A = a[rows.long(), :k]
    assert torch.allclose(out.cpu().double(), (A.double() if exact else bf16(A).double()) @ w[0].double().T, atol=1e-4, rtol=1e-4)


@pytest.mark.parametrize("W,groups", [(48, 3), (64, 1), (250, 5), (4096, 2)])
def test_gated_postnorm_and_depth_mix(dev, W, groups):
    from vllm_i64_amd import ops_dense as D
    g = torch.Generator().manual_seed(W)
    n, idx = 5, 3
    x, y, gp = torch.randn(n, W, generator=g), torch.randn(n, W + 2, generator=g), torch.randn(n, W + 7, generator=g)
    b, nw = torch.randn(W, generator=g), torch.randn(W, generator=g)
    hist = torch.randn(idx + 2, n, W, generator=g)
    mw = torch.randn(idx + 1, generator=g)
    hd = hist.to(dev)
    out, mix = torch.empty(n, W, device=dev), torch.empty(n, W, device=dev)
    D.gated_postnorm(x.to(dev), nw.to(dev), groups, 1e-3, alpha=1.75, y=y.to(dev), ldy=W + 2, gate_pre=gp.to(dev), gate_off=4, ldg=W + 7, gate_bias=b.to(dev),
                     out=out, hist=hd, hist_index=idx, mix_w=mw.to(dev), mix_out=mix)
    v = 1.75 * x.double() + torch.sigmoid(gp[:, 4:4 + W].double() + b.double()) * y[:, :W].double()
    ref = R.rms_norm(v, nw.double(), 1e-3, groups)
    assert torch.allclose(out.cpu().double(), ref, atol=2e-6, rtol=2e-6)
    assert torch.allclose(hd[idx].cpu().double(), ref, atol=2e-6, rtol=2e-6) and torch.equal(hd[idx + 1].cpu(), hist[idx + 1])
    want = sum(mw[j].double() * hist[j].double() for j in range(idx)) + mw[idx].double() * ref
    assert torch.allclose(mix.cpu().double(), want, atol=1e-5, rtol=1e-5)
    # plain norm of gathered rows (the final norm): no sublayer, no gate
    rows = torch.tensor([4, 1], dtype=torch.int32)
    out2 = torch.empty(2, W, device=dev)
    D.gated_postnorm(x.to(dev), nw.to(dev), groups, 1e-3, x_rows=rows.to(dev), out=out2)
    assert torch.allclose(out2.cpu().double(), R.rms_norm(x[rows.long()].double(), nw.double(), 1e-3, groups), atol=2e-6, rtol=2e-6)


@pytest.mark.parametrize("epilogue", [0, 1, 2, 3])
def test_linear_large_tiles(dev, epilogue):
    """A launch with enough 128 x 128 tiles for the large-tile kernel, edges in M, N and K, against the 64 x 64 kernel's result."""
    from vllm_i64_amd import ops_dense as D
    g = torch.Generator().manual_seed(epilogue)
    M, N, K = 2000, 2100, 104
    a = torch.randn(M, K, generator=g).to(dev)
    w = bf16(torch.randn(2 * N, K, generator=g) / math.sqrt(K)).to(dev)
    e = torch.randn(M, N, generator=g).to(dev)
    outs = []
    for knob in (7, 0):
        D.call_dense("i64h_set_linear_skinny", knob)
        out = torch.empty(M, N, device=dev)
        D.linear(a, w, out, n=N, k=K, epilogue=epilogue, e=e if epilogue == 2 else None, lde=N, softcap=1.3 if epilogue == 3 else 0.0)
        outs.append(out.cpu())
    D.call_dense("i64h_set_linear_skinny", 3)
    assert torch.equal(outs[0], outs[1])       # the same products summed in the same order
    ref = bf16(a.cpu()).double() @ w.cpu()[:N].double().T
    if epilogue == 1:
        ref = R.gelu_tanh(ref) * (bf16(a.cpu()).double() @ w.cpu()[N:].double().T)
    elif epilogue == 2:
        ref = ref * torch.sigmoid(e.cpu().double())
    elif epilogue == 3:
        ref = 1.3 * torch.tanh(ref / 1.3)
    assert torch.allclose(outs[0].double(), ref, atol=1e-4, rtol=1e-4)


def test_embed_scaled(dev):
    from vllm_i64_amd import ops_dense as D
    table = bf16(torch.randn(50, 37, generator=torch.Generator().manual_seed(1)))
    ids = torch.tensor([0, 49, 7, 7, 13])
    out = torch.empty(5, 37, device=dev)
    D.embed_scaled(ids.to(dev), table.to(dev), 12.5, out)
    assert torch.equal(out.cpu(), table[ids].float() * 12.5)


def _paged(dev, T, D_, dtype, seed=0, block=16, spare=3):
    """A cache of one sequence in slot 1 whose pages are scattered, plus a decoy slot 0."""
    nb = (T + block - 1) // block
    perm = torch.randperm(nb + spare, generator=torch.Generator().manual_seed(seed))[:nb].to(torch.int32)
    bt = torch.full((2, nb + 1), -1, dtype=torch.int32)
    bt[1, :nb] = perm
    cache = torch.zeros(nb + spare, block, D_, dtype=dtype, device=dev)
    return cache, bt, perm


def _cache_rows(cache, perm, T, block=16):
    return torch.cat([cache[int(b)] for b in perm]).cpu().double()[:T]


@pytest.mark.parametrize("cache_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,d,e,r,rdims", [(3, 10, 6, 20, 6), (2, 16, 8, 32, 4), (1, 5, 0, 9, 0), (4, 8, 32, 128, 32)])
def test_latent_prep_norm_rotation_and_cache_write(dev, cache_dtype, H, d, e, r, rdims):
    from vllm_i64_amd import ops_dense as D
    from vllm_i64_amd.morilorn import inverse_frequencies
    g = torch.Generator().manual_seed(5)
    T, base, eps = 37, 30000.0, 1e-4
    q_off, dkv_off = 3, 3 + H * (d + e) + 2
    P = torch.randn(T, dkv_off + r + e + 1, generator=g)
    nw = torch.randn(r, generator=g)
    pos = torch.arange(100, 100 + T, dtype=torch.int32)       # positions 100.. : crosses several pages, angles are not small
    cache, bt, perm = _paged(dev, 100 + T, r + e, cache_dtype)
    Q = torch.zeros(T, H, r + e, device=dev)
    D.latent_prep(P.to(dev), q_off=q_off, dkv_off=dkv_off, heads=H, dim=d, rot_dim=e, kv_rank=r, rot_dims=rdims, c_norm_w=nw.to(dev), eps=eps,
                  inv_freq=inverse_frequencies(base, rdims).to(dev) if rdims else None, positions=pos.to(dev), slot_ids=torch.ones(T, dtype=torch.int32, device=dev),
                  block_table=bt.to(dev), block_size=16, cache=cache, q=Q)
    rows = _cache_rows(cache, perm, 100 + T)[100:]
    lat = R.rms_norm(P[:, dkv_off:dkv_off + r].double(), nw.double(), eps)
    tol = 1e-5 if cache_dtype == torch.float32 else 1e-2
    assert torch.allclose(rows[:, :r], lat, atol=tol, rtol=tol)
    if e:
        k = P[:, dkv_off + r: dkv_off + r + e].double()
        assert torch.allclose(rows[:, r:], R.rotate_pairs(k, pos, base, rdims) if rdims else k, atol=tol * 4, rtol=tol)
        q = P[:, q_off: q_off + H * (d + e)].double().reshape(T, H, d + e)[..., d:]
        assert torch.allclose(Q[..., r:].cpu().double(), R.rotate_pairs(q, pos, base, rdims) if rdims else q, atol=4e-5, rtol=1e-5)
    assert bool((Q[..., :r] == 0).all())     # the latent-space part of the query is the caller's Linear's


def _ref_attn(Q, rows, positions, window, scale, r):
    out = torch.zeros(Q.shape[0], Q.shape[1], r, dtype=torch.float64)
    for i, p in enumerate(positions):
        lo = max(0, p - window + 1) if window > 0 else 0
        keys = rows[lo:p + 1]
        for h in range(Q.shape[1]):
            wgt = torch.softmax(scale * (keys @ Q[i, h].double()), dim=0)
            out[i, h] = wgt @ keys[:, :r]
    return out


@pytest.mark.parametrize("cache_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window", [0, 1, 7, 16, 17, 45])
@pytest.mark.parametrize("r,e", [(32, 8), (20, 6)])   # widths the matrix-core form takes (multiples of 16 and 8), and widths it leaves to the row form
def test_latent_attn_one_key_stands_out(dev, cache_dtype, window, r, e):
    """One cached row is made to dominate every head's softmax wherever it is visible.  It is placed far back, at page borders and
    just inside / just outside the window of rows in the middle of a run of rows (a prompt's portion) and of single rows (decode):
    one position off in the window or in the page arithmetic changes the result by the whole row."""
    from vllm_i64_amd import ops_dense as D
    H, T = 3, 150
    g = torch.Generator().manual_seed(window)
    u = torch.randn(r + e, generator=g)
    u = bf16(u / u.norm()).float()
    for star in sorted({0, 15, 16, 17, 63, 64, 100, 149}):
        rows = bf16(torch.randn(T, r + e, generator=g) * 0.5).float()
        rows -= (rows @ u)[:, None] * u[None, :] / (u @ u)      # no other row has a component along u ...
        rows[star] += 6.0 * u                                    # ... this one has a large one
        rows = bf16(rows).float()
        cache, bt, perm = _paged(dev, T, r + e, cache_dtype, seed=star)
        for b_i, b in enumerate(perm):
            part = rows[b_i * 16:(b_i + 1) * 16]
            cache[int(b), :part.shape[0]] = part.to(dev).to(cache_dtype)
        cand = {star, T - 1}
        if window:
            cand |= {star + window - 1, star + window}            # the last row that sees it, the first that does not
        positions = sorted(p for p in cand if star <= p < T)
        for pos_list in (positions, *[[p] for p in positions]):   # rows of one launch, then each alone
            n = len(pos_list)
            Q = torch.randn(n, H, r + e, generator=g) * 0.3 + 4.0 * u
            ref = _ref_attn(Q, rows.double(), pos_list, window, 0.9, r)
            for mode in (1, 2, 3):    # one wave per (row, head) in fp32; the matrix-core forms (bf16 caches of fitting widths)
                out = torch.empty(n, H, r, device=dev)
                D.latent_attn(Q.to(dev), cache, bt.to(dev), torch.ones(n, dtype=torch.int32, device=dev), torch.tensor(pos_list, dtype=torch.int32, device=dev),
                              window=window, scale=0.9, heads=H, kv_rank=r, rot_dim=e, out=out, mode=mode)
                tol = 2e-4 if mode == 1 else 1e-3     # there the query and the weights are carried with 16 bits of mantissa
                assert torch.allclose(out.cpu().double(), ref, atol=tol, rtol=tol), (window, star, pos_list, mode)
            for i, p in enumerate(pos_list):    # the construction works: the row dominates exactly where it is visible
                sees = p - star < window if window else True
                close = torch.allclose(ref[i, 0], rows[star, :r].double(), atol=0.2)
                assert close == sees, (window, star, p)


@pytest.mark.parametrize("H,r,e", [(5, 48, 16), (16, 256, 32), (18, 240, 80)])    # the last two: the widest rows the matrix-core forms take
def test_latent_attn_keys_dealt_to_several_waves(dev, H, r, e):
    """Decode rows whose keys are split over waves and merged: same result as one wave per token, also when some shares are empty;
    and the same rows through the form made for prompt portions."""
    from vllm_i64_amd import ops_dense as D
    g = torch.Generator().manual_seed(2)
    lens = [1, 40, 333, 64]
    nb = [(t + 15) // 16 for t in lens]
    bt = torch.full((4, max(nb)), -1, dtype=torch.int32)
    perm = torch.randperm(sum(nb), generator=g).to(torch.int32)
    rows_of, at = [], 0
    cache = torch.zeros(sum(nb), 16, r + e, dtype=torch.bfloat16, device=dev)
    for s_, t in enumerate(lens):
        bt[s_, :nb[s_]] = perm[at:at + nb[s_]]
        rows = bf16(torch.randn(t, r + e, generator=g) * 0.7).float()
        for b_i in range(nb[s_]):
            part = rows[b_i * 16:(b_i + 1) * 16]
            cache[int(perm[at + b_i]), :part.shape[0]] = part.to(dev).to(torch.bfloat16)
        rows_of.append(rows.double())
        at += nb[s_]
    Q = torch.randn(4, H, r + e, generator=g)
    pos = torch.tensor([t - 1 for t in lens], dtype=torch.int32)
    for window in (0, 100):
        ref = torch.cat([_ref_attn(Q[i:i + 1], rows_of[i], [lens[i] - 1], window, 0.4, r) for i in range(4)])
        for form in (1, 0):      # the kernel that requests its fragments a tile ahead, and the general matrix-core kernel
            D.call_dense("i64h_set_latent_attn_decode_form", form)
            for splits in (1, 2, 5, 64):
                out = torch.empty(4, H, r, device=dev)
                D.latent_attn(Q.to(dev), cache, bt.to(dev), torch.arange(4, dtype=torch.int32, device=dev), pos.to(dev), window=window, scale=0.4, heads=H,
                              kv_rank=r, rot_dim=e, out=out, mode=2, splits=splits)
                assert torch.allclose(out.cpu().double(), ref, atol=1e-3, rtol=1e-3), (window, splits, form)
        out = torch.empty(4, H, r, device=dev)
        D.latent_attn(Q.to(dev), cache, bt.to(dev), torch.arange(4, dtype=torch.int32, device=dev), pos.to(dev), window=window, scale=0.4, heads=H,
                      kv_rank=r, rot_dim=e, out=out, mode=3)
        assert torch.allclose(out.cpu().double(), ref, atol=1e-3, rtol=1e-3), (window, "row tiles")
    D.call_dense("i64h_set_latent_attn_decode_form", 1)


def test_sample_rows(dev):
    from vllm_i64_amd import ops_dense as D
    g = torch.Generator().manual_seed(3)
    x = torch.randn(6, 301, generator=g)
    x[0, 7] = x[0, 200] = 9.0         # a tie: the first index wins
    xd = x.to(dev)
    assert D.sample_rows(xd).tolist() == [7] + x[1:].argmax(-1).tolist()
    f = lambda v, dt: torch.tensor(v, dtype=dt, device=dev)
    one = D.sample_rows(xd, temperature=f([1.0] * 6, torch.float32), top_k=f([1] * 6, torch.int32), top_p=f([1.0] * 6, torch.float32), u=f([0.9] * 6, torch.float32))
    assert one.tolist()[1:] == x[1:].argmax(-1).tolist() and one.tolist()[0] in (7, 200)
    tiny = D.sample_rows(xd, temperature=f([0.5] * 6, torch.float32), top_k=f([0] * 6, torch.int32), top_p=f([1e-6] * 6, torch.float32), u=f([0.3] * 6, torch.float32))
    assert tiny.tolist()[1:] == x[1:].argmax(-1).tolist()
    # the draw follows the distribution: u sweeps the cumulative sums of softmax(x / T) over the 5 largest, in index order
    T, k = 0.7, 5
    row = x[1].double()
    keep = torch.zeros(301, dtype=torch.bool)
    keep[row.topk(k).indices] = True
    p = torch.where(keep, torch.exp((row - row.max()) / T), torch.zeros((), dtype=torch.float64))
    cum = torch.cumsum(p / p.sum(), 0)
    us = [0.01, 0.2, 0.4, 0.6, 0.8, 0.99]
    xs = x[1:2].repeat(6, 1).contiguous().to(dev)
    got = D.sample_rows(xs, temperature=f([T] * 6, torch.float32), top_k=f([k] * 6, torch.int32), top_p=f([1.0] * 6, torch.float32), u=f(us, torch.float32)).tolist()
    for uu, tok in zip(us, got):
        want = int((cum > uu).nonzero()[0])
        assert keep[tok] and (tok == want or abs(float(cum[tok]) - uu) < 1e-4 or abs(float(cum[want]) - uu) < 1e-4)
    # top-p: the smallest set of most likely tokens that reaches p
    ps = torch.softmax(row / T, 0)
    order = ps.argsort(descending=True)
    m = int((torch.cumsum(ps[order], 0) < 0.5).sum()) + 1
    allowed = set(order[:m].tolist())
    got = D.sample_rows(xs, temperature=f([T] * 6, torch.float32), top_k=f([0] * 6, torch.int32), top_p=f([0.5] * 6, torch.float32), u=f(us, torch.float32)).tolist()
    assert set(got) <= allowed and len(set(got)) > 1


# ---- whole models ------------------------------------------------------------------------------------------------------------------
@pytest.fixture(scope="module", params=sorted(SHAPES))
def shape(request):
    cfg = R.make_config(**SHAPES[request.param])
    w = R.make_weights(cfg, seed=len(request.param))
    reqs = {"a": tokens(cfg, 75, 1), "b": tokens(cfg, 41, 2), "c": tokens(cfg, 1, 3), "d": tokens(cfg, 18, 4), "e": tokens(cfg, 50, 5)}
    want = {i: R.forward(cfg, w, t) for i, t in reqs.items()}
    return cfg, w, reqs, want


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_prompts_and_layer_streams(dev, shape, dtype):
    from vllm_i64_amd.engine import Engine
    cfg, w, reqs, want = shape
    m = make_model(cfg, w, dtype, dev)
    eng = Engine(m)
    got = replay(eng, reqs, [[(i, len(t))] for i, t in reqs.items()])
    for i in reqs:
        assert rel_err(got[i], want[i]) < TOL[dtype], i
    # the stream after every layer, in 32 bits
    if dtype == "float32":
        t = reqs["b"]
        streams, rec = [], {}
        R.forward(cfg, w, t, streams)
        m.kv.reserve(2, len(t))
        m.forward(torch.tensor(t, device=dev), torch.arange(len(t), dtype=torch.int32, device=dev), torch.full((len(t),), 2, dtype=torch.int32, device=dev), record=rec)
        m.kv.free(2)
        for l, s in enumerate(streams):
            assert torch.allclose(rec[f"l{l}.out"].cpu().double(), s, atol=2e-4, rtol=2e-4), l


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_token_by_token_and_portions(dev, shape, dtype):
    """Prefill against token-by-token decoding from the first token on, and portions of 2, 3, 5, 16, 17 ... tokens: cuts fall inside
    pages and windows, and every position is asked for."""
    from vllm_i64_amd.engine import Engine
    cfg, w, reqs, want = shape
    eng = Engine(make_model(cfg, w, dtype, dev))
    t = reqs["a"]
    got = replay(eng, {"a": t}, [[("a", 1)] for _ in t])
    assert rel_err(got["a"], want["a"]) < TOL[dtype]
    for sizes in ([2] * 37 + [1], [3, 5, 16, 17, 2, 30, 2], [40] + [1] * 35, [16, 16, 16, 16, 11]):
        assert sum(sizes) == len(t)
        got = replay(eng, {"a": t}, [[("a", k)] for k in sizes])
        assert rel_err(got["a"], want["a"]) < TOL[dtype], sizes
    assert not eng.seqs and eng.kv.free_blocks == eng.kv.num_blocks


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_mixed_batches_reuse_slots_and_pages(dev, shape, dtype):
    """Up to four live requests, portions beside single tokens, in a pool that only fits if ended requests' pages are used again;
    'e' starts in the slot and pages 'b' and 'c' gave back.  Each request must come out as if it had run alone."""
    from vllm_i64_amd.engine import Engine
    cfg, w, reqs, want = shape
    eng = Engine(make_model(cfg, w, dtype, dev, max_tokens=80 + 48 + 16 + 32, max_seqs=4))
    sched = [[("c", 1), ("a", 2), ("b", 17)],
             [("a", 30), ("b", 1), ("d", 3)],
             [("b", 1), ("d", 2), ("a", 1)],
             [("b", 22), ("a", 1)],                       # b (41) ends -> its three pages return
             [("e", 33), ("a", 1), ("d", 1)],              # e is admitted into freed slot and pages
             [("e", 1), ("d", 12), ("a", 16)],             # d (18) ends
             [("a", 24), ("e", 2)],                        # a (75) ends
             [("e", 14)]]
    got = replay(eng, reqs, sched)
    for i in reqs:
        assert got[i].shape[0] == len(reqs[i])
        assert rel_err(got[i], want[i]) < TOL[dtype], i
    assert not eng.seqs and eng.kv.free_blocks == eng.kv.num_blocks
    with pytest.raises(RuntimeError):        # a fifth live request has no slot
        for k in range(5):
            eng.step([(f"x{k}", [1], [])])
    for k in range(4):
        eng.release(f"x{k}")


def test_long_decode_past_windows_and_pages(dev):
    """300 decoded tokens after a 5-token prompt: the window slides over decoded tokens only, many page borders are crossed."""
    from vllm_i64_amd.engine import Engine
    cfg = R.make_config(**SHAPES["mixed_layers"])
    w = R.make_weights(cfg, seed=9)
    t = tokens(cfg, 305, 6)
    want = R.forward(cfg, w, t)
    for dtype in ("float32", "bfloat16"):
        eng = Engine(make_model(cfg, w, dtype, dev, max_tokens=320))
        got = replay(eng, {"a": t}, [[("a", 5)]] + [[("a", 1)] for _ in range(300)])
        assert rel_err(got["a"], want) < TOL[dtype]


def test_greedy_generation_through_the_scheduler(dev):
    """Engine.generate: more prompts than slots, a token budget that cuts prompts into portions, pages for prompt + answer only.
    In 32 bits the tokens are the oracle's wherever its own top two logits are not within rounding of each other."""
    from vllm_i64_amd.engine import Engine, SamplingParams
    cfg = R.make_config(**SHAPES["odd"])
    w = R.make_weights(cfg, seed=4)
    prompts = [tokens(cfg, n, 20 + n) for n in (9, 30, 1, 17, 23, 4)]
    steps = 12
    eng = Engine(make_model(cfg, w, "float32", dev, max_tokens=4 * 48, max_seqs=3), max_batch_tokens=16)
    outs = eng.generate(prompts, SamplingParams(max_new_tokens=steps))
    assert not eng.seqs and eng.kv.free_blocks == eng.kv.num_blocks
    for p, out in zip(prompts, outs):
        assert len(out) == steps
        seq = list(p)
        for tok in out:
            lg = R.forward(cfg, w, seq)[-1]
            top = lg.topk(2).values
            assert tok == int(lg.argmax()) or float(top[0] - top[1]) < 1e-3
            seq.append(tok)
    # sampling with a temperature: reproducible for a seed, inside the top-k set
    a = Engine(make_model(cfg, w, "float32", dev), max_batch_tokens=64).generate(prompts[:2], SamplingParams(max_new_tokens=6, temperature=0.8, top_k=4, seed=1))
    b = Engine(make_model(cfg, w, "float32", dev), max_batch_tokens=7).generate(prompts[:2], SamplingParams(max_new_tokens=6, temperature=0.8, top_k=4, seed=1))
    assert a == b
    for p, out in zip(prompts[:2], a):
        seq = list(p)
        for tok in out:
            assert tok in R.forward(cfg, w, seq)[-1].topk(4).indices.tolist()
            seq.append(tok)


def test_trace_replay_command_on_a_checkpoint_folder(dev, tmp_path):
    """bin/trace_run on a folder with config.json + model.safetensors: registry, loader, engine and output files end to end."""
    from safetensors.torch import save_file
    cfg = R.make_config(**SHAPES["odd"])
    w = R.make_weights(cfg, seed=2)
    model_dir, out_dir = tmp_path / "model", tmp_path / "out"
    model_dir.mkdir()
    save_file({k: v.contiguous() for k, v in w.items()}, str(model_dir / "model.safetensors"))
    (model_dir / "config.json").write_text(json.dumps(cfg))
    a, b = tokens(cfg, 40, 1), tokens(cfg, 19, 2)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:21], "want": [0, 20]}], "end": []},
             {"step": 1, "entries": [{"id": "b", "tokens": b[:2], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": a[21:], "want": [18]}, {"id": "b", "tokens": b[2:], "want": [0, 16]}], "end": ["a", "b"]}]
    for dtype in ("float32", "bfloat16"):
        p = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", str(model_dir), "--dtype", dtype, "--out", str(out_dir), "--max-tokens", "128"],
                           input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
        assert p.returncode == 0, p.stderr[-2000:]
        assert [ln for ln in p.stdout.splitlines() if ln.startswith("done")] == ["done 0", "done 1", "done 2"]
        assert not (out_dir / "1.f32").exists()
        wa, wb = R.forward(cfg, w, a), R.forward(cfg, w, b)
        g0 = np.fromfile(out_dir / "0.f32", dtype="<f4").reshape(2, -1)
        g2 = np.fromfile(out_dir / "2.f32", dtype="<f4").reshape(3, -1)
        assert rel_err(g0, wa[[0, 20]]) < TOL[dtype]
        assert rel_err(g2, torch.stack([wa[39], wb[2], wb[18]])) < TOL[dtype]
        for f in out_dir.iterdir():
            f.unlink()
