"""Host-side parts of serving the Morilorn design, on the CPU: configuration, registry, page pool, the engine's batching and
scheduling (with a stand-in runner), and the algebra the GPU path relies on, checked in the oracle's own terms."""
import pytest
import torch

from oracle import morilorn_ref as R
from vllm_i64_amd.config import MorilornConfig
from vllm_i64_amd.engine import Engine, SamplingParams
from vllm_i64_amd.paged_cache import LatentCache, PagePool
from vllm_i64_amd import registry


def test_config_reads_every_size_and_constant():
    d = R.make_config(vocab=77, width=36, layers=2, groups=3, alpha=1.25, embed_scale=2.0, softcap=5.0, eps=1e-4, per_layer=[
        dict(heads=2, dim=6, rot_dim=4, vdim=5, kv_rank=9, window=3, ff=10, rot_base=123.0, scale=0.5),
        dict(heads=1, dim=3, rot_dim=8, vdim=7, kv_rank=11, window=0, ff=None, rot_dims=4)])
    c = MorilornConfig.from_dict(d)
    assert (c.vocab, c.width, c.num_layers, c.norm_groups, c.postln_alpha, c.embedding_scale, c.logit_softcap, c.norm_eps) == (77, 36, 2, 3, 1.25, 2.0, 5.0, 1e-4)
    m0, m1 = c.layers[0].mixer, c.layers[1].mixer
    assert (m0.heads, m0.dim, m0.rot_dim, m0.vdim, m0.kv_rank, m0.window, m0.rot_base, m0.rot_dims, m0.scale) == (2, 6, 4, 5, 9, 3, 123.0, 4, 0.5)
    assert (m1.window, m1.rot_dims, m1.cache_width, m1.q_width) == (0, 4, 19, 11) and c.layers[1].mlp is None and c.layers[0].mlp.ff == 10
    assert MorilornConfig.from_dict(c.to_dict()) == c
    bad = R.make_config()
    bad["layers"][0]["type"] = "something_else"
    with pytest.raises(ValueError):
        MorilornConfig.from_dict(bad)
    bad = R.make_config()
    bad["layers"][0]["mlp"]["kind"] = "sparse"
    with pytest.raises(ValueError):
        MorilornConfig.from_dict(bad)
    with pytest.raises(ValueError):
        MorilornConfig.from_dict(R.make_config(width=50, groups=3))


def test_registry_picks_the_runner_by_config():
    assert registry.architecture_of({"architecture": "Morilorn"}) == "Morilorn"
    assert registry.architecture_of({"model_type": "complexity-deep"}) == "complexity-deep"
    assert "morilorn" in registry.architectures() and "complexity-deep" in registry.architectures()
    with pytest.raises(ValueError):
        registry.load_model("/nonexistent", config={"architecture": "NoSuchDesign"})
    with pytest.raises(ValueError):
        registry.architecture_of({})


def test_page_pool_hands_freed_pages_out_again():
    pool = PagePool(num_blocks=6, block=16, max_seqs=3, max_blocks_per_seq=6, device="cpu")
    pool.reserve(0, 17)
    pool.reserve(1, 40)
    assert pool.blocks_of(0) == [0, 1] and pool.blocks_of(1) == [2, 3, 4] and pool.free_blocks == 1
    pool.reserve(0, 32)                       # no new page inside the last one
    assert pool.free_blocks == 1
    with pytest.raises(RuntimeError):
        pool.reserve(2, 33)
    pool.free(1)
    assert pool.free_blocks == 4 and pool.block_table[1].tolist() == [-1] * 6
    pool.reserve(2, 33)                       # the pages sequence 1 gave back, last freed first
    assert pool.blocks_of(2) == [4, 3, 2]
    pool.reserve(0, 33)
    assert pool.blocks_of(0) == [0, 1, 5] and pool.free_blocks == 0
    lc = LatentCache([10, 24], num_blocks=4, max_seqs=2, device="cpu", dtype=torch.float32)
    assert [tuple(r.shape) for r in lc.rows] == [(4, 16, 10), (4, 16, 24)] and lc.max_blocks_per_seq == 4


class _FakeRunner:
    """Stands in for a GPU runner: remembers what each step was given; logits put all mass on (token + position) % vocab."""

    class _Cfg:
        vocab_size = 50

    def __init__(self, num_blocks=8, max_seqs=3):
        self.cfg, self.device = self._Cfg(), torch.device("cpu")
        self.kv = PagePool(num_blocks, 16, max_seqs, num_blocks, "cpu")
        self.calls = []

    def check_sync(self, force=True):
        pass

    def forward(self, ids, pos, slots, ctx_len, logit_rows=None, max_ctx_hint=0, tokens_per_seq=None, **kw):
        self.calls.append(dict(ids=ids.tolist(), pos=pos.tolist(), slots=slots.tolist(), rows=logit_rows.tolist(), tps=list(tokens_per_seq)))
        for s, p in zip(slots.tolist(), pos.tolist()):       # every position the kernels would touch has a page
            assert self.kv._bt_host[s, p // 16] >= 0
        out = torch.zeros(len(logit_rows), 50)
        for k, r in enumerate(logit_rows.tolist()):
            out[k, (ids[r] + pos[r]) % 50] = 1.0
        return out


def test_engine_step_lays_out_rows_positions_and_slots():
    m = _FakeRunner()
    e = Engine(m)
    lg = e.step([("a", [5, 6, 7], [0, 2]), ("b", [9], [])])
    assert lg.shape == (2, 50)
    c = m.calls[-1]
    assert c == dict(ids=[5, 6, 7, 9], pos=[0, 1, 2, 0], slots=[0, 0, 0, 1], rows=[0, 2], tps=[3, 1])
    e.step([("b", [1, 2], [1]), ("a", [8], [0])], end=["a"])
    c = m.calls[-1]
    assert c == dict(ids=[1, 2, 8], pos=[1, 2, 3], slots=[1, 1, 0], rows=[1, 2], tps=[2, 1])
    assert "a" not in e.seqs and m.kv.blocks_of(0) == []
    e.step([("c", [3] * 20, [19])])                                     # 'c' takes the slot and the page 'a' gave back
    assert m.calls[-1]["slots"] == [0] * 20 and m.kv.blocks_of(0)[0] == 0
    assert e.step([("b", [4], [])]).shape == (0, 50)                    # nothing asked for: the step still runs
    assert m.calls[-1]["pos"] == [3]
    with pytest.raises(ValueError):
        e.step([("b", [1], [1])])
    with pytest.raises(ValueError):
        e.step([("b", [50], [0])])


def test_engine_schedules_portions_under_a_budget_and_queues_requests(monkeypatch):
    monkeypatch.setattr(Engine, "_sample", lambda self, logits, seqs: logits.argmax(-1).tolist())
    m = _FakeRunner(num_blocks=6, max_seqs=2)
    e = Engine(m, max_batch_tokens=8)
    prompts = [[7, 8, 9], list(range(1, 21)), list(range(30, 42))]
    outs = e.generate(prompts, SamplingParams(max_new_tokens=3))
    assert not e.seqs and m.kv.free_blocks == 6
    for p, out in zip(prompts, outs):                                    # the fake model's next token is (token + position) % 50
        seq, want = list(p), []
        for _ in range(3):
            want.append((seq[-1] + len(seq) - 1) % 50)
            seq.append(want[-1])
        assert out == want
    assert all(sum(c["tps"]) <= 8 for c in m.calls)
    assert any(1 in c["tps"] and max(c["tps"]) > 1 for c in m.calls)    # decoded tokens rode beside a prompt's portion
    assert max(len(c["tps"]) for c in m.calls) <= 2                      # never more live requests than slots
    # a stop token ends a request early
    e2 = Engine(_FakeRunner(), max_batch_tokens=8)
    assert e2.generate([[7, 8, 9]], SamplingParams(max_new_tokens=5, stop_token=(9 + 2) % 50)) == [[11]]


def test_scores_and_values_through_latent_space_equal_the_written_out_form():
    """What the GPU path relies on: q . (U c) = (U^T q) . c per head, and sum_j w_j (V c_j) = V (sum_j w_j c_j)."""
    g = torch.Generator().manual_seed(0)
    H, d, v, r, T = 3, 5, 4, 7, 6
    q = torch.randn(T, H, d, generator=g, dtype=torch.float64)
    c = torch.randn(T, r, generator=g, dtype=torch.float64)
    uk = torch.randn(H * d, r, generator=g, dtype=torch.float64)
    uv = torch.randn(H * v, r, generator=g, dtype=torch.float64)
    k = (c @ uk.T).reshape(T, H, d)
    val = (c @ uv.T).reshape(T, H, v)
    see = R.visible(T, 3)
    assert see[4].tolist() == [False, False, True, True, True, False] and R.visible(3, 0)[2].tolist() == [True] * 3
    for h in range(H):
        s = (q[:, h] @ k[:, h].T).masked_fill(~see, float("-inf"))
        q_lat = q[:, h] @ uk[h * d:(h + 1) * d]                    # [T, r]
        s2 = (q_lat @ c.T).masked_fill(~see, float("-inf"))
        assert torch.allclose(s, s2)
        wgt = torch.softmax(s, -1)
        assert torch.allclose(wgt @ val[:, h], (wgt @ c) @ uv[h * v:(h + 1) * v].T)
