"""CPU-side pieces of the Dogalorn design: configuration, registry, the hybrid cache's pages and slots, the distance buckets, and
properties of the oracle's own mechanisms."""
import pytest
import torch

from oracle import dogalorn_ref as R
from vllm_i64_amd.config import DogalornConfig
from vllm_i64_amd.paged_cache import HybridCache

MAMBA = {"type": "mamba2", "mixer": {"heads": 2, "vdim": 6, "state": 5, "groups": 2, "conv": 3, "norm_groups": 2}, "mlp": {"kind": "dense", "ff": 20}}
PAR = {"type": "parallel", "mixer": {"left": {"heads": 4, "kv_heads": 2, "dim": 6, "vdim": 6, "scale": 0.3, "bias_max": 12, "mask": {"size": 9}},
                                     "right": {"width": 10}}, "mlp": None}
BASE = {"architecture": "Dogalorn", "vocab": 30, "width": 12, "streams": 3, "logit_scale": 1.5, "norm": {"eps": 1e-5},
        "embedding": {"bigram": {"buckets": 11, "mul_prev": 7, "mul_cur": 3}}, "layers": [MAMBA, PAR, dict(MAMBA, weights_of=0), dict(PAR, weights_of=1)]}


def test_config_round_trip_and_defaults():
    c = DogalornConfig.from_dict(BASE)
    assert DogalornConfig.from_dict(c.to_dict()) == c
    assert (c.streams, c.bigram.buckets, c.layers[1].mixer.left.chunk, c.layers[2].weights_of, c.layers[0].mixer.in_width) == (3, 11, 9, 0, 2 * 12 + 2 * 2 * 5 + 2)
    bare = DogalornConfig.from_dict({"architecture": "Dogalorn", "vocab": 30, "width": 12, "layers": [dict(PAR, mixer={"left": {"heads": 1, "dim": 4, "scale": 1.0},
                                                                                                                   "right": {"width": 3}})]})
    assert (bare.streams, bare.bigram, bare.logit_scale, bare.layers[0].mixer.left.chunk, bare.layers[0].mixer.left.kv_heads) == (0, None, 1.0, 0, 1)


@pytest.mark.parametrize("edit,msg", [
    (lambda d: d["layers"].__setitem__(3, dict(PAR, weights_of=2)), "borrows"),
    (lambda d: d["layers"].__setitem__(3, dict(PAR, weights_of=0)), "borrows"),
    (lambda d: d["layers"].__setitem__(0, dict(MAMBA, type="lstm")), "not built"),
    (lambda d: d["layers"].__setitem__(1, dict(PAR, mixer={"left": dict(PAR["mixer"]["left"], vdim=8), "right": {"width": 10}})), "values are the keys"),
    (lambda d: d["layers"].__setitem__(0, dict(MAMBA, mixer=dict(MAMBA["mixer"], groups=3))), "bad sizes"),
])
def test_config_refuses(edit, msg):
    import copy
    d = copy.deepcopy(BASE)
    edit(d)
    with pytest.raises(ValueError, match=msg):
        DogalornConfig.from_dict(d)


def test_registry_knows_the_design():
    from vllm_i64_amd import registry
    assert "dogalorn" in registry.architectures()
    assert registry.architecture_of(BASE) == "Dogalorn"


def test_hybrid_cache_pages_slots_and_state():
    kv = HybridCache([{"state": {"conv": (2, 16), "ssm": (2, 5, 6)}}, {"rows": 12, "state": {"gru": (10,)}}], num_blocks=6, max_seqs=3, device="cpu",
                     dtype=torch.bfloat16, block=4, seq_state={"prev_token": ((), torch.int64)})
    assert kv.rows[0] is None and tuple(kv.rows[1].shape) == (6, 4, 12) and tuple(kv.kscale[1].shape) == (6, 4) and kv.kscale[1].dtype == torch.float32
    assert tuple(kv.state[0]["ssm"].shape) == (3, 2, 5, 6) and tuple(kv.state[1]["gru"].shape) == (3, 10) and tuple(kv.seq_state["prev_token"].shape) == (3,)
    kv.reserve(0, 9), kv.reserve(2, 4)
    first = kv.blocks_of(0)
    assert len(first) == 3 and kv.free_blocks == 2
    with pytest.raises(RuntimeError):
        kv.reserve(1, 13)
    kv.free(0)
    kv.reserve(1, 13)         # the pages that slot 0 gave back, last freed first
    assert kv.blocks_of(1)[:3] == first[::-1] and kv.free_blocks == 1


def test_distance_buckets_match_the_oracle():
    from vllm_i64_amd.dogalorn import distance_bias_table
    for rows, far in ((8, 20), (9, 11), (32, 240), (2, 3), (6, 40.5), (16, 64)):
        rel = torch.arange(rows, dtype=torch.float32).reshape(rows, 1)
        table = distance_bias_table(rel, far)
        for n in range(0, 400):
            assert int(table[min(n, table.shape[0] - 1), 0]) == R.distance_bucket(n, rows, far), (rows, far, n)


def test_oracle_sink_and_candidate():
    g = torch.Generator().manual_seed(0)
    H, d, T = 2, 4, 6
    w = {"q": torch.eye(H * d), "k": torch.eye(H * d), "o": torch.eye(H * d), "q.norm": torch.ones(H * d), "k.norm": torch.ones(H * d),
         "rel": torch.full((4, H), -30.0), "temp": torch.ones(H)}
    h = torch.randn(T, H * d, generator=g)
    out = R.chunked_bias_attention({k: v.double() for k, v in w.items()}, "", {"heads": H, "kv_heads": H, "dim": d, "scale": 0.1, "bias_max": 8}, 1e-6, h.double())
    assert float(out.abs().max()) < 1e-9          # every score far below the sink's zero: nothing gets through
    w1 = {"z": torch.zeros(1, 1), "z.b": torch.tensor([50.0]), "x": torch.eye(1), "x.b": torch.zeros(1), "g": torch.zeros(1, 1), "o": torch.eye(1)}
    # z = 1: the state is the candidate; the gate silu(0) = 0 hides it, so look at the candidate's two branches through a gate of one
    w1["g"] = torch.tensor([[0.0]])
    u = torch.tensor([[-1e-9], [0.0], [2.0]], dtype=torch.float64)
    cand = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    assert abs(float(cand[0] - cand[1])) < 1e-8 and float(cand[2]) == 2.5
