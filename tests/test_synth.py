import torch
from forge import synth


def test_dense_outlier_is_seeded_and_has_outlier_channels():
    a, b = synth.dense_outlier(R=64, C=256, n=128), synth.dense_outlier(R=64, C=256, n=128)
    assert torch.equal(a.W, b.W) and torch.equal(a.X, b.X)
    col_rms = a.X.pow(2).mean(0).sqrt()
    assert int((col_rms > 10).sum()) == round(0.01 * 256)


def test_routing_is_ragged_top8():
    rows = synth.route_topk(1024, 32, 8, torch.Generator().manual_seed(0))
    counts = [len(r) for r in rows]
    assert sum(counts) == 8 * 1024 and max(counts) > 3 * min(counts)
    assert all(len(set(r.tolist())) == len(r) for r in rows)


def test_fp8_roundtrip_is_close_and_bf16():
    W = (0.02 * torch.randn(200, 300)).bfloat16()
    Q = synth.fp8_block_roundtrip(W)
    assert Q.dtype == torch.bfloat16 and Q.shape == W.shape
    assert ((Q.float() - W.float()).abs() <= 0.07 * W.float().abs() + 1e-4).all()


def test_moe_case_shapes():
    m = synth.qwen3_moe(experts=2, n_experts=16, hidden=128, inter=64, tokens=256)
    x, h = m.expert_inputs(0)
    assert x.shape[1] == 128 and h.shape == (x.shape[0], 64) and h.dtype == torch.bfloat16
