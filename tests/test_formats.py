"""fp8 block-scale dequant (into the path) and the 1:4 sparse u64x2 words (out of it)."""
import numpy as np
import pytest
import torch

import oracle

DEV = "cuda"


def _sparse_case(R, C, seed):
    g = torch.Generator().manual_seed(seed)
    q = torch.randint(0, 16, (R, C), dtype=torch.uint8, generator=g)
    G32 = (C + 31) // 32
    pos = torch.randint(0, 4, (G32 * 8, R), generator=g)                 # kept column per group of 4
    bits = (1 << pos).view(G32, 8, R)
    bits[0, 3] = 0                                                        # a group with nothing kept
    M = sum(bits[:, i] << (4 * i) for i in range(8)).to(torch.int64)
    M = (M & 0xFFFFFFFF).to(torch.int64)
    M32 = M.to(torch.int32) if False else torch.from_numpy(M.numpy().astype(np.uint32).view(np.int32))
    scales = torch.rand(G32, R, generator=g) * 0.02 + 1e-4
    return q, M32, scales, pos.view(G32, 8, R)


def test_oracle_sparse_pack_layout():
    """Pins the oracle's packer with an independent numpy decode of every field."""
    R, C = 17, 200
    q, M32, scales, pos = _sparse_case(R, C, 0)
    out = oracle.pack_sparsegptq14_to_u64x2(q, M32, scales).numpy().astype(np.uint64)
    G32 = (C + 31) // 32
    assert out.shape == ((G32 + 1) // 2, R, 2)
    for gid in range(G32):
        word = out[gid // 2, :, gid % 2]
        qw32 = word & np.uint64(0xFFFFFFFF)
        idx16 = (word >> np.uint64(32)) & np.uint64(0xFFFF)
        sbits = ((word >> np.uint64(48)) & np.uint64(0xFFFF)).astype(np.uint32) << 16
        s = sbits.view(np.float32) if sbits.dtype == np.uint32 else None
        assert np.allclose(s, scales[gid].numpy(), rtol=2 ** -8)
        assert np.array_equal(s, scales[gid].bfloat16().float().numpy())
        for i in range(8):
            nib = (qw32 >> np.uint64(4 * i)) & np.uint64(0xF)
            p2 = (idx16 >> np.uint64(2 * i)) & np.uint64(3)
            if gid == 0 and i == 3:
                assert np.all(nib == 8) and np.all(p2 == 0)               # empty group: code 8
                continue
            c = pos[gid, i].numpy()
            assert np.array_equal(p2, c.astype(np.uint64))
            cid = gid * 32 + 4 * i + c
            want = np.where(cid < C, q.numpy()[np.arange(R), np.minimum(cid, C - 1)], 8)
            assert np.array_equal(nib, want.astype(np.uint64))
    if G32 % 2:
        assert np.all(out[-1, :, 1] == 0)                                 # missing partner word


def test_oracle_fp8_dequant_matches_tile_loop():
    g = torch.Generator().manual_seed(1)
    O, I = 300, 256
    w = (torch.randn(O, I, generator=g) * 50).to(torch.float8_e4m3fn)
    s = torch.rand(3, 2, generator=g) * 0.01 + 1e-4
    got = oracle.fp8_block_dequant(w, s)
    want = torch.empty(O, I)
    for bo in range(3):
        for bi in range(2):
            blk = w[bo * 128:(bo + 1) * 128, bi * 128:(bi + 1) * 128].float()
            want[bo * 128:(bo + 1) * 128, bi * 128:(bi + 1) * 128] = blk * s[bo, bi]
    assert torch.equal(got, want.bfloat16())


@pytest.mark.gpu
@pytest.mark.parametrize("R,C", [(64, 256), (17, 200), (130, 96), (100, 1100), (33, 2080), (70, 4100)])
def test_gpu_sparse_pack_bit_exact(hip, R, C):
    q, M32, scales, _ = _sparse_case(R, C, R + C)
    want = oracle.pack_sparsegptq14_to_u64x2(q, M32, scales)
    got = hip.pack_sparsegptq14_to_u64x2(q.to(DEV), M32.view(torch.uint32).to(DEV), scales.to(DEV))
    assert got.dtype == torch.uint64 and tuple(got.shape) == tuple(want.shape)
    assert torch.equal(got.view(torch.int64).cpu(), want)


@pytest.mark.gpu
@pytest.mark.parametrize("O,I,dtype", [(256, 512, torch.bfloat16), (300, 384, torch.bfloat16),
                                       (77, 128, torch.float32), (50, 200, torch.bfloat16),
                                       (40, 136, torch.float32), (3, 20480, torch.bfloat16)])
def test_gpu_fp8_block_dequant_bit_exact(hip, O, I, dtype):
    g = torch.Generator().manual_seed(O)
    raw = torch.randint(0, 256, (2, O, I), dtype=torch.uint8, generator=g)      # every byte pattern
    w = raw.view(torch.float8_e4m3fn)
    s = torch.rand(2, (O + 127) // 128, I // 128, generator=g) * 0.01 + 1e-4
    got = hip.fp8_block_dequant(w.to(DEV), s.to(DEV), dtype).cpu()
    for b in range(2):
        want = oracle.fp8_block_dequant(w[b], s[b], dtype)
        a, c = got[b].float(), want.float()
        nan = torch.isnan(c)
        assert torch.equal(torch.isnan(a), nan)
        assert torch.equal(a[~nan], c[~nan])


@pytest.mark.gpu
def test_gpu_fp8_roundtrip_feeds_the_solver(hip):
    """Config-3 pre-step: encode to fp8 + 128x128 scales as the generator does, decode on
    the GPU, and get exactly the bf16 weights the CPU round trip produces."""
    from forge import synth
    W = (0.02 * torch.randn(256, 384)).bfloat16()
    blk = W.float().view(2, 128, 3, 128)
    s_inv = blk.abs().amax(dim=(1, 3)).clamp_min(1e-12) / 448.0
    q = (blk / s_inv[:, None, :, None]).to(torch.float8_e4m3fn).reshape(256, 384)
    got = hip.fp8_block_dequant(q.to(DEV), s_inv.to(DEV)).cpu()
    assert torch.equal(got, synth.fp8_block_roundtrip(W))


@pytest.mark.gpu
@pytest.mark.parametrize("sym", [True, False])
def test_layer_record_and_consumer_tensors(hip, sym):
    """The per-layer dict of quant.py:498-511 and the tensor set of pack_quantized.py:279-313
    built from a quantize() result: dtypes and shapes as the reference writes them, the record
    dequantises to the same weights, and weight_packed decodes back to code - zero."""
    from forge.gptq import GPTQ
    from forge import export
    from helpers import linear
    g = torch.Generator().manual_seed(9)
    R, C, gs = 96, 328, 128
    W = 0.02 * torch.randn(R, C, generator=g)
    h = GPTQ(linear(W).to(DEV), device=DEV, bits=4, group_size=gs, symmetric=sym,
             quantization_scale="absmax", quantization_order="activation")
    h.update(torch.randn(512, C, generator=g).to(DEV))
    q, s, z = h.quantize()
    G = h.G
    rec = export.layer_record(q, s, z, gs, 4, W.shape)
    assert rec["qweight"].dtype == torch.int8 and tuple(rec["qweight"].shape) == (R, C)
    assert rec["scales"].dtype == torch.float32 and rec["qzeros"].dtype == torch.int32
    assert rec["scales"].numel() == R * G and rec["group_size"] == gs and rec["bits"] == 4
    assert rec["shape"] == (R, C)
    assert torch.equal(rec["qzeros"].float(), z)                      # zeros are whole numbers
    deq = oracle.dequantize(rec["qweight"].cpu().to(torch.uint8), rec["scales"].cpu(),
                            rec["qzeros"].cpu().float(), gs)
    assert torch.equal(deq, oracle.dequantize(q.cpu(), s.cpu(), z.cpu(), gs))
    out = export.pack_weight(rec, bits=4, sym=sym, group_size=gs)
    assert set(out) == {"weight_packed", "weight_shape", "weight_scale"} | (set() if sym else {"weight_zero_point"})
    assert out["weight_shape"].tolist() == [R, C] and out["weight_shape"].dtype == torch.int64
    assert tuple(out["weight_scale"].shape) == (R, G) and torch.equal(out["weight_scale"].reshape(-1), s)
    pk = out["weight_packed"].cpu()
    assert pk.dtype == torch.int32 and tuple(pk.shape) == (R, (C + 7) // 8)
    nib = torch.stack([(pk.to(torch.int64) >> (4 * k)) & 0xF for k in range(8)], dim=-1).reshape(R, -1)[:, :C]
    zz = z.cpu().view(R, G).repeat_interleave(gs, 1)[:, :C].to(torch.int64)
    # offset binary of code - zero; a difference outside [-8, 7] (possible with asymmetric
    # zeros) wraps in the nibble, as it does in the reference's int8 subtraction + 4-bit pack
    assert torch.equal(nib, (q.cpu().to(torch.int64) - zz + 8) & 0xF)
    inside = (q.cpu().to(torch.int64) - zz).abs() < 8
    assert torch.equal((nib - 8)[inside], (q.cpu().to(torch.int64) - zz)[inside])
    if not sym:
        assert torch.equal(out["weight_zero_point"].reshape(-1).float(), z)
    # the reference's own key names are read too
    alt = export.pack_weight({"qweight": rec["qweight"], "scale": rec["scales"].view(R, G),
                              "zero": rec["qzeros"].view(R, G).to(torch.int8)}, 4, sym, gs)
    assert torch.equal(alt["weight_packed"], out["weight_packed"])
    with pytest.raises(NotImplementedError):
        export.pack_weight(rec, bits=3, sym=sym, group_size=gs)
