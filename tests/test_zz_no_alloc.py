"""forge_hessian_update_static, the entry point that allocates nothing (its workspace is a
device array inside the library), against forge_hessian_update_grouped with one group: the
same kernels, so the same bits.  Two calls in a row on the same array, the second with a
smaller input, then a running-mean update (beta != 0), for bf16 and f32 tokens."""
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _grouped(hip, X, H, alpha, beta):
    Hb = H.clone().view(1, *H.shape)
    hip.hessian_update_grouped(X, [0, X.shape[0]], Hb, [alpha], [beta])
    return Hb[0]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "f32"])
def test_static_entry_point_matches_the_grouped_one(hip, dtype):
    g = torch.Generator().manual_seed(5)
    for n, C in ((700, 1024), (130, 328), (33, 1024)):        # larger first, then smaller ones
        X = torch.randn(n, C, generator=g).to(dtype).to(DEV)
        H0 = torch.randn(C, C, generator=g).to(DEV)
        H0 = (H0 + H0.t()).contiguous()
        for alpha, beta in ((2.0 / n, 0.0), (2.0 / (n + 50), 50.0 / (n + 50))):
            want = _grouped(hip, X, H0, alpha, beta)
            got = hip.hessian_update_static(X, H0.clone(), alpha, beta)
            torch.cuda.synchronize()
            assert torch.equal(got, want), (n, C, alpha, beta)
            ref = beta * H0.double() + alpha * (X.double().t() @ X.double())
            assert ((got.double() - ref).norm() / ref.norm()).item() < 2e-6
    # no rows: H untouched
    H1 = H0.clone()
    hip.hessian_update_static(X[:0], H1, 1.0, 0.0)
    assert torch.equal(H1, H0)


def test_static_entry_point_rejects_what_does_not_fit(hip):
    from forge.backend.hip import load_library
    lib = load_library()
    assert lib.forge_hessian_update_static_max_rows(7168, 1) == 2336
    assert lib.forge_hessian_update_static_max_rows(2048, 1) == 8192
    assert lib.forge_hessian_update_static_max_rows(20000, 1) == 0
    X = torch.zeros(16, 64, dtype=torch.bfloat16, device=DEV)
    H = torch.zeros(64, 64, device=DEV)
    rc = lib.forge_hessian_update_static(X.data_ptr(), 1, 7168, 2337, 7168, 1.0, 0.0, H.data_ptr(), None)
    assert rc == 1 and b"exceeds the static workspace" in lib.forge_last_error()
    rc = lib.forge_hessian_update_static(X.data_ptr(), 0, 20000, 4, 20000, 1.0, 0.0, H.data_ptr(), None)
    assert rc == 1 and b"columns" in lib.forge_last_error()


def test_static_entry_point_allocates_nothing_and_creates_no_events(hip):
    """What the entry point is for: across its calls (after the first on the device, which looks
    the array's address up) the device's free memory and torch's reserved memory do not move,
    and with per-kernel timing switched on it files no record (a record is a pair of events)."""
    g = torch.Generator().manual_seed(9)
    X = torch.randn(300, 512, generator=g).bfloat16().to(DEV)
    Xf = torch.randn(90, 512, generator=g).to(DEV)
    H = torch.zeros(512, 512, device=DEV)
    hip.hessian_update_static(X, H, 1.0, 0.0)              # first call on this device
    torch.cuda.synchronize()
    free0, reserved0 = torch.cuda.mem_get_info()[0], torch.cuda.memory_reserved()
    hip.timing_enable(True)
    try:
        for _ in range(3):
            hip.hessian_update_static(X, H, 0.5, 0.5)
            hip.hessian_update_static(Xf, H, 0.5, 0.5)
        torch.cuda.synchronize()
        records = hip.timing_collect()
    finally:
        hip.timing_enable(False)
    assert records == {}
    assert torch.cuda.mem_get_info()[0] == free0 and torch.cuda.memory_reserved() == reserved0
