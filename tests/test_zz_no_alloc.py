"""cute_spmm_run_static -- the entry point that allocates nothing -- through the C ABI, against
cute_spmm_run on the same plans: two calls in a row, the second on a smaller input, every output
poisoned first.  Both entry points launch the same kernels and add the partial tiles of cut panels in
the same fixed order, so the bar is equality bit for bit (and the oracle's tolerance for both)."""
import numpy as np
import pytest

from helpers import random_csr

pytestmark = pytest.mark.gpu

BERR = 2e-6


def _both(cs, torch, h, B, **kw):
    N = B.shape[1]
    dB = torch.from_numpy(np.ascontiguousarray(B)).cuda()
    plan = cs.SPMM_TC(h, N, **kw)
    dC = torch.full((h.M, N), float("nan"), device="cuda")
    plan.run(dB, dC)
    torch.cuda.synchronize()
    want = dC.cpu().numpy().copy()
    dC.fill_(float("nan"))
    plan.run_static(dB, dC)
    torch.cuda.synchronize()
    return want, dC.cpu().numpy(), plan


def test_static_scratch_entry_point(cs, orc):
    import torch
    assert torch.cuda.is_available()
    rng = np.random.default_rng(77)
    # first call: long panels that the planner cuts (partial tiles in use), 128 columns
    M, K, N = 1024, 4096, 128
    rp, cl, vl = random_csr(rng, M, K, row_nnz=lambda r: 1500 if r in (5, 300, 900) else 6)
    B = rng.standard_normal((K, N)).astype(np.float32)
    ref = orc.spmm_csr(rp, cl, vl, B)
    h = cs.HRPB(M, K, rp, cl, vl)
    # second call: a smaller matrix and a narrower N, so that stale tiles of the first call lie all around its own
    M2, K2, N2 = 256, 1024, 48
    rp2, cl2, vl2 = random_csr(rng, M2, K2, row_nnz=lambda r: 600 if r == 17 else 3)
    B2 = rng.standard_normal((K2, N2)).astype(np.float32)
    ref2 = orc.spmm_csr(rp2, cl2, vl2, B2)
    h2 = cs.HRPB(M2, K2, rp2, cl2, vl2)
    for kw in (dict(path=cs.PATH_BRICK, mfma_shape=1), dict(path=cs.PATH_BRICK, mfma_shape=2),
               dict(path=cs.PATH_BRICK, mfma_shape=1, pipeline=2), dict(), dict(path=cs.PATH_BRICK, mfma_shape=2, max_chunk_blocks=2)):
        want, got, plan = _both(cs, torch, h, B, **kw)
        assert plan.info["numAtomicChunks"] > 0 and 0 < plan.info["partialTileKiB"] * 1024 <= cs.STATIC_SCRATCH_BYTES, kw
        assert got.tobytes() == want.tobytes(), kw
        assert cs.backward_error(rp, cl, vl, B, ref, got) <= BERR, kw
        want2, got2, plan2 = _both(cs, torch, h2, B2, **kw)
        assert plan2.info["numAtomicChunks"] > 0 and plan2.info["partialTileKiB"] < plan.info["partialTileKiB"], kw
        assert got2.tobytes() == want2.tobytes(), kw
        assert cs.backward_error(rp2, cl2, vl2, B2, ref2, got2) <= BERR, kw
    # a plan without cut panels uses no scratch at all and runs the same way
    want, got, plan = _both(cs, torch, h2, B2, path=cs.PATH_ROWS)
    assert plan.info["partialTileKiB"] == 0 and got.tobytes() == want.tobytes()


def test_static_entry_point_allocates_nothing(cs):
    """Free device memory as the driver reports it does not move across many calls, on a plan that uses the scratch."""
    import torch
    rng = np.random.default_rng(3)
    M, K, N = 1024, 4096, 128
    rp, cl, vl = random_csr(rng, M, K, row_nnz=lambda r: 1500 if r in (5, 300, 900) else 6)
    h = cs.HRPB(M, K, rp, cl, vl)
    plan = cs.SPMM_TC(h, N, path=cs.PATH_BRICK, mfma_shape=2)
    assert plan.info["numAtomicChunks"] > 0
    dB = torch.randn((K, N), device="cuda")
    dC = torch.empty((M, N), device="cuda")
    stream = torch.cuda.current_stream()
    plan.run_static(dB, dC, stream=stream)
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    for _ in range(200):
        plan.run_static(dB, dC, stream=stream)
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before


def test_caller_scratch_on_two_streams(cs, orc):
    """cute_spmm_run_scratch: one plan, two streams at the same time, each call with a buffer of its own; the bits
    of cute_spmm_run.  Too small a buffer is refused before anything is launched."""
    import torch
    rng = np.random.default_rng(21)
    M, K, N = 2048, 4096, 256
    rp, cl, vl = random_csr(rng, M, K, row_nnz=lambda r: 2500 if r % 256 == 3 else 5)
    h = cs.HRPB(M, K, rp, cl, vl)
    Bs = [rng.standard_normal((K, N)).astype(np.float32) for _ in range(2)]
    refs = [orc.spmm_csr(rp, cl, vl, B) for B in Bs]
    for kw in (dict(path=cs.PATH_BRICK, mfma_shape=2), dict(path=cs.PATH_BRICK, mfma_shape=1), dict()):
        plan = cs.SPMM_TC(h, N, **kw)
        need = plan.scratch_bytes
        assert plan.info["numAtomicChunks"] > 0 and need > 0 and (need + 1023) // 1024 == plan.info["partialTileKiB"]
        dBs = [torch.from_numpy(B).cuda() for B in Bs]
        want = []
        for dB in dBs:
            dC = torch.full((M, N), float("nan"), device="cuda")
            plan.run(dB, dC)
            torch.cuda.synchronize()
            want.append(dC.cpu().numpy())
        streams = [torch.cuda.Stream(), torch.cuda.Stream()]
        scratch = [torch.empty(need, dtype=torch.uint8, device="cuda") for _ in streams]
        outs = [torch.full((M, N), float("nan"), device="cuda") for _ in streams]
        torch.cuda.synchronize()
        for rep in range(10):                      # overlapping launches of the one plan
            for i, st in enumerate(streams):
                plan.run_scratch(dBs[i], outs[i], scratch[i], stream=st)
        torch.cuda.synchronize()
        for i in range(2):
            got = outs[i].cpu().numpy()
            assert got.tobytes() == want[i].tobytes(), (kw, i)
            assert cs.backward_error(rp, cl, vl, Bs[i], refs[i], got) <= BERR
        small = torch.empty(need - 16, dtype=torch.uint8, device="cuda")
        with pytest.raises(cs.CuteError) as e:
            plan.run_scratch(dBs[0], outs[0], small)
        assert e.value.status == -10
    # a plan without cut panels needs no buffer
    plan = cs.SPMM_TC(h, N, path=cs.PATH_ROWS)
    assert plan.scratch_bytes == 0
    dC = torch.full((M, N), float("nan"), device="cuda")
    plan.run_scratch(torch.from_numpy(Bs[0]).cuda(), dC, None)
    torch.cuda.synchronize()
    assert cs.backward_error(rp, cl, vl, Bs[0], refs[0], dC.cpu().numpy()) <= BERR


def test_static_scratch_limit(cs):
    """A plan whose partial tiles exceed the static array is refused by the entry point, with both sizes in the message."""
    import torch
    A = cs.gen_config(2, 1 / 4.0)                                   # 16 384-row stencil
    h = cs.HRPB(A.M, A.K, A.rowPtr, A.cols, A.vals)
    N = 512
    plan = cs.SPMM_TC(h, N, path=cs.PATH_BRICK, mfma_shape=1, max_chunk_blocks=1)    # every block a piece of its own
    assert plan.info["partialTileKiB"] * 1024 > cs.STATIC_SCRATCH_BYTES
    dB = torch.zeros((A.K, N), device="cuda")
    dC = torch.full((A.M, N), 7.0, device="cuda")
    with pytest.raises(cs.CuteError) as e:
        plan.run_static(dB, dC)
    assert e.value.status == -10 and str(cs.STATIC_SCRATCH_BYTES) in str(e.value)
    torch.cuda.synchronize()
    assert (dC == 7.0).all().item()                                 # nothing was launched
    plan.run(dB, dC)                                                # the allocating entry point still serves the plan
    torch.cuda.synchronize()
    assert (dC == 0.0).all().item()
