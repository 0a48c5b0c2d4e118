"""Randomised differential test of the launch paths: random small matrices of seven shapes (uniform, banded, power-law
rows, dense 16x16 blocks, hub columns, nearly empty, one full row), random widths 1..1000, random tunables (kernel family,
MFMA shape, brick variant, chunk policy and order, row-kernel thresholds, residency hint), host-built and device-built
handles, and the three run entry points.  Operands are small integers (explicit zeros included), so every order of
summation gives the same float32 bits and each product must EQUAL the oracle's."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

KINDS = ("uniform", "banded", "powerlaw", "blocks", "hub", "sparse_rows", "one_dense_row")
WIDTHS = (1, 2, 3, 4, 7, 8, 16, 31, 32, 33, 48, 64, 100, 128, 130, 256, 512, 1000)


def _matrix(rng, kind):
    M = int(rng.choice([16, 32, 48, 64, 128, 256, 512, 1024, 2048]))
    K = int(rng.choice([16, 32, 64, 128, 256, 1024, 4096, 16384]))
    rows = []
    for r in range(M):
        if kind == "uniform":
            c = rng.choice(K, rng.integers(0, min(K, 24) + 1), replace=False)
        elif kind == "banded":
            w = min(K, 40)
            lo = min(max(0, int(r * K / M) - w // 2), K - w)
            c = lo + rng.choice(w, rng.integers(0, min(w, 12) + 1), replace=False)
        elif kind == "powerlaw":
            c = rng.choice(K, min(K, int(rng.pareto(1.2) * 2)), replace=False)
        elif kind == "blocks":
            c = ((r // 16) % max(1, K // 16)) * 16 + rng.choice(16, rng.integers(8, 17), replace=False)
            if rng.random() < 0.2:
                c = np.concatenate([c, rng.choice(K, 2)])
        elif kind == "hub":
            c = np.concatenate([rng.choice(min(K, 8), min(int(rng.integers(0, 6)), min(K, 8)), replace=False), rng.choice(K, 2)])
        elif kind == "sparse_rows":
            c = rng.choice(K, 1) if rng.random() < 0.3 else np.zeros(0, np.int64)
        else:
            c = np.arange(K) if r == M // 2 else rng.choice(K, rng.integers(0, 3), replace=False)
        rows.append(np.unique(np.asarray(c, np.int64)))
    rp = np.zeros(M + 1, np.uint32)
    rp[1:] = np.cumsum([len(c) for c in rows])
    cl = (np.concatenate(rows) if rp[-1] else np.zeros(0, np.int64)).astype(np.uint32)
    vl = rng.integers(-2, 3, len(cl)).astype(np.float32)
    return M, K, rp, cl, vl


@pytest.mark.parametrize("kind", KINDS)
def test_random_plans_equal_the_oracle(cs, orc, torch_cuda, kind):
    torch = torch_cuda
    rng = np.random.default_rng(20240 + KINDS.index(kind))
    launches = 0
    for case in range(10):
        M, K, rp, cl, vl = _matrix(rng, kind)
        N = int(rng.choice(WIDTHS))
        if M * N > (1 << 20):
            N = max(1, (1 << 20) // M)
        B = rng.integers(-3, 4, (K, N)).astype(np.float32)
        ref = orc.spmm_csr(rp, cl, vl, B)
        dB = torch.from_numpy(B).cuda()
        if case % 2:
            h = cs.DeviceHRPB(M, K, torch.from_numpy(rp.astype(np.int64).astype(np.int32)).cuda(),
                              torch.from_numpy(cl.view(np.int32).copy()).cuda(), torch.from_numpy(vl.copy()).cuda(),
                              quad_layout=int(rng.choice([0, 1, 2])))
        else:
            h = cs.HRPB(M, K, rp, cl, vl)
        for rep in range(4):
            kw = dict(path=int(rng.choice([cs.PATH_AUTO, cs.PATH_AUTO, cs.PATH_BRICK, cs.PATH_ROWS])), mfma_shape=int(rng.choice([0, 1, 2])),
                      pipeline=int(rng.choice([0, 0, 1, 2])), chunk_order=int(rng.choice([0, 0, 1, 2, 3])),
                      slots=int(rng.choice([0, 0, 0, 1, 3, 7, 64])), max_chunk_blocks=int(rng.choice([0, 0, 1, 2, 5])),
                      operand_residency=int(rng.choice([0, 1, 2])), brick_groups=int(rng.choice([0, 0, 1, 2])),
                      min_reuse=float(rng.choice([0.0, 0.0, 0.5, 4.0])), max_row_nnz=int(rng.choice([0, 0, 4, 64])))
            how = ("run", "static", "scratch")[int(rng.integers(0, 3))]
            what = "%s case %d: M %d K %d nnz %d N %d, %s, %s" % (kind, case, M, K, len(cl), N, how, kw)
            p = cs.SPMM_TC(h, N, **kw)
            dC = torch.full((M, N), float("nan"), device="cuda")
            if how == "static" and p.scratch_bytes > cs.STATIC_SCRATCH_BYTES:
                how = "run"
            if how == "run":
                p.run(dB, dC)
            elif how == "static":
                p.run_static(dB, dC)
            else:
                p.run_scratch(dB, dC, torch.empty(p.scratch_bytes // 4 + 64, device="cuda"))
            torch.cuda.synchronize()
            assert np.array_equal(dC.cpu().numpy(), ref), what + " -> " + p.kernel_name
            launches += 1
    assert launches == 40


def test_random_special_paths_equal_the_oracle(cs, orc, torch_cuda):
    """The same on the paths a default plan never takes: the bf16x3 brick kernel (small integers split into an exact
    high part and a zero low part), the hub kernel on strip lists, the hybrid call under both split rules, and the
    three plain CSR kernels."""
    torch = torch_cuda
    rng = np.random.default_rng(77001)
    for case in range(14):
        kind = KINDS[case % len(KINDS)]
        M, K, rp, cl, vl = _matrix(rng, kind)
        N = int(rng.choice(WIDTHS[:-1]))
        if M * N > (1 << 20):
            N = max(1, (1 << 20) // M)
        B = rng.integers(-3, 4, (K, N)).astype(np.float32)
        ref = orc.spmm_csr(rp, cl, vl, B)
        dB = torch.from_numpy(B).cuda()
        h = cs.HRPB(M, K, rp, cl, vl)
        strips = cs.DeviceHRPB(M, K, torch.from_numpy(rp.astype(np.int64).astype(np.int32)).cuda(),
                               torch.from_numpy(cl.view(np.int32).copy()).cuda(), torch.from_numpy(vl.copy()).cuda(), quad_layout=2)
        for handle, kw in ((h, dict(precision=cs.PREC_BF16X3)), (h, dict(precision=cs.PREC_BF16X3, slots=3, max_chunk_blocks=1)),
                           (strips, dict(path=cs.PATH_BRICK, mfma_shape=2, hub_rows=int(rng.choice([1, 8, 64, 256]))))):
            p = cs.SPMM_TC(handle, N, **kw)
            dC = torch.full((M, N), float("nan"), device="cuda")
            p.run(dB, dC)
            torch.cuda.synchronize()
            assert np.array_equal(dC.cpu().numpy(), ref), (kind, case, M, K, N, kw, p.kernel_name)
        csr = cs.CSR_Matrix(nrows=M, ncols=K, rowPtr=rp.astype(np.int32), cols=cl.astype(np.int32), values=vl)
        for kw in (dict(), dict(nnz_threshold=int(rng.integers(1, 60))),
                   dict(mode=cs.HYBRID_CLASSIFIER, deviation_threshold=float(rng.random()), underload_dominance=float(rng.random()))):
            dC = torch.full((M, N), float("nan"), device="cuda")
            cs.HybridSpMM(csr, **kw).spmm(dB, dC)
            torch.cuda.synchronize()
            assert np.array_equal(dC.cpu().numpy(), ref), (kind, case, M, K, N, kw)
        for alg in (0, 1, 2):
            dC = torch.full((M, N), float("nan"), device="cuda")
            cs.csr_spmm_dev(alg, h, dB, dC)
            torch.cuda.synchronize()
            assert np.array_equal(dC.cpu().numpy(), ref), (kind, case, M, K, N, "csr kernel", alg)
