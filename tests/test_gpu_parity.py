"""GPU parity tests: the HIP path, called through the C ABI, against the CPU oracle on the
same seeded inputs.

Tolerances (fp32 MFMA / fp32 FMA paths):
  * componentwise backward error  max |dC_ij| / sum_k |a_ik||b_kj|  <= 2e-6
    (a row with n nonzeros summed in any order in fp32 is within n * 2^-24 of exact);
  * the reference's own metric (inc.h:84-109), max relative error over non-zero reference
    entries, <= 1e-5 on inputs without cancellation (A = 1, B in [0,1), the only regime the
    reference ever evaluated it in, run.cu:24-27 + IO.cu:68);
  * exact equality where every product and partial sum is exactly representable.
"""
import numpy as np
import pytest

from helpers import csr_from_dense, random_csr

pytestmark = pytest.mark.gpu

BERR = 2e-6


def _run(cs, torch, h, B, **kw):
    N = B.shape[1]
    dB = torch.from_numpy(np.ascontiguousarray(B)).cuda()
    dC = torch.full((h.M, N), float("nan"), device="cuda")      # every element must be written
    plan = cs.SPMM_TC(h, N, **kw)
    plan.run(dB, dC)
    torch.cuda.synchronize()
    return dC.cpu().numpy(), plan


def _paths(cs):
    mfma = dict(path=cs.PATH_BRICK)
    return [("quad", dict(mfma, mfma_shape=2)),
            ("brick_rolling", dict(mfma, mfma_shape=1, pipeline=1)),
            ("brick_rolling_g2", dict(mfma, mfma_shape=1, pipeline=1, brick_groups=2)),
            ("brick_pipelined", dict(mfma, mfma_shape=1, pipeline=2)),
            ("brick_pipelined_g2", dict(mfma, mfma_shape=1, pipeline=2, brick_groups=2)),
            ("mfma_default", mfma), ("rows", dict(path=cs.PATH_ROWS)), ("auto", dict())]


def test_device_is_gfx950(cs, torch_cuda):
    info = cs.device_info()
    assert info["arch"].startswith("gfx950") and info["wave_size"] == 64 and info["num_cus"] > 0


@pytest.mark.parametrize("cfg,scale", [(1, 1.0), (2, 1 / 16.0), (3, 1 / 16.0), (4, 1 / 32.0), (5, 1 / 128.0)])
def test_configs_against_oracle(cs, orc, torch_cuda, cfg, scale):
    A = cs.gen_config(cfg, scale)
    N = cs.CONFIGS[cfg]["N"]
    B = cs.gen_dense(cs.SEED_BASE + 100 + cfg, A.K, N, 2)
    ref = orc.spmm_csr(A.rowPtr, A.cols, A.vals, B)
    h = cs.HRPB(A.M, A.K, A.rowPtr, A.cols, A.vals)
    for name, kw in _paths(cs):
        out, _ = _run(cs, torch_cuda, h, B, **kw)
        err = cs.backward_error(A.rowPtr, A.cols, A.vals, B, ref, out)
        assert np.isfinite(out).all() and err <= BERR, (cfg, name, err)


@pytest.mark.parametrize("N", [1, 3, 16, 20, 32, 48, 64, 100, 128, 130, 131, 192, 256, 320, 512, 1024])
def test_every_width(cs, orc, torch_cuda, N):
    rng = np.random.default_rng(N)
    M, K = 160, 256
    rp, cl, vl = random_csr(rng, M, K, density=0.08)
    B = rng.standard_normal((K, N)).astype(np.float32)
    ref = orc.spmm_csr(rp, cl, vl, B)
    h = cs.HRPB(M, K, rp, cl, vl)
    for name, kw in _paths(cs):
        out, plan = _run(cs, torch_cuda, h, B, **kw)
        err = cs.backward_error(rp, cl, vl, B, ref, out)
        assert err <= BERR, (N, name, err, plan.info)


def test_exact_cases(cs, torch_cuda):
    torch = torch_cuda
    rng = np.random.default_rng(3)
    K, N = 128, 64
    B = rng.standard_normal((K, N)).astype(np.float32)
    # A = I  =>  C = B bit for bit
    I = csr_from_dense(np.eye(K, dtype=np.float32))
    h = cs.HRPB(K, K, *I)
    for name, kw in _paths(cs):
        out, _ = _run(cs, torch, h, B, **kw)
        assert (out == B).all(), name
    # all-ones A and B  =>  row nonzero counts, exact in any summation order
    rp, cl, vl = random_csr(rng, 96, K, density=0.3, values="ones")
    h = cs.HRPB(96, K, rp, cl, vl)
    ones = np.ones((K, N), np.float32)
    for name, kw in _paths(cs):
        out, _ = _run(cs, torch, h, ones, **kw)
        assert (out == np.diff(rp.astype(np.int64))[:, None]).all(), name
    # one-hot B picks out a column of A (catches a transposed or permuted operand)
    rp, cl, vl = random_csr(rng, 64, K, density=0.2, values="ints")
    h = cs.HRPB(64, K, rp, cl, vl)
    E = np.zeros((K, 16), np.float32)
    picks = rng.choice(K, 16, replace=False)
    E[picks, np.arange(16)] = 1
    D = np.zeros((64, K), np.float32)
    for r in range(64):
        D[r, cl[rp[r]:rp[r + 1]]] = vl[rp[r]:rp[r + 1]]
    for name, kw in _paths(cs):
        out, _ = _run(cs, torch, h, E, **kw)
        assert (out == D[:, picks]).all(), name
    # small integers: equal to the oracle's HRPB-stream SpMM and to CSR exactly


def test_integer_inputs_equal_oracle_bit_for_bit(cs, orc, torch_cuda):
    rng = np.random.default_rng(17)
    M, K, N = 256, 320, 96
    rp, cl, vl = random_csr(rng, M, K, density=0.05, values="ints")
    B = rng.integers(-4, 5, (K, N)).astype(np.float32)
    ref = orc.spmm_csr(rp, cl, vl, B)
    h = cs.HRPB(M, K, rp, cl, vl)
    assert (orc.spmm_hrpb(h.as_dict(), B) == ref).all()
    for name, kw in _paths(cs):
        out, _ = _run(cs, torch_cuda, h, B, **kw)
        assert (out == ref).all(), name


def test_reference_regime_metric(cs, orc, torch_cuda):
    """A = 1 everywhere it is non-zero, B uniform in [0,1): the reference's own check."""
    import os
    from test_oracle_pins import GOLD
    r = cs.MTX_READER(os.path.join(GOLD, "G67.mtx"))
    for N in (32, 128, 512):                     # run.cu:16
        B = cs.gen_dense(5 + N, r.K, N, 0)
        ref = orc.spmm_csr(r.rowPtr, r.cols, r.vals, B)
        h = cs.HRPB(r.M, r.K, r.rowPtr, r.cols, r.vals)
        for name, kw in _paths(cs):
            out, _ = _run(cs, torch_cuda, h, B, **kw)
            assert cs.check_gemm_correctness_coo(ref, out) <= 1e-5, (N, name)


@pytest.mark.parametrize("cfg,scale", [(1, 1.0), (2, 1.0), (3, 1.0), (4, 1.0), (5, 1 / 8.0)])
def test_literal_tolerance_on_every_config_pattern(cs, orc, torch_cuda, cfg, scale):
    """The reference's metric (inc.h:84-109) at its literal fp32 bar, 1e-5, on the sparsity pattern of every
    benchmark configuration in the regime the reference evaluates it in: values |a| (no cancellation) and
    B uniform in [0,1) (run.cu:24-27).  Every kernel path; the backward error is recorded beside it."""
    A = cs.gen_config(cfg, scale)
    vals = np.abs(A.vals)
    N = cs.CONFIGS[cfg]["N"]
    B = cs.gen_dense(cs.SEED_BASE + 300 + cfg, A.K, N, 0)
    ref = orc.spmm_csr(A.rowPtr, A.cols, vals, B)
    h = cs.HRPB(A.M, A.K, A.rowPtr, A.cols, vals)
    worst = {}
    big = A.nnz > 4_000_000
    for name, kw in _paths(cs):
        if big and name in ("brick_rolling_g2", "brick_pipelined_g2", "mfma_default"):
            continue                                   # the largest pattern: one variant per kernel family is enough
        out, _ = _run(cs, torch_cuda, h, B, **kw)
        worst[name] = cs.check_gemm_correctness_coo(ref, out)
        assert worst[name] <= 1e-5, (cfg, name, worst[name])
    out, _ = _run(cs, torch_cuda, h, B)
    print("cfg%d literal metric max %.3g, backward error %.3g" %
          (cfg, max(worst.values()), cs.backward_error(A.rowPtr, A.cols, vals, B, ref, out)))


@pytest.mark.parametrize("cfg,scale", [(1, 1.0), (2, 1 / 4.0), (3, 1 / 4.0), (4, 1 / 4.0), (5, 1 / 32.0)])
@pytest.mark.parametrize("N", [32, 128, 512])
def test_literal_tolerance_at_the_reference_widths(cs, orc, torch_cuda, cfg, scale, N):
    """The three feature widths of the reference's driver (run.cu:16) on each (scaled) configuration pattern."""
    A = cs.gen_config(cfg, scale)
    vals = np.abs(A.vals)
    B = cs.gen_dense(cs.SEED_BASE + 400 + cfg + N, A.K, N, 0)
    ref = orc.spmm_csr(A.rowPtr, A.cols, vals, B)
    h = cs.HRPB(A.M, A.K, A.rowPtr, A.cols, vals)
    for name, kw in _paths(cs):
        out, _ = _run(cs, torch_cuda, h, B, **kw)
        m = cs.check_gemm_correctness_coo(ref, out)
        assert m <= 1e-5, (cfg, N, name, m)


BERR_BF16X3 = 5e-5      # three bf16 products per block: what is dropped is below 2^-16 of each product (measured 2e-5)


def test_bf16x3_precision_path(cs, orc, torch_cuda):
    """CUTE_PREC_BF16X3: the brick kernel on the bf16 matrix pipeline.  Backward error in the 2^-15 class on every
    benchmark pattern, the reference's metric within its reduced-precision bar of 1e-3 (in fact 1e-4) in the
    reference's regime, exact on small integers (their hi parts are exact and their lo parts zero), every
    width, cut panels, and fp32 wherever the kernel does not exist."""
    for cfg, scale in [(1, 1.0), (2, 1 / 16.0), (3, 1 / 8.0), (4, 1 / 32.0), (5, 1 / 128.0)]:
        A = cs.gen_config(cfg, scale)
        N = cs.CONFIGS[cfg]["N"]
        B = cs.gen_dense(cs.SEED_BASE + 100 + cfg, A.K, N, 2)
        ref = orc.spmm_csr(A.rowPtr, A.cols, A.vals, B)
        h = cs.HRPB(A.M, A.K, A.rowPtr, A.cols, A.vals)
        for kw in (dict(path=cs.PATH_BRICK), dict(path=cs.PATH_BRICK, brick_groups=1), dict()):
            out, plan = _run(cs, torch_cuda, h, B, precision=cs.PREC_BF16X3, **kw)
            err = cs.backward_error(A.rowPtr, A.cols, A.vals, B, ref, out)
            assert np.isfinite(out).all() and err <= BERR_BF16X3, (cfg, kw, err)
            if "path" in kw and N > 32:                             # narrower products take two-column tiles, in fp32
                assert plan.info["precision"] == cs.PREC_BF16X3 and plan.kernel_name == "hrpb_brick_bf16x3"
                assert err > 1e-6                                   # it really is the reduced-precision kernel
        # the reference's regime: A = |a|, B in [0,1)
        vals = np.abs(A.vals)
        B0 = cs.gen_dense(cs.SEED_BASE + 500 + cfg, A.K, N, 0)
        ref0 = orc.spmm_csr(A.rowPtr, A.cols, vals, B0)
        h0 = cs.HRPB(A.M, A.K, A.rowPtr, A.cols, vals)
        out, _ = _run(cs, torch_cuda, h0, B0, precision=cs.PREC_BF16X3, path=cs.PATH_BRICK)
        assert cs.check_gemm_correctness_coo(ref0, out) <= 1e-4, cfg
    rng = np.random.default_rng(23)
    M, K = 160, 256
    rp, cl, vl = random_csr(rng, M, K, density=0.08, values="ints")
    h = cs.HRPB(M, K, rp, cl, vl)
    for N in (4, 20, 64, 100, 128, 192, 260, 512):
        B = rng.integers(-4, 5, (K, N)).astype(np.float32)
        ref = orc.spmm_csr(rp, cl, vl, B)
        out, plan = _run(cs, torch_cuda, h, B, precision=cs.PREC_BF16X3, path=cs.PATH_BRICK)
        assert plan.info["precision"] == (cs.PREC_BF16X3 if N > 32 else cs.PREC_FP32) and (out == ref).all(), N
    # widths the kernel does not exist for (N not a multiple of 4), the quad kernel, the pipelined brick kernel: fp32
    B = rng.standard_normal((K, 30)).astype(np.float32)
    out, plan = _run(cs, torch_cuda, h, B, precision=cs.PREC_BF16X3, path=cs.PATH_BRICK)
    assert plan.info["precision"] == cs.PREC_FP32 and cs.backward_error(rp, cl, vl, B, orc.spmm_csr(rp, cl, vl, B), out) <= BERR
    B = rng.standard_normal((K, 64)).astype(np.float32)
    for kw in (dict(mfma_shape=2), dict(pipeline=2)):
        out, plan = _run(cs, torch_cuda, h, B, precision=cs.PREC_BF16X3, path=cs.PATH_BRICK, **kw)
        assert plan.info["precision"] == cs.PREC_FP32 and cs.backward_error(rp, cl, vl, B, orc.spmm_csr(rp, cl, vl, B), out) <= BERR
    # cut panels: partial tiles added in fp32, in a fixed order
    M, K, N = 512, 4096, 128
    rp, cl, vl = random_csr(rng, M, K, row_nnz=lambda r: 1500 if r in (5, 300) else 4)
    B = rng.standard_normal((K, N)).astype(np.float32)
    ref = orc.spmm_csr(rp, cl, vl, B)
    h = cs.HRPB(M, K, rp, cl, vl)
    outs = []
    for kw in (dict(), dict(max_chunk_blocks=3), dict(max_chunk_blocks=3)):
        out, plan = _run(cs, torch_cuda, h, B, precision=cs.PREC_BF16X3, path=cs.PATH_BRICK, **kw)
        assert plan.info["numAtomicChunks"] > 0 and cs.backward_error(rp, cl, vl, B, ref, out) <= BERR_BF16X3
        outs.append(out)
    assert (outs[1] == outs[2]).all()
    with pytest.raises(cs.CuteError):
        cs.SPMM_TC(h, N, precision=2)


def test_non_finite_b_rows(cs, torch_cuda):
    """What an Inf in B does, path by path.  The row kernel is exact: only rows of C that reference the B row see it.
    The MFMA kernels multiply stored zeros into real B rows (as the reference's kernel does, kernel.cu:26-27,149):
    the Inf spreads as NaN over the rows that share a panel (brick kernels) or a 4-row group (quad kernels) with a
    row that references it -- never further -- and an Inf in B row 0 reaches every panel that pads its last block."""
    rng = np.random.default_rng(5)
    M, K, N = 64, 128, 64
    # three entries per row, none in column 0, column 77 referenced by row 21 only
    pool = np.array([c for c in range(1, K) if c != 77])
    cols = [np.sort(rng.choice(pool, 3, replace=False)) for _ in range(M)]
    cols[21] = np.sort(np.append(rng.choice(pool, 2, replace=False), 77))
    rp2 = (3 * np.arange(M + 1)).astype(np.uint32)
    cl2 = np.concatenate(cols).astype(np.uint32)
    vl2 = rng.standard_normal(3 * M).astype(np.float32)
    h = cs.HRPB(M, K, rp2, cl2, vl2)
    B = rng.standard_normal((K, N)).astype(np.float32)
    B[77, 5] = np.inf
    out, _ = _run(cs, torch_cuda, h, B, path=cs.PATH_ROWS)
    bad = ~np.isfinite(out)
    assert bad[21, 5] and bad.sum() == 1
    for name, kw, rows_hit in (("brick", dict(path=cs.PATH_BRICK, mfma_shape=1), range(16, 32)),
                               ("brick_pipelined", dict(path=cs.PATH_BRICK, mfma_shape=1, pipeline=2), range(16, 32)),
                               ("quad", dict(path=cs.PATH_BRICK, mfma_shape=2), range(20, 24))):
        out, _ = _run(cs, torch_cuda, h, B, **kw)
        bad = ~np.isfinite(out)
        assert bad[21, 5] and set(np.nonzero(bad.any(1))[0]) <= set(rows_hit) and not bad[:, :5].any() and not bad[:, 6:].any(), name
    # B row 0 is what padding slots point at
    B[77, 5] = 1.0
    B[0, 9] = np.inf
    out, _ = _run(cs, torch_cuda, h, B, path=cs.PATH_ROWS)
    assert np.isfinite(out).all()                                  # no row references column 0
    out, _ = _run(cs, torch_cuda, h, B, path=cs.PATH_BRICK, mfma_shape=1)
    assert not np.isfinite(out[:, 9]).all() and np.isfinite(np.delete(out, 9, axis=1)).all()


def test_edge_shapes(cs, orc, torch_cuda):
    from test_oracle_pins import _edge_cases
    rng = np.random.default_rng(0)
    for name, (M, K, rp, cl, vl) in sorted(_edge_cases().items()):
        B = rng.standard_normal((K, 64)).astype(np.float32)
        ref = orc.spmm_csr(rp, cl, vl, B)
        h = cs.HRPB(M, K, rp, cl, vl)
        for pname, kw in _paths(cs):
            out, _ = _run(cs, torch_cuda, h, B, **kw)
            assert cs.backward_error(rp, cl, vl, B, ref, out) <= BERR, (name, pname)
            assert (out[np.diff(rp.astype(np.int64)) == 0] == 0).all()      # empty rows are written as zeros


def test_split_panels_add_up(cs, orc, torch_cuda):
    """A few very long panels among short ones: the planner cuts them and the pieces add up."""
    rng = np.random.default_rng(8)
    M, K, N = 512, 4096, 128
    rp, cl, vl = random_csr(rng, M, K, row_nnz=lambda r: 1500 if r in (5, 300) else 4)
    B = rng.standard_normal((K, N)).astype(np.float32)
    ref = orc.spmm_csr(rp, cl, vl, B)
    h = cs.HRPB(M, K, rp, cl, vl)
    for shape in (1, 2):
        out, plan = _run(cs, torch_cuda, h, B, path=cs.PATH_BRICK, mfma_shape=shape)
        assert plan.info["numAtomicChunks"] > 0
        assert cs.backward_error(rp, cl, vl, B, ref, out) <= BERR
        # forcing tiny chunks everywhere, and the reference's own partition arithmetic
        for kw in (dict(max_chunk_blocks=1), dict(max_chunk_blocks=3), dict(slots=64), dict(slots=864)):
            out, plan = _run(cs, torch_cuda, h, B, path=cs.PATH_BRICK, mfma_shape=shape, **kw)
            assert cs.backward_error(rp, cl, vl, B, ref, out) <= BERR, (shape, kw)
    # a second launch on the same output buffer must not accumulate on top of the first, and the pieces of a
    # cut panel are added in a fixed order: the same product gives the same bits every time
    import torch
    dB = torch.from_numpy(B).cuda()
    for shape in (1, 2):
        dC = torch.zeros((M, N), device="cuda")
        plan = cs.SPMM_TC(h, N, path=cs.PATH_BRICK, mfma_shape=shape, max_chunk_blocks=2)
        plan.run(dB, dC)
        plan.run(dB, dC)
        torch.cuda.synchronize()
        first = dC.cpu().numpy().copy()
        assert cs.backward_error(rp, cl, vl, B, ref, first) <= BERR
        for _ in range(3):
            dC.fill_(float("nan"))
            plan.run(dB, dC)
            torch.cuda.synchronize()
            assert (dC.cpu().numpy() == first).all()


def test_work_items_dealt_by_length(cs, orc, torch_cuda):
    """The order in which the MFMA work items are listed decides where they run, not what they compute: panel
    order, the planner's choice and a forced deal give the same bits, with panels of very different lengths,
    with cut panels (partial tiles) among them, for one and for several column slabs, alone and fused with rows."""
    rng = np.random.default_rng(21)
    M, K = 4096, 4096
    lengths = rng.integers(1, 40, M // 16)
    rp, cl, vl = random_csr(rng, M, K, row_nnz=lambda r: 700 if r in (40, 2000) else int(lengths[r // 16]))
    h = cs.HRPB(M, K, rp, cl, vl)
    for N in (32, 128, 200):
        B = rng.standard_normal((K, N)).astype(np.float32)
        ref = orc.spmm_csr(rp, cl, vl, B)
        for kw in (dict(path=cs.PATH_BRICK, mfma_shape=1), dict(path=cs.PATH_BRICK, mfma_shape=2), dict()):
            outs = {}
            for order in (1, 0, 2, 3):
                outs[order], plan = _run(cs, torch_cuda, h, B, chunk_order=order, **kw)
                assert plan.info["dealtChunks"] == (0 if order == 1 else 1 if order == 2 else 2 if order == 3 else plan.info["dealtChunks"])
                if order == 1 and "path" in kw:
                    assert plan.info["numAtomicChunks"] > 0
            assert cs.backward_error(rp, cl, vl, B, ref, outs[1]) <= BERR, (N, kw)
            assert (outs[0] == outs[1]).all() and (outs[2] == outs[1]).all() and (outs[3] == outs[1]).all(), (N, kw)
    # several work items per SIMD, of very different lengths, all on the device at once: the planner deals them by itself
    M3, K3 = 32768, 2048
    lengths = rng.integers(1, 24, M3 // 16)
    rp3, cl3, vl3 = random_csr(rng, M3, K3, row_nnz=lambda r: int(lengths[r // 16]))
    h3 = cs.HRPB(M3, K3, rp3, cl3, vl3)
    B3 = rng.standard_normal((K3, 64)).astype(np.float32)
    ref3 = orc.spmm_csr(rp3, cl3, vl3, B3)
    for shape in (1, 2):
        out, plan = _run(cs, torch_cuda, h3, B3, path=cs.PATH_BRICK, mfma_shape=shape)
        assert plan.info["dealtChunks"] == 1 and plan.info["numChunks"] >= 2048
        assert cs.backward_error(rp3, cl3, vl3, B3, ref3, out) <= BERR
        same, plan = _run(cs, torch_cuda, h3, B3, path=cs.PATH_BRICK, mfma_shape=shape, chunk_order=1)
        assert plan.info["dealtChunks"] == 0 and (same == out).all()
    # a launch larger than the device with a heavy tail of long panels: the planner lists the long items first by
    # itself, and cuts at a multiple of the per-slot share; same bits as panel order
    M4, K4 = 65536, 8192
    hub = set(int(x) for x in rng.choice(M4, 40, replace=False))
    rp4, cl4, vl4 = random_csr(rng, M4, K4, row_nnz=lambda r: 3000 if r in hub else 3)
    h4 = cs.HRPB(M4, K4, rp4, cl4, vl4)
    B4 = rng.standard_normal((K4, 192)).astype(np.float32)
    ref4 = orc.spmm_csr(rp4, cl4, vl4, B4)
    for shape in (1, 2):
        out, plan = _run(cs, torch_cuda, h4, B4, path=cs.PATH_BRICK, mfma_shape=shape)
        assert plan.info["dealtChunks"] == 2 and plan.info["numAtomicChunks"] > 0, plan.info
        assert cs.backward_error(rp4, cl4, vl4, B4, ref4, out) <= BERR
        same, plan = _run(cs, torch_cuda, h4, B4, path=cs.PATH_BRICK, mfma_shape=shape, chunk_order=1)
        assert plan.info["dealtChunks"] == 0 and (same == out).all()
    # equal panels stay in panel order
    rp2, cl2, vl2 = random_csr(rng, 1024, 1024, row_nnz=lambda r: 8)
    h2 = cs.HRPB(1024, 1024, rp2, cl2, vl2)
    _, plan = _run(cs, torch_cuda, h2, rng.standard_normal((1024, 64)).astype(np.float32), path=cs.PATH_BRICK, mfma_shape=1)
    assert plan.info["dealtChunks"] == 0
    with pytest.raises(cs.CuteError):
        cs.SPMM_TC(h2, 64, chunk_order=4)
    # where the operands live only changes which MFMA kernel runs
    A5 = cs.gen_config(2, 1 / 16.0)
    h5 = cs.HRPB(A5.M, A5.K, A5.rowPtr, A5.cols, A5.vals)
    B5 = rng.standard_normal((A5.K, 128)).astype(np.float32)
    ref5 = orc.spmm_csr(A5.rowPtr, A5.cols, A5.vals, B5)
    # (unknown is planned like "from HBM": a product on fresh data finds its operands there whatever their size)
    for res, name in ((0, "hrpb_brick_f32_rolling"), (1, "hrpb_brick_f32_rolling"), (2, "hrpb_quad_f32")):
        out, plan = _run(cs, torch_cuda, h5, B5, operand_residency=res)
        assert plan.kernel_name == name, (res, plan.kernel_name)
        assert cs.backward_error(A5.rowPtr, A5.cols, A5.vals, B5, ref5, out) <= BERR
    with pytest.raises(cs.CuteError):
        cs.SPMM_TC(h5, 128, operand_residency=3)


def _stencil5(g):
    """5-point stencil on a g x g grid (rows padded to a multiple of 16), the shape of the reference's `obstclae`."""
    idx = np.arange(g * g).reshape(g, g)
    rows, cols = [], []
    for di, dj in ((0, 0), (-1, 0), (1, 0), (0, -1), (0, 1)):
        src = idx[max(0, -di):g - max(0, di), max(0, -dj):g - max(0, dj)]
        dst = idx[max(0, di):g - max(0, -di), max(0, dj):g - max(0, -dj)]
        rows.append(src.ravel())
        cols.append(dst.ravel())
    r, c = np.concatenate(rows), np.concatenate(cols)
    o = np.lexsort((c, r))
    r, c = r[o], c[o]
    M = ((g * g + 15) // 16) * 16
    rp = np.zeros(M + 1, np.int64)
    np.add.at(rp, r + 1, 1)
    vals = np.random.default_rng(g).uniform(-1, 1, len(c)).astype(np.float32)
    return M, np.cumsum(rp).astype(np.uint32), c.astype(np.uint32), vals


def test_default_kernel_choice(cs, orc, torch_cuda):
    """The planner's default on the headline shape, pinned: the 65 536-row 9-point stencil at N = 128 goes to the
    brick kernel unless the caller says that its operands stay cache-resident (its quad lists ask for 1.25 B-row
    pieces per piece the brick kernel asks for); a 5-point stencil (1.0) stays on the quad kernel either way."""
    A = cs.gen_config(2)
    h = cs.HRPB(A.M, A.K, A.rowPtr, A.cols, A.vals)
    assert cs.SPMM_TC(h, 128).kernel_name == "hrpb_brick_f32_rolling"
    assert cs.SPMM_TC(h, 128, operand_residency=1).kernel_name == "hrpb_brick_f32_rolling"
    assert cs.SPMM_TC(h, 128, operand_residency=2).kernel_name == "hrpb_quad_f32"
    assert cs.SPMM_TC(h, 1024, operand_residency=2).kernel_name == "hrpb_brick_f32_rolling"   # 512 MiB: no cache holds that
    # the banded benchmark matrix (an eighth of it) at its own width: wide and large, but its panels read a window of B the
    # L2s hold, so the rule for wide products of short rows leaves it with the row kernel
    A5 = cs.gen_config(5, 1 / 8.0)
    assert cs.SPMM_TC(cs.HRPB(A5.M, A5.K, A5.rowPtr, A5.cols, A5.vals), 256).kernel_name == "csr_rows_batched"
    M, rp, cl, vl = _stencil5(200)
    h5 = cs.HRPB(M, M, rp, cl, vl)
    B = np.random.default_rng(5).standard_normal((M, 128)).astype(np.float32)
    ref = orc.spmm_csr(rp, cl, vl, B)
    for res in (0, 1, 2):
        out, plan = _run(cs, torch_cuda, h5, B, operand_residency=res)
        assert plan.info["mfmaShape"] == 2 and plan.kernel_name.startswith("hrpb_quad"), (res, plan.kernel_name)
        assert cs.backward_error(rp, cl, vl, B, ref, out) <= BERR


def test_a_handful_of_mfma_panels_goes_to_the_row_kernel(cs, orc, torch_cuda):
    """9-point stencil at N = 32: only the panels on the grid's boundary (fewer columns, more reuse) would pass the bar
    for the matrix cores -- 16 of 1 024 -- and the fused launch they would cause costs the other panels more than they
    gain, so the whole matrix goes to the row kernel.  A panel with a row too long for a lane group keeps its MFMA kernel
    (and the plan its fused launch).  Same product either way."""
    A = cs.gen_matrix(2, 0xC07E5B02, 128)
    h = cs.HRPB(A.M, A.K, A.rowPtr, A.cols, A.vals)
    B = np.random.default_rng(8).standard_normal((A.K, 32)).astype(np.float32)
    ref = orc.spmm_csr(A.rowPtr, A.cols, A.vals, B)
    out, plan = _run(cs, torch_cuda, h, B)
    assert plan.kernel_name == "csr_rows_batched" and plan.info["numBrickPanels"] == 0 and plan.info["numRowPanelsSparse"] == A.M // 16
    assert cs.backward_error(A.rowPtr, A.cols, A.vals, B, ref, out) <= BERR
    forced, fplan = _run(cs, torch_cuda, h, B, path=cs.PATH_BRICK)
    assert fplan.info["numBrickPanels"] == A.M // 16 and cs.backward_error(A.rowPtr, A.cols, A.vals, B, ref, forced) <= BERR
    # the same matrix with one row of 64 entries: its panel cannot go to the row kernel, so the plan stays mixed
    rp, cl, vl = np.asarray(A.rowPtr).copy(), np.asarray(A.cols), np.asarray(A.vals)
    r, long_row = 4000, 64
    cols2 = np.concatenate([cl[:rp[r]], np.arange(long_row, dtype=np.uint32) * 3, cl[rp[r + 1]:]])
    vals2 = np.concatenate([vl[:rp[r]], np.ones(long_row, np.float32), vl[rp[r + 1]:]])
    rp2 = rp.copy()
    rp2[r + 1:] += np.uint32(long_row - (rp[r + 1] - rp[r]))
    h2 = cs.HRPB(A.M, A.K, rp2, cols2, vals2)
    ref2 = orc.spmm_csr(rp2, cols2, vals2, B)
    out2, plan2 = _run(cs, torch_cuda, h2, B)
    assert plan2.info["numBrickPanels"] >= 1 and plan2.info["numRowPanelsSparse"] >= A.M // 16 - 20, plan2.info
    assert cs.backward_error(rp2, cols2, vals2, B, ref2, out2) <= BERR
    # and the other way round: the FEM benchmark matrix at N = 16, where 53 of 3 000 panels (0.5 % of the entries) would go
    # to the row kernel and cost a fused launch -- they join the brick kernel; a stricter bar that sends a good part
    # of the panels to the row kernel keeps the plan mixed
    F = cs.gen_config(3)
    hf = cs.HRPB(F.M, F.K, F.rowPtr, F.cols, F.vals)
    Bf = np.random.default_rng(9).standard_normal((F.K, 16)).astype(np.float32)
    reff = orc.spmm_csr(F.rowPtr, F.cols, F.vals, Bf)
    outf, planf = _run(cs, torch_cuda, hf, Bf)
    assert planf.kernel_name == "hrpb_brick_f32_rolling" and planf.info["numRowPanelsSparse"] == 0, planf.info
    assert cs.backward_error(F.rowPtr, F.cols, F.vals, Bf, reff, outf) <= BERR
    shares = [cs.SPMM_TC(hf, 64, min_reuse=bar, max_row_nnz=200).info for bar in (1.6, 2.0, 2.4, 2.8, 3.2)]
    assert any(i["numRowPanelsSparse"] > 100 and i["numBrickPanels"] > 100 for i in shares), [(i["numRowPanelsSparse"], i["numBrickPanels"]) for i in shares]


def test_panels_with_one_long_row_leave_the_row_kernel_at_narrow_widths(cs, orc, torch_cuda):
    """Rows of 3 entries with one row of 40 in every other panel, all at random columns (no reuse for the matrix cores):
    up to N = 128 several rows share a wavefront of the row kernel, which would wait for the long one, so those panels go
    to the MFMA kernel; at N = 256 (one row per wavefront) and for evenly long rows (all 40) they stay."""
    rng = np.random.default_rng(12)
    M, K = 4096, 16384
    rp, cl, vl = random_csr(rng, M, K, row_nnz=lambda r: 40 if r % 32 == 5 else 3)
    h = cs.HRPB(M, K, rp, cl, vl)
    for N, uneven_to_mfma in ((32, True), (128, True), (256, False)):
        B = rng.standard_normal((K, N)).astype(np.float32)
        out, plan = _run(cs, torch_cuda, h, B)
        if uneven_to_mfma:
            assert plan.info["numBrickPanels"] == M // 32 and plan.info["numRowPanelsSparse"] == M // 32, (N, plan.info)
        else:
            assert plan.info["numBrickPanels"] == 0, (N, plan.info)
        assert cs.backward_error(rp, cl, vl, B, orc.spmm_csr(rp, cl, vl, B), out) <= BERR
        # the caller's own limit on row lengths switches the rule off
        assert cs.SPMM_TC(h, N, max_row_nnz=48).info["numBrickPanels"] == 0
    rp2, cl2, vl2 = random_csr(rng, 1024, K, row_nnz=40)
    assert cs.SPMM_TC(cs.HRPB(1024, K, rp2, cl2, vl2), 32).info["numBrickPanels"] == 0


def test_wide_products_of_short_rows_go_to_the_quad_kernel(cs, orc, torch_cuda):
    """50 000 rows of 7 entries at random columns: no reuse for the matrix cores to harvest, and at N = 128 the row
    kernel keeps them; at N = 512 the launch is several times the device and the quad kernel's deeper pipeline wins
    (93 against 116 us), so the planner sends the panels there.  Same product either way."""
    rng = np.random.default_rng(3)
    M = K = 50000 // 16 * 16
    cols = np.sort(rng.integers(0, K - 64, (M, 7)), axis=1)
    cols += np.arange(7)[None, :] * 8 * (np.diff(cols, axis=1, prepend=-1) == 0).cumsum(1)      # make equal neighbours distinct
    cols = np.sort(cols, axis=1)
    keep = (np.diff(cols, axis=1) > 0).all(1)
    cols[~keep] = np.arange(7)[None, :] * 3 + 5                                                 # the rare leftover rows
    rp = (np.arange(M + 1) * 7).astype(np.uint32)
    cl, vl = cols.ravel().astype(np.uint32), rng.standard_normal(M * 7).astype(np.float32)
    h = cs.HRPB(M, K, rp, cl, vl)
    narrow = cs.SPMM_TC(h, 128)
    assert narrow.kernel_name == "csr_rows_batched" and narrow.info["numChunks"] == 0
    B = rng.standard_normal((K, 512)).astype(np.float32)
    out, wide = _run(cs, torch_cuda, h, B)
    assert wide.info["mfmaShape"] == 2 and wide.kernel_name.startswith("hrpb_quad"), wide.info
    assert wide.info["numBrickPanels"] > 0.9 * (M // 16)
    ref = orc.spmm_csr(rp, cl, vl, B)
    assert cs.backward_error(rp, cl, vl, B, ref, out) <= BERR
    same, rows = _run(cs, torch_cuda, h, B, path=cs.PATH_ROWS)
    assert cs.backward_error(rp, cl, vl, B, ref, same) <= BERR
    # a caller's own bar overrides the rule
    assert cs.SPMM_TC(h, 512, min_reuse=1.25).info["numChunks"] == 0


def test_hub_rows_staged_in_lds(cs, orc, torch_cuda):
    """cute_tunables.hub_rows: the quad kernel on strip lists as persistent work-groups with the most referenced B
    rows in LDS.  A graph-like matrix (a few columns in most rows, a few very long rows): exact on integers, within
    tolerance on real values, widths that are and are not multiples of the 64-column slab, cut strips included."""
    torch = torch_cuda
    rng = np.random.default_rng(31)
    M, K = 2048, 6000 // 16 * 16
    hubs = rng.choice(K, 40, replace=False)

    def row(r):
        n = 1500 if r in (9, 700, 701) else 4
        mine = set(int(x) for x in rng.choice(K, n, replace=False))
        mine.update(int(x) for x in hubs[rng.random(40) < 0.5])
        return sorted(mine)
    lists = [row(r) for r in range(M)]
    rp = np.concatenate([[0], np.cumsum([len(x) for x in lists])]).astype(np.uint32)
    cl = np.concatenate(lists).astype(np.uint32)
    for values, exact in (("ints", True), ("normal", False)):
        vl = rng.integers(-4, 5, len(cl)).astype(np.float32) if exact else rng.standard_normal(len(cl)).astype(np.float32)
        h = cs.HRPB(M, K, rp, cl, vl)
        assert h.upload(quad_layout=2)
        for N in (64, 128, 200):
            B = (rng.integers(-3, 4, (K, N)) if exact else rng.standard_normal((K, N))).astype(np.float32)
            ref = orc.spmm_csr(rp, cl, vl, B)
            for hub_rows in (256, 16, 1000):
                out, plan = _run(cs, torch, h, B, path=cs.PATH_BRICK, mfma_shape=2, hub_rows=hub_rows)
                assert plan.kernel_name == "hrpb_quad_hub_f32" and 0 < plan.info["hubRows"] <= min(hub_rows, 256), plan.info
                assert plan.info["numAtomicChunks"] > 0
                if exact:
                    assert (out == ref).all(), (N, hub_rows)
                else:
                    assert cs.backward_error(rp, cl, vl, B, ref, out) <= BERR, (N, hub_rows)
            # mixed with the row kernel (the planner's own split) and as the plain quad kernel: the same product
            out, plan = _run(cs, torch, h, B, hub_rows=128)
            assert cs.backward_error(rp, cl, vl, B, ref, out) <= BERR
    # plans that are not the quad kernel on strip lists ignore the tunable
    A = cs.gen_config(2, 1 / 16.0)
    h2 = cs.HRPB(A.M, A.K, A.rowPtr, A.cols, A.vals)
    assert cs.SPMM_TC(h2, 128, hub_rows=256).info["hubRows"] == 0


def test_layouts_are_built_when_first_needed(cs, orc, torch_cuda):
    """An upload sends the CSR arrays and the one MFMA layout the planner's default rules would use (none when every
    panel would go to the row kernel); a plan that asks for the other one builds it then, from the device copy of the
    CSR arrays -- also after the host arrays the format was made from have been overwritten."""
    rng = np.random.default_rng(12)
    A = cs.gen_config(2, 1 / 16.0)                                  # 9-point stencil: the default rules pick the brick tiles
    rp, cl, vl = A.rowPtr.copy(), A.cols.copy(), A.vals.copy()
    h = cs.HRPB(A.M, A.K, rp, cl, vl)
    B = rng.standard_normal((A.K, 64)).astype(np.float32)
    ref = orc.spmm_csr(A.rowPtr, A.cols, A.vals, B)
    csr_bytes = (A.M + 1) * 4 + A.nnz * 8
    h.upload()
    after_upload = h.device_bytes()
    assert after_upload > csr_bytes
    out, plan = _run(cs, torch_cuda, h, B)
    assert plan.info["mfmaShape"] == 1 and h.device_bytes() == after_upload           # nothing more was needed
    h.cols[:] = 0                                                                      # the borrowed host arrays go away
    h.vals[:] = 0
    out2, plan2 = _run(cs, torch_cuda, h, B, path=cs.PATH_BRICK, mfma_shape=2)
    assert h.device_bytes() > after_upload                                             # the quad lists were built now
    for o in (out, out2):
        assert cs.backward_error(A.rowPtr, A.cols, A.vals, B, ref, o) <= BERR
    grown = h.device_bytes()
    _run(cs, torch_cuda, h, B, path=cs.PATH_BRICK, mfma_shape=2, max_chunk_blocks=2)
    assert h.device_bytes() == grown                                                   # built once
    # every panel to the row kernel: the upload holds the CSR arrays only, until a plan forces an MFMA kernel
    U = cs.gen_config(1)
    hu = cs.HRPB(U.M, U.K, U.rowPtr, U.cols, U.vals)
    hu.upload()
    assert hu.device_bytes() == (U.M + 1) * 4 + U.nnz * 8
    Bu = rng.standard_normal((U.K, 32)).astype(np.float32)
    refu = orc.spmm_csr(U.rowPtr, U.cols, U.vals, Bu)
    for kw in (dict(), dict(path=cs.PATH_BRICK, mfma_shape=2), dict(path=cs.PATH_BRICK, mfma_shape=1)):
        out, _ = _run(cs, torch_cuda, hu, Bu, **kw)
        assert cs.backward_error(U.rowPtr, U.cols, U.vals, Bu, refu, out) <= BERR, kw
    assert hu.device_bytes() > (U.M + 1) * 4 + U.nnz * 8


def test_csr_comparison_kernels(cs, orc, torch_cuda):
    torch = torch_cuda
    A = cs.gen_config(2, 1 / 16.0)
    for N in (32, 100, 128):
        B = cs.gen_dense(3, A.K, N, 2)
        ref = orc.spmm_csr(A.rowPtr, A.cols, A.vals, B)
        h = cs.HRPB(A.M, A.K, A.rowPtr, A.cols, A.vals)
        dB = torch.from_numpy(B).cuda()
        for alg in (0, 1, 2):
            dC = torch.full((A.M, N), float("nan"), device="cuda")
            cs.csr_spmm_dev(alg, h, dB, dC)
            torch.cuda.synchronize()
            assert cs.backward_error(A.rowPtr, A.cols, A.vals, B, ref, dC.cpu().numpy()) <= BERR, (N, alg)
        hC = np.zeros((A.M, N), np.float32)
        ms = cs.GPU_CSR_cuSPARSE_NEW(A.rowPtr, A.cols, A.vals, A.nnz, B, hC, A.M, A.K, N, 3)
        assert ms > 0 and cs.backward_error(A.rowPtr, A.cols, A.vals, B, ref, hC) <= BERR


def test_full_size_headline_config(cs, orc, torch_cuda):
    """The benchmark workload itself (65536-row stencil, N=128): oracle comparison plus two
    size-independent properties -- column sums (1^T C = (1^T A) B) and linearity in B."""
    torch = torch_cuda
    A = cs.gen_config(2)
    N = 128
    B = cs.gen_dense(cs.SEED_BASE + 102, A.K, N, 2)
    h = cs.HRPB(A.M, A.K, A.rowPtr, A.cols, A.vals)
    ref = orc.spmm_csr(A.rowPtr, A.cols, A.vals, B)
    out, plan = _run(cs, torch, h, B)
    assert plan.info["numAtomicChunks"] == 0
    assert cs.backward_error(A.rowPtr, A.cols, A.vals, B, ref, out) <= BERR
    colsum = np.zeros(A.K, np.float64)
    np.add.at(colsum, A.cols.astype(np.int64), A.vals.astype(np.float64))
    expect = colsum @ B.astype(np.float64)
    got = out.astype(np.float64).sum(0)
    scale = np.abs(colsum) @ np.abs(B.astype(np.float64))
    assert (np.abs(got - expect) <= 1e-5 * scale).all()
    B2 = cs.gen_dense(99, A.K, N, 1)
    out2, _ = _run(cs, torch, h, B2)
    out3, _ = _run(cs, torch, h, (2.0 * B + B2).astype(np.float32))
    # 2B is exact in fp32, so A(2B + B2) differs from 2AB + AB2 only by rounding of the sums
    lin = np.abs(out3.astype(np.float64) - (2.0 * out + out2))
    assert lin.max() <= 1e-4 * max(1.0, float(np.abs(out3).max()))


def test_plan_rejects_bad_arguments(cs, torch_cuda):
    import torch
    rp, cl, vl = random_csr(np.random.default_rng(1), 32, 32, density=0.2)
    h = cs.HRPB(32, 32, rp, cl, vl)
    with pytest.raises(cs.CuteError) as e:
        cs.SPMM_TC(h, 0)
    assert e.value.status == -2
    with pytest.raises(cs.CuteError):
        cs.SPMM_TC(h, 32, path=7)
    plan = cs.SPMM_TC(h, 32)
    with pytest.raises(ValueError):
        plan.run(torch.zeros((32, 16), device="cuda"), torch.zeros((32, 32), device="cuda"))
    # a cut panel's partial tiles are added up by a launch that walks a tile along grid.y: widths it cannot
    # cover are refused when the plan is made (without cut panels the same width is accepted)
    rp, cl, vl = random_csr(np.random.default_rng(2), 64, 4096, row_nnz=lambda r: 2000 if r == 3 else 2)
    long_panel = cs.HRPB(64, 4096, rp, cl, vl)
    assert cs.SPMM_TC(long_panel, 128, path=cs.PATH_BRICK).info["numAtomicChunks"] > 0
    with pytest.raises(cs.CuteError) as e:
        cs.SPMM_TC(long_panel, 300000, path=cs.PATH_BRICK, max_chunk_blocks=4)
    assert e.value.status == -2
    assert cs.SPMM_TC(h, 300000, path=cs.PATH_BRICK).info["numAtomicChunks"] == 0


def test_driver_and_sweep_tool(cs, torch_cuda, tmp_path):
    """The C++ driver (counterpart of run.cu's main) on the golden matrix, through the sweep tool:
    three widths, results checked by the driver itself against the plain CSR kernel, and a second
    pass that reads the converted matrix from the cache file."""
    import os
    from cutespmm_ae_amd import sweep
    from test_oracle_pins import GOLD
    mtx = os.path.join(GOLD, "G67.mtx")
    cache = str(tmp_path / "g67.hrpb")
    first = sweep.run_one(mtx, [32, 128, 512], 5, cache)
    again = sweep.run_one(mtx, [32, 128, 512], 5, cache)
    assert [r["N"] for r in first] == [32, 128, 512] and os.path.getsize(cache) > 0
    for a, b in zip(first, again):
        assert not a["from_cache"] and b["from_cache"]
        assert (a["M"], a["K"], a["nnz"], a["blocks"], a["bricks"]) == (10000, 10000, 40000, 2500, b["bricks"])
        assert (b["M"], b["nnz"], b["blocks"]) == (10000, 40000, 2500)
        for r in (a, b):
            assert r["gflops"] > 0 and r["max_rel_err"] <= 1e-5 and r["backward_err"] <= BERR
    text = sweep.table([("G67", r) for r in first])
    assert text.splitlines()[0] == "matrix, N(feature size), cuTeSpMM GFLOPS, CSR GFLOPS" and len(text.splitlines()) == 4


def test_sweep_kernel_durations_from_rocprofv3(cs, torch_cuda):
    """The sweep tool's --rocprof column: one (matrix, N) under rocprofv3 --kernel-trace --stats, the plan's kernels
    of one step added up and the CSR comparison kernel, against the driver's own event times."""
    import os
    import shutil
    from cutespmm_ae_amd import sweep
    from test_oracle_pins import GOLD
    if not (shutil.which("rocprofv3") or os.path.exists("/opt/rocm/bin/rocprofv3")):
        pytest.skip("rocprofv3 is not installed")
    mtx = os.path.join(GOLD, "G67.mtx")
    events = sweep.run_one(mtx, [128], 20)[0]
    plan_us, csr_us = sweep.kernel_durations(mtx, 128, 20)
    # kernel durations leave out what the event bracket adds per launch, so they are the smaller figures
    assert 0 < plan_us <= 1.5 * events["kernel_us"] and 0 < csr_us <= 1.5 * events["csr_kernel_us"]
    text = sweep.table([("G67", dict(events, kernel_us_rocprof=plan_us, csr_kernel_us_rocprof=csr_us))], rocprof=True)
    assert text.splitlines()[1].startswith("G67, 128, ")


def test_driver_extras_through_the_cpp_mirror(cs, torch_cuda):
    """`run_cute --extras`: the C++ classes HRPB_DEVICE (format built on the device from CSR arrays that live there),
    SPMM_TC::run with a caller's scratch buffer and HybridSpMM, on the golden matrix and on the R-MAT benchmark
    matrix (cut panels: the scratch buffer is used).  The device-built format's product must equal the
    host-built one's bit for bit; the hybrid is held to the reference's metric."""
    import os
    from cutespmm_ae_amd import sweep
    from test_oracle_pins import GOLD
    rows = sweep.run_one(os.path.join(GOLD, "G67.mtx"), [32, 100], 3, extras=True) + sweep.run_one("gen:4", [64], 3, extras=True)
    assert [r["N"] for r in rows] == [32, 100, 64] and rows[2]["atomic_chunks"] > 0
    for r in rows:
        assert r["device_built_equal"] == 1, r
        assert 0 <= r["hybrid_max_rel_err"] <= 1e-5 and r["max_rel_err"] <= 1e-5, r


@pytest.mark.parametrize("block_size", [16, 32])
def test_blocked_ell_spmm(cs, orc, torch_cuda, block_size):
    """Blocked-ELL device SpMM against the CSR oracle: random values (tolerance), integer values
    (bit for bit), every vector width of N, and C += on top of a previous result."""
    torch = torch_cuda
    rng = np.random.default_rng(40 + block_size)
    M, K = 192, 256
    for values, Ns in (("normal", (1, 6, 64, 100, 128)), ("ints", (32,))):
        rp, cl, vl = random_csr(rng, M, K, density=0.06, empty_rows=set(range(64, 96)), values=values)
        csr = cs.CSR_Matrix(nrows=M, ncols=K, rowPtr=rp.astype(np.int32), cols=cl.astype(np.int32), values=vl)
        ell = cs.preprocess(csr, block_size)
        assert ell.get_ellColIdx_height() * block_size == M
        for N in Ns:
            B = (rng.integers(-4, 5, (K, N)) if values == "ints" else rng.standard_normal((K, N))).astype(np.float32)
            ref = orc.spmm_csr(rp, cl, vl, B)
            dB = torch.from_numpy(B).cuda()
            dC = torch.full((M, N), float("nan"), device="cuda")
            ell.spmm(dB, dC)
            torch.cuda.synchronize()
            out = dC.cpu().numpy()
            if values == "ints":
                assert (out == ref).all()
            else:
                assert cs.backward_error(rp, cl, vl, B, ref, out) <= BERR, (block_size, N)
            ell.spmm(dB, dC, accumulate=True)
            torch.cuda.synchronize()
            twice = dC.cpu().numpy()
            assert np.allclose(twice, 2 * out, rtol=1e-6, atol=0) if values != "ints" else (twice == 2 * ref).all()


def test_split_matrix_spmm(cs, orc, torch_cuda):
    """Splitter: heavy tiles through the Blocked-ELL kernel, light tiles through the CSR kernel,
    added into one C -- equal to the product with the unsplit matrix."""
    torch = torch_cuda
    rng = np.random.default_rng(77)
    M = K = 256
    N = 64
    D = np.zeros((M, K), np.float32)
    D[rng.random((M, K)) < 0.01] = 1.0                      # light background
    for t in rng.choice(256, 40, replace=False):            # some dense 16x16 tiles
        r, c = (t // 16) * 16, (t % 16) * 16
        D[r:r + 16, c:c + 16] = (rng.random((16, 16)) < 0.7)
    D *= rng.integers(1, 4, D.shape)
    rp, cl, vl = csr_from_dense(D)
    csr = cs.CSR_Matrix(nrows=M, ncols=K, rowPtr=rp.astype(np.int32), cols=cl.astype(np.int32), values=vl)
    sp = cs.Splitter(csr, 16, 64)
    assert sp.get_num_heavy_tiles() > 0 and sp.get_num_light_tiles() > 0
    heavy, light = cs.CSR_Matrix(sp.get_heavyMatrix()), cs.CSR_Matrix(sp.get_lightMatrix())
    assert heavy.nnz + light.nnz == len(vl)
    B = rng.integers(-3, 4, (K, N)).astype(np.float32)
    dB = torch.from_numpy(B).cuda()
    dC = torch.full((M, N), float("nan"), device="cuda")
    lp = torch.from_numpy(light.rowPtr.astype(np.int32)).cuda()
    lc = torch.from_numpy(light.cols.astype(np.int32)).cuda()
    lv = torch.from_numpy(light.values).cuda()
    cs.csr_spmm_tensors(2, lp, lc, lv, dB, dC)               # C = light . B
    cs.preprocess(heavy, 16).spmm(dB, dC, accumulate=True)   # C += heavy . B
    torch.cuda.synchronize()
    assert (dC.cpu().numpy() == orc.spmm_csr(rp, cl, vl, B)).all()


def test_hybrid_spmm(cs, orc, torch_cuda):
    """cute_hybrid_*: heavy tiles through the Blocked-ELL MFMA kernel, the remainder through the row kernel, one call.
    Exact on integer-valued inputs (every sum is exact in fp32), for both split rules and for thresholds that send
    everything, nothing and some of the matrix to the matrix cores; within tolerance on real values."""
    torch = torch_cuda
    rng = np.random.default_rng(78)
    M, K, N = 256, 320, 64
    D = np.zeros((M, K), np.float32)
    D[rng.random((M, K)) < 0.01] = 1.0                      # light background
    for t in rng.choice((M // 16) * (K // 16), 50, replace=False):   # some dense 16x16 tiles
        r, c = (t // (K // 16)) * 16, (t % (K // 16)) * 16
        D[r:r + 16, c:c + 16] = (rng.random((16, 16)) < 0.7)
    D *= rng.integers(1, 4, D.shape)
    rp, cl, vl = csr_from_dense(D)
    csr = cs.CSR_Matrix(nrows=M, ncols=K, rowPtr=rp.astype(np.int32), cols=cl.astype(np.int32), values=vl)
    B = rng.integers(-3, 4, (K, N)).astype(np.float32)
    ref = orc.spmm_csr(rp, cl, vl, B)
    dB = torch.from_numpy(B).cuda()
    seen = set()
    for kw in (dict(), dict(nnz_threshold=1), dict(nnz_threshold=257), dict(nnz_threshold=40), dict(tile_size=32),
               dict(mode=cs.HYBRID_CLASSIFIER, deviation_threshold=0.5, underload_dominance=0.8),
               dict(mode=cs.HYBRID_CLASSIFIER, deviation_threshold=0.1, underload_dominance=0.5)):
        hy = cs.HybridSpMM(csr, **kw)
        info = hy.info
        assert info["heavyElems"] + info["lightElems"] == len(vl) and info["heavyTiles"] + info["lightTiles"] == info["totalTiles"]
        dC = torch.full((M, N), float("nan"), device="cuda")
        hy.spmm(dB, dC)
        torch.cuda.synchronize()
        assert (dC.cpu().numpy() == ref).all(), kw
        seen.add((info["heavyElems"] > 0, info["lightElems"] > 0))
    assert seen == {(True, True), (True, False), (False, True)}
    # the default threshold: 15 % of the tile's cells (measured break-even); the harness's block statistics ride along
    hy = cs.HybridSpMM(csr)
    st = cs.GET_STATS(csr, 16)
    assert hy.info["threshold"] == 39 and hy.info["stats"][2] == st[2] and hy.info["stats"][3] == st[3]
    sp = cs.Splitter(csr, 16, hy.info["threshold"])
    assert (hy.info["heavyTiles"], hy.info["heavyElems"]) == (sp.get_num_heavy_tiles(), sp.get_num_heavy_elems())
    # real values, a wider N that is not a multiple of the slab
    vr = rng.standard_normal(len(vl)).astype(np.float32)
    csr_r = cs.CSR_Matrix(nrows=M, ncols=K, rowPtr=rp.astype(np.int32), cols=cl.astype(np.int32), values=vr)
    Br = rng.standard_normal((K, 100)).astype(np.float32)
    dC = torch.full((M, 100), float("nan"), device="cuda")
    cs.HybridSpMM(csr_r).spmm(torch.from_numpy(Br).cuda(), dC)
    torch.cuda.synchronize()
    assert cs.backward_error(rp, cl, vr, Br, orc.spmm_csr(rp, cl, vr, Br), dC.cpu().numpy()) <= BERR
    # shapes the Blocked-ELL part cannot take are refused
    odd = cs.CSR_Matrix(nrows=40, ncols=64, rowPtr=np.zeros(41, np.int32), cols=np.zeros(0, np.int32), values=np.zeros(0, np.float32))
    with pytest.raises(cs.CuteError) as e:
        cs.HybridSpMM(odd)
    assert e.value.status == -2


@pytest.mark.timeout(600)
@pytest.mark.parametrize("cfg", [3, 4, 5])
def test_full_size_other_configs(cs, orc, torch_cuda, cfg):
    """The other benchmark workloads at full size through the planner's own choice: comparison with
    the oracle, and the column-sum identity 1^T C = (1^T A) B, which does not depend on the oracle."""
    torch = torch_cuda
    A = cs.gen_config(cfg)
    N = cs.CONFIGS[cfg]["N"]
    B = cs.gen_dense(cs.SEED_BASE + 100 + cfg, A.K, N, 2)
    h = cs.HRPB(A.M, A.K, A.rowPtr, A.cols, A.vals)
    out, plan = _run(cs, torch, h, B)
    ref = orc.spmm_csr(A.rowPtr, A.cols, A.vals, B)
    assert cs.backward_error(A.rowPtr, A.cols, A.vals, B, ref, out) <= BERR, plan.info
    colsum = np.zeros(A.K, np.float64)
    np.add.at(colsum, A.cols.astype(np.int64), A.vals.astype(np.float64))
    scale = np.zeros(A.K, np.float64)
    np.add.at(scale, A.cols.astype(np.int64), np.abs(A.vals.astype(np.float64)))
    expect = colsum @ B.astype(np.float64)
    bound = scale @ np.abs(B.astype(np.float64))
    got = out.sum(0, dtype=np.float64)
    assert (np.abs(got - expect) <= 1e-5 * bound).all()


def test_strip_layout_of_the_quad_kernel(cs, orc, torch_cuda):
    """The quad kernel on one list per 4-row strip (forced, and chosen by the library for a matrix
    with a few very long rows), including strips that are cut into several chunks."""
    torch = torch_cuda
    rng = np.random.default_rng(21)
    M, K = 512, 4096
    rp, cl, vl = random_csr(rng, M, K, row_nnz=lambda r: 2500 if r in (7, 130, 131) else 3)
    for N in (64, 100):
        B = rng.standard_normal((K, N)).astype(np.float32)
        ref = orc.spmm_csr(rp, cl, vl, B)
        dB = torch.from_numpy(B).cuda()
        for layout, kw in ((2, {}), (2, dict(max_chunk_blocks=3)), (2, dict(slots=64)), (0, {}), (1, {})):
            h = cs.HRPB(M, K, rp, cl, vl)
            h.upload(quad_layout=layout)
            dC = torch.full((M, N), float("nan"), device="cuda")
            plan = cs.SPMM_TC(h, N, path=cs.PATH_BRICK, mfma_shape=2, **kw)
            plan.run(dB, dC)
            plan.run(dB, dC)                        # a second launch must not add onto the first
            torch.cuda.synchronize()
            assert cs.backward_error(rp, cl, vl, B, ref, dC.cpu().numpy()) <= BERR, (N, layout, kw, plan.info)
    # integer inputs: bit for bit, strips forced on an ordinary matrix
    rp, cl, vl = random_csr(rng, 256, 320, density=0.05, values="ints")
    B = rng.integers(-4, 5, (320, 96)).astype(np.float32)
    h = cs.HRPB(256, 320, rp, cl, vl)
    h.upload(quad_layout=2)
    out, _ = _run(cs, torch, h, B, path=cs.PATH_BRICK, mfma_shape=2)
    assert (out == orc.spmm_csr(rp, cl, vl, B)).all()


def test_mixed_plans_at_narrow_widths(cs, orc, torch_cuda):
    """Dense panels next to sparse ones, so the planner mixes the MFMA and the row kernel: one fused
    launch whenever N is a multiple of 4 (from one lane per row on), narrow brick tiles for N <= 32."""
    rng = np.random.default_rng(33)
    M, K = 640, 2048
    dense_rows = set(range(64, 160)) | set(range(400, 432))
    rp, cl, vl = random_csr(rng, M, K, row_nnz=lambda r: 60 if r in dense_rows else 3)
    # the dense panels share their columns, as blocks of a stiffness matrix do
    for r in dense_rows:
        s, e = int(rp[r]), int(rp[r + 1])
        cl[s:e] = np.sort(rng.choice(np.arange((r // 16) * 8, (r // 16) * 8 + 64), e - s, replace=False)).astype(cl.dtype)
    h = cs.HRPB(M, K, rp, cl, vl)
    for N in (4, 8, 16, 20, 24, 32, 40, 64):
        B = rng.standard_normal((K, N)).astype(np.float32)
        ref = orc.spmm_csr(rp, cl, vl, B)
        for kw in (dict(), dict(mfma_shape=1), dict(mfma_shape=2)):
            out, plan = _run(cs, torch_cuda, h, B, **kw)
            info = plan.info
            assert info["numChunks"] > 0 and info["numRowPanelsSparse"] > 0, (N, kw, info)
            assert cs.backward_error(rp, cl, vl, B, ref, out) <= BERR, (N, kw, info)
            assert info["fusedLaunch"] == (1 if N % 4 == 0 else 0), (N, info)   # whenever the row kernel's lanes hold four floats
            if info["mfmaShape"] == 1:
                vec = 4 if N % 4 == 0 else 2 if N % 2 == 0 else 1
                while vec > 1 and 8 * vec >= N:         # the narrowest tile that still covers N
                    vec //= 2
                assert info["slabWidth"] == 16 * vec * (2 if vec == 4 and N >= 128 else 1), (N, info)


def test_mixed_and_row_plans_at_wide_widths(cs, orc, torch_cuda):
    """Products wider than one lane group of the row kernel (256 columns): its rows are walked slab by slab, on their
    own and as the row blocks of the fused launches.  Integer operands, so every path must equal the oracle bit for bit;
    widths that are and are not multiples of the slab, and of four."""
    torch = torch_cuda
    rng = np.random.default_rng(77)
    M, K = 320, 1024
    dense_rows = set(range(32, 96)) | set(range(208, 240))
    rp, cl, vl = random_csr(rng, M, K, row_nnz=lambda r: 48 if r in dense_rows else 3, values="ints")
    for r in dense_rows:
        s, e = int(rp[r]), int(rp[r + 1])
        cl[s:e] = np.sort(rng.choice(np.arange((r // 16) * 8, (r // 16) * 8 + 64), e - s, replace=False)).astype(cl.dtype)
    h = cs.HRPB(M, K, rp, cl, vl)
    for N in (260, 512, 516, 770, 1024):
        B = rng.integers(-3, 4, (K, N)).astype(np.float32)
        ref = orc.spmm_csr(rp, cl, vl, B)
        for kw in (dict(), dict(mfma_shape=1), dict(mfma_shape=2), dict(path=cs.PATH_ROWS), dict(mfma_shape=1, brick_groups=2)):
            out, plan = _run(cs, torch, h, B, **kw)
            info = plan.info
            assert (out == ref).all(), (N, kw, info)
            if "path" not in kw:
                assert info["numChunks"] > 0 and info["numRowPanelsSparse"] > 0, (N, kw, info)
                if N % 4 == 0 and "brick_groups" not in kw:
                    assert info["fusedLaunch"] == 1, (N, kw, info)
        # the same through a row list that leaves rows out (every second panel forced to the MFMA side by its long rows)
        plan = cs.SPMM_TC(h, N, max_row_nnz=8)
        dB = torch.from_numpy(B).cuda()
        dC = torch.full((M, N), float("nan"), device="cuda")
        plan.run(dB, dC)
        torch.cuda.synchronize()
        assert (dC.cpu().numpy() == ref).all(), (N, plan.info)


def test_few_huge_panels_are_still_cut(cs, orc, torch_cuda):
    """A handful of dense rows among many short ones: only their panels go to the MFMA kernel, all of
    them long.  Their mean length must not become the chunk length, or one wavefront walks a panel alone."""
    rng = np.random.default_rng(34)
    M, K, N = 4096, 8192, 32
    rp, cl, vl = random_csr(rng, M, K, row_nnz=lambda r: 6000 if r in (100, 2000, 3000) else 2)
    B = rng.standard_normal((K, N)).astype(np.float32)
    ref = orc.spmm_csr(rp, cl, vl, B)
    h = cs.HRPB(M, K, rp, cl, vl)
    out, plan = _run(cs, torch_cuda, h, B)
    assert plan.info["numBrickPanels"] == 3 and plan.info["numAtomicChunks"] >= 3 * 10, plan.info
    assert cs.backward_error(rp, cl, vl, B, ref, out) <= BERR


def _structured_csr(rng, kind, M, K):
    """A few sparsity structures the planner treats differently (all rows sorted, distinct columns)."""
    if kind == "uniform":
        return random_csr(rng, M, K, density=rng.choice([0.002, 0.01, 0.05]))
    if kind == "banded":
        half = int(rng.choice([4, 24, 100]))
        rp, cl, vl = random_csr(rng, M, K, row_nnz=lambda r: min(half, int(rng.integers(1, 12))))    # a clipped window still holds `half` columns
        for r in range(M):
            s, e = int(rp[r]), int(rp[r + 1])
            centre = int(r * K / M)
            window = np.arange(max(0, centre - half), min(K, centre + half))
            cl[s:e] = np.sort(rng.choice(window, e - s, replace=False))
        return rp, cl, vl
    if kind == "blocks":           # dense little blocks on a coarse random pattern, like a stiffness matrix
        b = int(rng.choice([3, 6, 8]))
        D = np.zeros((M, K), np.float32)
        for i in range(0, M - b + 1, b):
            for j in rng.choice(max(1, K // b), size=min(4, max(1, K // b)), replace=False):
                D[i:i + b, j * b:(j + 1) * b] = rng.standard_normal((b, min(b, K - j * b)))
        return csr_from_dense(D)
    if kind == "hubs":             # a few very long rows among short ones, and some empty panels
        long_rows = set(rng.choice(M, 3, replace=False).tolist())
        empty = set(range(32, 64)) if M > 96 else set()
        return random_csr(rng, M, K, row_nnz=lambda r: min(K, 700) if r in long_rows else 0 if r in empty else int(rng.integers(0, 5)))
    raise ValueError(kind)


@pytest.mark.parametrize("seed", range(10))
def test_planner_choices_on_varied_structures(cs, orc, torch_cuda, seed):
    """Whatever the planner picks (kernel, tile width, fused launch, split panels), the product is right:
    varied structures, sizes and widths through the default plan and with either MFMA shape forced."""
    rng = np.random.default_rng(1000 + seed)
    for kind in ("uniform", "banded", "blocks", "hubs"):
        M = 16 * int(rng.integers(1, 70))
        K = 16 * int(rng.integers(4, 90))
        rp, cl, vl = _structured_csr(rng, kind, M, K)
        h = cs.HRPB(M, K, rp, cl, vl)
        for N in sorted(set(int(x) for x in rng.choice([1, 2, 4, 7, 8, 12, 16, 24, 32, 36, 48, 64, 72, 96, 128, 130, 160, 256, 260], 4, replace=False))):
            B = rng.standard_normal((K, N)).astype(np.float32)
            ref = orc.spmm_csr(rp, cl, vl, B)
            for kw in (dict(), dict(mfma_shape=1), dict(mfma_shape=2)):
                out, plan = _run(cs, torch_cuda, h, B, **kw)
                err = cs.backward_error(rp, cl, vl, B, ref, out)
                assert np.isfinite(out).all() and err <= BERR, (seed, kind, M, K, N, kw, err, plan.info)


@pytest.mark.parametrize("K,N", [((1 << 24) + 64, 8), ((1 << 22) + 16, 264)])
def test_dimensions_beyond_the_32_bit_offsets(cs, orc, torch_cuda, K, N):
    """The rolling brick kernel and the quad kernel address B with 32-bit byte offsets from 24-bit products: with
    2^24 columns or more, or a B of 4 GiB or more, the planner has to fall back to the pipelined brick kernel
    (64-bit addresses, like the row kernel).  B lives on the device only; the oracle sees the rows that are used."""
    torch = torch_cuda
    rng = np.random.default_rng(31)
    M = 256
    pool = np.unique(np.concatenate([rng.integers(0, 1000, 200), rng.integers(K - 1000, K, 200), rng.integers(0, K, 400),
                                     np.array([0, K - 1])]))
    rowPtr, cols = np.zeros(M + 1, np.uint32), []
    for r in range(M):
        n = 0 if r in (7, 100) else 300 if r == 50 else int(rng.integers(1, 40))
        cols.append(np.sort(rng.choice(len(pool), n, replace=False)))
        rowPtr[r + 1] = rowPtr[r] + n
    small_cols = np.concatenate(cols).astype(np.uint32)            # column ids inside the pool
    vals = rng.standard_normal(len(small_cols)).astype(np.float32)
    Bpool = rng.standard_normal((len(pool), N)).astype(np.float32)
    ref = orc.spmm_csr(rowPtr, small_cols, vals, Bpool)
    big_cols = pool[small_cols].astype(np.uint32)
    assert big_cols.max() == K - 1
    h = cs.HRPB(M, K, rowPtr, big_cols, vals)
    dB = torch.zeros((K, N), device="cuda")
    dB[torch.from_numpy(pool.astype(np.int64)).cuda()] = torch.from_numpy(Bpool).cuda()
    for kw in (dict(path=cs.PATH_BRICK), dict(path=cs.PATH_BRICK, mfma_shape=2), dict(path=cs.PATH_BRICK, pipeline=1),
               dict(path=cs.PATH_BRICK, max_chunk_blocks=2), dict(path=cs.PATH_ROWS), dict()):
        plan = cs.SPMM_TC(h, N, **kw)
        if plan.info["numChunks"]:
            assert plan.info["mfmaShape"] == 1 and plan.info["pipeline"] == 2, (kw, plan.info)
        dC = torch.full((M, N), float("nan"), device="cuda")
        plan.run(dB, dC)
        torch.cuda.synchronize()
        out = dC.cpu().numpy()
        assert np.isfinite(out).all() and cs.backward_error(rowPtr, small_cols, vals, Bpool, ref, out) <= BERR, kw


def test_row_count_beyond_the_32_bit_offsets(cs, orc, torch_cuda):
    """2^24 rows or more (almost all of them empty here): C is addressed with 64 bits, every row is still written."""
    torch = torch_cuda
    rng = np.random.default_rng(32)
    M, K, N = (1 << 24) + 32, 1024, 4
    busy = np.unique(np.concatenate([rng.integers(0, M, 3000), np.arange(M - 40, M), np.arange(0, 20)]))
    counts = np.zeros(M, np.int64)
    counts[busy] = rng.integers(1, 30, len(busy))
    counts[M - 1] = 200
    rowPtr = np.concatenate([[0], np.cumsum(counts)]).astype(np.uint32)
    cols = np.concatenate([np.sort(rng.choice(K, int(c), replace=False)) for c in counts[busy]]).astype(np.uint32)
    vals = rng.standard_normal(len(cols)).astype(np.float32)
    B = rng.standard_normal((K, N)).astype(np.float32)
    ref = orc.spmm_csr(rowPtr, cols, vals, B)
    h = cs.HRPB(M, K, rowPtr, cols, vals)
    dB = torch.from_numpy(B).cuda()
    for kw in (dict(), dict(path=cs.PATH_BRICK), dict(path=cs.PATH_ROWS)):
        plan = cs.SPMM_TC(h, N, **kw)
        if plan.info["numChunks"]:
            assert plan.info["mfmaShape"] == 1 and plan.info["pipeline"] == 2, (kw, plan.info)
        dC = torch.full((M, N), float("nan"), device="cuda")
        plan.run(dB, dC)
        torch.cuda.synchronize()
        out = dC.cpu().numpy()
        assert np.isfinite(out).all() and (out[counts == 0] == 0).all()
        assert cs.backward_error(rowPtr, cols, vals, B, ref, out) <= BERR, kw


def test_launches_can_be_captured_in_a_graph(cs, orc, torch_cuda):
    """cute_spmm_run only enqueues kernels (zeroing included), so a caller may capture it in a HIP
    graph: every replay, with B changed in place between replays, equals the eager result."""
    torch = torch_cuda
    rng = np.random.default_rng(9)
    M, K, N = 512, 4096, 128
    rp, cl, vl = random_csr(rng, M, K, row_nnz=lambda r: 1200 if r in (5, 300) else 6)     # cut panels: partial tiles + the reduce kernel
    h = cs.HRPB(M, K, rp, cl, vl)
    for kw in (dict(), dict(path=cs.PATH_BRICK, mfma_shape=1), dict(path=cs.PATH_BRICK, mfma_shape=2)):
        plan = cs.SPMM_TC(h, N, **kw)
        dB = torch.zeros((K, N), device="cuda")
        dC = torch.full((M, N), float("nan"), device="cuda")
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            plan.run(dB, dC, stream=side)                   # warm-up outside the capture
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            plan.run(dB, dC, stream=torch.cuda.current_stream())
        for rep in range(3):
            B = rng.standard_normal((K, N)).astype(np.float32)
            dB.copy_(torch.from_numpy(B))
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            got = dC.cpu().numpy()
            eager = torch.full((M, N), float("nan"), device="cuda")
            plan.run(dB, eager)
            torch.cuda.synchronize()
            ref = orc.spmm_csr(rp, cl, vl, B)
            assert cs.backward_error(rp, cl, vl, B, ref, got) <= BERR, (kw, rep)
            if not plan.info["numAtomicChunks"]:
                assert (got == eager.cpu().numpy()).all(), (kw, rep)
