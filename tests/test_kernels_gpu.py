"""Parity of the HIP kernel families (called through the C-ABI launcher)
against the CPU oracle, on seeded inputs.

Tolerances: bit-exact for integer / index / byte-moving outputs; <= 1e-5
relative for fp32 outputs; <= 2e-2 absolute for bf16 outputs.  Shapes follow
the reference's own test shapes where it has them (cited per test).
"""
import os

import numpy as np
import pytest
import torch

from tests.helpers import announce, bits

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


@pytest.fixture(scope="module")
def K():
    from inductor_x_amd import kernels

    return kernels


@pytest.fixture(scope="module")
def O():
    from oracle import oracle

    return oracle


# ---------------------------------------------------------------- graph 1
# last-dim sums incl. odd outer shapes, as reference test/npu_indexing/reduction_test.py:12-33
@pytest.mark.parametrize("shape", [(3, 8), (1024, 4096), (7, 9, 1024), (2053, 64), (33, 12), (1, 7168), (513, 100)])
def test_rowsum_vs_oracle(K, O, shape):
    announce(f"rowsum shape={shape}")
    torch.manual_seed(0)
    x = torch.randn(*shape)
    y = K.fused_relu_sigmoid_rowsum(x.to(DEV)).cpu().numpy()
    ref = O.relu_sigmoid_rowsum(x.numpy())
    assert y.shape == ref.shape
    np.testing.assert_allclose(y, ref, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("variant", [(256, 256), (256, 128), (256, 64), (512, 512), (1024, 1024)])
def test_rowsum_variants(K, O, variant):
    announce(f"rowsum variant={variant}")
    torch.manual_seed(1)
    x = torch.randn(301, 2048)
    y = K.fused_relu_sigmoid_rowsum(x.to(DEV), variant=variant).cpu().numpy()
    np.testing.assert_allclose(y, O.relu_sigmoid_rowsum(x.numpy()), rtol=1e-5, atol=1e-6)


def test_rowsum_empty_and_nan(K):
    announce("rowsum empty / nan")
    assert K.fused_relu_sigmoid_rowsum(torch.empty(0, 64, device=DEV)).shape == (0,)
    x = torch.randn(4, 64)
    x[2, 5] = float("nan")
    y = K.fused_relu_sigmoid_rowsum(x.to(DEV)).cpu()
    assert torch.isnan(y[2]) and not torch.isnan(y[[0, 1, 3]]).any()


def test_rowsum_rejects_bad_operands(K):
    with pytest.raises(ValueError):
        K.fused_relu_sigmoid_rowsum(torch.randn(4, 6, device=DEV))  # row not a multiple of 4
    with pytest.raises(ValueError):
        K.fused_relu_sigmoid_rowsum(torch.randn(8, 8, device=DEV).t())  # not contiguous
    with pytest.raises(ValueError):
        K.fused_relu_sigmoid_rowsum(torch.randn(8, 8, device=DEV).half())


# ---------------------------------------------------------------- graph 2
@pytest.mark.parametrize("rows,cols", [(1, 8), (5, 64), (64, 4096), (129, 1024), (3, 2056), (257, 512), (8, 8192)])
def test_add_rmsnorm_vs_oracle(K, O, rows, cols):
    announce(f"add_rmsnorm rows={rows} cols={cols}")
    torch.manual_seed(0)
    h = torch.randn(rows, cols).bfloat16()
    r = torch.randn(rows, cols).bfloat16()
    w = (1 + 0.02 * torch.randn(cols)).bfloat16()
    out, s = K.add_rmsnorm(h.to(DEV), r.to(DEV), w.to(DEV), 1e-6)
    o_ref, s_ref = O.add_rmsnorm_bf16(bits(h), bits(r), bits(w), 1e-6)
    assert np.array_equal(bits(s), s_ref)  # h + r is exactly rounded: bit-exact
    err = np.abs(O.bf16_bits_to_f32(bits(out)) - O.bf16_bits_to_f32(o_ref)).max()
    assert err <= 2e-2
    # and almost everywhere identical bits (differences are single bf16 roundings)
    assert (bits(out) != o_ref).mean() < 0.01


@pytest.mark.parametrize("variant", [(256, 256, 2), (256, 128, 4), (256, 64, 8), (512, 512, 1), (256, 256, 4)])
def test_add_rmsnorm_variants(K, O, variant):
    announce(f"add_rmsnorm variant={variant}")
    torch.manual_seed(2)
    rows, cols = 77, 4096
    h = torch.randn(rows, cols).bfloat16()
    r = torch.randn(rows, cols).bfloat16()
    w = (1 + 0.02 * torch.randn(cols)).bfloat16()
    out, s = K.add_rmsnorm(h.to(DEV), r.to(DEV), w.to(DEV), 1e-6, variant=variant)
    o_ref, s_ref = O.add_rmsnorm_bf16(bits(h), bits(r), bits(w), 1e-6)
    assert np.array_equal(bits(s), s_ref)
    assert np.abs(O.bf16_bits_to_f32(bits(out)) - O.bf16_bits_to_f32(o_ref)).max() <= 2e-2


def test_add_rmsnorm_full_size_properties(K):
    """BASELINE shape [8192, 4096]: w = 1, r = 0 reduces to textbook RMSNorm
    (every output row has mean square 1), and h + 0 returns h bit-for-bit."""
    announce("add_rmsnorm full size properties")
    torch.manual_seed(0)
    h = torch.randn(8192, 4096).bfloat16().to(DEV)
    r = torch.zeros_like(h)
    w = torch.ones(4096, dtype=torch.bfloat16, device=DEV)
    out, s = K.add_rmsnorm(h, r, w, 1e-6)
    assert torch.equal(s, h)
    ms = out.float().pow(2).mean(-1)
    assert (ms - 1).abs().max().item() < 5e-3
    # scale invariance: normalising 4*h gives the same result as h
    out4, _ = K.add_rmsnorm(h * 4, r, w, 1e-6)
    assert (out4.float() - out.float()).abs().max().item() <= 2e-2


def test_add_rmsnorm_empty(K):
    out, s = K.add_rmsnorm(
        torch.empty(0, 64, dtype=torch.bfloat16, device=DEV),
        torch.empty(0, 64, dtype=torch.bfloat16, device=DEV),
        torch.ones(64, dtype=torch.bfloat16, device=DEV),
    )
    assert out.shape == (0, 64) and s.shape == (0, 64)


# ---------------------------------------------------------------- graph 3
def _check_col(K, O, x, correction=0.0, **kw):
    mean, var, arg = K.col_mean_var_argmax(x.to(DEV), correction, **kw)
    m_ref, v_ref, a_ref = O.col_mean_var_argmax(x.numpy(), correction)
    assert np.array_equal(arg.cpu().numpy(), a_ref)  # bit-exact, first index on ties
    # means of N(0,1) columns are ~0: relative 1e-5 of the column's scale (its
    # standard deviation), i.e. an absolute floor of 1e-5 * sqrt(var)
    scale = np.sqrt(np.maximum(v_ref, 1e-30))
    assert (np.abs(mean.cpu().numpy() - m_ref) <= 1e-5 * np.maximum(np.abs(m_ref), scale) + 1e-12).all()
    np.testing.assert_allclose(var.cpu().numpy(), v_ref, rtol=1e-5, atol=1e-12)


# shapes: reference test/npu_indexing/var_mean_test.py:28-36 reduces (128,8,64) style
# tensors; argmax shapes 513x64 / 513x1024 from argmax_unalign_test.py:37,58
@pytest.mark.parametrize("rows,cols", [(1, 4), (2, 512), (513, 64), (513, 1024), (4096, 512), (65536, 512), (1000, 12), (300, 2048), (70000, 8)])
def test_col_stats_vs_oracle(K, O, rows, cols):
    announce(f"col stats rows={rows} cols={cols}")
    torch.manual_seed(0)
    _check_col(K, O, torch.randn(rows, cols))


def test_col_stats_correction_and_offset(K, O):
    announce("col stats correction=1, shifted data")
    torch.manual_seed(3)
    x = torch.randn(5000, 64) * 0.5 + 100.0  # large mean relative to spread
    _check_col(K, O, x, correction=1.0)


def test_col_argmax_ties_and_nan(K, O):
    """Planted ties across thread / row-lane / split boundaries and NaNs."""
    announce("col argmax ties / nan")
    torch.manual_seed(4)
    rows, cols = 4096, 64
    x = torch.randn(rows, cols).clamp_(-3, 3)
    x[:, 0] = 1.0  # all equal -> index 0
    x[100, 1] = 10.0
    x[3000, 1] = 10.0  # tie far apart -> 100
    x[4095, 2] = 10.0
    x[17, 2] = 10.0  # later planted first in memory order anyway -> 17
    x[2000, 3] = float("nan")
    x[50, 3] = 50.0  # NaN beats numbers -> 2000
    x[7, 4] = float("nan")
    x[9, 4] = float("nan")  # first NaN -> 7
    x[:, 5] = float("-inf")  # all -inf -> 0
    x[1234, 6] = float("inf")
    mean, var, arg = K.col_mean_var_argmax(x.to(DEV))
    a = arg.cpu().numpy()
    assert list(a[:7]) == [0, 100, 17, 2000, 7, 0, 1234]
    assert np.array_equal(a, torch.argmax(x, 0).numpy())
    assert np.array_equal(a, O.col_mean_var_argmax(x.numpy())[2])
    assert torch.isnan(var.cpu()[3]) and torch.isnan(mean.cpu()[3])


@pytest.mark.parametrize("ct,rl,u", [(128, 2, 4), (128, 4, 8), (128, 8, 4), (64, 16, 4), (64, 1, 8), (16, 16, 4), (1, 64, 4)])
def test_col_stats_variants(K, O, ct, rl, u):
    from inductor_x_amd.hip_heuristics import SplitPlan, cdiv

    announce(f"col stats variant ct={ct} rl={rl} u={u}")
    torch.manual_seed(5)
    rows, cols = 3001, 256
    x = torch.randn(rows, cols)
    rps = cdiv(cdiv(rows, 7), rl * u) * rl * u
    plan = SplitPlan(ct, rl, u, cdiv(rows, rps), rps, cdiv(cols, ct * 4))
    for fv in [(16, 16), (8, 32), (4, 64), (64, 4)]:
        _check_col(K, O, x, plan=plan, final_variant=fv)


@pytest.mark.parametrize("rows", [1, 7, 16, 17, 64, 65, 4099])
@pytest.mark.parametrize("nsplit", [1, 7, 64])
def test_col_stats_batch_cyclic_row_order(K, O, rows, nsplit):
    """Rows go to the splits in batches of RL * UNROLL, batch b to split b % nsplit: fewer rows than
    one batch, a partly filled last batch, whole batches only, and more splits than batches (splits
    without any row), with NaNs and ties planted so the rare re-walk of a column runs too."""
    from inductor_x_amd.hip_heuristics import SplitPlan, cdiv

    announce(f"col stats cyclic rows={rows} nsplit={nsplit}")
    torch.manual_seed(rows * 100 + nsplit)
    cols = 64
    x = torch.randn(rows, cols)
    if rows > 16:
        x[rows - 1, 3] = float("nan")
        x[5, 3] = float("nan")  # first NaN wins -> 5
        x[rows - 2, 4] = 9.0
        x[2, 4] = 9.0  # tie -> 2
        x[1, 5] = float("inf")
        x[9, 5] = float("-inf")  # inf - inf makes the shifted sum NaN without a NaN sample
    for ct, rl, u in [(128, 2, 8), (128, 4, 4), (64, 8, 4), (16, 16, 4)]:
        plan = SplitPlan(ct, rl, u, nsplit, cdiv(rows, nsplit), cdiv(cols, ct * 4))
        mean, var, arg = K.col_mean_var_argmax(x.to(DEV), 0.0, plan=plan)
        assert np.array_equal(arg.cpu().numpy(), torch.argmax(x, 0).numpy()), (ct, rl, u)
        assert np.array_equal(arg.cpu().numpy(), O.col_mean_var_argmax(x.numpy(), 0.0)[2])
        v_ref, m_ref = torch.var_mean(x.double(), 0, unbiased=False)
        ok = torch.isfinite(m_ref)
        # same bar as _check_col: 1e-5 of the column's scale for the (near-zero) means, 1e-5 relative for var
        scale = v_ref[ok].sqrt().clamp_min(1e-15)
        assert ((mean.cpu().double()[ok] - m_ref[ok]).abs() <= 1e-5 * torch.maximum(m_ref[ok].abs(), scale) + 1e-12).all()
        assert torch.allclose(var.cpu().double()[ok], v_ref[ok], rtol=1e-5, atol=1e-12)
        if rows > 16:
            assert torch.isnan(mean.cpu()[3]) and torch.isnan(var.cpu()[3])


def test_col_stats_invariants_full_size(K):
    """BASELINE shape: var(x + c) == var(x), var(k x) == k^2 var(x), argmax unchanged."""
    announce("col stats invariants 65536x512")
    torch.manual_seed(0)
    x = torch.randn(65536, 512).to(DEV)
    m0, v0, a0 = K.col_mean_var_argmax(x)
    m1, v1, a1 = K.col_mean_var_argmax(x + 3.0)
    m2, v2, a2 = K.col_mean_var_argmax(x * 2.0)
    assert torch.equal(a0, a2)
    assert ((v1 - v0).abs() / v0).max().item() < 1e-4  # x + 3 rounds the inputs themselves
    assert ((v2 - 4 * v0).abs() / (4 * v0)).max().item() < 1e-6
    assert (m1 - m0 - 3.0).abs().max().item() < 1e-5
    assert torch.equal(a0, torch.argmax(x, 0))


# ---------------------------------------------------------------- graph 4
@pytest.mark.parametrize("nrows,width,n", [(10, 8, 1), (50304, 1024, 4096), (17, 128, 1000), (3, 2048, 33), (100, 264, 77)])
def test_gather_vs_oracle(K, O, nrows, width, n):
    announce(f"gather nrows={nrows} width={width} n={n}")
    torch.manual_seed(0)
    table = (0.02 * torch.randn(nrows, width)).bfloat16()
    idx = torch.randint(0, nrows, (n,), dtype=torch.int64)
    idx[0] = 0
    idx[-1] = nrows - 1
    out = K.gather_rows(table.to(DEV), idx.to(DEV))
    assert np.array_equal(bits(out), O.gather_rows(bits(table), idx.numpy()))


def test_gather_duplicates_negative_2d_index_fp32(K, O):
    announce("gather duplicates / negative / 2-D idx / fp32")
    torch.manual_seed(1)
    table = torch.randn(9, 64).bfloat16()
    idx = torch.tensor([[0, 0, 8, -1], [3, 3, -9, 8]], dtype=torch.int64)
    out = K.gather_rows(table.to(DEV), idx.to(DEV))
    assert out.shape == (2, 4, 64)
    assert torch.equal(out.cpu(), table[idx])
    t32 = torch.randn(9, 64)
    assert torch.equal(K.gather_rows(t32.to(DEV), idx.to(DEV)).cpu(), t32[idx])
    assert K.gather_rows(table.to(DEV), torch.empty(0, dtype=torch.int64, device=DEV)).shape == (0, 64)


@pytest.mark.parametrize("variant", [(256, 128, 1), (256, 128, 4), (256, 64, 2), (256, 16, 4)])
def test_gather_variants(K, variant):
    announce(f"gather variant={variant}")
    torch.manual_seed(2)
    table = torch.randn(301, 1024).bfloat16()
    idx = torch.randint(0, 301, (999,), dtype=torch.int64)
    out = K.gather_rows(table.to(DEV), idx.to(DEV), variant=variant)
    assert torch.equal(out.cpu(), table[idx])


# permute (0,2,1,3): reference test/npu_indexing/permute_test.py:19 on (8,8,512,128)
@pytest.mark.parametrize("shape", [(8, 8, 512, 128), (2, 3, 5, 8), (1, 33, 7, 64), (16, 2048, 32, 128), (3, 100, 9, 120)])
def test_permute_vs_oracle(K, O, shape):
    announce(f"permute shape={shape}")
    torch.manual_seed(0)
    t = torch.randn(*shape).bfloat16()
    out = K.permute_0213_contiguous(t.to(DEV))
    assert out.shape == (shape[0], shape[2], shape[1], shape[3])
    assert np.array_equal(bits(out), O.permute4(bits(t), (0, 2, 1, 3)))


def test_permute_involution_full_size_and_fp32(K):
    announce("permute involution 16x2048x32x128")
    torch.manual_seed(0)
    t = torch.randn(16, 2048, 32, 128, device=DEV).bfloat16()
    once = K.permute_0213_contiguous(t)
    assert torch.equal(K.permute_0213_contiguous(once), t)
    assert torch.equal(once, t.permute(0, 2, 1, 3).contiguous())
    f = torch.randn(4, 50, 6, 64, device=DEV)
    assert torch.equal(K.permute_0213_contiguous(f), f.permute(0, 2, 1, 3).contiguous())


@pytest.mark.parametrize("variant", [(256, 16, 32, 8), (256, 16, 8, 8), (256, 16, 1, 64), (256, 16, 2, 8), (256, 64, 4, 4), (256, 8, 1, 32)])
def test_permute_variants(K, variant):
    announce(f"permute variant={variant}")
    torch.manual_seed(1)
    inner = min(variant[1] * 8, 128)
    t = torch.randn(3, 70, 37, inner, device=DEV).bfloat16()
    out = K.permute_0213_contiguous(t, variant=variant)
    assert torch.equal(out, t.permute(0, 2, 1, 3).contiguous())


def test_copy_probe(K):
    announce("copy probe")
    src = torch.randint(0, 255, (1 << 20,), dtype=torch.uint8, device=DEV)
    dst = torch.zeros_like(src)
    K.copy_bytes(dst, src)
    assert torch.equal(dst, src)


# ------------------------------------------------- autotune cache, bandwidth print
# counterpart of the reference's cached autotune and .best_config record
# (inductor_x/npu_triton_heuristics.py:302-393) and of its bandwidth print
# (NPUDebugAutotuner, :268-299)
def _gather_family(K, tmp_path, monkeypatch, variants):
    from inductor_x_amd import codecache
    from inductor_x_amd.hip_heuristics import CachingLauncher, LaunchConfig

    cfgs = [LaunchConfig(f"gather_rows_b16_b{b}_t{t}_r{r}", b, meta={"BLOCK": b, "TPR": t, "RPT": r}) for b, t, r in variants]
    fam = CachingLauncher(
        "gather_rows", codecache.aot_source("copy_kernels.hip"), "PPPiii", cfgs,
        bytes_fn=lambda table, idx, out, n, width, nrows: 2 * n * width * 2 + 8 * n, prefer_intree=True,
    )
    monkeypatch.setattr(fam, "_best_path", lambda: str(tmp_path / "gather_rows.best_config"))
    return fam


def test_autotune_winner_is_recorded_and_reused(K, tmp_path, monkeypatch):
    import json

    from inductor_x_amd import config
    from inductor_x_amd.hip_heuristics import cdiv

    announce("autotune record")
    monkeypatch.setattr(config, "autotune", True)
    torch.manual_seed(5)
    table = torch.randn(4096, 1024, device=DEV).bfloat16()
    idx = torch.randint(0, 4096, (8192,), device=DEV)
    out = torch.empty(8192, 1024, dtype=torch.bfloat16, device=DEV)
    args = (table.data_ptr(), idx.data_ptr(), out.data_ptr(), 8192, 1024, 4096)
    grid = lambda meta: (cdiv(8192, (meta["BLOCK"] // meta["TPR"]) * meta["RPT"]), 1, 1)  # noqa: E731
    variants = [(256, 128, 1), (256, 128, 2), (256, 64, 2), (256, 16, 4)]
    stream = torch.cuda.current_stream().cuda_stream

    fam = _gather_family(K, tmp_path, monkeypatch, variants)
    fam.run(*args, grid=grid, stream=stream)
    torch.cuda.synchronize()
    assert torch.equal(out, table[idx])
    rec = json.loads((tmp_path / "gather_rows.best_config").read_text())
    assert rec["symbol"] == fam.best_config().symbol
    assert set(rec["timings_ms"]) == {f"gather_rows_b16_b{b}_t{t}_r{r}" for b, t, r in variants}
    assert rec["timings_ms"][rec["symbol"]] == min(rec["timings_ms"].values())

    # a second launcher object (another process would look the same) reads the record and times nothing
    again = _gather_family(K, tmp_path, monkeypatch, variants)
    monkeypatch.setattr(again, "bench", lambda *a, **k: pytest.fail("timed again despite a valid record"))
    out.zero_()
    again.run(*args, grid=grid, stream=stream)
    torch.cuda.synchronize()
    assert again.best_config().symbol == rec["symbol"]
    assert torch.equal(out, table[idx])

    # a record made for another configuration list is not trusted
    other = _gather_family(K, tmp_path, monkeypatch, variants[:3])
    other.precompile()
    assert other._best is None


def test_bandwidth_print(K, tmp_path, monkeypatch, capsys):
    from inductor_x_amd import config

    announce("bandwidth print")
    monkeypatch.setattr(config, "profile_bandwidth", True)
    table = torch.randn(1024, 1024, device=DEV).bfloat16()
    idx = torch.arange(1024, device=DEV)
    out = torch.empty_like(table)
    fam = _gather_family(K, tmp_path, monkeypatch, [(256, 128, 2)])
    fam.run(table.data_ptr(), idx.data_ptr(), out.data_ptr(), 1024, 1024, 1024, grid=(256, 1, 1),
            stream=torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    line = [l for l in capsys.readouterr().out.splitlines() if l.startswith("gather_rows:")]
    assert len(line) == 1 and line[0].endswith("GB/s") and " ms " in line[0]
    assert torch.equal(out, table)


def test_autotune_reaches_the_product_entry_points(K, O, tmp_path, monkeypatch):
    """With config.autotune on, kernels.fused_relu_sigmoid_rowsum and kernels.add_rmsnorm time the
    instantiated shapes that fit the problem once per extents, write a per-shape record beside the
    code object, launch the winner, and return the same numbers as without tuning."""
    import glob
    import json
    import shutil

    from inductor_x_amd import config, kernels
    from inductor_x_amd.hip_heuristics import CachingLauncher

    announce("autotune through kernels.*")
    torch.manual_seed(8)
    x = torch.randn(300, 2048, device=DEV)
    h, r = (torch.randn(129, 1024, device=DEV).bfloat16() for _ in range(2))
    w = torch.ones(1024, device=DEV).bfloat16()
    plain_sum = K.fused_relu_sigmoid_rowsum(x)
    plain_norm = K.add_rmsnorm(h, r, w, 1e-6)
    # a private copy of each family's code object, so the records land in tmp_path
    for getter in (kernels._rowsum_launcher, kernels._rmsnorm_launcher):
        fam = getter()
        fam.precompile()
        private = str(tmp_path / os.path.basename(fam._hsaco_path))
        shutil.copyfile(fam._hsaco_path, private)
        monkeypatch.setattr(fam, "_hsaco_path", private)
        monkeypatch.setattr(fam, "_tuned", {}, raising=False)
    monkeypatch.setattr(config, "autotune", True)
    launched = []
    real = CachingLauncher._launch
    monkeypatch.setattr(CachingLauncher, "_launch",
                        lambda self, idx, *a, **k: (launched.append(self.launchers[idx][0].symbol), real(self, idx, *a, **k))[1])
    tuned_sum = K.fused_relu_sigmoid_rowsum(x)
    last_of_sum = launched[-1]  # the timing launches come first, the launch that counts last
    tuned_norm = K.add_rmsnorm(h, r, w, 1e-6)
    last_of_norm = launched[-1]
    torch.cuda.synchronize()
    np.testing.assert_allclose(tuned_sum.cpu().numpy(), plain_sum.cpu().numpy(), rtol=1e-6)
    assert torch.equal(tuned_norm[1], plain_norm[1])
    assert (tuned_norm[0].float() - plain_norm[0].float()).abs().max().item() <= 2e-2
    records = {os.path.basename(p).split(".", 1)[1]: json.loads(open(p).read()) for p in glob.glob(str(tmp_path / "*.best_config"))}
    assert set(records) == {"300x2048.best_config", "129x1024.best_config"}
    rs, rn = records["300x2048.best_config"], records["129x1024.best_config"]
    assert len(rs["timings_ms"]) == len(kernels._ROWSUM_VARIANTS) and rs["timings_ms"][rs["symbol"]] == min(rs["timings_ms"].values())
    # rows of 1024 bf16 = 128 vectors: only shapes with TPR * ITERS >= 128 are candidates
    assert all(int(s.split("_t")[1].split("_i")[0]) * int(s.rsplit("_i", 1)[1]) >= 128 for s in rn["timings_ms"])
    assert (last_of_sum, last_of_norm) == (rs["symbol"], rn["symbol"])
    # the second call of a shape times nothing
    monkeypatch.setattr(CachingLauncher, "bench", lambda *a, **k: pytest.fail("timed a second time"))
    again = K.fused_relu_sigmoid_rowsum(x)
    assert torch.equal(again, tuned_sum) and launched[-1] == rs["symbol"]


def test_attention_resource_probes_run():
    """The probe kernels behind `bench.py --attention-ceiling` load, run and report every rate as a
    positive finite number (their values are measurements, not pass criteria)."""
    announce("attention resource probes")
    import math

    import bench

    r = bench._attention_ceiling(torch)
    ns = r["ns_per_step_per_simd"]
    assert set(ns) >= {"mfma_only", "fragment_per_mfma", "mfma_with_vector_work", "fragment_per_mfma_with_vector_work"}
    assert all(math.isfinite(v) and v > 0 for v in ns.values())
    assert all(math.isfinite(v) and v > 0 for v in r["lds_bytes_per_clock_per_cu"].values())
    assert math.isfinite(r["ceiling_of_datasheet_peak"]) and r["ceiling_of_datasheet_peak"] > 0


def test_attention_timeline_probe_matches_the_shipped_kernel():
    """The measurement build behind `bench.py --attention-timeline` is the shipped kernel template plus clock
    reads: its outputs are bit-identical to `kernels.fused_attention` and every query block of both launches
    leaves a complete, ordered record (the durations themselves are measurements, not pass criteria)."""
    announce("attention timeline probe")
    import math

    import bench

    r = bench._attention_timeline(torch)
    for mode in ("causal", "full"):
        row = r[mode]
        assert row["matches_shipped_kernel"], mode
        seg = row["mean_us_per_query_block"]
        assert all(math.isfinite(v) for v in seg.values()) and seg["whole_block"] > 0 and seg["unguarded_steps"] > 0
        assert 0 < row["us_per_unguarded_tile_step"] < 50
        assert row["workgroup_end_us"]["max"] >= row["workgroup_end_us"]["mean"] > 0
