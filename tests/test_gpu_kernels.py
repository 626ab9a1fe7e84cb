"""Parity of the HIP kernels (called through the C ABI) with the CPU oracle.

Tolerances: survivor sets, column order and values bit-exact; encoder pre-activations and
reconstructions rel-L2 <= 1e-2 in bf16 and <= 1e-5 in fp32.
"""
import math

import numpy as np
import pytest
import torch

import crosslayer_coding_amd as cca
from crosslayer_coding_amd import _native as nat
from crosslayer_coding_amd import engine
from oracle import clt_oracle as orc

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-5, torch.bfloat16: 1e-2, torch.float16: 2e-3}
DTYPES = [torch.float32, torch.bfloat16, torch.float16]
# relative width of the band around a ranking threshold inside which two correct implementations may differ
BAND = {torch.float32: 1e-5, torch.bfloat16: 2.0 ** -6, torch.float16: 2.0 ** -9}


def dense_from(surv):
    return engine.densify(surv).cpu()


def check_rows_sorted(surv):
    rp = surv.row_ptr.cpu().numpy()
    col = surv.col.cpu().numpy()
    assert rp[0] == 0 and np.all(np.diff(rp) >= 0) and rp[-1] == len(col)
    for r in range(len(rp) - 1):
        seg = col[rp[r]:rp[r + 1]]
        assert np.all(np.diff(seg) > 0), f"row {r} not strictly ascending"


# ---- encoder --------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("L,T,d,F", [(1, 30, 8, 16), (2, 300, 64, 136), (3, 257, 96, 260), (1, 5, 7, 9), (2, 512, 768, 512),
                                     (2, 40, 256, 512), (1, 1, 128, 256), (3, 255, 128, 260),     # short batches: padded to a tile
                                     # an odd number of 128-byte stages along d (1, 3, 5 for 16-bit elements)
                                     (1, 256, 64, 256), (2, 512, 192, 512), (2, 300, 320, 520), (1, 256, 32, 256),
                                     (1, 700, 1600, 768),
                                     # shapes the matrix kernel takes only as zero-padded copies (d, F, T or all three)
                                     (2, 300, 200, 1092), (1, 100, 72, 7000), (3, 512, 100, 516), (1, 260, 1000, 250)])
def test_encode_parity(dev, dtype, L, T, d, F):
    g = torch.Generator().manual_seed(L * 1000 + T)
    x = torch.randn(L, T, d, generator=g).to(dtype)
    w = (torch.randn(L, F, d, generator=g) / math.sqrt(d)).to(dtype)
    b = torch.randn(L, F, generator=g).to(dtype)
    got = engine.encode(x.to(dev), w.to(dev), b.to(dev)).cpu()
    for l in range(L):
        ref = orc.encoder_preactivations(x[l], w[l], b[l])
        ref64 = torch.from_numpy(orc.affine_f64(x[l].float().numpy(), w[l].float().numpy(), b[l].float().numpy()))
        assert orc.rel_l2(got[l], ref) <= TOL[dtype]
        assert orc.rel_l2(got[l], ref64) <= TOL[dtype]
    nob = engine.encode(x.to(dev), w.to(dev), None).cpu()
    assert orc.rel_l2(nob[0], orc.encoder_preactivations(x[0], w[0], None)) <= TOL[dtype]


# ---- BatchTopK per layer ---------------------------------------------------------------------
def run_select(pre, k, dev, global_mode=False):
    surv = engine.batchtopk_select(pre.to(dev), k, global_mode)
    torch.cuda.synchronize()
    return surv


def oracle_per_layer(pre, k):
    return torch.stack([orc.batchtopk_forward(pre[l], float(k), pre[l]) for l in range(pre.shape[0])])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,F,d,n,pitch,tied", [(512, 512, 128, 3, 192, False), (256, 768, 256, 4, 320, True),
                                                 (300, 260, 64, 2, 64, False), (512, 256, 768, 5, 832, False)])
def test_encode_segmented_equals_product_of_stacked_operands(dev, dtype, T, F, d, n, pitch, tied):
    """K cut into n segments that live in separate matrices (a gradient slab [n, T, d] and padded
    feature-major decoders [n, F, pitch]; `tied`: one decoder for all segments): bit for bit the product
    of the operands copied side by side, and within the encoder tolerance of an fp64 matmul."""
    g = torch.Generator().manual_seed(T + F + d + n)
    x = torch.randn(n, T, d, generator=g).to(dtype).to(dev)
    w = (torch.randn(1 if tied else n, F, pitch, generator=g) / math.sqrt(n * d)).to(dtype).to(dev)
    got = engine.encode_segmented(x, w, n, d, T * d, d, 0 if tied else F * pitch, pitch, T, F)
    xs = torch.cat([x[q] for q in range(n)], dim=1).unsqueeze(0).contiguous()                       # [1, T, n d]
    wsd = torch.cat([w[0 if tied else q][:, :d] for q in range(n)], dim=1).unsqueeze(0).contiguous()  # [1, F, n d]
    side_by_side = engine.encode(xs, wsd, None)[0]
    assert torch.equal(got, side_by_side)
    ref = xs[0].double().cpu() @ wsd[0].double().cpu().T
    rel = (got.double().cpu() - ref).norm() / ref.norm()
    assert rel <= TOL[dtype], rel


def test_encode_segmented_rejects_shapes_the_matrix_kernel_cannot_take(dev):
    x = torch.zeros(2, 100, 64, device=dev)
    w = torch.zeros(2, 256, 64, device=dev)
    with pytest.raises(nat.CLTNativeError):
        engine.encode_segmented(x, w, 2, 64, 100 * 64, 64, 256 * 64, 64, 100, 256)   # fewer than 256 tokens
    x = torch.zeros(3, 256, 32, device=dev)
    w = torch.zeros(3, 256, 32, device=dev)
    with pytest.raises(nat.CLTNativeError):
        engine.encode_segmented(x, w, 3, 32, 256 * 32, 32, 256 * 32, 32, 256, 256)   # an odd number of K pieces


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("L,T,F,k", [(1, 2, 4, 2), (2, 64, 256, 8), (3, 100, 1000, 17), (1, 33, 77, 5),
                                     (2, 16, 64, 64), (2, 16, 64, 100), (1, 1, 8, 3), (2, 512, 2048, 40)])
def test_batchtopk_per_layer_bit_exact(dev, dtype, L, T, F, k):
    g = torch.Generator().manual_seed(T * 7 + F)
    pre = torch.randn(L, T, F, generator=g).to(dtype)
    surv = run_select(pre, k, dev)
    check_rows_sorted(surv)
    assert surv.nnz == L * min(k * T, T * F)
    got = dense_from(surv)
    ref = oracle_per_layer(pre, k)
    assert torch.equal(got, ref)


def test_batchtopk_reference_known_answer(dev):
    # reference tests/unit/models/test_activations.py:10-25 : survivors at flat indices {3,4,7,2}
    x = torch.tensor([[[1.0, 2.0, 3.0, 4.0], [5.0, 1.0, 2.5, 3.5]]])
    surv = run_select(x, 2, dev)
    rows = engine.survivor_rows(surv).cpu() * 4 + surv.col.cpu().long()
    assert sorted(rows.tolist()) == [2, 3, 4, 7]
    assert torch.equal(dense_from(surv)[0], torch.tensor([[0.0, 0.0, 3.0, 4.0], [5.0, 0.0, 0.0, 3.5]]))


@pytest.mark.parametrize("dtype", DTYPES)
def test_batchtopk_heavy_ties_lowest_index(dev, dtype):
    g = torch.Generator().manual_seed(11)
    pre = (torch.randint(-4, 5, (2, 96, 520), generator=g).float() * 0.25).to(dtype)
    for k in (3, 50, 300):
        surv = run_select(pre, k, dev)
        check_rows_sorted(surv)
        assert torch.equal(dense_from(surv).to(dtype), oracle_per_layer(pre, k))
        # zero-valued survivors vanish in the dense form: compare the index sets as well
        for l in range(2):
            m = orc.batchtopk_mask(pre[l], k, pre[l])
            rows = engine.survivor_rows(surv).cpu()
            sel = (rows >= l * 96) & (rows < (l + 1) * 96)
            flat = (rows[sel] - l * 96) * 520 + surv.col.cpu().long()[sel]
            assert torch.equal(torch.sort(flat).values, m.view(-1).nonzero().view(-1))


@pytest.mark.parametrize("dtype", DTYPES)
def test_batchtopk_special_values(dev, dtype):
    g = torch.Generator().manual_seed(5)
    pre = torch.randn(1, 40, 128, generator=g).to(dtype)
    pre[0, 0, 0], pre[0, 1, 5] = float("nan"), float("inf")
    pre[0, 2, 7], pre[0, 3, 9] = float("-inf"), -0.0
    pre[0, 5, :64] = 0.0
    pre[0, 6, :64] = -0.0
    for k in (1, 20, 100, 128):
        surv = run_select(pre, k, dev)
        m = orc.batchtopk_mask(pre[0], k, pre[0])
        rows = engine.survivor_rows(surv).cpu()
        flat = rows * 128 + surv.col.cpu().long()
        assert torch.equal(torch.sort(flat).values, m.view(-1).nonzero().view(-1)), k


def test_batchtopk_all_equal_and_constant_rows(dev):
    pre = torch.full((2, 50, 96), 1.5)
    surv = run_select(pre, 10, dev)
    # all tie: the lowest flat indices win -> the first 500 elements of each layer
    got = dense_from(surv)
    ref = oracle_per_layer(pre, 10)
    assert torch.equal(got, ref) and int((got != 0).sum()) == 2 * 500


@pytest.mark.parametrize("dtype", DTYPES)
def test_batchtopk_outlier_rows_overflow_segments(dev, dtype):
    # a few rows hold nearly all survivors: their candidate segments overflow and are re-read
    g = torch.Generator().manual_seed(9)
    L, T, F, k = 2, 256, 4096, 16
    pre = torch.randn(L, T, F, generator=g)
    pre[:, 3] += 6.0
    pre[0, 200] += 8.0
    pre = pre.to(dtype)
    surv = run_select(pre, k, dev)
    check_rows_sorted(surv)
    assert torch.equal(dense_from(surv), oracle_per_layer(pre, k))


@pytest.mark.parametrize("dtype", DTYPES)
def test_batchtopk_candidate_pool_overflow_falls_back_to_dense_rows(dev, dtype):
    # half of all values tie at the top: the sampled cut admits ~500x more candidates than the
    # pool holds, so most rows are re-read from the matrix; the result must not change
    g = torch.Generator().manual_seed(13)
    L, T, F, k = 2, 512, 2048, 4
    pre = torch.randn(L, T, F, generator=g).clamp(max=0.0)
    pre[1] = pre[1].clamp(min=-0.5)
    pre = pre.to(dtype)
    surv = run_select(pre, k, dev)
    check_rows_sorted(surv)
    for l in range(L):
        m = orc.batchtopk_mask(pre[l], k, pre[l])
        rows = engine.survivor_rows(surv).cpu()
        sel = (rows >= l * T) & (rows < (l + 1) * T)
        flat = (rows[sel] - l * T) * F + surv.col.cpu().long()[sel]
        assert torch.equal(torch.sort(flat).values, m.view(-1).nonzero().view(-1))


def test_batchtopk_k_zero_and_empty(dev):
    pre = torch.randn(2, 8, 16)
    surv = run_select(pre, 0, dev)
    assert surv.nnz == 0 and int(surv.row_ptr.abs().sum()) == 0
    surv = engine.batchtopk_select(torch.empty(2, 0, 16, device=dev), 3, False)
    assert surv.nnz == 0


# ---- encoder with the per-feature-threshold epilogue (JumpReLU) ---------------------------------
def threshold_fused_vs_separate(x, w, b, theta, dev, density_ppm=200000):
    xd, wd, td = x.to(dev), w.to(dev), theta.to(dev)
    bd = b.to(dev) if b is not None else None
    pre = engine.encode(xd, wd, bd)
    ref = engine.threshold_select(pre, td, nat.PRED_GE_THETA)
    got = engine.encode_threshold(xd, wd, bd, td, engine.Workspace(xd.device), density_ppm)
    torch.cuda.synchronize()
    return pre.cpu(), ref, got


def assert_same_list(got, ref, dtype):
    iv = torch.int32 if dtype == torch.float32 else torch.int16
    assert torch.equal(got.row_ptr.cpu(), ref.row_ptr.cpu())
    assert torch.equal(got.col.cpu(), ref.col.cpu())
    assert torch.equal(got.val.cpu().view(iv), ref.val.cpu().view(iv))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("L,T,d,F", [(1, 256, 128, 256), (2, 512, 256, 1024), (3, 256, 768, 512),
                                     # token counts that are not whole tiles: the last tile is shifted back
                                     (2, 257, 128, 256), (3, 300, 256, 512), (1, 511, 128, 1024), (2, 1000, 128, 256),
                                     # an odd number of stages along d
                                     (2, 512, 320, 512), (1, 300, 64, 256),
                                     # feature counts that are not whole tiles: the last feature tile is shifted back
                                     (2, 256, 128, 384), (1, 300, 128, 520), (2, 512, 64, 1096), (1, 257, 128, 264),
                                     # more token tiles than feature tiles, in eights: the token-major tile map
                                     (1, 2000, 128, 256), (1, 4000, 64, 520)])
def test_encode_threshold_matches_separate_and_oracle(dev, dtype, L, T, d, F):
    g = torch.Generator().manual_seed(L * 17 + T + F)
    x = torch.randn(L, T, d, generator=g).to(dtype)
    w = (torch.randn(L, F, d, generator=g) / math.sqrt(d)).to(dtype)
    b = (0.1 * torch.randn(L, F, generator=g)).to(dtype)
    theta = torch.exp(0.5 * torch.randn(L, F, generator=g) + 0.3).to(dtype)
    pre, ref, got = threshold_fused_vs_separate(x, w, b, theta, dev)
    assert got is not None
    assert_same_list(got, ref, dtype)
    check_rows_sorted(got)
    dense = engine.densify(got, out_f32=True).cpu()
    for l in range(L):
        assert torch.equal(dense[l], orc.jumprelu_forward(pre[l], theta[l]))


@pytest.mark.parametrize("dtype", DTYPES)
def test_encode_threshold_special_thresholds_and_values(dev, dtype):
    # zero / huge / infinite thresholds and NaN, +-inf, -0.0 pre-activations (reached through
    # crafted inputs: one-hot weights copy input values into the pre-activations)
    g = torch.Generator().manual_seed(4)
    L, T, d, F = 1, 256, 128, 256
    x = torch.randn(L, T, d, generator=g)
    x[0, 3, 0] = float("nan"); x[0, 5, 1] = float("inf"); x[0, 7, 2] = float("-inf"); x[0, 9, 3] = -0.0
    w = torch.zeros(L, F, d)
    for f in range(F):
        w[0, f, f % d] = 1.0                       # pre[t, f] = x[t, f % d] (plus NaN/inf propagation rules)
    theta = torch.exp(0.5 * torch.randn(L, F, generator=g))
    theta[0, 0] = 0.0; theta[0, 1] = float("inf"); theta[0, 2] = 3e38; theta[0, 130] = 0.0
    pre, ref, got = threshold_fused_vs_separate(x.to(dtype), w.to(dtype), None, theta.to(dtype), dev)
    assert got is not None
    assert_same_list(got, ref, dtype)


def test_encode_threshold_pool_too_small_reports_it(dev):
    g = torch.Generator().manual_seed(6)
    L, T, d, F = 1, 256, 128, 256
    x = torch.randn(L, T, d, generator=g).to(torch.bfloat16)
    w = (torch.randn(L, F, d, generator=g) / math.sqrt(d)).to(torch.bfloat16)
    theta = torch.full((L, F), 1e-3).to(torch.bfloat16)          # about half of all values survive
    pre, ref, got = threshold_fused_vs_separate(x, w, None, theta, dev, density_ppm=1)
    assert got is None
    pre, ref, got = threshold_fused_vs_separate(x, w, None, theta, dev, density_ppm=600000)
    assert got is not None and got.nnz == ref.nnz
    assert_same_list(got, ref, torch.bfloat16)


@pytest.mark.parametrize("T", [300, 700])
def test_encode_threshold_ragged_batch_overflow_is_redone_densely(dev, T):
    # the device-side fallback (pool overflow -> dense route) on a token count that is not a whole number of tiles
    g = torch.Generator().manual_seed(T)
    L, d, F = 2, 128, 512
    x = torch.randn(L, T, d, generator=g).to(torch.bfloat16).to(dev)
    w = (torch.randn(L, F, d, generator=g) / math.sqrt(d)).to(torch.bfloat16).to(dev)
    theta = torch.full((L, F), 1e-3).to(torch.bfloat16).to(dev)
    pre = engine.encode(x, w, None)
    ref = engine.threshold_select(pre, theta, nat.PRED_GE_THETA)
    for ppm in (1, 600000):        # 1: overflows and is redone from the dense scratch; 600000: fits
        scratch = torch.full_like(pre, float("nan"))
        got = engine.encode_threshold(x, w, None, theta, engine.Workspace(dev), ppm, pre_scratch=scratch)
        torch.cuda.synchronize()
        n = int(got.row_ptr[-1])
        assert n == ref.nnz
        assert torch.equal(got.row_ptr.cpu(), ref.row_ptr.cpu())
        assert torch.equal(got.col[:n].cpu(), ref.col.cpu())
        assert torch.equal(got.val[:n].cpu().view(torch.int16), ref.val.cpu().view(torch.int16))


# ---- BatchTopK global ------------------------------------------------------------------------
# ---- encoder with the collecting epilogue + BatchTopK on the candidates --------------------
def fused_vs_separate(x, w, b, k, dev):
    """The fused path must give the survivor list of encode -> batchtopk_select, bit for bit."""
    xd, wd, bd = x.to(dev), w.to(dev), (b.to(dev) if b is not None else None)
    assert engine.encode_collect_supported(xd, wd, bd, k)
    pre = engine.encode(xd, wd, bd)
    ref = engine.batchtopk_select(pre, k, False)
    ws = engine.Workspace(xd.device)
    scratch = torch.full_like(pre, float("nan"))
    got = engine.collect_select(engine.encode_collect(xd, wd, bd, k, scratch, ws))
    torch.cuda.synchronize()
    assert torch.equal(got.row_ptr.cpu(), ref.row_ptr.cpu())
    assert torch.equal(got.col.cpu(), ref.col.cpu())
    assert torch.equal(got.val.cpu().view(torch.int32 if x.dtype == torch.float32 else torch.int16),
                       ref.val.cpu().view(torch.int32 if x.dtype == torch.float32 else torch.int16))
    return pre.cpu(), got


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("L,T,d,F,k", [(1, 256, 128, 256, 3), (2, 512, 256, 1024, 20), (3, 256, 768, 512, 64),
                                       (2, 768, 128, 2048, 200),
                                       # token counts that are not whole tiles: the last tile is shifted back
                                       (2, 257, 128, 256, 5), (3, 300, 256, 512, 20), (1, 511, 128, 1024, 64),
                                       (2, 1000, 128, 256, 7), (1, 833, 256, 2048, 300),
                                       # an odd number of stages along d
                                       (2, 512, 192, 512, 20), (1, 300, 64, 256, 5), (1, 512, 1600, 512, 16),
                                       # feature counts that are not whole tiles: the last feature tile is shifted back
                                       (2, 256, 128, 384, 9), (1, 300, 128, 520, 30), (2, 512, 64, 1096, 17), (1, 257, 128, 264, 4),
                                       (1, 600, 128, 448, 100), (2, 256, 128, 320, 3),
                                       # more token tiles than feature tiles, in eights: the token-major tile map
                                       (1, 2000, 128, 256, 6), (1, 4000, 64, 520, 11), (2, 2048, 128, 512, 9)])
def test_encode_collect_matches_separate_and_oracle(dev, dtype, L, T, d, F, k):
    g = torch.Generator().manual_seed(L * 31 + T + F + k)
    x = torch.randn(L, T, d, generator=g).to(dtype)
    w = (torch.randn(L, F, d, generator=g) / math.sqrt(d)).to(dtype)
    b = (0.1 * torch.randn(L, F, generator=g)).to(dtype)
    pre, got = fused_vs_separate(x, w, b, k, dev)
    check_rows_sorted(got)
    assert got.nnz == L * min(k * T, T * F)
    assert torch.equal(dense_from(got), oracle_per_layer(pre, k))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T", [512, 333])
def test_encode_collect_heavy_ties(dev, dtype, T):
    # small-integer inputs and weights: the pre-activations are exact small integers, so
    # thousands of them tie at the threshold and the lowest flat indices must win
    g = torch.Generator().manual_seed(5)
    L, d, F, k = 2, 128, 1024, 30
    x = torch.randint(-1, 2, (L, T, d), generator=g).to(dtype)
    w = torch.randint(-1, 2, (L, F, d), generator=g).to(dtype)
    pre, got = fused_vs_separate(x, w, None, k, dev)
    assert torch.equal(dense_from(got), oracle_per_layer(pre, k))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T", [512, 450])
def test_encode_collect_unusable_cut_takes_streaming_route(dev, dtype, T):
    # almost every pre-activation is exactly 0 and K reaches into the zeros: every element
    # reaches the sampled cut, the candidate pool overflows, and the layer must be redone from
    # the dense pre-activations (written to the scratch buffer for that purpose)
    g = torch.Generator().manual_seed(9)
    L, d, F, k = 2, 128, 2048, 8
    x = torch.zeros(L, T, d)
    x[:, ::64] = torch.randn(L, (T + 63) // 64, d, generator=g)
    w = (torch.randn(L, F, d, generator=g) / math.sqrt(d))
    pre, got = fused_vs_separate(x.to(dtype), w.to(dtype), None, k, dev)
    assert got.nnz == L * k * T
    assert torch.equal(dense_from(got), oracle_per_layer(pre, k))


def test_encode_collect_all_selected_and_shape_gate(dev):
    g = torch.Generator().manual_seed(2)
    L, T, d, F = 1, 256, 128, 256
    x = torch.randn(L, T, d, generator=g).to(torch.bfloat16)
    w = torch.randn(L, F, d, generator=g).to(torch.bfloat16)
    pre, got = fused_vs_separate(x, w, None, F + 5, dev)          # k >= F: everything survives
    assert got.nnz == T * F
    # shapes the collecting epilogue does not take
    assert not engine.encode_collect_supported(x[:, :200].contiguous().to(dev), w.to(dev), None, 4)   # less than a tile
    assert not engine.encode_collect_supported(x.to(dev), w[:, :136].contiguous().to(dev), None, 4)
    assert not engine.encode_collect_supported(x.to(dev), w.to(dev), None, 0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("L,T,F,k", [(2, 2, 2, 1), (3, 64, 128, 6), (4, 200, 520, 12)])
def test_batchtopk_global(dev, dtype, L, T, F, k):
    g = torch.Generator().manual_seed(L + T + F)
    pre = (torch.randn(L, T, F, generator=g) * (1 + torch.arange(L).view(L, 1, 1))).to(dtype)
    surv = run_select(pre, k, dev, global_mode=True)
    check_rows_sorted(surv)
    assert surv.nnz == min(k * T, T * F * L)
    got = dense_from(surv)
    ref = orc.global_batchtopk({l: pre[l] for l in range(L)}, L, k)
    ref = torch.stack([ref[l] for l in range(L)])
    # ranking uses per-feature mean/std reductions, whose last-bit rounding differs between
    # implementations: elements whose z-score is within a relative 2^-6 (bf16) / 1e-5 (fp32)
    # of the threshold may legitimately differ; everything else must agree exactly.
    z = torch.cat([orc.zscore_for_ranking(pre[l]) for l in range(L)], dim=1).double()
    flat = z.reshape(-1)
    kth = torch.topk(flat, min(k * T, flat.numel())).values[-1]
    band = BAND[dtype] * max(abs(float(kth)), 1e-3)
    zl = torch.stack([z[:, l * F:(l + 1) * F] for l in range(L)])
    sure = (zl - kth).abs() > band
    assert torch.equal((got != 0) & sure, (ref != 0) & sure)
    assert torch.equal(got[got != 0], torch.stack([pre[l] for l in range(L)])[got != 0])
    if dtype == torch.float32 and (L, T, F) == (2, 2, 2):
        assert torch.equal(got, ref)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("L,T,F,k", [(4, 200, 520, 12), (3, 512, 2048, 20)])
def test_batchtopk_global_is_bit_exact_given_the_column_statistics(dev, dtype, L, T, F, k):
    # The only thing that can differ between two correct implementations of the global helper is the last
    # bit of the per-feature mean / std reductions.  Given the statistics the kernel itself used, the ranking
    # values are fixed (each step rounded to the model dtype, activations.py:283) and the selection must be
    # exactly the k*T largest of them over the [T, L*F] block, ties to the lowest flat index.
    g = torch.Generator().manual_seed(L * 7 + F)
    pre = (torch.randn(L, T, F, generator=g) * (1 + torch.arange(L).view(L, 1, 1))).to(dtype)
    if dtype != torch.float32:
        pre[1, :, 5] = pre[0, :, 5]                 # equal columns: equal z-scores, ties across layers
    pre_dev = pre.to(dev)
    mean, denom = engine.colstats(pre_dev)
    surv = engine.batchtopk_select(pre_dev, k, True, stats=(mean, denom))
    check_rows_sorted(surv)
    got = dense_from(surv) != 0
    mean, denom = mean.cpu(), denom.cpu()
    z = torch.cat([((pre[l].float() - mean[l]).to(dtype).float() / denom[l]).to(dtype).float() for l in range(L)], dim=1)
    order = torch.sort(z.reshape(-1), descending=True, stable=True).indices[:k * T]
    want = torch.zeros(T * L * F, dtype=torch.bool)
    want[order] = True
    want = torch.stack([want.view(T, L * F)[:, l * F:(l + 1) * F] for l in range(L)])
    assert torch.equal(got, want)


@pytest.mark.parametrize("dtype", DTYPES)
def test_batchtopk_global_outlier_tokens(dev, dtype):
    # two tokens stand far out of the batch in every feature: under the batch-wide cut nearly all of
    # their values are candidates, more per step of the streaming pass than its buffer holds
    g = torch.Generator().manual_seed(21)
    L, T, F, k = 2, 256, 4096, 24
    pre = torch.randn(L, T, F, generator=g)
    pre[:, 7] += 9.0
    pre[1, 130] += 12.0
    pre = pre.to(dtype)
    surv = run_select(pre, k, dev, global_mode=True)
    check_rows_sorted(surv)
    assert surv.nnz == k * T
    got = dense_from(surv)
    ref = orc.global_batchtopk({l: pre[l] for l in range(L)}, L, k)
    ref = torch.stack([ref[l] for l in range(L)])
    z = torch.cat([orc.zscore_for_ranking(pre[l]) for l in range(L)], dim=1).double()
    kth = torch.topk(z.reshape(-1), k * T).values[-1]
    band = BAND[dtype] * max(abs(float(kth)), 1e-3)
    zl = torch.stack([z[:, l * F:(l + 1) * F] for l in range(L)])
    sure = (zl - kth).abs() > band
    assert torch.equal((got != 0) & sure, (ref != 0) & sure)
    assert torch.equal(got[got != 0], pre[got != 0])
    # the outlying tokens do hold most of the survivors
    assert int((got[:, 7] != 0).sum()) + int((got[1, 130] != 0).sum()) > k * T // 2


def test_batchtopk_global_closed_form(dev):
    # hand-computed case of tests/test_oracle_pins.py::test_zscore_closed_form_and_global_selection
    pre = torch.tensor([[[0.0, 5.0], [2.0, 5.0]], [[10.0, -1.0], [10.0, 3.0]]])
    got = dense_from(run_select(pre, 1, dev, global_mode=True))
    assert torch.equal(got[0], torch.tensor([[0.0, 0.0], [2.0, 0.0]]))
    assert torch.equal(got[1], torch.tensor([[0.0, 0.0], [0.0, 3.0]]))


# ---- TokenTopK -----------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("L,T,F,kk", [(1, 2, 4, 2), (2, 40, 256, 7), (3, 33, 1000, 50), (1, 5, 77, 77), (2, 9, 64, 100)])
def test_tokentopk_per_layer_bit_exact(dev, dtype, L, T, F, kk):
    g = torch.Generator().manual_seed(T * 3 + F)
    pre = torch.randn(L, T, F, generator=g)
    pre[0, 0, : F // 2] = 0.5                      # ties inside a row
    pre = pre.to(dtype)
    surv = engine.tokentopk_select(pre.to(dev), kk, False)
    check_rows_sorted(surv)
    assert surv.nnz == L * T * min(kk, F)
    for l in range(L):
        m = orc.tokentopk_mask(pre[l], float(kk), pre[l])
        rows = engine.survivor_rows(surv).cpu()
        sel = (rows >= l * T) & (rows < (l + 1) * T)
        flat = (rows[sel] - l * T) * F + surv.col.cpu().long()[sel]
        assert torch.equal(torch.sort(flat).values, m.view(-1).nonzero().view(-1))
    assert torch.equal(dense_from(surv).to(dtype), torch.stack([orc.tokentopk_forward(pre[l], float(kk), pre[l]) for l in range(L)]))


def test_tokentopk_reference_known_answers(dev):
    # reference tests/unit/models/test_activations.py:158-190, 255-272
    x = torch.tensor([[1.0, 2.0, 3.0, 4.0], [5.0, 1.0, 2.5, 3.5]], device=dev)
    m = cca.TokenTopK._compute_mask(x, 0.5).cpu()
    assert torch.equal(m, torch.tensor([[False, False, True, True], [True, False, False, True]]))
    m = cca.TokenTopK._compute_mask(x, 1.0).cpu()
    assert torch.equal(m, torch.tensor([[False, False, False, True], [True, False, False, False]]))
    assert cca.TokenTopK._compute_mask(x, 0.0).sum() == 0 and bool(cca.TokenTopK._compute_mask(x, 5.0).all())
    xx = torch.tensor([[1.0, 2.0, 3.0, 4.0], [10.0, 10.0, 10.0, 10.0]], device=dev)
    r = torch.tensor([[4.0, 3.0, 2.0, 1.0], [1.0, 2.0, 3.0, 4.0]], device=dev)
    out = cca.TokenTopK.apply(xx, 0.5, True, r).cpu()
    assert torch.equal(out, torch.tensor([[1.0, 2.0, 0.0, 0.0], [0.0, 0.0, 10.0, 10.0]]))
    # BatchTopK operator surface too (test_activations.py:66-152)
    xb = torch.tensor([[1.0, 2.0, 3.0, 4.0], [5.0, 1.0, 2.5, 3.5]], device=dev, requires_grad=True)
    ob = cca.BatchTopK.apply(xb, 2.0, True, None)
    assert torch.equal(ob.detach().cpu(), torch.tensor([[0.0, 0.0, 3.0, 4.0], [5.0, 0.0, 0.0, 3.5]]))
    gout = torch.ones_like(ob)
    ob.backward(gout)
    assert torch.equal(xb.grad.cpu(), torch.tensor([[0.0, 0.0, 1.0, 1.0], [1.0, 0.0, 0.0, 1.0]]))


@pytest.mark.parametrize("dtype", DTYPES)
def test_tokentopk_global(dev, dtype):
    g = torch.Generator().manual_seed(4)
    L, T, F, kk = 3, 50, 128, 9
    pre = (torch.randn(L, T, F, generator=g) * (1 + torch.arange(L).view(L, 1, 1))).to(dtype)
    surv = engine.tokentopk_select(pre.to(dev), kk, True)
    check_rows_sorted(surv)
    assert surv.nnz == T * kk
    got = dense_from(surv)
    per_tok = (engine.survivor_rows(surv).cpu() % T).bincount(minlength=T)
    assert torch.equal(per_tok, torch.full((T,), kk))
    ref = orc.global_tokentopk({l: pre[l] for l in range(L)}, L, float(kk))
    ref = torch.stack([ref[l] for l in range(L)])
    z = torch.stack([orc.zscore_for_ranking(pre[l]) for l in range(L)]).double()       # [L, T, F]
    zt = z.permute(1, 0, 2).reshape(T, L * F)
    kth = torch.topk(zt, kk, dim=1).values[:, -1]                                        # per token
    band = BAND[dtype] * kth.abs().clamp(min=1e-3)
    sure = (z - kth.view(1, T, 1)).abs() > band.view(1, T, 1)
    assert torch.equal((got != 0) & sure, (ref != 0) & sure)


# ---- threshold activations ---------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("L,T,F", [(1, 7, 7), (2, 100, 264), (3, 64, 1000)])
def test_jumprelu_and_relu_exact(dev, dtype, L, T, F):
    g = torch.Generator().manual_seed(T + F)
    pre = torch.randn(L, T, F, generator=g).to(dtype)
    log_t = torch.log(torch.rand(L, F, generator=g) + 0.3)
    theta = torch.stack([orc.theta_from_log(log_t[l], dtype) for l in range(L)])
    pre[0, 0, 0] = theta[0, 0]                     # equality must pass
    surv = engine.threshold_select(pre.to(dev), theta.to(dev), nat.PRED_GE_THETA)
    check_rows_sorted(surv)
    got = engine.densify(surv, out_f32=True).cpu()
    ref = torch.stack([orc.jumprelu_forward(pre[l], theta[l]) for l in range(L)])
    assert got.dtype == torch.float32 and torch.equal(got, ref)
    assert got[0, 0, 0] == theta[0, 0].float()
    relu = engine.densify(engine.threshold_select(pre.to(dev), None, nat.PRED_GT_ZERO)).cpu()
    assert torch.equal(relu, torch.relu(pre))
    nz = engine.densify(engine.threshold_select(relu.to(dev), None, nat.PRED_NONZERO)).cpu()
    assert torch.equal(nz, relu)


def test_jumprelu_reference_known_answer(dev):
    # reference tests/unit/models/test_activations.py:304-315
    x = torch.tensor([-2.0, -1.0, -0.4, 0.0, 0.4, 1.0, 2.0], device=dev)
    out = cca.JumpReLU.apply(x, torch.tensor([0.5], device=dev), 1.0)
    assert torch.equal(out.cpu(), torch.tensor([0.0, 0.0, 0.0, 0.0, 0.0, 1.0, 2.0]))


# ---- pack / densify / norms -------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
def test_pack_is_transpose(dev, dtype):
    w = torch.randn(70, 130).to(dtype)
    out = engine.alloc_packed(1, 130, 70, dtype, dev)[0]
    engine.pack_decoder(w.to(dev), out)
    assert torch.equal(out.cpu()[:, :70], w.T.contiguous())
    # a row of whole, evenly many cache lines gets one more line of pitch; the matrix sits in the leading columns
    w2 = torch.randn(128, 40).to(dtype)
    out2 = engine.alloc_packed(1, 40, 128, dtype, dev)[0]
    assert out2.shape[1] == 128 + 128 // w2.element_size()
    engine.pack_decoder(w2.to(dev), out2)
    assert torch.equal(out2.cpu()[:, :128], w2.T.contiguous()) and float(out2[:, 128:].abs().max()) == 0.0


# ---- sparse decode -------------------------------------------------------------------------------
def make_decoder(L, d, F, tying, dtype, g):
    names = [f"{s}->{t}" for s in range(L) for t in range(s, L)] if tying == "none" else [str(i) for i in range(L)]
    w = {n: (torch.randn(d, F, generator=g) / math.sqrt(F)).to(dtype) for n in names}
    b = {n: torch.randn(d, generator=g).to(dtype) for n in names}
    return names, w, b


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("tying", ["none", "per_source", "per_target"])
@pytest.mark.parametrize("L,T,d,F", [(2, 30, 8, 16), (3, 70, 768, 256), (4, 33, 100, 72), (3, 20, 2048, 64)])
def test_decode_sparse_parity(dev, dtype, tying, L, T, d, F):
    g = torch.Generator().manual_seed(L * 31 + d)
    names, w, b = make_decoder(L, d, F, tying, dtype, g)
    acts = torch.randn(L, T, F, generator=g) * (torch.rand(L, T, F, generator=g) < 0.1)
    acts = acts.to(dtype)
    tied = tying != "none"
    off = torch.randn(L, F, generator=g).to(dtype) if tied else None
    sc = torch.randn(L, F, generator=g).to(dtype) if tied else None
    surv = engine.threshold_select(acts.to(dev), None, nat.PRED_NONZERO)
    slab = engine.alloc_packed(len(names), F, d, dtype, dev)
    for i, n in enumerate(names):
        engine.pack_decoder(w[n].to(dev), slab[i])
    B = torch.stack([b[n].float() for n in names])
    bias_sum = torch.zeros(L, d)
    for t in range(L):
        if tying == "none":
            for s in range(t + 1):
                bias_sum[t] += B[names.index(f"{s}->{t}")]
        elif tying == "per_source":
            bias_sum[t] = B[: t + 1].sum(0)
        else:
            bias_sum[t] = B[t]
    got = engine.decode_sparse(surv, slab, tying, d, bias_sum=bias_sum.to(dev),
                               feat_offset=off.to(dev) if tied else None,
                               feat_scale=sc.to(dev) if tied else None).cpu()
    for t in range(L):
        ref = orc.decode({s: acts[s] for s in range(L)}, t, tying=tying, weights=w, biases=b, d_model=d,
                         num_features=F, dtype=dtype,
                         feature_offset=list(off) if tied else None, feature_scale=list(sc) if tied else None)
        assert orc.rel_l2(got[t], ref) <= TOL[dtype], (t, orc.rel_l2(got[t], ref))
    # fp32 output and a source subset
    mask = 0b101 if L >= 3 else 0b01
    sub = engine.decode_sparse(surv, slab, tying, d, src_mask=mask, out_f32=True).cpu()
    t = L - 1
    zero_b = {n: torch.zeros_like(v) for n, v in b.items()}
    ref = orc.decode({s: acts[s] for s in range(L) if (mask >> s) & 1}, t, tying=tying, weights=w, biases=zero_b,
                     d_model=d, num_features=F, dtype=dtype)
    if tying != "per_target":
        assert sub.dtype == torch.float32 and orc.rel_l2(sub[t], ref) <= TOL[dtype]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("tying,d", [("none", 768), ("per_source", 768), ("none", 1024), ("none", 512), ("per_source", 2048),
                                     ("none", 640), ("per_source", 320), ("per_target", 768), ("none", 192),
                                     ("per_source", 4096), ("none", 200)])
def test_decode_sliced_matches_single_pass(dev, dtype, tying, d):
    # the XCD-sliced schedules (workspace given) against the one-wavefront-per-row kernel and the oracle:
    # d a multiple of 256 takes the quarter-row kernel (2 feature slices x 4 column quarters); other widths
    # that are whole cache lines take the line kernel (640 and 320: 10 / 5 column parts in bf16, dealt to the
    # XCDs in rounds with a remainder; 192: 3 parts, all XCDs share each; 4096: more columns than the
    # whole-row kernels hold); per-target tying and the remaining widths take the 8-slice kernel
    g = torch.Generator().manual_seed(21)
    L, T, F = 3, 161, 1024
    names, w, b = make_decoder(L, d, F, tying, dtype, g)
    acts = (torch.randn(L, T, F, generator=g) * (torch.rand(L, T, F, generator=g) < 0.05)).to(dtype)
    acts[0, 5] = 0                                     # an empty row
    acts[1, 7, :] = torch.randn(F, generator=g).to(dtype)   # a full row (more than 64 per slice)
    surv = engine.threshold_select(acts.to(dev), None, nat.PRED_NONZERO)
    slab = engine.alloc_packed(len(names), F, d, dtype, dev)
    for i, n in enumerate(names):
        engine.pack_decoder(w[n].to(dev), slab[i])
    bias = torch.randn(L, d, generator=g)
    skip = torch.randn(L, T, d, generator=g)
    ws = engine.Workspace(dev)
    old = engine.SLICED_DECODE_MIN_ROWS
    try:
        engine.SLICED_DECODE_MIN_ROWS = 1
        sliced = engine.decode_sparse(surv, slab, tying, d, bias_sum=bias.to(dev), skip_add=skip.to(dev), ws=ws)
        sliced32 = engine.decode_sparse(surv, slab, tying, d, out_f32=True, t_begin=1, t_end=3, src_mask=0b110, ws=ws)
    finally:
        engine.SLICED_DECODE_MIN_ROWS = old
    single = engine.decode_sparse(surv, slab, tying, d, bias_sum=bias.to(dev), skip_add=skip.to(dev))
    single32 = engine.decode_sparse(surv, slab, tying, d, out_f32=True, t_begin=1, t_end=3, src_mask=0b110)
    assert orc.rel_l2(sliced, single) <= (1e-6 if dtype == torch.float32 else 4e-3)
    assert orc.rel_l2(sliced32[1:], single32[1:]) <= 1e-6
    zero_b = {n: torch.zeros(d, dtype=dtype) for n in names}
    for t in range(L):
        ref = orc.decode({s: acts[s] for s in range(L)}, t, tying=tying, weights=w, biases=zero_b, d_model=d,
                         num_features=F, dtype=dtype).float() + bias[t] + skip[t]
        assert orc.rel_l2(sliced[t], ref) <= TOL[dtype]


@pytest.mark.parametrize("dtype", DTYPES)
def test_decode_line_schedule_with_feature_slices(dev, dtype):
    # F x 128 bytes above 3.25 MiB: the line kernel cuts the feature axis in two and keeps two partial rows
    g = torch.Generator().manual_seed(4)
    L, T, F, d = 2, 300, 28672, 192
    assert engine.decode_route(T, d, F, L, "none", dtype, rows=10 ** 6) == nat.ROUTE_LINE
    names, w, b = make_decoder(L, d, F, "none", dtype, g)
    acts = torch.zeros(L, T, F)
    for l in range(L):
        for t in range(T):
            idx = torch.randint(0, F, (40,), generator=g)
            acts[l, t, idx] = torch.randn(40, generator=g)
    acts[1, 3] = 0
    acts = acts.to(dtype)
    surv = engine.threshold_select(acts.to(dev), None, nat.PRED_NONZERO)
    slab = engine.alloc_packed(len(names), F, d, dtype, dev)
    for i, n in enumerate(names):
        engine.pack_decoder(w[n].to(dev), slab[i])
    ws = engine.Workspace(dev)
    old = engine.SLICED_DECODE_MIN_ROWS
    try:
        engine.SLICED_DECODE_MIN_ROWS = 1
        sliced = engine.decode_sparse(surv, slab, "none", d, out_f32=True, ws=ws)
    finally:
        engine.SLICED_DECODE_MIN_ROWS = old
    single = engine.decode_sparse(surv, slab, "none", d, out_f32=True)
    assert orc.rel_l2(sliced, single) <= 1e-6
    zero_b = {n: torch.zeros(d, dtype=dtype) for n in names}
    for t in range(L):
        ref = orc.decode({s: acts[s] for s in range(L)}, t, tying="none", weights=w, biases=zero_b, d_model=d,
                         num_features=F, dtype=dtype).float()
        assert orc.rel_l2(sliced[t].cpu(), ref) <= TOL[dtype]


def test_decode_linearity_property(dev):
    # decode(2 * a) - bias == 2 * (decode(a) - bias), exact in fp32 for power-of-two scaling
    g = torch.Generator().manual_seed(2)
    L, T, d, F = 3, 64, 768, 512
    names, w, b = make_decoder(L, d, F, "none", torch.float32, g)
    acts = torch.randn(L, T, F, generator=g) * (torch.rand(L, T, F, generator=g) < 0.05)
    slab = engine.alloc_packed(len(names), F, d, torch.float32, dev)
    for i, n in enumerate(names):
        engine.pack_decoder(w[n].to(dev), slab[i])
    s1 = engine.threshold_select(acts.to(dev), None, nat.PRED_NONZERO)
    s2 = engine.threshold_select((2 * acts).to(dev), None, nat.PRED_NONZERO)
    o1 = engine.decode_sparse(s1, slab, "none", d)
    o2 = engine.decode_sparse(s2, slab, "none", d)
    assert torch.equal(o2, 2 * o1)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("tying", ["none", "per_source", "per_target"])
def test_decoder_norms(dev, dtype, tying):
    g = torch.Generator().manual_seed(8)
    L, d, F = 3, 40, 50
    names, w, _ = make_decoder(L, d, F, tying, dtype, g)
    slab = engine.alloc_packed(len(names), F, d, dtype, dev)
    for i, n in enumerate(names):
        engine.pack_decoder(w[n].to(dev), slab[i])
    got = engine.decoder_norms(slab, L, tying, d).cpu()
    ref = orc.decoder_norms(w, L, F, tying, dtype)
    assert orc.rel_l2(got, ref) <= TOL[dtype]


def test_gather_probe_runs_and_rejects_bad_arguments(dev):
    # calibration entry point: results are not meaningful numbers, the call must just be safe
    from crosslayer_coding_amd import _native as nat
    lib = nat.load()
    table = torch.arange(64 * 1536 // 4, dtype=torch.int32, device=dev)
    idx = torch.tensor([0, 63, 5, 1 << 20, -3], dtype=torch.int32, device=dev)     # two indices outside the table: clamped
    out = torch.empty(8 * 256, dtype=torch.float32, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    for to_lds in (0, 1):
        assert lib.clt_probe_gather(table.data_ptr(), 64, 1536, idx.data_ptr(), 5, 8, to_lds, out.data_ptr(), stream) == 0
    torch.cuda.synchronize()
    assert torch.isfinite(out).all()
    assert lib.clt_probe_gather(table.data_ptr(), 64, 1530, idx.data_ptr(), 5, 8, 0, out.data_ptr(), stream) != 0   # not 16-byte rows
    assert lib.clt_probe_gather(table.data_ptr(), 64, 512, idx.data_ptr(), 5, 8, 1, out.data_ptr(), stream) != 0    # LDS variant needs >= 1 KB
    assert lib.clt_probe_gather(None, 64, 1536, idx.data_ptr(), 5, 8, 0, out.data_ptr(), stream) != 0
