"""Pins the CPU oracle: the reference's own known-answer vectors, brute force on small
inputs, and closed forms.  Vector sources are cited per test (paths relative to the
reference checkout)."""
import math

import numpy as np
import pytest
import torch

from oracle import clt_oracle as orc


# ---- BatchTopK: reference tests/unit/models/test_activations.py -------------------------
def test_batchtopk_mask_known_answer():
    # test_activations.py:10-25 : indices {3, 4, 7, 2}
    x = torch.tensor([[1.0, 2.0, 3.0, 4.0], [5.0, 1.0, 2.5, 3.5]])
    mask = orc.batchtopk_mask(x, 2)
    expect = torch.zeros(8, dtype=torch.bool)
    expect[torch.tensor([3, 4, 7, 2])] = True
    assert mask.dtype == torch.bool and mask.shape == x.shape
    assert torch.equal(mask.view(-1), expect)


def test_batchtopk_edge_cases():
    # test_activations.py:28-63
    x = torch.randn(2, 4)
    assert orc.batchtopk_mask(x, 0).sum() == 0
    assert bool(orc.batchtopk_mask(x, 4).all())
    assert bool(orc.batchtopk_mask(x, 5).all())
    assert orc.batchtopk_mask(torch.empty(0, 4), 2).shape == (0, 4)
    assert orc.batchtopk_mask(torch.empty(2, 0), 2).shape == (2, 0)


def test_batchtopk_forward_known_answer():
    # test_activations.py:66-90 : [[0,0,3,4],[5,0,0,3.5]]
    x = torch.tensor([[1.0, 2.0, 3.0, 4.0], [5.0, 1.0, 2.5, 3.5]])
    out = orc.batchtopk_forward(x, 2.0)
    assert torch.equal(out, torch.tensor([[0.0, 0.0, 3.0, 4.0], [5.0, 0.0, 0.0, 3.5]]))


def test_batchtopk_ranking_override_known_answer():
    # test_activations.py:92-111 : the second row is selected, the values come from x
    x = torch.tensor([[1.0, 2.0, 3.0, 4.0], [0.0, 0.0, 0.0, 0.0]])
    r = torch.tensor([[0.0, 0.0, 0.0, 0.0], [5.0, 6.0, 7.0, 8.0]])
    mask = orc.batchtopk_mask(x, 2, r)
    assert torch.equal(mask, torch.tensor([[False] * 4, [True] * 4]))
    assert torch.equal(orc.batchtopk_forward(x, 2.0, r), torch.zeros(2, 4))


def test_batchtopk_keeps_negatives():
    x = torch.tensor([[-1.0, -2.0, -3.0]])
    assert torch.equal(orc.batchtopk_forward(x, 2.0), torch.tensor([[-1.0, -2.0, 0.0]]))


def _brute_force_topk(values, k_total):
    """Independent selector: python sort on (value desc, index asc) with explicit float rules."""
    def sort_key(iv):
        i, v = iv
        if math.isnan(v):
            return (0, 0.0, i)       # NaN first (largest)
        return (1, -(v + 0.0), i)    # -0.0 + 0.0 == +0.0
    order = sorted(enumerate(values), key=sort_key)
    return sorted(i for i, _ in order[:k_total])


@pytest.mark.parametrize("seed", range(6))
def test_batchtopk_matches_brute_force_with_ties(seed):
    g = torch.Generator().manual_seed(seed)
    B, F, k = 7, 13, 3
    x = torch.randint(-3, 4, (B, F), generator=g).float() * 0.5   # heavy ties
    if seed % 2:
        x[0, 0], x[1, 1] = float("nan"), float("inf")
        x[2, 2], x[3, 3] = -0.0, 0.0
    got = orc.batchtopk_mask(x, k).view(-1).nonzero().view(-1).tolist()
    assert got == _brute_force_topk(x.view(-1).tolist(), k * B)


def test_batchtopk_invariants_bf16():
    g = torch.Generator().manual_seed(3)
    x = torch.randn(32, 64, generator=g).to(torch.bfloat16)
    mask = orc.batchtopk_mask(x, 5)
    assert int(mask.sum()) == 5 * 32
    assert float(x[mask].float().min()) >= float(x[~mask].float().max())


# ---- TokenTopK: test_activations.py:158-283 ------------------------------------------------
def test_tokentopk_known_answers():
    x = torch.tensor([[1.0, 2.0, 3.0, 4.0], [5.0, 1.0, 2.5, 3.5]])
    assert torch.equal(orc.tokentopk_mask(x, 0.5),
                       torch.tensor([[False, False, True, True], [True, False, False, True]]))
    assert torch.equal(orc.tokentopk_mask(x, 1.0),
                       torch.tensor([[False, False, False, True], [True, False, False, False]]))
    assert orc.tokentopk_mask(x, 0.0).sum() == 0 and orc.tokentopk_mask(x, -0.5).sum() == 0
    assert bool(orc.tokentopk_mask(x, 4.0).all()) and bool(orc.tokentopk_mask(x, 5.0).all())
    y = torch.randn(2, 5)
    assert orc.tokentopk_mask(y, 0.6).sum(dim=1).tolist() == [3, 3]   # ceil(3.0)
    assert orc.tokentopk_mask(y, 0.5).sum(dim=1).tolist() == [3, 3]   # ceil(2.5)
    assert orc.tokentopk_mask(torch.empty(0, 4), 0.5).shape == (0, 4)


def test_tokentopk_ranking_override_known_answer():
    # test_activations.py:255-272
    x = torch.tensor([[1.0, 2.0, 3.0, 4.0], [10.0, 10.0, 10.0, 10.0]])
    r = torch.tensor([[4.0, 3.0, 2.0, 1.0], [1.0, 2.0, 3.0, 4.0]])
    assert torch.equal(orc.tokentopk_forward(x, 0.5, r), torch.tensor([[1.0, 2.0, 0.0, 0.0], [0.0, 0.0, 10.0, 10.0]]))


# ---- JumpReLU: test_activations.py:304-315, test_theta.py:79-92 --------------------------------
def test_jumprelu_known_answer():
    x = torch.tensor([-2.0, -1.0, -0.4, 0.0, 0.4, 1.0, 2.0])
    out = orc.jumprelu_forward(x, torch.tensor([0.5]))
    assert torch.equal(out, torch.tensor([0.0, 0.0, 0.0, 0.0, 0.0, 1.0, 2.0]))
    assert out.dtype == torch.float32


def test_jumprelu_is_where_ge_theta_and_fp32():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(10, 16, generator=g).to(torch.bfloat16)
    log_t = torch.full((16,), math.log(0.5))
    theta = orc.theta_from_log(log_t, torch.bfloat16)
    out = orc.jumprelu_forward(x, theta)
    assert out.dtype == torch.float32
    assert torch.equal(out, torch.where(x >= theta, x, torch.zeros_like(x)).float())
    x[0, 0] = theta[0]      # equality passes (>=)
    assert orc.jumprelu_forward(x, theta)[0, 0] == theta[0].float()


# ---- encoder: affine map ---------------------------------------------------------------------
def test_encoder_matches_float64_contraction():
    g = torch.Generator().manual_seed(1)
    x, w, b = torch.randn(9, 8, generator=g), torch.randn(16, 8, generator=g), torch.randn(16, generator=g)
    got = orc.encoder_preactivations(x, w, b)
    ref = orc.affine_f64(x.numpy(), w.numpy(), b.numpy())
    assert np.allclose(got.numpy(), ref, rtol=1e-5, atol=1e-5)
    assert orc.encoder_preactivations(x.view(3, 3, 8), w, b).shape == (9, 16)
    # transposed-operand mistake would fail this: a one-hot input picks a weight column
    e = torch.zeros(1, 8); e[0, 2] = 1.0
    assert torch.allclose(orc.encoder_preactivations(e, w, None)[0], w[:, 2])


# ---- global helper: closed form of the z-score -----------------------------------------------
def test_zscore_closed_form_and_global_selection():
    # column 0: values 0,2 -> mean 1, unbiased std sqrt(2); column 1 constant -> std 0 -> /1e-6
    pre = torch.tensor([[0.0, 5.0], [2.0, 5.0]])
    z = orc.zscore_for_ranking(pre)
    s = math.sqrt(2.0)
    assert torch.allclose(z[:, 0], torch.tensor([-1.0 / (s + 1e-6), 1.0 / (s + 1e-6)]))
    assert torch.equal(z[:, 1], torch.zeros(2))
    # two layers, k=1 per token -> 2 survivors over the [2, 4] block ranked on z, raw values kept
    pre0 = torch.tensor([[0.0, 5.0], [2.0, 5.0]])
    pre1 = torch.tensor([[10.0, -1.0], [10.0, 3.0]])
    out = orc.global_batchtopk({0: pre0, 1: pre1}, 2, 1)
    # z: layer0 col0 = -.707/+.707, col1 = 0,0 ; layer1 col0 = 0,0, col1 = -.707/+.707
    # top-2 z are (t=1,l=0,f=0) and (t=1,l=1,f=1); the large raw 10.0 is not selected
    assert torch.equal(out[0], torch.tensor([[0.0, 0.0], [2.0, 0.0]]))
    assert torch.equal(out[1], torch.tensor([[0.0, 0.0], [0.0, 3.0]]))


# ---- decoder -------------------------------------------------------------------------------------
def _dec_params(L, d, F, tying, g, dtype=torch.float32):
    names = [f"{s}->{t}" for s in range(L) for t in range(s, L)] if tying == "none" else [str(i) for i in range(L)]
    w = {n: torch.randn(d, F, generator=g).to(dtype) for n in names}
    b = {n: torch.randn(d, generator=g).to(dtype) for n in names}
    return w, b


def test_decode_additivity_and_loop_reference():
    # additivity over sources: reference tests/unit/models/test_decoder.py:62-81
    g = torch.Generator().manual_seed(2)
    L, d, F, T = 3, 4, 6, 5
    w, b = _dec_params(L, d, F, "none", g)
    a = {s: torch.randn(T, F, generator=g) * (torch.rand(T, F, generator=g) > 0.5) for s in range(L)}
    kw = dict(tying="none", weights=w, biases=b, d_model=d, num_features=F, dtype=torch.float32)
    full = orc.decode(a, 2, **kw)
    parts = sum(orc.decode({s: a[s]}, 2, **kw) for s in range(3))
    assert torch.allclose(full, parts, atol=1e-5)
    # explicit float64 loops (target 1: sources 0 and 1, one bias per decoder)
    ref = np.zeros((T, d))
    for s in (0, 1):
        W = w[f"{s}->1"].double().numpy()
        for tok in range(T):
            for f in range(F):
                ref[tok] += float(a[s][tok, f]) * W[:, f]
        ref += b[f"{s}->1"].double().numpy()
    assert np.allclose(orc.decode(a, 1, **kw).numpy(), ref, atol=1e-5)
    assert orc.decode({}, 1, **kw).shape == (0, d)                    # test_decoder.py:83-92
    bad = dict(a); bad[1] = torch.randn(T, F + 1)                      # test_decoder.py:94-112
    assert torch.allclose(orc.decode(bad, 1, **kw), orc.decode({0: a[0]}, 1, **kw))


def test_decode_tied_variants():
    g = torch.Generator().manual_seed(4)
    L, d, F, T = 3, 4, 6, 5
    a = {s: torch.randn(T, F, generator=g) * (torch.rand(T, F, generator=g) > 0.5) for s in range(L)}
    # zero-initialised tied decoders give zero output (test_tied_decoders.py:138-166)
    zw = {str(i): torch.zeros(d, F) for i in range(L)}
    zb = {str(i): torch.zeros(d) for i in range(L)}
    for tying in ("per_source", "per_target"):
        out = orc.decode(a, 2, tying=tying, weights=zw, biases=zb, d_model=d, num_features=F, dtype=torch.float32)
        assert torch.equal(out, torch.zeros(T, d))
    w, b = _dec_params(L, d, F, "per_target", g)
    off = [torch.randn(F, generator=g) for _ in range(L)]
    sc = [torch.randn(F, generator=g) for _ in range(L)]
    out = orc.decode(a, 1, tying="per_target", weights=w, biases=b, d_model=d, num_features=F,
                     dtype=torch.float32, feature_offset=off, feature_scale=sc)
    summed = torch.zeros(T, F)
    for s in (0, 1):
        summed += torch.where(a[s] != 0, (a[s] + off[1]) * sc[1], torch.zeros(()))
    assert torch.allclose(out, summed @ w["1"].T + b["1"], atol=1e-5)
    out_ps = orc.decode(a, 1, tying="per_source", weights=w, biases=b, d_model=d, num_features=F,
                        dtype=torch.float32, feature_offset=off, feature_scale=sc)
    ref = sum(torch.where(a[s] != 0, (a[s] + off[1]) * sc[1], torch.zeros(())) @ w[str(s)].T + b[str(s)] for s in (0, 1))
    assert torch.allclose(out_ps, ref, atol=1e-5)


def test_decoder_norms_closed_form():
    L, d, F = 2, 2, 2
    w = {"0->0": torch.tensor([[3.0, 0.0], [4.0, 1.0]]), "0->1": torch.tensor([[0.0, 2.0], [0.0, 0.0]]),
         "1->1": torch.tensor([[1.0, 1.0], [1.0, 1.0]])}
    n = orc.decoder_norms(w, L, F, "none", torch.float32)
    assert torch.allclose(n, torch.tensor([[5.0, math.sqrt(5.0)], [math.sqrt(2.0), math.sqrt(2.0)]]))


def test_forward_wiring_small():
    g = torch.Generator().manual_seed(5)
    L, d, F, T = 2, 8, 16, 30
    enc_w = [torch.randn(F, d, generator=g) for _ in range(L)]
    enc_b = [torch.randn(F, generator=g) for _ in range(L)]
    w, b = _dec_params(L, d, F, "none", g)
    x = {l: torch.randn(T, d, generator=g) for l in range(L)}
    recs, acts = orc.forward(x, enc_w=enc_w, enc_b=enc_b, dec_w=w, dec_b=b, activation_fn="batchtopk",
                             dtype=torch.float32, num_layers=L, d_model=d, num_features=F, k=3, topk_mode="global")
    assert set(recs) == {0, 1} and recs[0].shape == (T, d) and acts[1].shape == (T, F)
    assert sum(int((a != 0).sum()) for a in acts.values()) == 3 * T
    r1 = acts[0] @ w["0->1"].T + b["0->1"] + acts[1] @ w["1->1"].T + b["1->1"]
    assert torch.allclose(recs[1], r1, atol=1e-5)


# ---- post-hoc theta estimation: hand-computed case + the reference test's properties ------------
def test_theta_estimation_hand_computed():
    # one layer, two features, four tokens, k = 1 per token -> 4 survivors over the [4, 2] block.
    # feature 0: 10, 11, 12, 13  (mean 11.5, unbiased std sqrt(5/3)); feature 1: 0, 0, 0, 4 (mean 1, std 2)
    pre = {0: torch.tensor([[10.0, 0.0], [11.0, 0.0], [12.0, 0.0], [13.0, 4.0]])}
    s, c, mu, sg = orc.theta_estimate_posthoc([pre], activation_fn="batchtopk", k=1, num_layers=1, num_features=2,
                                              dtype=torch.float32)
    sd0 = math.sqrt(5.0 / 3.0)
    z0 = [(v - 11.5) / (sd0 + 1e-6) for v in (10.0, 11.0, 12.0, 13.0)]      # -1.16, -0.39, 0.39, 1.16
    z1 = [(v - 1.0) / (2.0 + 1e-6) for v in (0.0, 0.0, 0.0, 4.0)]           # -0.5, -0.5, -0.5, 1.5
    # the four largest z-scores: 1.5 (f1,t3), 1.16 (f0,t3), 0.39 (f0,t2), then -0.39 (f0,t1)
    assert c.tolist() == [[1.0, 1.0]]
    assert abs(float(s[0, 0]) - z0[1]) < 1e-6 and abs(float(s[0, 1]) - z1[3]) < 1e-6
    assert torch.allclose(mu, torch.tensor([[11.5, 1.0]])) and torch.allclose(sg, torch.tensor([[sd0, 2.0]]))
    # conversion: feature 0's theta is negative, so the layer scalar is the mean of the positive ones = z1[3]
    log_t = orc.theta_convert(s, c, mu, sg)
    expect = torch.tensor([[z1[3] * sd0 + 11.5, z1[3] * 2.0 + 1.0]])
    assert torch.allclose(torch.exp(log_t), expect, rtol=1e-5)


def test_theta_estimation_reference_test_properties():
    # reference tests/unit/models/test_theta.py:110-175: consistently selected features end up with
    # higher thresholds than the others; all thresholds finite and positive
    g = torch.Generator().manual_seed(0)
    l0 = torch.cat([torch.randn(4, 2, generator=g) + 5, torch.randn(4, 2, generator=g)], dim=1)
    l1 = torch.cat([torch.randn(4, 2, generator=g), torch.randn(4, 2, generator=g) + 5], dim=1)
    s, c, mu, sg = orc.theta_estimate_posthoc([{0: l0, 1: l1}], activation_fn="batchtopk", k=2, num_layers=2,
                                              num_features=4, dtype=torch.float32)
    theta = torch.exp(orc.theta_convert(s, c, mu, sg))
    assert bool(torch.isfinite(theta).all()) and bool((theta > 0).all())
    assert bool((theta[0, :2].min() > theta[0, 2:].max())) and bool((theta[1, 2:].min() > theta[1, :2].max()))


# ---- MSE loss gradients: finite differences in float64 on a tiny model ---------------------------
@pytest.mark.parametrize("tying", ["none", "per_source", "per_target"])
def test_mse_gradients_match_finite_differences(tying):
    g = torch.Generator().manual_seed(3)
    L, T, d, F_, k = 2, 6, 3, 5, 2
    x = {l: torch.randn(T, d, generator=g) for l in range(L)}
    tgt = {l: torch.randn(T, d, generator=g) for l in range(L)}
    enc_w = [torch.randn(F_, d, generator=g) for _ in range(L)]
    enc_b = [0.1 * torch.randn(F_, generator=g) for _ in range(L)]
    names = ["0->0", "0->1", "1->1"] if tying == "none" else ["0", "1"]
    dec_w = {n: torch.randn(d, F_, generator=g) for n in names}
    dec_b = {n: 0.1 * torch.randn(d, generator=g) for n in names}
    loss, grads = orc.mse_loss_and_gradients(x, tgt, enc_w=enc_w, enc_b=enc_b, dec_w=dec_w, dec_b=dec_b,
                                             activation_fn="batchtopk", num_layers=L, k=k, tying=tying)
    masks = {l: orc.batchtopk_mask(torch.nn.functional.linear(x[l], enc_w[l], enc_b[l]), k) for l in range(L)}

    def loss64(ew, eb, dw, db):     # independent float64 numpy forward with the gate held fixed
        acts = {l: (x[l].double().numpy() @ ew[l].T + eb[l]) * masks[l].numpy() for l in range(L)}
        total = 0.0
        for t in range(L):
            if tying == "none":
                rec = sum(acts[s] @ dw[f"{s}->{t}"].T + db[f"{s}->{t}"] for s in range(t + 1))
            elif tying == "per_source":      # the source's decoder and bias, once per contributing source
                rec = sum(acts[s] @ dw[str(s)].T + db[str(s)] for s in range(t + 1))
            else:                            # the target's decoder over the summed activations, bias once
                rec = sum(acts[s] for s in range(t + 1)) @ dw[str(t)].T + db[str(t)]
            total += float(np.mean((rec - tgt[t].double().numpy()) ** 2))
        return total

    ew = [w.double().numpy().copy() for w in enc_w]; eb = [b.double().numpy().copy() for b in enc_b]
    dw = {n: w.double().numpy().copy() for n, w in dec_w.items()}; db = {n: b.double().numpy().copy() for n, b in dec_b.items()}
    assert abs(loss64(ew, eb, dw, db) - float(loss)) < 1e-5
    eps = 1e-6
    wn, bn = (("0->1", "1->1") if tying == "none" else ("0", "1"))
    checks = [("encoder_module.encoders.0.weight", ew[0], (1, 2)), ("encoder_module.encoders.1.bias_param", eb[1], (3,)),
              (f"decoder_module.decoders.{wn}.weight", dw[wn], (2, 4)), (f"decoder_module.decoders.{bn}.bias_param", db[bn], (0,)),
              (f"decoder_module.decoders.{wn}.bias_param", db[wn], (1,))]
    for name, arr, idx in checks:
        old = arr[idx]
        arr[idx] = old + eps; up = loss64(ew, eb, dw, db)
        arr[idx] = old - eps; dn = loss64(ew, eb, dw, db)
        arr[idx] = old
        fd = (up - dn) / (2 * eps)
        assert abs(fd - float(grads[name][idx])) <= 1e-4 * max(1.0, abs(fd)), (name, fd, float(grads[name][idx]))


def test_evaluator_reductions_hand_computed():
    # layer 0: 3 tokens x 4 features; layer 1 the same shape, one feature never fires
    a0 = torch.tensor([[0.0, 2.0, -1.0, 0.0], [1e-7, 0.0, 3.0, 0.0], [0.0, 0.0, 0.5, 0.0]])
    a1 = torch.tensor([[1.0, 1.0, 0.0, 0.0], [1.0, 0.0, 0.0, 0.0], [1.0, 0.0, 0.0, 0.0]])
    sp = orc.sparsity_metrics({0: a0, 1: a1}, num_features=4, num_layers=2)
    # non-zeros per token: layer 0 -> 2, 2, 1 (the 1e-7 and the negative count); layer 1 -> 2, 1, 1
    assert sp["layerwise/l0"]["layer_0"] == pytest.approx(5 / 3)
    assert sp["layerwise/l0"]["layer_1"] == pytest.approx(4 / 3)
    assert sp["sparsity/total_l0"] == pytest.approx(3.0)
    assert sp["sparsity/avg_l0"] == pytest.approx(1.5)
    assert sp["sparsity/sparsity_fraction"] == pytest.approx(1 - 1.5 / 4)
    fd = orc.feature_density_metrics({0: a0, 1: a1})
    # firing (> 1e-6): layer 0 feature counts 0, 1, 2, 0 (1e-7 and -1 do not fire)
    want = [math.log10(c / 3 + 1e-10) for c in (0, 1, 2, 0)]
    assert fd["layerwise/log_feature_density"]["layer_0"] == pytest.approx(want, rel=1e-6)
    assert fd["layerwise/consistent_activation_heuristic"]["layer_0"] == pytest.approx([0, 1, 2, 0])
    assert fd["layerwise/consistent_activation_heuristic"]["layer_1"] == pytest.approx([3, 1, 0, 0])
    n = torch.tensor([[5, 5, 5, 5], [0, 2, 7, 1]])
    got = orc.dead_feature_update(n, {0: a0, 1: a1})
    assert got.tolist() == [[6, 0, 0, 6], [0, 0, 8, 2]]
    # a layer that is absent keeps its counters
    assert orc.dead_feature_update(n, {1: a1}).tolist() == [[5, 5, 5, 5], [0, 0, 8, 2]]
    empty = orc.sparsity_metrics({}, 4, 2)
    assert empty["sparsity/sparsity_fraction"] == 1.0 and empty["layerwise/l0"] == {"layer_0": 0.0, "layer_1": 0.0}


def test_reconstruction_metrics_closed_forms_and_numpy():
    g = torch.Generator().manual_seed(3)
    tgt = {0: torch.randn(50, 6, generator=g) * 2 + 1, 1: torch.randn(50, 6, generator=g)}
    rec = {l: t + 0.3 * torch.randn(50, 6, generator=g) for l, t in tgt.items()}
    # perfect reconstruction: EV 1, NMSE 0
    m = orc.reconstruction_metrics(tgt, tgt)
    assert m["reconstruction/explained_variance"] == pytest.approx(1.0)
    assert m["reconstruction/normalized_mean_reconstruction_error"] == pytest.approx(0.0)
    # numpy float64: per-column population variances
    m = orc.reconstruction_metrics(tgt, rec)
    for l in (0, 1):
        t, r = tgt[l].double().numpy(), rec[l].double().numpy()
        tvar, evar = np.var(t, axis=0).mean(), np.var(t - r, axis=0).mean()
        assert m["layerwise/explained_variance"][f"layer_{l}"] == pytest.approx(1 - evar / tvar, rel=1e-5)
        assert m["layerwise/normalized_mse"][f"layer_{l}"] == pytest.approx(((t - r) ** 2).mean() / tvar, rel=1e-5)
    # an all-zero reconstruction of a centred target: MSE equals the variance, NMSE 1, EV 0
    c = {0: tgt[1] - tgt[1].mean(dim=0, keepdim=True)}
    z = orc.reconstruction_metrics(c, {0: torch.zeros_like(c[0])})
    assert z["layerwise/normalized_mse"]["layer_0"] == pytest.approx(1.0, rel=1e-5)
    assert z["layerwise/explained_variance"]["layer_0"] == pytest.approx(0.0, abs=1e-6)
    # de-normalisation with per-column std changes the weighting of the columns: numpy on x * std + mean
    mean = {0: torch.arange(6.0), 1: torch.zeros(6)}
    std = {0: torch.tensor([1.0, 2.0, 3.0, 0.5, 0.25, 4.0]), 1: torch.ones(6)}
    m = orc.reconstruction_metrics(tgt, rec, method="mean_std", mean_tg=mean, std_tg=std)
    t = (tgt[0] * std[0] + mean[0]).double().numpy()
    r = (rec[0] * std[0] + mean[0]).double().numpy()
    assert m["layerwise/explained_variance"]["layer_0"] == pytest.approx(
        1 - np.var(t - r, axis=0).mean() / np.var(t, axis=0).mean(), rel=1e-5)
    # sqrt(d_model) scaling leaves the ratios alone
    s = orc.reconstruction_metrics(tgt, rec, method="sqrt_d_model", d_model=6)
    base = orc.reconstruction_metrics(tgt, rec)
    assert s["reconstruction/explained_variance"] == pytest.approx(base["reconstruction/explained_variance"], rel=1e-5)
    # constant target, reconstruction off by a constant: both variances 0 -> EV 1, NMSE inf; an error
    # that varies -> EV 0 (the reference's branches, evaluator.py:309-325)
    k = orc.reconstruction_metrics({0: torch.ones(4, 2)}, {0: torch.zeros(4, 2)})
    assert k["layerwise/explained_variance"]["layer_0"] == 1.0 and math.isinf(k["layerwise/normalized_mse"]["layer_0"])
    k = orc.reconstruction_metrics({0: torch.ones(4, 2)}, {0: torch.arange(8.0).view(4, 2)})
    assert k["layerwise/explained_variance"]["layer_0"] == 0.0 and math.isinf(k["layerwise/normalized_mse"]["layer_0"])


def _chunk_store(chunks, dtype):
    """fetch_slice over in-memory chunks [L, 2, rows, d]: the wire bytes Layer0_Inputs | Layer0_Targets | ..."""
    def fetch(chunk_id, sorted_rows):
        sel = chunks[chunk_id][:, :, torch.as_tensor(np.asarray(sorted_rows, dtype=np.int64)), :].contiguous()
        return sel.view(torch.uint8).numpy().tobytes() if dtype != torch.float32 else sel.numpy().tobytes()
    return fetch


def test_store_batch_assembly_hand_written():
    # value = 1000*chunk + 100*layer + 50*is_target + row + col/4: every expected row can be written down
    L, d, rows = 2, 2, 6
    chunks = {}
    for c in (0, 1):
        t = torch.zeros(L, 2, rows, d)
        for l in range(L):
            for k in range(2):
                for r in range(rows):
                    for j in range(d):
                        t[l, k, r, j] = 1000 * c + 100 * l + 50 * k + r + j / 4
        chunks[c] = t
    idxs = np.array([(1, 3), (0, 2), (1, 0), (0, 5)], dtype=np.uint32)
    ins, tgs = orc.store_parse_batch(idxs, _chunk_store(chunks, torch.float32), num_layers=L, d_model=d, dtype=torch.float32)
    # chunks in ascending order; inside a chunk the sampler's order: (0,2), (0,5), (1,3), (1,0)
    assert ins[0].tolist() == [[2.0, 2.25], [5.0, 5.25], [1003.0, 1003.25], [1000.0, 1000.25]]
    assert tgs[0].tolist() == [[52.0, 52.25], [55.0, 55.25], [1053.0, 1053.25], [1050.0, 1050.25]]
    assert ins[1].tolist() == [[102.0, 102.25], [105.0, 105.25], [1103.0, 1103.25], [1100.0, 1100.25]]
    assert tgs[1][:, 0].tolist() == [152.0, 155.0, 1153.0, 1150.0]
    # normalisation by hand: (x - mean) / std in fp32, only where the layer has statistics; sqrt(d) scaling
    mean_in, std_in = {0: torch.tensor([[1.0, 2.0]])}, {0: torch.tensor([[2.0, 4.0]])}
    ins, tgs = orc.store_parse_batch(idxs, _chunk_store(chunks, torch.float32), num_layers=L, d_model=d, dtype=torch.float32,
                                     method="mean_std", mean_in=mean_in, std_in=std_in)
    assert ins[0][0].tolist() == [0.5, 0.0625]
    assert ins[1][0].tolist() == [102.0, 102.25] and tgs[0][0].tolist() == [52.0, 52.25]
    ins, _ = orc.store_parse_batch(idxs, _chunk_store(chunks, torch.float32), num_layers=L, d_model=d, dtype=torch.float32,
                                   method="sqrt_d_model")
    assert ins[0][1].tolist() == [float(np.float32(5.0) * np.float32(math.sqrt(2))), float(np.float32(5.25) * np.float32(math.sqrt(2)))]
    # 16-bit store: arithmetic in fp32, one rounding at the end (here 3.0 / 7.0 -> nearest bfloat16)
    c16 = {0: torch.full((1, 2, 2, 2), 3.0, dtype=torch.bfloat16)}
    ins, _ = orc.store_parse_batch(np.array([(0, 1)], dtype=np.uint32), _chunk_store(c16, torch.bfloat16), num_layers=1, d_model=2,
                                   dtype=torch.bfloat16, method="mean_std", mean_in={0: torch.zeros(1, 2)},
                                   std_in={0: torch.full((1, 2), 7.0)})
    assert ins[0].dtype == torch.bfloat16 and ins[0][0, 0].item() == torch.tensor(3.0 / 7.0).to(torch.bfloat16).item()


def test_store_batch_properties_of_the_reference_tests():
    # every row exactly once across sequential batches that span chunk boundaries
    # (tests/unit/data/test_data_integrity.py:215-294: the first element encodes the global position)
    L, d, per_chunk, n_chunks = 2, 4, 50, 3
    chunks = {}
    for c in range(n_chunks):
        t = torch.zeros(L, 2, per_chunk, d)
        for l in range(L):
            t[l, 0, :, 0] = torch.arange(per_chunk) + c * per_chunk
            t[l, 0, :, 1], t[l, 0, :, 2], t[l, 0, :, 3] = c, l, torch.arange(per_chunk)
            t[l, 1] = t[l, 0] + 1000
        chunks[c] = t
    manifest = np.array([(c, i) for c in range(n_chunks) for i in range(per_chunk)], dtype=np.uint32)
    seen = []
    for b in range(0, len(manifest), 25):
        ins, tgs = orc.store_parse_batch(manifest[b:b + 25], _chunk_store(chunks, torch.float32), num_layers=L, d_model=d,
                                         dtype=torch.float32)
        seen += ins[0][:, 0].tolist()
        assert torch.equal(tgs[1], ins[1] + 1000) and bool((ins[1][:, 2] == 1).all())
    assert seen == list(range(per_chunk * n_chunks))
    # normalised batches have mean ~ 0 and std ~ 1 (test_data_integrity.py:137-213, same generator and seed)
    d, n = 8, 1000
    stats = {0: (10.0, 2.0), 1: (-5.0, 0.5)}
    t = torch.zeros(2, 2, n, d)
    for l, (mu, sd) in stats.items():
        rng = np.random.RandomState(42)
        t[l, 0] = torch.from_numpy(rng.normal(mu, sd, (n, d)).astype(np.float32))
        t[l, 1] = torch.from_numpy(rng.normal(mu + 1, sd, (n, d)).astype(np.float32))
    mean_in = {l: torch.full((1, d), mu) for l, (mu, sd) in stats.items()}
    mean_tg = {l: torch.full((1, d), mu + 1) for l, (mu, sd) in stats.items()}
    std = {l: torch.full((1, d), sd) + 1e-6 for l, (mu, sd) in stats.items()}
    idxs = np.array([(0, i) for i in range(100)], dtype=np.uint32)
    ins, tgs = orc.store_parse_batch(idxs, _chunk_store({0: t}, torch.float32), num_layers=2, d_model=d, dtype=torch.float32,
                                     method="mean_std", mean_in=mean_in, std_in=std, mean_tg=mean_tg, std_tg=std)
    for l in (0, 1):
        for x in (ins[l], tgs[l]):
            assert abs(x.mean().item()) < 0.1 and abs(x.std().item() - 1.0) < 0.1
