"""Evaluation reductions from the survivor list against the oracle's dense restatement
(reference clt/training/evaluator.py:194-405, clt/training/trainer.py:693-712)."""
import math

import pytest
import torch

import crosslayer_coding_amd as cca
from crosslayer_coding_amd import engine, synth
from oracle import clt_oracle as orc

pytestmark = pytest.mark.gpu

BASE = synth.WORKLOADS["c0"]


def close_lists(a, b, rel=1e-6, abs_=1e-6):
    assert len(a) == len(b)
    for x, y in zip(a, b):
        assert x == pytest.approx(y, rel=rel, abs=abs_)


def dense_cases(dtype):
    g = torch.Generator().manual_seed(21)
    a = torch.randn(3, 70, 130, generator=g)
    a[a.abs() < 1.2] = 0.0
    a[0, 0, 0] = 1e-7          # non-zero but not firing
    a[1, :, 5] = 0.0           # a dead feature
    a[2, 3, 7] = float("nan")  # counts as non-zero, does not fire
    a[2, :, 9] = -1.0          # negatives: non-zero, never firing
    return a.to(dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_sparsity_density_and_dead_counters_from_dense_activations(dev, dtype):
    a = dense_cases(dtype)
    L, T, F = a.shape
    acts = {l: a[l] for l in range(L)}
    cfg = cca.CLTConfig(num_layers=L, d_model=8, num_features=F, activation_fn="relu",
                        clt_dtype=str(dtype).split(".")[1])
    model = cca.CrossLayerTranscoder(cfg, None, dev)
    ev = cca.CLTEvaluator(model, dev)
    dev_acts = {l: v.to(dev) for l, v in acts.items()}
    got = ev._compute_sparsity(dev_acts)
    want = orc.sparsity_metrics(acts, F, L)
    for key in ("sparsity/total_l0", "sparsity/avg_l0", "sparsity/sparsity_fraction"):
        assert got[key] == pytest.approx(want[key], rel=1e-6)
    assert got["layerwise/l0"].keys() == want["layerwise/l0"].keys()
    for k in want["layerwise/l0"]:
        assert got["layerwise/l0"][k] == pytest.approx(want["layerwise/l0"][k], rel=1e-6)
    gd, wd = ev._compute_feature_density(dev_acts), orc.feature_density_metrics(acts)
    for key in ("layerwise/log_feature_density", "layerwise/consistent_activation_heuristic"):
        assert gd[key].keys() == wd[key].keys()
        for k in wd[key]:
            close_lists(gd[key][k], wd[key][k])
    # counters: exact integers
    surv = engine.threshold_select(a.to(dev).contiguous(), None, 2)
    tr = cca.DeadFeatureTracker(L, F, dead_feature_window=2, device=dev)
    tr.n_forward_passes_since_fired += torch.arange(L * F, device=dev).view(L, F) % 4
    before = tr.n_forward_passes_since_fired.cpu().clone()
    tr.update(surv)
    assert torch.equal(tr.n_forward_passes_since_fired.cpu(), orc.dead_feature_update(before, acts))
    assert torch.equal(tr.dead_neurons_mask.cpu(), orc.dead_feature_update(before, acts) > 2)
    # the raw counts themselves
    nonzero, fired = engine.survivor_metrics(surv)
    assert nonzero.tolist() == [(a[l] != 0).sum().item() for l in range(L)]
    assert torch.equal(fired.cpu().long(), (a.float() > 1e-6).sum(dim=1))


def test_empty_inputs_follow_the_reference_branches(dev):
    cfg = cca.CLTConfig(num_layers=2, d_model=8, num_features=16, activation_fn="relu")
    ev = cca.CLTEvaluator(cca.CrossLayerTranscoder(cfg, None, dev), dev)
    assert ev._compute_sparsity({}) == orc.sparsity_metrics({}, 16, 2)
    assert ev._compute_feature_density({}) == orc.feature_density_metrics({})
    e = {0: torch.zeros(0, 16, device=dev)}
    assert ev._compute_sparsity(e) == orc.sparsity_metrics({0: torch.zeros(0, 16)}, 16, 2)
    z = {0: torch.zeros(5, 16, device=dev), 1: torch.zeros(5, 16, device=dev)}
    got = ev._compute_sparsity(z)
    assert got["sparsity/total_l0"] == 0.0 and got["sparsity/sparsity_fraction"] == 1.0
    with pytest.raises(ValueError):
        cca.CLTEvaluator(ev.model, dev, normalization_method="bogus")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("method", ["none", "mean_std", "sqrt_d_model"])
def test_reconstruction_metrics_match_the_oracle(dev, dtype, method):
    g = torch.Generator().manual_seed(8)
    L, T, d = 3, 150, 72
    tgt = {l: (torch.randn(T, d, generator=g) * (1 + l) + 0.5 * l).to(dtype) for l in range(L)}
    rec = {l: (t.float() + 0.4 * torch.randn(T, d, generator=g)).to(dtype) for l, t in tgt.items()}
    del rec[1]                                        # a layer without a reconstruction is skipped
    mean = {0: torch.randn(d, generator=g), 2: torch.randn(1, d, generator=g)}
    std = {0: torch.rand(d, generator=g) + 0.5, 2: torch.rand(1, d, generator=g) + 0.5}
    cfg = cca.CLTConfig(num_layers=L, d_model=d, num_features=16, activation_fn="relu")
    ev = cca.CLTEvaluator(cca.CrossLayerTranscoder(cfg, None, dev), dev, mean_tg=mean, std_tg=std,
                          normalization_method=method, d_model=d)
    got = ev._compute_reconstruction_metrics({l: t.to(dev) for l, t in tgt.items()}, {l: r.to(dev) for l, r in rec.items()})
    want = orc.reconstruction_metrics(tgt, rec, method=method, mean_tg=mean, std_tg=std, d_model=d)
    tol = 1e-5 if dtype == torch.float32 else 1e-4     # fp64 sums here, fp32 sums of the same rounded values there
    for key in ("reconstruction/explained_variance", "reconstruction/normalized_mean_reconstruction_error"):
        assert got[key] == pytest.approx(want[key], rel=tol)
    for key in ("layerwise/normalized_mse", "layerwise/explained_variance"):
        assert got[key].keys() == want[key].keys()
        for k in want[key]:
            assert got[key][k] == pytest.approx(want[key][k], rel=tol, abs=tol)


def test_reconstruction_metric_branches_for_constant_targets(dev):
    cfg = cca.CLTConfig(num_layers=1, d_model=4, num_features=16, activation_fn="relu")
    ev = cca.CLTEvaluator(cca.CrossLayerTranscoder(cfg, None, dev), dev)
    ones = torch.ones(6, 4, device=dev)
    m = ev._compute_reconstruction_metrics({0: ones}, {0: torch.zeros_like(ones)})
    assert m["layerwise/explained_variance"]["layer_0"] == 1.0 and math.isinf(m["layerwise/normalized_mse"]["layer_0"])
    m = ev._compute_reconstruction_metrics({0: ones}, {0: torch.arange(24.0, device=dev).view(6, 4)})
    assert m["layerwise/explained_variance"]["layer_0"] == 0.0 and math.isinf(m["layerwise/normalized_mse"]["layer_0"])
    m = ev._compute_reconstruction_metrics({0: ones}, {0: ones.clone()})
    assert m["layerwise/explained_variance"]["layer_0"] == 1.0 and m["layerwise/normalized_mse"]["layer_0"] == 0.0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16", "float16"])
def test_compute_metrics_on_a_model_matches_the_oracle_end_to_end(dev, dtype):
    wl = BASE.scaled("ev", dtype=dtype, num_layers=3, d_model=128, num_features=512, tokens=256, k=12)
    model, inputs, _ = synth.build_model(wl, dev)
    model.eval()
    g = torch.Generator().manual_seed(4)
    targets = {l: torch.randn(wl.tokens, wl.d_model, generator=g).to(getattr(torch, dtype)).to(dev) for l in range(3)}
    mask = torch.zeros(3, 512, dtype=torch.bool)
    mask[1, :7] = True
    ev = cca.CLTEvaluator(model, dev)
    got = ev.compute_metrics(inputs, targets, dead_neuron_mask=mask)
    # the oracle's formulas on the model's own dense outputs: this checks the reductions, the forward
    # itself is checked elsewhere
    acts = {l: a.cpu() for l, a in model.get_feature_activations(inputs).items()}
    recs = {l: r.cpu() for l, r in model(inputs).items()}
    want = {**orc.reconstruction_metrics({l: t.cpu() for l, t in targets.items()}, recs),
            **orc.sparsity_metrics(acts, 512, 3), **orc.feature_density_metrics(acts)}
    assert got["sparsity/avg_l0"] == pytest.approx(12.0)          # BatchTopK keeps k per token on average
    for key in ("sparsity/total_l0", "sparsity/avg_l0", "sparsity/sparsity_fraction",
                "reconstruction/explained_variance", "reconstruction/normalized_mean_reconstruction_error"):
        assert got[key] == pytest.approx(want[key], rel=1e-4), key
    for key in ("layerwise/log_feature_density", "layerwise/consistent_activation_heuristic"):
        for k in want[key]:
            close_lists(got[key][k], want[key][k])
    assert got["layerwise/dead_features"] == {"layer_0": 0, "layer_1": 7, "layer_2": 0}
    assert got["dead_features/total_eval"] == 7
    flat = [v for k in sorted(want["layerwise/log_feature_density"]) for v in want["layerwise/log_feature_density"][k]]
    assert got["sparsity/feature_density_mean"] == pytest.approx(sum(flat) / len(flat), rel=1e-5)
    assert len(got["sparsity/log_feature_density_agg_hist"]) == 3 * 512
