"""Post-hoc theta estimation and BatchTopK / TokenTopK -> JumpReLU conversion on the device
against the oracle's dense restatement (reference clt/models/theta.py:82-636)."""
import pytest
import torch

import crosslayer_coding_amd as cca
from crosslayer_coding_amd import synth
from crosslayer_coding_amd.config import CLTConfig
from crosslayer_coding_amd.theta import ThetaManager
from oracle import clt_oracle as orc

pytestmark = pytest.mark.gpu


def make_batches(L, T, F, n, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    out = []
    for _ in range(n):
        out.append({l: (torch.randn(T, F, generator=g) * (1.0 + 0.3 * l) + 0.2 * l).to(dtype) for l in range(L)})
    return out


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("fn,k", [("batchtopk", 5), ("topk", 0.05)])
def test_estimation_buffers_and_thresholds_match_the_oracle(dev, dtype, fn, k):
    L, T, F, nb = 3, 64, 128, 3
    batches = make_batches(L, T, F, nb, dtype, seed=11)
    cfg = CLTConfig(num_layers=L, d_model=8, num_features=F, activation_fn=fn,
                    batchtopk_k=k if fn == "batchtopk" else None, topk_k=k if fn == "topk" else None,
                    clt_dtype=str(dtype).split(".")[1])
    tm = ThetaManager(cfg, None, dev, dtype)
    it = iter(batches)
    data = [({0: torch.zeros(1, 8)}, None) for _ in range(nb)]      # the encoder is mocked: inputs are ignored

    def encode_fn(_inputs):
        return {l: p.to(dev) for l, p in next(it).items()}, []

    theta = tm.estimate_theta_posthoc(encode_fn, data, num_batches=nb)
    s, c, mu, sg = orc.theta_estimate_posthoc(batches, activation_fn=fn, k=k, num_layers=L, num_features=F, dtype=dtype)
    assert torch.equal(tm._count_min_selected_preact.cpu(), c)
    if dtype == torch.float32:
        assert torch.allclose(tm._sum_min_selected_preact.cpu(), s, rtol=1e-5, atol=1e-6)
        assert torch.allclose(tm._avg_layer_means.cpu(), mu, rtol=1e-5, atol=1e-6)
        assert torch.allclose(tm._avg_layer_stds.cpu(), sg, rtol=1e-5)
    else:   # bf16: identical roundings at every step
        assert torch.equal(tm._sum_min_selected_preact.cpu(), s)
        assert orc.rel_l2(tm._avg_layer_stds.float().cpu(), sg.float()) <= 1e-2
    log_t = orc.theta_convert(tm._sum_min_selected_preact.cpu(), tm._count_min_selected_preact.cpu(),
                              tm._avg_layer_means.cpu(), tm._avg_layer_stds.cpu())
    assert tm.config.activation_fn == "jumprelu" and tm.log_threshold.shape == (L, F)
    assert torch.allclose(tm.log_threshold.detach().float().cpu(), log_t.float(), rtol={torch.float32: 1e-5, torch.bfloat16: 1e-2, torch.float16: 2e-3}[dtype],
                          atol={torch.float32: 1e-6, torch.bfloat16: 1e-2, torch.float16: 2e-3}[dtype])
    assert bool(torch.isfinite(theta).all()) and bool((theta > 0).all())


def test_model_level_flow_and_the_reference_test_properties(dev):
    # reference tests/unit/models/test_theta.py:110-175 through the model API, then a JumpReLU forward
    wl = synth.Workload("est", 9, 2, 64, 256, 256, "float32", k=8, topk_mode="global")
    model, inputs, _ = synth.build_model(wl, dev)
    data = [(inputs, None), (inputs, None)]
    theta = model.estimate_theta_posthoc(data, num_batches=2)
    assert model.config.activation_fn == "jumprelu" and theta.shape == (2, 256)
    assert bool(torch.isfinite(theta).all()) and bool((theta > 0).all())
    acts = model.get_feature_activations(inputs)
    pre, _ = model._encode_all_layers(inputs)
    for l in acts:
        th = torch.exp(model.log_threshold[l]).to(model.dtype)
        assert torch.equal(acts[l], torch.where(pre[l] >= th, pre[l], torch.zeros_like(pre[l])).float())
    recs = model(inputs)
    assert sorted(recs) == [0, 1] and all(torch.isfinite(r).all() for r in recs.values())


def test_missing_and_mismatched_layers_are_zero_filled(dev):
    L, T, F = 3, 32, 64
    cfg = CLTConfig(num_layers=L, d_model=8, num_features=F, activation_fn="batchtopk", batchtopk_k=4)
    tm = ThetaManager(cfg, None, dev, torch.float32)
    g = torch.Generator().manual_seed(3)
    batch = {0: torch.randn(T, F, generator=g) + 1.0, 2: torch.randn(T // 2, F, generator=g)}   # layer 1 absent, layer 2 short

    def encode_fn(_inputs):
        return {l: p.to(dev) for l, p in batch.items()}, []

    tm.estimate_theta_posthoc(encode_fn, [({0: torch.zeros(1, 8)}, None)], num_batches=1)
    assert tm._processed_batches_for_stats.tolist() == [1, 0, 0]
    assert float(tm._count_min_selected_preact[1:].sum()) == 0.0 and float(tm._count_min_selected_preact[0].sum()) > 0
    # the same through the oracle with explicit zeros for layers 1 and 2
    ref_batch = {0: batch[0], 1: torch.zeros(T, F), 2: torch.zeros(T, F)}
    s, c, _, _ = orc.theta_estimate_posthoc([ref_batch], activation_fn="batchtopk", k=4, num_layers=L, num_features=F,
                                            dtype=torch.float32)
    assert torch.equal(tm._count_min_selected_preact.cpu(), c)
    assert torch.allclose(tm._sum_min_selected_preact.cpu(), s, rtol=1e-5, atol=1e-6)
