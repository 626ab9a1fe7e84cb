"""Decoders tied per target: the dense route (survivors scattered into the summed activation, then one
product on the MFMA kernel - the reference's own formulation, clt/models/decoder.py:208-251) against the
oracle and against the row-gather route, through the host mirror and through the C ABI."""
import math

import pytest
import torch

import crosslayer_coding_amd as cca
from crosslayer_coding_amd import _native as nat
from crosslayer_coding_amd import engine, synth
from oracle import clt_oracle as orc

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-5, torch.bfloat16: 1e-2, torch.float16: 2e-3}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_accumulate_dense_is_the_running_sum_in_the_model_dtype(dev, dtype):
    g = torch.Generator().manual_seed(3)
    L, T, F = 3, 70, 200
    acts = (torch.randn(L, T, F, generator=g) * (torch.rand(L, T, F, generator=g) < 0.3)).to(dtype)
    acts[1, 4] = 0
    off = torch.randn(F, generator=g).to(dtype)
    sc = torch.randn(F, generator=g).to(dtype)
    surv = engine.threshold_select(acts.to(dev), None, nat.PRED_NONZERO)
    acc = torch.full((T, F), 7.0, dtype=dtype, device=dev)
    want = torch.zeros(T, F, dtype=dtype)
    for s in range(L):
        engine.accumulate_dense(surv, s, acc, init=(s == 0))
        want = want + acts[s]                       # the reference's `summed_activation += activation_tensor`
        assert torch.equal(acc.cpu(), want)
    # the target's affine terms touch the non-zero entries only (decoder.py:228-244)
    engine.accumulate_dense(surv, -1, acc, init=True)
    assert float(acc.abs().max()) == 0.0
    want = torch.zeros(T, F, dtype=dtype)
    for s in range(L):
        engine.accumulate_dense(surv, s, acc, False, off.to(dev), sc.to(dev))
        a = acts[s].clone()
        nz = a != 0
        a[nz] = ((a + off)[nz].to(dtype) * sc.expand(T, F)[nz]).to(dtype)
        want = want + a
    assert torch.equal(acc.cpu(), want)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16", "float16"])
@pytest.mark.parametrize("affine", [False, True])
@pytest.mark.parametrize("features", [512, 576])      # 576: an odd number of 128-byte stages along the product's K
def test_dense_route_matches_the_oracle_and_the_gather_route(dev, dtype, affine, features):
    tdt = getattr(torch, dtype)
    wl = synth.Workload("dense-route", 7, 4, 256, features, 512, dtype, k=24, decoder_tying="per_target")
    cfg = wl.config()
    cfg.enable_feature_offset = cfg.enable_feature_scale = affine
    x = synth.make_inputs(wl, "cpu")
    sd = synth.make_state_dict(wl, "cpu")
    g = torch.Generator().manual_seed(9)
    L, F, d = wl.num_layers, wl.num_features, wl.d_model
    for i in range(L):
        sd[f"decoder_module.decoders.{i}.bias_param"] = (torch.randn(d, generator=g) * 0.1).to(tdt)
        if affine:
            sd[f"decoder_module.feature_offset.{i}"] = (torch.randn(F, generator=g) * 0.2).to(tdt)
            sd[f"decoder_module.feature_scale.{i}"] = (1 + 0.3 * torch.randn(F, generator=g)).to(tdt)
    model = cca.CrossLayerTranscoder(cfg, None, dev)
    model.load_state_dict(sd)
    inputs = {l: x[l].to(dev) for l in range(L)}
    # rates of a large shape: at this size the measured ones would (rightly) keep every target on the gather
    model.decoder_module.rate_override = (14.5e12, 1.0e14 if tdt == torch.float32 else 1.0e15)
    dense = model(inputs)
    route = dict(model.decoder_module.last_route)
    assert route["dense_targets"][0] < route["dense_targets"][1] == L      # the dense route was taken
    model.decoder_module.dense_route = False
    sparse = model(inputs)
    assert model.decoder_module.last_route["dense_targets"] == (L, L)
    acts = {l: a.cpu() for l, a in model.get_feature_activations(inputs).items()}
    names = synth.decoder_names(wl)
    for t in range(L):
        ref = orc.decode(acts, t, tying="per_target", weights={n: sd[f"decoder_module.decoders.{n}.weight"] for n in names},
                         biases={n: sd[f"decoder_module.decoders.{n}.bias_param"] for n in names}, d_model=d,
                         num_features=F, dtype=tdt,
                         feature_offset=[sd[f"decoder_module.feature_offset.{i}"] for i in range(L)] if affine else None,
                         feature_scale=[sd[f"decoder_module.feature_scale.{i}"] for i in range(L)] if affine else None)
        assert orc.rel_l2(dense[t].cpu(), ref) <= TOL[tdt], (t, "dense")
        assert orc.rel_l2(sparse[t].cpu(), ref) <= TOL[tdt], (t, "gather")
    # a subset of layers: the missing source contributes nothing, the missing target is not produced
    model.decoder_module.dense_route = True
    part = model({l: inputs[l] for l in (0, 2, 3)})
    assert sorted(part) == [0, 2, 3]
    model.decoder_module.dense_route = False
    want = model({l: inputs[l] for l in (0, 2, 3)})
    for t in part:
        assert orc.rel_l2(part[t].float().cpu(), want[t].float().cpu()) <= TOL[tdt]


def test_dense_split_follows_the_measured_rates(dev):
    # The split between the row gather and the dense product is decided from rates measured on this GPU
    # (Decoder.route_rates: the product itself on the matrix cores, a bare row gather), cached per shape;
    # with the two rates swapped the decision flips.
    wl = synth.Workload("dense-split", 7, 6, 512, 4096, 1024, "bfloat16", k=64, decoder_tying="per_target")
    model = cca.CrossLayerTranscoder(wl.config(), None, dev)
    dec = model.decoder_module
    L, T, F, d = wl.num_layers, wl.tokens, wl.num_features, wl.d_model
    gather, mfma = dec.route_rates(T, F, d, torch.bfloat16)
    assert 1e12 < gather < 4e13 and 5e13 < mfma < 2.5e15, (gather, mfma)        # plausible for one MI355X
    assert dec.route_rates(T, F, d, torch.bfloat16) == (gather, mfma)           # cached: measured once
    total = L * wl.k * T
    surv = engine.SurvivorList(torch.zeros(L * T + 1, dtype=torch.int32, device=dev),
                               torch.zeros(total, dtype=torch.int32, device=dev),
                               torch.zeros(total, dtype=torch.bfloat16, device=dev), T, F, L, torch.bfloat16, None, total)
    mask = (1 << L) - 1

    def first_dense(rates):
        dec.rate_override = rates
        return dec.dense_split(surv, mask, 0, L, None)

    # target t gathers (t + 1) k T rows of d elements; the product costs 2 T F d whatever t is
    def expected(g_rate, m_rate):
        for t in range(L):
            if (t + 1) * wl.k * T * d * 2 / g_rate > 2.0 * T * F * d / m_rate:
                return t
        return L

    for rates in ((gather, mfma), (1e12, 1e15), (1e15, 1e12), (mfma, gather)):
        assert first_dense(rates) == expected(*rates), rates
    assert first_dense((1e12, 1e15)) == 0 and first_dense((1e15, 1e12)) == L      # the decision flips with the rates
    dec.rate_override = None
    assert dec.dense_split(surv, mask, 0, L, None) == expected(gather, mfma)
    dec.dense_route = False
    assert dec.dense_split(surv, mask, 0, L, None) == L


def test_route_query_names_the_schedules(dev):
    big = 12 * 4096
    # GPT-2-small x32: a quarter of the columns of half the rows is 4.7 MiB, about one L2: quarter-row schedule
    assert engine.decode_route(4096, 768, 24576, 12, "none", torch.bfloat16) == nat.ROUTE_QUARTER
    assert engine.decode_route(4096, 768, 24576, 12, "none", torch.float32) == nat.ROUTE_LINE      # 9.4 MiB in fp32
    assert engine.decode_route(1024, 768, 6144, 12, "none", torch.float32) == nat.ROUTE_QUARTER
    # Pythia-410m shape: the same piece would be 8.4 MiB: one cache line of columns per XCD instead
    assert engine.decode_route(4096, 1024, 32768, 24, "none", torch.bfloat16) == nat.ROUTE_LINE
    assert engine.decode_route(8192, 2048, 16384, 16, "per_target", torch.bfloat16) == nat.ROUTE_SLICED_ALL_SOURCES
    assert engine.decode_route(4096, 640, 24576, 12, "per_source", torch.bfloat16) == nat.ROUTE_LINE
    assert engine.decode_route(4096, 4096, 24576, 12, "none", torch.bfloat16) == nat.ROUTE_LINE     # wider than a wavefront's registers hold
    assert engine.decode_route(4096, 200, 24576, 12, "per_source", torch.bfloat16) == nat.ROUTE_SLICED
    # a short batch keeps the XCD-partitioned schedule when the decoders are far larger than the caches (3.2 GB
    # here) and takes the one-pass kernel when they are small
    assert engine.decode_route(16, 768, 24576, 12, "none", torch.bfloat16, rows=16) == nat.ROUTE_QUARTER
    assert engine.decode_route(16, 768, 2048, 4, "none", torch.bfloat16, rows=16) == nat.ROUTE_SINGLE
    assert engine.decode_route(4096, 100, 24576, 12, "none", torch.bfloat16, rows=big) == nat.ROUTE_GENERIC


@pytest.mark.parametrize("tying", ["none", "per_source"])
@pytest.mark.parametrize("case", ["relu", "jumprelu-low-thresholds", "batchtopk-large-k"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_dense_pair_route_at_high_density(dev, dtype, case, tying):
    """Untied and per-source decoders at densities far above what the gather is made for: the decode takes the
    reference's dense products (clt/models/decoder.py:253-338) on the matrix-core kernel; result against the oracle
    and against the gather route of the same model."""
    tdt = getattr(torch, dtype)
    fn = {"relu": "relu", "jumprelu-low-thresholds": "jumprelu", "batchtopk-large-k": "batchtopk"}[case]
    wl = synth.Workload("dense-pairs", 8, 3, 256, 512, 600, dtype, activation_fn=fn, k=200 if fn == "batchtopk" else None,
                        decoder_tying=tying)
    x = synth.make_inputs(wl, "cpu")
    sd = synth.make_state_dict(wl, "cpu", inputs=x)
    g = torch.Generator().manual_seed(3)
    for key in list(sd):
        if key.endswith("bias_param") and "decoder" in key:
            sd[key] = (torch.randn(sd[key].shape, generator=g) * 0.1).to(tdt)
        if case == "jumprelu-low-thresholds" and key.endswith("bias_param") and "encoder" in key:
            sd[key] = sd[key] + 2.0            # most pre-activations pass their thresholds
    model = cca.CrossLayerTranscoder(wl.config(), None, dev)
    model.load_state_dict(sd)
    L, F, d = wl.num_layers, wl.num_features, wl.d_model
    inputs = {l: x[l].to(dev) for l in range(L)}
    # rates of a large shape: at this size the measured ones may keep the gather
    model.decoder_module.rate_override = (14.5e12, 1.0e14 if tdt == torch.float32 else 1.0e15)
    with torch.no_grad():
        model(inputs)                            # threshold activations: the density is known from the second forward on
        torch.cuda.synchronize()
        model(inputs)
        torch.cuda.synchronize()
        dense = model(inputs)
        assert model.decoder_module.last_route["dense_targets"] == (0, L), model.decoder_module.last_route
        # threshold activations make no survivor list at all on this route
        assert model.decoder_module.last_route.get("survivor_list", True) == (fn == "batchtopk")
        acts_dense = model.get_feature_activations(inputs)        # (threshold models: the gated slab itself)
        model.decoder_module.dense_route = False
        sparse = model(inputs)
        assert model.decoder_module.last_route["dense_targets"] == (L, L)
        acts = {l: a.cpu() for l, a in model.get_feature_activations(inputs).items()}
        for l in acts:
            assert acts_dense[l].dtype == acts[l].dtype and torch.equal(acts_dense[l].cpu(), acts[l])
        assert float((acts[0] != 0).float().mean()) > 0.2
        # a subset of layers
        model.decoder_module.dense_route = True
        part = model({l: inputs[l] for l in (0, 2)})
        model.decoder_module.dense_route = False
        want = model({l: inputs[l] for l in (0, 2)})
    names = synth.decoder_names(wl)
    for t in range(L):
        ref = orc.decode(acts, t, tying=tying, weights={n: sd[f"decoder_module.decoders.{n}.weight"] for n in names},
                         biases={n: sd[f"decoder_module.decoders.{n}.bias_param"] for n in names}, d_model=d,
                         num_features=F, dtype=tdt)
        assert orc.rel_l2(dense[t].cpu(), ref) <= TOL[tdt], (t, "dense")
        assert orc.rel_l2(sparse[t].cpu(), ref) <= TOL[tdt], (t, "gather")
    assert sorted(part) == [0, 2]
    for t in part:
        assert orc.rel_l2(part[t].float().cpu(), want[t].float().cpu()) <= TOL[tdt]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("L,T,F", [(2, 300, 520), (1, 77, 250), (3, 64, 1024)], ids=["vector", "element-wise", "vector-small"])
def test_threshold_dense_gates_in_place_and_counts(dev, dtype, L, T, F):
    """clt_threshold_dense against the reference's expressions (clt/models/activations.py:177-180 for JumpReLU, F.relu
    for ReLU): the tensor keeps x where the predicate holds and 0 elsewhere, and the count is the number kept."""
    g = torch.Generator().manual_seed(L * 100 + T + F)
    x = torch.randn(L, T, F, generator=g).to(dtype)
    x[0, 0, :4] = torch.tensor([0.0, -0.0, float("inf"), float("-inf")]).to(dtype)
    theta = torch.exp(0.5 * torch.randn(L, F, generator=g) - 0.5).to(dtype)
    theta[0, 0] = 0.0
    for pred, th in ((nat.PRED_GE_THETA, theta), (nat.PRED_GT_ZERO, None)):
        buf = x.clone().to(dev)
        total = engine.threshold_dense(buf, th.to(dev) if th is not None else None, pred)
        keep = (x >= theta.unsqueeze(1)) if th is not None else (x > 0)
        want = torch.where(keep, x, torch.zeros_like(x))
        iv = torch.int32 if dtype == torch.float32 else torch.int16
        assert torch.equal(buf.cpu().view(iv), want.view(iv))
        assert int(total) == int(keep.sum())


@pytest.mark.parametrize("tying", ["none", "per_source", "per_target"])
def test_dense_routes_carry_skip_connections(dev, tying):
    """A ReLU model with skip connections at 50 % density: reconstructions, loss and every gradient (skip matrices
    included) of the dense routes against the gather / survivor-list routes of the same model."""
    wl = synth.Workload("dense-skip", 8, 3, 256, 512, 320, "float32", activation_fn="relu", k=None, decoder_tying=tying)
    cfg = wl.config()
    cfg.skip_connection = True
    x = synth.make_inputs(wl, "cpu")
    sd = synth.make_state_dict(wl, "cpu", inputs=x)
    model = cca.CrossLayerTranscoder(cfg, None, dev)
    missing = [k for k in model.state_dict() if k not in sd]
    g = torch.Generator().manual_seed(4)
    for k in missing:                                   # the skip matrices
        sd[k] = torch.randn(model.state_dict()[k].shape, generator=g) * 0.05
    model.load_state_dict(sd)
    model.decoder_module.rate_override = (14.5e12, 1.0e14)
    L = wl.num_layers
    inputs = {l: x[l].to(dev) for l in range(L)}
    targets = {l: torch.randn(wl.tokens, wl.d_model, generator=g).to(dev) for l in range(L)}
    with torch.no_grad():
        model(inputs); torch.cuda.synchronize(); model(inputs); torch.cuda.synchronize()
        dense = model(inputs)
        assert model.decoder_module.last_route["dense_targets"][1] == L and model.decoder_module.last_route["dense_targets"][0] < L
    loss_d, grads_d = model.loss_and_gradients(inputs, targets)
    model.decoder_module.dense_route = False
    with torch.no_grad():
        sparse = model(inputs)
        assert model.decoder_module.last_route["dense_targets"] == (L, L)
    loss_s, grads_s = model.loss_and_gradients(inputs, targets)
    for t in range(L):
        assert orc.rel_l2(dense[t].cpu(), sparse[t].cpu()) <= 1e-5, t
    assert abs(float(loss_d) - float(loss_s)) <= 1e-5 * abs(float(loss_s))
    assert any("skip_weights" in k for k in grads_d)
    for k in grads_s:
        assert orc.rel_l2(grads_d[k].float().cpu(), grads_s[k].float().cpu()) <= 2e-5, k
