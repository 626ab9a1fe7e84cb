"""The behaviours the reference's own unit tests pin for this path, asserted on this build's classes.

Each test names the reference test it follows (file:lines under the reference's ``tests/``).  The CPU part needs
no kernel: like the reference's registry tests it replaces the autograd Functions by mocks and checks what they
are called with.  The GPU part runs the same small shapes the reference uses (2 layers, d_model 8, 16 features,
30 tokens) through the HIP path.
"""
import logging
from unittest.mock import MagicMock, patch

import pytest
import torch

import crosslayer_coding_amd as cca
from crosslayer_coding_amd import registry


# ---- activation registry (unit/activation_generation/test_activation_registry.py) ----------------------------
@pytest.fixture
def fresh_registry():
    saved = dict(registry.ACTIVATION_REGISTRY)
    yield registry.ACTIVATION_REGISTRY
    registry.ACTIVATION_REGISTRY.clear()
    registry.ACTIVATION_REGISTRY.update(saved)


@pytest.fixture
def model_stub():
    m = MagicMock()
    m.config = cca.CLTConfig(d_model=16, num_features=32, num_layers=2, activation_fn="relu")
    m.rank = 0
    m.device = torch.device("cpu")
    m.dtype = torch.float32
    return m


def test_registering_twice_overwrites_and_warns(fresh_registry, caplog):
    # test_activation_registry.py:36-59
    @cca.register_activation_fn("probe_act")
    def first(model, preact, layer_idx):
        return preact * 2

    assert fresh_registry["probe_act"] is first
    caplog.clear()
    with caplog.at_level(logging.WARNING):

        @cca.register_activation_fn("probe_act")
        def second(model, preact, layer_idx):
            return preact * 3

    assert fresh_registry["probe_act"] is second
    assert len(caplog.records) == 1 and caplog.records[0].levelname == "WARNING"
    assert "Activation function 'probe_act' is already registered. Overwriting." in caplog.records[0].message


def test_lookup_returns_the_function_or_raises_with_the_name(fresh_registry):
    # test_activation_registry.py:62-74
    @cca.register_activation_fn("probe_lookup")
    def fn(model, preact, layer_idx):
        return preact

    assert cca.get_activation_fn("probe_lookup") is fn
    with pytest.raises(ValueError, match="Activation function 'non_existent_act' not found in registry."):
        cca.get_activation_fn("non_existent_act")


def test_jumprelu_entry_delegates_to_the_model(model_stub):
    # test_activation_registry.py:101-111
    preact = torch.tensor([-1.0, 1.0, 2.0])
    model_stub.jumprelu = MagicMock(return_value=torch.tensor([0.0, 1.0, 2.0]))
    out = cca.get_activation_fn("jumprelu")(model_stub, preact, 0)
    model_stub.jumprelu.assert_called_once_with(preact, 0)
    assert torch.equal(out, model_stub.jumprelu.return_value)


@pytest.mark.parametrize("k_set", [True, False])
def test_batchtopk_entry_calls_the_function_per_layer(model_stub, caplog, k_set):
    # test_activation_registry.py:114-161: k from the config (all features when unset), the pre-activations as the
    # ranking tensor, a warning that the scope is one layer
    preact = torch.tensor([[1.0, 2.0, 3.0, 4.0]])
    model_stub.config.activation_fn = "batchtopk"
    model_stub.config.batchtopk_k = 2 if k_set else None
    model_stub.config.batchtopk_straight_through = k_set
    ret = torch.tensor([[0.0, 0.0, 3.0, 4.0]])
    with patch("crosslayer_coding_amd.activations.BatchTopK") as fn_cls:
        fn_cls.apply = MagicMock(return_value=ret)
        caplog.clear()
        with caplog.at_level(logging.WARNING):
            out = cca.get_activation_fn("batchtopk")(model_stub, preact, 0)
        fn_cls.apply.assert_called_once_with(preact, 2.0 if k_set else float(preact.size(1)), k_set, preact)
    assert torch.equal(out, ret)
    assert any("This applies TopK per-layer, not globally." in r.message for r in caplog.records)
    assert any("batchtopk_k not set in config" in r.message for r in caplog.records) == (not k_set)


@pytest.mark.parametrize("k_set", [True, False])
def test_topk_entry_calls_the_function_per_layer(model_stub, caplog, k_set):
    # test_activation_registry.py:164-212
    preact = torch.tensor([[1.0, 2.0, 3.0, 4.0]])
    model_stub.config.activation_fn = "topk"
    if k_set:
        model_stub.config.topk_k = 0.5
    elif hasattr(model_stub.config, "topk_k"):
        delattr(model_stub.config, "topk_k")
    model_stub.config.topk_straight_through = k_set
    ret = torch.tensor([[0.0, 0.0, 3.0, 4.0]])
    with patch("crosslayer_coding_amd.activations.TokenTopK") as fn_cls:
        fn_cls.apply = MagicMock(return_value=ret)
        caplog.clear()
        with caplog.at_level(logging.WARNING):
            out = cca.get_activation_fn("topk")(model_stub, preact, 0)
        fn_cls.apply.assert_called_once_with(preact, 0.5 if k_set else float(preact.size(1)), k_set, preact)
    assert torch.equal(out, ret)
    assert any("This applies TopK per-layer, not globally." in r.message for r in caplog.records)
    assert any("topk_k not set in config" in r.message for r in caplog.records) == (not k_set)


def test_inputs_of_unexpected_rank_are_answered_with_zeros_and_a_warning(caplog):
    # unit/models/test_encoder.py:145-162: 1-D and 4-D inputs - the first dimension counts as the batch
    m = cca.CrossLayerTranscoder(cca.CLTConfig(num_layers=2, d_model=8, num_features=16, activation_fn="relu"), None,
                                 torch.device("cpu"))
    for x in (torch.randn(8), torch.randn(2, 3, 4, 8)):
        caplog.clear()
        with caplog.at_level(logging.WARNING):
            out = m.get_preactivations(x, 0)
        assert "Cannot handle input shape" in caplog.text
        assert out.shape == (x.shape[0], 16) and float(out.abs().sum()) == 0.0


# ---- the same small model on the device ------------------------------------------------------------------------
@pytest.fixture(params=["relu", "jumprelu", "batchtopk"])
def small_model(request, dev):
    # unit/models/test_clt_encode_decode.py:27-56
    cfg = cca.CLTConfig(num_layers=2, d_model=8, num_features=16, activation_fn=request.param, jumprelu_threshold=0.5,
                        batchtopk_k=4)
    return cca.CrossLayerTranscoder(cfg, process_group=None, device=dev).to(dev)


@pytest.fixture
def small_inputs(dev):
    g = torch.Generator().manual_seed(5)
    return {0: torch.randn(30, 8, generator=g).to(dev), 1: torch.randn(30, 8, generator=g).to(dev)}


@pytest.mark.gpu
def test_activation_decode_and_forward_shapes(small_model, small_inputs):
    # test_clt_encode_decode.py:70-116
    acts = small_model.get_feature_activations(small_inputs)
    assert isinstance(acts, dict) and sorted(acts) == sorted(small_inputs)
    assert acts[0].shape == (30, 16) and acts[1].shape == (30, 16)
    if small_model.config.activation_fn == "relu":
        assert all(bool((a >= 0).all()) for a in acts.values())
    rec1 = small_model.decode(acts, layer_idx=1)
    assert rec1.shape == (30, 8)
    recs = small_model.forward(small_inputs)
    assert isinstance(recs, dict) and sorted(recs) == sorted(small_inputs)
    assert recs[0].shape == (30, 8) and recs[1].shape == (30, 8)


@pytest.mark.gpu
def test_decoder_norms_shape_sign_and_cache(dev):
    # unit/models/test_decoder_norms.py:13-33
    from crosslayer_coding_amd.decoder import Decoder
    cfg = cca.CLTConfig(num_layers=3, d_model=8, num_features=12)
    dec = Decoder(config=cfg, process_group=None, device=dev, dtype=torch.float32)
    norms = dec.get_decoder_norms()
    assert norms.shape == (3, 12) and bool((norms >= 0).all())
    assert dec.get_decoder_norms() is norms           # cached: the same tensor object


@pytest.mark.gpu
def test_encode_all_layers_reports_the_original_shapes(dev):
    # unit/models/test_encoder.py:119-143: a 2-D and a 3-D input; (layer, batch, sequence) in layer order
    m = cca.CrossLayerTranscoder(cca.CLTConfig(num_layers=2, d_model=8, num_features=16, activation_fn="relu"), None, dev)
    inputs = {1: torch.randn(2, 5, 8, device=dev), 0: torch.randn(4, 8, device=dev)}
    pre, shapes = m._encode_all_layers(inputs)
    assert sorted(pre) == [0, 1] and pre[0].shape == (4, 16) and pre[1].shape == (10, 16)
    assert shapes == [(0, 4, 1), (1, 2, 5)]
    for l in (0, 1):
        torch.testing.assert_close(pre[l], m.get_preactivations(inputs[l], l))


@pytest.mark.gpu
def test_parallel_linear_layers_alone(dev):
    # unit/models/test_parallel_layers.py:37-60, and the plain products they stand for (:96-97)
    from crosslayer_coding_amd.parallel import ColumnParallelLinear, RowParallelLinear
    g = torch.Generator().manual_seed(6)
    col = ColumnParallelLinear(in_features=10, out_features=20, process_group=None, device=dev)
    x = torch.randn(5, 10, generator=g).to(dev)
    y = col(x)
    assert y.shape == (5, 20) and y.device.type == dev.type
    torch.testing.assert_close(y, x @ col.weight.detach().t() + col.bias_param.detach(), rtol=1e-5, atol=1e-6)
    row = RowParallelLinear(in_features=10, out_features=20, process_group=None, d_model_for_init=20,
                            num_layers_for_init=1, device=dev)
    y = row(x)
    assert y.shape == (5, 20) and y.device.type == dev.type
    torch.testing.assert_close(y, x @ row.weight.detach().t() + row.bias_param.detach(), rtol=1e-5, atol=1e-6)
    with pytest.raises(ValueError, match="unexpectedly greater"):
        row(torch.randn(5, 11, device=dev))


@pytest.mark.gpu
def test_decoder_edge_cases(dev, caplog):
    # unit/models/test_decoder.py:83-131
    from crosslayer_coding_amd.decoder import Decoder
    cfg = cca.CLTConfig(num_layers=2, d_model=8, num_features=16, activation_fn="relu")
    dec = Decoder(config=cfg, process_group=None, device=dev, dtype=torch.float32)
    with torch.no_grad():
        for lin in dec._ordered():
            lin.weight.uniform_(-0.3, 0.3)
    assert dec.decode({}, layer_idx=0).shape == (0, 8)
    assert dec.decode({0: torch.randn(0, 16, device=dev)}, layer_idx=0).shape == (0, 8)      # a tensor with no rows
    # a source whose feature dimension is wrong is skipped with a warning
    acts = {0: torch.randn(4, 12, device=dev), 1: torch.randn(4, 16, device=dev)}
    with caplog.at_level(logging.WARNING):
        rec = dec.decode(acts, 1)
    torch.testing.assert_close(rec, dec.decode({1: acts[1]}, 1))
    assert "incorrect feature dimension" in caplog.text and "12" in caplog.text
    # the norm cache is dropped by clearing the attribute, as the trainer does
    n1 = dec.get_decoder_norms()
    assert dec.get_decoder_norms() is n1
    dec._cached_decoder_norms = None
    assert dec.get_decoder_norms() is not n1


@pytest.mark.gpu
def test_tied_decoders_start_at_zero_and_follow_their_weights(dev):
    # unit/models/test_tied_decoders.py:138-183, :185-219
    from crosslayer_coding_amd.decoder import Decoder
    cfg = cca.CLTConfig(num_features=128, num_layers=4, d_model=64, activation_fn="relu", decoder_tying="per_source")
    dec = Decoder(config=cfg, process_group=None, device=dev, dtype=torch.float32)
    acts = {0: torch.randn(8, 128, device=dev), 1: torch.randn(8, 128, device=dev)}
    rec = dec.decode(acts, layer_idx=1)
    assert rec.shape == (8, 64) and float(rec.abs().max()) == 0.0           # tied decoders are initialised to zero
    for lin in dec.decoders:
        lin.weight.data.fill_(0.1)
    assert float(dec.decode(acts, layer_idx=1).abs().max()) > 0.0
    norms = dec.get_decoder_norms()
    assert norms.shape == (4, 128) and bool((norms >= 0).all())
    cfg2 = cca.CLTConfig(num_features=128, num_layers=2, d_model=64, activation_fn="relu", enable_feature_offset=True,
                         enable_feature_scale=True, decoder_tying="per_source")
    dec2 = Decoder(config=cfg2, process_group=None, device=dev, dtype=torch.float32)
    dec2.feature_offset[0].data.fill_(0.5)
    dec2.feature_scale[0].data.fill_(2.0)
    assert dec2.decode({0: torch.randn(4, 128, device=dev), 1: torch.randn(4, 128, device=dev)}, layer_idx=1).shape == (4, 64)


@pytest.mark.gpu
def test_jumprelu_with_a_layer_out_of_range_returns_its_input(dev, caplog):
    # unit/models/test_theta.py:94-102
    from crosslayer_coding_amd.theta import ThetaManager
    cfg = cca.CLTConfig(num_layers=2, d_model=8, num_features=16, activation_fn="jumprelu", jumprelu_threshold=0.5)
    tm = ThetaManager(cfg, None, dev, torch.float32)
    x = torch.randn(2, 16, device=dev)
    with caplog.at_level(logging.ERROR):
        out = tm.jumprelu(x, layer_idx=cfg.num_layers)
    assert "Invalid layer_idx" in caplog.text
    torch.testing.assert_close(out, x)


def test_a_config_without_the_newer_fields_gets_their_defaults():
    # unit/models/test_tied_decoders.py:221-238
    c = cca.CLTConfig(**{"num_features": 128, "num_layers": 4, "d_model": 64, "activation_fn": "relu"})
    assert c.decoder_tying == "none"
    assert c.enable_feature_offset is False and c.enable_feature_scale is False and c.skip_connection is False


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_writes_through_data_show_in_the_next_forward(dev, dtype):
    # The reference reads its parameters in place, so its own tests change them through ``.data`` and expect the
    # next result to follow (unit/models/test_tied_decoders.py:160-166, integration/test_tp_equivalence.py:59, 228).
    # Such writes bump no version counter; the packed decoder copy follows them through a fingerprint check and a
    # repack that both run on the device.
    from crosslayer_coding_amd import synth
    from oracle import clt_oracle as orc
    wl = synth.WORKLOADS["c0"].scaled("data-writes", dtype=dtype, num_layers=3, d_model=64, num_features=256, tokens=96, k=8)
    model, inputs, _ = synth.build_model(wl, dev)
    model.eval()
    tol = 1e-5 if dtype == "float32" else 1e-2

    def reference():
        sd = {k: v.detach().cpu() for k, v in model.state_dict().items()}
        names = synth.decoder_names(wl)
        recs, _ = orc.forward({l: x.cpu() for l, x in inputs.items()},
                              enc_w=[sd[f"encoder_module.encoders.{l}.weight"] for l in range(3)],
                              enc_b=[sd[f"encoder_module.encoders.{l}.bias_param"] for l in range(3)],
                              dec_w={n: sd[f"decoder_module.decoders.{n}.weight"] for n in names},
                              dec_b={n: sd[f"decoder_module.decoders.{n}.bias_param"] for n in names},
                              activation_fn="batchtopk", dtype=getattr(torch, dtype), num_layers=3, d_model=64,
                              num_features=256, k=8, topk_mode="per_layer")
        return recs

    before = model(inputs)
    dec = model.decoder_module
    assert int(dec._fp_changed.sum()) == 0
    model(inputs)
    assert int(dec._fp_changed.sum()) == 0                      # nothing written: nothing repacked
    w = dec.decoders["0->1"].weight
    b = dec.decoders["1->2"].bias_param
    v_w, v_b = w._version, b._version
    w.data.mul_(-1.5)                                           # one matrix through .data ...
    b.data.add_(0.25)                                           # ... and one bias
    model.encoder_module.encoders[2].weight.data.mul_(0.5)      # the encoder reads its parameters in place anyway
    assert (w._version, b._version) == (v_w, v_b)
    after = model(inputs)
    assert int(dec._fp_changed.sum()) == 1 and int(dec._fp_changed[1]) == 1      # slot of "0->1"
    want = reference()
    for t in range(3):
        assert orc.rel_l2(after[t].float().cpu(), want[t].float()) <= tol, t
    assert not torch.equal(after[1], before[1]) and not torch.equal(after[2], before[2])
    model(inputs)
    assert int(dec._fp_changed.sum()) == 0
    # a whole-matrix copy, the way the reference's tests load weights
    with torch.no_grad():
        new = torch.randn_like(w) * 0.05
    w.data.copy_(new)
    again = model(inputs)
    want = reference()
    for t in range(3):
        assert orc.rel_l2(again[t].float().cpu(), want[t].float()) <= tol, t


# ---- the autograd Functions (unit/models/test_activations.py) ----------------------------------------------------
@pytest.mark.gpu
def test_masks_of_empty_inputs_are_empty(dev):
    # test_activations.py:53-63, :243-253
    for fn, k in ((cca.BatchTopK, 2), (cca.TokenTopK, 2.0)):
        for shape in ((0, 4), (2, 0)):
            x = torch.empty(*shape, device=dev)
            m = fn._compute_mask(x, k)
            assert m.shape == x.shape and m.dtype == torch.bool and int(m.sum()) == 0


@pytest.mark.gpu
@pytest.mark.parametrize("straight_through", [True, False])
def test_top_k_backward_passes_the_gradient_where_the_gate_kept(dev, straight_through):
    # test_activations.py:114-152 (BatchTopK; the non-straight-through flag behaves the same), :286-301 (TokenTopK)
    g = torch.Generator().manual_seed(3)
    for fn, k in ((cca.BatchTopK, 2.0), (cca.TokenTopK, 2.0)):
        x = torch.randn(2, 4, generator=g).to(dev).requires_grad_(True)
        out = fn.apply(x, k, straight_through, None)
        gout = torch.randn(2, 4, generator=g).to(dev)
        out.backward(gout)
        mask = fn._compute_mask(x.detach(), int(k) if fn is cca.BatchTopK else k, None)
        assert x.grad is not None and torch.allclose(x.grad, gout * mask.to(x.dtype))
        assert int(mask.sum()) == 4


@pytest.mark.gpu
def test_jumprelu_backward_table_and_grad_flags(dev):
    # test_activations.py:318-381 (the table, quoted in tests/golden/reference_known_answers.json), :384-420 (flags)
    import json
    import os
    table = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_known_answers.json")))["jumprelu_backward"]
    for case in table:
        x = torch.tensor([case["input"]], device=dev, requires_grad=True)
        thr = torch.tensor([case["threshold"]], device=dev, requires_grad=True)
        out = cca.JumpReLU.apply(x, thr, case["bandwidth"])
        out.backward(torch.tensor([case["grad_output"]], device=dev))
        assert x.grad.item() == pytest.approx(case["expected_grad_input"] * case["grad_output"])
        near = abs(case["input"] - case["threshold"]) <= case["bandwidth"] / 2.0
        want = (-case["input"] / case["bandwidth"]) * case["grad_output"] if near else 0.0
        assert thr.grad.item() == pytest.approx(want, abs=1e-6), case
    one = torch.tensor([1.0], device=dev)
    x = torch.tensor([1.5], device=dev, requires_grad=True)
    thr = torch.tensor([0.5], device=dev)
    cca.JumpReLU.apply(x, thr, 1.0).backward(one)
    assert x.grad is not None and thr.grad is None
    x = torch.tensor([1.5], device=dev)
    thr = torch.tensor([0.5], device=dev, requires_grad=True)
    cca.JumpReLU.apply(x, thr, 1.0).backward(one)
    assert x.grad is None and thr.grad is not None

    class Ctx:            # neither input asked for its gradient, the threshold did: backward called by hand
        needs_input_grad = [False, True, False]
        saved_tensors = (torch.tensor([1.5], device=dev), torch.tensor([0.5], device=dev))
        bandwidth = 1.0

    gx, gthr, _ = cca.JumpReLU.backward(Ctx(), one)
    assert gx is None and gthr is not None


@pytest.mark.gpu
def test_data_writes_are_seen_next_to_other_kinds_of_writes_and_between_training_steps(dev):
    # a versioned in-place write to one matrix and a .data write to another before the same forward; a .data write
    # after an optimiser step (whose kernels write the parameters themselves)
    from crosslayer_coding_amd import synth
    wl = synth.WORKLOADS["c0"].scaled("data-writes-2", dtype="bfloat16", num_layers=3, d_model=128, num_features=256, tokens=256, k=8)
    model, inputs, _ = synth.build_model(wl, dev)
    twin, _, _ = synth.build_model(wl, dev)
    dec, dec2 = model.decoder_module, twin.decoder_module
    model(inputs)
    with torch.no_grad():
        dec.decoders["0->0"].weight.mul_(0.5)                   # bumps the version counter
    dec.decoders["1->2"].weight.data.mul_(-2.0)                 # does not
    out = model(inputs)
    with torch.no_grad():
        dec2.decoders["0->0"].weight.mul_(0.5)
        dec2.decoders["1->2"].weight.mul_(-2.0)
    want = twin(inputs)
    for t in range(3):
        assert torch.equal(out[t], want[t]), t
    # training: each route's own kernels write the parameters; a .data write after the step must still count
    targets = {l: torch.randn_like(x) for l, x in inputs.items()}
    for fused in (False, True):
        opts = []
        for m in (model, twin):
            opt = cca.CLTAdam(m, lr=1e-3)
            opt.fuse_decoder_step = fused
            m.training_step(inputs, targets, opt)
            opts.append(opt)
        w = dec.decoders["0->1"].weight          # (a fused step left the parameters behind: this access refreshes them)
        w.data.add_(0.125)
        with torch.no_grad():
            dec2.decoders["0->1"].weight.add_(0.125)
        out, want = model(inputs), twin(inputs)
        for t in range(3):
            assert torch.equal(out[t], want[t]), (fused, t)


@pytest.mark.gpu
def test_forward_then_backward_fills_the_gradients(dev):
    # integration/test_clt_end_to_end.py:63-101: a ReLU model, the mean squared error of every reconstruction
    # against its own input, loss.backward(), gradients on encoder weights, decoder weights and decoder biases
    cfg = cca.CLTConfig(num_layers=2, d_model=8, num_features=16, activation_fn="relu")
    model = cca.CrossLayerTranscoder(cfg, process_group=None, device=dev)
    for p in model.parameters():
        p.requires_grad = True
    model = model.to(dev)
    g = torch.Generator().manual_seed(9)
    inputs = {0: torch.randn(20, 8, generator=g).to(dev), 1: torch.randn(20, 8, generator=g).to(dev)}
    recs = model.forward(inputs)
    loss = torch.tensor(0.0, device=dev, dtype=torch.float32)
    for l, r in recs.items():
        loss = loss + torch.mean((r - inputs[l]) ** 2)
    loss.backward()
    w_enc = model.encoder_module.encoders[0].weight
    assert w_enc.grad is not None and bool(torch.isfinite(w_enc.grad).all())
    # the reference initialises untied decoders to small random values, so the encoder sees a gradient
    assert not bool((w_enc.grad == 0).all())
    w_dec = model.decoder_module.decoders["0->1"].weight
    assert w_dec.grad is not None and bool(torch.isfinite(w_dec.grad).all()) and not bool((w_dec.grad == 0).all())
    b_dec = model.decoder_module.decoders["1->1"].bias_param
    assert b_dec.grad is not None and bool(torch.isfinite(b_dec.grad).all())
    # a parameter changed in place between forward and backward is reported, as autograd does for saved tensors
    recs = model(inputs)
    with torch.no_grad():
        w_dec.mul_(2.0)
    with pytest.raises(RuntimeError, match="modified in place"):
        sum(r.sum() for r in recs.values()).backward()


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_autograd_route_equals_loss_and_gradients(dev, dtype):
    from crosslayer_coding_amd import synth
    wl = synth.WORKLOADS["c0"].scaled("graph", dtype=dtype, num_layers=3, d_model=128, num_features=512, tokens=256, k=12)
    model, inputs, _ = synth.build_model(wl, dev)
    g = torch.Generator().manual_seed(2)
    targets = {l: torch.randn(256, 128, generator=g).to(dev).to(model.dtype) for l in range(3)}
    _, want = model.loss_and_gradients(inputs, targets)
    recs = model(inputs)
    assert all(r.requires_grad for r in recs.values())
    loss = sum(((recs[l].float() - targets[l].float()) ** 2).mean() for l in range(3))
    loss.backward()
    for name, p in model.named_parameters():
        if want.get(name) is None:
            continue
        assert p.grad is not None and p.grad.dtype == p.dtype, name
        ref = want[name].float()
        err = float((p.grad.float() - ref).norm() / ref.norm().clamp_min(1e-20))
        # bfloat16: d loss / d reconstruction reaches the kernels rounded to bfloat16, as it does in the reference
        assert err <= (1e-4 if dtype == "float32" else 2e-2), (name, err)
