"""Host-side mirror of the reference interface: config, parameter names and shapes,
registry, construction-time behaviour.  CPU only; nothing here computes on a device."""
import json
import math

import logging

import numpy as np
import pytest
import torch

import crosslayer_coding_amd as cca
from crosslayer_coding_amd import synth


def cfg(**kw):
    base = dict(num_features=16, num_layers=3, d_model=8, activation_fn="batchtopk", batchtopk_k=3)
    base.update(kw)
    return cca.CLTConfig(**base)


def test_config_validation_and_json_round_trip(tmp_path):
    with pytest.raises(ValueError):
        cca.CLTConfig(num_features=4, num_layers=1, d_model=2, activation_fn="batchtopk")
    with pytest.raises(ValueError):
        cca.CLTConfig(num_features=4, num_layers=1, d_model=2, activation_fn="topk")
    with pytest.raises(AssertionError):
        cca.CLTConfig(num_features=0, num_layers=1, d_model=2)
    with pytest.raises(AssertionError):
        cca.CLTConfig(num_features=4, num_layers=1, d_model=2, decoder_tying="bogus")
    c = cfg(clt_dtype="bfloat16", decoder_tying="per_target")
    p = tmp_path / "cfg.json"
    c.to_json(str(p))
    assert cca.CLTConfig.from_json(str(p)) == c
    # legacy keys of older checkpoints (reference clt/config/clt_config.py:91-112)
    legacy = {"num_features": 4, "num_layers": 1, "d_model": 2, "normalization_method": "auto",
              "sqrt_d_model_normalize": False}
    p.write_text(json.dumps(legacy))
    old = cca.CLTConfig.from_json(str(p))
    assert old.normalization_method == "mean_std" and old.decoder_tying == "none"
    legacy["sqrt_d_model_normalize"] = True
    p.write_text(json.dumps(legacy))
    assert cca.CLTConfig.from_json(str(p)).normalization_method == "sqrt_d_model"


def test_state_dict_schema_untied():
    # key names and shapes pinned by the reference's tests
    # (tests/unit/models/test_tied_decoders.py:39-57, test_distributed_checkpoint_weights.py:159-169)
    m = cca.CrossLayerTranscoder(cfg(), None, torch.device("cpu"))
    sd = m.state_dict()
    L, F, d = 3, 16, 8
    expect = {}
    for l in range(L):
        expect[f"encoder_module.encoders.{l}.weight"] = (F, d)
        expect[f"encoder_module.encoders.{l}.bias_param"] = (F,)
    for s in range(L):
        for t in range(s, L):
            expect[f"decoder_module.decoders.{s}->{t}.weight"] = (d, F)
            expect[f"decoder_module.decoders.{s}->{t}.bias_param"] = (d,)
    assert {k: tuple(v.shape) for k, v in sd.items()} == expect
    assert len(m.decoder_module.decoders) == L * (L + 1) // 2
    assert m.log_threshold is None


def test_state_dict_schema_tied_jumprelu_and_inits():
    c = cfg(activation_fn="jumprelu", batchtopk_k=None, jumprelu_threshold=0.5, decoder_tying="per_target",
            enable_feature_offset=True, enable_feature_scale=True, skip_connection=True)
    m = cca.CrossLayerTranscoder(c, None, torch.device("cpu"))
    sd = m.state_dict()
    assert sd["theta_manager.log_threshold"].shape == (3, 16)
    assert torch.allclose(sd["theta_manager.log_threshold"], torch.full((3, 16), math.log(0.5)))   # test_theta.py:63-72
    for i in range(3):
        assert sd[f"decoder_module.decoders.{i}.weight"].shape == (8, 16)
        assert float(sd[f"decoder_module.decoders.{i}.weight"].abs().sum()) == 0                     # tied: zero init
        assert sd[f"decoder_module.skip_weights.{i}"].shape == (8, 8)
        assert float(sd[f"decoder_module.skip_weights.{i}"].abs().sum()) == 0
        assert float(sd[f"decoder_module.feature_offset.{i}"].abs().sum()) == 0
    assert torch.equal(sd["decoder_module.feature_scale.0"], torch.ones(16))                           # test_tied_decoders.py:100-136
    assert torch.allclose(sd["decoder_module.feature_scale.1"], torch.full((16,), 0.1))
    assert m.log_threshold is m.theta_manager.log_threshold


def test_init_bounds_follow_reference_law():
    m = cca.CrossLayerTranscoder(cfg(num_features=64, d_model=32), None, torch.device("cpu"))
    w = m.encoder_module.encoders[0].weight
    assert float(w.abs().max()) <= 1 / math.sqrt(64) and float(w.abs().max()) > 0.5 / math.sqrt(64)
    wd = m.decoder_module.decoders["0->1"].weight
    assert float(wd.abs().max()) <= 1 / math.sqrt(3 * 32)
    assert float(m.encoder_module.encoders[0].bias_param.abs().sum()) == 0


def test_encoder_parameters_alias_one_slab_and_survive_to():
    m = cca.CrossLayerTranscoder(cfg(), None, torch.device("cpu"))
    w, b = m.encoder_module.stacked()
    for l, enc in enumerate(m.encoder_module.encoders):
        assert enc.weight.data_ptr() == w[l].data_ptr() and enc.bias_param.data_ptr() == b[l].data_ptr()
    before = [e.weight.detach().clone() for e in m.encoder_module.encoders]
    m = m.to(torch.float64).to(torch.float32)   # replaces parameter storage
    w2, _ = m.encoder_module.stacked()
    for l, enc in enumerate(m.encoder_module.encoders):
        assert enc.weight.data_ptr() == w2[l].data_ptr()
        assert torch.equal(enc.weight, before[l])
    sd = {k: torch.randn_like(v) for k, v in m.state_dict().items()}
    m.load_state_dict(sd)
    assert torch.equal(m.encoder_module.stacked()[0][1], sd["encoder_module.encoders.1.weight"])


def test_registry_api():
    assert set(cca.ACTIVATION_REGISTRY) >= {"relu", "jumprelu", "batchtopk", "topk"}
    with pytest.raises(ValueError):
        cca.get_activation_fn("nope")

    @cca.register_activation_fn("probe_identity")
    def ident(model, preact, layer_idx):
        return preact

    assert cca.get_activation_fn("probe_identity") is ident
    del cca.ACTIVATION_REGISTRY["probe_identity"]


def test_token_k_rule():
    from crosslayer_coding_amd.activations import resolve_token_k
    # reference tests/unit/models/test_activations.py:196-224
    assert resolve_token_k(0.6, 5) == 3 and resolve_token_k(0.5, 5) == 3
    assert resolve_token_k(1.0, 4) == 1 and resolve_token_k(5.0, 4) == 4
    assert resolve_token_k(0.0, 4) == 0 and resolve_token_k(-0.5, 4) == 0


def test_cpu_fallback_shapes_without_kernels(caplog):
    # inputs that never reach a kernel keep the reference's zero fallbacks even on CPU
    m = cca.CrossLayerTranscoder(cfg(), None, torch.device("cpu"))
    out = m.get_preactivations(torch.randn(5, 9), 0)          # wrong d_model
    assert out.shape == (5, 16) and float(out.abs().sum()) == 0
    out = m.get_preactivations(torch.randn(2, 3, 4, 8), 0)    # 4-D
    assert out.shape == (2, 16)
    assert m.decode({}, 0).shape == (0, 8)
    # conversion before any estimation: no statistics yet (reference tests/unit/models/test_theta.py:104-108)
    with pytest.raises(RuntimeError, match="Required buffer"):
        m.convert_to_jumprelu_inplace()


def test_workload_table_matches_baseline_shapes():
    w = synth.WORKLOADS
    assert (w["c1"].num_layers, w["c1"].d_model, w["c1"].num_features, w["c1"].tokens, w["c1"].k) == (12, 768, 24576, 4096, 200)
    assert (w["c0"].num_features, w["c0"].tokens, w["c0"].dtype) == (6144, 1024, "float32")
    assert (w["c2"].num_layers, w["c2"].d_model, w["c2"].num_features, w["c2"].activation_fn) == (24, 1024, 32768, "jumprelu")
    assert (w["c3"].num_layers, w["c3"].d_model, w["c3"].num_features, w["c3"].tokens, w["c3"].decoder_tying) == (16, 2048, 16384, 8192, "per_target")
    small = w["c0"].scaled("s", num_layers=2, d_model=16, num_features=32, tokens=64)
    x = synth.make_inputs(small)
    assert x.shape == (2, 64, 16) and abs(float(x[0].mean())) < 1e-5 and abs(float(x[0].std()) - 1) < 1e-3
    sd = synth.make_state_dict(small)
    assert float(sd["encoder_module.encoders.0.weight"].abs().max()) <= 1 / math.sqrt(16)
    assert sd["decoder_module.decoders.0->1.weight"].shape == (16, 32)


def test_convert_to_jumprelu_requires_estimation_first():
    # reference tests/unit/models/test_theta.py:104-108
    import pytest
    from crosslayer_coding_amd.config import CLTConfig
    from crosslayer_coding_amd.theta import ThetaManager

    cfg = CLTConfig(num_layers=2, d_model=8, num_features=4, activation_fn="batchtopk", batchtopk_k=2)
    tm = ThetaManager(cfg, None, torch.device("cpu"), torch.float32)
    with pytest.raises(RuntimeError, match="Required buffer .* not found"):
        tm.convert_to_jumprelu_inplace()


def test_manifest_formats_and_fallback(tmp_path):
    from crosslayer_coding_amd.feed import read_manifest
    # legacy pairs (tests/unit/data/test_data_integrity.py:296-357 writes both formats)
    legacy = np.array([(0, 0), (0, 1), (1, 0), (1, 1), (1, 2)], dtype=np.uint32)
    p = tmp_path / "legacy.bin"
    legacy.tofile(p)
    assert np.array_equal(read_manifest(p), legacy)      # 40 bytes: not a multiple of 16
    # 16-byte records expand to per-row entries, empty chunks are skipped
    rec = np.array([(0, 2, 0), (1, 0, 2), (2, 3, 2)], dtype=[("chunk_id", np.int32), ("num_tokens", np.int32), ("offset", np.int64)])
    p3 = tmp_path / "records.bin"
    rec.tofile(p3)
    want = np.array([(0, 0), (0, 1), (2, 0), (2, 1), (2, 2)], dtype=np.uint32)
    assert np.array_equal(read_manifest(p3), want)
    assert np.array_equal(read_manifest(p3, total_tokens=5), want)
    # a legacy file whose size happens to be a multiple of 16: the token total tells the formats apart
    even = np.array([(0, 0), (0, 1), (1, 0), (1, 1)], dtype=np.uint32)
    pe = tmp_path / "even.bin"
    even.tofile(pe)
    assert np.array_equal(read_manifest(pe, total_tokens=4), even)
    assert read_manifest(tmp_path / "absent.bin") is None
    (tmp_path / "odd.bin").write_bytes(bytes(12))
    assert read_manifest(tmp_path / "odd.bin") is None


def test_normalisation_tables_follow_prep_norm():
    from crosslayer_coding_amd.feed import prepare_normalization
    good = {"0": {"inputs": {"mean": [1.0, 2.0], "std": [0.5, 0.0]}, "targets": {"mean": [0.0, 0.0], "std": [1.0, 1.0]}},
            "1": {"inputs": {"mean": [3.0, 4.0], "std": [2.0, 2.0]}, "targets": {"mean": [1.0, 1.0], "std": [3.0, 3.0]}},
            "7": {"inputs": {"mean": [0.0, 0.0], "std": [1.0, 1.0]}}}       # unknown layer: skipped
    ok, mi, si, mt, st = prepare_normalization(good, [0, 1], 2)
    assert ok and mi.tolist() == [[1.0, 2.0], [3.0, 4.0]]
    assert torch.equal(si, torch.tensor([[0.5, 0.0], [2.0, 2.0]]) + 1e-6)
    assert torch.equal(st, torch.tensor([[1.0, 1.0], [3.0, 3.0]]) + 1e-6) and mt.tolist() == [[0.0, 0.0], [1.0, 1.0]]
    assert si[0, 1].item() == pytest.approx(1e-6)                           # std 0 survives thanks to the epsilon
    for bad in (None, {}, {"0": good["0"]},                                  # nothing, or layer 1 missing
                {"0": good["0"], "1": {"inputs": good["1"]["inputs"]}},      # no targets
                {"0": good["0"], "1": {**good["1"], "targets": {"mean": [0.0, 0.0], "std": [-1.0, 1.0]}}}):
        assert prepare_normalization(bad, [0, 1], 2)[0] is False


def test_feed_rejects_bad_arguments_and_needs_a_gpu():
    from crosslayer_coding_amd import DeviceActivationFeed
    from crosslayer_coding_amd._native import CLTNativeError
    with pytest.raises(ValueError):
        DeviceActivationFeed(2, 8, normalization_method="bogus")
    with pytest.raises(ValueError):
        DeviceActivationFeed(2, 8, dtype="float64")
    feed = DeviceActivationFeed(2, 8, dtype="float32", device="cpu", normalization_method="mean_std", norm_stats=None)
    assert feed.apply_normalization is False
    if not torch.cuda.is_available():
        with pytest.raises(CLTNativeError):
            feed.parse_batch(np.zeros((4, 2), dtype=np.uint32))
    with pytest.raises(ValueError):
        feed.add_chunk(0, torch.zeros(2, 2, 5, 7))


def test_more_than_64_layers_are_constructed():
    # deeper models run on the dense formulations
    import pytest
    m = cca.CrossLayerTranscoder(cfg(num_layers=65, decoder_tying="per_source"), None, torch.device("cpu"))
    assert len(m.decoder_module.decoders) == 65
    cca.CrossLayerTranscoder(cfg(num_layers=65, decoder_tying="per_source", skip_connection=True), None, torch.device("cpu"))
    cca.CrossLayerTranscoder(cfg(num_layers=65, decoder_tying="per_source", activation_fn="topk", topk_k=4.0,
                                 batchtopk_k=None), None, torch.device("cpu"))
