"""The oracle against tests/golden/reference_fixtures.json: inputs, parameters and outputs of tiny
seeded runs of the reference's own code on the CPU (written by tests/golden/make_reference_fixtures.py).
These pin what the reference's unit tests leave open: the full forward wiring for every tying / skip /
affine variant, the global BatchTopK / TokenTopK helper, post-hoc theta estimation, the gradients of the
reconstruction loss (straight-through gate, JumpReLU threshold gradient, tied decoders) and the
evaluator's metric formulas."""
import json
import math
import os

import pytest
import torch

from oracle import clt_oracle as orc

FIX = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_fixtures.json")))


def T(x):
    return torch.tensor(x, dtype=torch.float32)


def unpack(case):
    cfg, sd = case["config"], {k: T(v) for k, v in case["state_dict"].items()}
    L = cfg["num_layers"]
    tying = cfg.get("decoder_tying", "none")
    names = [f"{s}->{t}" for s in range(L) for t in range(s, L)] if tying == "none" else [str(i) for i in range(L)]
    kw = dict(enc_w=[sd[f"encoder_module.encoders.{l}.weight"] for l in range(L)],
              enc_b=[sd[f"encoder_module.encoders.{l}.bias_param"] for l in range(L)],
              dec_w={n: sd[f"decoder_module.decoders.{n}.weight"] for n in names},
              dec_b={n: sd[f"decoder_module.decoders.{n}.bias_param"] for n in names})
    return cfg, sd, L, tying, names, kw


def model_kwargs(cfg, sd, L, tying, names):
    fn = cfg["activation_fn"]
    k = cfg.get("batchtopk_k") if fn == "batchtopk" else cfg.get("topk_k")
    extra = dict(activation_fn=fn, num_layers=L, tying=tying, k=k)
    if fn == "jumprelu":
        extra["log_threshold"] = sd["theta_manager.log_threshold"]
    if cfg.get("skip_connection"):
        extra["skip_weights"] = {n: sd[f"decoder_module.skip_weights.{n}"] for n in names}
    if cfg.get("enable_feature_offset"):
        extra["feature_offset"] = [sd[f"decoder_module.feature_offset.{i}"] for i in range(L)]
    if cfg.get("enable_feature_scale"):
        extra["feature_scale"] = [sd[f"decoder_module.feature_scale.{i}"] for i in range(L)]
    return extra


@pytest.mark.parametrize("case", FIX["forward"], ids=lambda c: c["name"])
def test_oracle_forward_matches_the_reference(case):
    cfg, sd, L, tying, names, kw = unpack(case)
    dtype = getattr(torch, cfg.get("clt_dtype", "float32"))
    if dtype != torch.float32:
        kw = {k: ([w.to(dtype) for w in v] if isinstance(v, list) else {n: w.to(dtype) for n, w in v.items()}) for k, v in kw.items()}
    inputs = {int(l): T(v).to(dtype) for l, v in case["inputs"].items()}
    extra = model_kwargs(cfg, sd, L, tying, names)
    recs, acts = orc.forward(inputs, **kw, dtype=dtype, d_model=cfg["d_model"], num_features=cfg["num_features"],
                             topk_mode="global", **extra)
    for l in range(L):
        want_a, want_r = T(case["activations"][str(l)]), T(case["reconstructions"][str(l)])
        pre = orc.encoder_preactivations(inputs[l], kw["enc_w"][l], kw["enc_b"][l])
        if dtype == torch.float32:
            assert torch.allclose(pre, T(case["preactivations"][str(l)]), rtol=1e-5, atol=1e-6)
            assert torch.equal(acts[l] != 0, want_a != 0), f"selected set of layer {l}"
            assert torch.allclose(acts[l], want_a, rtol=1e-5, atol=1e-6)
            assert torch.allclose(recs[l], want_r, rtol=1e-5, atol=1e-5)
        else:   # the same torch-CPU ops on the same bf16 values: equal
            assert torch.equal(pre.float(), T(case["preactivations"][str(l)]))
            assert torch.equal(acts[l].float(), want_a)
            assert orc.rel_l2(recs[l].float(), want_r) <= 1e-2
    got_n = orc.decoder_norms(kw["dec_w"], L, cfg["num_features"], tying, dtype).float()
    assert torch.allclose(got_n, T(case["decoder_norms"]), rtol=2e-2 if dtype != torch.float32 else 1e-5, atol=1e-6)


@pytest.mark.parametrize("case", FIX["theta_estimation"], ids=lambda c: c["config"]["activation_fn"])
def test_oracle_theta_estimation_matches_the_reference(case):
    cfg, sd, L, tying, names, kw = unpack(case)
    fn = cfg["activation_fn"]
    k = cfg["batchtopk_k"] if fn == "batchtopk" else cfg["topk_k"]
    batches = [{int(l): orc.encoder_preactivations(T(v), kw["enc_w"][int(l)], kw["enc_b"][int(l)]) for l, v in b.items()}
               for b in case["batches"]]
    s, c, mu, sg = orc.theta_estimate_posthoc(batches, activation_fn=fn, k=k, num_layers=L, num_features=cfg["num_features"],
                                              dtype=torch.float32)
    log_theta = orc.theta_convert(s, c, mu, sg)
    assert case["activation_fn_after"] == "jumprelu"
    assert torch.allclose(log_theta, T(case["log_threshold_after"]), rtol=1e-4, atol=1e-5)
    assert torch.allclose(torch.exp(log_theta), T(case["theta"]), rtol=1e-4, atol=1e-6)     # the method's return value


@pytest.mark.parametrize("case", FIX["gradients"] + FIX["gradients_normalized"] + FIX["gradients_skip_affine"] + FIX["gradients_jumprelu_affine"],
                         ids=lambda c: c["name"])
def test_oracle_gradients_match_the_reference(case):
    cfg, sd, L, tying, names, kw = unpack(case)
    fn = cfg["activation_fn"]
    inputs = {int(l): T(v) for l, v in case["inputs"].items()}
    targets = {int(l): T(v) for l, v in case["targets"].items()}
    masks = None
    if fn == "batchtopk":      # the reference's default scope is global: the gate comes from the global helper
        pre = {l: orc.encoder_preactivations(inputs[l], kw["enc_w"][l], kw["enc_b"][l]) for l in range(L)}
        masks = {l: a != 0 for l, a in orc.global_batchtopk(pre, L, cfg["batchtopk_k"]).items()}
    extra = {}
    if "normalization_method" in case:      # the loss on de-normalised tensors (losses.py:70-86)
        extra = dict(normalization_method=case["normalization_method"],
                     mean_tg={int(l): T(v) for l, v in case["mean_tg"].items()},
                     std_tg={int(l): T(v) for l, v in case["std_tg"].items()})
    if cfg.get("skip_connection"):
        extra["skip_w"] = {n: sd[f"decoder_module.skip_weights.{n}"] for n in names}
    if cfg.get("enable_feature_offset"):
        extra["feature_offset"] = [sd[f"decoder_module.feature_offset.{i}"] for i in range(L)]
    if cfg.get("enable_feature_scale"):
        extra["feature_scale"] = [sd[f"decoder_module.feature_scale.{i}"] for i in range(L)]
    loss, grads = orc.mse_loss_and_gradients(inputs, targets, **kw, activation_fn=fn, num_layers=L, k=cfg.get("batchtopk_k"),
                                             masks=masks, tying=tying, **extra,
                                             log_threshold=sd.get("theta_manager.log_threshold") if fn == "jumprelu" else None)
    assert float(loss) == pytest.approx(case["loss"], rel=1e-5)
    assert set(case["gradients"]) <= set(grads), set(case["gradients"]) - set(grads)
    for name, want in case["gradients"].items():
        assert torch.allclose(grads[name], T(want), rtol=1e-4, atol=1e-6), name


@pytest.mark.parametrize("method", ["none", "mean_std", "sqrt_d_model"])
def test_oracle_evaluator_metrics_match_the_reference(method):
    ev = FIX["evaluator"]
    acts = {int(l): T(v) for l, v in ev["activations"].items()}
    tg = {int(l): T(v) for l, v in ev["targets"].items()}
    rc = {int(l): T(v) for l, v in ev["reconstructions"].items()}
    mean = {int(l): T(v) for l, v in ev["mean_tg"].items()}
    std = {int(l): T(v) for l, v in ev["std_tg"].items()}
    got = {**orc.sparsity_metrics(acts, ev["num_features"], ev["num_layers"]), **orc.feature_density_metrics(acts),
           **orc.reconstruction_metrics(tg, rc, method=method, mean_tg=mean, std_tg=std, d_model=ev["d_model"])}
    want = ev["metrics"][method]
    assert got.keys() == want.keys()

    def same(a, b, path):
        if isinstance(b, dict):
            assert a.keys() == b.keys(), path
            for k in b:
                same(a[k], b[k], f"{path}/{k}")
        elif isinstance(b, list):
            assert len(a) == len(b), path
            for i, (x, y) in enumerate(zip(a, b)):
                same(x, y, f"{path}[{i}]")
        else:
            assert a == pytest.approx(b, rel=1e-6, abs=1e-9) or (math.isinf(a) and math.isinf(b)), (path, a, b)

    same(got, want, method)


@pytest.mark.parametrize("case", FIX["global_select"], ids=lambda c: c["dtype"])
def test_oracle_global_selection_matches_the_reference_in_each_dtype(case):
    # pre-activations handed over as they are: the selected set must be the reference's, bit for bit
    dtype = getattr(torch, case["dtype"])
    pre = {int(l): T(v).to(dtype) for l, v in case["preactivations"].items()}
    L = len(pre)
    got_b = orc.global_batchtopk(pre, L, case["batchtopk_k"])
    got_t = orc.global_tokentopk(pre, L, float(case["topk_k"]))
    for l in range(L):
        assert torch.equal(got_b[l].float(), T(case["batchtopk"][str(l)])), ("batchtopk", l)
        assert torch.equal(got_t[l].float(), T(case["tokentopk"][str(l)])), ("tokentopk", l)


@pytest.mark.parametrize("case", FIX["config_json"], ids=lambda c: c["kwargs"]["activation_fn"])
def test_config_json_round_trip_matches_the_reference(case, tmp_path):
    # cfg.json as the reference writes it: this build reads it to the same field values, and writes the
    # same file for the same constructor arguments
    import json as _json
    from crosslayer_coding_amd import CLTConfig
    path = tmp_path / "cfg.json"
    path.write_text(_json.dumps(case["json"]))
    cfg = CLTConfig.from_json(str(path))
    for key, want in case["fields_after_reload"].items():
        assert getattr(cfg, key) == want, key
    out = tmp_path / "mine.json"
    CLTConfig(**case["kwargs"]).to_json(str(out))
    assert _json.loads(out.read_text()) == case["json"]


@pytest.mark.parametrize("case", FIX["per_layer"], ids=lambda c: c["name"])
def test_oracle_per_layer_scope_matches_the_reference_registry(case):
    # the registry's per-layer BatchTopK / TokenTopK on given pre-activations: bit for bit, in the model dtype
    cfg = case["config"]
    dtype = getattr(torch, cfg.get("clt_dtype", "float32"))
    for l, pre in case["preactivations"].items():
        pre = T(pre).to(dtype)
        if cfg["activation_fn"] == "batchtopk":
            got = orc.batchtopk_forward(pre, float(cfg["batchtopk_k"]), pre)
        else:
            got = orc.tokentopk_forward(pre, float(cfg["topk_k"]), pre)
        assert torch.equal(got.float(), T(case["activations"][l])), l
