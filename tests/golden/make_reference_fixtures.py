#!/usr/bin/env python3
"""Writes tests/golden/reference_fixtures.json: inputs, parameters and outputs of tiny seeded runs of
the reference's own code, for the functions that nothing else pins (full forward wiring, the global
BatchTopK / TokenTopK helper, post-hoc theta estimation, gradients of the reconstruction loss, the
evaluator's metric formulas).

Runs only where the reference checkout is present (default /root/reference, or the path given as
the first argument); it imports the reference on the CPU and nothing else.  The JSON it writes is
data only and is what travels: the tests read the JSON, never the reference.

    python tests/golden/make_reference_fixtures.py [/path/to/reference] [--only=section,section]

With --only the named top-level sections are (re)computed and merged into the existing file; the other
sections keep the values they have.
"""
import json
import os
import sys

import torch

sys.dont_write_bytecode = True     # the reference checkout is read-only for this build: no __pycache__ there
_ARGS = [a for a in sys.argv[1:] if not a.startswith("--")]
REF = _ARGS[0] if _ARGS else "/root/reference"
sys.path.insert(0, REF)

from clt.config import CLTConfig, TrainingConfig          # noqa: E402
from clt.models.activations import _apply_batch_topk_helper, _apply_token_topk_helper   # noqa: E402
from clt.activations.registry import get_activation_fn    # noqa: E402
from clt.models.clt import CrossLayerTranscoder           # noqa: E402
from clt.training.evaluator import CLTEvaluator           # noqa: E402
from clt.training.losses import LossManager               # noqa: E402

torch.set_num_threads(1)
CPU = torch.device("cpu")


def lists(obj):
    if isinstance(obj, torch.Tensor):
        return obj.detach().to(torch.float64).tolist()
    if isinstance(obj, dict):
        return {str(k): lists(v) for k, v in obj.items()}
    if isinstance(obj, (list, tuple)):
        return [lists(v) for v in obj]
    return obj


def build(cfg_kw, seed):
    torch.manual_seed(seed)
    cfg = CLTConfig(**cfg_kw)
    model = CrossLayerTranscoder(cfg, process_group=None, device=CPU)
    g = torch.Generator().manual_seed(seed + 1)
    with torch.no_grad():
        for name, p in model.named_parameters():
            if name.endswith("log_threshold"):
                p.copy_(torch.log(0.05 + 0.3 * torch.rand(p.shape, generator=g)))
            elif "feature_scale" in name:
                p.copy_(0.5 + torch.rand(p.shape, generator=g))
            else:
                p.copy_(torch.randn(p.shape, generator=g) * 0.4)
    model.eval()
    return cfg, model, g


def forward_case(name, cfg_kw, seed, tokens=5, save_as=None):
    cfg, model, g = build(cfg_kw, seed)
    if save_as:      # the reference's own checkpoint format (BaseTranscoder.save): one torch file
        model.save(os.path.join(os.path.dirname(os.path.abspath(__file__)), save_as))
    L, d = cfg.num_layers, cfg.d_model
    dtype = next(model.parameters()).dtype
    inputs = {l: torch.randn(tokens, d, generator=g).to(dtype) for l in range(L)}
    with torch.no_grad():
        recs = model(inputs)
        acts = model.get_feature_activations(inputs)
        pre = {l: model.get_preactivations(inputs[l], l) for l in range(L)}
        norms = model.get_decoder_norms()
        # the per-layer entry points: encode(x, layer) and decode(activations up to a layer, layer)
        encoded = {l: model.encode(inputs[l], l) for l in range(L)}
        mid = L // 2
        decoded_mid = model.decode({l: acts[l] for l in range(mid + 1)}, mid)
    return {"name": name, "config": cfg_kw, "state_dict": lists(dict(model.state_dict())), "inputs": lists(inputs),
            "reconstructions": lists(recs), "activations": lists(acts), "preactivations": lists(pre),
            "decoder_norms": lists(norms), "encode": lists(encoded), "decode_layer": mid, "decode": lists(decoded_mid)}


def irregular_cases(seed):
    """Inputs the reference answers with its fallbacks: a missing layer, 3-D inputs, a layer whose width
    is wrong, a layer with another token count."""
    out = {"models": {}, "cases": []}
    for fn_kw in (dict(activation_fn="relu"), dict(activation_fn="batchtopk", batchtopk_k=3)):
        cfg_kw = dict(num_features=16, num_layers=3, d_model=8, **fn_kw)
        cfg, model, g = build(cfg_kw, seed)
        out["models"][fn_kw["activation_fn"]] = {"config": cfg_kw, "state_dict": lists(dict(model.state_dict()))}
        variants = {
            "missing-layer-1": {0: torch.randn(5, 8, generator=g), 2: torch.randn(5, 8, generator=g)},
            "three-dimensional": {l: torch.randn(2, 3, 8, generator=g) for l in range(3)},
            "wrong-width-layer-1": {0: torch.randn(5, 8, generator=g), 1: torch.randn(5, 7, generator=g),
                                    2: torch.randn(5, 8, generator=g)},
            "other-token-count-layer-2": {0: torch.randn(5, 8, generator=g), 1: torch.randn(5, 8, generator=g),
                                          2: torch.randn(4, 8, generator=g)},
        }
        for vname, inputs in variants.items():
            with torch.no_grad():
                try:
                    recs = lists(model(inputs))
                    acts = lists(model.get_feature_activations(inputs))
                    err = None
                except Exception as e:      # the reference itself fails on this input: recorded as such
                    recs, acts, err = None, None, type(e).__name__
            out["cases"].append({"name": f"{fn_kw['activation_fn']}-{vname}", "model": fn_kw["activation_fn"],
                                 "inputs": lists(inputs), "reconstructions": recs, "activations": acts, "raises": err})
    return out


def config_json_cases():
    """cfg.json as the reference writes it, for two configurations."""
    import tempfile
    out = []
    for kw in (dict(num_features=16, num_layers=3, d_model=8, activation_fn="batchtopk", batchtopk_k=3),
               dict(num_features=32, num_layers=2, d_model=4, activation_fn="jumprelu", decoder_tying="per_target",
                    enable_feature_offset=True, enable_feature_scale=True, skip_connection=True, clt_dtype="bfloat16",
                    model_name="gpt2", jumprelu_threshold=0.05)):
        cfg = CLTConfig(**kw)
        with tempfile.TemporaryDirectory() as tmp:
            path = os.path.join(tmp, "cfg.json")
            cfg.to_json(path)
            written = json.load(open(path))
            back = CLTConfig.from_json(path)
        out.append({"kwargs": kw, "json": written, "fields_after_reload": {k: getattr(back, k) for k in written}})
    return out


def migration_case(seed):
    """An untied checkpoint, with its feature affine parameters under the old encoder_module names, loaded
    into a per-source model by the reference's load_state_dict (clt.py:347-432)."""
    base = dict(num_features=16, num_layers=3, d_model=8, activation_fn="relu")
    _, untied, g = build(base, seed)
    tied_kw = dict(base, decoder_tying="per_source", enable_feature_offset=True, enable_feature_scale=True)
    _, tied, _ = build(tied_kw, seed + 5)
    old = {k: v.clone() for k, v in untied.state_dict().items()}
    for i in range(3):
        old[f"encoder_module.feature_offset.{i}"] = torch.randn(16, generator=g) * 0.1
        old[f"encoder_module.feature_scale.{i}"] = 0.5 + torch.rand(16, generator=g)
    tied.load_state_dict(dict(old))
    tied.eval()
    inputs = {l: torch.randn(5, 8, generator=g) for l in range(3)}
    with torch.no_grad():
        recs = tied(inputs)
    return {"config": tied_kw, "old_state_dict": lists(old), "state_dict_after": lists(dict(tied.state_dict())),
            "inputs": lists(inputs), "reconstructions": lists(recs)}


def per_layer_case(name, cfg_kw, seed, tokens=16):
    """The per-layer scope of BatchTopK / TokenTopK, assembled from the reference's own pieces: the registry's
    per-layer activation (clt/activations/registry.py:43-98) on the model's pre-activations, then
    Decoder.decode per target.  (The model's own forward does not reach the registry function for this scope in
    this snapshot.)  Seeds with a tie at the threshold are skipped."""
    while True:
        cfg, model, g = build(cfg_kw, seed)
        dtype = next(model.parameters()).dtype
        L, d = cfg.num_layers, cfg.d_model
        inputs = {l: torch.randn(tokens, d, generator=g).to(dtype) for l in range(L)}
        fn = get_activation_fn(cfg.activation_fn)
        with torch.no_grad():
            pre = {l: model.get_preactivations(inputs[l], l) for l in range(L)}
            ok = True
            for l in range(L):
                if cfg.activation_fn == "batchtopk":
                    flat = torch.sort(pre[l].float().reshape(-1), descending=True).values
                    K = int(cfg.batchtopk_k) * tokens
                    ok = ok and bool(flat[K - 1] != flat[K])
                else:
                    rows = torch.sort(pre[l].float(), dim=1, descending=True).values
                    kk = int(cfg.topk_k)
                    ok = ok and bool((rows[:, kk - 1] != rows[:, kk]).all())
            if not ok:
                seed += 1000
                continue
            acts = {l: fn(model, pre[l], l) for l in range(L)}
            recs = {t: model.decode({s_: acts[s_] for s_ in range(t + 1)}, t) for t in range(L)}
        return {"name": name, "config": dict(cfg_kw, topk_mode="per_layer"), "seed": seed,
                "state_dict": lists(dict(model.state_dict())), "inputs": lists(inputs), "preactivations": lists(pre),
                "activations": lists(acts), "reconstructions": lists(recs)}


def theta_case(cfg_kw, seed, tokens=6, batches=3):
    cfg, model, g = build(cfg_kw, seed)
    L, d = cfg.num_layers, cfg.d_model
    data = [({l: torch.randn(tokens, d, generator=g) for l in range(L)},
             {l: torch.randn(tokens, d, generator=g) for l in range(L)}) for _ in range(batches)]
    sd_before = lists(dict(model.state_dict()))
    theta = model.estimate_theta_posthoc(iter(data), num_batches=batches, default_theta_value=1e6, device=CPU)
    return {"config": cfg_kw, "state_dict": sd_before, "batches": [lists(b[0]) for b in data],
            "theta": lists(theta), "log_threshold_after": lists(model.log_threshold),
            "activation_fn_after": model.config.activation_fn}


def gradient_case(name, cfg_kw, seed, tokens=6):
    cfg, model, g = build(cfg_kw, seed)
    model.train()
    L, d = cfg.num_layers, cfg.d_model
    inputs = {l: torch.randn(tokens, d, generator=g) for l in range(L)}
    targets = {l: torch.randn(tokens, d, generator=g) for l in range(L)}
    tc = TrainingConfig(learning_rate=1e-4, training_steps=10, activation_source="local_manifest",
                        activation_path="unused", normalization_method="none")
    lm = LossManager(tc, clt_config=cfg)
    loss = lm.compute_reconstruction_loss(model(inputs), targets)
    loss.backward()
    grads = {n: p.grad for n, p in model.named_parameters() if p.grad is not None}
    return {"name": name, "config": cfg_kw, "state_dict": lists(dict(model.state_dict())), "inputs": lists(inputs),
            "targets": lists(targets), "loss": float(loss), "gradients": lists(grads)}


def gradient_case_normalized(name, cfg_kw, seed, method, tokens=6, stat_layers=None):
    """Loss and gradients with the de-normalisation of LossManager.compute_reconstruction_loss
    (clt/training/losses.py:70-86): target statistics as the trainer takes them from the activation store
    ([1, d_model] per layer), or the 1 / sqrt(d_model) scaling.  ``stat_layers``: only these layers have
    statistics (the reference de-normalises those and leaves the others alone)."""
    cfg, model, g = build(cfg_kw, seed)
    model.train()
    L, d = cfg.num_layers, cfg.d_model
    inputs = {l: torch.randn(tokens, d, generator=g) for l in range(L)}
    targets = {l: torch.randn(tokens, d, generator=g) for l in range(L)}
    mean = {l: torch.randn(1, d, generator=g) * 0.5 for l in range(L)}
    std = {l: torch.rand(1, d, generator=g) + 0.5 for l in range(L)}
    if stat_layers is not None:
        mean = {l: v for l, v in mean.items() if l in stat_layers}
        std = {l: v for l, v in std.items() if l in stat_layers}
    tc = TrainingConfig(learning_rate=1e-4, training_steps=10, activation_source="local_manifest",
                        activation_path="unused", normalization_method=method)
    lm = LossManager(tc, mean_tg=mean, std_tg=std, clt_config=cfg)
    loss = lm.compute_reconstruction_loss(model(inputs), targets)
    loss.backward()
    grads = {n: p.grad for n, p in model.named_parameters() if p.grad is not None}
    return {"name": name, "config": cfg_kw, "normalization_method": method, "mean_tg": lists(mean), "std_tg": lists(std),
            "state_dict": lists(dict(model.state_dict())), "inputs": lists(inputs), "targets": lists(targets),
            "loss": float(loss), "gradients": lists(grads)}


def evaluator_subset_case(seed):
    """CLTEvaluator.compute_metrics when the batch holds only some of the layers: the reference's
    metrics run over the layers get_feature_activations returned (evaluator.py:194-244, 350-405)."""
    cfg_kw = dict(num_features=16, num_layers=4, d_model=8, activation_fn="relu")
    cfg, model, g = build(cfg_kw, seed)
    layers = [0, 2]
    inputs = {l: torch.randn(9, 8, generator=g) for l in layers}
    targets = {l: torch.randn(9, 8, generator=g) for l in layers}
    ev = CLTEvaluator(model, CPU)
    metrics = ev.compute_metrics(inputs, targets)
    return {"config": cfg_kw, "state_dict": lists(dict(model.state_dict())), "inputs": lists(inputs),
            "targets": lists(targets), "metrics": lists(metrics)}


def evaluator_case(seed):
    cfg_kw = dict(num_features=12, num_layers=2, d_model=6, activation_fn="relu")
    cfg, model, g = build(cfg_kw, seed)
    acts = {l: torch.relu(torch.randn(7, 12, generator=g) - 0.3) for l in range(2)}
    acts[1][:, 4] = 0.0
    acts[0][2, 1] = 5e-7
    targets = {l: torch.randn(7, 6, generator=g) * (1 + l) + 0.5 for l in range(2)}
    recs = {l: targets[l] + 0.3 * torch.randn(7, 6, generator=g) for l in range(2)}
    mean = {l: torch.randn(1, 6, generator=g) for l in range(2)}
    std = {l: torch.rand(1, 6, generator=g) + 0.5 for l in range(2)}
    out = {"activations": lists(acts), "targets": lists(targets), "reconstructions": lists(recs), "mean_tg": lists(mean),
           "std_tg": lists(std), "num_features": 12, "num_layers": 2, "d_model": 6, "metrics": {}}
    for method in ("none", "mean_std", "sqrt_d_model"):
        ev = CLTEvaluator(model, CPU, mean_tg=mean, std_tg=std, normalization_method=method, d_model=6)
        m = {}
        m.update(ev._compute_sparsity(acts))
        m.update(ev._compute_feature_density(acts))
        m.update(ev._compute_reconstruction_metrics(targets, recs))
        out["metrics"][method] = lists(m)
    return out


def global_select_case(dtype, seed, L=3, tokens=16, F=32, k=5, kk=6):
    """The global helpers fed pre-activations directly, in ``dtype``: pins the rounding sequence of the
    ranking values.  Seeds whose k-th and (k+1)-th ranking values coincide are skipped, because
    torch.topk's choice among equal values is unspecified."""
    while True:
        g = torch.Generator().manual_seed(seed)
        pre = {l: (torch.randn(tokens, F, generator=g) * (0.5 + l) + 0.3 * l).to(dtype) for l in range(L)}
        z = torch.cat([(p - p.mean(dim=0, keepdim=True)) / (p.std(dim=0, keepdim=True) + 1e-6) for p in pre.values()], dim=1)
        flat = torch.sort(z.float().reshape(-1), descending=True).values
        rows = torch.sort(z.float(), dim=1, descending=True).values
        if flat[k * tokens - 1] != flat[k * tokens] and bool((rows[:, kk - 1] != rows[:, kk]).all()):
            break
        seed += 1000
    name = str(dtype).split(".")[-1]
    cfg_b = CLTConfig(num_features=F, num_layers=L, d_model=8, activation_fn="batchtopk", batchtopk_k=k, clt_dtype=name)
    cfg_t = CLTConfig(num_features=F, num_layers=L, d_model=8, activation_fn="topk", topk_k=float(kk), clt_dtype=name)
    out_b = _apply_batch_topk_helper(pre, cfg_b, CPU, dtype, 0, None)
    out_t = _apply_token_topk_helper(pre, cfg_t, CPU, dtype, 0, None)
    return {"dtype": name, "seed": seed, "batchtopk_k": k, "topk_k": kk, "preactivations": lists(pre),
            "batchtopk": lists(out_b), "tokentopk": lists(out_t)}


def compute_metrics_case(seed):
    """CLTEvaluator.compute_metrics end to end on a seeded model (global BatchTopK)."""
    cfg_kw = dict(num_features=16, num_layers=3, d_model=8, activation_fn="batchtopk", batchtopk_k=3)
    cfg, model, g = build(cfg_kw, seed)
    inputs = {l: torch.randn(12, 8, generator=g) for l in range(3)}
    targets = {l: torch.randn(12, 8, generator=g) for l in range(3)}
    mask = torch.zeros(3, 16, dtype=torch.bool)
    mask[0, :3] = True
    mask[2, 5] = True
    ev = CLTEvaluator(model, CPU)
    metrics = ev.compute_metrics(inputs, targets, dead_neuron_mask=mask)
    return {"config": cfg_kw, "state_dict": lists(dict(model.state_dict())), "inputs": lists(inputs), "targets": lists(targets),
            "dead_neuron_mask": mask.int().tolist(), "metrics": lists(metrics)}


def c0_summary():
    """The full-size fp32 configuration (12 layers, d_model 768, 6144 features, 1024 tokens, k = 200) through the
    reference, on the weights and inputs of this build's own generator drawn on the CPU (so the test can
    rebuild them anywhere).  Too large to store: kept are, per layer, the sum and sum of squares of the
    reconstruction, the number of non-zero activations, and four token rows of three layers in full; for the
    global scope (the model's own forward) and for the per-layer scope (registry function + decode)."""
    sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__)))))
    from crosslayer_coding_amd import synth
    wl = synth.WORKLOADS["c0"]
    sd = synth.make_state_dict(wl, "cpu")
    x = synth.make_inputs(wl, "cpu")
    L = wl.num_layers
    rows = [0, 333, 700, 1023]
    out = {"workload": "c0", "rows": rows, "layers_in_full": [0, 6, 11]}
    for scope in ("global", "per_layer"):
        cfg = CLTConfig(num_features=wl.num_features, num_layers=L, d_model=wl.d_model, activation_fn="batchtopk",
                        batchtopk_k=wl.k)
        model = CrossLayerTranscoder(cfg, process_group=None, device=CPU)
        model.load_state_dict(sd)
        model.eval()
        inputs = {l: x[l] for l in range(L)}
        with torch.no_grad():
            if scope == "global":
                recs = model(inputs)
                acts = model.get_feature_activations(inputs)
            else:
                fn = get_activation_fn("batchtopk")
                acts = {l: fn(model, model.get_preactivations(inputs[l], l), l) for l in range(L)}
                recs = {t: model.decode({s_: acts[s_] for s_ in range(t + 1)}, t) for t in range(L)}
        out[scope] = {"sum": [float(recs[l].double().sum()) for l in range(L)],
                      "sumsq": [float((recs[l].double() ** 2).sum()) for l in range(L)],
                      "nonzero": [int((acts[l] != 0).sum()) for l in range(L)],
                      "rows": {str(l): lists(recs[l][rows]) for l in out["layers_in_full"]}}
    return out


def c1_summary():
    """The headline configuration (bf16, 12 layers, d_model 768, 24576 features, 4096 tokens, k = 200, per-layer
    scope) through the reference's registry function and decode, on this build's CPU-drawn weights and inputs.
    Kept: per layer the sum of squares of the reconstruction and the number of non-zero activations, and 16
    token rows of three layers in full, each with a flag: whether, in any source layer up to the row's layer,
    that token holds a pre-activation equal to the layer's threshold value (the smallest kept value) or one
    bf16 step beside it.  torch.topk's choice among equal values is unspecified, and two encoders that sum in
    different orders can put such an element on either side of the threshold; rows without the flag have the
    same survivors whatever the implementation.  Takes a few minutes."""
    sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__)))))
    from crosslayer_coding_amd import synth
    torch.set_num_threads(8)
    wl = synth.WORKLOADS["c1"]
    sd = synth.make_state_dict(wl, "cpu")
    x = synth.make_inputs(wl, "cpu")
    L = wl.num_layers
    rows = [0, 257, 513, 770, 1026, 1333, 1539, 1796, 2052, 2309, 2700, 2822, 3078, 3335, 3591, 4095]
    cfg = CLTConfig(num_features=wl.num_features, num_layers=L, d_model=wl.d_model, activation_fn="batchtopk",
                    batchtopk_k=wl.k, clt_dtype="bfloat16")
    model = CrossLayerTranscoder(cfg, process_group=None, device=CPU)
    model.load_state_dict(sd)
    model.eval()
    fn = get_activation_fn("batchtopk")
    near = torch.zeros(L, len(rows), dtype=torch.bool)      # [source layer, kept row]
    acts = {}
    with torch.no_grad():
        for l in range(L):
            pre = model.get_preactivations(x[l], l)
            acts[l] = fn(model, pre, l)
            kept = acts[l] != 0
            thr = pre[kept].float().min()                    # the layer's threshold value (a bf16 number)
            bits = thr.to(torch.bfloat16).view(torch.int16).to(torch.int32)
            lo = (bits - 1).to(torch.int16).view(torch.bfloat16).float()
            hi = (bits + 1).to(torch.int16).view(torch.bfloat16).float()
            sub = pre[rows].float()
            near[l] = ((sub >= lo) & (sub <= hi)).any(dim=1)
        recs = {t: model.decode({s_: acts[s_] for s_ in range(t + 1)}, t) for t in range(L)}
    torch.set_num_threads(1)
    flags = {str(t): near[:t + 1].any(dim=0).int().tolist() for t in (0, 6, 11)}
    return {"workload": "c1", "rows": rows, "layers_in_full": [0, 6, 11],
            "sumsq": [float((recs[l].double() ** 2).sum()) for l in range(L)],
            "nonzero": [int((acts[l] != 0).sum()) for l in range(L)],
            "rows_full": {str(l): lists(recs[l][rows]) for l in (0, 6, 11)},
            "rows_near_threshold": flags}


def sections():
    base = dict(num_features=16, num_layers=3, d_model=8)
    tied_affine = dict(base, activation_fn="relu", enable_feature_offset=True, enable_feature_scale=True)
    return {
        "forward": lambda: [
            forward_case("batchtopk-global", dict(base, activation_fn="batchtopk", batchtopk_k=3), 11),
            forward_case("tokentopk-global", dict(base, activation_fn="topk", topk_k=4), 12),
            forward_case("jumprelu", dict(base, activation_fn="jumprelu"), 13),
            forward_case("relu-per-target-affine-skip", dict(base, activation_fn="relu", decoder_tying="per_target",
                                                             enable_feature_offset=True, enable_feature_scale=True,
                                                             skip_connection=True), 14,
                         save_as="reference_checkpoint.pt"),
            forward_case("batchtopk-global-per-source", dict(base, activation_fn="batchtopk", batchtopk_k=3,
                                                             decoder_tying="per_source"), 15),
            forward_case("relu-untied-skip", dict(base, activation_fn="relu", skip_connection=True), 16),
            # bf16 on the CPU: sums run in another order than on the GPU, so these are held to the
            # rel-L2 tolerance of the bf16 path, not to equality
            forward_case("jumprelu-bf16", dict(num_features=32, num_layers=3, d_model=16, activation_fn="jumprelu",
                                               clt_dtype="bfloat16"), 17, tokens=16),
            forward_case("batchtopk-global-bf16", dict(num_features=32, num_layers=3, d_model=16,
                                                       activation_fn="batchtopk", batchtopk_k=4,
                                                       clt_dtype="bfloat16"), 18, tokens=16),
            # float16 likewise
            forward_case("jumprelu-f16", dict(num_features=32, num_layers=3, d_model=16, activation_fn="jumprelu",
                                              clt_dtype="float16"), 23, tokens=16),
            forward_case("batchtopk-global-f16", dict(num_features=32, num_layers=3, d_model=16,
                                                      activation_fn="batchtopk", batchtopk_k=4,
                                                      clt_dtype="float16"), 24, tokens=16),
        ],
        "per_layer": lambda: [
            per_layer_case("batchtopk", dict(num_features=32, num_layers=3, d_model=8, activation_fn="batchtopk",
                                             batchtopk_k=4), 71),
            per_layer_case("batchtopk-bf16", dict(num_features=32, num_layers=3, d_model=8, activation_fn="batchtopk",
                                                  batchtopk_k=4, clt_dtype="bfloat16"), 72),
            per_layer_case("tokentopk", dict(num_features=32, num_layers=3, d_model=8, activation_fn="topk",
                                             topk_k=5.0), 73),
            per_layer_case("batchtopk-f16", dict(num_features=32, num_layers=3, d_model=8, activation_fn="batchtopk",
                                                 batchtopk_k=4, clt_dtype="float16"), 74),
        ],
        "forward_irregular": lambda: irregular_cases(19),
        "config_json": config_json_cases,
        "checkpoint_migration": lambda: migration_case(61),
        "theta_estimation": lambda: [theta_case(dict(base, activation_fn="batchtopk", batchtopk_k=3), 21),
                                     theta_case(dict(base, activation_fn="topk", topk_k=4), 22)],
        "gradients": lambda: [
            gradient_case("batchtopk-global", dict(base, activation_fn="batchtopk", batchtopk_k=3), 31),
            gradient_case("jumprelu", dict(base, activation_fn="jumprelu"), 32),
            gradient_case("relu-per-source", dict(base, activation_fn="relu", decoder_tying="per_source"), 33),
            gradient_case("relu-per-target", dict(base, activation_fn="relu", decoder_tying="per_target"), 34),
        ],
        # the loss on de-normalised tensors (losses.py:70-86)
        "gradients_normalized": lambda: [
            gradient_case_normalized("mean-std", dict(base, activation_fn="relu"), 35, "mean_std"),
            gradient_case_normalized("sqrt-d-model", dict(base, activation_fn="batchtopk", batchtopk_k=3), 36, "sqrt_d_model"),
            gradient_case_normalized("mean-std-some-layers", dict(base, activation_fn="relu"), 44, "mean_std", stat_layers=(0, 2)),
        ],
        # the JumpReLU threshold gradient (activations.py:183-220) behind the per-target feature offset / scale
        "gradients_jumprelu_affine": lambda: [
            gradient_case("jumprelu-per-target-affine", dict(tied_affine, activation_fn="jumprelu", decoder_tying="per_target"), 45),
            gradient_case("jumprelu-per-source-scale", dict(base, activation_fn="jumprelu", decoder_tying="per_source",
                                                            enable_feature_scale=True), 46),
            gradient_case("jumprelu-per-target-offset-skip", dict(base, activation_fn="jumprelu", decoder_tying="per_target",
                                                                  enable_feature_offset=True, skip_connection=True), 47),
        ],
        # gradients through skip connections and the per-target feature offset / scale (decoder.py:228-338)
        "gradients_skip_affine": lambda: [
            gradient_case("untied-skip", dict(base, activation_fn="relu", skip_connection=True), 37),
            gradient_case("per-target-affine-skip", dict(tied_affine, decoder_tying="per_target", skip_connection=True), 38),
            gradient_case("per-source-affine", dict(tied_affine, decoder_tying="per_source"), 39),
            gradient_case("per-target-offset-only", dict(base, activation_fn="batchtopk", batchtopk_k=3, decoder_tying="per_target",
                                                         enable_feature_offset=True), 40),
        ],
        "global_select": lambda: [global_select_case(torch.float32, 51), global_select_case(torch.bfloat16, 52),
                                  global_select_case(torch.float16, 53)],
        "evaluator": lambda: evaluator_case(41),
        "compute_metrics": lambda: compute_metrics_case(42),
        "compute_metrics_subset": lambda: evaluator_subset_case(43),
        "c0_summary": c0_summary,
        "c1_summary": c1_summary,
    }


def main():
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_fixtures.json")
    only = [a.split("=", 1)[1].split(",") for a in sys.argv[1:] if a.startswith("--only=")]
    table = sections()
    if only:
        fixtures = json.load(open(out))
        names = only[0]
    else:
        fixtures = {"_about": "Produced by tests/golden/make_reference_fixtures.py from the reference's own code on the CPU "
                              "(fp32, tiny shapes, fixed seeds).  Data only."}
        names = list(table)
    for name in names:
        print("section", name, flush=True)
        fixtures[name] = table[name]()
    with open(out, "w") as f:
        json.dump(fixtures, f)
    print("wrote", out, os.path.getsize(out), "bytes")


if __name__ == "__main__":
    main()
