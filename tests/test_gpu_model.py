"""CrossLayerTranscoder (host mirror over the HIP kernels) against the CPU oracle's forward."""
import logging

import pytest
import torch

import crosslayer_coding_amd as cca
from crosslayer_coding_amd import _native as nat
from crosslayer_coding_amd import engine, synth
from oracle import clt_oracle as orc

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-5, torch.bfloat16: 1e-2}


def oracle_forward(wl, sd, x, **extra):
    dtype = getattr(torch, wl.dtype)
    L = wl.num_layers
    enc_w = [sd[f"encoder_module.encoders.{l}.weight"] for l in range(L)]
    enc_b = [sd[f"encoder_module.encoders.{l}.bias_param"] for l in range(L)]
    names = synth.decoder_names(wl)
    dec_w = {n: sd[f"decoder_module.decoders.{n}.weight"] for n in names}
    dec_b = {n: sd[f"decoder_module.decoders.{n}.bias_param"] for n in names}
    return orc.forward({l: x[l] for l in range(L)}, enc_w=enc_w, enc_b=enc_b, dec_w=dec_w, dec_b=dec_b,
                       activation_fn=wl.activation_fn, dtype=dtype, num_layers=L, d_model=wl.d_model,
                       num_features=wl.num_features, tying=wl.decoder_tying, k=wl.k, topk_mode=wl.topk_mode,
                       log_threshold=sd.get("theta_manager.log_threshold"), **extra)


def build(wl, dev, bias_noise=True):
    x = synth.make_inputs(wl, "cpu")
    sd = synth.make_state_dict(wl, "cpu", inputs=x)
    if bias_noise:
        g = torch.Generator().manual_seed(77)
        for k in list(sd):
            if k.endswith("bias_param") and "decoder" in k:
                sd[k] = (torch.randn(sd[k].shape, generator=g) * 0.1).to(sd[k].dtype)
    model = cca.CrossLayerTranscoder(wl.config(), None, dev)
    model.load_state_dict(sd)
    return model, sd, x


BASE = synth.Workload("tiny", 9, 3, 64, 256, 96, "float32", k=8)
CASES = [
    BASE,
    BASE.scaled("tiny-bf16", dtype="bfloat16"),
    BASE.scaled("tiny-global", topk_mode="global"),
    BASE.scaled("tiny-jump", activation_fn="jumprelu", k=None),
    BASE.scaled("tiny-jump-bf16", activation_fn="jumprelu", k=None, dtype="bfloat16"),
    BASE.scaled("tiny-relu", activation_fn="relu", k=None),
    BASE.scaled("tiny-per-target", decoder_tying="per_target", dtype="bfloat16"),
    BASE.scaled("tiny-per-source", decoder_tying="per_source"),
    BASE.scaled("tiny-topk", activation_fn="topk", k=6),
    BASE.scaled("tiny-topk-global", activation_fn="topk", k=6, topk_mode="global", dtype="bfloat16"),
    BASE.scaled("ref-shape", num_layers=2, d_model=8, num_features=16, tokens=30, k=3),   # the reference's own test shape
    BASE.scaled("mid", num_layers=4, d_model=768, num_features=2048, tokens=300, k=20, dtype="bfloat16"),
    # shapes that take the routes fused into the encoder epilogue (at least one 256 x 256 tile)
    BASE.scaled("fused-topk", num_layers=3, d_model=128, num_features=512, tokens=256, k=12),
    BASE.scaled("fused-topk-bf16", num_layers=3, d_model=256, num_features=1024, tokens=512, k=24, dtype="bfloat16"),
    # a short prompt on a model whose shapes take the matrix-core encoder: the batch is padded to one tile
    BASE.scaled("short-prompt-bf16", num_layers=3, d_model=256, num_features=1024, tokens=40, k=8, dtype="bfloat16"),
    BASE.scaled("short-prompt-jump", num_layers=3, d_model=256, num_features=1024, tokens=7, activation_fn="jumprelu", k=None),
    BASE.scaled("fused-jump", num_layers=3, d_model=128, num_features=512, tokens=256, activation_fn="jumprelu", k=None),
    BASE.scaled("fused-jump-bf16", num_layers=3, d_model=256, num_features=1024, tokens=512, activation_fn="jumprelu",
                k=None, dtype="bfloat16"),
]


@pytest.mark.parametrize("wl", CASES, ids=lambda w: w.name)
def test_forward_matches_oracle(dev, wl):
    dtype = getattr(torch, wl.dtype)
    model, sd, x = build(wl, dev)
    inputs = {l: x[l].to(dev) for l in range(wl.num_layers)}
    recs = model(inputs)
    ref_recs, ref_acts = oracle_forward(wl, sd, x)
    assert sorted(recs) == sorted(ref_recs)
    for t in recs:
        assert recs[t].shape == ref_recs[t].shape and recs[t].dtype == dtype
        err = orc.rel_l2(recs[t], ref_recs[t])
        assert err <= TOL[dtype], (t, err)
    acts = model.get_feature_activations(inputs)
    assert sorted(acts) == sorted(ref_acts)
    if dtype == torch.float32 and wl.topk_mode == "per_layer" or wl.activation_fn in ("relu",):
        pass
    for l in acts:
        assert acts[l].shape == ref_acts[l].shape
        assert acts[l].dtype == ref_acts[l].dtype
    # selection parity is judged on identical pre-activations: feed the oracle the GPU's own
    pre, _ = model._encode_all_layers(inputs)
    pre_cpu = {l: p.cpu() for l, p in pre.items()}
    if wl.activation_fn == "batchtopk" and wl.topk_mode == "per_layer":
        for l in acts:
            assert torch.equal(acts[l].cpu(), orc.batchtopk_forward(pre_cpu[l], float(wl.k), pre_cpu[l]))
    elif wl.activation_fn == "jumprelu":
        lt = sd["theta_manager.log_threshold"]
        for l in acts:
            assert torch.equal(acts[l].cpu(), orc.jumprelu_forward(pre_cpu[l], orc.theta_from_log(lt[l], dtype)))
    elif wl.activation_fn == "relu":
        for l in acts:
            assert torch.equal(acts[l].cpu(), torch.relu(pre_cpu[l]))
    elif wl.activation_fn == "topk" and wl.topk_mode == "per_layer":
        for l in acts:
            assert torch.equal(acts[l].cpu(), orc.tokentopk_forward(pre_cpu[l], float(wl.k), pre_cpu[l]))
    for l in pre:
        assert orc.rel_l2(pre[l], orc.encoder_preactivations(x[l], sd[f"encoder_module.encoders.{l}.weight"],
                                                              sd[f"encoder_module.encoders.{l}.bias_param"])) <= TOL[dtype]


HALF_CASES = [
    BASE.scaled("half-topk", dtype="float16"),
    BASE.scaled("half-global", dtype="float16", topk_mode="global"),
    BASE.scaled("half-jump", dtype="float16", activation_fn="jumprelu", k=None),
    BASE.scaled("half-per-target", dtype="float16", decoder_tying="per_target"),
    BASE.scaled("half-fused-shape", dtype="float16", num_layers=3, d_model=128, num_features=512, tokens=256, k=12),
    # large-batch schedules: quarter rows (d = 768), line parts (d = 640), the dense per-target route, fused thresholds
    BASE.scaled("half-quarter", dtype="float16", num_layers=4, d_model=768, num_features=1024, tokens=2304, k=16),
    BASE.scaled("half-line", dtype="float16", num_layers=4, d_model=640, num_features=1024, tokens=2304, k=16,
                decoder_tying="per_source"),
    BASE.scaled("half-dense-route", dtype="float16", num_layers=3, d_model=256, num_features=1024, tokens=512, k=24,
                decoder_tying="per_target"),
    BASE.scaled("half-fused-jump", dtype="float16", num_layers=3, d_model=256, num_features=1024, tokens=512,
                activation_fn="jumprelu", k=None),
]


@pytest.mark.parametrize("wl", HALF_CASES, ids=lambda w: w.name)
def test_float16_model_forward_matches_oracle(dev, wl):
    # float16 parameters and outputs on the float16 kernels (fp32 accumulation, one rounding per product, like
    # bfloat16); the oracle runs the reference's algorithm in float16 on the CPU
    model, sd, x = build(wl, dev)
    assert model.dtype == torch.float16 and all(v.dtype == torch.float16 for v in model.state_dict().values()
                                                if v.is_floating_point())
    inputs = {l: x[l].to(dev) for l in range(wl.num_layers)}
    recs = model(inputs)
    ref_recs, ref_acts = oracle_forward(wl, sd, x)
    for t in recs:
        assert recs[t].dtype == torch.float16 and recs[t].shape == ref_recs[t].shape
        err = orc.rel_l2(recs[t], ref_recs[t])
        assert err <= 5e-3, (t, err)
    acts = model.get_feature_activations(inputs)
    pre_cpu = {l: model.get_preactivations(inputs[l], l).cpu() for l in range(wl.num_layers)}
    for l in acts:
        # JumpReLU's `(input >= threshold).float() * input` promotes to float32 (activations.py:177-180)
        assert acts[l].dtype == (torch.float32 if wl.activation_fn == "jumprelu" else torch.float16)
        assert pre_cpu[l].dtype == torch.float16
        # pre-activations: the float32 sum rounded once to float16
        want_pre = orc.encoder_preactivations(x[l], sd[f"encoder_module.encoders.{l}.weight"],
                                              sd[f"encoder_module.encoders.{l}.bias_param"])
        assert orc.rel_l2(pre_cpu[l], want_pre) <= 2e-3
        if wl.activation_fn == "batchtopk" and wl.topk_mode == "per_layer":
            assert torch.equal(acts[l].cpu(), orc.batchtopk_forward(pre_cpu[l], float(wl.k), pre_cpu[l]))
        elif wl.activation_fn == "jumprelu":
            lt = sd["theta_manager.log_threshold"]
            assert torch.equal(acts[l].cpu(), orc.jumprelu_forward(pre_cpu[l], orc.theta_from_log(lt[l], torch.float16)))
    norms = model.get_decoder_norms()
    assert norms.dtype == torch.float16 and bool(torch.isfinite(norms).all())
    # parameters changed in place are picked up by the next forward
    with torch.no_grad():
        model.decoder_module._ordered()[0].bias_param.add_(1.0)
    recs2 = model(inputs)
    assert not torch.equal(recs2[0], recs[0])
    # module.half() on a float32 model takes the same route
    wl32 = wl.scaled(wl.name + "-32", dtype="float32")
    m32, _, _ = build(wl32, dev)
    m32.half()
    out = m32(inputs)
    assert m32.dtype == torch.float16 and all(v.dtype == torch.float16 for v in out.values())
    # what is not built for float16 says so
    with pytest.raises(NotImplementedError):
        model.loss_and_gradients(inputs, inputs)


@pytest.mark.parametrize("tokens", [512, 600])
@pytest.mark.parametrize("fn", ["batchtopk", "jumprelu"])
def test_fused_routes_equal_separate_kernels_in_the_model(dev, fn, tokens):
    # same model, same inputs: with and without the encoder-epilogue routes, all layers and a subset; a whole
    # number of encoder token tiles, and a batch whose last tile is partial (with a d_model of five 128-byte stages)
    wl = BASE.scaled("f", num_layers=3, d_model=256 if tokens == 512 else 320, num_features=1024, tokens=tokens, k=24 if fn == "batchtopk" else None,
                     activation_fn=fn, dtype="bfloat16")
    model, sd, x = build(wl, dev)
    for layers in ([0, 1, 2], [0, 2]):
        inputs = {l: x[l].to(dev) for l in layers}
        model.fuse_encode_select = True
        if fn == "batchtopk":
            assert engine.encode_collect_supported(*model.encoder_module.prepare_slab(inputs)[1:], int(wl.k))
        a1 = model.get_feature_activations(inputs)
        r1 = model(inputs)
        model.fuse_encode_select = False
        a2 = model.get_feature_activations(inputs)
        r2 = model(inputs)
        assert sorted(a1) == sorted(a2) == layers
        for l in layers:
            assert torch.equal(a1[l], a2[l])
            assert torch.equal(r1[l], r2[l])


def test_decode_api_matches_forward(dev):
    wl = BASE
    model, sd, x = build(wl, dev)
    inputs = {l: x[l].to(dev) for l in range(wl.num_layers)}
    acts = model.get_feature_activations(inputs)
    recs = model(inputs)
    for t in range(wl.num_layers):
        rel = {s: a for s, a in acts.items() if s <= t}
        out = model.decode(rel, t)
        assert orc.rel_l2(out, recs[t]) <= 1e-6
    # additivity over sources (reference tests/unit/models/test_decoder.py:62-81)
    zero_bias = {k: torch.zeros_like(v) for k, v in sd.items() if k.endswith("bias_param") and "decoder" in k}
    model.load_state_dict({**sd, **zero_bias})
    full = model.decode(acts, 2)
    parts = sum(model.decode({s: acts[s]}, 2) for s in range(3))
    assert orc.rel_l2(parts, full) <= 1e-5


def test_encode_api_and_fallbacks(dev, caplog):
    wl = BASE.scaled("j", activation_fn="jumprelu", k=None)
    model, sd, x = build(wl, dev)
    out = model.encode(x[1].to(dev), 1)
    pre = model.get_preactivations(x[1].to(dev), 1).cpu()
    assert out.dtype == torch.float32
    assert torch.equal(out.cpu(), orc.jumprelu_forward(pre, orc.theta_from_log(sd["theta_manager.log_threshold"][1], torch.float32)))
    # 3-D input is flattened (reference tests/unit/models/test_encoder.py:50-73)
    x3 = x[0][:90].view(3, 30, wl.d_model).to(dev)
    assert model.get_preactivations(x3, 0).shape == (90, wl.num_features)
    # wrong d_model -> zeros + warning (test_encoder.py:89-103)
    with caplog.at_level(logging.WARNING):
        bad = model.get_preactivations(torch.randn(5, wl.d_model + 1, device=dev), 0)
    assert bad.shape == (5, wl.num_features) and float(bad.abs().sum()) == 0
    assert "Input d_model" in caplog.text
    caplog.clear()
    # out-of-range layer -> zeros + error (test_encoder.py:105-117)
    with caplog.at_level(logging.ERROR):
        bad = model.get_preactivations(x[0].to(dev), 99)
    assert bad.shape == (wl.tokens, wl.num_features) and float(bad.abs().sum()) == 0
    assert "Invalid layer index" in caplog.text
    # 1-D input (test_encoder.py:145-162)
    bad = model.get_preactivations(torch.randn(wl.d_model, device=dev), 0)
    assert bad.shape == (wl.d_model, wl.num_features)
    # empty activation dict (test_decoder.py:83-92)
    assert model.decode({}, 0).shape == (0, wl.d_model)


def test_forward_subset_of_layers_and_bad_layer(dev):
    wl = BASE
    model, sd, x = build(wl, dev)
    inputs = {0: x[0].to(dev), 2: x[2].to(dev)}
    recs = model(inputs)
    ref, _ = oracle_forward(wl, sd, {0: x[0], 2: x[2]}) if False else (None, None)
    assert sorted(recs) == [0, 2]
    L = wl.num_layers
    enc_w = [sd[f"encoder_module.encoders.{l}.weight"] for l in range(L)]
    enc_b = [sd[f"encoder_module.encoders.{l}.bias_param"] for l in range(L)]
    names = synth.decoder_names(wl)
    ref, _ = orc.forward({0: x[0], 2: x[2]}, enc_w=enc_w, enc_b=enc_b,
                         dec_w={n: sd[f"decoder_module.decoders.{n}.weight"] for n in names},
                         dec_b={n: sd[f"decoder_module.decoders.{n}.bias_param"] for n in names},
                         activation_fn="batchtopk", dtype=torch.float32, num_layers=L, d_model=wl.d_model,
                         num_features=wl.num_features, k=wl.k, topk_mode="per_layer")
    for t in recs:
        assert orc.rel_l2(recs[t], ref[t]) <= 1e-5


def test_state_dict_round_trip_and_tied_migration(dev, tmp_path):
    from safetensors.torch import load_file, save_file

    wl = BASE.scaled("s", num_layers=2, d_model=8, num_features=16, tokens=10, k=3)
    model, sd, x = build(wl, dev)
    path = str(tmp_path / "clt.safetensors")
    save_file({k: v.contiguous() for k, v in model.state_dict().items()}, path)
    loaded = load_file(path)
    assert set(loaded) == set(sd)
    for k in sd:
        assert loaded[k].shape == sd[k].shape and torch.equal(loaded[k], sd[k])
    m2 = cca.CrossLayerTranscoder(wl.config(), None, dev)
    m2.load_state_dict(loaded)
    inputs = {l: x[l].to(dev) for l in range(2)}
    a, b = model(inputs), m2(inputs)
    assert all(torch.equal(a[t], b[t]) for t in a)
    # untied checkpoint into a per_source model keeps the diagonal decoders
    tied_cfg = wl.scaled("t", decoder_tying="per_source").config()
    m3 = cca.CrossLayerTranscoder(tied_cfg, None, dev)
    m3.load_state_dict(loaded, strict=False)
    assert torch.equal(m3.decoder_module.decoders[1].weight.cpu(), sd["decoder_module.decoders.1->1.weight"])


def test_model_to_device_keeps_results(dev):
    wl = BASE.scaled("m", tokens=40)
    x = synth.make_inputs(wl, "cpu")
    sd = synth.make_state_dict(wl, "cpu")
    model = cca.CrossLayerTranscoder(wl.config(), None, torch.device("cpu"))
    model.load_state_dict(sd)
    model = model.to(dev)
    recs = model({l: x[l].to(dev) for l in range(wl.num_layers)})
    ref, _ = oracle_forward(wl, sd, x)
    for t in recs:
        assert orc.rel_l2(recs[t], ref[t]) <= 1e-5


@pytest.mark.parametrize("name", ["fused-topk-bf16", "fused-jump-bf16", "tiny-jump", "tiny-relu", "tiny-global", "tiny-per-target"])
def test_forward_reads_nothing_back_from_the_device(dev, name):
    # The forward is a sequence of launches on the current stream - from the first one on.  The survivor count
    # of a threshold activation depends on the data: its arrays are sized for any batch of the shape.
    wl = next(c for c in CASES if c.name == name)
    model, sd, x = build(wl, dev)
    inputs = {l: x[l].to(dev) for l in range(wl.num_layers)}
    other = {l: (1.05 * v).to(v.dtype) for l, v in inputs.items()}                 # other data, same shape
    model.decoder_module.packed()                      # the one-off repack of the decoders is not the forward
    torch.cuda.synchronize()
    torch.cuda.set_sync_debug_mode("error")
    try:
        with torch.no_grad():        # inference: with gradients enabled the forward keeps its survivor list for the backward
            first = model(inputs)
            second = model(inputs)
            third = model(other)
    finally:
        torch.cuda.set_sync_debug_mode("default")
    torch.cuda.synchronize()
    for t in first:
        assert torch.equal(first[t], second[t])
        assert torch.isfinite(third[t]).all()
    if wl.activation_fn in ("jumprelu", "relu"):
        model(inputs)                                   # polls the totals of the forwards above
        assert model._thr_last_total is not None and not model._thr_pending[:-1]
        # with a budget that the arrays of the shape exceed, every forward reads the total back: same result
        model.threshold_list_budget_bytes = 1024
        exact = model(inputs)
        for t in first:
            assert torch.equal(first[t], exact[t])


def dense_compare_forward(model, inputs, L):
    """The reference's formulation on the device: dense pre-activations, compare, decode of the dense result."""
    pre = {l: model.get_preactivations(inputs[l], l) for l in range(L)}
    theta = model.theta_manager.thresholds(model.dtype)
    acts = {l: torch.where(pre[l] >= theta[l], pre[l], torch.zeros_like(pre[l])) for l in range(L)}
    return acts, {t: model.decoder_module.decode({l: acts[l] for l in range(t + 1)}, t) for t in range(L)}


def test_threshold_forward_is_exact_when_the_survivors_outgrow_the_pool(dev):
    # A batch with many times the active features of any seen before (clt.py:271-277, theta.py:70-79: exact
    # for any batch).  The fused route's candidate pool, sized from the density seen so far, overflows; the
    # device itself redoes the batch on the dense route.  The forward reads nothing back and is exact.
    wl = next(c for c in CASES if c.name == "fused-jump-bf16")
    model, sd, x = build(wl, dev)
    L = wl.num_layers
    inputs = {l: x[l].to(dev) for l in range(L)}
    want_small = {t: v.clone() for t, v in model(inputs).items()}
    model(inputs)
    torch.cuda.synchronize()
    model(inputs)                                                       # the pool now follows the density seen
    small_total = model._thr_last_total
    ppm = model._density_ppm
    big = {l: (40.0 * v).to(v.dtype) for l, v in inputs.items()}        # scales every pre-activation: far more survivors
    acts_ref, rec_ref = dense_compare_forward(model, big, L)
    torch.cuda.synchronize()
    torch.cuda.set_sync_debug_mode("error")
    try:
        res = model.forward_with_survivors(big)
    finally:
        torch.cuda.set_sync_debug_mode("default")
    assert res is not None
    overflowed, surv = res
    torch.cuda.synchronize()
    assert model._density_ppm == ppm                                    # the pool was the small one
    total = surv.nnz
    assert total > 8 * small_total
    assert int(surv.status.item()) == 0
    dense = engine.densify(surv)
    for l in range(L):
        assert torch.equal(dense[l], acts_ref[l])                       # the survivor set and values, bit for bit
    for t in range(L):
        assert orc.rel_l2(overflowed[t].float().cpu(), rec_ref[t].float().cpu()) <= 1e-2
    # the same batch again: the pool has grown, the fused route holds it, the result is the same list
    again, surv2 = model.forward_with_survivors(big)
    torch.cuda.synchronize()
    assert model._density_ppm > ppm
    assert torch.equal(surv2.row_ptr, surv.row_ptr)
    assert torch.equal(surv2.col[:total], surv.col[:total])
    assert torch.equal(surv2.val[:total].view(torch.int16), surv.val[:total].view(torch.int16))
    for t in range(L):
        assert torch.equal(again[t], overflowed[t])
    acts = model.get_feature_activations(big)
    for l in range(L):
        assert torch.equal(acts[l].to(acts_ref[l].dtype), acts_ref[l])
    back = model(inputs)
    for t in range(L):
        assert torch.equal(back[t], want_small[t])


def test_threshold_batch_beyond_any_list_is_poisoned_not_returned(dev):
    # clt_survivors_fit / clt_poison_if: a list that cannot be represented must not decode as "nothing fired".
    # Forced here through a tiny capacity on a real count; the model uses the largest list of the shape.
    g = torch.Generator().manual_seed(3)
    pre = torch.randn(2, 64, 256, generator=g).to(dev)
    lib = nat.load()
    row_ptr = torch.empty(2 * 64 + 1, dtype=torch.int32, device=dev)
    wbuf = torch.empty(2 * 64 * 4, dtype=torch.uint8, device=dev)
    s = torch.cuda.current_stream().cuda_stream
    nat.check(lib.clt_threshold_count(pre.data_ptr(), 64, 256, 2, 64 * 256, None, nat.PRED_GT_ZERO, nat.CLT_F32,
                                      row_ptr.data_ptr(), wbuf.data_ptr(), wbuf.numel(), s), "count")
    total = int(row_ptr[-1].item())
    status = engine._fit(row_ptr, total - 1)
    out = torch.ones(5, 7, device=dev, dtype=torch.bfloat16)
    engine.poison_if(out, status)
    assert int(status.item()) == 1 and int(row_ptr.abs().sum()) == 0 and torch.isnan(out).all()
    surv = engine.SurvivorList(row_ptr, torch.empty(1, dtype=torch.int32, device=dev), torch.empty(1, device=dev), 64, 256, 2,
                               torch.float32, status)
    with pytest.raises(nat.CLTNativeError):
        surv.trimmed()
    # a list that fits: flag clear, nothing touched
    nat.check(lib.clt_threshold_count(pre.data_ptr(), 64, 256, 2, 64 * 256, None, nat.PRED_GT_ZERO, nat.CLT_F32,
                                      row_ptr.data_ptr(), wbuf.data_ptr(), wbuf.numel(), s), "count")
    status = engine._fit(row_ptr, total)
    out = torch.ones(5, 7, device=dev, dtype=torch.bfloat16)
    engine.poison_if(out, status)
    assert int(status.item()) == 0 and int(row_ptr[-1].item()) == total and bool((out == 1).all())


def test_profiler_hook_receives_the_reference_timer_names(dev):
    # the `profiler=` argument of the constructor (clt.py:30-36): timers "batchtopk_activation" (clt.py:254-257)
    # and, inside the global helper, "batchtopk_compute_mask" (activations.py:335-341)
    class Timer:
        def __init__(self):
            self.elapsed = 0.0

        def __enter__(self):
            return self

        def __exit__(self, *exc):
            self.elapsed = 1.0
            return False

    class Profiler:
        def __init__(self):
            self.records = []

        def timer(self, name):
            return Timer()

        def record(self, name, elapsed):
            self.records.append(name)

    wl = next(c for c in CASES if c.name == "tiny-global")
    x = synth.make_inputs(wl, "cpu")
    sd = synth.make_state_dict(wl, "cpu", inputs=x)
    prof = Profiler()
    model = cca.CrossLayerTranscoder(wl.config(), None, dev, profiler=prof)
    model.load_state_dict(sd)
    model({l: x[l].to(dev) for l in range(wl.num_layers)})
    assert "batchtopk_activation" in prof.records and "batchtopk_compute_mask" in prof.records


@pytest.mark.parametrize("kw", [dict(), dict(activation_fn="jumprelu", k=None), dict(topk_mode="global"),
                                dict(decoder_tying="per_target")], ids=["topk", "jumprelu", "global", "per-target"])
def test_inference_forward_replays_from_a_graph(dev, kw):
    # The inference forward is launches on the current stream and nothing else (no allocation inside the library,
    # no memset, nothing read back), so it can be captured once and replayed.  Every replay - on new inputs, with
    # eager forwards and synchronisations in between - must equal the eager result bit for bit.
    wl = BASE.scaled("graph", dtype="bfloat16", num_layers=3, d_model=256, num_features=1024, tokens=512,
                     **({"k": 16} if "k" not in kw else {}), **kw)
    model, sd, x = build(wl, dev)
    model.eval()
    inputs = {l: x[l].to(dev) for l in range(wl.num_layers)}
    static_in = {l: v.clone() for l, v in inputs.items()}
    with torch.no_grad():
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                model(static_in)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            out = model(static_in)
        for rep in range(4):
            new = {l: (v * (1.0 + 0.1 * rep)).to(v.dtype) for l, v in inputs.items()}
            for l in new:
                static_in[l].copy_(new[l])
            graph.replay()
            torch.cuda.synchronize()
            got = {l: o.clone() for l, o in out.items()}
            want = model(new)
            torch.cuda.synchronize()
            for l in want:
                assert torch.equal(got[l], want[l]), (rep, l)


@pytest.mark.parametrize("tying,fn", [("per_target", "batchtopk"), ("per_source", "jumprelu"), ("none", "batchtopk"),
                                      ("per_source", "topk-global")])
def test_more_than_64_layers_run_on_the_dense_formulations(dev, tying, fn):
    """The gather and survivor-list kernels take 64 layers; a deeper model decodes and trains through the dense
    products at any density.  Forward against the oracle; loss and gradients against autograd through the oracle."""
    L = 66
    mode = "global" if fn == "topk-global" else "per_layer"
    fn = fn.split("-")[0]
    wl = BASE.scaled("deep", num_layers=L, d_model=32, num_features=64, tokens=20, k=4 if fn != "jumprelu" else None,
                     activation_fn=fn, decoder_tying=tying, topk_mode=mode)
    model, sd, x = build(wl, dev)
    inputs = {l: x[l].to(dev) for l in range(L)}
    with torch.no_grad():
        recs = model(inputs)
        recs = model(inputs)        # (a threshold model knows its density from the second forward on)
    assert model.decoder_module.last_route["dense_targets"] == (0, L)
    ref_recs, _ = oracle_forward(wl, sd, x)
    for t in (0, 1, 31, 64, 65):
        assert orc.rel_l2(recs[t], ref_recs[t]) <= 1e-5, t
    g = torch.Generator().manual_seed(6)
    targets = {l: torch.randn(wl.tokens, wl.d_model, generator=g) for l in range(L)}
    loss, grads = model.loss_and_gradients(inputs, {l: t.to(dev) for l, t in targets.items()})
    names = synth.decoder_names(wl)
    theta = log_theta = masks = None
    if fn == "jumprelu":
        theta = torch.exp(sd["theta_manager.log_threshold"].float())
        log_theta = sd["theta_manager.log_threshold"]
    if fn == "topk":
        masks = {l: (a != 0).cpu() for l, a in model.get_feature_activations(inputs).items()}
    ref_loss, ref = orc.mse_loss_and_gradients(
        {l: x[l] for l in range(L)}, targets,
        enc_w=[sd[f"encoder_module.encoders.{l}.weight"] for l in range(L)],
        enc_b=[sd[f"encoder_module.encoders.{l}.bias_param"] for l in range(L)],
        dec_w={n: sd[f"decoder_module.decoders.{n}.weight"] for n in names},
        dec_b={n: sd[f"decoder_module.decoders.{n}.bias_param"] for n in names},
        activation_fn=fn, num_layers=L, k=wl.k, theta=theta, masks=masks, tying=tying, log_threshold=log_theta,
        model_dtype=torch.float32)
    assert abs(float(loss) - float(ref_loss)) <= 1e-4 * abs(float(ref_loss))
    for name in (f"encoder_module.encoders.0.weight", f"encoder_module.encoders.{L - 1}.bias_param",
                 f"decoder_module.decoders.{names[0]}.weight", f"decoder_module.decoders.{names[-1]}.weight",
                 f"decoder_module.decoders.{names[len(names) // 2]}.bias_param"):
        assert orc.rel_l2(grads[name].float().cpu(), ref[name]) <= (1e-3 if name.endswith("log_threshold") else 2e-5), name
    opt = cca.CLTAdam(model, lr=1e-3)
    before = model.state_dict()["encoder_module.encoders.3.weight"].clone()
    model.training_step(inputs, {l: t.to(dev) for l, t in targets.items()}, opt)
    assert not torch.equal(model.state_dict()["encoder_module.encoders.3.weight"], before)
