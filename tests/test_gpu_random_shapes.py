"""Seeded random shapes through the whole forward, every stage judged on its own: pre-activations against an fp64
product, the selection exactly against the oracle on the GPU's own pre-activations, the routes fused into the
encoder epilogue against the separate kernels bit for bit, and the reconstructions against fp64 dense products of
the model's own activations (the reference's formulation, clt/models/decoder.py:176-338).  The draws cover token
counts below, at and between whole encoder tiles, d_model with odd and even numbers of 128-byte stages and values
the matrix-core kernels do not take, all activations, selection modes, tyings and element types."""
import random

import pytest
import torch

import crosslayer_coding_amd as cca
from crosslayer_coding_amd import synth
from oracle import clt_oracle as orc

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 2e-5, torch.bfloat16: 1.2e-2, torch.float16: 2e-3}


def draw(rng, case):
    dtype = rng.choice(["float32", "bfloat16", "bfloat16", "float16"])
    fn = rng.choice(["batchtopk", "batchtopk", "jumprelu", "jumprelu", "relu", "topk"])
    mode = rng.choice(["per_layer", "per_layer", "global"]) if fn in ("batchtopk", "topk") else "per_layer"
    tying = rng.choice(["none", "none", "per_source", "per_target"])
    L = rng.randint(1, 4)
    d = rng.choice([64, 128, 192, 256, 320, 448, 640, 768, 72, 1600])
    F = rng.choice([256, 512, 768, 1024, 1280, 2048, 520, 136])
    T = rng.choice([rng.randint(1, 255), rng.randint(256, 1300), 256, 512, 1024, rng.randint(256, 700)])
    k = None
    if fn == "batchtopk":
        k = rng.choice([1, 3, 8, 20, 64, F // 2])
    if fn == "topk":
        k = rng.choice([1, 4, 16])
    return synth.Workload("rs%d" % case, 20 + case % 7, L, d, F, T, dtype, activation_fn=fn, k=k, topk_mode=mode,
                          decoder_tying=tying)


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_random_shapes_stage_by_stage(dev, seed):
    rng = random.Random(seed)
    for case in range(16):
        wl = draw(rng, case)
        tag = f"seed {seed} case {case}: {wl}"
        dt = getattr(torch, wl.dtype)
        L, T, d = wl.num_layers, wl.tokens, wl.d_model
        x = synth.make_inputs(wl, "cpu")
        sd = synth.make_state_dict(wl, "cpu", inputs=x)
        g = torch.Generator().manual_seed(77 + case)
        for key in list(sd):
            if key.endswith("bias_param") and "decoder" in key:
                sd[key] = (torch.randn(sd[key].shape, generator=g) * 0.1).to(sd[key].dtype)
        model = cca.CrossLayerTranscoder(wl.config(), None, dev)
        model.load_state_dict(sd)
        layers = list(range(L)) if rng.random() < 0.8 or L == 1 else sorted(rng.sample(range(L), L - 1))
        inputs = {l: x[l].to(dev) for l in layers}
        with torch.no_grad():
            model.fuse_encode_select = True
            r1, a1 = model(inputs), model.get_feature_activations(inputs)
            model.fuse_encode_select = False
            r2, a2 = model(inputs), model.get_feature_activations(inputs)
            pre, _ = model._encode_all_layers(inputs)
        # under a threshold activation the decode moves between the gather and dense products with the density seen
        # so far (always possible for decoders tied per target, at high densities for the others), so two calls
        # may differ in the last bits there
        route_may_move = wl.activation_fn in ("relu", "jumprelu")
        for l in layers:
            assert torch.equal(a1[l], a2[l]), tag
        for t in r1:
            assert route_may_move or torch.equal(r1[t], r2[t]), tag
        dd = lambda name: sd[name].to(dev).double()
        for l in layers:
            ref = x[l].to(dev).double() @ dd(f"encoder_module.encoders.{l}.weight").T + dd(f"encoder_module.encoders.{l}.bias_param")
            assert float((pre[l].double() - ref).norm() / ref.norm().clamp_min(1e-30)) <= TOL[dt], tag
        for l in layers:
            p = pre[l].cpu()
            want = None
            if wl.activation_fn == "batchtopk" and wl.topk_mode == "per_layer":
                want = orc.batchtopk_forward(p, float(wl.k), p)
            elif wl.activation_fn == "jumprelu":
                want = orc.jumprelu_forward(p, orc.theta_from_log(sd["theta_manager.log_threshold"][l], dt))
            elif wl.activation_fn == "relu":
                want = torch.relu(p)
            elif wl.activation_fn == "topk" and wl.topk_mode == "per_layer":
                want = orc.tokentopk_forward(p, float(wl.k), p)
            assert want is None or torch.equal(a1[l].cpu(), want), tag
        for t in r1:
            if wl.decoder_tying == "per_target":
                acc = sum(a1[s].double() for s in layers if s <= t) @ dd(f"decoder_module.decoders.{t}.weight").T \
                    + dd(f"decoder_module.decoders.{t}.bias_param")
            else:
                acc = torch.zeros(T, d, dtype=torch.float64, device=dev)
                for s in layers:
                    if s <= t:
                        nm = f"{s}->{t}" if wl.decoder_tying == "none" else f"{s}"
                        acc += a1[s].double() @ dd(f"decoder_module.decoders.{nm}.weight").T + dd(f"decoder_module.decoders.{nm}.bias_param")
            assert float((r1[t].double() - acc).norm() / acc.norm().clamp_min(1e-30)) <= TOL[dt], tag
        del model
