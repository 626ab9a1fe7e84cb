"""Gradients of the MSE reconstruction loss from the survivor list (C ABI kernels) against torch
autograd through the oracle's dense forward.  fp32: rel-L2 <= 1e-5; bf16: <= 1e-2 (the kernels read
bf16 weights / inputs and accumulate in fp32; the oracle runs in fp32 on the same bf16 values)."""
import pytest
import torch

from crosslayer_coding_amd import engine, synth
from oracle import clt_oracle as orc

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-5, torch.bfloat16: 1e-2}
BASE = synth.Workload("bw", 9, 3, 64, 256, 96, "float32", k=8)


def build(wl, dev):
    import crosslayer_coding_amd as cca
    x = synth.make_inputs(wl, "cpu")
    sd = synth.make_state_dict(wl, "cpu", inputs=x)
    g = torch.Generator().manual_seed(5)
    for k in list(sd):
        if k.endswith("bias_param"):
            sd[k] = (torch.randn(sd[k].shape, generator=g) * 0.05).to(sd[k].dtype)
    model = cca.CrossLayerTranscoder(wl.config(), None, dev)
    model.load_state_dict(sd)
    tg = torch.Generator().manual_seed(6)
    targets = {l: torch.randn(wl.tokens, wl.d_model, generator=tg).to(x.dtype) for l in range(wl.num_layers)}
    return model, sd, x, targets


@pytest.mark.parametrize("wl", [
    BASE,
    BASE.scaled("bw-bf16", dtype="bfloat16"),
    BASE.scaled("bw-wide", num_layers=2, d_model=768, num_features=512, tokens=64, k=20),
    BASE.scaled("bw-jump", activation_fn="jumprelu", k=None),
    BASE.scaled("bw-fused", num_layers=2, d_model=128, num_features=512, tokens=256, k=10, dtype="bfloat16"),
], ids=lambda w: w.name)
def test_loss_and_gradients_match_autograd(dev, wl):
    dtype = getattr(torch, wl.dtype)
    model, sd, x, targets = build(wl, dev)
    L = wl.num_layers
    inputs = {l: x[l].to(dev) for l in range(L)}
    loss, grads = model.loss_and_gradients(inputs, {l: t.to(dev) for l, t in targets.items()})
    # in bf16 the oracle's fp32 pre-activations would select a slightly different set at the
    # threshold; the comparison here is about gradients, so it gets the model's gate
    masks = None
    if dtype == torch.bfloat16:
        masks = {l: (a != 0).cpu() for l, a in model.get_feature_activations(inputs).items()}
    names = synth.decoder_names(wl)
    theta = None
    if wl.activation_fn == "jumprelu":
        theta = torch.exp(sd["theta_manager.log_threshold"].float()).to(dtype)
    ref_loss, ref = orc.mse_loss_and_gradients(
        {l: x[l] for l in range(L)}, targets,
        enc_w=[sd[f"encoder_module.encoders.{l}.weight"] for l in range(L)],
        enc_b=[sd[f"encoder_module.encoders.{l}.bias_param"] for l in range(L)],
        dec_w={n: sd[f"decoder_module.decoders.{n}.weight"] for n in names},
        dec_b={n: sd[f"decoder_module.decoders.{n}.bias_param"] for n in names},
        activation_fn=wl.activation_fn, num_layers=L, k=wl.k, theta=theta, masks=masks)
    tol = TOL[dtype]
    assert abs(float(loss) - float(ref_loss)) <= max(tol, 1e-6) * abs(float(ref_loss)) * 10
    for name, gref in ref.items():
        got = grads[name]
        assert got is not None and tuple(got.shape) == tuple(gref.shape), name
        err = orc.rel_l2(got.float().cpu(), gref)
        assert err <= tol * (5 if dtype == torch.bfloat16 else 1), (name, err)


def test_feature_lists_are_a_permutation_grouped_by_feature(dev):
    g = torch.Generator().manual_seed(2)
    L, T, F = 2, 300, 128
    pre = torch.randn(L, T, F, generator=g).to(dev)
    surv = engine.batchtopk_select(pre, 9, False)
    ptr, tok, src = engine.feature_lists(surv)
    ptr, tok, src = ptr.cpu().long(), tok.cpu().long(), src.cpu().long()
    assert ptr[0] == 0 and ptr[-1] == surv.nnz and bool((ptr[1:] >= ptr[:-1]).all())
    assert torch.equal(torch.sort(src).values, torch.arange(surv.nnz))
    rows = engine.survivor_rows(surv).cpu().long()
    col = surv.col.cpu().long()
    for q in range(L * F):
        b, e = int(ptr[q]), int(ptr[q + 1])
        if e > b:
            l, f = divmod(q, F)
            assert bool((col[src[b:e]] == f).all()) and bool((rows[src[b:e]] // T == l).all())
            assert torch.equal(rows[src[b:e]] % T, tok[b:e])
            if e - b <= 64:
                assert bool((tok[b + 1:e] > tok[b:e - 1]).all())
