"""The other benchmark configurations at their own sizes: Pythia-410m-shaped JumpReLU (24 layers,
d_model 1024, 32768 features, 300 untied decoders), Pythia-1B-shaped per-target tying (16 layers,
d_model 2048, 16384 features, 8192 tokens) and the training step at the GPT-2-small x32 shape in bf16
with fp32 Adam moments.

A CPU forward at these sizes takes many minutes, so results are checked through properties that do not
depend on size and against independent dense formulations with torch matmuls on the GPU (fp32), the way
the reference itself computes them.
"""
import pytest
import torch

import crosslayer_coding_amd as cca
from crosslayer_coding_amd import _native as nat
from crosslayer_coding_amd import engine, synth
from oracle import clt_oracle as orc

pytestmark = pytest.mark.gpu


def _free():
    import gc
    gc.collect()
    torch.cuda.empty_cache()


# ---- C2: JumpReLU, 300 untied decoders ----------------------------------------------------------------
def test_c2_jumprelu_forward_at_full_size(dev):
    wl = synth.WORKLOADS["c2"]
    L, T, F, d = wl.num_layers, wl.tokens, wl.num_features, wl.d_model
    model, inputs, _ = synth.build_model(wl, dev)
    model.eval()
    dec = model.decoder_module
    # the packed decoders: 300 * 32768 * 1024 = 1.0e10 elements, past 32-bit offsets
    n_elems = nat.load().clt_decoder_slab_elems(d, F, L, nat.TYING["none"], nat.CLT_BF16)
    pitch = engine.decoder_pitch(d, torch.bfloat16)
    assert pitch == d + 64                              # 16 cache lines per row: padded to 17
    assert n_elems == 300 * F * pitch > 2 ** 32 and dec.packed().numel() == n_elems
    assert engine.decode_route(T, d, F, L, "none", torch.bfloat16) == nat.ROUTE_LINE

    # thresholds in the encoder epilogue == dense pre-activations + threshold pass, bit for bit
    _, x, w, b = model.encoder_module.prepare_slab(inputs)
    theta = model.theta_manager.thresholds(model.dtype)
    ws = model._workspace()
    fused = engine.encode_threshold(x, w, b, theta, ws, density_ppm=20000)
    assert fused is not None, "the encoder-epilogue route must take this shape"
    pre = engine.encode(x, w, b)
    ref = engine.threshold_select(pre, theta, nat.PRED_GE_THETA)
    torch.cuda.synchronize()
    assert torch.equal(fused.row_ptr, ref.row_ptr)
    assert torch.equal(fused.col, ref.col)
    assert torch.equal(fused.val.view(torch.int16), ref.val.view(torch.int16))
    nnz = fused.nnz
    density = nnz / (L * T * F)
    print(f"c2: {nnz} survivors, density {100 * density:.3f} % ({nnz / (L * T):.1f} per token and layer)")
    assert 0.003 <= density <= 0.012                    # calibrated for about 0.6 %
    # the survivors are exactly the elements with x >= theta (dense torch compare, layer by layer)
    rp = fused.row_ptr.long()
    for l in (0, 11, L - 1):
        keep = pre[l] >= theta[l]
        assert int(keep.sum()) == int(rp[(l + 1) * T] - rp[l * T])
        rows, cols = keep.nonzero(as_tuple=True)
        seg = slice(int(rp[l * T]), int(rp[(l + 1) * T]))
        assert torch.equal(fused.col[seg].long(), cols)
        assert torch.equal(fused.val[seg].view(torch.int16), pre[l][rows, cols].view(torch.int16))
    del pre, ref, keep, rows, cols
    _free()

    # the model's forward takes the same route (no dense pre-activations) and gives the same list
    res = model._survivors(inputs)
    assert res is not None
    _, _, surv = res
    # (the model's arrays are sized for any batch of the shape: 2^31 - 1 entries here, nothing is read back)
    assert surv.status is not None and surv.capacity == 2 ** 31 - 1
    assert torch.equal(surv.row_ptr, fused.row_ptr) and torch.equal(surv.col[:nnz], fused.col)
    assert torch.equal(surv.val[:nnz].view(torch.int16), fused.val.view(torch.int16))
    surv = fused
    # nothing is read back from the device in an inference forward (with gradients enabled the forward keeps an
    # exact copy of the survivor list for its backward, which takes one read-back)
    torch.cuda.synchronize()
    torch.cuda.set_sync_debug_mode("error")
    try:
        with torch.no_grad():
            recs = model(inputs)
    finally:
        torch.cuda.set_sync_debug_mode("default")
    dense = engine.densify(surv)                         # [L, T, F] in the model dtype
    for t in (0, 12, L - 1):
        want = torch.zeros(T, d, dtype=torch.float32, device=dev)
        for s in range(t + 1):
            lin = dec.decoders[f"{s}->{t}"]
            want += dense[s].float() @ lin.weight.float().t() + lin.bias_param.float()
        err = orc.rel_l2(recs[t].float().cpu(), want.cpu())
        assert err <= 1e-2, (t, err)
    del dense, want, recs
    _free()

    # the largest offset: one survivor at (last layer, token 0, last feature) must read the last row of
    # the last matrix of the slab, on the sliced schedule and on the single-pass one
    row_ptr = torch.zeros(L * T + 1, dtype=torch.int32, device=dev)
    row_ptr[(L - 1) * T + 1:] = 1
    one = engine.SurvivorList(row_ptr, torch.tensor([F - 1], dtype=torch.int32, device=dev),
                              torch.tensor([1.0], dtype=torch.bfloat16, device=dev), T, F, L, torch.bfloat16)
    want_row = dec.decoders[f"{L - 1}->{L - 1}"].weight[:, F - 1].float()
    for workspace in (ws, None):
        out = engine.decode_sparse(one, dec.packed(), "none", d, t_begin=L - 1, t_end=L, out_f32=True, ws=workspace)
        assert torch.equal(out[L - 1, 0], want_row)
        assert float(out[L - 1, 1:].abs().max()) == 0.0
    del model, inputs
    _free()


def test_c2_training_step_at_full_size(dev):
    """One optimisation step of the JumpReLU configuration at its own size: the backward kernels index a
    decoder slab and moment slabs of 1.0e10 elements, the threshold gradient takes its dense product from
    24 K-segments of the gradient slab and of the packed decoders, and the untied decoder weights take their
    Adam step inside the weight-gradient kernel (no 40 GB fp32 gradient).  The weight gradients of the first,
    a middle and the LAST decoder pair are checked against dense torch formulations, the in-place step against
    torch.optim.Adam on those gradients, and the step as a whole through the loss."""
    wl = synth.WORKLOADS["c2"]
    L, T, F, d = wl.num_layers, wl.tokens, wl.num_features, wl.d_model
    model, inputs, _ = synth.build_model(wl, dev)
    model.eval()
    tgt = synth.make_targets(wl, dev)
    targets = {l: tgt[l] for l in range(L)}
    lr = 1e-3
    opt = cca.CLTAdam(model, lr=lr)
    assert opt.fuses_decoder_step()
    pairs = [(0, 0), (7, 19), (L - 1, L - 1)]                    # slots 0, a middle one, 299
    slot_of = lambda s, t: s * L - (s * (s - 1)) // 2 + (t - s)  # noqa: E731
    # the gradients as separate tensors first (the two-step route: 40 GB of fp32 decoder gradients)
    recs, surv = model.forward_with_survivors(inputs)
    diff = torch.stack([recs[l] for l in range(L)]).float() - tgt.float()
    want_loss = float((diff.double() ** 2).mean(dim=(1, 2)).sum())
    g32 = 2.0 * diff / (T * d)                                   # d loss / d rec, [L, T, d]
    del recs, diff
    dense = engine.densify(surv)                                 # kept activations, [L, T, F] bf16 (6.4 GB)
    loss_l, raw = model._loss_and_raw_gradients(inputs, targets)
    assert abs(float(loss_l.sum()) - want_loss) <= 1e-4 * want_loss
    kept = {}
    for s, t in pairs:
        got = raw["dec_w"][slot_of(s, t)]                        # [F, d]
        want = dense[s].float().t() @ g32[t]                     # dW[s->t] = a[s]^T g[t]
        err = orc.rel_l2(got.cpu(), want.cpu())
        assert err <= 2e-2, (s, t, err)                          # the kernel reads g rounded to bf16
        kept[(s, t)] = got.t().contiguous().clone()              # checkpoint layout [d, F]
    assert raw["theta"] is not None and bool(torch.isfinite(raw["theta"]).all())
    del dense, g32, raw, surv, want, got
    _free()
    before = {k: model.decoder_module.decoders[f"{k[0]}->{k[1]}"].weight.detach().float().clone() for k in pairs}
    theta_before = model.theta_manager.log_threshold.detach().float().clone()
    # the step itself, with the decoder weights updated inside the weight-gradient kernel
    loss0 = float(model.training_step(inputs, targets, opt))
    assert abs(loss0 - want_loss) <= 1e-4 * want_loss
    # ... over column tiles where the batch's slice fits the LDS (4096 tokens do), else row by row
    assert (opt._dec_layout == "tiles") == (engine.decoder_tile_width(T, d, F, torch.bfloat16) > 0)
    assert opt._dec_layout == ("tiles" if T <= 4096 else "rows")
    for (s, t) in pairs:
        p = torch.nn.Parameter(before[(s, t)].clone())
        p.grad = kept[(s, t)]
        torch.optim.Adam([p], lr=lr, betas=(0.9, 0.999), eps=1e-8).step()
        want = p.detach().to(torch.bfloat16)
        got = model.decoder_module.decoders[f"{s}->{t}"].weight.detach()
        same = (got.view(torch.int16) == want.view(torch.int16)).float().mean()
        # fp32 rounding differences can move a value that sits on a bf16 rounding boundary by one ulp (the
        # gradients here are of the order of eps, so the step is not simply lr * sign(g))
        assert float(same) >= 0.99, (s, t, float(same))
        assert orc.rel_l2(got.float().cpu(), want.float().cpu()) <= 1e-3
        assert float((got.float() != before[(s, t)]).float().mean()) > 0.1     # the step did change bf16 values
        assert torch.equal(model.decoder_module.packed()[slot_of(s, t)][:, :d], got.t())
    del before, kept
    _free()
    theta_after = model.theta_manager.log_threshold.detach().float()
    # (log_threshold is a bf16 parameter near -1: a step of lr = 1e-3 is below half an ulp for most elements)
    assert bool(torch.isfinite(theta_after).all()) and float((theta_after != theta_before).float().mean()) > 0.01
    loss1, _ = model._loss_and_raw_gradients(inputs, targets)
    assert float(loss1.sum()) < loss0, (float(loss1.sum()), loss0)
    print(f"c2 training step: loss {loss0:.5f} -> {float(loss1.sum()):.5f}")
    del model, inputs, opt
    _free()


# ---- C3: decoders tied per target, 8192 tokens, d_model 2048 -------------------------------------------
def test_c3_per_target_forward_at_full_size(dev):
    wl = synth.WORKLOADS["c3"]
    L, T, F, d, k = wl.num_layers, wl.tokens, wl.num_features, wl.d_model, wl.k
    model, inputs, _ = synth.build_model(wl, dev)
    model.eval()
    dec = model.decoder_module
    res = model._survivors(inputs)
    assert res is not None
    _, _, surv = res
    rp = surv.row_ptr.long()
    assert (rp[T::T] - rp[:-1:T]).tolist() == [k * T] * L             # exactly k*T survivors per layer
    recs = model(inputs)
    first_dense = dec.last_route["dense_targets"][0]
    assert first_dense <= 2 and dec.last_route["dense_targets"][1] == L, dec.last_route
    # the row-gather route on the same survivors: all sources in one launch, 8 feature slices
    assert engine.decode_route(T, d, F, L, "per_target", torch.bfloat16) == nat.ROUTE_SLICED_ALL_SOURCES
    dec.dense_route = False
    gathered = model(inputs)
    dec.dense_route = True
    dense = engine.densify(surv)
    for t in (0, 8, L - 1):
        summed = torch.zeros(T, F, dtype=torch.float32, device=dev)
        for s in range(t + 1):
            summed += dense[s].float()
        lin = dec.decoders[t]
        want = (summed @ lin.weight.float().t() + lin.bias_param.float()).cpu()     # decoder.py:208-251
        for name, got in (("dense route", recs), ("gather route", gathered)):
            err = orc.rel_l2(got[t].float().cpu(), want)
            assert err <= 1e-2, (name, t, err)
    del model, inputs, dense, recs, gathered
    _free()


def test_c3_training_step_at_full_size(dev):
    """Gradients and one optimisation step with decoders tied per target at the configuration's own size
    (d_model 2048 is the widest row the backward kernels take, 8192 tokens): a decoder matrix sums the token
    lists of all its sources, the value gradients walk all sources of a target.  Against dense torch
    formulations of the reference's computation (decoder.py:208-251 differentiated)."""
    wl = synth.WORKLOADS["c3"]
    L, T, F, d, k = wl.num_layers, wl.tokens, wl.num_features, wl.d_model, wl.k
    model, inputs, _ = synth.build_model(wl, dev)
    model.eval()
    tgt = synth.make_targets(wl, dev)
    targets = {l: tgt[l] for l in range(L)}
    loss, grads = model.loss_and_gradients(inputs, targets)
    recs, surv = model.forward_with_survivors(inputs)
    diff = torch.stack([recs[l] for l in range(L)]).float() - tgt.float()
    want_loss = float((diff.double() ** 2).mean(dim=(1, 2)).sum())
    assert abs(float(loss) - want_loss) <= 1e-4 * want_loss
    g32 = 2.0 * diff / (T * d)
    del recs, diff
    dense = engine.densify(surv)                                  # [L, T, F] bf16, 4.3 GB
    # decoder t: rec[t] = (sum over s <= t of a[s]) W[t]^T + b[t]   =>   dW[t] = g[t]^T sum_s a[s]
    for t in (0, 8, L - 1):
        summed = torch.zeros(T, F, dtype=torch.float32, device=dev)
        for s_ in range(t + 1):
            summed += dense[s_].float()
        want = g32[t].t() @ summed
        err = orc.rel_l2(grads[f"decoder_module.decoders.{t}.weight"].float().cpu(), want.cpu())
        assert err <= 2e-2, (t, err)
        err_b = orc.rel_l2(grads[f"decoder_module.decoders.{t}.bias_param"].cpu(), g32[t].sum(dim=0).cpu())
        assert err_b <= 1e-3, (t, err_b)
    del summed, want
    # encoder s: d loss / d a[s] = sum over t >= s of g[t] W[t], through the straight-through gate
    for s_ in (0, L - 1, 9):
        dact = None
        for t in range(s_, L):
            term = g32[t] @ model.decoder_module.decoders[t].weight.float()
            dact = term if dact is None else dact + term
        dpre = dact * (dense[s_] != 0)
        err_w = orc.rel_l2(grads[f"encoder_module.encoders.{s_}.weight"].cpu(), (dpre.t() @ inputs[s_].float()).cpu())
        err_b = orc.rel_l2(grads[f"encoder_module.encoders.{s_}.bias_param"].cpu(), dpre.sum(dim=0).cpu())
        assert err_w <= 2e-2 and err_b <= 2e-2, (s_, err_w, err_b)
    names = ["decoder_module.decoders.8.weight", f"decoder_module.decoders.{L - 1}.weight", "encoder_module.encoders.9.weight"]
    params = dict(model.named_parameters())
    g_ref = {n: grads[n].float().contiguous().clone() for n in names}
    before = {n: params[n].detach().float().clone() for n in names}
    del dense, dact, dpre, term, g32, grads, surv
    _free()
    # one optimisation step (two-step route: a tied matrix collects its gradient over several launches)
    opt = cca.CLTAdam(model, lr=1e-4)
    assert not opt.fuses_decoder_step()
    loss0 = float(model.training_step(inputs, targets, opt))
    assert abs(loss0 - want_loss) <= 1e-4 * want_loss
    for n in names:
        p = torch.nn.Parameter(before[n].clone())
        p.grad = g_ref[n]
        torch.optim.Adam([p], lr=1e-4, betas=(0.9, 0.999), eps=1e-8).step()
        want = p.detach().to(torch.bfloat16)
        got = params[n].detach()
        same = (got.view(torch.int16) == want.view(torch.int16)).float().mean()
        assert float(same) >= 0.99, (n, float(same))
        assert orc.rel_l2(got.float().cpu(), want.float().cpu()) <= 1e-3
        assert float((got.float() != before[n]).float().mean()) > 0.05    # the step did change bf16 values
    print(f"c3 training step: loss {loss0:.5f}")
    del model, inputs, opt, params, before, g_ref
    _free()


# ---- C4: training step at the GPT-2-small x32 shape, bf16 parameters, fp32 Adam moments ------------------
def _dense_dact(model, g32, s, L):
    """d loss / d activation of source layer s as the reference's autograd forms it: sum over the targets
    t >= s of g[t] @ W[s->t]   ([T, d] x [d, F])."""
    out = None
    for t in range(s, L):
        term = g32[t] @ model.decoder_module.decoders[f"{s}->{t}"].weight.float()
        out = term if out is None else out + term
    return out


def test_c4_training_step_at_full_size_in_bf16(dev):
    wl = synth.WORKLOADS["c1"]
    L, T, F, d, k = wl.num_layers, wl.tokens, wl.num_features, wl.d_model, wl.k
    model, inputs, _ = synth.build_model(wl, dev)
    model.eval()
    tgt = synth.make_targets(wl, dev)
    targets = {l: tgt[l] for l in range(L)}
    loss, grads = model.loss_and_gradients(inputs, targets)
    recs, surv = model.forward_with_survivors(inputs)
    rec32 = torch.stack([recs[l] for l in range(L)]).float()
    diff = rec32 - tgt.float()
    # loss: sum over layers of the per-layer mean squared error of the bf16 reconstructions (losses.py:45-92)
    want_loss = float((diff.double() ** 2).mean(dim=(1, 2)).sum())
    assert abs(float(loss) - want_loss) <= 1e-5 * want_loss
    g32 = 2.0 * diff / (T * d)                                   # d loss / d rec, [L, T, d]
    # decoder biases: column sums of g[t]
    for t in (0, 5, L - 1):
        got = grads[f"decoder_module.decoders.{t}->{t}.bias_param"]
        assert orc.rel_l2(got.cpu(), g32[t].sum(dim=0).cpu()) <= 1e-3
    dense = engine.densify(surv)                                 # kept activations, [L, T, F] bf16
    # decoder weights: dW[s->t] = g[t]^T a[s]   ([d, T] x [T, F]); the kernel reads g rounded to bf16
    for s, t in ((0, 0), (3, 7), (L - 1, L - 1)):
        want = g32[t].t() @ dense[s].float()
        got = grads[f"decoder_module.decoders.{s}->{t}.weight"]
        err = orc.rel_l2(got.float().cpu(), want.cpu())
        assert err <= 2e-2, (s, t, err)
    # encoder: the straight-through gate hands d loss / d activation to the kept pre-activations only
    # (activations.py:82-90); dW_enc = (mask * dact)^T x, db_enc = column sums of mask * dact
    for s in (0, 6, L - 1):
        dpre = _dense_dact(model, g32, s, L) * (dense[s] != 0)
        want_w = dpre.t() @ inputs[s].float()
        want_b = dpre.sum(dim=0)
        err_w = orc.rel_l2(grads[f"encoder_module.encoders.{s}.weight"].cpu(), want_w.cpu())
        err_b = orc.rel_l2(grads[f"encoder_module.encoders.{s}.bias_param"].cpu(), want_b.cpu())
        assert err_w <= 2e-2 and err_b <= 2e-2, (s, err_w, err_b)
    del dense, dpre, want_w, want, rec32, diff, recs
    _free()

    # The loss is quadratic in the decoder weights and biases, so along a direction V
    #     loss(W + V) - loss(W - V) = 2 <grad(W), V>
    # with no step-size limit.  In bf16 W +- V must be representable: V is +-4 ulp of each weight whose
    # mantissa is far enough from its binade's ends (0 elsewhere), signed like the gradient.
    params = dict(model.named_parameters())
    names = ["decoder_module.decoders.0->0.weight", "decoder_module.decoders.3->7.weight",
             "decoder_module.decoders.11->11.weight"]
    predicted, dirs = 0.0, {}
    for n in names:
        p = params[n].detach()
        bits = p.view(torch.int16).to(torch.int32) & 0xFFFF
        mant, expo = bits & 0x7F, (bits >> 7) & 0xFF
        safe = (mant >= 8) & (mant <= 0x7F - 8) & (expo > 20)
        ulp = torch.ldexp(torch.ones_like(p, dtype=torch.float32), (expo - 127 - 7).to(torch.int32))
        v = torch.where(safe, 4.0 * ulp * torch.sign(grads[n].float()), torch.zeros_like(ulp))
        plus, minus = (p.float() + v).to(torch.bfloat16), (p.float() - v).to(torch.bfloat16)
        assert torch.equal(plus.float(), p.float() + v) and torch.equal(minus.float(), p.float() - v)
        dirs[n] = v
        predicted += 2.0 * float((grads[n].double() * v.double()).sum())
    del grads
    with torch.no_grad():
        for n in names:
            params[n].copy_((params[n].float() + dirs[n]).to(torch.bfloat16))
        plus_loss, _ = model.loss_and_gradients(inputs, targets)
        for n in names:
            params[n].copy_((params[n].float() - 2 * dirs[n]).to(torch.bfloat16))
        minus_loss, _ = model.loss_and_gradients(inputs, targets)
        for n in names:
            params[n].copy_((params[n].float() + dirs[n]).to(torch.bfloat16))
    measured = float(plus_loss.double() - minus_loss.double())
    print(f"c4: loss {float(loss):.6f}, loss(W+V) - loss(W-V) = {measured:.6e}, 2<grad, V> = {predicted:.6e}")
    assert abs(predicted) > 1e-4 * float(loss)
    # the reconstructions are rounded to bf16 before the loss, and the gradient was formed from bf16 g
    assert abs(measured - predicted) <= 3e-2 * abs(predicted), (measured, predicted)
    del dirs
    _free()

    # one optimisation step: every parameter family against torch.optim.Adam on the same fp32 gradients,
    # fp32 arithmetic from the bf16 parameter, one rounding (two full-size tensors)
    opt = cca.CLTAdam(model, lr=1e-4, betas=(0.9, 0.999))
    loss_l, raw = model._loss_and_raw_gradients(inputs, targets)
    slot = 3 * L - 3 + (7 - 3)                                         # "3->7"
    before = {"enc": model.encoder_module.encoders[5].weight.detach().float().clone(),
              "dec": model.decoder_module.decoders["3->7"].weight.detach().float().clone()}
    g_ref = {"enc": raw["enc_w"][5].clone(), "dec": raw["dec_w"][slot].t().contiguous().clone()}
    opt.step(raw)
    after = {"enc": model.encoder_module.encoders[5].weight.detach(),
             "dec": model.decoder_module.decoders["3->7"].weight.detach()}
    for key in ("enc", "dec"):
        p = torch.nn.Parameter(before[key].clone())
        p.grad = g_ref[key]
        torch.optim.Adam([p], lr=1e-4, betas=(0.9, 0.999), eps=1e-8).step()
        want = p.detach().to(torch.bfloat16)
        got = after[key]
        same = (got.view(torch.int16) == want.view(torch.int16)).float().mean()
        # fp32 rounding differences can move a value that sits on a bf16 rounding boundary by one ulp
        assert float(same) >= 0.999, (key, float(same))
        assert orc.rel_l2(got.float().cpu(), want.float().cpu()) <= 1e-3
        moved = (got.float() != before[key]).float().mean()
        assert float(moved) > 0.0                                     # the step did change bf16 values
    # the feature-major working copy of the decoder follows its parameter
    assert torch.equal(model.decoder_module.packed()[slot][:, :d], after["dec"].t())
    del raw, opt, before, after, g_ref
    _free()

    # The route training_step takes at this size (what `bench.py --train-step` times): the untied decoder weights
    # take their Adam step inside the column-tile weight-gradient kernel (d = 768: 48 column slices, T * 32 B =
    # 128 KB filling the LDS).  Three decoder pairs against torch.optim.Adam on separately computed gradients.
    pairs = [(0, 0), (3, 7), (L - 1, L - 1)]
    slot_of = lambda s_, t_: s_ * L - (s_ * (s_ - 1)) // 2 + (t_ - s_)  # noqa: E731
    loss_l, raw = model._loss_and_raw_gradients(inputs, targets)
    want_loss = float(loss_l.sum())
    kept = {k_: raw["dec_w"][slot_of(*k_)].t().contiguous().clone() for k_ in pairs}
    del raw
    _free()
    before = {k_: model.decoder_module.decoders[f"{k_[0]}->{k_[1]}"].weight.detach().float().clone() for k_ in pairs}
    opt = cca.CLTAdam(model, lr=1e-4, betas=(0.9, 0.999))
    assert opt.fuses_decoder_step() and engine.decoder_tile_width(T, d, F, torch.bfloat16) > 0
    loss0 = float(model.training_step(inputs, targets, opt))
    assert abs(loss0 - want_loss) <= 1e-5 * want_loss
    assert opt._dec_layout == "tiles"
    assert model.decoder_module._params_behind            # the parameters follow when they are read (below)
    for (s_, t_) in pairs:
        p = torch.nn.Parameter(before[(s_, t_)].clone())
        p.grad = kept[(s_, t_)]
        torch.optim.Adam([p], lr=1e-4, betas=(0.9, 0.999), eps=1e-8).step()
        want = p.detach().to(torch.bfloat16)
        got = model.decoder_module.decoders[f"{s_}->{t_}"].weight.detach()
        same = (got.view(torch.int16) == want.view(torch.int16)).float().mean()
        assert float(same) >= 0.99, (s_, t_, float(same))
        assert orc.rel_l2(got.float().cpu(), want.float().cpu()) <= 1e-3
        assert float((got.float() != before[(s_, t_)]).float().mean()) > 0.1
        assert torch.equal(model.decoder_module.packed()[slot_of(s_, t_)][:, :d], got.t())
    loss1, _ = model._loss_and_raw_gradients(inputs, targets)
    assert float(loss1.sum()) < loss0
    del model, inputs, opt, before, kept
    _free()
