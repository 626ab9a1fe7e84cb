"""The forward path at the full sizes of the benchmark workloads.

A dense CPU forward at these sizes takes minutes, so parity is checked through properties
that do not depend on size, and against independent formulations on the GPU:

* selection: the fused route (candidates collected by the encoder) and the streaming route
  (dense pre-activations, one pass) give the same survivor list bit for bit; each layer keeps
  exactly k*T entries; rows are strictly ascending; kept values equal the pre-activations;
  the smallest kept value is >= the largest value left out;
* decode: scaling the survivor values by 2 scales the output by exactly 2; the sliced schedule
  agrees with the single-pass schedule; the result agrees (rel-L2 <= 1e-2 in bf16) with a
  dense fp32 torch matmul over the densified activations;
* C0 (fp32, the size a CPU can run) end to end against the oracle, stage by stage on identical
  inputs: pre-activations rel-L2 <= 1e-5, survivor set bit-exact, reconstructions <= 1e-5.
"""
import pytest
import torch

from crosslayer_coding_amd import engine, synth
from oracle import clt_oracle as orc

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def c1(dev):
    wl = synth.WORKLOADS["c1"]
    model, inputs, slab = synth.build_model(wl, dev)
    model.eval()
    yield wl, model, inputs, slab
    del model, inputs, slab
    torch.cuda.empty_cache()


def test_c1_selection_routes_agree_and_hold_the_topk_properties(dev, c1):
    wl, model, inputs, _ = c1
    L, T, F, k = wl.num_layers, wl.tokens, wl.num_features, wl.k
    _, x, w, b = model.encoder_module.prepare_slab(inputs)
    assert engine.encode_collect_supported(x, w, b, k)
    pre = engine.encode(x, w, b)
    ref = engine.batchtopk_select(pre, k, False)
    ws = engine.Workspace(x.device)
    got = engine.collect_select(engine.encode_collect(x, w, b, k, torch.empty_like(pre), ws))
    torch.cuda.synchronize()
    assert torch.equal(got.row_ptr, ref.row_ptr)
    assert torch.equal(got.col, ref.col)
    assert torch.equal(got.val.view(torch.int16), ref.val.view(torch.int16))
    # exactly k*T per layer
    rp = got.row_ptr.long()
    per_layer = rp[T::T] - rp[:-1:T]
    assert per_layer.tolist() == [k * T] * L
    # strictly ascending columns inside every row
    rows = engine.survivor_rows(got).long()
    col = got.col.long()
    same_row = rows[1:] == rows[:-1]
    assert bool(((col[1:] > col[:-1]) | ~same_row).all())
    assert bool((rows[1:] >= rows[:-1]).all())
    # values are the pre-activations at those positions; threshold property per layer
    flat = rows * F + col
    assert torch.equal(pre.view(-1)[flat].view(torch.int16), got.val.view(torch.int16))
    mask = torch.zeros(L * T * F, dtype=torch.bool, device=pre.device)
    mask[flat] = True
    mask = mask.view(L, T * F)
    pf = pre.view(L, T * F).float()
    kept_min = torch.where(mask, pf, torch.full_like(pf, float("inf"))).min(dim=1).values
    left_max = torch.where(mask, torch.full_like(pf, float("-inf")), pf).max(dim=1).values
    assert bool((kept_min >= left_max).all())


def test_c1_decode_linearity_schedules_and_dense_reference(dev, c1):
    wl, model, inputs, _ = c1
    L, T, F, d = wl.num_layers, wl.tokens, wl.num_features, wl.d_model
    res = model._survivors(inputs)
    _, _, surv = res
    dec = model.decoder_module
    ws = model._workspace()
    mask = (1 << L) - 1
    tying = wl.decoder_tying

    def run(sv, workspace, bias=None):
        return engine.decode_sparse(sv, dec.packed(), tying, d, bias_sum=bias, src_mask=mask, out_f32=True, ws=workspace)

    # linearity: doubling the activations doubles the (bias-free) output exactly
    plain = run(surv, ws).clone()
    doubled = engine.SurvivorList(surv.row_ptr, surv.col, (surv.val.float() * 2).to(surv.val.dtype), T, F, L, surv.dtype)
    assert torch.equal(run(doubled, ws), 2 * plain)
    # the single-pass schedule (no workspace) agrees up to fp32 summation order
    out = run(surv, ws, dec.bias_sum(mask)).clone()
    single = run(surv, None, dec.bias_sum(mask))
    assert orc.rel_l2(single.cpu(), out.cpu()) <= 1e-5
    # dense fp32 torch reference for three targets
    dense = engine.densify(surv)
    for t in (0, 5, L - 1):
        ref = torch.zeros(T, d, dtype=torch.float32, device=dense.device)
        for s in range(t + 1):
            lin = dec.decoders[f"{s}->{t}"]
            ref += dense[s].float() @ lin.weight.float().t() + lin.bias_param.float()
        assert orc.rel_l2(out[t].cpu(), ref.cpu()) <= 1e-2
    rec = model(inputs)
    assert orc.rel_l2(rec[L - 1].float().cpu(), out[L - 1].cpu()) <= 1e-2


def test_c0_full_size_against_the_oracle_stage_by_stage(dev):
    wl = synth.WORKLOADS["c0"]
    L, T, F, d, k = wl.num_layers, wl.tokens, wl.num_features, wl.d_model, wl.k
    model, inputs, _ = synth.build_model(wl, dev)
    model.eval()
    sd = {n: v.detach().cpu() for n, v in model.state_dict().items()}
    pre_dict, _ = model._encode_all_layers(inputs)
    for l in (0, L - 1):
        ref = orc.encoder_preactivations(inputs[l].cpu(), sd[f"encoder_module.encoders.{l}.weight"],
                                         sd[f"encoder_module.encoders.{l}.bias_param"])
        assert orc.rel_l2(pre_dict[l].cpu(), ref) <= 1e-5
    acts = model.get_feature_activations(inputs)
    for l in range(L):
        pre_l = pre_dict[l].cpu()
        assert torch.equal(acts[l].cpu(), orc.batchtopk_forward(pre_l, float(k), pre_l))
    recs = model(inputs)
    names = synth.decoder_names(wl)
    dec_w = {n: sd[f"decoder_module.decoders.{n}.weight"] for n in names}
    dec_b = {n: sd[f"decoder_module.decoders.{n}.bias_param"] for n in names}
    cpu_acts = {l: acts[l].cpu() for l in range(L)}
    for t in (0, L // 2, L - 1):
        ref = orc.decode(cpu_acts, t, tying="none", weights=dec_w, biases=dec_b, d_model=d, num_features=F,
                         dtype=torch.float32)
        assert orc.rel_l2(recs[t].cpu(), ref) <= 1e-5


def test_c1_sized_gradients_against_exact_differences_of_the_quadratic_loss(dev):
    # The loss is quadratic in the decoder weights and biases, so along any direction V
    #     loss(W + V) - loss(W - V) = 2 <grad(W), V>
    # holds exactly (no step-size limit), and the encoder / selection do not move.  fp32 so that W +- V
    # is what the kernels read; C1's shape otherwise.
    wl = synth.WORKLOADS["c1"].scaled("c1-f32", dtype="float32")
    L, T, d, F = wl.num_layers, wl.tokens, wl.d_model, wl.num_features
    model, inputs, _ = synth.build_model(wl, dev)
    model.eval()
    g = torch.Generator(device=dev).manual_seed(17)
    targets = {l: torch.randn(T, d, generator=g, device=dev) for l in range(L)}
    loss, grads = model.loss_and_gradients(inputs, targets)
    params = dict(model.named_parameters())
    names = ["decoder_module.decoders.0->0.weight", "decoder_module.decoders.3->7.weight",
             "decoder_module.decoders.11->11.weight", "decoder_module.decoders.2->5.bias_param"]
    # direction: the gradient itself, scaled to the size of the parameter (a random direction is almost
    # orthogonal to the gradient and its effect drowns in the rounding of the loss)
    predicted, dirs = 0.0, {}
    for n in names:
        p, gr = params[n], grads[n]
        v = gr * (float(p.detach().norm().clamp_min(1.0)) / float(gr.norm()))
        dirs[n] = v
        predicted += 2.0 * float((gr.double() * v.double()).sum())
    del grads
    with torch.no_grad():
        for n in names:
            params[n].add_(dirs[n])
        plus, _ = model.loss_and_gradients(inputs, targets)
        for n in names:
            params[n].sub_(2 * dirs[n])
        minus, _ = model.loss_and_gradients(inputs, targets)
    measured = float(plus.double() - minus.double())
    assert abs(predicted) > 1e-2 * float(loss)              # the direction is not degenerate
    assert abs(measured - predicted) <= 1e-4 * abs(predicted), (measured, predicted)
    # the bias gradient of target t is the column sum of d loss / d rec[t] = 2 (rec - target) / (T d)
    with torch.no_grad():
        for n in names:
            params[n].add_(dirs[n])
    loss2, grads = model.loss_and_gradients(inputs, targets)
    assert abs(float(loss2) - float(loss)) <= 1e-5 * float(loss)
    rec = model(inputs)
    for t in (0, 5, L - 1):
        want = (2.0 * (rec[t].double() - targets[t].double()) / (T * d)).sum(dim=0)
        assert orc.rel_l2(grads[f"decoder_module.decoders.{t}->{t}.bias_param"].double().cpu(), want.cpu()) <= 1e-4
    del model, grads, params, dirs
    torch.cuda.empty_cache()


def test_c1_evaluator_counts_against_dense_scans(dev, c1):
    # the reductions on the survivor list against the reference's own formulation (dense scans with torch
    # ops) on the GPU, layer by layer, at full size
    wl, model, inputs, _ = c1
    L, T, F, k = wl.num_layers, wl.tokens, wl.num_features, wl.k
    recs, surv = model.forward_with_survivors(inputs)
    nonzero, fired = engine.survivor_metrics(surv)
    dense = engine.densify(surv)
    for l in range(L):
        a = dense[l]
        assert int(nonzero[l]) == int((a != 0).sum())
        assert torch.equal(fired[l].long(), (a.float() > 1e-6).sum(dim=0))
    assert int(nonzero.sum()) <= L * k * T        # a kept value can be an exact zero, never more than k*T entries
    passes = torch.randint(0, 5, (L, F), device=dev)
    want = torch.where(fired > 0, torch.zeros_like(passes), passes + 1)
    engine.dead_feature_update(fired, passes)
    assert torch.equal(passes, want)
    # reconstruction statistics against torch's own variance / mse on the same tensors
    tgt = torch.stack([inputs[l] for l in range(L)]).contiguous()        # any [L, T, d] tensor serves as target
    rec = torch.stack([recs[l] for l in range(L)]).contiguous()
    stats = engine.reconstruction_stats(rec, tgt)
    for l in (0, L - 1):
        t, r = tgt[l].float(), rec[l].float()
        assert float(stats[l, 0]) == pytest.approx(float(torch.nn.functional.mse_loss(r, t)), rel=1e-4)
        assert float(stats[l, 1]) == pytest.approx(float(torch.var(t, dim=0, unbiased=False).mean()), rel=1e-4)
        assert float(stats[l, 2]) == pytest.approx(float(torch.var(t - r, dim=0, unbiased=False).mean()), rel=1e-4)


def test_c1_sized_feed_round_trip(dev):
    # rows gathered without normalisation are the stored rows, bit for bit; with sqrt(d) scaling they
    # equal torch's own fp32 multiply and cast on the GPU
    import numpy as np
    import crosslayer_coding_amd as cca
    L, T, d, rows = 12, 4096, 768, 8192
    g = torch.Generator().manual_seed(3)
    chunks = [torch.randn(L, 2, rows, d, generator=g).to(torch.bfloat16) for _ in range(2)]
    rng = np.random.RandomState(4)
    idxs = np.stack([rng.randint(0, 2, T), rng.randint(0, rows, T)], axis=1).astype(np.uint32)
    order = np.concatenate([np.nonzero(idxs[:, 0] == c)[0] for c in (0, 1)])        # ascending chunk, sampler order inside
    for method in ("none", "sqrt_d_model"):
        feed = cca.DeviceActivationFeed(L, d, dtype="bfloat16", device=dev, normalization_method=method)
        for c, t in enumerate(chunks):
            feed.add_chunk(c, t)
        ins, tgs = feed.parse_batch(idxs)
        for kind, got in ((0, ins), (1, tgs)):
            for l in (0, 7, L - 1):
                want = torch.stack([chunks[int(idxs[i, 0])][l, kind, int(idxs[i, 1])] for i in order[:64]]).to(dev)
                if method == "sqrt_d_model":
                    want = (want.float() * (d ** 0.5)).to(torch.bfloat16)
                assert torch.equal(got[l][:64].view(torch.int16), want.view(torch.int16))
        full = torch.cat([chunks[c][5, 0, torch.as_tensor(idxs[idxs[:, 0] == c, 1].astype(np.int64))] for c in (0, 1)]).to(dev)
        if method == "sqrt_d_model":
            full = (full.float() * (d ** 0.5)).to(torch.bfloat16)
        assert torch.equal(ins[5].view(torch.int16), full.view(torch.int16))
