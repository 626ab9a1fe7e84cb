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
