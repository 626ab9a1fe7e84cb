"""Gradients of the MSE reconstruction loss from the survivor list (C ABI kernels) against torch
autograd through the oracle's dense forward.  fp32: rel-L2 <= 1e-5; bf16: <= 1e-2 (the kernels read
bf16 weights / inputs and accumulate in fp32; the oracle runs in fp32 on the same bf16 values)."""
import pytest
import torch

from crosslayer_coding_amd import _native as nat
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
    BASE.scaled("bw-jump-bf16", activation_fn="jumprelu", k=None, dtype="bfloat16", num_layers=2, d_model=128, num_features=512, tokens=256),
    BASE.scaled("bw-jump-per-target", activation_fn="jumprelu", k=None, decoder_tying="per_target"),
    BASE.scaled("bw-fused", num_layers=2, d_model=128, num_features=512, tokens=256, k=10, dtype="bfloat16"),
    # one layer of inputs / loss gradient larger than an XCD's L2: the weight-gradient kernels split the columns
    BASE.scaled("bw-split", num_layers=2, d_model=768, num_features=512, tokens=4096, k=12, dtype="bfloat16"),
    BASE.scaled("bw-split-f32", num_layers=2, d_model=200, num_features=256, tokens=4096, k=6),
    # other gates: the survivor list is whatever the forward selected, the backward does not care how
    BASE.scaled("bw-global", topk_mode="global"),
    BASE.scaled("bw-tokentopk", activation_fn="topk", k=5),
    BASE.scaled("bw-tokentopk-global", activation_fn="topk", k=5, topk_mode="global", dtype="bfloat16"),
    BASE.scaled("bw-relu", activation_fn="relu", k=None),
    # tied decoders: one matrix per source (collects its targets) or per target (sums its sources)
    BASE.scaled("bw-per-source", decoder_tying="per_source"),
    BASE.scaled("bw-per-target", decoder_tying="per_target"),
    BASE.scaled("bw-per-source-bf16", decoder_tying="per_source", dtype="bfloat16", num_layers=4),
    BASE.scaled("bw-per-target-split", decoder_tying="per_target", num_layers=3, d_model=200, num_features=256, tokens=4096, k=6),
    # rows beyond 2048 elements (up to 4096: eight 16-byte pieces per lane in bf16, up to sixteen in fp32)
    BASE.scaled("bw-d4096-bf16", num_layers=2, d_model=4096, num_features=256, tokens=96, k=8, dtype="bfloat16"),
    BASE.scaled("bw-d2304-f32", num_layers=2, d_model=2304, num_features=256, tokens=64, k=8),
    BASE.scaled("bw-d4096-f32-jump", num_layers=2, d_model=4096, num_features=256, tokens=64, activation_fn="jumprelu", k=None),
    BASE.scaled("bw-d3072-f32-per-source", num_layers=2, d_model=3072, num_features=128, tokens=64, k=6, decoder_tying="per_source"),
    # a batch beyond 65536 tokens (the per-feature lists are ordered with fewer wavefronts per workgroup)
    BASE.scaled("bw-66000-tokens", num_layers=2, d_model=64, num_features=128, tokens=66000, k=4),
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
    if dtype == torch.bfloat16 or wl.topk_mode == "global" or wl.activation_fn == "topk":
        masks = {l: (a != 0).cpu() for l, a in model.get_feature_activations(inputs).items()}
    names = synth.decoder_names(wl)
    theta, log_theta = None, None
    if wl.activation_fn == "jumprelu":
        # the oracle then runs the reference's JumpReLU backward, threshold gradient included
        theta = torch.exp(sd["theta_manager.log_threshold"].float()).to(dtype)
        log_theta = sd["theta_manager.log_threshold"]
        masks = None
    ref_loss, ref = orc.mse_loss_and_gradients(
        {l: x[l] for l in range(L)}, targets,
        enc_w=[sd[f"encoder_module.encoders.{l}.weight"] for l in range(L)],
        enc_b=[sd[f"encoder_module.encoders.{l}.bias_param"] for l in range(L)],
        dec_w={n: sd[f"decoder_module.decoders.{n}.weight"] for n in names},
        dec_b={n: sd[f"decoder_module.decoders.{n}.bias_param"] for n in names},
        activation_fn=wl.activation_fn, num_layers=L, k=wl.k, theta=theta, masks=masks, tying=wl.decoder_tying,
        log_threshold=log_theta, model_dtype=dtype)
    tol = TOL[dtype]
    assert abs(float(loss) - float(ref_loss)) <= max(tol, 1e-6) * abs(float(ref_loss)) * 10
    for name, gref in ref.items():
        got = grads[name]
        assert got is not None and tuple(got.shape) == tuple(gref.shape), name
        err = orc.rel_l2(got.float().cpu(), gref)
        bound = tol * (5 if dtype == torch.bfloat16 else 1)
        if name.endswith("log_threshold"):
            # band membership |x - theta| <= 1/2 is decided on pre-activations that differ in the last
            # bits between the two sides; an element that changes side moves the sum by its whole term
            bound = 1e-3 if dtype == torch.float32 else 1e-1
        assert err <= bound, (name, err)


@pytest.mark.parametrize("T,F,k", [(300, 128, 9), (4100, 96, 9), (70, 40960, 9), (40, 2048, 800), (8, 32768, 5000),
                                   (70000, 32, 2), (140000, 16, 1)],
                         ids=["blocks-of-tokens", "ragged-last-block", "feature-axis-beyond-lds", "rows-longer-than-a-workgroup",
                              "rows-longer-than-the-staging-buffer", "tokens-beyond-65536", "tokens-beyond-131072"])
def test_feature_lists_are_a_permutation_grouped_by_feature(dev, T, F, k):
    # the blocked construction (counters of a token block in LDS, token order by construction; 4100 tokens = 33
    # blocks, the last one ragged; rows of ~800 survivors against 512 threads), and for a feature axis whose
    # counters do not fit the LDS the atomic construction followed by the sort
    g = torch.Generator().manual_seed(2)
    L = 2
    pre = torch.randn(L, T, F, generator=g).to(dev)
    surv = engine.batchtopk_select(pre, k, False)
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
            assert bool((tok[b + 1:e] > tok[b:e - 1]).all())      # token order, whatever the length


def test_feature_lists_of_an_empty_survivor_list(dev):
    L, T, F = 2, 100, 256
    surv = engine.threshold_select(torch.zeros(L, T, F, device=dev), None, nat.PRED_NONZERO)
    assert surv.nnz == 0
    ptr, tok, src = engine.feature_lists(surv)
    assert ptr.numel() == L * F + 1 and not bool(ptr.any())


def test_long_feature_lists_are_in_token_order_and_gradients_repeat_bit_for_bit(dev):
    # a few features fire on most tokens: their lists are far longer than a wavefront; every list must come
    # out in token order, and two runs of the whole backward must give the same bits
    g = torch.Generator().manual_seed(12)
    L, T, F = 2, 1500, 64
    pre = torch.randn(L, T, F, generator=g)
    pre[:, :, 5] += 6.0
    pre[0, ::3, 17] += 6.0
    surv = engine.batchtopk_select(pre.to(dev), 4, False)
    ptr, tok, src = (t.cpu().long() for t in engine.feature_lists(surv))
    lens = ptr[1:] - ptr[:-1]
    assert int(lens.max()) > 1000 and int((lens > 64).sum()) >= 3
    rows = engine.survivor_rows(surv).cpu().long()
    col = surv.col.cpu().long()
    for q in range(L * F):
        b, e = int(ptr[q]), int(ptr[q + 1])
        if e > b:
            l, f = divmod(q, F)
            assert bool((tok[b + 1:e] > tok[b:e - 1]).all())
            assert bool((col[src[b:e]] == f).all()) and torch.equal(rows[src[b:e]], l * T + tok[b:e])
    wl = BASE.scaled("bw-repeat", num_layers=2, d_model=128, num_features=256, tokens=2048, k=16, dtype="bfloat16")
    model, sd, x, targets = build(wl, dev)
    with torch.no_grad():       # two features that fire on nearly every token
        for l in range(2):
            model.encoder_module.encoders[l].bias_param[:2] += 8.0
    inputs = {l: x[l].to(dev) for l in range(2)}
    tg = {l: t.to(dev) for l, t in targets.items()}
    _, g1 = model.loss_and_gradients(inputs, tg)
    g1 = {k: v.clone() for k, v in g1.items()}
    _, g2 = model.loss_and_gradients(inputs, tg)
    for k in g1:
        assert torch.equal(g1[k], g2[k]), k


def _assert_same_training(a, b, dtype, steps):
    """(losses, state dict, packed slab, moments) of two runs that differ only in the association of some fp32
    sums of the decoder weight gradient.  After ONE step from the same state everything agrees to rounding; later
    steps start from states that differ in last places, where an element at the selection threshold or a
    gradient near zero can move a parameter by a whole Adam step, so then nearly all elements must agree."""
    ulp = 2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -20
    # (even after one step: where a gradient sum cancels to nearly nothing, below Adam's eps, its last places
    # decide the step; fp32 parameters show that, bf16 ones round it away.  The moments below are the strict check.)
    allowed = (1e-4 if dtype == torch.bfloat16 else 2e-2) if steps == 1 else 2e-2

    def close(x, y, what):
        # one unit in the last place of the larger of the value and the size of an Adam step (lr 1e-2 here)
        x, y = x.float(), y.float()
        bad = (x - y).abs() > ulp * torch.maximum(x.abs(), y.abs()).clamp_min(0.05)
        assert float(bad.float().mean()) <= allowed, what
        if dtype == torch.bfloat16:
            assert float((x != y).float().mean()) <= 2e-3 * steps, what
    if a[0] is not None:
        assert a[0] == pytest.approx(b[0], rel=1e-3)
    for k, v in a[1].items():
        close(v, b[1][k], k)
    if a[2] is not None:
        close(a[2], b[2], "slab")
    for x, y in zip(a[3], b[3]):
        # moments: rounding of the gradient sums, measured against the size of the terms
        assert float((x - y).abs().max()) <= (1e-5 if steps == 1 else 1e-2) * float(x.abs().max())


@pytest.mark.parametrize("dtype,d_model,fn,tokens", [
    ("bfloat16", 128, "batchtopk", 256), ("bfloat16", 768, "batchtopk", 256), ("float32", 64, "batchtopk", 256),
    ("bfloat16", 128, "jumprelu", 256),
    ("bfloat16", 136, "batchtopk", 256),    # d not a multiple of the tile width: the tile route declines
    ("bfloat16", 80, "batchtopk", 300),     # d a multiple of the tile width, not of the 64-column conversion block
    ("float32", 72, "batchtopk", 4100),     # the slice of one target fills nearly all the LDS it may take
    ("bfloat16", 128, "batchtopk", 1501)])  # two features fire on nearly every token: lists cut over many lanes
def test_adam_inside_the_weight_gradient_kernel_equals_the_two_step_sequence(dev, dtype, d_model, fn, tokens):
    # untied decoders: training_step lets the decoder weights take their Adam step inside the weight-gradient
    # kernel (no fp32 gradient in memory, parameters rewritten from the working copy), over column tiles where
    # the shape allows and row by row otherwise; three steps must leave every parameter, the packed copy and
    # both moments bit-identical to gradient-then-Adam
    import crosslayer_coding_amd as cca
    wl = BASE.scaled("bw-fuse", num_layers=3, d_model=d_model, num_features=256, tokens=tokens, dtype=dtype,
                     activation_fn=fn, k=10 if fn == "batchtopk" else None)
    runs, first = [], []
    for fuse, tiles in ((True, True), (True, False), (False, False)):
        model, sd, x, targets = build(wl, dev)
        if tokens == 1501:
            with torch.no_grad():
                for l in range(3):
                    model.encoder_module.encoders[l].bias_param[5:7] += 8.0
        opt = cca.CLTAdam(model, lr=1e-2)
        opt.fuse_decoder_step = fuse
        opt.tile_decoder_step = tiles
        assert opt.fuses_decoder_step() == fuse
        inputs = {l: x[l].to(dev) for l in range(3)}
        tg = {l: t.to(dev) for l, t in targets.items()}
        def snapshot(losses):
            return (list(losses), {k: v.detach().clone() for k, v in model.state_dict().items()},
                    model.decoder_module.packed().clone(), [t.clone() for t in opt.decoder_moments()])
        losses = [float(model.training_step(inputs, tg, opt))]
        first.append(snapshot(losses))
        losses += [float(model.training_step(inputs, tg, opt)) for _ in range(2)]
        if fuse:
            took = engine.decoder_tile_width(tokens, d_model, 256, getattr(torch, dtype)) > 0
            assert (opt._dec_layout == "tiles") == (tiles and took)
            assert took == (d_model != 136)
        runs.append(snapshot(losses))
    # row by row inside the kernel == gradient-then-Adam, bit for bit
    assert runs[1][0] == runs[2][0]
    for k, v in runs[1][1].items():
        assert torch.equal(v, runs[2][1][k]), k
    assert torch.equal(runs[1][2], runs[2][2])
    for a, b in zip(runs[1][3], runs[2][3]):
        assert torch.equal(a, b)
    # over column tiles: a list cut between two lane pairs is summed in another association, so the gradient
    # agrees to fp32 rounding; parameters may differ where that moves a rounding decision
    _assert_same_training(first[0], first[1], getattr(torch, dtype), 1)
    _assert_same_training(runs[0], runs[1], getattr(torch, dtype), 3)
    # the parameters are what the packed copy holds
    model_keys = [k for k in runs[0][1] if k.startswith("decoder_module.decoders.") and k.endswith(".weight")]
    for i, k in enumerate(sorted(model_keys, key=lambda n: [int(p) for p in n.split(".")[2].split("->")])):
        assert torch.equal(runs[0][1][k].t(), runs[0][2][i][:, :d_model]), k


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_tiled_decoder_layout_round_trip(dev, dtype):
    # slab -> tiles -> slab + checkpoint layout, on a shape with ragged 64 x 64 conversion blocks
    import ctypes
    n_dec, F, d = 3, 200, 80 if dtype == torch.bfloat16 else 72
    g = torch.Generator().manual_seed(3)
    slab = engine.alloc_packed(n_dec, F, d, dtype, dev)
    w = torch.randn(n_dec, F, d, generator=g).to(dtype).to(dev)
    slab[:, :, :d] = w
    tiles = engine.tile_decoders(slab, d)
    cs = 32 // slab.element_size()
    assert tuple(tiles.shape) == (n_dec, d // cs, F, cs)
    assert torch.equal(tiles.permute(0, 2, 1, 3).reshape(n_dec, F, d), w)
    slab2 = engine.alloc_packed(n_dec, F, d, dtype, dev)
    refs = [torch.zeros(d, F, dtype=dtype, device=dev) for _ in range(n_dec)]
    host = (ctypes.c_void_p * n_dec)(*[r.data_ptr() for r in refs])
    table = torch.tensor([r.data_ptr() for r in refs], dtype=torch.int64, device=dev)
    engine.untile_decoders(tiles, slab2, table, host)
    assert torch.equal(slab2[:, :, :d], w) and not bool(slab2[:, :, d:].any())
    for i in range(n_dec):
        assert torch.equal(refs[i], w[i].t())
    slab3 = engine.alloc_packed(n_dec, F, d, dtype, dev)
    engine.untile_decoders(tiles, slab3)
    assert torch.equal(slab3, slab2)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("T,F", [(300, 200), (257, 2248)], ids=["ragged-row-block", "two-feature-chunks"])
def test_tiled_decoder_step_kernel_against_the_row_kernel(dev, dtype, T, F):
    # the two fused kernels on the same lists, loss gradient, weights and (non-zero) moments: feature counts that
    # leave the last block of 32 rows ragged and that cross the 2048-feature work units; one feature with a long list
    g = torch.Generator().manual_seed(21)
    L, d = 3, 64
    n_dec = L * (L + 1) // 2
    pre = torch.randn(L, T, F, generator=g)
    pre[:, :, 3] += 5.0
    pre[:, :, 64:128] -= 100.0          # two whole blocks of 32 rows whose lists are empty
    surv = engine.batchtopk_select(pre.to(dtype).to(dev), 11, False)
    lists = engine.feature_lists(surv)
    ptr = lists[0].cpu()
    assert int(ptr[128] - ptr[64]) == 0 and int(ptr[4] - ptr[3]) > 64
    g_model = (torch.randn(L, T, d, generator=g) * 1e-3).to(dtype).to(dev)
    w = (torch.randn(n_dec, F, d, generator=g) * 0.1).to(dtype).to(dev)
    m0 = (torch.randn(n_dec, F, d, generator=g) * 1e-4).to(dev)
    v0 = (torch.rand(n_dec, F, d, generator=g) * 1e-7).to(dev)
    slab = engine.alloc_packed(n_dec, F, d, dtype, dev)
    slab[:, :, :d] = w
    cs = engine.decoder_tile_width(T, d, F, dtype)
    assert cs == 32 // slab.element_size()
    # row kernel
    slab_r, m_r, v_r = slab.clone(), m0.clone(), v0.clone()
    engine.decoder_weight_grad_adam(lists, surv, g_model, slab_r, m_r, v_r, 1e-3, (0.9, 0.999), 1e-8, 3)
    # tile kernel on the tiled copies
    tiles = engine.tile_decoders(slab, d)
    to_tiles = lambda t: t.view(n_dec, F, d // cs, cs).permute(0, 2, 1, 3).contiguous()      # noqa: E731
    from_tiles = lambda t: t.permute(0, 2, 1, 3).contiguous().view(n_dec, F, d)               # noqa: E731
    m_t, v_t = to_tiles(m0), to_tiles(v0)
    engine.decoder_weight_grad_adam_tiled(lists, surv, g_model, tiles, m_t, v_t, 1e-3, (0.9, 0.999), 1e-8, 3)
    slab_t = engine.alloc_packed(n_dec, F, d, dtype, dev)
    engine.untile_decoders(tiles, slab_t)
    # the gradient enters m linearly: (m - 0.9 m0) / 0.1 is the gradient each kernel summed
    g_r, g_t = (m_r - 0.9 * m0) / 0.1, (from_tiles(m_t) - 0.9 * m0) / 0.1
    assert float((g_r - g_t).abs().max()) <= 2e-5 * float(g_r.abs().max())
    assert torch.allclose(from_tiles(v_t), v_r, rtol=1e-4, atol=1e-14)
    x, y = slab_t[:, :, :d].float(), slab_r[:, :, :d].float()
    ulp = 2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -20
    # (fp32: the step is lr * m / sqrt(v) with lr 1e-3, so gradient rounding shows at the 1e-7 level whatever |w|)
    floor = 1e-3 if dtype == torch.bfloat16 else 0.1
    assert bool(((x - y).abs() <= ulp * torch.maximum(x.abs(), y.abs()).clamp_min(floor)).all())
    assert float((x != y).float().mean()) <= (1e-3 if dtype == torch.bfloat16 else 0.5)
    assert float((y - w.float()).abs().max()) > 0          # and the step did move the weights


def test_optimiser_moves_between_the_tiled_and_the_row_route(dev):
    # one optimiser, steps taken in turn through the tiled kernel, the row kernel and gradient-then-Adam: the
    # moments change layout under way and the tiled weight copy is rebuilt when the slab changed behind it;
    # the result must be the one of three plain steps
    import crosslayer_coding_amd as cca
    wl = BASE.scaled("bw-mixed", num_layers=3, d_model=128, num_features=256, tokens=256, dtype="bfloat16", k=10)
    runs = []
    for mixed in (True, False):
        model, sd, x, targets = build(wl, dev)
        opt = cca.CLTAdam(model, lr=1e-2)
        inputs = {l: x[l].to(dev) for l in range(3)}
        tg = {l: t.to(dev) for l, t in targets.items()}
        for step in range(4):
            if mixed:
                opt.fuse_decoder_step = step != 2
                opt.tile_decoder_step = step != 1
            else:
                opt.fuse_decoder_step = False
            model.training_step(inputs, tg, opt)
        runs.append(({k: v.detach().clone() for k, v in model.state_dict().items()},
                     [t.clone() for t in opt.decoder_moments()]))
    _assert_same_training((None, runs[0][0], None, runs[0][1]), (None, runs[1][0], None, runs[1][1]), torch.bfloat16, 4)


@pytest.mark.parametrize("tiled", [True, False], ids=["tile-route", "row-route"])
def test_parameters_left_behind_by_the_decoder_step_are_current_whenever_they_are_read(dev, tiled):
    # The in-kernel decoder step rewrites the feature-major slab only; the checkpoint-layout parameters [d, F]
    # follow when something reads them.  Against an optimiser that rewrites them in every step
    # (trainer.py:751-778: the reference's parameters are always current): state_dict(), named_parameters(),
    # decoders[key] and the forward must all see the same bits.
    import crosslayer_coding_amd as cca
    wl = BASE.scaled("bw-lazy", num_layers=3, d_model=128, num_features=256, tokens=256, dtype="bfloat16", k=10)
    models, opts = [], []
    for defer in (True, False):
        model, sd, x, targets = build(wl, dev)
        opt = cca.CLTAdam(model, lr=1e-2)
        opt.defer_parameter_sync, opt.tile_decoder_step = defer, tiled
        models.append(model); opts.append(opt)
    inputs = {l: x[l].to(dev) for l in range(3)}
    tg = {l: t.to(dev) for l, t in targets.items()}
    lazy, eager = models
    for step in range(3):
        for m, o in zip(models, opts):
            m.training_step(inputs, tg, o)
        assert opts[0]._dec_layout == ("tiles" if tiled else "rows")
        dec = lazy.decoder_module
        assert dec._params_behind and not eager.decoder_module._params_behind
        raw = dec.decoders._modules["0->1"].weight.detach().clone()      # the registry itself: no sync
        want = eager.decoder_module.decoders["0->1"].weight.detach()
        assert not torch.equal(raw, want)                                 # really behind ...
        if step == 0:
            got = dec.decoders["0->1"].weight.detach()                    # ... until an entry is read
        elif step == 1:
            got = dict(lazy.named_parameters())["decoder_module.decoders.0->1.weight"].detach()
        else:
            got = lazy.state_dict()["decoder_module.decoders.0->1.weight"]
        assert not dec._params_behind and torch.equal(got, want)
        # the forward never depended on them
        a, b = lazy(inputs), eager(inputs)
        assert all(torch.equal(a[t], b[t]) for t in a)
    sa, sb = lazy.state_dict(), eager.state_dict()
    assert set(sa) == set(sb) and all(torch.equal(sa[k], sb[k]) for k in sa)
    # loading a checkpoint makes the parameters the truth again
    lazy.training_step(inputs, tg, opts[0])
    assert lazy.decoder_module._params_behind
    lazy.load_state_dict(sb)
    assert not lazy.decoder_module._params_behind
    a, b = lazy(inputs), eager(inputs)
    assert all(torch.equal(a[t], b[t]) for t in a)


def test_tied_decoders_do_not_fuse_the_step(dev):
    import crosslayer_coding_amd as cca
    wl = BASE.scaled("bw-nofuse", num_layers=2, d_model=64, num_features=128, tokens=64, decoder_tying="per_source")
    model, sd, x, targets = build(wl, dev)
    assert not cca.CLTAdam(model).fuses_decoder_step()


@pytest.mark.parametrize("fn", ["batchtopk", "jumprelu"])
def test_three_training_steps_repeat_bit_for_bit(dev, fn):
    # two models built from the same state take three optimisation steps on the same batches: every
    # parameter and both Adam moments must agree bit for bit (features that fire on nearly every token
    # give lists far longer than a wavefront, the case whose order used to depend on atomics)
    import crosslayer_coding_amd as cca
    wl = BASE.scaled("bw-det", num_layers=2, d_model=128, num_features=256, tokens=1024, dtype="bfloat16",
                     activation_fn=fn, k=12 if fn == "batchtopk" else None)
    runs = []
    for rep in range(2):
        model, sd, x, targets = build(wl, dev)
        with torch.no_grad():
            for l in range(2):
                model.encoder_module.encoders[l].bias_param[:2] += 8.0
        opt = cca.CLTAdam(model, lr=1e-2)
        inputs = {l: x[l].to(dev) for l in range(2)}
        tg = {l: t.to(dev) for l, t in targets.items()}
        losses = [float(model.training_step(inputs, tg, opt)) for _ in range(3)]
        runs.append((losses, {k: v.detach().clone() for k, v in model.state_dict().items()}))
    assert runs[0][0] == runs[1][0]
    assert runs[0][0][2] < runs[0][0][0]          # and the steps do reduce the loss
    for k, v in runs[0][1].items():
        assert torch.equal(v, runs[1][1][k]), k


@pytest.mark.parametrize("tying,fn", [("none", "batchtopk"), ("per_source", "batchtopk"), ("per_target", "batchtopk"),
                                      ("none", "jumprelu")])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_training_steps_match_torch_adam_on_autograd_gradients(dev, dtype, tying, fn):
    # two optimisation steps; reference: torch.optim.Adam over the oracle's autograd gradients, fp32
    # parameters, the gate of each step taken from the model (so both sides differentiate the same
    # function); bf16 parameters are compared after rounding the reference to bf16
    import crosslayer_coding_amd as cca
    wl = BASE.scaled("tr", dtype=dtype, num_layers=2, d_model=128, num_features=256, tokens=64, decoder_tying=tying,
                     activation_fn=fn, k=6 if fn == "batchtopk" else None)
    tdt = getattr(torch, dtype)
    model, sd, x, targets = build(wl, dev)
    L = wl.num_layers
    names = synth.decoder_names(wl)
    ref = {k: v.detach().float().clone().requires_grad_(True) for k, v in sd.items()}
    ropt = torch.optim.Adam(list(ref.values()), lr=1e-2, betas=(0.9, 0.999), eps=1e-8)
    opt = cca.CLTAdam(model, lr=1e-2)
    inputs = {l: x[l].to(dev) for l in range(L)}
    tg = {l: t.to(dev) for l, t in targets.items()}
    for step in range(2):
        masks = {l: (a != 0).cpu() for l, a in model.get_feature_activations(inputs).items()}
        loss = model.training_step(inputs, tg, opt)
        # the bf16 model computes with bf16-rounded parameters: give the reference the same view
        cur = {k: (v.detach().to(tdt).float() if tdt == torch.bfloat16 else v.detach()) for k, v in ref.items()}
        ref_loss, grads = orc.mse_loss_and_gradients(
            {l: x[l] for l in range(L)}, targets,
            enc_w=[cur[f"encoder_module.encoders.{l}.weight"] for l in range(L)],
            enc_b=[cur[f"encoder_module.encoders.{l}.bias_param"] for l in range(L)],
            dec_w={n: cur[f"decoder_module.decoders.{n}.weight"] for n in names},
            dec_b={n: cur[f"decoder_module.decoders.{n}.bias_param"] for n in names},
            activation_fn=fn, num_layers=L, k=wl.k, masks=masks if fn == "batchtopk" else None, tying=tying,
            log_threshold=cur.get("theta_manager.log_threshold"), model_dtype=tdt)
        assert abs(float(loss) - float(ref_loss)) <= (1e-4 if tdt == torch.float32 else 2e-2) * abs(float(ref_loss))
        ropt.zero_grad()
        for k, p in ref.items():
            p.grad = grads[k].clone()
        ropt.step()
    new_sd = model.state_dict()
    # Adam's first steps move a parameter by about lr * sign(gradient) whatever the gradient's size, so
    # an element whose gradient is zero up to rounding may move either way: compare the displacement
    # as a whole (rel-L2), and element by element where the reference gradient is not negligible
    for k, p in ref.items():
        got = new_sd[k].float().cpu()
        moved = got - sd[k].float()
        want = p.detach() - sd[k].float()
        err = orc.rel_l2(moved, want)
        print(k, "displacement rel-L2", err)
        bound = 2e-2 if tdt == torch.float32 else 0.15
        if k.endswith("log_threshold") and tdt == torch.bfloat16:
            bound = 0.3      # a threshold whose tiny gradient changes sign with the rounding moves the other way
        assert err <= bound, (k, err)
        if tdt == torch.float32:
            g = grads[k]
            clear = g.abs() > 1e-3 * g.abs().max()
            assert torch.allclose(got[clear], p.detach()[clear], rtol=1e-4, atol=1e-4), k
    # the feature-major working copy was updated together with the parameters
    packed = model.decoder_module.packed()
    for slot, n in enumerate(names):
        assert torch.equal(packed[slot][:, :wl.d_model], new_sd[f"decoder_module.decoders.{n}.weight"].t())
    # and a forward after the steps runs on the new weights
    rec = model(inputs)
    assert all(torch.isfinite(r).all() for r in rec.values())


@pytest.mark.parametrize("shape", [(96, 200), (50, 77), (96, 192), (1028, 128), (128, 200)],
                         ids=["vector", "scalar", "whole-tiles", "tall", "padded-pitch"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_adam_kernels_match_torch_adam_on_given_gradients(dev, dtype, shape):
    # same gradients on both sides (zeros and tiny values included): the update itself, three steps
    from crosslayer_coding_amd import _native
    lib = _native.load()
    gen = torch.Generator().manual_seed(5)
    # the first two are not multiples of the 64 x 64 tile, (50, 77) is not a multiple of 4 either
    d, F = shape
    p0 = (torch.randn(d, F, generator=gen) * 0.1).to(dtype)
    ref = p0.float().clone().requires_grad_(True)
    ropt = torch.optim.Adam([ref], lr=3e-3, betas=(0.9, 0.999), eps=1e-8)
    w_ref = p0.to(dev).contiguous()
    w_packed = engine.alloc_packed(1, F, d, dtype, dev)[0]         # [F, pitch], pitch > d for the last shape
    engine.pack_decoder(w_ref, w_packed)
    flat = p0.to(dev).clone().view(-1)
    m = torch.zeros(F, d, device=dev); v = torch.zeros(F, d, device=dev)
    m2 = torch.zeros(d * F, device=dev); v2 = torch.zeros(d * F, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    for step in range(1, 4):
        g = torch.randn(d, F, generator=gen) * 10.0 ** float(torch.randint(-9, 0, (1,), generator=gen))
        g[torch.rand(d, F, generator=gen) < 0.3] = 0.0
        if dtype == torch.bfloat16:
            # the reference keeps fp32 master values; the kernel rounds the parameter each step
            with torch.no_grad():
                ref.copy_(ref.to(dtype).float())
        ropt.zero_grad(); ref.grad = g.clone(); ropt.step()
        gp = g.t().contiguous().to(dev)
        rc = lib.clt_adam_step_decoder(w_ref.data_ptr(), w_packed.data_ptr(), gp.data_ptr(), m.data_ptr(), v.data_ptr(),
                                       d, F, 3e-3, 0.9, 0.999, 1e-8, step, _native.dtype_code(dtype), stream)
        assert rc == 0
        gf = g.contiguous().view(-1).to(dev)
        rc = lib.clt_adam_step(flat.data_ptr(), gf.data_ptr(), m2.data_ptr(), v2.data_ptr(), d * F,
                               3e-3, 0.9, 0.999, 1e-8, step, _native.dtype_code(dtype), stream)
        assert rc == 0
    torch.cuda.synchronize()
    assert torch.equal(w_ref, w_packed[:, :d].t())
    assert float(w_packed[:, d:].abs().sum()) == 0.0               # the padding columns are left alone
    assert torch.equal(w_ref.view(-1), flat)
    want = ref.detach().to(dtype).float()
    tol = dict(rtol=1e-5, atol=1e-6) if dtype == torch.float32 else dict(rtol=1e-2, atol=1e-3)
    assert torch.allclose(w_ref.float().cpu(), want, **tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_adam_batched_entry_points_equal_the_single_ones(dev, dtype):
    # three decoder matrices and their biases in one launch each against one call per tensor: same bits
    import ctypes
    from crosslayer_coding_amd import _native
    lib = _native.load()
    gen = torch.Generator().manual_seed(11)
    n, d, F = 3, 96, 200
    stream = torch.cuda.current_stream().cuda_stream
    code = _native.dtype_code(dtype)
    w0 = [(torch.randn(d, F, generator=gen) * 0.1).to(dtype) for _ in range(n)]
    b0 = [(torch.randn(d, generator=gen) * 0.1).to(dtype) for _ in range(n)]
    g = (torch.randn(n, F, d, generator=gen) * 1e-2).to(dev)
    gb = (torch.randn(n, d, generator=gen) * 1e-2).to(dev)
    out = []
    for batched in (False, True):
        ws = [w.to(dev).contiguous() for w in w0]
        bs = [b.to(dev).contiguous() for b in b0]
        packed = torch.stack([w.t().contiguous() for w in ws]).contiguous()
        m = torch.zeros(n, F, d, device=dev); v = torch.zeros(n, F, d, device=dev)
        mb = torch.zeros(n, d, device=dev); vb = torch.zeros(n, d, device=dev)
        for step in (1, 2):
            if batched:
                ptrs = [w.data_ptr() for w in ws]
                host = (ctypes.c_void_p * n)(*ptrs)
                devp = torch.tensor(ptrs, dtype=torch.int64, device=dev)
                assert lib.clt_adam_step_decoders(devp.data_ptr(), ctypes.addressof(host), n, packed.data_ptr(), g.data_ptr(),
                                                  m.data_ptr(), v.data_ptr(), d, F, 3e-3, 0.9, 0.999, 1e-8, step, code, stream) == 0
                bp = torch.tensor([b.data_ptr() for b in bs], dtype=torch.int64, device=dev)
                assert lib.clt_adam_step_many(bp.data_ptr(), gb.data_ptr(), mb.data_ptr(), vb.data_ptr(), n, d,
                                              3e-3, 0.9, 0.999, 1e-8, step, code, stream) == 0
            else:
                for i in range(n):
                    assert lib.clt_adam_step_decoder(ws[i].data_ptr(), packed[i].data_ptr(), g[i].data_ptr(), m[i].data_ptr(),
                                                     v[i].data_ptr(), d, F, 3e-3, 0.9, 0.999, 1e-8, step, code, stream) == 0
                    assert lib.clt_adam_step(bs[i].data_ptr(), gb[i].data_ptr(), mb[i].data_ptr(), vb[i].data_ptr(), d,
                                             3e-3, 0.9, 0.999, 1e-8, step, code, stream) == 0
        torch.cuda.synchronize()
        out.append((torch.stack(ws).cpu(), packed.cpu(), torch.stack(bs).cpu(), m.cpu(), vb.cpu()))
    for a, b in zip(*out):
        assert torch.equal(a, b)
    assert torch.equal(out[1][0], out[1][1].transpose(1, 2))
    # bad arguments are refused before anything is launched
    assert lib.clt_adam_step_decoders(None, None, 1, None, None, None, None, d, F, 3e-3, 0.9, 0.999, 1e-8, 1, code, stream) != 0
    assert lib.clt_adam_step_many(None, None, None, None, 2, d, 3e-3, 0.9, 0.999, 1e-8, 1, code, stream) != 0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,F", [(300, 520), (1000, 256), (77, 250), (4100, 1032)],
                         ids=["vector", "vector-whole", "one-column-per-thread", "long-slices"])
@pytest.mark.parametrize("bandwidth", [1.0, 0.3, 0.25])
def test_threshold_gradient_reduction(dev, dtype, T, F, bandwidth):
    """clt_jumprelu_theta_grad against the reference's tensor arithmetic (clt/models/activations.py:196-199): every
    elementwise step in the model dtype, the column sums in fp32.  Both kernels behind the entry point (16 bytes of
    a row per thread, or one column per thread when a row is not whole 16-byte pieces), power-of-two and other
    bandwidths."""
    g = torch.Generator().manual_seed(T + F)
    x = (torch.randn(T, F, generator=g) * 0.7).to(dtype)
    go = torch.randn(T, F, generator=g).to(dtype)
    theta = torch.exp(0.4 * torch.randn(F, generator=g) - 0.5).to(dtype)
    near = torch.abs(x - theta) <= (bandwidth / 2.0)
    want = (go * ((-x / bandwidth) * near.type_as(x))).float().sum(0)
    got = torch.empty(F, dtype=torch.float32, device=dev)
    engine.jumprelu_theta_grad(x.to(dev), go.to(dev), theta.to(dev), bandwidth, got)
    scale = float(want.abs().max())
    assert float((got.cpu() - want).abs().max()) <= 2e-5 * scale + (1e-6 if dtype == torch.float32 else 0.0)
    assert int(near.sum()) > 0


@pytest.mark.parametrize("tying", ["none", "per_source", "per_target"])
@pytest.mark.parametrize("case", ["relu", "jumprelu-low-thresholds", "batchtopk-large-k"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_gradients_on_the_dense_route_at_high_density(dev, dtype, case, tying):
    """Far above the densities the survivor-list kernels are made for, forward and gradients take the reference's
    dense formulation on the matrix-core kernel (Decoder.dense_pairs_wanted).  Loss and every gradient against
    autograd through the oracle; one optimisation step equal to the step taken from the same gradients."""
    tdt = getattr(torch, dtype)
    fn = {"relu": "relu", "jumprelu-low-thresholds": "jumprelu", "batchtopk-large-k": "batchtopk"}[case]
    wl = BASE.scaled("dense-bw", num_layers=3, d_model=256, num_features=512, tokens=320, dtype=dtype, activation_fn=fn,
                     k=200 if fn == "batchtopk" else None, decoder_tying=tying)
    import crosslayer_coding_amd as cca
    x = synth.make_inputs(wl, "cpu")
    sd = synth.make_state_dict(wl, "cpu", inputs=x)
    g = torch.Generator().manual_seed(5)
    for k in list(sd):
        if k.endswith("bias_param"):
            sd[k] = (torch.randn(sd[k].shape, generator=g) * 0.05).to(sd[k].dtype)
            if case == "jumprelu-low-thresholds" and "encoder" in k:
                sd[k] = sd[k] + 2.0
    L = wl.num_layers
    tg = torch.Generator().manual_seed(6)
    targets = {l: torch.randn(wl.tokens, wl.d_model, generator=tg).to(tdt) for l in range(L)}

    def fresh():
        m = cca.CrossLayerTranscoder(wl.config(), None, dev)
        m.load_state_dict(sd)
        m.decoder_module.rate_override = (14.5e12, 1.0e14 if tdt == torch.float32 else 1.0e15)
        return m

    model = fresh()
    inputs = {l: x[l].to(dev) for l in range(L)}
    tdev = {l: t.to(dev) for l, t in targets.items()}
    calls = []
    real = model._raw_gradients_dense
    model._raw_gradients_dense = lambda *a, **kw: (calls.append(1), real(*a, **kw))[1]
    loss, grads = model.loss_and_gradients(inputs, tdev)
    assert calls, "the dense gradient route was not taken"
    if tying != "per_target":       # (decoders tied per target choose target by target in the forward)
        assert model.decoder_module.last_route["dense_targets"] == (0, L)
    acts = model.get_feature_activations(inputs)
    assert float((acts[0] != 0).float().mean()) > 0.2
    masks, theta, log_theta = None, None, None
    if fn == "jumprelu":
        theta = torch.exp(sd["theta_manager.log_threshold"].float()).to(tdt)
        log_theta = sd["theta_manager.log_threshold"]
    else:
        masks = {l: (a != 0).cpu() for l, a in acts.items()}
    names = synth.decoder_names(wl)
    ref_loss, ref = orc.mse_loss_and_gradients(
        {l: x[l] for l in range(L)}, targets,
        enc_w=[sd[f"encoder_module.encoders.{l}.weight"] for l in range(L)],
        enc_b=[sd[f"encoder_module.encoders.{l}.bias_param"] for l in range(L)],
        dec_w={n: sd[f"decoder_module.decoders.{n}.weight"] for n in names},
        dec_b={n: sd[f"decoder_module.decoders.{n}.bias_param"] for n in names},
        activation_fn=fn, num_layers=L, k=wl.k, theta=theta, masks=masks, tying=tying, log_threshold=log_theta,
        model_dtype=tdt)
    tol = TOL[tdt]
    assert abs(float(loss) - float(ref_loss)) <= max(tol, 1e-6) * abs(float(ref_loss)) * 10
    for name, gref in ref.items():
        err = orc.rel_l2(grads[name].float().cpu(), gref)
        bound = tol * (5 if tdt == torch.bfloat16 else 1)
        if name.endswith("log_threshold"):
            bound = 1e-3 if tdt == torch.float32 else 1e-1
        assert err <= bound, (name, err)
    # threshold activations: once the density of the shape is known no survivor list is made; same gradients
    torch.cuda.synchronize()
    loss2, grads2 = model.loss_and_gradients(inputs, tdev)
    assert model.decoder_module.last_route.get("survivor_list", True) == (fn == "batchtopk" or tying == "per_target")
    assert float(loss2) == float(loss)
    for name in grads:
        assert torch.equal(grads2[name], grads[name]), name
    # the same route under training_step (an optimiser that would otherwise fuse the decoder step) == stepping on
    # the gradients just checked
    a, b = fresh(), fresh()
    oa, ob = cca.CLTAdam(a, lr=1e-3), cca.CLTAdam(b, lr=1e-3)
    ob.fuse_decoder_step = False
    la = a.training_step(inputs, tdev, oa)
    lb = b.training_step(inputs, tdev, ob)
    assert float(la) == float(lb)
    sa, sb = a.state_dict(), b.state_dict()
    for k in sa:
        assert torch.equal(sa[k], sb[k]), k
    assert not torch.equal(sa["encoder_module.encoders.0.weight"].cpu(), sd["encoder_module.encoders.0.weight"])


@pytest.mark.parametrize("tying", ["none", "per_target"])
def test_models_wider_than_the_list_kernels_train_through_the_dense_formulation(dev, tying):
    """d_model = 4352 > 4096: the gradient kernels that walk survivor lists do not hold such rows; loss and gradients
    come from the dense formulation at any density, against autograd through the oracle.  Decoders tied per target
    of that width also decode through the dense products (no gather kernel of that tying holds the rows)."""
    wl = BASE.scaled("wide", num_layers=2, d_model=4352, num_features=512, tokens=300, k=8, dtype="bfloat16", decoder_tying=tying)
    model, sd, x, targets = build(wl, dev)
    L = wl.num_layers
    inputs = {l: x[l].to(dev) for l in range(L)}
    calls = []
    real = model._raw_gradients_dense
    model._raw_gradients_dense = lambda *a, **kw: (calls.append(1), real(*a, **kw))[1]
    loss, grads = model.loss_and_gradients(inputs, {l: t.to(dev) for l, t in targets.items()})
    assert calls
    if tying == "per_target":
        assert model.decoder_module.last_route["dense_targets"] == (0, L)
    masks = {l: (a != 0).cpu() for l, a in model.get_feature_activations(inputs).items()}
    names = synth.decoder_names(wl)
    ref_loss, ref = orc.mse_loss_and_gradients(
        {l: x[l] for l in range(L)}, targets,
        enc_w=[sd[f"encoder_module.encoders.{l}.weight"] for l in range(L)],
        enc_b=[sd[f"encoder_module.encoders.{l}.bias_param"] for l in range(L)],
        dec_w={n: sd[f"decoder_module.decoders.{n}.weight"] for n in names},
        dec_b={n: sd[f"decoder_module.decoders.{n}.bias_param"] for n in names},
        activation_fn="batchtopk", num_layers=L, k=wl.k, theta=None, masks=masks, tying=tying, log_threshold=None,
        model_dtype=torch.bfloat16)
    assert abs(float(loss) - float(ref_loss)) <= 0.1 * abs(float(ref_loss)) * TOL[torch.bfloat16] * 10
    for name, gref in ref.items():
        assert orc.rel_l2(grads[name].float().cpu(), gref) <= 5 * TOL[torch.bfloat16], name
