"""Activation-store feed on the device against the oracle's restatement of the reference's batch
assembly (clt/training/data/manifest_activation_store.py:776-958): bit-exact rows, order and
normalisation for resident chunks (HBM, pinned host memory) and for fetched wire-format slices."""
import math

import numpy as np
import pytest
import torch

import crosslayer_coding_amd as cca
from crosslayer_coding_amd import synth
from oracle import clt_oracle as orc

pytestmark = pytest.mark.gpu

DT = {"float32": torch.float32, "bfloat16": torch.bfloat16, "float16": torch.float16}


def make_chunks(L, d, sizes, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    return {c: (torch.randn(L, 2, n, d, generator=g) * 3 + 1).to(dtype) for c, n in enumerate(sizes)}


def wire(chunks):
    def fetch(chunk_id, sorted_rows):
        sel = chunks[chunk_id][:, :, torch.as_tensor(np.asarray(sorted_rows, dtype=np.int64)), :].contiguous()
        return sel.view(torch.uint8).numpy().tobytes()
    return fetch


def stats_json(L, d, seed):
    g = torch.Generator().manual_seed(seed)
    out = {}
    for l in range(L):
        out[str(l)] = {k: {"mean": torch.randn(d, generator=g).tolist(), "std": (torch.rand(d, generator=g) + 0.3).tolist()}
                       for k in ("inputs", "targets")}
    return out


def oracle_tables(js, L):
    t = {k: {} for k in ("mean_in", "std_in", "mean_tg", "std_tg")}
    for l in range(L):
        t["mean_in"][l] = torch.tensor(js[str(l)]["inputs"]["mean"]).unsqueeze(0)
        t["std_in"][l] = (torch.tensor(js[str(l)]["inputs"]["std"]) + 1e-6).unsqueeze(0)
        t["mean_tg"][l] = torch.tensor(js[str(l)]["targets"]["mean"]).unsqueeze(0)
        t["std_tg"][l] = (torch.tensor(js[str(l)]["targets"]["std"]) + 1e-6).unsqueeze(0)
    return t


def same_bits(a, b):
    a, b = a.cpu().contiguous(), b.contiguous()
    assert a.dtype == b.dtype and a.shape == b.shape
    return torch.equal(a.view(torch.uint8), b.view(torch.uint8))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16", "float16"])
@pytest.mark.parametrize("method", ["none", "mean_std", "sqrt_d_model"])
@pytest.mark.parametrize("source", ["device", "pinned", "wire"])
def test_batches_equal_the_oracle_bit_for_bit(dev, dtype, method, source):
    L, d = 3, 72
    tdt = DT[dtype]
    out_dt = tdt
    chunks = make_chunks(L, d, [40, 17, 64], tdt, seed=3)
    js = stats_json(L, d, seed=4) if method == "mean_std" else None
    feed = cca.DeviceActivationFeed(L, d, dtype=dtype, device=dev, normalization_method=method, norm_stats=js, out_dtype=out_dt)
    if source != "wire":
        for c, t in chunks.items():
            feed.add_chunk(c, t if c != 1 else t.view(torch.uint8).numpy().tobytes(), rows=t.shape[2], where=source)
    rng = np.random.RandomState(9)
    manifest = np.array([(c, r) for c, t in chunks.items() for r in range(t.shape[2])], dtype=np.uint32)
    for batch in range(3):       # several batches: the pinned staging buffers take turns
        idxs = manifest[rng.permutation(len(manifest))[:50]]
        ins, tgs = feed.parse_batch(idxs, wire(chunks) if source == "wire" else None)
        tabs = oracle_tables(js, L) if js else {}
        # the oracle works in the store dtype, as the reference does
        want_in, want_tg = orc.store_parse_batch(idxs, wire(chunks), num_layers=L, d_model=d, dtype=tdt, method=method, **tabs)
        for l in range(L):
            assert same_bits(ins[l], want_in[l]), (batch, l)
            assert same_bits(tgs[l], want_tg[l]), (batch, l)


def test_odd_width_takes_the_scalar_kernel(dev):
    L, d = 2, 13
    chunks = make_chunks(L, d, [9, 11], torch.float32, seed=5)
    js = stats_json(L, d, seed=6)
    feed = cca.DeviceActivationFeed(L, d, dtype="float32", device=dev, normalization_method="mean_std", norm_stats=js)
    feed.add_chunk(0, chunks[0])
    idxs = np.array([(1, 10), (0, 8), (1, 0), (0, 0), (0, 8)], dtype=np.uint32)     # a row may repeat
    ins, tgs = feed.parse_batch(idxs, wire(chunks))                                 # chunk 0 resident, chunk 1 fetched
    want_in, want_tg = orc.store_parse_batch(idxs, wire(chunks), num_layers=L, d_model=d, dtype=torch.float32,
                                             method="mean_std", **oracle_tables(js, L))
    for l in range(L):
        assert same_bits(ins[l], want_in[l]) and same_bits(tgs[l], want_tg[l])


def test_errors_and_empty_batches(dev):
    L, d = 2, 8
    chunks = make_chunks(L, d, [6], torch.float32, seed=1)
    feed = cca.DeviceActivationFeed(L, d, dtype="float32", device=dev)
    feed.add_chunk(0, chunks[0])
    with pytest.raises(IndexError):
        feed.parse_batch(np.array([(0, 6)], dtype=np.uint32))
    with pytest.raises(RuntimeError):
        feed.parse_batch(np.array([(3, 0)], dtype=np.uint32))                       # unknown chunk, nothing to fetch with
    with pytest.raises(ValueError):
        feed.parse_batch(np.array([(3, 0)], dtype=np.uint32), lambda c, rows: b"123")   # wrong byte count
    ins, tgs = feed.parse_batch(np.zeros((0, 2), dtype=np.uint32))
    assert ins[0].shape == (0, d) and tgs[1].shape == (0, d)
    # the C entry refuses memory the device cannot reach instead of reading it
    from crosslayer_coding_amd import _native as nat
    host = torch.zeros(L, 2, 6, d)
    idx = torch.zeros(1, dtype=torch.int32, device=dev)
    out = torch.empty(L, 1, d, device=dev)
    code = nat.load().clt_feed_gather(host.data_ptr(), 0, 6, 2 * 6 * d, 6 * d, idx.data_ptr(), 1, d, L, 0, None, None, None, None,
                                      1.0, out.data_ptr(), out.data_ptr(), 0, 1, 0, torch.cuda.current_stream().cuda_stream)
    assert code != 0
    # an index outside the chunk handed straight to the C entry gives a NaN row, the rest is untouched
    src = chunks[0].to(dev)
    idx = torch.tensor([2, 99, -1, 5], dtype=torch.int32, device=dev)
    x = torch.zeros(L, 4, d, device=dev)
    t = torch.zeros(L, 4, d, device=dev)
    code = nat.load().clt_feed_gather(src.data_ptr(), 0, 6, 2 * 6 * d, 6 * d, idx.data_ptr(), 4, d, L, 0, None, None, None, None,
                                      1.0, x.data_ptr(), t.data_ptr(), 0, 4, 0, torch.cuda.current_stream().cuda_stream)
    assert code == 0
    assert torch.isnan(x[:, 1:3]).all() and torch.equal(x[:, 0].cpu(), chunks[0][:, 0, 2]) and torch.equal(t[:, 3].cpu(), chunks[0][:, 1, 5])


def test_a_fed_batch_runs_through_the_model_without_a_copy(dev):
    wl = synth.WORKLOADS["c0"].scaled("feed", dtype="bfloat16", num_layers=3, d_model=128, num_features=512, tokens=256, k=8)
    model, _, _ = synth.build_model(wl, dev)
    model.eval()
    chunks = make_chunks(3, 128, [300], torch.bfloat16, seed=2)
    feed = cca.DeviceActivationFeed(3, 128, dtype="bfloat16", device=dev, normalization_method="sqrt_d_model")
    feed.add_chunk(0, chunks[0])
    idxs = np.array([(0, r) for r in np.random.RandomState(0).permutation(300)[:256]], dtype=np.uint32)
    ins, tgs = feed.parse_batch(idxs)
    prep = model.encoder_module.prepare_slab(ins)
    assert prep[1].data_ptr() == ins[0].data_ptr()          # the slab is used where the feed wrote it
    rec = model(ins)
    want = {l: (chunks[0][l, 0, idxs[:, 1].astype(np.int64)].float() * math.sqrt(128)).to(torch.bfloat16) for l in range(3)}
    assert all(same_bits(ins[l], want[l]) for l in range(3))
    assert all(torch.isfinite(rec[l]).all() for l in range(3))
