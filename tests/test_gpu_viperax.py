"""Viperax on the GPU against the plain implementation (tests/plain_viperax.py): each new kernel
alone; the attention kernels with sinks, with a key that stands out far back, at page borders and
just inside and just outside a window, for prompt portions and for single tokens; whole prompts
against token-by-token decoding, portions down to two tokens and mixed batches with pages and
request slots used again, in 32-bit and bfloat16; greedy generation through LLMEngine."""

import json
import math

import numpy as np
import pytest
import torch

import helpers
import plain_viperax as V
import test_gpu_kernels as K
import viperax_cases as cases
from mini_gpt_inference_amd import EngineConfig, SamplingParams
from mini_gpt_inference_amd.engine.llm_engine import LLMEngine
from mini_gpt_inference_amd.engine.replay import TraceReplayer
from mini_gpt_inference_amd.ops import kernels

pytestmark = pytest.mark.gpu
DEV = "cuda"
TDT = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def _rnd(g, *shape, dtype="float32", scale=1.0):
    return (torch.randn(*shape, generator=g) * scale).to(TDT[dtype])


# ---------------------------------------------------------------- kernels, one at a time
@pytest.mark.parametrize("streams,width,n", [(1, 40, 3), (2, 64, 70), (3, 192, 9), (8, 24, 5)])
def test_streams_read_and_write(streams, width, n):
    g = torch.Generator().manual_seed(streams)
    x = _rnd(g, n + 2, streams * width)
    coef, out, mix = _rnd(g, streams), _rnd(g, streams), _rnd(g, streams, streams)
    y = _rnd(g, n + 2, width)
    xd = x.to(DEV)
    u = torch.full((n + 2, width), 9.0, device=DEV)
    z = torch.full((n + 2, width), 9.0, device=DEV)
    kernels.streams_read(xd, coef.to(DEV), u, n, streams, zero=z)
    as_streams = x[:n].view(n, streams, width).transpose(0, 1)
    helpers.assert_close(u[:n], V.hyper_read(as_streams, coef), "float32", "read")
    assert (z[:n] == 0).all() and (z[n:] == 9.0).all() and (u[n:] == 9.0).all()
    kernels.streams_read(xd, None, u, n, streams)
    helpers.assert_close(u[:n], as_streams.sum(0), "float32", "sum")
    kernels.streams_write(xd, mix.to(DEV), out.to(DEV), y.to(DEV), n, streams)
    want = V.hyper_write(as_streams, mix, out, y[:n]).transpose(0, 1).reshape(n, streams * width)
    helpers.assert_close(xd[:n], want, "float32", "write")
    assert torch.equal(xd[n:].cpu(), x[n:])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("streams,width,n", [(1, 40, 3), (2, 64, 70), (3, 192, 9), (4, 4100, 2), (2, 5000, 3),
                                             (2, 4500, 130), (8, 1024, 8), (3, 17000, 2)])
def test_streams_write_read_and_norm_in_one_pass(dtype, streams, width, n):
    g = torch.Generator().manual_seed(streams + width)
    x = _rnd(g, n + 1, streams * width, scale=3.0)
    coef, out, mix = _rnd(g, streams), _rnd(g, streams), _rnd(g, streams, streams)
    gain, beta = _rnd(g, width) + 1.0, _rnd(g, width)
    y = _rnd(g, n + 1, width)
    as_streams = x[:n].view(n, streams, width).transpose(0, 1)
    for pending in (False, True):
        xd, yd = x.to(DEV), y.to(DEV)
        u = torch.zeros(n + 1, width, device=DEV)
        h = torch.full((n + 1, width), 5.0, dtype=TDT[dtype], device=DEV)
        kernels.streams_step(xd, (mix.to(DEV), out.to(DEV), yd) if pending else None, coef.to(DEV), u, gain.to(DEV),
                             beta.to(DEV) if pending else None, 1e-5, h, n, streams, zero=yd)
        new = V.hyper_write(as_streams, mix, out, y[:n]) if pending else as_streams
        helpers.assert_close(xd[:n], new.transpose(0, 1).reshape(n, streams * width), "float32", "streams")
        want_u = V.hyper_read(new, coef)
        helpers.assert_close(u[:n], want_u, "float32", "u")
        want_h = V.layer_norm(want_u, gain, 1e-5) + (beta if pending else 0.0)
        helpers.assert_close(h[:n], want_h, dtype, "normed")
        assert (yd[:n] == 0).all() and torch.equal(yd[n:].cpu(), y[n:]) and (h[n:] == 5.0).all()
        assert torch.equal(xd[n:].cpu(), x[n:])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_embed_scaled_fills_every_stream(dtype):
    g = torch.Generator().manual_seed(1)
    table = _rnd(g, 50, 36, dtype=dtype)
    ids = torch.tensor([3, 49, 0, 3, 17], dtype=torch.int32)
    x = torch.zeros(5, 3 * 36, device=DEV)
    kernels.embed_scaled(ids.to(DEV), table.to(DEV), x, 5, 2.5, copies=3)
    want = (table[ids.long()].float() * 2.5).repeat(1, 3)
    assert torch.equal(x.cpu(), want)


@pytest.mark.parametrize("cap", [0.0, 7.0])
def test_scale_softcap(cap):
    g = torch.Generator().manual_seed(2)
    logits = _rnd(g, 4, 103, scale=20.0)
    buf = torch.zeros(4, 104, device=DEV)[:, :103]
    for fast, dtype in ((False, "float32"), (True, "bfloat16")):
        buf.copy_(logits)
        kernels.scale_softcap(buf, 3, 0.5, cap, fast=fast)
        want = logits[:3] * 0.5
        if cap:
            want = cap * torch.tanh(want / cap)
        helpers.assert_close(buf[:3], want, dtype, "softcap")
        assert torch.equal(buf[3].cpu(), logits[3])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("rank,page", [(24, 4), (96, 16), (200, 8)])
def test_rms_norm_store(dtype, rank, page):
    g = torch.Generator().manual_seed(rank)
    n = 7
    src = _rnd(g, n, 50 + rank, dtype=dtype, scale=3.0)
    gain = _rnd(g, rank) + 1.0
    pool = torch.full((5, 1, page, rank), 7.0, dtype=TDT[dtype], device=DEV)
    slots = torch.tensor([page + 1, 0, -1, 4 * page + page - 1, 2 * page, 3, 2], dtype=torch.int32)
    kernels.rms_norm_store(src.to(DEV)[:, 50:], gain.to(DEV), 1e-3, pool, slots.to(DEV), n)
    want = V.rms_norm(src[:, 50:].float(), gain, 1e-3)
    flat = pool.view(-1, rank)
    for i, s in enumerate(slots.tolist()):
        if s >= 0:
            helpers.assert_close(flat[s], want[i], dtype, f"token {i}")
    written = {s for s in slots.tolist() if s >= 0}
    assert all((flat[s] == 7.0).all() for s in range(flat.shape[0]) if s not in written)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("n,heads,n_out,k", [(1, 1, 40, 24), (19, 3, 16, 96), (70, 4, 96, 64), (5, 2, 7, 130),
                                             (200, 5, 72, 40), (65, 2, 128, 128)])
def test_heads_linear_with_and_without_gate(dtype, n, heads, n_out, k):
    g = torch.Generator().manual_seed(n)
    a = _rnd(g, n, heads * k + 8, dtype=dtype)
    w = _rnd(g, heads, n_out, k, dtype=dtype, scale=k ** -0.5)
    gate = _rnd(g, n, heads * n_out, dtype=dtype, scale=2.0)
    want = torch.einsum("nhk,hok->nho", a[:, :heads * k].float().view(n, heads, k), w.float()).reshape(n, -1)
    for use_gate in (False, True):
        out = torch.zeros(n, heads * n_out, dtype=TDT[dtype], device=DEV)
        kernels.heads_linear(a.to(DEV), w.to(DEV), out, n, gate=gate.to(DEV) if use_gate else None,
                             fast=dtype == "bfloat16")
        helpers.assert_close(out, want * torch.sigmoid(gate.float()) if use_gate else want, dtype, f"gate {use_gate}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_gated_unit(dtype):
    g = torch.Generator().manual_seed(3)
    z = _rnd(g, 9, 2 * 37, dtype=dtype, scale=3.0)
    act = torch.zeros(9, 37, dtype=TDT[dtype], device=DEV)
    kernels.gated_unit(z.to(DEV), act, 9, 37, fast=dtype == "bfloat16")
    helpers.assert_close(act, V.silu(z[:, :37].float()) * z[:, 37:].float(), dtype, "gated unit")


@pytest.mark.parametrize("dtype,tile,fast", [("float32", 16, False), ("bfloat16", 16, False), ("bfloat16", 64, True),
                                             ("float32", 64, False)])
@pytest.mark.parametrize("n,experts,top,width,hidden", [(1, 2, 1, 24, 8), (40, 5, 2, 64, 24), (300, 16, 1, 48, 40),
                                                        (7, 3, 3, 32, 16), (130, 4, 2, 100, 36), (130, 4, 2, 64, 256), (70, 3, 1, 512, 40)])
def test_experts_by_table(dtype, tile, fast, n, experts, top, width, hidden):
    """Route, both grouped products, the gated unit and the sum over a token's experts, against the
    plain loop; some tokens are padding (their request is -1) and an expert may get no token."""
    g = torch.Generator().manual_seed(n)
    vocab = 23
    table = torch.rand(vocab, experts, generator=g).argsort(dim=1)[:, :top].to(torch.int32)
    if experts > 2:
        table[table == 1] = 0 if top == 1 else table[table == 1]     # (top 1: expert 1 stays without tokens)
    ids = torch.randint(0, vocab, (n,), generator=g, dtype=torch.int32)
    q_req = torch.zeros(n, dtype=torch.int32)
    if n > 3:
        q_req[-2:] = -1
    h = _rnd(g, n, width, dtype=dtype)
    w_in = _rnd(g, experts, 2 * hidden, width, dtype=dtype, scale=width ** -0.5)
    w_down = _rnd(g, experts, width, hidden, dtype=dtype, scale=hidden ** -0.5)
    slots = kernels.expert_slots(n, top, experts, tile)
    st, sp = (torch.full((slots,), -7, dtype=torch.int32, device=DEV) for _ in range(2))
    te = torch.full((slots // tile,), -7, dtype=torch.int32, device=DEV)
    kernels.expert_route(ids.to(DEV), q_req.to(DEV), table.to(DEV), n, experts, st, sp, te, tile)
    z = torch.zeros(slots, 2 * hidden, dtype=TDT[dtype], device=DEV)
    kernels.grouped_linear(h.to(DEV), st, w_in.to(DEV), te, st, z, None, slots, tile, fast)
    act = torch.zeros(slots, hidden, dtype=TDT[dtype], device=DEV)
    kernels.gated_unit(z, act, slots, hidden, fast=dtype == "bfloat16")
    pair_out = torch.zeros(n * top, width, device=DEV)
    kernels.grouped_linear(act, None, w_down.to(DEV), te, st, pair_out, sp, slots, tile, fast)
    y = torch.ones(n, width, device=DEV)
    kernels.expert_combine(pair_out, y, n, top, 1.0 / top)
    live = [i for i in range(n) if q_req[i] >= 0]
    # every live pair has exactly one slot, in a tile of its expert
    st_h, sp_h, te_h = st.cpu(), sp.cpu(), te.cpu()
    used = [(int(sp_h[s]), int(te_h[s // tile])) for s in range(slots) if st_h[s] >= 0]
    assert sorted(p for p, _ in used) == sorted(i * top + j for i in live for j in range(top))
    assert all(e == int(table[ids[p // top], p % top]) for p, e in used)
    exp = [(w_in[e, :hidden].float(), w_in[e, hidden:].float(), w_down[e].float()) for e in range(experts)]
    want = 1.0 + V.table_moe(h.float(), ids.tolist(), table.long(), exp, None)
    helpers.assert_close(y[live], want[live], dtype, "experts")


@pytest.mark.parametrize("n,experts,top,width,hidden", [(700, 6, 2, 64, 96), (130, 4, 2, 64, 256), (1500, 8, 2, 128, 64),
                                                        (40, 3, 1, 32, 16)])
def test_experts_through_the_tiled_kernel(n, experts, top, width, hidden):
    """The same with every expert's run padded to tiles of 256 slots: rows copied into the experts'
    order, the dense layers' tiled MFMA kernel with a matrix per tile, and the sum through the
    pairs' slots."""
    g = torch.Generator().manual_seed(n)
    vocab, tile = 31, 256
    table = torch.rand(vocab, experts, generator=g).argsort(dim=1)[:, :top].to(torch.int32)
    ids = torch.randint(0, vocab, (n,), generator=g, dtype=torch.int32)
    q_req = torch.zeros(n, dtype=torch.int32)
    q_req[-3:] = -1
    h = _rnd(g, n, width, dtype="bfloat16")
    w_in = _rnd(g, experts, 2 * hidden, width, dtype="bfloat16", scale=width ** -0.5)
    w_down = _rnd(g, experts, width, hidden, dtype="bfloat16", scale=hidden ** -0.5)
    slots = kernels.expert_slots(n, top, experts, tile)
    st, sp = (torch.full((slots,), -7, dtype=torch.int32, device=DEV) for _ in range(2))
    ps = torch.full((n * top,), -7, dtype=torch.int32, device=DEV)
    te = torch.full((slots // tile,), -7, dtype=torch.int32, device=DEV)
    kernels.expert_route(ids.to(DEV), q_req.to(DEV), table.to(DEV), n, experts, st, sp, te, tile, pair_slot=ps)
    rows = torch.full((slots, width), float("nan"), dtype=torch.bfloat16, device=DEV)
    assert kernels.gather_rows(h.to(DEV), st, rows, slots)
    z = torch.full((slots, 2 * hidden), float("nan"), dtype=torch.bfloat16, device=DEV)
    assert kernels.grouped_linear_tiled(rows, w_in.to(DEV), te, st, z, slots)
    act = torch.zeros(slots, hidden, dtype=torch.bfloat16, device=DEV)
    kernels.gated_unit(z, act, slots, hidden, fast=True)
    out = torch.full((slots, width), float("nan"), device=DEV)
    assert kernels.grouped_linear_tiled(act, w_down.to(DEV), te, st, out, slots)
    y = torch.ones(n, width, device=DEV)
    kernels.expert_combine(out, y, n, top, 1.0 / top, pair_slot=ps, q_req=q_req.to(DEV))
    live = list(range(n - 3))
    st_h, sp_h, ps_h = st.cpu(), sp.cpu(), ps.cpu()
    assert all(int(sp_h[int(ps_h[p])]) == p and int(st_h[int(ps_h[p])]) == p // top for i in live for p in
               range(i * top, (i + 1) * top))
    exp = [(w_in[e, :hidden].float(), w_in[e, hidden:].float(), w_down[e].float()) for e in range(experts)]
    want = 1.0 + V.table_moe(h.float(), ids.tolist(), table.long(), exp, None)
    helpers.assert_close(y[live], want[live], "bfloat16", "experts, tiled")
    assert (y[n - 3:] == 1.0).all(), "a padded token's row was touched"


# ---------------------------------------------------------------- attention with sinks, kernel by kernel
def _sink_want(c, sinks, scale, window):
    outs = []
    for r, (s, ql) in enumerate(zip(c.seq_lens, c.q_lens)):
        rep = c.h // c.hk
        k = c.k[r].double().repeat_interleave(rep, dim=1)
        v = c.v[r].double().repeat_interleave(rep, dim=1)
        q = torch.zeros(s, c.h, c.d, dtype=torch.float64)
        q[s - ql:] = c.q[r].double()
        outs.append(V.sink_attention(q, k, v, sinks.double(), scale, window)[s - ql:].reshape(ql, -1))
    return torch.cat(outs)


# (seq_lens, q_lens, heads, kv heads, head size, page size, window, spikes as (request, query, key, head)).
# Spiked keys: far back among hundreds; the last slot of a page and the first of the next; the
# first key of a sequence; with a window w, position p - w + 1 (just inside) and p - w (just
# outside: the output must not be that key's value).
SINK_CASES = [
    dict(seq_lens=[300, 40], q_lens=[1, 1], h=4, hk=1, d=32, page=16, window=0, spikes=[(0, 0, 2, 1), (1, 0, 15, 0), (1, 0, 16, 3)]),
    dict(seq_lens=[200, 90], q_lens=[64, 2], h=3, hk=1, d=96, page=8, window=50,
         spikes=[(0, 63, 150, 0), (0, 10, 97, 1), (1, 1, 40, 2), (0, 0, 136, 2)]),
    dict(seq_lens=[131, 9], q_lens=[131, 9], h=2, hk=2, d=64, page=4, window=0, spikes=[(0, 130, 0, 1), (0, 70, 3, 0), (1, 8, 4, 1)]),
    dict(seq_lens=[77, 150, 33], q_lens=[1, 1, 1], h=2, hk=1, d=40, page=16, window=33,
         spikes=[(0, 0, 44, 0), (1, 0, 117, 1), (2, 0, 0, 0)]),
    dict(seq_lens=[260], q_lens=[130], h=4, hk=1, d=128, page=32, window=129, spikes=[(0, 129, 131, 0), (0, 129, 130, 3)]),
    # few tiles of a small head size: the tile kernel's two wave groups each see keys of their own
    dict(seq_lens=[400], q_lens=[300], h=2, hk=1, d=32, page=16, window=0, spikes=[(0, 299, 5, 0), (0, 200, 240, 1)]),
    dict(seq_lens=[700, 300], q_lens=[290, 300], h=3, hk=1, d=64, page=16, window=300, spikes=[(0, 289, 400, 0), (1, 150, 140, 1)]),
]


@pytest.mark.parametrize("case", range(len(SINK_CASES)))
@pytest.mark.parametrize("kernel", ["generic-float32", "generic-bfloat16", "split-bfloat16", "splitfast-bfloat16",
                                    "prefill-bfloat16", "decode-bfloat16"])
def test_attention_with_sinks(kernel, case):
    name, dtype = kernel.split("-")
    spec = dict(SINK_CASES[case])
    window = spec.pop("window")
    c = K.PagedCase(**spec, dtype=dtype, seed=case, poison=True)
    scale = 1.0 / math.sqrt(c.d)
    # sinks around the spiked scores (9 d * scale) and far below them
    sinks = torch.tensor([9.0 * math.sqrt(c.d) * f for f in (1.0, -1.0, 0.9, 0.2)][:c.h])
    out = torch.full((c.n, c.h * c.d), float("nan"), dtype=TDT[dtype], device=DEV)
    args = (c.q_flat, out, c.kp, c.vp, c.bt, c.cu, c.sl, c.q_req, c.n, len(c.seq_lens), c.h, scale, window)
    sd = sinks.to(DEV)
    if name == "generic":
        kernels.paged_attention_generic(*args, fast_exp=dtype == "bfloat16", sinks=sd)
    elif name == "prefill":
        if c.d not in (32, 64, 96, 128):
            pytest.skip("the tile kernel takes head sizes 32, 64, 96, 128")
        assert kernels.prefill_attention_bf16(c.q_flat, out, c.kp, c.vp, c.bt, c.cu, c.sl, len(c.seq_lens),
                                              max(c.q_lens), c.h, scale, window, sinks=sd)
    elif name == "decode":
        if c.d not in (16, 32, 64, 128) or any(q != 1 for q in c.q_lens):
            pytest.skip("single tokens with head sizes 16, 32, 64, 128")
        positions = K.i32([s - 1 for s in c.seq_lens])
        assert kernels.paged_attention_decode_bf16(c.q_flat, out, c.kp, c.vp, c.bt, positions, c.q_req, c.n, c.h,
                                                   scale, window, identity=True, sinks=sd)
    else:
        if name == "splitfast" and c.d not in (16, 32, 64, 128):
            pytest.skip("the wide-load variant takes head sizes 16, 32, 64, 128")
        assert kernels.paged_attention_split_bf16(*args, fast=name == "splitfast", sinks=sd)
    want = _sink_want(c, sinks, scale, window)
    helpers.assert_close(out, want, dtype, f"{kernel} case {case}")
    # the spikes did what they were made for: inside the reach the output is (nearly) the key's value
    # where no sink competes, outside it is not
    offsets = np.concatenate([[0], np.cumsum(c.q_lens)])
    for r, qi, key, head in spec["spikes"]:
        pos = c.seq_lens[r] - c.q_lens[r] + qi
        row = want[offsets[r] + qi, head * c.d:(head + 1) * c.d]
        value = c.v[r][key, head // (c.h // c.hk)].double()
        inside = window == 0 or pos - key < window
        if not inside:
            assert (row - value).abs().max() > 0.1, "a key outside the window must not be seen"
        elif float(sinks[head]) < 0:
            assert (row - value).abs().max() < 0.05


# ---------------------------------------------------------------- the model through the step function
LENGTHS = {"P": [5, 70, 23, 41, 2, 64, 37], "Q": [1, 9, 33, 17, 50], "R": [40, 3, 64, 21], "S": [75, 12, 30, 6, 49]}
_folders, _plain = {}, {}


def _folder(tmp_path_factory, name):
    if name not in _folders:
        _folders[name] = cases.write_model(str(tmp_path_factory.mktemp("viperax") / name), name)
    return _folders[name]


def _requests(name):
    rng = np.random.default_rng(len(name) + ord(name[0]))
    return {f"r{i}": helpers.random_ids(rng, cases.RAW[name]["vocab"], n) for i, n in enumerate(LENGTHS[name])}


def _plain_logits(folder, name):
    if name not in _plain:
        cfg, w = V.read_model_folder(folder)
        _plain[name] = {rid: V.forward(cfg, w, ids)[0].numpy() for rid, ids in _requests(name).items()}
    return _plain[name]


def _row_errors(got, want):
    """Per position: root mean square over the vocabulary of the difference, its mean taken off."""
    d = np.asarray(got, dtype=np.float64) - np.asarray(want, dtype=np.float64)
    d = d - d.mean(axis=1, keepdims=True)
    return np.sqrt((d * d).mean(axis=1))


def _rounded_twin(cfg, w, ids):
    """The plain implementation with every matrix product rounded to bfloat16: what rounding alone does."""
    V.ROUNDING = torch.bfloat16
    try:
        return V.forward(cfg, w, ids)[0].numpy()
    finally:
        V.ROUNDING = None


_twin = {}


def _assert_within_rounding(folder, name, rid, ids, got, want, what):
    """bfloat16: a position's error may be three times what rounding alone causes at the request's
    worst position, and the request's mean error three times the mean of that."""
    assert np.isfinite(got).all(), f"{what}: non-finite logits"
    key = (name, rid, len(ids))
    if key not in _twin:
        cfg, w = V.read_model_folder(folder)
        _twin[key] = _row_errors(_rounded_twin(cfg, w, ids), want)
    noise, err = _twin[key], _row_errors(got, want)
    assert err.max() <= 3.0 * noise.max(), f"{what}: worst position {err.max():.3e} > 3 * {noise.max():.3e}"
    assert err.mean() <= 3.0 * noise.mean(), f"{what}: mean {err.mean():.3e} > 3 * {noise.mean():.3e}"


@pytest.mark.parametrize("page_size", [16, 4])
@pytest.mark.parametrize("way", ["whole", "tail", "portions", "mixed"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(cases.RAW))
def test_every_way_of_cutting_matches_the_plain_implementation(tmp_path_factory, name, dtype, way, page_size):
    folder = _folder(tmp_path_factory, name)
    reqs = _requests(name)
    want = _plain_logits(folder, name)
    plan = helpers.PLANS[way](reqs, np.random.default_rng(5))
    # the pool holds just what the live requests need and starts as NaN; four request slots
    replayer = TraceReplayer(folder, dtype, plan.tight_tokens(page_size), page_size=page_size, max_live=4, poison=True)
    got = plan.assemble(helpers.run_plan_in_process(replayer, plan), {r: len(t) for r, t in reqs.items()},
                        cases.RAW[name]["vocab"])
    for rid in reqs:
        if dtype == "float32":
            helpers.assert_close(got[rid], want[rid], dtype, f"{name} {dtype} {way} {rid}")
        else:
            _assert_within_rounding(folder, name, rid, reqs[rid], got[rid], want[rid], f"{name} {way} {rid}")
    assert replayer.cache.check() == 0 and not replayer.live
    assert all(replayer.cache.num_free_pages(g) == replayer.num_pages for g in range(len(replayer.cache.groups)))


@pytest.mark.parametrize("seed", range(8))
def test_random_configurations(tmp_path, seed):
    """Configurations drawn at random (tests/viperax_cases.py: random_raw), five requests of lengths
    1 to 200 each, whole, in portions and mixed, in both dtypes.  bfloat16: a position may be one and
    a half times over three times what rounding alone does, the mean may not."""
    rng = np.random.default_rng(1000 + seed)
    raw = cases.random_raw(rng)
    folder = cases.write_raw_model(str(tmp_path / "m"), raw, seed)
    cfg, w = V.read_model_folder(folder)
    lens = [int(x) for x in rng.choice([1, 2, 5, 17, 33, 64, 70, 97, 130, 200], size=5)]
    reqs = {f"r{i}": helpers.random_ids(rng, raw["vocab"], n) for i, n in enumerate(lens)}
    want = {rid: V.forward(cfg, w, ids)[0].numpy() for rid, ids in reqs.items()}
    noise = {rid: _row_errors(_rounded_twin(cfg, w, ids), want[rid]) for rid, ids in reqs.items()}
    for dtype in ("float32", "bfloat16"):
        for way in ("whole", "portions", "mixed"):
            plan = helpers.PLANS[way](reqs, np.random.default_rng(5))
            replayer = TraceReplayer(folder, dtype, plan.tight_tokens(16), page_size=16, max_live=4, poison=True)
            got = plan.assemble(helpers.run_plan_in_process(replayer, plan), {r: len(t) for r, t in reqs.items()},
                                raw["vocab"])
            for rid in reqs:
                what = f"seed {seed} {dtype} {way} {rid} ({json.dumps(raw)})"
                if dtype == "float32":
                    helpers.assert_close(got[rid], want[rid], dtype, what)
                    continue
                assert np.isfinite(got[rid]).all(), what
                err = _row_errors(got[rid], want[rid])
                assert err.max() <= 4.5 * noise[rid].max() and err.mean() <= 3.0 * noise[rid].mean(), \
                    f"{err.max():.3e} / {noise[rid].max():.3e}, mean {err.mean():.3e} / {noise[rid].mean():.3e}: {what}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_past_every_window(tmp_path_factory, dtype):
    """Three tokens of prompt, then 120 tokens one by one: the windows of 9, 20 and 33 pass over
    decoded tokens only, and the pages behind them are given back on the way."""
    folder = _folder(tmp_path_factory, "P")
    rng = np.random.default_rng(9)
    ids = helpers.random_ids(rng, cases.RAW["P"]["vocab"], 123)
    cfg, w = V.read_model_folder(folder)
    want = V.forward(cfg, w, ids)[0].numpy()
    plan = helpers.plan_tail({"a": ids}, tail=120)
    replayer = TraceReplayer(folder, dtype, 128, page_size=4, max_live=4, poison=True)
    got = plan.assemble(helpers.run_plan_in_process(replayer, plan), {"a": len(ids)}, cases.RAW["P"]["vocab"])
    if dtype == "float32":
        helpers.assert_close(got["a"], want, dtype, "long decoding")
    else:
        _assert_within_rounding(folder, "P", "long", ids, got["a"], want, "long decoding")


def test_a_long_portion_takes_the_tiled_experts(tmp_path_factory, monkeypatch):
    """A portion of 300 tokens with two experts each is beyond the bound from which the experts'
    products go through the tiled kernel; the same prompt in short portions stays below it."""
    folder = _folder(tmp_path_factory, "P")
    ids = helpers.random_ids(np.random.default_rng(21), cases.RAW["P"]["vocab"], 300)
    cfg, w = V.read_model_folder(folder)
    want = V.forward(cfg, w, ids)[0].numpy()
    calls = []
    tiled = kernels.grouped_linear_tiled
    monkeypatch.setattr(kernels, "grouped_linear_tiled", lambda *a, **k: calls.append(1) or tiled(*a, **k))
    for cut in (300, 60):
        plan = helpers.TracePlan()
        for at in range(0, 300, cut):
            plan.add_step([("a", ids[at:at + cut], 300)], end=["a"] if at + cut >= 300 else [])
        replayer = TraceReplayer(folder, "bfloat16", 320, page_size=16, max_live=4, poison=True)
        before = len(calls)
        got = plan.assemble(helpers.run_plan_in_process(replayer, plan), {"a": 300}, cases.RAW["P"]["vocab"])
        assert (len(calls) > before) == (cut == 300)
        _assert_within_rounding(folder, "P", "tiled", ids, got["a"], want, f"portions of {cut}")


def test_the_sink_and_the_far_latents_matter(tmp_path_factory, tmp_path):
    """The test models are made so that leaving out a sink, or a window's last key, shows: the plain
    logits move by far more than the tolerance when either is changed."""
    folder = _folder(tmp_path_factory, "P")
    cfg, w = V.read_model_folder(folder)
    ids = _requests("P")["r1"]
    base = V.forward(cfg, w, ids)[0]
    w2 = dict(w)
    w2["l0.mix.sink"] = w["l0.mix.sink"] - 30.0
    assert float((V.forward(cfg, w2, ids)[0] - base).abs().max()) > 0.5
    cfg2 = {**cfg, "layers": [dict(layer) for layer in cfg["layers"]]}
    cfg2["layers"][1] = {**cfg["layers"][1], "mixer": {**cfg["layers"][1]["mixer"], "mask": {"size": 19}}}
    assert float((V.forward(cfg2, w, ids)[0] - base).abs().max()) > 0.05


@pytest.mark.parametrize("name", ["P", "R"])
def test_greedy_generation_through_the_engine(tmp_path_factory, name):
    folder = _folder(tmp_path_factory, name)
    cfg, w = V.read_model_folder(folder)
    vocab = cases.RAW[name]["vocab"]
    rng = np.random.default_rng(2)
    prompts = [helpers.random_ids(rng, vocab, n) for n in (7, 19, 3, 11, 26)]
    want = [V.greedy(cfg, w, p, 10) for p in prompts]
    # three request slots for five prompts, portions of at most 8 tokens, small pages: requests
    # wait, prompts are cut, slots and pages are used again
    engine = LLMEngine.from_folder(folder, EngineConfig(block_size=4, num_blocks=48, max_batch_size=3,
                                                        prefill_chunk=8, dtype="float32"))
    got = engine.generate(prompts, SamplingParams(max_tokens=10, temperature=0.0))
    assert got == want
    engine = LLMEngine.from_folder(folder, EngineConfig(block_size=16, num_blocks=32, max_batch_size=3, dtype="bfloat16"))
    got = engine.generate(prompts, SamplingParams(max_tokens=10, temperature=0.0))
    for prompt, tokens in zip(prompts, got):
        seq = list(prompt)
        assert len(tokens) == 10
        for tok in tokens:
            logits = V.forward(cfg, w, seq)[0][-1].numpy()
            margin = 2 * helpers.TOL["bfloat16"] * max(1.0, float(abs(logits).max()))
            assert logits[tok] >= logits.max() - margin
            seq.append(tok)
