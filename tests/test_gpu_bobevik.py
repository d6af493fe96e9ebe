"""Bobevik on the GPU against the plain implementation (tests/plain_bobevik.py): each new kernel
alone (RMS norms, the step between two sublayers, rotation / head norm / value mixing / page store,
the decaying state, capped scores and the gate per head in the attention kernels, the gated unit's activations); whole prompts
against token-by-token decoding, portions down to two tokens and mixed batches with pages, request
slots and states used again, steps that want no logits, in 32-bit and bfloat16; long decoding;
configurations drawn at random; greedy generation through LLMEngine."""

import json

import numpy as np
import pytest
import torch

import bobevik_cases as cases
import helpers
import plain_bobevik as P
from mini_gpt_inference_amd import EngineConfig, SamplingParams
from mini_gpt_inference_amd.engine.llm_engine import LLMEngine
from mini_gpt_inference_amd.engine.replay import TraceReplayer
from mini_gpt_inference_amd.ops import kernels

pytestmark = pytest.mark.gpu
DEV = "cuda"
TDT = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def _rnd(g, *shape, dtype="float32", scale=1.0):
    return (torch.randn(*shape, generator=g) * scale).to(TDT[dtype])


def _d(t):
    return t.to(P.DTYPE)


# ---------------------------------------------------------------- kernels, one at a time
@pytest.mark.parametrize("out_dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("n,width", [(1, 8), (5, 40), (70, 256), (3, 1000), (2, 4100), (4, 2048), (2, 300)])
def test_rms_norm_rows(out_dtype, n, width):
    g = torch.Generator().manual_seed(width)
    x = _rnd(g, n + 1, width, scale=3.0)
    gain = _rnd(g, width, scale=0.3)
    rows = torch.randint(0, n, (n,), generator=g, dtype=torch.int32)
    for one_plus in (False, True):
        for gather in (False, True):
            out = torch.full((n + 1, width), 5.0, dtype=TDT[out_dtype], device=DEV)
            zero = torch.full((n + 1, 24), 7.0, device=DEV)
            kernels.rms_norm(x.to(DEV), gain.to(DEV), out, n, 1e-5, width, offset=1.0 if one_plus else 0.0,
                             rows=rows.to(DEV) if gather else None, zero=zero)
            src = x[rows.long()] if gather else x[:n]
            helpers.assert_close(out[:n], P.rms_norm(_d(src), _d(gain), 1e-5, one_plus), out_dtype, "rms norm")
            assert (out[n] == 5.0).all() and (zero[:n] == 0).all() and (zero[n] == 7.0).all()
    # without a gain, in place, a large eps
    xd = x.to(DEV)
    kernels.rms_norm(xd, None, xd, n, 0.5, width)
    helpers.assert_close(xd[:n], P.unit_rms(_d(x[:n]), 0.5), "float32", "in place")
    assert torch.equal(xd[n].cpu(), x[n])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("groups,width,stride", [(1, 24, 24), (3, 20, 20), (4, 64, 96), (2, 130, 136)])
def test_rms_norm_segments_gate_and_accumulate(dtype, groups, width, stride):
    g = torch.Generator().manual_seed(groups * width)
    n = 6
    x = _rnd(g, n, groups * stride + 8, scale=2.0)
    gain = _rnd(g, groups * width) + 1.0
    gate = _rnd(g, n, groups * width + 3, dtype=dtype, scale=2.0)
    segs = torch.stack([x[:, i * stride:i * stride + width] for i in range(groups)], dim=1)      # [n, groups, width]
    base = P.unit_rms(_d(segs), 1e-6) * _d(gain).view(groups, width)
    for act, f in ((None, None), ("silu", P.silu), ("sigmoid", P.sigmoid)):
        out = torch.zeros(n, groups * width, dtype=TDT[dtype], device=DEV)
        kernels.rms_norm(x.to(DEV), gain.to(DEV), out, n, 1e-6, width, groups=groups, x_group_stride=stride,
                         gate=gate.to(DEV) if act else None, gate_act=act)
        want = base if f is None else base * f(_d(gate[:, :groups * width])).view(n, groups, width)
        helpers.assert_close(out, want.reshape(n, -1), dtype, f"gate {act}")
    acc = _rnd(g, n, groups * width)
    out = acc.to(DEV)
    kernels.rms_norm(x.to(DEV), gain.to(DEV), out, n, 1e-6, width, groups=groups, x_group_stride=stride, mult=0.5,
                     accumulate=True)
    helpers.assert_close(out, _d(acc) + 0.5 * base.reshape(n, -1), "float32", "accumulate")


@pytest.mark.parametrize("h_dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("branches,n,width", [(1, 3, 40), (2, 70, 64), (3, 5, 300), (4, 2, 1030), (1, 9, 2048), (1, 5, 3000),
                                              (1, 2, 5000), (1, 4, 1024), (2, 3, 2048), (2, 2, 2100)])
def test_the_step_between_two_sublayers(h_dtype, branches, n, width):
    g = torch.Generator().manual_seed(branches + width)
    x = _rnd(g, n + 1, width, scale=3.0)
    ys = [_rnd(g, n + 1, width, scale=1.0 + b) for b in range(branches)]
    joins = [_rnd(g, width) + 1.0 for _ in range(branches)]
    post, nxt = _rnd(g, width, scale=0.2), _rnd(g, width, scale=0.2)
    eps, mult = 1e-5, 0.7
    if branches == 1:
        y = _d(ys[0][:n])
    else:
        y = sum(P.rms_norm(_d(yb[:n]), _d(jb), eps, False) for yb, jb in zip(ys, joins)) / branches
    want_x = _d(x[:n]) + mult * P.rms_norm(y, _d(post), eps, True)
    for with_next in (True, False):
        xd = x.to(DEV)
        yd = [yb.to(DEV) for yb in ys]
        h = torch.full((n + 1, width), 5.0, dtype=TDT[h_dtype], device=DEV)
        kernels.rms_post_norm([(yb, jb.to(DEV) if branches > 1 else None) for yb, jb in zip(yd, joins)], xd, post.to(DEV),
                              n, eps, 1.0, mult, gain_next=nxt.to(DEV) if with_next else None, h=h if with_next else None)
        helpers.assert_close(xd[:n], want_x, "float32", "residual")
        assert torch.equal(xd[n].cpu(), x[n])
        for yb, y0 in zip(yd, ys):
            assert (yb[:n] == 0).all() and torch.equal(yb[n].cpu(), y0[n])
        if with_next:
            helpers.assert_close(h[:n], P.rms_norm(want_x, _d(nxt), eps, True), h_dtype, "next norm")
            assert (h[n] == 5.0).all()


def _freq(dims, base, factor=1.0):
    return torch.tensor([base ** (-2.0 * i / dims) / factor for i in range(dims // 2)], dtype=torch.float64).float()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H,G,D,E,stride,dims,page", [(4, 2, 16, 32, 32, 8, 4), (2, 2, 64, 64, 64, 64, 16),
                                                      (3, 1, 20, 12, 24, 20, 8), (8, 1, 48, 64, 64, 48, 16),
                                                      (1, 1, 130, 40, 136, 2, 4)])
def test_rotation_head_norm_value_mixing_and_page_store(dtype, H, G, D, E, stride, dims, page):
    g = torch.Generator().manual_seed(H * D + E)
    n, pages = 9, 6
    q_off, k_off, v_off = 0, H * stride, (H + G) * stride
    z = torch.zeros(n, (H + 2 * G) * stride + 16)
    q, k, v = _rnd(g, n, H, D, dtype=dtype), _rnd(g, n, G, D, dtype=dtype), _rnd(g, n, G, E, dtype=dtype)
    z[:, q_off:k_off].view(n, H, stride)[:, :, :D] = q.float()
    z[:, k_off:v_off].view(n, G, stride)[:, :, :D] = k.float()
    z[:, v_off:v_off + G * stride].view(n, G, stride)[:, :, :E] = v.float()
    z = z.to(TDT[dtype])
    # positions up to a thousand (beyond, the rounding of a 32-bit angle is itself larger than the bound);
    # slots scattered, one token without
    positions = torch.tensor([0, 1, 1100, 1025, 33, 2, 511, 7, 8], dtype=torch.int32)
    slots = torch.tensor([page + 1, 0, 5 * page + page - 1, -1, 2 * page, 3, 2, 4 * page + 1, 1], dtype=torch.int32)
    freq = _freq(dims, 10000.0, 4.0)
    other = _rnd(g, n, G * E + 4, dtype=dtype)
    lam = torch.tensor(0.3)

    def rotated(x):     # [n, heads, D] at the given positions, through the plain function one position at a time
        out = torch.zeros(n, x.shape[1], D, dtype=P.DTYPE)
        for i, p in enumerate(positions.tolist()):
            seq = torch.zeros(p + 1, x.shape[1], D, dtype=P.DTYPE)
            seq[p] = _d(x[i])
            out[i] = P.rotate_half(seq[max(p - 1, 0):], dims, 10000.0, 4.0)[-1] if p == 0 else \
                _rotate_at(_d(x[i]), p, dims, 10000.0, 4.0)
        return out

    for norm_eps in (None, 1e-5):
        for mode in (0, 1, 2):
            zd = z.to(DEV)
            kp = torch.full((pages, G, page, stride), 7.0, dtype=TDT[dtype], device=DEV)
            vp = torch.full((pages, G, page, stride), 7.0, dtype=TDT[dtype], device=DEV)
            od = other.to(DEV)
            kernels.qk_prepare(zd, q_off, k_off, v_off, H, G, D, E, stride, n, positions=positions.to(DEV), freq=freq.to(DEV),
                               norm_eps=norm_eps, mix_lambda=lam.to(DEV) if mode == 2 else None,
                               v_other=od if mode else None, mix_mode=mode, k_pool=kp, v_pool=vp, slot_mapping=slots.to(DEV))
            want_q, want_k = rotated(q), rotated(k)
            if norm_eps is not None:
                want_q, want_k = P.unit_rms(want_q, norm_eps), P.unit_rms(want_k, norm_eps)
            want_v = _d(v)
            if mode == 2:
                want_v = 0.7 * want_v + 0.3 * _d(other[:, :G * E]).view(n, G, E)
            got_q = zd[:, q_off:k_off].view(n, H, stride)
            helpers.assert_close(got_q[:, :, :D], want_q, dtype, f"q norm {norm_eps}")
            assert (got_q[:, :, D:] == 0).all()
            if mode == 1:
                assert torch.equal(od[:, :G * E].cpu().view(n, G, E), v) and torch.equal(od[:, G * E:].cpu(), other[:, G * E:])
            else:
                assert torch.equal(od.cpu(), other)
            kf, vf = kp.permute(0, 2, 1, 3).reshape(pages * page, G, stride), vp.permute(0, 2, 1, 3).reshape(pages * page, G, stride)
            for i, s in enumerate(slots.tolist()):
                if s < 0:
                    continue
                helpers.assert_close(kf[s][:, :D], want_k[i], dtype, f"key {i}")
                helpers.assert_close(vf[s][:, :E], want_v[i], dtype, f"value {i} mode {mode}")
                assert (kf[s][:, D:] == 0).all() and (vf[s][:, E:] == 0).all()
            written = {s for s in slots.tolist() if s >= 0}
            assert all((kf[s] == 7.0).all() and (vf[s] == 7.0).all() for s in range(pages * page) if s not in written)


def _rotate_at(x, p, dims, base, factor):
    """One position of the plain rotation, without building the sequence before it."""
    half = dims // 2
    freq = torch.tensor([base ** (-2.0 * i / dims) / factor for i in range(half)], dtype=P.DTYPE)
    c, s = torch.cos(p * freq), torch.sin(p * freq)
    a, b = x[..., :half], x[..., half:dims]
    return torch.cat([a * c - b * s, b * c + a * s, x[..., dims:]], dim=-1)


def test_the_plain_rotation_agrees_with_its_one_position_form():
    g = torch.Generator().manual_seed(0)
    x = _d(_rnd(g, 7, 2, 12))
    whole = P.rotate_half(x, 8, 100.0, 2.0)
    for p in range(7):
        assert torch.allclose(whole[p], _rotate_at(x[p], p, 8, 100.0, 2.0), atol=1e-12)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kind,f", [("silu", P.silu), ("relu", lambda z: torch.clamp(z, min=0.0)),
                                    ("gelu_tanh", lambda z: 0.5 * z * (1 + torch.tanh(0.7978845608028654 * (z + 0.044715 * z ** 3))))])
def test_gated_unit_activations(dtype, kind, f):
    g = torch.Generator().manual_seed(4)
    for hidden in (36, 40, 320):          # (multiples of 8 take the kernel with 16-byte loads in bfloat16)
        z = _rnd(g, 7, 2 * hidden, dtype=dtype, scale=2.0)
        for fast in (False, True):
            act = torch.full((8, hidden), 3.0, dtype=TDT[dtype], device=DEV)
            kernels.gated_unit(z.to(DEV), act, 7, hidden, fast=fast, activation=kind)
            helpers.assert_close(act[:7], f(_d(z[:, :hidden])) * _d(z[:, hidden:]), dtype if not fast else "bfloat16",
                                 f"{kind} {hidden}")
            assert (act[7] == 3.0).all()


def _state_case(g, dtype, lens, H, D, E):
    n = sum(lens)
    width = 2 * H * D + 2 * H * E
    z = _rnd(g, n, width + 8, dtype=dtype)
    return z, H * D, 2 * H * D, 2 * H * D + H * E


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H,D,E", [(2, 16, 24), (1, 64, 64), (2, 128, 128), (3, 20, 12), (1, 256, 64), (2, 8, 256),
                                   (1, 1, 1)])
def test_decaying_state_whole_in_portions_and_slots_used_again(dtype, H, D, E):
    """Three requests of unequal lengths in one step against the plain recurrence; then the same
    requests cut into portions (down to one token) over several steps, their states carried in
    slots that held other requests' states before (poisoned with NaN first)."""
    g = torch.Generator().manual_seed(H * D + E)
    lens = [37, 1, 12]
    z, k_off, v_off, g_off = _state_case(g, dtype, lens, H, D, E)
    n = sum(lens)
    decay = torch.tensor(([0.999, 0.6, 0.9] * 3)[:H])
    dims = D - D % 2 if D >= 2 else 0
    freq = _freq(dims, 1000.0) if dims else None
    for variant in ("retention", "lightning"):
        silu_in = variant == "lightning"
        want = torch.zeros(n, H * E, dtype=P.DTYPE)
        at = 0
        for T in lens:
            rows = _d(z[at:at + T])
            f = P.silu if silu_in else (lambda t: t)
            q, k = f(rows[:, :H * D]).view(T, H, D), f(rows[:, k_off:k_off + H * D]).view(T, H, D)
            v = f(rows[:, v_off:v_off + H * E]).view(T, H, E)
            if variant == "retention":
                if dims:
                    q, k = P.rotate_half(q, dims, 1000.0), P.rotate_half(k, dims, 1000.0)
                k = k * 0.25
                o = P.unit_rms(P.decaying_state(q, k, v, decay.tolist()), 1e-5).reshape(T, H * E)
                o = o * P.silu(rows[:, g_off:g_off + H * E])
            else:
                o = P.decaying_state(q, k, v, decay.tolist()).reshape(T, H * E)
            want[at:at + T] = o
            at += T
        out_dtype = dtype if variant == "retention" else "float32"
        kwargs = dict(silu_inputs=silu_in, freq=freq.to(DEV) if (variant == "retention" and dims) else None,
                      k_scale=0.25 if variant == "retention" else 1.0, norm_eps=1e-5 if variant == "retention" else None)
        gate = g_off if variant == "retention" else -1

        def run(steps, state, out):
            """steps: [[(request, first token, tokens)]]; request r uses slot 3 - r."""
            for step in steps:
                rows, pos, cu, slots = [], [], [0], []
                for r, first, count in step:
                    base = sum(lens[:r])
                    rows += list(range(base + first, base + first + count))
                    pos += list(range(first, first + count))
                    cu.append(len(rows))
                    slots.append(3 - r)
                # two empty requests of a padding at the end
                cu += [len(rows)] * 2
                slots += [-1, 0]
                zs = z[rows].to(DEV)
                o = torch.zeros(len(rows), H * E, dtype=TDT[out_dtype], device=DEV)
                kernels.decay_state(zs, 0, k_off, v_off, gate, H, D, E, decay.to(DEV), state,
                                    torch.tensor(slots, dtype=torch.int32, device=DEV),
                                    torch.tensor(cu, dtype=torch.int32, device=DEV), len(slots),
                                    torch.tensor(pos, dtype=torch.int32, device=DEV), o, **kwargs)
                out[rows] = o.float().cpu().to(P.DTYPE)

        state = torch.full((5, H * D * E), float("nan"), device=DEV)
        got = torch.zeros(n, H * E, dtype=P.DTYPE)
        run([[(0, 0, 37), (1, 0, 1), (2, 0, 12)]], state, got)
        helpers.assert_close(got, want, out_dtype, f"{variant} whole")
        assert torch.isnan(state[0]).all() and torch.isnan(state[4]).all() and torch.isfinite(state[1:4]).all()
        whole_state = state.clone()
        # the same again in portions, in the slots that now hold the finished requests' states
        got2 = torch.zeros(n, H * E, dtype=P.DTYPE)
        run([[(0, 0, 2), (2, 0, 5)], [(0, 2, 9), (1, 0, 1)], [(2, 5, 1), (0, 11, 1)], [(0, 12, 17), (2, 6, 6)],
             [(0, 29, 8)]], state, got2)
        helpers.assert_close(got2, want, out_dtype, f"{variant} portions")
        helpers.assert_close(state[1:4], whole_state[1:4], "float32", f"{variant} state")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H,D,E", [(2, 16, 24), (1, 64, 64), (2, 128, 128), (3, 20, 12), (1, 128, 200), (2, 8, 256),
                                   (1, 1, 1), (1, 30, 33), (8, 16, 200), (9, 64, 160)])     # (the last two: 32 channels a workgroup)
def test_decaying_state_a_chunk_at_a_time(dtype, H, D, E):
    """The matrix-core form for prompt portions against the plain recurrence: requests whose lengths are
    below, at and beyond the chunk of 32 tokens, in one step; then cut into portions that end inside
    chunks, beside single tokens, the states carried in slots poisoned before."""
    g = torch.Generator().manual_seed(H * D + E + 1)
    lens = [70, 1, 32, 33]
    n = sum(lens)
    z, k_off, v_off, g_off = _state_case(g, dtype, lens, H, D, E)
    decay = torch.tensor(([0.999, 0.6, 0.9] * 3)[:H])
    dims = D - D % 2 if D >= 2 else 0
    for variant in ("rotated", "silu"):
        f = P.silu if variant == "silu" else (lambda t: t)
        want = torch.zeros(n, H * E, dtype=P.DTYPE)
        at = 0
        for T in lens:
            rows = _d(z[at:at + T])
            q, k = f(rows[:, :H * D]).view(T, H, D), f(rows[:, k_off:k_off + H * D]).view(T, H, D)
            v = f(rows[:, v_off:v_off + H * E]).view(T, H, E)
            if variant == "rotated":
                if dims:
                    q, k = P.rotate_half(q, dims, 1000.0), P.rotate_half(k, dims, 1000.0)
                k = k * 0.25
            want[at:at + T] = P.decaying_state(q, k, v, decay.tolist()).reshape(T, H * E)
            at += T
        freq = _freq(dims, 1000.0).to(DEV) if (variant == "rotated" and dims) else None

        def run(steps, state, out):
            for step in steps:
                rows, pos, cu, slots = [], [], [0], []
                for r, first, count in step:
                    base = sum(lens[:r])
                    rows += list(range(base + first, base + first + count))
                    pos += list(range(first, first + count))
                    cu.append(len(rows))
                    slots.append(4 - r)
                cu += [len(rows)] * 2
                slots += [-1, 0]
                zs = z[rows].to(DEV)
                o = torch.zeros(len(rows), H * E, device=DEV)
                qk = torch.zeros(len(rows), 2 * H * D, device=DEV)
                assert kernels.decay_state_chunked(zs, 0, k_off, v_off, H, D, E, decay.to(DEV), state,
                                                   torch.tensor(slots, dtype=torch.int32, device=DEV),
                                                   torch.tensor(cu, dtype=torch.int32, device=DEV), len(slots), len(rows),
                                                   torch.tensor(pos, dtype=torch.int32, device=DEV), qk, o,
                                                   silu_inputs=variant == "silu", freq=freq,
                                                   k_scale=0.25 if variant == "rotated" else 1.0)
                out[rows] = o.cpu().to(P.DTYPE)

        state = torch.full((6, H * D * E), float("nan"), device=DEV)
        got = torch.zeros(n, H * E, dtype=P.DTYPE)
        run([[(0, 0, 70), (1, 0, 1), (2, 0, 32), (3, 0, 33)]], state, got)
        helpers.assert_close(got, want, "float32", f"{variant} whole")
        assert torch.isnan(state[0]).all() and torch.isnan(state[5]).all() and torch.isfinite(state[1:5]).all()
        whole_state = state.clone()
        got2 = torch.zeros(n, H * E, dtype=P.DTYPE)
        run([[(0, 0, 31), (3, 0, 2)], [(0, 31, 2), (1, 0, 1), (3, 2, 30)], [(3, 32, 1), (0, 33, 36), (2, 0, 17)],
             [(0, 69, 1), (2, 17, 15)]], state, got2)
        helpers.assert_close(got2, want, "float32", f"{variant} portions")
        helpers.assert_close(state[1:5], whole_state[1:5], "float32", f"{variant} state")
        # and the token-by-token kernel goes on from a state that the chunked one left
        if variant == "silu":
            extra = _rnd(g, 3, z.shape[1], dtype=dtype)
            rows = _d(torch.cat([z[:70], extra]))
            q, k = P.silu(rows[:, :H * D]).view(73, H, D), P.silu(rows[:, k_off:k_off + H * D]).view(73, H, D)
            v = P.silu(rows[:, v_off:v_off + H * E]).view(73, H, E)
            ref = P.decaying_state(q, k, v, decay.tolist()).reshape(73, H * E)[70:]
            o = torch.zeros(3, H * E, device=DEV)
            kernels.decay_state(extra.to(DEV), 0, k_off, v_off, -1, H, D, E, decay.to(DEV), state,
                                torch.tensor([4], dtype=torch.int32, device=DEV), torch.tensor([0, 3], dtype=torch.int32, device=DEV),
                                1, torch.tensor([70, 71, 72], dtype=torch.int32, device=DEV), o, silu_inputs=True)
            helpers.assert_close(o, ref, "float32", "token by token behind chunks")


def test_the_state_far_back_matters():
    """With a decay near one the first token's key and value are still in the output after hundreds
    of tokens (a lost or restarted state shows), with a fast decay they are gone."""
    g = torch.Generator().manual_seed(5)
    T = 400
    q, k, v = _d(_rnd(g, T, 2, 8)), _d(_rnd(g, T, 2, 8)), _d(_rnd(g, T, 2, 8))
    base = P.decaying_state(q, k, v, [0.9995, 0.5])
    k2 = k.clone()
    k2[0] *= 20.0
    moved = P.decaying_state(q, k2, v, [0.9995, 0.5])
    assert float((moved[-1, 0] - base[-1, 0]).abs().max()) > 1.0
    assert float((moved[-1, 1] - base[-1, 1]).abs().max()) < 1e-9


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_capped_scores_in_attention_with_a_key_that_stands_out(dtype):
    """The general attention kernel with cap * tanh(score / cap): one key far back (at a page border)
    and the query are scaled so that its score is many times the cap; without the cap it would take
    all the weight, with it the other keys keep theirs."""
    g = torch.Generator().manual_seed(6)
    H, G, D, page, T = 4, 2, 32, 8, 200
    q, k, v = _rnd(g, T, H, D, dtype=dtype), _rnd(g, T, G, D, dtype=dtype), _rnd(g, T, G, D, dtype=dtype)
    far = 2 * page - 1
    k[far] *= 6.0
    q[-1] = (k[far].float().repeat_interleave(H // G, dim=0)).to(TDT[dtype])
    cap, scale = 3.0, 0.2
    want = P.causal_softmax_attention(_d(q), _d(k), _d(v), scale, cap)
    uncapped = P.causal_softmax_attention(_d(q), _d(k), _d(v), scale, None)
    assert float((want[-1] - uncapped[-1]).abs().max()) > 0.3
    gate = _rnd(g, T, H + 3, dtype=dtype, scale=2.0)        # one number a token and head, behind a sigmoid
    gated = want * P.sigmoid(_d(gate[:, :H]))[:, :, None]
    pages = T // page
    perm = torch.randperm(pages, generator=g)
    kp = torch.zeros(pages, G, page, D, dtype=TDT[dtype])
    vp = torch.zeros(pages, G, page, D, dtype=TDT[dtype])
    for j in range(T):
        kp[perm[j // page], :, j % page], vp[perm[j // page], :, j % page] = k[j], v[j]
    out = torch.zeros(T, H * D, dtype=TDT[dtype], device=DEV)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)
    # the last 70 queries as a portion on top of 130 cached tokens
    first = 130
    kernels.paged_attention_generic(q[first:].reshape(T - first, H * D).to(DEV), out, kp.to(DEV), vp.to(DEV),
                                    perm.to(torch.int32).view(1, pages).to(DEV), i32([0, T - first]), i32([T]),
                                    i32([0] * (T - first)), T - first, 1, H, scale, softcap=cap)
    helpers.assert_close(out[:T - first], want[first:].reshape(T - first, H * D), dtype, "capped attention")
    kernels.paged_attention_generic(q[first:].reshape(T - first, H * D).to(DEV), out, kp.to(DEV), vp.to(DEV),
                                    perm.to(torch.int32).view(1, pages).to(DEV), i32([0, T - first]), i32([T]),
                                    i32([0] * (T - first)), T - first, 1, H, scale, softcap=cap, gate=gate[first:].to(DEV))
    helpers.assert_close(out[:T - first], gated[first:].reshape(T - first, H * D), dtype, "capped and gated attention")


@pytest.mark.parametrize("D", [32, 64, 128])
def test_capped_scores_in_the_bfloat16_attention_kernels(D):
    """The same construction through the matrix-core kernel for portions, the decode kernel and the
    kernel that splits a query's keys over waves: the cap must bite in each."""
    g = torch.Generator().manual_seed(7 + D)
    H, G, page, T = 4, 2, 16, 208
    q, k, v = _rnd(g, T, H, D, dtype="bfloat16"), _rnd(g, T, G, D, dtype="bfloat16"), _rnd(g, T, G, D, dtype="bfloat16")
    far = 2 * page - 1
    k[far] *= 4.0
    q[-1] = k[far].float().repeat_interleave(H // G, dim=0).to(torch.bfloat16)
    cap, scale = 3.0, D ** -0.5
    want = P.causal_softmax_attention(_d(q), _d(k), _d(v), scale, cap)
    assert float((want[-1] - P.causal_softmax_attention(_d(q), _d(k), _d(v), scale, None)[-1]).abs().max()) > 0.3
    pages = T // page
    perm = torch.randperm(pages, generator=g)
    kp = torch.zeros(pages, G, page, D, dtype=torch.bfloat16)
    vp = torch.zeros(pages, G, page, D, dtype=torch.bfloat16)
    for j in range(T):
        kp[perm[j // page], :, j % page], vp[perm[j // page], :, j % page] = k[j], v[j]
    kp, vp, bt = kp.to(DEV), vp.to(DEV), perm.to(torch.int32).view(1, pages).to(DEV)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)
    first = 100
    n = T - first
    qd = q[first:].reshape(n, H * D).to(DEV)
    gate = _rnd(g, n, H + 5, dtype="bfloat16", scale=2.0)
    for gd in (None, gate.to(DEV)):
        ref = want[first:] if gd is None else want[first:] * P.sigmoid(_d(gate[:, :H]))[:, :, None]
        ref = ref.reshape(n, H * D)
        out = torch.zeros(n, H * D, dtype=torch.bfloat16, device=DEV)
        assert kernels.prefill_attention_bf16(qd, out, kp, vp, bt, i32([0, n]), i32([T]), 1, n, H, scale, softcap=cap, gate=gd)
        helpers.assert_close(out, ref, "bfloat16", "tile kernel")
        out.zero_()
        assert kernels.paged_attention_split_bf16(qd, out, kp, vp, bt, i32([0, n]), i32([T]), i32([0] * n), n, 1, H, scale,
                                                  softcap=cap, gate=gd)
        helpers.assert_close(out, ref, "bfloat16", "split kernel")
        out.zero_()
        assert kernels.paged_attention_split_bf16(qd, out, kp, vp, bt, i32([0, n]), i32([T]), i32([0] * n), n, 1, H, scale,
                                                  fast=False, softcap=cap, gate=gd)
        helpers.assert_close(out, ref, "bfloat16", "split kernel, general variant")
        one = torch.zeros(1, H * D, dtype=torch.bfloat16, device=DEV)
        assert kernels.paged_attention_decode_bf16(qd[n - 1:], one, kp, vp, bt, i32([T - 1]), i32([0]), 1, H, scale,
                                                   identity=True, softcap=cap, gate=None if gd is None else gd[n - 1:])
        helpers.assert_close(one, ref[n - 1:], "bfloat16", "decode kernel")


# ---------------------------------------------------------------- the model through the step function
LENGTHS = {"A": [5, 70, 23, 41, 2, 64, 37], "B": [1, 9, 33, 17, 150], "C": [40, 3, 64, 21], "D": [75, 12, 30, 6, 49]}
_folders, _plain, _twin = {}, {}, {}


def _folder(tmp_path_factory, name):
    if name not in _folders:
        _folders[name] = cases.write_model(str(tmp_path_factory.mktemp("bobevik") / name), name)
    return _folders[name]


def _requests(name):
    rng = np.random.default_rng(len(name) + ord(name[0]))
    return {f"r{i}": helpers.random_ids(rng, cases.RAW[name]["vocab"], n) for i, n in enumerate(LENGTHS[name])}


def _plain_logits(folder, name):
    if name not in _plain:
        cfg, w = P.read_model_folder(folder)
        _plain[name] = {rid: P.forward(cfg, w, ids).numpy() for rid, ids in _requests(name).items()}
    return _plain[name]


def _row_errors(got, want):
    """Per position: root mean square over the vocabulary of the difference, its mean taken off."""
    d = np.asarray(got, dtype=np.float64) - np.asarray(want, dtype=np.float64)
    d = d - d.mean(axis=1, keepdims=True)
    return np.sqrt((d * d).mean(axis=1))


def _rounded_twin(cfg, w, ids):
    """The plain implementation with every matrix product rounded to bfloat16: what rounding alone does."""
    P.ROUNDING = torch.bfloat16
    try:
        return P.forward(cfg, w, ids).numpy()
    finally:
        P.ROUNDING = None


def _assert_within_rounding(folder, key, ids, got, want, what, worst=3.0):
    """bfloat16: a position's error may be `worst` times what rounding alone causes at the request's
    worst position, and the request's mean error three times the mean of that."""
    assert np.isfinite(got).all(), f"{what}: non-finite logits"
    if key not in _twin:
        cfg, w = P.read_model_folder(folder)
        _twin[key] = _row_errors(_rounded_twin(cfg, w, ids), want)
    noise, err = _twin[key], _row_errors(got, want)
    assert err.max() <= worst * noise.max(), f"{what}: worst position {err.max():.3e} > {worst} * {noise.max():.3e}"
    assert err.mean() <= 3.0 * noise.mean(), f"{what}: mean {err.mean():.3e} > 3 * {noise.mean():.3e}"


def _check(folder, name, dtype, rid, ids, got, want, what):
    if dtype == "float32":
        assert np.isfinite(got).all(), what
        err = _row_errors(got, want)
        assert err.max() <= 5e-5 * max(1.0, float(np.abs(want).max())), f"{what}: {err.max():.3e}"
    else:
        _assert_within_rounding(folder, (name, rid, len(ids)), ids, got, want, what)


@pytest.mark.parametrize("page_size", [16, 4])
@pytest.mark.parametrize("way", ["whole", "tail", "portions", "mixed"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(cases.RAW))
def test_every_way_of_cutting_matches_the_plain_implementation(tmp_path_factory, name, dtype, way, page_size):
    folder = _folder(tmp_path_factory, name)
    reqs = _requests(name)
    want = _plain_logits(folder, name)
    plan = helpers.PLANS[way](reqs, np.random.default_rng(5))
    # the pool holds just what the live requests need and starts as NaN, and so do the states; four request slots
    replayer = TraceReplayer(folder, dtype, plan.tight_tokens(page_size), page_size=page_size, max_live=4, poison=True)
    got = plan.assemble(helpers.run_plan_in_process(replayer, plan), {r: len(t) for r, t in reqs.items()},
                        cases.RAW[name]["vocab"])
    for rid in reqs:
        _check(folder, name, dtype, rid, reqs[rid], got[rid], want[rid], f"{name} {dtype} {way} {rid}")
    assert replayer.cache.check() == 0 and not replayer.live
    assert all(replayer.cache.num_free_pages(g) == replayer.num_pages for g in range(len(replayer.cache.groups)))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_steps_that_want_no_logits_leave_the_state_right(tmp_path_factory, name, dtype):
    """Token-by-token steps of which only every fourth wants its logits, and mixed steps likewise:
    step shapes come back often enough to be replayed from recorded launches and from graphs, of
    the exact shape and of its bucket, and a request's state must have seen every token once."""
    folder = _folder(tmp_path_factory, name)
    reqs = _requests(name)
    want = _plain_logits(folder, name)
    for way in ("tail", "mixed"):
        plan = helpers.PLANS[way](reqs, np.random.default_rng(7))
        kept = {}
        for rec in plan.steps:
            rows, keep, at = plan.wanted[rec["step"]], [], 0
            for entry in rec["entries"]:
                n = len(entry["tokens"])
                entry["want"] = [i for i in range(n) if (rec["step"] + i) % 4 == 0]
                keep += [rows[at + i] for i in entry["want"]]
                at += n
            kept[rec["step"]] = keep
        plan.wanted = {s: rows for s, rows in kept.items() if rows}
        replayer = TraceReplayer(folder, dtype, plan.tight_tokens(16), page_size=16, max_live=4, poison=True)
        outputs = helpers.run_plan_in_process(replayer, plan)
        assert replayer.runner.num_replayed_steps > 0
        vocab = cases.RAW[name]["vocab"]
        for step, rows in plan.wanted.items():
            out = np.asarray(outputs[step], dtype=np.float64).reshape(len(rows), vocab)
            for (rid, pos), row in zip(rows, out):
                ref = want[rid][pos:pos + 1]
                err = float(_row_errors(row[None], ref)[0])
                bound = 5e-5 * max(1.0, float(np.abs(ref).max())) if dtype == "float32" else 0.1
                assert np.isfinite(row).all() and err <= bound, f"{name} {dtype} {way} {rid} position {pos}: {err:.3e}"


@pytest.mark.parametrize("seed", range(8))
def test_random_configurations(tmp_path, seed):
    """Configurations drawn at random (tests/bobevik_cases.py: random_raw), five requests of lengths
    1 to 200 each, whole, in portions and mixed, in both dtypes.  bfloat16: a position may be one and
    a half times over three times what rounding alone does, the mean may not."""
    rng = np.random.default_rng(2000 + seed)
    raw = cases.random_raw(rng)
    folder = cases.write_raw_model(str(tmp_path / "m"), raw, seed)
    cfg, w = P.read_model_folder(folder)
    lens = [int(x) for x in rng.choice([1, 2, 5, 17, 33, 64, 70, 97, 130, 200], size=5)]
    reqs = {f"r{i}": helpers.random_ids(rng, raw["vocab"], n) for i, n in enumerate(lens)}
    want = {rid: P.forward(cfg, w, ids).numpy() for rid, ids in reqs.items()}
    noise = {rid: _row_errors(_rounded_twin(cfg, w, ids), want[rid]) for rid, ids in reqs.items()}
    for dtype in ("float32", "bfloat16"):
        for way in ("whole", "portions", "mixed"):
            plan = helpers.PLANS[way](reqs, np.random.default_rng(5))
            replayer = TraceReplayer(folder, dtype, plan.tight_tokens(16), page_size=16, max_live=4, poison=True)
            got = plan.assemble(helpers.run_plan_in_process(replayer, plan), {r: len(t) for r, t in reqs.items()},
                                raw["vocab"])
            for rid in reqs:
                what = f"seed {seed} {dtype} {way} {rid} ({json.dumps(raw)})"
                assert np.isfinite(got[rid]).all(), what
                err = _row_errors(got[rid], want[rid])
                if dtype == "float32":
                    assert err.max() <= 5e-5 * max(1.0, float(np.abs(want[rid]).max())), f"{err.max():.3e}: {what}"
                    continue
                assert err.max() <= 4.5 * noise[rid].max() and err.mean() <= 3.0 * noise[rid].mean(), \
                    f"{err.max():.3e} / {noise[rid].max():.3e}, mean {err.mean():.3e} / {noise[rid].mean():.3e}: {what}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(tmp_path_factory, dtype):
    """Three tokens of prompt, then 300 tokens one by one through pages of four tokens: states are
    carried over hundreds of steps, the decode steps come from graphs."""
    folder = _folder(tmp_path_factory, "A")
    ids = helpers.random_ids(np.random.default_rng(9), cases.RAW["A"]["vocab"], 303)
    cfg, w = P.read_model_folder(folder)
    want = P.forward(cfg, w, ids).numpy()
    plan = helpers.plan_tail({"a": ids}, tail=300)
    replayer = TraceReplayer(folder, dtype, 304, page_size=4, max_live=4, poison=True)
    got = plan.assemble(helpers.run_plan_in_process(replayer, plan), {"a": len(ids)}, cases.RAW["A"]["vocab"])
    _check(folder, "A", dtype, "long", ids, got["a"], want, "long decoding")


@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_through_the_engine(tmp_path_factory, name):
    folder = _folder(tmp_path_factory, name)
    cfg, w = P.read_model_folder(folder)
    vocab = cases.RAW[name]["vocab"]
    rng = np.random.default_rng(2)
    prompts = [helpers.random_ids(rng, vocab, n) for n in (7, 19, 3, 11, 26)]
    want = [P.greedy(cfg, w, p, 10) for p in prompts]
    # three request slots for five prompts, portions of at most 8 tokens, small pages: requests
    # wait, prompts are cut, slots, pages and states are used again
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
            logits = P.forward(cfg, w, seq)[-1].numpy()
            margin = 2 * helpers.TOL["bfloat16"] * max(1.0, float(abs(logits).max()))
            assert logits[tok] >= logits.max() - margin
            seq.append(tok)


def test_generation_with_evictions_recomputes_the_state(tmp_path_factory):
    """A page pool too small for all running requests: the newest is evicted and later recomputed
    from its prompt and outputs, its state starting over; the tokens are those of an engine with room."""
    folder = _folder(tmp_path_factory, "D")
    rng = np.random.default_rng(3)
    prompts = [helpers.random_ids(rng, cases.RAW["D"]["vocab"], n) for n in (9, 14, 5, 12)]
    roomy = LLMEngine.from_folder(folder, EngineConfig(block_size=4, num_blocks=64, max_batch_size=4, dtype="float32"))
    want = roomy.generate(prompts, SamplingParams(max_tokens=24, temperature=0.0))
    tight = LLMEngine.from_folder(folder, EngineConfig(block_size=4, num_blocks=22, max_batch_size=4, dtype="float32"))
    got = tight.generate(prompts, SamplingParams(max_tokens=24, temperature=0.0))
    assert got == want
    assert tight.stats()["num_preemptions"] > 0
