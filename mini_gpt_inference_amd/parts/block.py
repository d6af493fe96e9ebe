"""Arrangements: how a layer's norm, mixer and feed-forward sit around the residual stream."""

from __future__ import annotations

from typing import Dict, Mapping, Optional, Tuple

import torch

from ..ops import kernels, residual
from ..ops.linear import LazyNorm
from .base import CacheBinding, Part, StepContext, VECTOR, WeightRequest, register_arrangement
from .feedforward import FeedForward
from .mixers import Mixer
from .positions import PositionEncoding


class Arrangement(Part):
    """How a layer's parts sit around the residual stream.  `roles` names the parts it arranges (the
    model refuses a layer whose parts are others); run() gets them by role, and for every mixer role
    the binding of this run's cache."""

    category = "arrangement"
    roles: Optional[Tuple[str, ...]] = None     # None: whatever the layer brings

    def run(self, ctx: StepContext, x: torch.Tensor, parts: Mapping[str, Part],
            bindings: Mapping[str, CacheBinding], position: PositionEncoding) -> None:
        raise NotImplementedError


@register_arrangement("pre_norm")
class PreNorm(Arrangement):
    """x = x + mixer(norm1(x)); x = x + ff(norm2(x)) (reference: src/minigpt_infer/model.py:112-115)."""

    graph_safe = True

    plan_safe = True
    takes_pending_residual = True
    roles = ("norm1", "mixer", "norm2", "feed_forward")

    def __init__(self, width: int) -> None:
        self.width = int(width)

    def run(self, ctx, x, parts, bindings, position) -> None:
        norm1, mixer, norm2, feed_forward = (parts[r] for r in self.roles)
        binding = bindings["mixer"]
        # the norms are handed on uncomputed: a linear layer that can normalise in its prologue
        # does, everything else calls .tensor(ctx) and gets the normed rows.  A part that does not
        # know of a residual whose sums are still pending gets a plain one.
        n = ctx.n_rows
        if not mixer.takes_pending_residual:
            residual.settle(ctx, x, n)
        mixer.forward_add(ctx, LazyNorm(norm1, x, n), x, binding, position)
        if not feed_forward.takes_pending_residual:
            residual.settle(ctx, x, n)
        feed_forward.forward_add(ctx, LazyNorm(norm2, x, n), x)


@register_arrangement("pre_norm_mixer")
class PreNormMixerOnly(Arrangement):
    """x = x + mixer(norm1(x)): a pre-norm layer that has no feed-forward."""

    graph_safe = True
    plan_safe = True
    takes_pending_residual = True
    roles = ("norm1", "mixer")

    def __init__(self, width: int) -> None:
        self.width = int(width)

    def run(self, ctx, x, parts, bindings, position) -> None:
        mixer = parts["mixer"]
        if not mixer.takes_pending_residual:
            residual.settle(ctx, x, ctx.n_rows)
        mixer.forward_add(ctx, LazyNorm(parts["norm1"], x, ctx.n_rows), x, bindings["mixer"], position)


def flush_streams(ctx: StepContext, x: torch.Tensor, streams: int) -> None:
    """Makes the write into the residual streams that a sublayer has left pending, if any."""
    if ctx.pending_streams is not None:
        mix, out, y = ctx.pending_streams
        ctx.pending_streams = None
        kernels.streams_write(x, mix, out, y, ctx.n_rows, streams)


@register_arrangement("hyper_connections")
class HyperConnections(Arrangement):
    """A pre-norm layer over several residual streams.  A token's residual is S rows x_1 .. x_S.
    For sublayer q (1: the mixer, 2: the feed-forward, which a layer may lack) with its own
    a_q [S], M_q [S, S] and b_q [S]:

        u = sum_s a_q[s] x_s;  y = sublayer_q(norm_q(u));  x_t <- sum_s M_q[s, t] x_s + b_q[t] y

    every new stream from the old ones, all in float32.  With S = 1, a = b = 1 and M = 1 this is
    the plain pre-norm layer.  The sublayers are the framework's ordinary parts: they add their
    output into a cleared buffer that stands for y.  A sublayer's write is left pending
    (ctx.pending_streams) and made by the kernel that reads the streams next: the next sublayer's
    read and LayerNorm, or the model before the final norm."""

    graph_safe = True
    plan_safe = True

    def __init__(self, width: int, streams: int, feed_forward: bool = True) -> None:
        self.width, self.streams = int(width), int(streams)
        if not 1 <= self.streams <= kernels.MAX_STREAMS:
            raise ValueError(f"{self.streams} residual streams: the kernels take 1 to {kernels.MAX_STREAMS}")
        self.has_feed_forward = bool(feed_forward)
        self.roles = ("norm1", "mixer", "norm2", "feed_forward") if self.has_feed_forward else ("norm1", "mixer")

    def weight_requests(self) -> Dict[str, WeightRequest]:
        s, req = self.streams, {}
        for q in ("1", "2") if self.has_feed_forward else ("1",):
            req["in" + q] = WeightRequest((s,), VECTOR)
            req["out" + q] = WeightRequest((s,), VECTOR)
            req["mix" + q] = WeightRequest((s, s), VECTOR)
        return req

    # the arrangement reads ctx.pending_streams: a write that the sublayer before (of this layer or of
    # the one before) has left to be made together with this sublayer's read
    takes_pending_streams = True

    def _sublayer(self, ctx: StepContext, x: torch.Tensor, q: str, norm: Part, call) -> None:
        n, ws = ctx.n_rows, ctx.workspace
        u = ws.get("streams_read", n, self.width, torch.float32)
        y = ws.get("streams_update", n, self.width, torch.float32)
        if getattr(norm, "fusable_layer_norm", False):
            # one kernel: the write left over from the sublayer before, y cleared, this sublayer's
            # read and its LayerNorm
            h = ws.get("normed", n, self.width, ctx.dtype)
            kernels.streams_step(x, ctx.pending_streams, getattr(self, "in" + q), u, norm.weight, norm.bias, norm.eps,
                                 h, n, self.streams, zero=y)
            ctx.pending_streams = None
        else:
            flush_streams(ctx, x, self.streams)
            kernels.streams_read(x, getattr(self, "in" + q), u, n, self.streams, zero=y)
            h = LazyNorm(norm, u, n)
        call(h, y)
        ctx.pending_streams = (getattr(self, "mix" + q), getattr(self, "out" + q), y)

    def run(self, ctx, x, parts, bindings, position) -> None:
        mixer = parts["mixer"]
        self._sublayer(ctx, x, "1", parts["norm1"],
                       lambda h, y: mixer.forward_add(ctx, h, y, bindings["mixer"], position))
        if self.has_feed_forward:
            feed_forward = parts["feed_forward"]
            self._sublayer(ctx, x, "2", parts["norm2"], lambda h, y: feed_forward.forward_add(ctx, h, y))
