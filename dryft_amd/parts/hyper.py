"""Several copies of a float32 residual stream, read and written through learned weights (hyper-connections).

Instead of one stream ``x`` there are ``n`` copies ``x_1 .. x_n``, all equal to the embedding's output at the start.
A sublayer reads ``u = sum_s read[s] x_s`` through its norm, and its output ``y`` goes back to all copies at once:
``x_t <- sum_s mix[s, t] x_s + write[t] y`` (``mix`` is indexed ``[from, to]``). At the end the stream is the sum of
the copies. As with one stream, every update is folded into the read that follows it: a block hands its last
sublayer's output on unadded (``Deferred`` with the ``route`` it has to take), and the next read mixes the copies,
adds the output, writes them back, forms the weighted sum and norms it, in one launch.

``StreamRoute``   the three small tensors of one sublayer: ``read [n]``, ``write [n]``, ``mix [n, n]``.
``HyperBlock``    mixer and feed-forward, each behind a route and a norm; ``HyperMixerBlock`` has the mixer alone.
"""

from __future__ import annotations

import torch

from ..csrc import ops
from ..weights.spec import VECTOR
from . import register_block, register_part
from .base import Deferred, FeedForward, Mixer, Norm, Part, Partials, StepContext
from .stream import as_deferred


class StreamRoute(Part):
    def __init__(self, streams: int):
        self.streams = int(streams)
        if not 1 <= self.streams <= ops.HYPER_MAX_STREAMS:
            raise ValueError(f"1..{ops.HYPER_MAX_STREAMS} copies of the stream, got {streams}")
        self.read = self.write = self.mix = None

    def tensor_specs(self):
        n = self.streams
        return {"read": ((n,), VECTOR, "ones"), "write": ((n,), VECTOR, "ones"), "mix": ((n, n), VECTOR, "eye")}

    def load(self, tensors):
        self.read, self.write, self.mix = (tensors[k].float().contiguous() for k in ("read", "write", "mix"))

    def kernel_modules(self, dtype):
        return ("hyper",)

    def reads_whole(self) -> bool:
        return False


def _copies(x: torch.Tensor, pending: Deferred) -> int:
    if x.dim() == 3:
        return x.shape[0]
    if pending.route is not None:
        return pending.route.streams
    return 1


def read_streams(x: torch.Tensor, pending: Deferred, route: StreamRoute | None, norm, act: torch.dtype,
                 keep: bool = True, copies: int | None = None):
    """``(copies, h)``: the copies after ``pending`` has entered them (float32 ``[n, rows, width]``; updated in place
    where ``x`` already is such a tensor, None when not kept), and ``h = norm(sum_s read[s] x_s)`` in ``act``
    (``route`` None: the plain sum). ``x`` may still be the embedding's output ``[rows, width]``, which every copy
    equals."""
    if pending.norm is not None or pending.rows is not None or pending.vector is not None:
        raise ValueError("a stream of several copies takes a sublayer's output and nothing else")
    n = copies or (route.streams if route is not None else _copies(x, pending))
    rows, width = x.shape[-2:]
    out = None
    if keep:
        out = x if (x.dim() == 3 and x.dtype == torch.float32) else \
            torch.empty((n, rows, width), dtype=torch.float32, device=x.device)
    h = torch.empty((rows, width), dtype=act, device=x.device)
    delta = pending.delta
    if isinstance(delta, Partials):
        delta = (delta.data, delta.count)
    taken = pending.route
    ops.hyper_norm(x, n, delta, taken.mix if taken else None, taken.write if taken else None,
                   route.read if route is not None else None, norm.weight, norm.eps, out, h, normed=True)
    return out, h


def summed_streams(x: torch.Tensor, pending: Deferred) -> torch.Tensor:
    """The sum of the copies with what is pending entered, float32 ``[rows, width]`` (for looking at the stream)."""
    n = _copies(x, pending)
    rows, width = x.shape[-2:]
    out = torch.empty((rows, width), dtype=torch.float32, device=x.device)
    delta = pending.delta
    if isinstance(delta, Partials):
        delta = (delta.data, delta.count)
    taken = pending.route
    ops.hyper_norm(x, n, delta, taken.mix if taken else None, taken.write if taken else None, None, None, 0.0, None,
                   out, normed=False, act=taken.compute_dtype if taken else None)
    return out


class HyperBlock:
    roles = ("mixer_route", "mixer_norm", "mixer", "ffn_route", "ffn_norm", "ffn")

    def __init__(self, mixer_route: StreamRoute, mixer_norm: Norm, mixer: Mixer, ffn_route: StreamRoute | None = None,
                 ffn_norm: Norm | None = None, ffn: FeedForward | None = None):
        self.mixer_route, self.mixer_norm, self.mixer = mixer_route, mixer_norm, mixer
        self.ffn_route, self.ffn_norm, self.ffn = ffn_route, ffn_norm, ffn

    def parts(self):
        return {role: getattr(self, role) for role in self.roles}

    def forward(self, x, pending, ctx: StepContext, line, writes_cache: bool):
        x, h = read_streams(x, as_deferred(pending), self.mixer_route, self.mixer_norm, ctx.dtype)
        pending = Deferred(delta=self.mixer.forward(h, ctx, line, writes_cache), route=self.mixer_route)
        if self.ffn is None:
            return x, pending
        x, h = read_streams(x, pending, self.ffn_route, self.ffn_norm, ctx.dtype)
        return x, Deferred(delta=self.ffn.forward(h, ctx), route=self.ffn_route)


class HyperMixerBlock(HyperBlock):
    roles = ("mixer_route", "mixer_norm", "mixer")


register_part("stream_route", StreamRoute)
register_block("hyper", HyperBlock)
register_block("hyper_mixer", HyperMixerBlock)
