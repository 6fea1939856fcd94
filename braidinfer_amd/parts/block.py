"""Arrangements of a layer's parts.  `prenorm_residual`: x += mixer(norm(x)), then
x += feed_forward(norm(x)), with the layer's norms of the roles "mixer" and "feed_forward"
(reference: the per-layer emit order, megakernel/megakernel_compile.rs:115-236,
compile_attention.rs:78-376, compile_layers.rs:373-386).  The parts add into `x`
themselves, so the sum is part of their last projection.

`sandwich_residual` norms a half's output too before the sum; `parallel_residual` runs both halves on one
normed input, x += mixer(norm(x)) + feed_forward(norm(x)).

An arrangement is an object with `run(layer, x, step, mixer_ctx)`; it reads whatever roles
of `layer.norms` it likes.  It may also have `first_norm(layer)`: the norm that reads the
residual rows first when the layer runs, which lets the layer before prepare that norm
inside its last product (see `parts.base.ResidualSink`); arrangements without it, and plain
functions `f(layer, x, step, mixer_ctx)`, work the same without that shortcut.  After the
mixer half and after the whole layer it calls `step.probe(name, x)` when the step carries
a probe (names as the reference's tracer, crates/braidinfer-runtime/src/tracer.rs:94-160).
"""
from __future__ import annotations

from .base import NormedInput, ResidualSink, register_part


def run_residual_branch(part, norm, next_norm, x, step, dtype, *extra) -> None:
    """One residual branch: x += part(norm(x)).  A part that works through `linear` only gets
    the norm unrun (with what the product before prepared for it, if that was this norm and
    these rows) and the residual rows together with the norm that reads them next."""
    prepared, step.prepared_norm = step.prepared_norm, None
    if not part.through_linear_only:
        h = x
        if norm is not None:
            h = step.ws.get("block_h", tuple(x.shape), dtype)
            norm.forward(x, h)
        part.forward(h, x, step, *extra)
        return
    h = x
    if norm is not None:
        mine = prepared[2] if prepared is not None and prepared[0] is norm and prepared[1] is x else None
        if isinstance(mine, tuple) and mine[:1] == ("normed",):
            mine = None            # rows another arrangement normed ahead: not a product's preparation; norm again
        h = NormedInput(x, norm, step.ws, dtype, mine)
    sink = ResidualSink(x, next_norm)
    part.forward(h, sink, step, *extra)
    if sink.prepared is not None:
        step.prepared_norm = (next_norm, x, sink.prepared)


class PrenormResidual:
    def first_norm(self, layer):
        return layer.norms.get("mixer") if layer.mixer is not None else layer.norms.get("feed_forward")

    def run(self, layer, x, step, mixer_ctx) -> None:
        after = step.norm_after_layer          # the norm that reads x after this layer, if known
        ffn_norm = layer.norms.get("feed_forward")
        if layer.mixer is not None:
            nxt = ffn_norm if layer.feed_forward is not None else after
            run_residual_branch(layer.mixer, layer.norms.get("mixer"), nxt, x, step, layer.rt.dtype, mixer_ctx)
        if step.probe is not None:
            step.probe(f"L{step.schedule_index}.post_mixer", x)
        if layer.feed_forward is not None:
            run_residual_branch(layer.feed_forward, ffn_norm, after, x, step, layer.rt.dtype)
        if step.probe is not None:
            step.probe(f"L{step.schedule_index}.post_ffn", x)


class SandwichResidual:
    """x += norm_out(part(norm_in(x))) for the mixer and then for the feed-forward: a norm in front
    of each half and one behind it, before the sum.  Roles of `layer.norms`: "mixer", "mixer_out",
    "feed_forward", "feed_forward_out" (an absent one is left out).  The half writes its output
    into float rows of its own; the norm behind it adds the normed rows to the residual rows, so
    the sum is a float add in that kernel, and where it can it also leaves the norm that reads the
    rows next (the other half's, or the next layer's first) in the same pass."""

    def first_norm(self, layer):
        return layer.norms.get("mixer") if layer.mixer is not None else layer.norms.get("feed_forward")

    def run(self, layer, x, step, mixer_ctx) -> None:
        after = step.norm_after_layer          # the norm that reads x after this layer, if known
        ffn_norm = layer.norms.get("feed_forward")
        if layer.mixer is not None:
            nxt = ffn_norm if layer.feed_forward is not None else after
            self.branch(layer.mixer, layer.norms.get("mixer"), layer.norms.get("mixer_out"), nxt, x, step, layer.rt.dtype, mixer_ctx)
        if step.probe is not None:
            step.probe(f"L{step.schedule_index}.post_mixer", x)
        if layer.feed_forward is not None:
            self.branch(layer.feed_forward, ffn_norm, layer.norms.get("feed_forward_out"), after, x, step, layer.rt.dtype)
        if step.probe is not None:
            step.probe(f"L{step.schedule_index}.post_ffn", x)

    @staticmethod
    def branch(part, norm_in, norm_out, next_norm, x, step, dtype, *extra) -> None:
        prepared, step.prepared_norm = step.prepared_norm, None
        h = x
        if norm_in is not None:
            # two buffers in turn: the norm behind this half writes the next half's input while this one's is read
            if isinstance(prepared, tuple) and len(prepared) == 3 and prepared[0] is norm_in and prepared[1] is x \
                    and isinstance(prepared[2], tuple) and prepared[2][0] == "normed":
                h = prepared[2][1]
            else:
                h = step.ws.get("block_h", tuple(x.shape), dtype)
                norm_in.forward(x, h)
        if norm_out is None:
            part.forward(h, x, step, *extra)
            return
        y = step.ws.get("branch_out", tuple(x.shape), x.dtype)
        if part.through_linear_only:
            part.forward(h, ResidualSink(y, None, overwrite=True), step, *extra)
        else:
            y.zero_()
            part.forward(h, y, step, *extra)
        h_next = None
        if next_norm is not None and next_norm.then_args() is not None:
            name = "block_h2" if h is not x and h.data_ptr() == step.ws.get("block_h", tuple(x.shape), dtype).data_ptr() else "block_h"
            h_next = step.ws.get(name, tuple(x.shape), dtype)
        if norm_out.add_normed(y, x, next_norm if h_next is not None else None, h_next):
            step.prepared_norm = (next_norm, x, ("normed", h_next))


class ParallelResidual:
    """x += mixer(n) + feed_forward(n) with n = norm(x): one norm (role "mixer") whose output both halves read.
    Each half adds its output into the residual rows in its last product, the mixer first; neither reads the rows."""

    def first_norm(self, layer):
        return None          # the norm's output is kept for both halves: nothing a product before could prepare in passing

    def run(self, layer, x, step, mixer_ctx) -> None:
        step.prepared_norm = None
        dtype = layer.rt.dtype
        norm = layer.norms.get("mixer")
        h = x
        if norm is not None:
            h = step.ws.get("block_h", tuple(x.shape), dtype)
            norm.forward(x, h)
        if layer.mixer is not None:
            layer.mixer.forward(h, x, step, mixer_ctx)
        if step.probe is not None:
            step.probe(f"L{step.schedule_index}.post_mixer", x)
        if layer.feed_forward is not None:
            layer.feed_forward.forward(h, x, step)
        if step.probe is not None:
            step.probe(f"L{step.schedule_index}.post_ffn", x)


class PrenormSideBySide:
    """x += sum over the layer's mixers of norm_out(mixer(n)) with n = norm(x), then x += feed_forward(norm(x)): several
    mixers side by side on one normed input (`layer.mixer` and `layer.more_mixers`), each with a norm of its own
    behind it before the sum.  Roles of `layer.norms`: "mixer" (in front), "mixer_out" for `layer.mixer` and
    "mixer_out.<role>" for the others (an absent one: the mixer adds into the rows itself), "feed_forward".  A
    weighting of the sum (a mean, a residual multiplier) is the norms' business (`scale` of an RMS norm).  Each mixer
    writes float rows of its own; the norm behind it adds the normed rows to the residual rows."""

    def first_norm(self, layer):
        return None          # the norm's output is kept for all mixers: nothing a product before could prepare in passing

    def run(self, layer, x, step, mixer_ctx) -> None:
        step.prepared_norm = None
        dtype = layer.rt.dtype
        norm = layer.norms.get("mixer")
        h = x
        if norm is not None:
            h = step.ws.get("block_h", tuple(x.shape), dtype)
            norm.forward(x, h)
        mixers = ([(None, layer.mixer, mixer_ctx)] if layer.mixer is not None else []) + \
                 [(role, m, mixer_ctx.others[role]) for role, m in layer.more_mixers.items()]
        for role, mixer, ctx in mixers:
            norm_out = layer.norms.get("mixer_out" if role is None else "mixer_out." + role)
            if norm_out is None:
                mixer.forward(h, x, step, ctx)
                continue
            y = step.ws.get("branch_out", tuple(x.shape), x.dtype)
            if mixer.through_linear_only:
                mixer.forward(h, ResidualSink(y, None, overwrite=True), step, ctx)
            else:
                y.zero_()
                mixer.forward(h, y, step, ctx)
            norm_out.add_normed(y, x)
        if step.probe is not None:
            step.probe(f"L{step.schedule_index}.post_mixer", x)
        if layer.feed_forward is not None:
            run_residual_branch(layer.feed_forward, layer.norms.get("feed_forward"), step.norm_after_layer, x, step, dtype)
        if step.probe is not None:
            step.probe(f"L{step.schedule_index}.post_ffn", x)


register_part("block", "prenorm_residual", PrenormResidual, replace=True)
register_part("block", "prenorm_side_by_side", PrenormSideBySide, replace=True)
register_part("block", "parallel_residual", ParallelResidual, replace=True)
register_part("block", "sandwich_residual", SandwichResidual, replace=True)
