"""A block: a mixer, a feed-forward and their norm(s) in one of the known arrangements."""

from __future__ import annotations

from typing import Callable, Dict, Optional

import torch

from .base import LayerCache, Part, SideLinear, build_part
from .specs import LayerSpec, ParamSpec


def _parallel_few_rows(block: "Block", x, batch, cache, normed, then, handed) -> bool:
    """The parallel block for a few bf16 rows in three launches: norm + both first linears, the
    mixer's core, both last linears + residual. Needs a mixer and a feed-forward that offer their
    stages (``input_projection`` / ``output_projection``); returns ``False`` otherwise.
    ``normed``: the block's norm of ``x``, where the block before has computed it; ``then``: the norm
    the next block starts with, which the last launch computes as well where it pays (``handed``, a
    list, then gets the normalised rows)."""
    from ..ops import fast
    from ..ops.linear import linear

    n = x.shape[0]
    if block.dtype != torch.bfloat16 or n > fast.SKINNY_MAX_ROWS or block.feed_forward is None:
        return False
    m_in, f_in = block.mixer.input_projection(), block.feed_forward.input_projection()
    m_out, f_out = block.mixer.output_projection(), block.feed_forward.output_projection()
    if m_in is None or f_in is None or m_out is None or f_out is None:
        return False
    ws = batch.workspace
    projected = ws.get("block.mixer_in", (n, m_in[2]), block.dtype)
    hidden = ws.get("block.ff_hidden", (n, f_in[2]), block.dtype)
    norm = block.norm
    fused = False
    beside = None
    if normed is not None:
        fused = fast.linear_two_outputs(normed, m_in[0], m_in[1], projected, 0, f_in[0], f_in[1], hidden, f_in[3])
    ln = norm.layernorm_operands()            # (a norm of another form is run through its own forward below)
    rms = norm.rms_operands() if ln is None and callable(getattr(norm, "rms_operands", None)) else None
    if not fused and fast.FUSE_LAYERNORM_PROLOGUE and rms is not None:
        # a root-mean-square norm in the prologue of the launch that projects for the mixer and the feed-forward
        fused = fast.layernorm_linear(x, rms[0], None, rms[1], m_in[0], m_in[1], projected, 0, f_in[0], f_in[1], hidden, f_in[3],
                                      centred=False)
    if not fused and fast.FUSE_LAYERNORM_PROLOGUE and ln is not None:
        # the feed-forward's first linear goes into the mixer's launch where the mixer takes it (the
        # launch of the mixer's first linear then leaves the normalised rows for it), else into the
        # launch of the mixer's first linear
        h = ws.get("block.h", tuple(x.shape), block.dtype)
        job = SideLinear(h, f_in[0], f_in[1], hidden, f_in[3])
        if block.mixer.takes_beside(job, batch, cache) and \
                fast.layernorm_linear(x, *ln, m_in[0], m_in[1], projected, 0, store=h):
            fused, beside = True, job
        else:
            fused = fast.layernorm_linear(x, *ln, m_in[0], m_in[1], projected, 0, f_in[0], f_in[1], hidden, f_in[3])
    if not fused:
        h = ws.get("block.h", tuple(x.shape), block.dtype)
        norm.forward(x, h)
        if not fast.linear_two_outputs(h, m_in[0], m_in[1], projected, 0, f_in[0], f_in[1], hidden, f_in[3]):
            linear(h, m_in[0], m_in[1], projected)
            linear(h, f_in[0], f_in[1], hidden, act=f_in[3])
    mixed = block.mixer.attend(projected, batch, cache, beside) if beside is not None \
        else block.mixer.attend(projected, batch, cache)
    # More rows than the next block's first launch normalises by itself, or a last launch of this block that
    # ends in a kernel that finishes whole rows anyway: the next block's norm is computed here, by that
    # kernel, instead of in a launch or a prologue of its own (9 to 16 rows of 2048: 1 to 2 % of a step;
    # rows of 2560, which leave the prologue's kernel no registers for a third strip of weights in flight, from
    # 5 rows on: 3 to 4 %).
    handing = n > fast.SKINNY_LN_MAX_ROWS or fast.pair_finishes_rows(n, x.shape[1])
    then_ln = then.layernorm_operands() if then is not None and handing else None
    if then_ln is not None:
        rows = ws.get("block.handed", tuple(x.shape), block.dtype)
        if fast.linear_pair_accumulate(mixed, m_out[0], m_out[1], hidden, f_out[0], f_out[1], x,
                                       then_norm=(*then_ln, rows)):
            handed.append(rows)
            return True
    if not fast.linear_pair_accumulate(mixed, m_out[0], m_out[1], hidden, f_out[0], f_out[1], x):
        linear(mixed, m_out[0], m_out[1], x, accumulate=True)
        linear(hidden, f_out[0], f_out[1], x, accumulate=True)
    return True


def _parallel(block: "Block", x, batch, cache, normed=None, then=None):
    """``x + mixer(norm(x)) + ff(norm(x))``: both branches read the same normalised input (a block without a
    feed-forward has the first branch only).

    Reference: ``kestrel/models/moondream/text.py:222-275``.
    """
    handed = []
    if _parallel_few_rows(block, x, batch, cache, normed, then, handed):
        return handed[0] if handed else None
    h = normed
    if h is None:
        h = batch.workspace.get("block.h", tuple(x.shape), block.dtype)
        block.norm.forward(x, h)
    block.mixer.forward(h, batch, cache, x)
    if block.feed_forward is not None:
        block.feed_forward.forward(h, batch, x)
    return None


_parallel.hands_over = True


def _sequential_few_rows(block: "Block", x, batch, cache) -> bool:
    """The sequential block for a few bf16 rows: each norm in the prologue of the launch that reads it (the mixer's first
    linear; the feed-forward's first linear where it offers ``from_stream``). Needs a root-mean-square norm and a mixer
    that offers its stages; returns ``False`` (nothing was run) otherwise."""
    from ..ops import fast
    from ..ops.linear import linear

    n = x.shape[0]
    if block.dtype != torch.bfloat16 or n > fast.SKINNY_LN_MAX_ROWS or not fast.FUSE_LAYERNORM_PROLOGUE:
        return False
    rms = block.norm.rms_operands() if callable(getattr(block.norm, "rms_operands", None)) else None
    m_in, m_out = block.mixer.input_projection(), block.mixer.output_projection()
    if rms is None or m_in is None or m_out is None:
        return False
    ws = batch.workspace
    projected = ws.get("block.mixer_in", (n, m_in[2]), block.dtype)
    if not fast.layernorm_linear(x, rms[0], None, rms[1], m_in[0], m_in[1], projected, 0, centred=False):
        return False
    linear(block.mixer.attend(projected, batch, cache), m_out[0], m_out[1], x, accumulate=True)
    if block.feed_forward is not None:
        from_stream = getattr(block.feed_forward, "from_stream", None)
        if from_stream is None or not from_stream(x, block.norm2, batch):
            h = ws.get("block.h", tuple(x.shape), block.dtype)
            block.norm2.forward(x, h)
            block.feed_forward.forward(h, batch, x)
    return True


def _sequential(block: "Block", x, batch, cache) -> None:
    """``x += mixer(norm(x)); x += ff(norm2(x))``; without a feed-forward the first half only."""
    if _sequential_few_rows(block, x, batch, cache):
        return
    h = batch.workspace.get("block.h", tuple(x.shape), block.dtype)
    block.norm.forward(x, h)
    block.mixer.forward(h, batch, cache, x)
    if block.feed_forward is not None:
        block.norm2.forward(x, h)
        block.feed_forward.forward(h, batch, x)


# Whether a block of weighted branches leaves the sum ``x += scale * delta`` to whoever reads the stream next (the
# next such block adds it in the pass that computes its norms; anything else calls ``settle`` first) instead of
# adding it in a launch of its own. Off: every block leaves the stream complete (what a test that reads the
# stream between blocks needs).
DEFER_RESIDUAL = True
_PENDING = "residual_pending"


def settle(x, batch) -> None:
    """Add what a block before has left to be added into the fp32 stream ``x``."""
    from ..ops import core

    host = getattr(batch, "host", None)
    pending = host.pop(_PENDING, None) if host else None
    if pending is not None:
        core.add_scaled(x, pending[0], pending[1])


def _two_branches_by_stages(block: "Block", h1, h2, batch, cache, delta) -> bool:
    """Both branches through the stages that mixer and feed-forward offer, so that the first of the last linears
    writes ``delta`` and nobody has to clear it: for a few bf16 rows the two last linears are one launch.
    ``False``: a part offers no stages (its ``forward`` then adds into a cleared ``delta``)."""
    from ..ops import fast
    from ..ops.linear import linear

    n = h1.shape[0]
    ff = block.feed_forward
    m_in, m_out = block.mixer.input_projection(), block.mixer.output_projection()
    f_in, f_out = (ff.input_projection(), ff.output_projection()) if ff is not None else (None, None)
    if m_in is None or m_out is None or (ff is not None and (f_in is None or f_out is None)):
        return False
    ws = batch.workspace
    projected = ws.get("block.mixer_in", (n, m_in[2]), block.dtype)
    linear(h1, m_in[0], m_in[1], projected)
    hidden = None
    if ff is not None:
        hidden = ws.get("block.ff_hidden", (n, f_in[2]), block.dtype)
        linear(h2, f_in[0], f_in[1], hidden, act=f_in[3])
    mixed = block.mixer.attend(projected, batch, cache)
    if ff is not None and block.dtype == torch.bfloat16 and n <= fast.SKINNY_MAX_ROWS and \
            fast.linear_pair_accumulate(mixed, m_out[0], m_out[1], hidden, f_out[0], f_out[1], delta, accumulate=False):
        return True
    linear(mixed, m_out[0], m_out[1], delta)
    if ff is not None:
        linear(hidden, f_out[0], f_out[1], delta, accumulate=True)
    return True


def _parallel_two_norms(block: "Block", x, batch, cache) -> None:
    """``x + residual_scale * (mixer(norm(x)) + ff(norm2(x)))``: two branches, each with a norm of its own of the
    same ``x``; without a feed-forward, ``x + residual_scale * mixer(norm(x))``.

    Both norms come from one pass over ``x`` where they are LayerNorms of one eps; that pass also adds what the
    block before has left to be added (``DEFER_RESIDUAL``). The branches' sum is kept in a buffer of its own and
    enters the stream with the weight in fp32, like the stream."""
    from ..ops import core

    ws = batch.workspace
    h1 = ws.get("block.h", tuple(x.shape), block.dtype)
    delta = ws.get("block.delta", tuple(x.shape), torch.float32)
    ff = block.feed_forward
    ln1 = block.norm.layernorm_operands()
    ln2 = block.norm2.layernorm_operands() if ff is not None else None
    h2 = ws.get("block.h2", tuple(x.shape), block.dtype) if ff is not None else None
    host = batch.host
    pending = host.get(_PENDING)
    if pending is not None and pending[0].data_ptr() != delta.data_ptr():
        settle(x, batch)              # (left in another buffer than this block's)
        pending = None
    # parts that offer their stages write the buffer; parts that only add need it cleared
    staged = block.mixer.input_projection() is not None and block.mixer.output_projection() is not None and \
        (ff is None or (ff.input_projection() is not None and ff.output_projection() is not None))
    sum_args = dict(delta=delta if (pending is not None or not staged) else None, scale=pending[1] if pending else 1.0,
                    apply=pending is not None, clear=not staged)
    if ln1 is not None and (ff is None or (ln2 is not None and float(ln2[2]) == float(ln1[2]))):
        core.layernorm_pair(x, ln1, ln2, h1, h2, **sum_args)
    else:
        core.layernorm_pair(x, None, None, None, None, **sum_args)
        block.norm.forward(x, h1)
        if ff is not None:
            block.norm2.forward(x, h2)
    host.pop(_PENDING, None)
    if not (staged and _two_branches_by_stages(block, h1, h2, batch, cache, delta)):
        block.mixer.forward(h1, batch, cache, delta)
        if ff is not None:
            ff.forward(h2, batch, delta)
    if DEFER_RESIDUAL:
        host[_PENDING] = (delta, float(block.spec.residual_scale))
    else:
        core.add_scaled(x, delta, block.spec.residual_scale)


_parallel_two_norms.defers = True


def _output_norms(block: "Block", x, batch, cache) -> None:
    """``x += norm(mixer(x)); x += norm2(ff(x))``: the parts read the stream itself (rounded to the activation type, or,
    for a mixer that says ``reads_stream``, as it is) and the norms stand behind them. Each part writes its output into
    an fp32 buffer (``mix``; a part without it adds into a cleared buffer through ``forward``), and the norm's kernel adds
    the normalised rows into the stream (``Norm.add_normed``)."""
    from ..ops import core

    ws = batch.workspace
    delta = ws.get("block.delta", tuple(x.shape), torch.float32)

    def rounded():
        if block.dtype == torch.float32:
            return x
        h = ws.get("block.h", tuple(x.shape), block.dtype)
        core.cast_columns(x, h)
        return h

    def add(norm, also_rounded: bool = False) -> bool:
        """``x += norm(delta)``; with ``also_rounded`` the stream's rounding is left in ``block.h`` by the same launch where
        the norm offers that (returns whether it did)."""
        if callable(getattr(norm, "add_normed", None)):
            if also_rounded and block.dtype != torch.float32:
                norm.add_normed(delta, x, rounded=ws.get("block.h", tuple(x.shape), block.dtype))
                return True
            norm.add_normed(delta, x)
            return False
        normed = ws.get("block.normed", tuple(x.shape), torch.float32)
        norm.forward(delta, normed)
        core.add_scaled(x, normed, 1.0)
        return False

    mixer = block.mixer
    source = x if getattr(mixer, "reads_stream", False) else rounded()
    if callable(getattr(mixer, "mix", None)):
        mixer.mix(source, batch, cache, delta, False)
    else:
        delta.zero_()
        mixer.forward(source, batch, cache, delta)
    ff = block.feed_forward
    left = add(block.norm, also_rounded=ff is not None)
    if ff is not None:
        # (the feed-forward reads the stream's rounding, which the launch before has left where the norm could)
        h = ws.get("block.h", tuple(x.shape), block.dtype) if left else rounded()
        if callable(getattr(ff, "mix", None)):
            ff.mix(h, batch, delta, False)
        else:
            delta.zero_()
            ff.forward(h, batch, delta)
        add(block.norm2)


ARRANGEMENTS: Dict[str, Callable] = {"parallel": _parallel, "sequential": _sequential,
                                     "parallel_two_norms": _parallel_two_norms, "output_norms": _output_norms}


def register_arrangement(name: str, fn: Callable) -> None:
    """``fn(block, x, batch, cache)`` updates the fp32 residual ``x`` in place. A function with the
    attribute ``hands_over = True`` is called as ``fn(block, x, batch, cache, normed=, then=)``:
    ``normed`` is ``block.norm`` of ``x`` if the block before has computed it (else ``None``), ``then``
    the first norm of the block that follows (or ``None``); it may return that norm of its result, or
    ``None``."""
    ARRANGEMENTS[name] = fn


class Block:
    """Parts of one layer, built from its specification through the registries."""

    def __init__(self, spec: LayerSpec) -> None:
        if spec.arrangement not in ARRANGEMENTS:
            raise ValueError(f"unknown arrangement {spec.arrangement!r}; known: {', '.join(sorted(ARRANGEMENTS))}")
        self.spec = spec
        self.norm = build_part("norm", spec.norm)
        self.norm2 = build_part("norm", spec.norm2) if spec.norm2 is not None else None
        if spec.arrangement == "sequential" and self.norm2 is None and spec.feed_forward is not None:
            raise ValueError("the sequential arrangement needs norm2 for its feed-forward")
        self.mixer = build_part("mixer", spec.mixer)
        if spec.arrangement == "output_norms" and self.norm2 is None and spec.feed_forward is not None:
            raise ValueError("the output_norms arrangement needs norm2 for its feed-forward")
        if spec.feed_forward is None and spec.arrangement not in ("parallel_two_norms", "parallel", "sequential", "output_norms"):
            raise ValueError(f"the {spec.arrangement} arrangement needs a feed-forward")
        if spec.arrangement == "parallel_two_norms" and spec.feed_forward is not None and self.norm2 is None:
            raise ValueError("the parallel_two_norms arrangement needs norm2 for its feed-forward")
        self.feed_forward = build_part("feed_forward", spec.feed_forward) if spec.feed_forward is not None else None
        self.dtype: Optional[torch.dtype] = None
        self._run = ARRANGEMENTS[spec.arrangement]

    def parts(self) -> Dict[str, Part]:
        out = {"norm": self.norm, "mixer": self.mixer}
        if self.feed_forward is not None:
            out["feed_forward"] = self.feed_forward
        if self.norm2 is not None:
            out["norm2"] = self.norm2
        return out

    def params(self) -> Dict[str, ParamSpec]:
        """Checkpoint tensor name -> spec, for every tensor of this layer."""
        out = {}
        for part_name, part in self.parts().items():
            for local, pspec in part.params().items():
                key = f"{part_name}.{local}"
                if key not in self.spec.names:
                    raise ValueError(f"the architecture names no tensor for {key!r}")
                out[self.spec.names[key]] = pspec
        return out

    def bind(self, tensors: Dict[str, torch.Tensor], dtype, device) -> None:
        self.dtype = dtype
        for part_name, part in self.parts().items():
            local = {name: tensors[self.spec.names[f"{part_name}.{name}"]] for name in part.params()}
            part.bind(local, dtype, device)

    def forward(self, x: torch.Tensor, batch, cache: LayerCache, normed: Optional[torch.Tensor] = None,
                then: Optional[Part] = None) -> Optional[torch.Tensor]:
        """Updates the fp32 residual ``x`` in place. ``normed``: this block's first norm of ``x``, if the
        block before has computed it; ``then``: the first norm of the block that follows. Returns that
        norm of the result where the block's last launch computed it, else ``None``."""
        if not getattr(self._run, "defers", False):
            settle(x, batch)          # (an arrangement that knows nothing of sums left to be added)
        if getattr(self._run, "hands_over", False):
            return self._run(self, x, batch, cache, normed=normed, then=then)
        self._run(self, x, batch, cache)
        return None
