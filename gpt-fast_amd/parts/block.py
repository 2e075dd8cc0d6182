"""How norms, mixer, feed-forward and the residual stream are wired in one layer."""
import torch

from ..config.spec import LayerSpec
from ..ops import kernels as K
from ..ops import linear as L
from .base import (FEED_FORWARDS, MIXERS, NORMS, Param, Part, ResidualStream, Runtime, check_bound,
                   register_block)


class PreNormBlock(Part):
    """``h = x + mixer(norm1(x)); out = h + ffn(norm2(h))`` (reference model.py:161-164).
    The residual stream is float32 and updated in place; the sums happen in the
    parts' epilogues.  A spec without a feed-forward gives ``out = h``."""

    def __init__(self, spec: LayerSpec, runtime: Runtime):
        self.spec = spec
        self.mixer_norm = NORMS.build(spec.mixer_norm, runtime)
        self.mixer = MIXERS.build(spec.mixer, runtime)
        self.feed_forward_norm = self.feed_forward = None
        if spec.feed_forward is not None:
            self.feed_forward_norm = NORMS.build(spec.feed_forward_norm, runtime)
            self.feed_forward = FEED_FORWARDS.build(spec.feed_forward, runtime)

    def children(self):
        s = self.spec
        out = {s.mixer_norm_name: self.mixer_norm, s.mixer_name: self.mixer}
        if self.feed_forward is not None:
            out[s.feed_forward_norm_name] = self.feed_forward_norm
            out[s.feed_forward_name] = self.feed_forward
        return out

    def parameters(self):
        out = {}
        for child_name, child in self.children().items():
            for name, p in child.parameters().items():
                out[f"{child_name}.{name}"] = p
        return out

    def bind(self, tensors):
        for child_name, child in self.children().items():
            prefix = child_name + "."
            child.bind({k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)})

    def cache_need(self):
        return self.mixer.cache_need()

    def step_flops(self, q_lens, starts) -> float:
        """Matrix-product work of one run of this block (parts that do not say count as 0)."""
        return sum(getattr(c, "step_flops", lambda q, s: 0.0)(q_lens, starts)
                   for c in self.children().values())

    def unread_bytes(self, rows: int) -> int:
        """Bytes of this block's parameters that a step of ``rows`` tokens does not read."""
        return sum(getattr(c, "unread_bytes", lambda r: 0)(rows) for c in self.children().values())

    def step_fields(self):
        out = []
        for child in self.children().values():
            out += list(getattr(child, "step_fields", lambda: ())())
        return out

    # Reads the stream through ``stream.normed`` so that the kernel which completed it can
    # hand over the norm's rows (parts.base.ResidualStream); parts that do not put off their
    # sum get the plain tensor.
    takes_stream = True

    @property
    def replayable(self):
        return all(getattr(c, "replayable", False) for c in self.children().values())

    @property
    def takes_prepared(self):
        return getattr(self.mixer, "takes_prepared", False)

    @staticmethod
    def _residual_for(part, stream):
        return stream if getattr(part, "defers_sum", False) else stream.tensor

    def forward(self, residual, batch, entry):
        stream = residual if isinstance(residual, ResidualStream) else ResidualStream(residual)
        x = stream.normed(self.mixer_norm, reader=self.mixer)
        self.mixer.forward(x, batch, entry, self._residual_for(self.mixer, stream))
        if self.feed_forward is not None:
            h = stream.normed(self.feed_forward_norm, reader=self.feed_forward)
            self.feed_forward.forward(h, batch, self._residual_for(self.feed_forward, stream))
        if stream is not residual:
            stream.tensor                    # a caller with a plain tensor gets the sums now


# up to this many rows a sandwich block takes a sublayer's result as its last product's float32
# sums (the few-row kernels store them directly); measured on a 4,096-wide stack: 1.51 -> 1.44 ms
# a step at 8 rows, but 2.26 -> 2.82 ms at 64 rows and 12.5 -> 13.6 ms for 2,048 tokens
DIRECT_MAX_ROWS = 16


class ResultGate(Part):
    """``sigmoid(W h + b)``, which multiplies a sublayer's result element by element; h is what
    the sublayer reads.  This part makes the float32 sums ``W h``; the sigmoid, the bias and
    the multiplication belong to the kernel that joins the result to the stream."""

    replayable = True

    def __init__(self, dim: int, runtime: Runtime):
        self.dim = dim
        self.weight = self.bias = None

    def parameters(self):
        return {"weight": Param((self.dim, self.dim)),
                "bias": Param((self.dim,), role="vector", init="around_zero")}

    def bind(self, tensors):
        check_bound("ResultGate", self.parameters(), tensors)
        self.weight = tensors["weight"]
        self.bias = tensors["bias"].to(torch.float32).contiguous()

    def step_flops(self, q_lens, starts) -> float:
        return 2.0 * sum(q_lens) * self.dim * self.dim

    def sums(self, x):
        return L.linear(x, self.weight, out_dtype=torch.float32)


class SandwichNormBlock(PreNormBlock):
    """``h = x + norm1b(mixer(norm1(x))); out = h + norm2b(ffn(norm2(h)))``: a norm before
    each sublayer and a second one on its result, before that joins the stream.  A sublayer
    that offers ``forward_rows(x, batch[, entry]) -> float32 [N, D]`` hands its result over as
    its last product's float32 sums where that product is one of the library's own kernels
    with a float32 store (few rows, or the float32 engine); else it adds into a float32 tensor
    of its own, which starts at zero (with many bfloat16 rows the vendor library's bfloat16
    result plus the kernel that adds it is faster than its float32 result).  One kernel then norms the result, adds it to the stream and, where the
    block knows which norm reads the stream next (its own feed-forward's), applies that one in
    the same pass.

    With ``result_gate`` each sublayer's result is first multiplied, element by element, by
    ``sigmoid(W h + b)`` of what the sublayer read (the same kernel does it).  Such a block
    reads the stream through ``stream.normed`` and puts its last join off until the stream is
    read next, so that this kernel also makes the next reader's rows.  A norm of kind "none"
    before a sublayer hands it the stream itself, in the compute type."""

    takes_prepared = False

    @property
    def takes_stream(self):
        return self.gated

    def __init__(self, spec: LayerSpec, runtime: Runtime):
        super().__init__(spec, runtime)
        if spec.mixer_out_norm is None or (spec.feed_forward is not None
                                           and spec.feed_forward_out_norm is None):
            raise ValueError("a sandwich_norm block needs a norm on each sublayer's result")
        self.rt = runtime
        self.mixer_out_norm = NORMS.build(spec.mixer_out_norm, runtime)
        self.feed_forward_out_norm = None
        if spec.feed_forward is not None:
            self.feed_forward_out_norm = NORMS.build(spec.feed_forward_out_norm, runtime)
        self.gated = bool(getattr(spec, "result_gate", False))
        self.mixer_gate = self.feed_forward_gate = None
        if self.gated:
            dim = spec.mixer_out_norm.dim
            self.mixer_gate = ResultGate(dim, runtime)
            if spec.feed_forward is not None:
                self.feed_forward_gate = ResultGate(dim, runtime)

    def children(self):
        out = super().children()
        out[self.spec.mixer_out_norm_name] = self.mixer_out_norm
        if self.feed_forward is not None:
            out[self.spec.feed_forward_out_norm_name] = self.feed_forward_out_norm
        if self.mixer_gate is not None:
            out[self.spec.mixer_gate_name] = self.mixer_gate
        if self.feed_forward_gate is not None:
            out[self.spec.feed_forward_gate_name] = self.feed_forward_gate
        return out

    def _gated_join(self, residual, y, gate, gate_sums, out_norm, next_norm):
        """residual += out_norm(y * sigmoid(gate_sums + bias)); what ``next_norm`` makes of the
        sum, from the same kernel where it can (a norm per row and column, or none), else by
        the norm's own kernel; None without a next norm."""
        weight, eps = out_norm.row_and_column_form()
        bias = gate.bias if gate is not None else None
        if next_norm is None:
            K.gated_normed_add(residual, y, weight, eps, gate_sums, bias)
            return None
        if getattr(next_norm, "plain_rows", False):
            return K.gated_normed_add(residual, y, weight, eps, gate_sums, bias, next_plain=True,
                                      out_dtype=self.rt.dtype)
        form = getattr(next_norm, "row_and_column_form", None)
        if form is not None:
            next_weight, next_eps = form()
            return K.gated_normed_add(residual, y, weight, eps, gate_sums, bias,
                                      next_weight=next_weight, next_eps=next_eps,
                                      out_dtype=self.rt.dtype)
        K.gated_normed_add(residual, y, weight, eps, gate_sums, bias)
        return next_norm.forward(residual)

    def _forward_gated(self, stream, batch, entry):
        x = stream.normed(self.mixer_norm, reader=None)
        rows = stream.tensor
        y = self._result(self.mixer, (x, batch, entry), rows)
        g = self.mixer_gate.sums(x)
        if self.feed_forward is None:
            stream.defer(lambda r, then_norm, halves: self._gated_join(
                r, y, self.mixer_gate, g, self.mixer_out_norm, then_norm))
            return
        h = self._gated_join(rows, y, self.mixer_gate, g, self.mixer_out_norm, self.feed_forward_norm)
        y2 = self._result(self.feed_forward, (h, batch), rows)
        g2 = self.feed_forward_gate.sums(h)
        stream.defer(lambda r, then_norm, halves: self._gated_join(
            r, y2, self.feed_forward_gate, g2, self.feed_forward_out_norm, then_norm))

    @staticmethod
    def _result(part, args, like):
        """A sublayer's result alone, float32 [N, D]."""
        if hasattr(part, "forward_rows"):
            return part.forward_rows(*args)
        y = torch.zeros_like(like)
        part.forward(*args, y)
        return y

    def _join(self, residual, y, out_norm, next_norm):
        """residual += out_norm(y); the rows of ``next_norm`` over the sum, or None."""
        form = getattr(out_norm, "row_and_column_form", None)
        next_form = getattr(next_norm, "row_and_column_form", None)
        if form is None:
            K.add_into(residual, out_norm.forward(y))
            return None if next_norm is None else next_norm.forward(residual)
        weight, eps = form()
        if next_form is None:
            K.normed_add(residual, y, weight, eps)
            return None if next_norm is None else next_norm.forward(residual)
        next_weight, next_eps = next_form()
        return K.normed_add(residual, y, weight, eps, next_weight, next_eps, self.rt.dtype)

    def forward(self, residual, batch, entry):
        if self.gated:
            stream = residual if isinstance(residual, ResidualStream) else ResidualStream(residual)
            self._forward_gated(stream, batch, entry)
            if stream is not residual:
                stream.tensor                # a caller with a plain tensor gets the sums now
            return
        if isinstance(residual, ResidualStream):
            residual = residual.tensor
        direct = self.rt.is_float32 or residual.shape[0] <= DIRECT_MAX_ROWS
        x = self.mixer_norm.forward(residual)
        if direct and hasattr(self.mixer, "forward_rows"):
            y = self.mixer.forward_rows(x, batch, entry)
        else:
            y = torch.zeros_like(residual)
            self.mixer.forward(x, batch, entry, y)
        h = self._join(residual, y, self.mixer_out_norm, self.feed_forward_norm)
        if self.feed_forward is not None:
            if direct and hasattr(self.feed_forward, "forward_rows"):
                y = self.feed_forward.forward_rows(h, batch)
            else:
                y = torch.zeros_like(residual)
                self.feed_forward.forward(h, batch, y)
            self._join(residual, y, self.feed_forward_out_norm, None)


class LayerScale(Part):
    """A stored weight per element that multiplies a sublayer's result before it joins the
    stream; the multiplication belongs to the kernel that joins."""

    replayable = True

    def __init__(self, dim: int, runtime: Runtime):
        self.dim = dim
        self.weight = None

    def parameters(self):
        return {"weight": Param((self.dim,), role="vector", init="norm")}

    def bind(self, tensors):
        check_bound("LayerScale", self.parameters(), tensors)
        self.weight = tensors["weight"].to(torch.float32).contiguous()


class PostNormBlock(PreNormBlock):
    """``h = norm1(a x + ls1 * mixer(read(x))); out = norm2(a h + ls2 * ffn(read(h)))``: the
    norm stands after the sum, so the stream itself is normed; ``a`` is the spec's
    ``residual_scale``, ``ls`` a stored weight per element (``layer_scale``), ``read`` the
    spec's ``mixer_norm`` / ``feed_forward_norm`` (kind "none": the sublayers read the stream
    itself).  A sublayer hands over its result alone (``forward_rows``); one kernel scales,
    adds, norms, writes the stream back and makes the next reader's rows in the compute type.
    The last join of a layer is put off until the stream is read next, so that it serves the
    next layer's reader (or leaves the rows to the final norm).  A mixer that offers
    ``forward_branches`` (two results that are each RMS-normed and averaged) has that
    combination done by the same kernel."""

    takes_stream = True
    takes_prepared = False

    def __init__(self, spec: LayerSpec, runtime: Runtime):
        super().__init__(spec, runtime)
        if spec.mixer_out_norm is None or (spec.feed_forward is not None
                                           and spec.feed_forward_out_norm is None):
            raise ValueError("a post_norm block needs the norm of each sum")
        self.rt = runtime
        self.mixer_out_norm = NORMS.build(spec.mixer_out_norm, runtime)
        self.feed_forward_out_norm = None
        if spec.feed_forward is not None:
            self.feed_forward_out_norm = NORMS.build(spec.feed_forward_out_norm, runtime)
        for norm in (self.mixer_out_norm, self.feed_forward_out_norm):
            if norm is not None and not hasattr(norm, "layer_form"):
                raise TypeError("a post_norm block's sums take a norm with layer_form() (kind 'layer')")
        self.alpha = float(spec.residual_scale)
        self.mixer_scale = self.feed_forward_scale = None
        if spec.layer_scale:
            dim = spec.mixer_out_norm.dim
            self.mixer_scale = LayerScale(dim, runtime)
            if spec.feed_forward is not None:
                self.feed_forward_scale = LayerScale(dim, runtime)

    def children(self):
        out = super().children()
        out[self.spec.mixer_out_norm_name] = self.mixer_out_norm
        if self.feed_forward is not None:
            out[self.spec.feed_forward_out_norm_name] = self.feed_forward_out_norm
        if self.mixer_scale is not None:
            out[self.spec.mixer_scale_name] = self.mixer_scale
        if self.feed_forward_scale is not None:
            out[self.spec.feed_forward_scale_name] = self.feed_forward_scale
        return out

    def _join(self, residual, result, scale, out_norm, next_norm):
        """residual <- out_norm(alpha * residual + scale * result); what ``next_norm`` makes of
        the new stream, from the same kernel where that is the rows themselves, else by the
        norm's own kernel; None without a next norm.  ``result`` is a tensor or a
        ``(first, second, (w_first, w_second), eps)`` of two branches."""
        weight, eps = out_norm.layer_form()
        ls = scale.weight if scale is not None else None
        plain = next_norm is not None and getattr(next_norm, "plain_rows", False)
        args = dict(alpha=self.alpha, layer_scale=ls, out_dtype=self.rt.dtype if plain else None)
        if isinstance(result, tuple):
            first, second, weights, branch_eps = result
            out = K.post_norm_join(residual, first, weight, eps, second=second,
                                   branch_weights=weights, branch_eps=branch_eps, **args)
        else:
            out = K.post_norm_join(residual, result, weight, eps, **args)
        if next_norm is None or plain:
            return out
        return next_norm.forward(residual)

    @staticmethod
    def _result(part, args, like):
        if hasattr(part, "forward_branches"):
            return part.forward_branches(*args)
        if hasattr(part, "forward_rows"):
            return part.forward_rows(*args)
        y = torch.zeros_like(like)
        part.forward(*args, y)
        return y

    def forward(self, residual, batch, entry):
        stream = residual if isinstance(residual, ResidualStream) else ResidualStream(residual)
        x = stream.normed(self.mixer_norm, reader=None)
        rows = stream.tensor
        y = self._result(self.mixer, (x, batch, entry), rows)
        if self.feed_forward is None:
            stream.defer(lambda r, then_norm, halves: self._join(
                r, y, self.mixer_scale, self.mixer_out_norm, then_norm))
        else:
            h = self._join(rows, y, self.mixer_scale, self.mixer_out_norm, self.feed_forward_norm)
            y2 = self._result(self.feed_forward, (h, batch), rows)
            stream.defer(lambda r, then_norm, halves: self._join(
                r, y2, self.feed_forward_scale, self.feed_forward_out_norm, then_norm))
        if stream is not residual:
            stream.tensor                    # a caller with a plain tensor gets the sums now


register_block("pre_norm", PreNormBlock)
register_block("post_norm", PostNormBlock)
register_block("sandwich_norm", SandwichNormBlock)
