"""Position encodings of attention.

A position encoding turns the fused projection ``qkv`` of a step into rotated queries and
writes keys and values into the cache entry.  Rotary encodings differ only in their
frequency vector, pair layout and rotary width, all parameters of one kernel.
"""
import math

import torch

from ..config.spec import PositionSpec
from ..ops import kernels as K
from ..ops import linear as L
from .base import Param, Part, Runtime, check_bound, register_position


def rotary_frequencies(rotary_dim: int, base: float) -> torch.Tensor:
    """f_i = 1 / base^(2i / rotary_dim) in float32 (reference model.py:271)."""
    idx = torch.arange(0, rotary_dim, 2)[: rotary_dim // 2].float()
    return 1.0 / (base ** (idx / rotary_dim))


def llama3_scaled(freqs: torch.Tensor, factor: float, low_freq_factor: float,
                  high_freq_factor: float, original_max_position_embeddings: float,
                  **_ignored) -> torch.Tensor:
    """Llama-3.1 rescale by wavelength (reference model.py:244-263): wavelengths below
    orig/high are kept, above orig/low divided by ``factor``, between blended."""
    orig = original_max_position_embeddings
    low_wavelen = orig / low_freq_factor
    high_wavelen = orig / high_freq_factor
    wavelen = 2 * math.pi / freqs
    if high_freq_factor == low_freq_factor:
        blended = freqs
    else:
        smooth = (orig / wavelen - low_freq_factor) / (high_freq_factor - low_freq_factor)
        blended = (1 - smooth) * freqs / factor + smooth * freqs
    return torch.where(wavelen < high_wavelen, freqs,
                       torch.where(wavelen > low_wavelen, freqs / factor, blended))


def linear_scaled(freqs: torch.Tensor, factor: float, **_ignored) -> torch.Tensor:
    """Position interpolation: every frequency divided by ``factor``."""
    return freqs / float(factor)


def yarn_scaled(freqs: torch.Tensor, factor: float, original: float, fast: float, slow: float,
                base: float, **_ignored) -> torch.Tensor:
    """The slow end of the ladder divided by ``factor`` along a linear ramp.  With n = 2 len(freqs)
    rotated elements, ``place(t) = n ln(original / (2 pi t)) / (2 ln base)`` is the index whose
    pair makes ``t`` full turns over ``original`` positions; from ``lo = max(floor(place(fast)),
    0)`` to ``hi = min(ceil(place(slow)), n - 1)`` the ramp rises from 0 to 1 (at least 0.001
    wide), and ``f_i <- f_i / factor * ramp_i + f_i (1 - ramp_i)``.  Worked out in double
    precision."""
    n = 2 * freqs.numel()

    def place(turns):
        return n * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(place(float(fast))), 0)
    hi = min(math.ceil(place(float(slow))), n - 1)
    i = torch.arange(freqs.numel(), dtype=torch.float64)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    f = freqs.to(torch.float64)
    return (f / float(factor) * ramp + f * (1.0 - ramp)).to(torch.float32)


FREQUENCY_SCALINGS = {"llama3": llama3_scaled, "linear": linear_scaled, "yarn": yarn_scaled}
# rules that also multiply cos and sin by a number: rule -> function of the rule's constants
TRIG_SCALINGS = {"yarn": lambda factor, **_ignored: 0.1 * math.log(float(factor)) + 1.0}


def frequencies_and_trig_scale(spec: PositionSpec):
    """(float32 frequencies [rotary_dim / 2] on the host, the factor on cos and sin) of a rope
    spec, with its scaling rule applied.  The plain ladder is worked out in double precision."""
    if spec.layout not in RotaryPosition.LAYOUTS:
        raise ValueError(f"rotary layout '{spec.layout}': {sorted(RotaryPosition.LAYOUTS)}")
    if spec.rotary_dim <= 0 or spec.rotary_dim % 2:
        raise ValueError(f"rotary_dim {spec.rotary_dim} must be positive and even")
    idx = torch.arange(0, spec.rotary_dim, 2, dtype=torch.float64)[: spec.rotary_dim // 2]
    freqs = (1.0 / (float(spec.base) ** (idx / spec.rotary_dim))).to(torch.float32)
    trig = 1.0
    scaling = spec.scaling_dict()
    if scaling is not None:
        kind = scaling.get("rope_type")
        if kind not in FREQUENCY_SCALINGS:
            raise ValueError(f"rope scaling '{kind}': {sorted(FREQUENCY_SCALINGS)}")
        constants = {k: v for k, v in scaling.items() if k != "rope_type"}
        if kind == "yarn":
            idx64 = 1.0 / (float(spec.base) ** (idx / spec.rotary_dim))
            freqs = yarn_scaled(idx64, base=float(spec.base), **constants)
        else:
            freqs = FREQUENCY_SCALINGS[kind](freqs, **constants)
        if kind in TRIG_SCALINGS:
            trig = float(TRIG_SCALINGS[kind](**constants))
    return freqs.to(torch.float32), trig


# the kernel that rotates, stores and attends in one (csrc/attention_bf16.hip: gfa_attention_sliced_bf16)
# is not used: see RotaryPosition.rotate_store_attend
FUSED_SLICED_ATTENTION = False


class RotaryPosition(Part):
    LAYOUTS = {"interleaved": 0, "half": 1}
    replayable = True

    def __init__(self, spec: PositionSpec, runtime: Runtime):
        if spec.layout not in self.LAYOUTS:
            raise ValueError(f"rotary layout '{spec.layout}': {sorted(self.LAYOUTS)}")
        if spec.rotary_dim <= 0 or spec.rotary_dim % 2:
            raise ValueError(f"rotary_dim {spec.rotary_dim} must be positive and even")
        self.spec = spec
        self.rt = runtime
        freqs = rotary_frequencies(spec.rotary_dim, spec.base)
        scaling = spec.scaling_dict()
        if scaling is not None:
            kind = scaling.get("rope_type")
            if kind not in FREQUENCY_SCALINGS:
                raise ValueError(f"rope scaling '{kind}': {sorted(FREQUENCY_SCALINGS)}")
            if kind in TRIG_SCALINGS:
                raise ValueError(f"rope scaling '{kind}' also scales cos and sin, which this part's "
                                 f"kernels do not; mixers that take it ask frequencies_and_trig_scale")
            freqs = FREQUENCY_SCALINGS[kind](
                freqs, **{k: v for k, v in scaling.items() if k != "rope_type"})
        self.freqs_host = freqs.to(torch.float32)
        self.freqs = self.freqs_host.to(runtime.device)

    # qkv may come as ops.linear.SlicedRows (a sliced product's partial sums): they are added
    # on the way where the kernel for that fits
    takes_sliced = True

    def rotate_and_store(self, qkv, batch, entry, n_heads, n_kv_heads, head_dim):
        write = entry is not None and entry.writes
        pages = (entry.k_pages if write else None, entry.v_pages if write else None)
        if isinstance(qkv, L.SlicedRows):
            if (self.spec.layout == "interleaved" and qkv.dtype == torch.bfloat16
                    and head_dim % 8 == 0 and self.spec.rotary_dim % 8 == 0):
                return K.rope_cache_write_sliced(
                    qkv.part, self.freqs, batch.tok_seq, batch.tok_pos, batch.table(entry.group_id),
                    *pages, n_heads, n_kv_heads, head_dim, self.spec.rotary_dim)
            qkv = qkv.rows()
        return K.rope_cache_write(
            qkv, self.freqs, batch.tok_seq, batch.tok_pos, batch.table(entry.group_id), *pages,
            n_heads, n_kv_heads, head_dim, self.spec.rotary_dim, self.LAYOUTS[self.spec.layout])

    def rotate_store_attend(self, qkv, batch, entry, n_heads, n_kv_heads, head_dim, scale, window):
        """For a step of one token per sequence whose ``qkv`` is still an
        ``ops.linear.SlicedRows``: rotation, cache write and attention in one kernel.  None:
        not available for this step (the caller rotates, stores and attends apart).

        Switched off (``FUSED_SLICED_ATTENTION``): the kernel puts the token's own key into the
        operand registers of the block it has loaded from the cache, and in some sequences of
        a step - other ones from run to run - what the cache held at that place reaches the
        product instead: with the pool's never-written slots holding bytes that are no number,
        20 sequences decoding together gave rows that are no number; with other bytes the
        token's own score is quietly that of a stale key.  Rotating and storing apart and then
        attending (3 us more a layer at 17..64 rows) reads the key back from the cache and does
        not show it."""
        if not FUSED_SLICED_ATTENTION:
            return None
        # a run that reads another run's cache attends to that run's keys and values, also at
        # the token's own position: not to the ones this kernel would make of its own rows
        if (self.spec.layout != "interleaved" or not isinstance(qkv, L.SlicedRows)
                or qkv.dtype != torch.bfloat16 or entry is None or not entry.writes):
            return None
        from ..ops import attention_bf16 as AB
        return AB.attention_sliced(qkv.part, self.freqs, self.spec.rotary_dim, entry.k_pages,
                                   entry.v_pages, True, batch, batch.table(entry.group_id),
                                   scale, window or 0, n_heads)

    def project_rotate_store(self, x, wqkv, batch, entry, n_heads, n_kv_heads, head_dim):
        """Projection + rotation + cache write in one kernel for few rows (interleaved
        pairs only: both elements of a pair are then in one lane).  None: not available."""
        if self.spec.layout != "interleaved":
            return None
        write = entry is not None and entry.writes
        return L.qkv_rope_store(
            x, wqkv, self.freqs, batch.tok_seq, batch.tok_pos,
            batch.table(entry.group_id), entry.k_pages if write else None,
            entry.v_pages if write else None, n_heads, n_kv_heads, head_dim, self.spec.rotary_dim)


class NoPosition(Part):
    """No position information: q, k, v pass through unchanged into q and the cache."""
    replayable = True

    def __init__(self, spec: PositionSpec, runtime: Runtime):
        self.spec = spec

    def rotate_and_store(self, qkv, batch, entry, n_heads, n_kv_heads, head_dim):
        write = entry is not None and entry.writes
        return K.rope_cache_write(
            qkv, None, batch.tok_seq, batch.tok_pos, batch.table(entry.group_id),
            entry.k_pages if write else None, entry.v_pages if write else None,
            n_heads, n_kv_heads, head_dim, 0, 0)


class LearnedPosition(Part):
    """A learned vector per position, added to the embedded rows: ``x[n] += table[pos(n)]``
    (not scaled).  Used as a plan's ``input_position``; positions beyond the table are refused
    by the plan's ``max_positions``, which the engine checks against the table's rows."""
    replayable = True

    def __init__(self, spec: PositionSpec, runtime: Runtime):
        if spec.dim <= 0 or spec.max_positions <= 0:
            raise ValueError("a learned position table needs dim and max_positions")
        self.spec = spec
        self.table = None

    def parameters(self):
        return {"table": Param((self.spec.max_positions, self.spec.dim))}

    def bind(self, tensors):
        check_bound("LearnedPosition", self.parameters(), tensors)
        self.table = tensors["table"]

    def unread_bytes(self, rows: int) -> int:
        """Each token takes one row of the table."""
        return max(0, self.table.shape[0] - rows) * self.table.shape[1] * self.table.element_size()

    def add_to_stream(self, residual, batch):
        if batch.max_kv_len > self.spec.max_positions:
            raise ValueError(f"a sequence of {batch.max_kv_len} tokens is longer than the "
                             f"{self.spec.max_positions} learned positions")
        K.add_table_rows(residual, self.table, batch.tok_pos)


register_position("rope", RotaryPosition)
register_position("learned", LearnedPosition)
register_position("none", NoPosition)
