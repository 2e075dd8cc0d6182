"""Several mixers side by side that read the same input."""
import torch

from ..cache.store import JointNeed
from ..config.spec import ParallelMixerSpec
from ..ops import kernels as K
from .base import MIXERS, Param, Part, Runtime, check_bound, register_mixer


class ParallelMixer(Part):
    """``y = mean_b( rms(branch_b(x)) * out_b )``: every branch is a mixer of its own kind with
    its own parameters (named ``<branch>.<parameter>``) and its own cache (member b of the
    run's joint cache entry); its result, float32 [N, D], is divided by its root mean square
    over the model width and multiplied by the weight ``<branch>_out`` before the mean.

    A block that joins results by a kernel of its own asks ``forward_branches`` and gets the
    two results apart (the combination then rides on that kernel); ``forward_rows`` and
    ``forward`` combine here."""

    def __init__(self, spec: ParallelMixerSpec, runtime: Runtime):
        if len(spec.branches) < 2:
            raise ValueError("a parallel mixer has at least two branches")
        self.spec = spec
        self.rt = runtime
        self.names = [name for name, _ in spec.branches]
        self.branches = [MIXERS.build(branch, runtime) for _, branch in spec.branches]
        for name, part in zip(self.names, self.branches):
            if not hasattr(part, "forward_rows"):
                raise TypeError(f"branch '{name}' of a parallel mixer must offer forward_rows")
        self.out_weights = None
        if len(self.branches) == 2:
            self.forward_branches = self._forward_branches

    @property
    def replayable(self):
        return all(getattr(b, "replayable", False) for b in self.branches)

    def children(self):
        return dict(zip(self.names, self.branches))

    def parameters(self):
        out = {}
        for name, part in zip(self.names, self.branches):
            for pname, p in part.parameters().items():
                out[f"{name}.{pname}"] = p
            out[f"{name}_out"] = Param((self.spec.dim,), role="vector", init="norm")
        return out

    def bind(self, tensors):
        check_bound("ParallelMixer", self.parameters(), tensors)
        for name, part in zip(self.names, self.branches):
            prefix = name + "."
            part.bind({k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)})
        self.out_weights = [tensors[f"{name}_out"].to(torch.float32).contiguous() for name in self.names]

    def cache_need(self):
        return JointNeed(tuple(part.cache_need() for part in self.branches))

    def step_flops(self, q_lens, starts) -> float:
        return sum(getattr(p, "step_flops", lambda q, s: 0.0)(q_lens, starts) for p in self.branches)

    def unread_bytes(self, rows: int) -> int:
        return sum(getattr(p, "unread_bytes", lambda r: 0)(rows) for p in self.branches)

    def step_fields(self):
        out = []
        for part in self.branches:
            out += list(getattr(part, "step_fields", lambda: ())())
        return out

    def _results(self, x, batch, entry):
        return [part.forward_rows(x, batch, entry.part(i) if entry is not None else None)
                for i, part in enumerate(self.branches)]

    def _forward_branches(self, x, batch, entry):
        """(first result, second result, (weight of the first, of the second), eps)."""
        first, second = self._results(x, batch, entry)
        return first, second, tuple(self.out_weights), self.spec.eps

    def forward_rows(self, x, batch, entry):
        """The mean of the normed branch results, float32 [N, D]."""
        results = self._results(x, batch, entry)
        y = torch.zeros_like(results[0])
        share = 1.0 / len(results)
        for r, w in zip(results, self.out_weights):
            K.normed_add(y, r, w * share, self.spec.eps)
        return y

    def forward(self, x, batch, entry, residual):
        K.add_into(residual.tensor if hasattr(residual, "tensor") else residual,
                   self.forward_rows(x, batch, entry))


register_mixer("parallel", ParallelMixer)
