"""Parts that add to the embedded rows of a step (a plan's ``input_adds``)."""
from ..cache.store import StateNeed
from ..config.spec import PairEmbeddingSpec
from ..ops import kernels as K
from .base import Param, Part, Runtime, check_bound, register_input_add


class PairEmbedding(Part):
    """An embedding of the pair (previous token, token): row ``(previous * mul_prev + token *
    mul_cur) mod buckets`` of a table of ``buckets + 1`` rows is added to the token's embedded
    row; a sequence's first token takes the last row.  The previous token of the first token
    that a step brings is state of the sequence: one int32 in the cache's state slot, left
    there by the step before, on the device, so that single-token steps whose tokens never
    reach the host (a recorded step) find it."""

    replayable = True

    def __init__(self, spec: PairEmbeddingSpec, runtime: Runtime):
        if spec.buckets < 1 or spec.mul_prev < 0 or spec.mul_cur < 0:
            raise ValueError("a pair embedding needs buckets >= 1 and multipliers >= 0")
        self.spec = spec
        self.table = None

    def parameters(self):
        return {"table": Param((self.spec.buckets + 1, self.spec.dim))}

    def bind(self, tensors):
        check_bound("PairEmbedding", self.parameters(), tensors)
        self.table = tensors["table"]

    def unread_bytes(self, rows: int) -> int:
        """Each token takes one row of the table."""
        return max(0, self.table.shape[0] - rows) * self.table.shape[1] * self.table.element_size()

    def cache_need(self):
        return StateNeed((1,), "int32")

    def add_to_stream(self, residual, batch, entry):
        s = self.spec
        K.pair_embed_add(residual, self.table, batch.tokens, batch.tok_seq, batch.tok_pos,
                         batch.q_start, batch.slots, entry.state.view(-1), s.buckets, s.mul_prev,
                         s.mul_cur)


register_input_add("pair_embedding", PairEmbedding)
