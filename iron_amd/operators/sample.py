"""Sample: the next token drawn on the device from a row of logits, carried into the next call.

The reference's operator (iron/operators/sample.py:106-336).  A draw row is four int32
words (temperature bits, top-k, a 53-bit number); an all-zero row is greedy, the first
largest logit -- the draw this build runs (``iron_argmax_bf16``).  The token is written
to ``token`` and recorded in ``tokens[at]``.
"""

from __future__ import annotations

import numpy as np

from ..common.declare import Built, In, InOut, Operator, Out, param, per_call, tunable
from ..common.testing import Case, Testing
from ..common.verify import Tolerance

ROW_WORDS = 4  # int32 words of one draw row


class Sample(Operator):
    test = Testing([Case(dict(vocab=4096, steps=3), id="small"), Case(dict(vocab=128256), id="llama", bench=True),
                    Case(dict(vocab=51866), id="uneven"), Case(dict(vocab=151670, drawable=151669), id="padded")])

    vocab: int = param(array=True)
    k_max: int = param(default=64, array=True)
    # The logits that are tokens'; the rest pad an odd vocabulary.
    drawable: int = param(default=lambda op: op.vocab, array=True)
    # Positions the draws and the record hold; a call picks one.
    steps: int = param(default=1)
    cores: int = tunable(default=4)

    logits = In(vocab)
    draws = In(steps, ROW_WORDS, dtype=np.int32)
    tokens = InOut(steps, dtype=np.int32)
    token = Out(1, dtype=np.int32)
    # The word of `draws` the call's row starts at, and the record slot it writes.
    row = per_call(bounds=None)
    at = per_call(bounds=None)

    @classmethod
    def infer(cls, shapes, **kw):
        return dict(vocab=int(np.prod(shapes["logits"])), steps=int(np.prod(shapes["tokens"])))

    def bind_views(self, inputs, outputs):
        return {}

    def output_valid(self, name, inputs):
        return {}

    def ops(self) -> int:
        return 0  # a draw, not arithmetic: its figure is latency

    def tolerance(self) -> Tolerance:
        return Tolerance.exact()

    def build(self) -> Built:
        from .. import kernels

        drawable = self.drawable

        def launch(t, words):
            # "__carry_token__": the scratchpad word a compiled loop carries the draw in, if it does.
            kernels.argmax(t["logits"].reshape(-1), t["token"].reshape(-1), n=drawable,
                           record=t["tokens"].reshape(-1), at=words.get("at"),
                           token_copy=words.get("__carry_token__"))

        return Built("iron_argmax_bf16", launch)
