"""Sample: the next token drawn on the device from a row of logits, carried into the next call.

The reference's operator (iron/operators/sample.py:106-336).  A draw row is four int32
words (temperature bits, top-k, a 53-bit number) the host writes ahead of time per position;
an all-zero row is greedy, the first largest logit.  With a temperature the token is drawn
from the top-k logits' softmax by that number (``iron_sample_bf16``, which states the
arithmetic).  The token is written to ``token`` and recorded in ``tokens[at]``.
"""

from __future__ import annotations

import numpy as np

from ..common.declare import Built, In, InOut, Operator, Out, Scratch, param, per_call, tunable
from ..common.testing import Case, Testing
from ..common.verify import Tolerance

ROW_WORDS = 4  # int32 words of one draw row
K_MAX = 64     # the most candidates the device weighs


def draw_row(temperature, top_k: int, n53: int) -> np.ndarray:
    """One draw row: ``temperature`` as float32 bits, ``top_k``, and ``n53`` (a uniform number's
    53 bits) as a low and a high word."""
    if not 0 <= int(n53) < 1 << 53:
        raise ValueError(f"n53 {n53} is not a 53-bit number")
    row = np.empty(ROW_WORDS, dtype=np.uint32)
    row[0] = np.array([temperature], dtype=np.float32).view(np.uint32)[0]
    row[1] = int(top_k)
    row[2] = int(n53) & 0xFFFFFFFF
    row[3] = int(n53) >> 32
    return row.view(np.int32)


def _logits(op: "Sample") -> dict:
    """Logits with a few ties at the top, padding above every token's logit (which no draw may
    take), and one draw row per position (iron/operators/sample.py:82-103)."""
    from ..bf16 import round_bf16

    rng = np.random.default_rng(11)
    logits = round_bf16(rng.normal(0, 3, op.vocab))
    logits[rng.choice(op.vocab, 8, replace=False)] = logits.max()
    logits[op.drawable:] = logits.max() + 1
    temperatures, top_ks = rng.choice([0.0, 0.7, 1.0], op.steps), rng.integers(1, 51, op.steps)
    draws = np.stack([draw_row(t, k, int(rng.integers(0, 1 << 53))) for t, k in zip(temperatures, top_ks)])
    return dict(given={op.logits: logits, op.draws: draws, op.tokens: np.full(op.steps, -1, dtype=np.int32)})


class Sample(Operator):
    test = Testing([Case(dict(vocab=4096, steps=3), id="small"), Case(dict(vocab=128256), id="llama", bench=True),
                    Case(dict(vocab=51866), id="uneven"), Case(dict(vocab=151670, drawable=151669), id="padded")],
                   draw=_logits)

    vocab: int = param(array=True)
    k_max: int = param(default=64, array=True)
    # The logits that are tokens'; the rest pad an odd vocabulary.
    drawable: int = param(default=lambda op: op.vocab, array=True)
    # Positions the draws and the record hold; a call picks one.
    steps: int = param(default=1)
    cores: int = tunable(default=4)
    workspace_words: int = param(derive=lambda op: op._workspace_words(), repr=False)

    logits = In(vocab)
    draws = In(steps, ROW_WORDS, dtype=np.int32)
    tokens = InOut(steps, dtype=np.int32)
    token = Out(1, dtype=np.int32)
    # The blocks' candidate lists behind the word that counts the blocks, which every launch finds
    # and leaves at zero: kept from call to call.
    workspace = Scratch(workspace_words, dtype=np.float32, kept=True)
    # The word of `draws` the call's row starts at, and the record slot it writes.
    row = per_call(bounds=None)
    at = per_call(bounds=None)

    def _workspace_words(self) -> int:
        from .._lib import lib

        return int(lib().iron_sample_workspace_bytes(self.drawable)) // 4

    def validate(self) -> None:
        if not 1 <= self.k_max <= K_MAX:
            raise ValueError(f"Sample: k_max ({self.k_max}) must be from 1 to {K_MAX}")
        if not self.k_max <= self.drawable <= self.vocab:
            raise ValueError(f"Sample: drawable ({self.drawable}) must be from k_max ({self.k_max}) "
                             f"to vocab ({self.vocab})")

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

        drawable, k_max = self.drawable, self.k_max

        own = {}

        def launch(t, words):
            ws = t.get("workspace")
            if ws is None:  # a call outside a graph: allocated once, kept
                ws = own.get("ws")
                if ws is None:
                    ws = own["ws"] = kernels.sample_workspace(drawable, t["logits"].device)
            # "__carry_token__": the scratchpad word a compiled loop carries the draw in, if it does;
            # "__carry_eval__": the loop's word expressions, where the draw is the step's last launch.
            kernels.sample(t["logits"].reshape(-1), t["draws"].reshape(-1), t["token"].reshape(-1), n=drawable,
                           row=words.get("row"), k_max=k_max, workspace=ws, record=t["tokens"].reshape(-1),
                           at=words.get("at"), token_copy=words.get("__carry_token__"),
                           advance=words.get("__carry_eval__"))

        return Built("iron_sample_bf16", launch)
