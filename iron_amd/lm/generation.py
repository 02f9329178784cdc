"""How tokens are drawn, and the loops that generate and judge, for anything with ``logits(tokens)``.

Interface of the reference's iron/lm/generation.py:1-185 (``Sampler``, ``generate_on_host``,
``divergence``, ``accuracy``, ``determinism`` ...).  Here a ``Sampler`` is first of all a source of
*draw rows* for the device: the GPU draws every token itself from rows written ahead of time
(``Session.draw``), and the host-side ``Sampler.__call__`` exists to check that draw, token for
token, through the test oracle's restatement of the device arithmetic.  The product never samples on
the CPU.
"""

from __future__ import annotations

import numpy as np

from ..common.declare import REFERENCES
from ..operators.sample import ROW_WORDS, draw_row

SEED = 1608560892   # default seed: the same run twice gives the same text

_TWO_53 = float(1 << 53)


def _oracle(name: str):
    """A host restatement of the device's draw, present only when a test installed the oracle."""
    try:
        return REFERENCES[name]
    except KeyError:
        raise NotImplementedError(
            f"{name}: the host-side draw belongs to the test oracle (import oracle; oracle.install()); "
            "on the device a Sampler acts through its rows()") from None


def check_order_preserving(temperature) -> None:
    """Refuse a temperature the device could not honour.

    The device ranks the raw bf16 logits and only then scales the survivors' distance from the best
    by 1/temperature in float64, so ranking is untouched by any finite, normal, positive float32.

    Raises:
        ValueError: not finite, or below float32's smallest normal number.
    """
    value = np.float32(temperature)
    if not (np.isfinite(value) and value >= np.finfo(np.float32).tiny):
        raise ValueError(f"temperature {temperature} is not a finite, normal float32")


class Sampler:
    """Temperature / top-k sampling driven by a seeded stream of 53-bit numbers.

    ``temperature == 0`` is greedy.  ``top_k=None`` (the whole row) exists on the host only: the
    device weighs a bounded number of candidates, and ``rows`` refuses rather than clamps.
    """

    def __init__(self, temperature: float = 0.7, top_k: int | None = 50, seed: int = SEED):
        if temperature < 0:
            raise ValueError(f"temperature {temperature} is below zero")
        if temperature > 0:
            check_order_preserving(temperature)
        if top_k is not None and top_k < 1:
            raise ValueError(f"top_k {top_k} leaves nothing to draw from")
        self.temperature, self.top_k = np.float32(temperature), top_k
        self.rng = np.random.default_rng(seed)

    def _next_n53(self) -> int:
        # Generator.random() is (next 53 random bits) / 2^53, so scaling back recovers the integer.
        return int(self.rng.random() * _TWO_53)

    def _k(self, width: int) -> int:
        return width if self.top_k is None else self.top_k

    # -- what the device consumes
    def rows(self, count: int, k_max: int) -> np.ndarray:
        """``count`` consecutive draws as device rows, shape ``(count, ROW_WORDS)`` int32; they use up
        the same random numbers, in the same order, as ``count`` host draws would.

        Raises:
            ValueError: ``top_k`` is unbounded or above ``k_max``.
        """
        if self.top_k is None or self.top_k > k_max:
            raise ValueError(f"top_k {self.top_k} is not one the device draws (1..{k_max})")
        packed = [draw_row(self.temperature, self.top_k, self._next_n53()) for _ in range(count)]
        return np.asarray(packed, dtype=np.int32).reshape(count, ROW_WORDS)

    # -- host-side checks of the same draw (oracle-backed)
    def __call__(self, logits: np.ndarray) -> int:
        width = np.asarray(logits).size
        return _oracle("sample_ref")(logits, self.temperature, self._k(width), self._next_n53())

    def probabilities(self, logits: np.ndarray) -> np.ndarray:
        """The float64 distribution one draw from ``logits`` follows (zero outside the top-k)."""
        width = np.asarray(logits).size
        out = np.zeros(width, dtype=np.float64)
        if self.temperature > 0:
            ids, weights = _oracle("sample_weights")(logits, self.temperature, self._k(width))
            out[ids] = weights / weights.sum()
        else:
            out[_oracle("sample_ref")(logits, self.temperature, 1, 0)] = 1.0
        return out


def greedy(logits: np.ndarray) -> int:
    """Index of the largest logit (the first, of equals)."""
    return int(np.argmax(np.asarray(logits, dtype=np.float32)))


def _steps(model, tokens, count, pick):
    """``count`` steps from ``tokens``: yields the history fed to the model and the logits it
    returned, then extends the history by ``pick(logits)``."""
    seen = [int(t) for t in tokens]
    for _ in range(count):
        logits = model.logits(seen)
        yield list(seen), logits
        seen.append(int(pick(logits)))


def generate_on_host(model, tokens, num_tokens, sample) -> list[int]:
    """``num_tokens`` tokens after ``tokens``, each chosen by ``sample`` from ``model``'s logits."""
    chosen: list[int] = []

    def pick(logits):
        chosen.append(int(sample(logits)))
        return chosen[-1]

    for _ in _steps(model, tokens, num_tokens, pick):
        pass
    return chosen


def divergence(reference, logits) -> tuple[float, bool]:
    """``(KL(reference || model), same top token)`` for two rows of logits."""
    def log_probs(row):
        z = np.asarray(row, dtype=np.float64).ravel()
        z = z - z.max()
        return z - np.log(np.exp(z).sum())

    p, q = log_probs(reference), log_probs(logits)
    return float(np.sum(np.exp(p) * (p - q))), bool(np.argmax(p) == np.argmax(q))


def accuracy(model, reference, tokens, num_tokens, report=None) -> list[tuple[float, bool]]:
    """Per step, ``divergence`` of ``model`` from ``reference`` while both follow the reference's
    greedy continuation of ``tokens`` (teacher forcing: an early disagreement cannot snowball)."""
    out = []
    for step, (history, expected) in enumerate(_steps(reference, tokens, num_tokens, greedy)):
        out.append(divergence(expected, model.logits(history)))
        if report is not None:
            report(f"step {step:3d}  KL {out[-1][0]:.5f}  top-1 {'match' if out[-1][1] else 'MISMATCH'}")
    return out


def kl_stats(results) -> dict[str, float]:
    """Mean, 90th percentile and maximum of the KLs in ``accuracy``'s output."""
    values = np.array([kl for kl, _ in results], dtype=np.float64)
    return {"Mean": float(values.mean()), "P90": float(np.percentile(values, 90)), "Max": float(values.max())}


def greedy_logits(model, tokens, num_tokens) -> np.ndarray:
    """Logits of ``num_tokens`` greedy steps after ``tokens``, stacked (row 0: the prompt's)."""
    return np.stack([logits for _, logits in _steps(model, tokens, num_tokens, greedy)])


def differing_steps(run, first) -> list[int]:
    """Rows at which two ``greedy_logits`` results are not the same bytes (so NaN == NaN, 0 != -0)."""
    def as_bytes(rows):
        return np.ascontiguousarray(rows).view(np.uint8).reshape(len(rows), -1)

    return [i for i, (a, b) in enumerate(zip(as_bytes(run), as_bytes(first))) if not np.array_equal(a, b)]


def determinism(model, prompts, num_tokens, rounds) -> int:
    """Number of runs whose logits are not bitwise those of the first run on the same prompt.

    The prompts take turns within each of the ``rounds``, so that state leaking from one run into
    the next shows up as another prompt's data rather than as a harmless copy of the same."""
    first_run: dict[int, np.ndarray] = {}
    mismatches = 0
    for _ in range(rounds):
        for index, prompt in enumerate(prompts):
            logits = greedy_logits(model, prompt, num_tokens)
            if index in first_run:
                mismatches += bool(differing_steps(logits, first_run[index]))
            else:
                first_run[index] = logits
    return mismatches
