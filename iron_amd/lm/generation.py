"""Sampling, and the loops that generate and check, over any model (iron/lm/generation.py:1-185).

A model is anything with ``logits(tokens)``: the logits after the last of ``tokens``, the
whole history so far, as ``(vocab_size,)``.  A ``CausalLM`` on the GPU is one, and so is a CPU
reference.
"""

from __future__ import annotations

import numpy as np

from ..common.declare import REFERENCES
from ..operators.sample import ROW_WORDS, draw_row

#: Seeds the sampler, so a run's text is reproducible.
SEED = 1608560892


def _host(name: str):
    """The host's restatement of the device's draw: supplied by the test oracle, never by the product."""
    fn = REFERENCES.get(name)
    if fn is None:
        raise NotImplementedError(
            f"{name}: no host draw is registered; the oracle is test infrastructure (import oracle; "
            "oracle.install()).  On the device a Sampler's draws are its rows()."
        )
    return fn


def check_order_preserving(temperature) -> None:
    """The device ranks raw bf16 logits and divides only the candidates' distances from the best by
    the temperature, in float64: any finite positive float32 temperature keeps every logit's order.

    Raises:
        ValueError: ``temperature`` is not finite, or under the smallest normal float32.
    """
    t = np.float32(temperature)
    if not np.isfinite(t) or t < np.finfo(np.float32).tiny:
        raise ValueError(f"temperature {temperature} is not a finite, normal float32")


class Sampler:
    """Temperature, then top-k, then a draw from the softmax, exactly as the device draws
    (iron/lm/generation.py:24-94).

    Args:
        top_k: None keeps the whole row; only valid on the host, since the device's top-k is bounded.
    """

    def __init__(self, temperature: float = 0.7, top_k: int | None = 50, seed: int = SEED):
        if temperature < 0:
            raise ValueError(f"temperature {temperature} is negative")
        if temperature > 0:
            check_order_preserving(temperature)
        if top_k is not None and top_k < 1:
            raise ValueError(f"top_k {top_k} keeps no token")
        self.temperature = np.float32(temperature)
        self.top_k = top_k
        self.rng = np.random.default_rng(seed)

    def _top_k(self, size: int) -> int:
        return size if self.top_k is None else self.top_k

    def _n53(self) -> int:
        # random() is n53 * 2^-53 for the generator's next 53 bits, exactly.
        return int(self.rng.random() * 2.0**53)

    def probabilities(self, logits: np.ndarray) -> np.ndarray:
        """The distribution a token is drawn from, float64, over ``logits`` (1-D); a host check."""
        size = np.asarray(logits).size
        probs = np.zeros(size, dtype=np.float64)
        if self.temperature == 0:
            probs[_host("sample_ref")(logits, self.temperature, 1, 0)] = 1.0
            return probs
        candidates, weights = _host("sample_weights")(logits, self.temperature, self._top_k(size))
        probs[candidates] = weights / weights.sum()
        return probs

    def __call__(self, logits: np.ndarray) -> int:
        """One token id drawn on the host from a row of logits (any shape of one row); a host check."""
        top_k = self._top_k(np.asarray(logits).size)
        return _host("sample_ref")(logits, self.temperature, top_k, self._n53())

    def rows(self, count: int, k_max: int) -> np.ndarray:
        """``count`` draws for the device, ``(count, ROW_WORDS)`` int32, one per position: the
        uniforms ``count`` host draws would take, in order.

        Raises:
            ValueError: ``top_k`` is None or past ``k_max``, the device's largest, where it would be
                clamped rather than honoured.
        """
        if self.top_k is None or self.top_k > k_max:
            raise ValueError(f"top_k {self.top_k} is not one the device draws (1..{k_max})")
        rows = np.empty((count, ROW_WORDS), dtype=np.int32)
        for i in range(count):
            rows[i] = draw_row(self.temperature, self.top_k, self._n53())
        return rows


def greedy(logits: np.ndarray) -> int:
    """The id of the largest of ``logits``."""
    return int(np.asarray(logits, dtype=np.float32).argmax())


def _rollout(model, tokens, num_tokens, choose):
    """Yield ``(history, logits)`` for ``num_tokens`` steps from ``tokens``; ``choose(history, logits)``
    names the token each step appends."""
    history = list(map(int, tokens))
    for _ in range(num_tokens):
        row = model.logits(history)
        yield history, row
        history = [*history, int(choose(history, row))]


def generate_on_host(model, tokens, num_tokens, sample) -> list[int]:
    """The ``num_tokens`` drawn after ``tokens``, each from ``model``'s logits by ``sample``."""
    drawn: list[int] = []

    def choose(_, row):
        drawn.append(int(sample(row)))
        return drawn[-1]

    for _ in _rollout(model, tokens, num_tokens, choose):
        pass
    return drawn


def divergence(reference, logits) -> tuple[float, bool]:
    """KL(reference || model) of two rows of logits, and whether both rank the same token first."""
    from scipy.special import log_softmax

    want = log_softmax(np.asarray(reference, dtype=np.float64).ravel())
    got = log_softmax(np.asarray(logits, dtype=np.float64).ravel())
    return float(np.exp(want) @ (want - got)), bool(want.argmax() == got.argmax())


def accuracy(model, reference, tokens, num_tokens, report=None) -> list[tuple[float, bool]]:
    """``model``'s next-token distributions against ``reference``'s over ``num_tokens`` steps from
    ``tokens``, teacher-forced on the reference's greedy token so that a divergence is the model's
    own error and not an earlier different choice's consequence."""
    results = []
    for history, want in _rollout(reference, tokens, num_tokens, lambda _, row: greedy(row)):
        results.append(divergence(want, model.logits(history)))
        if report is not None:
            kl, same = results[-1]
            report(f"step {len(results) - 1:3d}  KL {kl:.5f}  top-1 {'match' if same else 'MISMATCH'}")
    return results


def kl_stats(results) -> dict[str, float]:
    """The mean, p90 and max KL of ``accuracy``'s results, over every step alike."""
    kl = np.fromiter((k for k, _ in results), dtype=np.float64)
    return {"Mean": float(kl.mean()), "P90": float(np.percentile(kl, 90)), "Max": float(kl.max())}


def greedy_logits(model, tokens, num_tokens) -> np.ndarray:
    """The logits of ``num_tokens`` greedy steps from ``tokens``, one row each, the first the prompt's."""
    return np.stack([row for _, row in _rollout(model, tokens, num_tokens, lambda _, row: greedy(row))])


def differing_steps(run, first) -> list[int]:
    """The steps at which two ``greedy_logits`` runs differ bitwise, NaNs and signed zeros included."""
    a, b = (np.ascontiguousarray(r).view(np.uint8).reshape(len(r), -1) for r in (run, first))
    return [i for i in range(len(a)) if not np.array_equal(a[i], b[i])]


def determinism(model, prompts, num_tokens, rounds) -> int:
    """How many runs' logits differ bitwise from the first run of their prompt, over ``rounds``
    repeats; the prompts alternate, so a host write that never reaches the device shows as the
    other prompt's data and not as a leftover copy of its own."""
    baseline: dict[int, np.ndarray] = {}
    differ = 0
    for _ in range(rounds):
        for p, prompt in enumerate(prompts):
            run = greedy_logits(model, prompt, num_tokens)
            if p not in baseline:
                baseline[p] = run
            elif differing_steps(run, baseline[p]):
                differ += 1
    return differ
