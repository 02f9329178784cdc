"""CPU oracle for the operator hot path -- TEST INFRASTRUCTURE, not product code.

A numpy restatement of the reference operators' ``reference()`` methods and of
the Llama graph wiring, each function citing the reference file:line it follows.
Only ``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s cpu_baseline leg
import this package; the ``iron_amd`` package never does, and its operators
raise if no HIP library is loaded rather than fall back to anything here.

``install()`` registers these functions as the operator classes' ``reference()``
providers (the numpy-reference API the operator tests use).
"""

from . import ops  # noqa: F401


def install() -> None:
    """Register the oracle as the ``reference()`` provider of ``iron_amd``'s operators."""
    from . import references

    references.install()
