"""CPU oracle (test infrastructure; see oracle.py). Product code must not import this."""
from . import oracle  # noqa: F401
