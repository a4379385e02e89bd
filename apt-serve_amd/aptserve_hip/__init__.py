"""Host side of the MI355X hybrid-cache library (Python over a C ABI)."""

from . import ops  # noqa: F401

__all__ = ["ops"]
