"""Helpers shared by the dispatch modules (reference: src/scorch/utils.py)."""
from .format import parse_format  # noqa: F401  (same import path as the reference's utils.parse_format)
