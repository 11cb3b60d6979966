"""Helpers around the layers (mirror of the parts of sharktank/sharktank/utils the MoE path touches)."""

from . import debugging

__all__ = ["debugging"]
