"""Minimal model counterparts of the reference's ``transformer`` package, built on the Fastmax operator."""
from .model import Attention, Transformer, TransformerBlock  # noqa: F401
