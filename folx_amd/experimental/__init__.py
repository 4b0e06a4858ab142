"""Helpers that choose something for the caller instead of asking (folx/experimental/)."""

from .vmap import auto_batched_vmap

__all__ = ['auto_batched_vmap']
