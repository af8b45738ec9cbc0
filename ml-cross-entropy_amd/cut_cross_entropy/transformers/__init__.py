"""Patch layer for Hugging Face ``transformers`` causal language models.

Mirrors the reference package ``cut_cross_entropy.transformers`` (ref: transformers/__init__.py:1-4).
"""

from cut_cross_entropy.transformers.patch import cce_patch

__all__ = ["cce_patch"]
