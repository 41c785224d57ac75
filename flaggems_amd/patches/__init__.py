"""Hooks that put this package's operators behind vLLM's layers
(reference: src/flag_gems/patches/__init__.py)."""
from .patch_vllm_all import apply_gems_patches_to_vllm

__all__ = ["apply_gems_patches_to_vllm"]
