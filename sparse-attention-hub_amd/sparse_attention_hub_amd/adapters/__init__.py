"""Adapters that plug the MI355X sparse-attention path into model frameworks."""
from .huggingface import ModelAdapterHF

__all__ = ["ModelAdapterHF"]
