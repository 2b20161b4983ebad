"""ResearchAttention and its maskers."""
from .base import ResearchAttention, ResearchAttentionConfig

__all__ = ["ResearchAttention", "ResearchAttentionConfig"]
