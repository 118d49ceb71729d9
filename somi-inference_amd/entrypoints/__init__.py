"""User-facing entry points."""

from .llm import LLM

__all__ = ["LLM"]
