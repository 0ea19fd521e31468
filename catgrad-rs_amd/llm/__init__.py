"""LLM building blocks and model definitions as catgrad `Module`s (mirror of catgrad-llm)."""
from . import helpers, llama, qwen_moe, gemma3, runner, random_init  # noqa: F401
from .helpers import Config  # noqa: F401
from .runner import CachedRunner  # noqa: F401
