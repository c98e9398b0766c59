from .llm import LLM, GenerationLoop, GenerationResult

__all__ = ["LLM", "GenerationLoop", "GenerationResult"]
