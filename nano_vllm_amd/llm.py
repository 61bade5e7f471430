"""The Python entry point, as the reference's nanovllm/llm.py:4-5: LLM is the engine."""
from .engine.llm_engine import LLMEngine


class LLM(LLMEngine):
    pass
