class LLMEngine:
    pass
