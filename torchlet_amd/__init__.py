"""torchlet_amd: a small, whole Qwen2.5 inference engine for one AMD MI355X."""
__version__ = "0.1.0"


def __getattr__(name):
    if name == "LLM":
        from .llm import LLM
        return LLM
    raise AttributeError(name)
