"""simply_amd: a Gemma 2 inference engine for one MI355X, after google-deepmind/simply."""
__version__ = "0.1.0"


def __getattr__(name):
    if name in ("LLM", "LMInterface", "SamplingParams", "ScoringParams", "SamplingOutput"):
        from .engine import llm as _llm

        return getattr(_llm, name)
    raise AttributeError(name)
