"""A small, whole inference engine for the Qwen3 dense decoder on one MI355X.

    from nanohybrid_vlm_amd import LLM, SamplingParams
"""


def __getattr__(name):
    # imported on first use, so that tools which need only a part of the package start fast
    if name == "LLM":
        from .engine.llm import LLM
        return LLM
    if name == "SamplingParams":
        from .sampling.params import SamplingParams
        return SamplingParams
    raise AttributeError(name)


__all__ = ["LLM", "SamplingParams"]
