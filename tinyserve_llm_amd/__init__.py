"""An inference engine for the Llama dense decoder on one AMD MI355X: hand-written HIP kernels
under a paged cache manager, a step function over mixed batches, and a cache-aware scheduler."""

__all__ = ["LLM", "SamplingParams"]


def __getattr__(name: str):
    # resolved on first use so that configuration, cache manager and scheduler import without the engine
    if name == "LLM":
        from tinyserve_llm_amd.engine.llm import LLM
        return LLM
    if name == "SamplingParams":
        from tinyserve_llm_amd.engine.sequence import SamplingParams
        return SamplingParams
    raise AttributeError(name)
