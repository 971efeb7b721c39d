"""tokamak_amd: a small LLM inference engine for one AMD MI355X GPU."""

from tokamak_amd.sampling.params import SamplingParams

__version__ = "0.1.0"
__all__ = ["LLM", "ModelRunner", "RequestOutput", "SamplingParams", "StepEntry", "__version__"]


def __getattr__(name):  # torch is imported only when the engine is asked for
    if name == "LLM":
        from tokamak_amd.engine.llm import LLM
        return LLM
    if name == "RequestOutput":
        from tokamak_amd.engine.outputs import RequestOutput
        return RequestOutput
    if name in ("ModelRunner", "StepEntry"):
        from tokamak_amd.engine import runner
        return getattr(runner, name)
    raise AttributeError(name)
