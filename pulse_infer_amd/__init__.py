"""pulse_infer_amd: a small, whole LLM inference engine for one AMD Instinct MI355X.

    from pulse_infer_amd import LLM
    llm = LLM.from_pretrained("model_dir", dtype="bfloat16")
    out = llm.generate([[1, 2, 3]], max_new_tokens=16)
"""
from .config import ConfigError, Qwen3Config, load_config, register_architecture
from .sampling.params import SamplingParams

__all__ = ["ConfigError", "Qwen3Config", "load_config", "register_architecture", "SamplingParams", "LLM",
           "ContinuousBatchEngine"]


def __getattr__(name):  # the engine pulls in torch.cuda pieces; load it on first use
    if name in ("LLM", "ContinuousBatchEngine"):
        from .engine import engine as _engine
        return getattr(_engine, name)
    raise AttributeError(name)
