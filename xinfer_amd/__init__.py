"""xinfer_amd: a small, whole LLM inference engine for one AMD MI355X (gfx950).

    from xinfer_amd import Engine, EngineConfig, SamplingParams
    engine = Engine(EngineConfig(weight_path="/path/to/model"), "bf16")
    outputs = engine.generate([[1, 2, 3]], SamplingParams(temperature=0.0, max_tokens=16))

Names follow the reference's Python package (xinfer.pyi).
"""
from .config.engine_config import (DType, EngineConfig, GenerationConfig, GenerationOutput, Message,
                                   SamplingParams, StreamItem)


def __getattr__(name):
    # the engine pulls in torch and the native libraries; import it on first use
    if name in ("Engine", "LLMEngine"):
        from .engine.llm_engine import LLMEngine
        return LLMEngine
    raise AttributeError(name)


__all__ = ["DType", "Engine", "EngineConfig", "GenerationConfig", "GenerationOutput", "LLMEngine", "Message",
           "SamplingParams", "StreamItem"]
