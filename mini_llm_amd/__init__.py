"""mini_llm_amd: a small, whole GPT-2 inference engine for one AMD MI355X (gfx950) GPU.

    from mini_llm_amd import Engine, SamplingParams
    engine = Engine.from_pretrained(model_dir, dtype="bfloat16")
    new_tokens = engine.generate([[15496, 11, 616]], SamplingParams(max_new_tokens=8))

``Engine`` composes the model from parts in Python (any registered part, also ones written in
Python) and runs it through the native step function; ``NativeEngine`` is the engine that is native
from the loader to the sampler (the architectures registered natively), the one behind ``bin/mini-llm``.
"""
from .engine.engine import Engine, EngineOptions, RequestOutput  # noqa: F401
from .engine.native_engine import NativeEngine  # noqa: F401
from .models import load_model  # noqa: F401
from .sampling.sampler import SamplingParams  # noqa: F401
from .weights.random_init import write_random_model  # noqa: F401
