"""mini_llm_amd: a small, whole GPT-2 inference engine for one AMD MI355X (gfx950) GPU.

    from mini_llm_amd import Engine, SamplingParams
    engine = Engine.from_pretrained(model_dir, dtype="bfloat16")
    new_tokens = engine.generate([[15496, 11, 616]], SamplingParams(max_new_tokens=8))

The engine is native (csrc/): configuration and registry, loader, parts, cache manager and storage,
step function, scheduler, sampler, kernels; ``bin/mini-llm`` is its command line. This package is the
thin Python entry over its C ABI.
"""
from .config import describe_config, load_plugin, read_preset, registered_architectures  # noqa: F401
from .engine.engine import Engine, EngineOptions, RequestOutput, SamplingParams  # noqa: F401
from .engine.runner import Runner, StepEntry  # noqa: F401
from .native import EngineError  # noqa: F401
from .weights import check_model_dir, write_random_model  # noqa: F401
