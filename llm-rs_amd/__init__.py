"""llm-rs_amd: a single-GPU inference engine for MI355X (gfx950) with the
capabilities of Leikoe/llm-rs for the Llama dense decoder.

    from llm_rs_amd import Engine
    engine = Engine.from_folder("model_dir", dtype="bfloat16")
    tokens = engine.generate([[1, 2, 3]], max_new_tokens=16)

    r = engine.submit([4, 5, 6], max_new_tokens=8)          # requests may come at any time
    while engine.has_unfinished():
        for e in engine.advance():                           # one step of the scheduler
            print(e.request, e.token, e.finished)
"""
from .cache import CacheManager, FixedState, PagedKV
from .config import (ConfigError, ExtraPart, LlamaConfig, ModelSpec, LayerSpec, PartSpec, RunSpec, load_config,
                     config_from_dict, register_architecture)
from .engine import Emitted, Engine, Model, OutOfPages, StepEntry, StepRunner, random_model_tensors
from .kernels import KernelError, kernels, use_kernels
from .sampling import SamplingParams
from .weights import WeightError, load_tensors, write_model_folder

__all__ = ["CacheManager", "FixedState", "PagedKV", "ConfigError", "ExtraPart", "LlamaConfig", "ModelSpec", "LayerSpec",
           "PartSpec", "RunSpec", "load_config", "config_from_dict", "register_architecture", "Emitted", "Engine", "Model",
           "OutOfPages", "StepEntry", "StepRunner", "random_model_tensors", "KernelError", "kernels",
           "use_kernels", "SamplingParams", "WeightError", "load_tensors", "write_model_folder"]
