"""ginfer_amd: a small, whole inference engine for one MI355X (gfx950).

    from ginfer_amd import Engine, EngineConfig, SamplingParams
    engine = Engine(EngineConfig(model_path="/path/to/model", dtype="bfloat16"))
    outputs = engine.generate([[1, 2, 3]], SamplingParams(max_tokens=16))
"""
from .config import config_from_folder, config_from_dict, register_architecture, Qwen2Config
from .sampling import SamplingParams
from .engine import Engine, EngineConfig, ModelRunner, StepEntry, RequestOutput
from .weights import write_random_model

__all__ = ["config_from_folder", "config_from_dict", "register_architecture", "Qwen2Config", "SamplingParams",
           "Engine", "EngineConfig", "ModelRunner", "StepEntry", "RequestOutput", "write_random_model"]
__version__ = "0.1.0"
