"""longbow-quarrel on MI355X: a small model library with its own generation.

Five architectures (the Llama 3 dense decoder; Vafodra, a hybrid of windowed attention with a sink, Mamba-2
and the gated delta rule; Vupelorn, gated linear attention and attention through a cached latent with a mixture
of experts; Mifidra, softmax attention beside the gated delta rule between norms on both sides of every sublayer,
with grouped experts and layers that run several times; Sofinex, differential attention under a sliding window
and attention with a learned sink beside the gated delta rule, experts chosen by softmax scores among identity
experts), one GPU, from a model folder
(config.json + model.safetensors) to generated tokens, on hand-written gfx950
kernels.
"""
from . import models  # noqa: F401  (registers the architectures)
from .api import QuarrelEngine, SamplerConfig, new_engine
from .config import ConfigError, LlamaConfig, MifidraConfig, ModelConfig, SofinexConfig, VafodraConfig, VupelornConfig
from .engine import Engine, GenerationResult, SequenceTooLong, StepEntry, generate
from .loading import load_engine, random_engine
from .sampling import NonFiniteLogits, SamplingParams
from .registry import register_architecture, registered_architectures
from .weights import WeightError, write_model_folder

__all__ = [
    "ConfigError", "LlamaConfig", "MifidraConfig", "SofinexConfig", "VafodraConfig", "VupelornConfig", "ModelConfig", "Engine", "StepEntry", "load_engine", "random_engine",
    "GenerationResult", "generate", "SamplingParams", "NonFiniteLogits", "SequenceTooLong", "QuarrelEngine", "SamplerConfig", "new_engine", "register_architecture", "registered_architectures", "WeightError", "write_model_folder",
]
