"""picolm_amd: a small text-generation library for the dense Llama decoder on AMD MI355X
(gfx950), in the manner of whoreson/picolm: token ids in, next tokens out."""
from .config import ConfigError, LlamaConfig, RopeScaling, known_architectures, register_architecture
from .weights import WeightsError, write_random_model

__version__ = "0.1.0"

__all__ = ["ConfigError", "LlamaConfig", "RopeScaling", "known_architectures", "register_architecture",
           "WeightsError", "write_random_model", "load_model", "Session"]


def __getattr__(name):
    # the engine pulls in the GPU kernels' bindings; import it on first use
    if name in ("load_model", "random_model", "Session", "DecoderModel", "LayerCall"):
        from . import engine
        return getattr(engine, name)
    if name in ("generate", "Generator", "SamplingParams"):
        from . import generation
        return getattr(generation, name)
    raise AttributeError(name)
