from .builder import build_from_config_dict, load_model, parse_dtype, random_model, tensor_specs_for
from .errors import StepError
from .model import DecoderModel, LayerCall
from .session import Session

__all__ = ["StepError", "build_from_config_dict", "load_model", "parse_dtype", "random_model",
           "tensor_specs_for", "DecoderModel", "LayerCall", "Session"]
