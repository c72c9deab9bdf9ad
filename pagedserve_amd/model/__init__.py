from .decoder import DecoderModel
from .loading import load_model, write_random_model

__all__ = ["DecoderModel", "load_model", "write_random_model"]
