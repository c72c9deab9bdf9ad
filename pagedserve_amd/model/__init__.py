from .decoder import DecoderModel
from .loading import load_model, random_model, write_random_model

__all__ = ["DecoderModel", "load_model", "random_model", "write_random_model"]
