from .decoder import DecoderModel, build_model, load_model

__all__ = ["DecoderModel", "build_model", "load_model"]
