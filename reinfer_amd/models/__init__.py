from .decoder import DecoderModel, declare_params

__all__ = ["DecoderModel", "declare_params"]
