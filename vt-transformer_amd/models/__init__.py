from .model import DecoderModel, build_part

__all__ = ["DecoderModel", "build_part"]
