from .decoder import DecoderModel, LayerSpec, ModelSpec, RunEntry
