from .decoder import DecoderModel, LayerCall
