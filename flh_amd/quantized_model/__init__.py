from .decoder_layer import StaticKVCache, W4A4DecoderLayer, rotary_tables  # noqa: F401
from .llama import LlamaShape, W4A4LlamaModel  # noqa: F401
