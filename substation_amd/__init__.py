"""MI355X-native fused BERT encoder layer with the module API of
spcl/substation's pytorch_module/encoder.py."""
from .layouts import load_layouts, mi355x_layouts, reference_layouts, save_layouts  # noqa: F401


def __getattr__(name):
    if name in ('Encoder', 'EncoderStack', 'causal_mask'):       # torch is imported only when the module is used
        from . import encoder
        return getattr(encoder, name)
    if name == 'DecoderLayer':
        from . import decoder
        return decoder.DecoderLayer
    raise AttributeError(name)
