"""MI355X-native fused disentangled attention for DeBERTa-v2/v3.

Import paths mirror TurboDeBERTa's: ``turbodeberta_amd.ops.flash_attention``,
``turbodeberta_amd.ops.flash_attention_varlen``, ``turbodeberta_amd.model``, ``turbodeberta_amd.padding``."""

__version__ = "0.1.0"
