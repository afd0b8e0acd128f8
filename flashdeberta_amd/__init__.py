"""MI355X-native DeBERTa disentangled-attention forward (hand-written HIP behind a C ABI).

Attributes resolve lazily so that `python -m flashdeberta_amd.csrc.build` can run before the
shared library exists; touching any operator or model name loads libfdb_hip.so and raises if it
is missing (there is no fallback path).
"""
_OPS = ("disentangled_attention_fwd", "flash_attention_with_disentangled",
        "flash_attention_with_disentangled_varlen", "quantize_e4m3_per_head", "quantize_e4m3_per_head_pair", "dequantize_e4m3_per_head")
_MODEL = ("FlashDisentangledSelfAttention", "DEBERTA_SELF_ATTENTION_CLASSES", "FlashDebertaV2Model",
          "patch_model", "DebertaV2Config")
__all__ = list(_OPS + _MODEL)


def __getattr__(name):
    if name in _OPS:
        from . import ops
        return getattr(ops, name)
    if name in _MODEL:  # needs transformers
        from . import model
        return getattr(model, name)
    raise AttributeError("module %r has no attribute %r" % (__name__, name))
