"""MI355X-native padding-free BERT encoder (drop-in for the hot path of
bytedance/effective_transformer).  The compute lives in lib/libet_hip.so (hand-written HIP
for gfx950 behind the C ABI of include/et.h); this package is the Python-side mirror of the
reference's op interface."""

from . import _lib  # noqa: F401


def __getattr__(name):
    # torch-facing API is imported lazily so that `import effective_transformer_amd` stays cheap
    if name in ("effective_transformer_input", "effective_transformer", "effective_transformer_output",
                "get_sequence_output", "EffectiveTransformerEncoder", "GraphedEncoder", "LayerWeights", "handle",
                "EmbeddingWeights", "effective_transformer_embedding_input"):
        from . import ops
        return getattr(ops, name)
    raise AttributeError(name)
