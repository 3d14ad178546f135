"""MI355X-native KV-cache scoring, selection and compaction (TriAttention hot path).

``ops``      tensor-level wrappers over the C ABI of libtriattention_hip.so
``core``     dense scoring / compressor API
``runtime``  TRIATTN_RUNTIME_* settings, selector, paged compaction, runner hook
"""
__version__ = "0.1.0"
