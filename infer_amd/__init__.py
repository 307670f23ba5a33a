"""MI355X-native paged KV-cache hot path (append + paged decode attention + block pool) behind
the Python entry points of Graylatzhou/Infer."""
__version__ = "0.1"
