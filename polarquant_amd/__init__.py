"""MI355X-native polar-key decode path (quantize-on-append, decode scores, fused decode attention)."""
__version__ = "0.1.0"
