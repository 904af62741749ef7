"""MI355X-native decode path for GeoRefine's lossless BF16 context codec."""
__all__ = ["bitexact_context_codec", "bitexact_context_gpu", "bitexact_predictive_codec",
           "bitexact_predictive_gpu", "bitexact_predictive_mix", "serving"]
