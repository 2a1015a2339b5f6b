"""torch_mlu_amd — MI355X-native flash-attention forward behind torch_mlu's operator interface."""
__version__ = "0.1.0"
