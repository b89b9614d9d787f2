"""MI355X-native scatter / segment / gather reductions (torch_scatter-compatible)."""
__version__ = "0.1.0"
