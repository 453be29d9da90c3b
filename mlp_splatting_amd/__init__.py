"""MI355X-native tile-based forward renderer for MLP Splatting (hand-written HIP behind a C ABI)."""
__version__ = "0.1.0"
