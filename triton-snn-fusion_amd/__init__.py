"""MI355X-native fused temporal SNN operators (libsnnf + the snn_custom operator layer)."""

__version__ = "0.1.0"
