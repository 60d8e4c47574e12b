"""berth_amd — MI355X-native EXL3 trellis linear and MoE hot path."""
__all__ = ["synth"]
