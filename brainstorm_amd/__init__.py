"""MI355X-native MoE routing hot path behind Brainstorm's Python API."""
