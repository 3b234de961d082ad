"""MI355X-native single-GPU MoE hot path behind picotron's ``MoELayer`` / ``megakernel`` API."""
