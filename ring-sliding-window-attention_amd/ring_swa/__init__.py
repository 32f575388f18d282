"""MI355X-native single-GPU attention path of ring_swa."""
