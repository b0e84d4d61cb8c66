"""MI355X-native attention kernels behind AXLearn's flash-attention dispatch API."""
