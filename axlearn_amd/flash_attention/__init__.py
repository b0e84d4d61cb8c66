"""HIP attention kernels behind AXLearn's flash-attention dispatch API."""
