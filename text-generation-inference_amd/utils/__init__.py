"""Checkpoint access for the int4 linear layer: safetensors slicing, shard arithmetic and
the quantizer configuration that selects the loader."""
