"""starrygl_amd -- MI355X-native temporal mini-batch hot path behind StarryGL's
Python API (graph / cache / utils.partition_book / nn.model.time_encoder)."""
__version__ = "0.1.0"
