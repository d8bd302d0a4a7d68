"""zse_amd: a small MI355X-native inference engine (one GPU, one architecture at a time)."""
__version__ = "0.1.0"
