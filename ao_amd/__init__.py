"""ao_amd: MI355X (gfx950) implementation of torchao's weight-only quantized linear path."""
__version__ = "0.1.0"
