"""MI355X (gfx950) native MXFP8 linear path behind torchtitan's model-converter API."""

__version__ = "0.1.0"
