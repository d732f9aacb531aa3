"""An inference engine for OPT-family decoders on one AMD MI355X."""
__version__ = "0.1.0"
