"""halite_amd: a small, whole inference engine for the Llama 3 decoder on one AMD
MI355X (gfx950), after the inference stack of rosinality/halite."""

__version__ = "0.1.0"
