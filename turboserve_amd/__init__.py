"""An inference engine for the Qwen2 dense decoder on one AMD MI355X."""

__version__ = "0.1.0"
