"""An inference engine for the Qwen2.5 dense decoder on AMD MI355X (gfx950)."""
__version__ = "0.1.0"
