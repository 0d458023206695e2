"""An inference engine on AMD MI355X (gfx950) for the architectures its registry names (`models/`)."""
__version__ = "0.1.0"
