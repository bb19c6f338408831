"""gfx950-native low-precision compute path with the ``primus_turbo`` op surface."""

__version__ = "0.1.0"
