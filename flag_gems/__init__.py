"""Drop-in alias: ``import flag_gems`` resolves to the gfx950 build (flaggems_amd) for the FP8
quantized-linear operators, so code written against the reference package runs unchanged."""
from flaggems_amd import *  # noqa: F401,F403
from flaggems_amd import __all__, __version__, device, vendor_name  # noqa: F401
