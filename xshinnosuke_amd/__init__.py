"""xshinnosuke_amd -- MI355X (gfx950) backend for xshinnosuke's conv / max-pool path."""
from . import backend  # noqa: F401
