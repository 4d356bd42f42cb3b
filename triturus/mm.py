"""Drop-in import path of the reference: ``from triturus.mm import mm``."""
from triturus_amd.mm import mm  # noqa: F401
