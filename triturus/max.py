"""Drop-in import path of the reference: ``from triturus.max import matmax, vamax, vmax``."""
from triturus_amd.max import matmax, vamax, vmax  # noqa: F401
