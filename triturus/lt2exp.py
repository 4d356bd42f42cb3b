"""Drop-in import path of the reference: ``from triturus.lt2exp import lt2exp``."""
from triturus_amd.lt2exp import lt2exp  # noqa: F401
