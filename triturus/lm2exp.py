"""Drop-in import path of the reference: ``from triturus.lm2exp import lm2exp``."""
from triturus_amd.lm2exp import lm2exp  # noqa: F401
