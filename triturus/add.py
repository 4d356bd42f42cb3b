"""Drop-in import path of the reference: ``from triturus.add import vadd``."""
from triturus_amd.add import vadd  # noqa: F401
