"""MI355X-native log-space contraction kernels behind the triturus entry points.

Modules (same names and signatures as the reference package):
    triturus_amd.lm2exp.lm2exp, triturus_amd.lt2exp.lt2exp,
    triturus_amd.max.{matmax, vmax, vamax}, triturus_amd.utils.

The function names ``lm2exp`` / ``lt2exp`` are deliberately not re-exported
here: they would shadow the submodules of the same name.
"""

from triturus_amd.max import matmax, vamax, vmax  # noqa: F401

__all__ = ["matmax", "vamax", "vmax"]
