"""Drop-in import path of the reference: ``from triturus.utils import ...``."""
from triturus_amd.utils import (  # noqa: F401
    ensure_reproducibility,
    is_torch_tf32_enabled,
    is_triturus_tf32_enabled,
    matrix_precision,
    set_matrix_precision,
    set_tf32_enabled,
)
