"""MI355X-native stochastic-rounding AdamW with the ``ramtorch.AdamW`` interface.

    from ramtorch_amd import AdamW

The update runs only as hand-written gfx950 HIP kernels behind a C ABI
(``include/ramtorch_sr_adamw.h``); build them with ``python -m ramtorch_amd.build``.
"""
from .stochastic_optimizers.adamw import AdamW, copy_stochastic_

__all__ = ["AdamW", "copy_stochastic_"]
__version__ = "0.1.0"
