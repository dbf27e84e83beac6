"""lpmm for AMD MI355X: the 4-bit optimizer-state path of thu-ml/low-bit-optimizers behind
the reference's own API (`lpmm.optim.AdamW`, `lpmm.functional.vectorwise_quant/dequant`),
running on hand-written gfx950 kernels in liblpmm_hip.so."""
from . import optim  # noqa: F401
from . import config, functional, utils  # noqa: F401
