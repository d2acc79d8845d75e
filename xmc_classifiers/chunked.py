"""Import alias: `from xmc_classifiers.chunked import XMCBCECHUNKEDLayer` (src/model.py:144-156)."""
from elmo_amd.xmc_classifiers.chunked import XMCBCECHUNKEDLayer, dtype_map  # noqa: F401
