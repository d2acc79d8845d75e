"""Drop-in classifier modules: same module, class, method and attribute names as the reference's
src/xmc_classifiers package (selected in src/model.py:144-156)."""
from .chunked_fp8xmc_clf import Fp8XMCBCEChunkedLayer  # noqa: F401
from .chunked import XMCBCECHUNKEDLayer  # noqa: F401
from .chunked_head_kahan_fp8xmc_clf import Fp8XMCBCEChunkedHeadKahanLayer  # noqa: F401
