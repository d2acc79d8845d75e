"""Import alias: `from xmc_classifiers.chunked_head_kahan_fp8xmc_clf import Fp8XMCBCEChunkedHeadKahanLayer`
(src/model.py:144-156)."""
from elmo_amd.xmc_classifiers.chunked_head_kahan_fp8xmc_clf import Fp8XMCBCEChunkedHeadKahanLayer, dtype_map  # noqa: F401
