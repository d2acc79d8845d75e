from elmo_amd.xmc_classifiers.chunked_fp8xmc_clf import Fp8XMCBCEChunkedLayer, dtype_map  # noqa: F401
