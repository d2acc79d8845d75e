"""MI355X-native implementation of the ELMO extreme-classifier training step.

Public surface
  elmo_amd.xmc_classifiers   drop-in classifier modules (same names as the reference's src/xmc_classifiers)
  elmo_amd.ops               thin tensor-level wrappers over the C ABI (include/elmo_xmc.h)
  elmo_amd.synth             seeded synthetic inputs of the benchmark shapes
"""
__version__ = "0.1.0"
