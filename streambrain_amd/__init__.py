"""MI355X-native implementation of StreamBrain's BCPNN layer training and inference step.

  streambrain_amd.backend.hip_backend   DenseLayer / StructuralPlasticityLayer / Network (the DSL)
  streambrain_amd.kernels_hip           numpy-facing single-kernel entry points (differential testing)
  streambrain_amd._capi                 ctypes view of libsbhip.so (include/sbhip.h)
  streambrain_amd.build                 builds libsbhip.so and the pybind11 module in-tree

Importing this package does not touch the GPU; importing the backend does.
"""
__version__ = "0.1.0"
