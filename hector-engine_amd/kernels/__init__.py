"""ctypes bindings of the hand-written HIP kernels."""
