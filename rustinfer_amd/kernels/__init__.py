"""ctypes bindings of the hand-written gfx950 kernels."""
