"""MI355X (gfx950) backend for the oneNew Conv / MatMul / Gemm operator path.

  onenew_amd.abi     ctypes mirror of the plugin ABI and of the kernel-level descriptors
  onenew_amd.ops     host side of the plugin boundary (slot arrays, operator objects)
  onenew_amd.hip     loader / front end of the kernel library (device pointers)
  onenew_amd.stacks  layer-shape tables of the benchmark configurations
  onenew_amd.build   in-place build of the shared objects
"""
__all__ = ["abi", "ops", "hip", "stacks", "datagen", "build"]
