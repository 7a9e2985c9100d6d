"""MI355X-native inference engine for the MiniCPM/FM9G decoder.

Sub-packages:
  config    typed configuration and the architecture registry
  weights   safetensors loading by tensor name, random-weights model folders
  parts     mixers, feed-forwards, norms, position encodings, blocks, the layered model
  cache     paged key/value cache, block tables, per-request state slots
  kernels   ctypes bindings of the HIP kernels under csrc/
  engine    the step function, scheduler, request tasks, trace replay
  sampling  sampling parameters, random draws and the device sampler
"""
__version__ = "0.1.0"
