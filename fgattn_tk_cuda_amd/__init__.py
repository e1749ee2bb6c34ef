"""MI355X-native block-sparse attention (gfx950 HIP kernels behind a C ABI).

Layers, bottom up:
  csrc/            HIP kernels and the extern "C" surface (libspattn_hip.so)
  capi             ctypes binding of that surface over torch device tensors
  spattn/          mirror of the reference's ``spattn`` Python package
                   (``spattn.cuda_attn`` operator extension, ``mask_utils``,
                   ``sparseattn_functionals``)
  workloads        seeded synthetic inputs of the benchmark configurations
"""
__version__ = "0.1.0"
