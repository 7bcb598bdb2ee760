"""recis_amd: the MI355X (gfx950) implementation of RecIS's sparse-embedding hot path.

``recis_amd.ops`` holds the operators RecIS registers as ``torch.ops.recis.*``;
``recis_amd.nn``, ``recis_amd.ragged``, ``recis_amd.optim``, ``recis_amd.features`` and
``recis_amd.hooks`` mirror the reference's Python modules of the same names for this
path. Everything runs on librecis_hip.so (hand-written HIP kernels behind a C ABI);
there is no CPU fallback.
"""
__version__ = "0.1.0"
