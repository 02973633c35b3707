"""tessera_amd — the MI355X (gfx950 / CDNA4) execution lane for Tessera's dense
ops: GEMM (f16 / bf16 / int8 / fp8), flash-attention forward and the MoE
grouped-GEMM block, as hand-written HIP kernels behind a C ABI.

Modules
-------
``lane``        ctypes binding of ``lib/libtessera_gfx950.so``
``ops``         the ``tessera.ops`` / ``nn.functional`` surface of the path
``resident``    the same ops on device-resident handles, for chains without host round trips
``executors``   the ``runtime.launch`` executor seam (execution-matrix rows)
``candidates``  gfx950 candidates for the host's measured arbiter (host API injected)
``install``     one call that registers candidates, matrix rows and executors with a host
``autotune``    the lane's autotune corpus (reference schema) and tuning through the host
``tile_table``  Tile-IR op -> gfx950 kernel table
``build``       in-tree hipcc build of the library
"""
from . import bf16, lane  # noqa: F401

__all__ = ["bf16", "lane", "ops", "resident", "executors", "candidates", "install", "autotune", "tile_table", "build"]
