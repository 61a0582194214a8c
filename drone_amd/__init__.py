"""drone_amd: MI355X (gfx950) kernels for DRONE's per-subgraph CSR pull aggregation.

The compute lives in csrc/libdrone_hip.so behind the C ABI declared in include/drone_hip.h.  The Python
modules here are thin host-side mirrors of the reference's two call sites:

* ``drone_amd.pagerank`` - the wrappers of DRONE/src/tools/cuda_convert.go (CUDA_build_graph,
  CUDA_LoadOutDegree, CUDA_PR_PEVal, CUDA_PR_IncEVal) plus the fp64 pull plan;
* ``drone_amd.gcn``      - the kernel-level calls behind cuda_gcn's CUDAGraphSum / CUDAMatmul modules.

There is no CPU fallback: importing works anywhere, but every compute call needs the built library
and a GPU, and raises otherwise.
"""
from ._lib import lib, DroneError, library_path  # noqa: F401
