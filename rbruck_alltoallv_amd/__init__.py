"""MI355X-native radix-r Bruck alltoallv for a virtual communicator of P ranks on one GPU.

`workloads` is host-only numpy; `api` (imported lazily) needs torch, a GPU and the built
librbruck_vc.so and has no fallback.
"""
__all__ = ["workloads", "api", "build"]
