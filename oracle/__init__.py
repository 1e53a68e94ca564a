"""CPU oracle for the xKV compressed-KV decode path.

TEST INFRASTRUCTURE ONLY.  Nothing in ``kernel_collections_amd`` imports this
package; only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline``
leg of ``bench.py`` may.  It restates, in eager PyTorch on the CPU (plus a small
brute-force C file, ``xkv_oracle.c``), what the reference's eager functions
compute, so the HIP kernels can be checked against it on identical inputs.
"""
from .xkv_oracle import *  # noqa: F401,F403
