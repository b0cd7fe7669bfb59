"""MI355X-native InfiniOP paged-attention decode, paged-attention prefill and paged_caching.

The product is the pair of C-ABI shared libraries built from ``csrc/`` into ``lib/``
(``libinfinirt.so``, ``libinfiniop.so``). This package is their Python host side:

* ``libinfiniop`` - ctypes declarations of every exported entry point and small RAII helpers;
* ``ops``         - ``paged_attention`` / ``paged_attention_prefill`` / ``paged_caching`` on torch CUDA
                    tensors, with the argument order of the reference's
                    ``python/infinicore/ops/paged_attention.py:5-40``, ``paged_attention_prefill.py:5-45`` and
                    ``paged_caching.py:5-21``;
* ``workloads``   - seeded synthetic inputs of the benchmark configurations;
* ``build``       - compiles the libraries with hipcc for gfx950.

Nothing here computes attention on the host: if the libraries are missing the import of
``libinfiniop`` raises, there is no fallback path.
"""

__all__ = ["libinfiniop", "ops", "workloads", "build"]
