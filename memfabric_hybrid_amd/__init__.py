"""MI355X-native data plane for MemFabric's batched xcopy path.

Python here is host-side glue over the C ABI of ``lib/libmf_hip_dataplane.so``
(``include/*.h``); the work is done by HIP kernels in ``csrc/kernels``.
Importing the package loads nothing; ``native.lib()`` loads the shared
library and raises if it has not been built.
"""

from . import native  # noqa: F401

__all__ = ["native", "bm", "transfer", "workloads"]
