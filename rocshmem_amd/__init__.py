"""MI355X-native symmetric-heap data movement behind rocSHMEM's API.

The product is the HIP library built from ``rocshmem_amd/csrc`` (device API
headers under ``include/rocshmem``, C entry points in ``include/rocshmem_amd.h``).
This package only loads that library for Python callers; there is no CPU
fallback: importing :mod:`rocshmem_amd.lib` raises if the library is not built.
"""

from .lib import Library, load  # noqa: F401
