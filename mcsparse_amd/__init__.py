"""MI355X-native CSR SpMV / SpMM / csr2csc / csr2coo behind mcSparse's C API.

The product is libmcsparse.so (mcsparse_amd/csrc, built by mcsparse_amd.build); this package
adds a ctypes view of its C ABI (api) and the seeded benchmark matrices (workloads).
"""
from . import api, workloads  # noqa: F401
from ._lib import PROTOTYPES, load  # noqa: F401
