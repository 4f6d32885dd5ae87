"""Loads libmcsparse.so and declares the prototypes of include/mcsparse.h for ctypes.

There is no fallback: if the library has not been built, importing a compute entry point
raises, so a caller can never end up on a silent CPU path.
"""
import ctypes
import os

from .build import LIB_PATH

c_int = ctypes.c_int
c_i64 = ctypes.c_int64
c_size = ctypes.c_size_t
vp = ctypes.c_void_p
P = ctypes.POINTER

# every symbol include/mcsparse.h declares: name -> (restype, argtypes)
PROTOTYPES = {
    "mcsparseCreate": (c_int, [P(vp)]),
    "mcsparseDestroy": (c_int, [vp]),
    "mcsparseGetVersion": (c_int, [vp, P(c_int)]),
    "mcsparseGetProperty": (c_int, [c_int, P(c_int)]),
    "mcsparseGetErrorName": (ctypes.c_char_p, [c_int]),
    "mcsparseGetErrorString": (ctypes.c_char_p, [c_int]),
    "mcsparseSetStream": (c_int, [vp, vp]),
    "mcsparseGetStream": (c_int, [vp, P(vp)]),
    "mcsparseSetPointerMode": (c_int, [vp, c_int]),
    "mcsparseGetPointerMode": (c_int, [vp, P(c_int)]),
    "mcsparseCreateDnVec": (c_int, [P(vp), c_i64, vp, c_int]),
    "mcsparseDestroyDnVec": (c_int, [vp]),
    "mcsparseDnVecGet": (c_int, [vp, P(c_i64), P(vp), P(c_int)]),
    "mcsparseDnVecGetValues": (c_int, [vp, P(vp)]),
    "mcsparseDnVecSetValues": (c_int, [vp, vp]),
    "mcsparseCreateCsr": (c_int, [P(vp), c_i64, c_i64, c_i64, vp, vp, vp, c_int, c_int, c_int, c_int]),
    "mcsparseCsrGet": (c_int, [vp, P(c_i64), P(c_i64), P(c_i64), P(vp), P(vp), P(vp), P(c_int), P(c_int), P(c_int),
                               P(c_int)]),
    "mcsparseCsrSetPointers": (c_int, [vp, vp, vp, vp]),
    "mcsparseCreateCsc": (c_int, [P(vp), c_i64, c_i64, c_i64, vp, vp, vp, c_int, c_int, c_int, c_int]),
    "mcsparseCscSetPointers": (c_int, [vp, vp, vp, vp]),
    "mcsparseCreateCoo": (c_int, [P(vp), c_i64, c_i64, c_i64, vp, vp, vp, c_int, c_int, c_int]),
    "mcsparseCooGet": (c_int, [vp, P(c_i64), P(c_i64), P(c_i64), P(vp), P(vp), P(vp), P(c_int), P(c_int), P(c_int)]),
    "mcsparseCooSetPointers": (c_int, [vp, vp, vp, vp]),
    "mcsparseDestroySpMat": (c_int, [vp]),
    "mcsparseSpMatGetSize": (c_int, [vp, P(c_i64), P(c_i64), P(c_i64)]),
    "mcsparseSpMatGetFormat": (c_int, [vp, P(c_int)]),
    "mcsparseSpMatGetIndexBase": (c_int, [vp, P(c_int)]),
    "mcsparseSpMatGetValues": (c_int, [vp, P(vp)]),
    "mcsparseSpMatSetValues": (c_int, [vp, vp]),
    "mcsparseCreateDnMat": (c_int, [P(vp), c_i64, c_i64, c_i64, vp, c_int, c_int]),
    "mcsparseDestroyDnMat": (c_int, [vp]),
    "mcsparseDnMatGet": (c_int, [vp, P(c_i64), P(c_i64), P(c_i64), P(vp), P(c_int), P(c_int)]),
    "mcsparseDnMatGetValues": (c_int, [vp, P(vp)]),
    "mcsparseDnMatSetValues": (c_int, [vp, vp]),
    "mcsparseCooSetStridedBatch": (c_int, [vp, c_int, c_i64]),
    "mcsparseCsrSetStridedBatch": (c_int, [vp, c_int, c_i64, c_i64]),
    "mcsparseDnMatSetStridedBatch": (c_int, [vp, c_int, c_i64]),
    "mcsparseDnMatGetStridedBatch": (c_int, [vp, P(c_int), P(c_i64)]),
    "mcsparseSpMV": (c_int, [vp, c_int, vp, vp, vp, vp, vp, c_int, c_int, vp]),
    "mcsparseSetSpMVDeterministic": (c_int, [vp, c_int]),
    "mcsparseGetSpMVDeterministic": (c_int, [vp, P(c_int)]),
    "mcsparseSetSpMVPreprocessTrial": (c_int, [vp, c_int]),
    "mcsparseGetSpMVPreprocessTrial": (c_int, [vp, P(c_int)]),
    "mcsparseXstreamProbe": (c_int, [vp, c_int, vp, vp, ctypes.c_size_t, vp, ctypes.c_size_t]),
    "mcsparseXtopologyOfCuCount": (c_int, [c_int, P(c_int)]),
    "mcsparseSpMV_staticBuffer": (c_int, [vp, c_int, vp, vp, vp, vp, vp, c_int, c_int]),
    "mcsparseSpMV_preprocess_bufferSize": (c_int, [vp, c_int, vp, vp, vp, vp, vp, c_int, c_int, P(c_size)]),
    "mcsparseSpMV_preprocess": (c_int, [vp, c_int, vp, vp, vp, vp, vp, c_int, c_int, vp]),
    "mcsparseSpMatSetSpMVBandBytes": (c_int, [vp, c_size]),
    "mcsparseSpMatGetSpMVPreprocess": (c_int, [vp, P(c_int), P(c_int), P(c_int)]),
    "mcsparseSpMV_bufferSize": (c_int, [vp, c_int, vp, vp, vp, vp, vp, c_int, c_int, P(c_size)]),
    "mcsparseSpMM_bufferSize": (c_int, [vp, c_int, c_int, vp, vp, vp, vp, vp, c_int, c_int, P(c_size)]),
    "mcsparseSpMM_preprocess": (c_int, [vp, c_int, c_int, vp, vp, vp, vp, vp, c_int, c_int, vp]),
    "mcsparseSpMM": (c_int, [vp, c_int, c_int, vp, vp, vp, vp, vp, c_int, c_int, vp]),
    "mcsparseXcoo2csr": (c_int, [vp, vp, c_int, c_int, vp, c_int]),
    "mcsparseXcsr2coo": (c_int, [vp, vp, c_int, c_int, vp, c_int]),
    "mcsparseCsr2cscEx2": (c_int, [vp, c_int, c_int, c_int, vp, vp, vp, vp, vp, vp, c_int, c_int, c_int, c_int, vp]),
    "mcsparseCsr2cscEx2_bufferSize": (c_int, [vp, c_int, c_int, c_int, vp, vp, vp, vp, vp, vp, c_int, c_int, c_int,
                                              c_int, P(c_size)]),
    "mcsparseXcsrsort_bufferSizeExt": (c_int, [vp, c_int, c_int, c_int, vp, vp, P(c_size)]),
    "mcsparseXcsrsort": (c_int, [vp, c_int, c_int, c_int, vp, vp, vp, vp, vp]),
    "mcsparseXcscsort_bufferSizeExt": (c_int, [vp, c_int, c_int, c_int, vp, vp, P(c_size)]),
    "mcsparseXcscsort": (c_int, [vp, c_int, c_int, c_int, vp, vp, vp, vp, vp]),
    "mcsparseXcoosort_bufferSizeExt": (c_int, [vp, c_int, c_int, c_int, vp, vp, P(c_size)]),
    "mcsparseXcoosortByRow": (c_int, [vp, c_int, c_int, c_int, vp, vp, vp, vp]),
    "mcsparseXcoosortByColumn": (c_int, [vp, c_int, c_int, c_int, vp, vp, vp, vp]),
    "mcsparseCreateIdentityPermutation": (c_int, [vp, c_int, vp]),
    "mcsparseSgthr": (c_int, [vp, c_int, vp, vp, vp, c_int]),
    "mcsparseDgthr": (c_int, [vp, c_int, vp, vp, vp, c_int]),
    "mcsparseCreateMatDescr": (c_int, [P(vp)]),
    "mcsparseDestroyMatDescr": (c_int, [vp]),
    "mcsparseCopyMatDescr": (c_int, [vp, vp]),
    "mcsparseSetMatIndexBase": (c_int, [vp, c_int]),
    "mcsparseGetMatIndexBase": (c_int, [vp]),
    "mcsparseSetMatType": (c_int, [vp, c_int]),
    "mcsparseGetMatType": (c_int, [vp]),
    "mcsparseSetMatFillMode": (c_int, [vp, c_int]),
    "mcsparseGetMatFillMode": (c_int, [vp]),
    "mcsparseSetMatDiagType": (c_int, [vp, c_int]),
    "mcsparseGetMatDiagType": (c_int, [vp]),
    "mcsparseSetStorageMode": (c_int, [vp, c_int]),
    "mcsparseGetStorageMode": (c_int, [vp, P(c_int)]),
    "mcsparseScsrmv": (c_int, [vp, c_int, c_int, c_int, c_int, vp, vp, vp, vp, vp, vp, vp, vp]),
    "mcsparseDcsrmv": (c_int, [vp, c_int, c_int, c_int, c_int, vp, vp, vp, vp, vp, vp, vp, vp]),
    "mcsparseCsrmvEx_bufferSize": (c_int, [vp, c_int, c_int, c_int, c_int, c_int, vp, c_int, vp, vp, c_int, vp, vp,
                                           vp, c_int, vp, c_int, vp, c_int, c_int, P(c_size)]),
    "mcsparseCsrmvEx": (c_int, [vp, c_int, c_int, c_int, c_int, c_int, vp, c_int, vp, vp, c_int, vp, vp, vp, c_int,
                                vp, c_int, vp, c_int, c_int, vp]),
    "mcsparseScsrmm2": (c_int, [vp, c_int, c_int, c_int, c_int, c_int, c_int, vp, vp, vp, vp, vp, vp, c_int, vp, vp,
                                c_int]),
    "mcsparseDcsrmm2": (c_int, [vp, c_int, c_int, c_int, c_int, c_int, c_int, vp, vp, vp, vp, vp, vp, c_int, vp, vp,
                                c_int]),
    "mcsparseScsrmm": (c_int, [vp, c_int, c_int, c_int, c_int, c_int, vp, vp, vp, vp, vp, vp, c_int, vp, vp, c_int]),
    "mcsparseDcsrmm": (c_int, [vp, c_int, c_int, c_int, c_int, c_int, vp, vp, vp, vp, vp, vp, c_int, vp, vp, c_int]),
    "mcsparseXcsrRowBinsPlan": (c_int, [vp, c_i64, c_i64, c_i64, P(c_int), P(c_int)]),
    "mcsparseXcsrRowBins": (c_int, [vp, c_int, vp, c_int, vp, vp]),
    "mcsparseSpMatGetSpMVPlan": (c_int, [vp, P(c_int), P(c_int)]),
    "mcsparseSpMatSetSpMVPlan": (c_int, [vp, c_int, c_int]),
    "mcsparseSpMatGetSpMMSchedule": (c_int, [vp, P(c_int), P(c_i64)]),
}

_lib = None


def load():
    """Returns the ctypes handle of libmcsparse.so with all prototypes set."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "libmcsparse.so is not built (%s). Run `python -c 'import __graft_entry__ as g; g.build()'` "
                "or `python -m mcsparse_amd.build`; there is no CPU fallback." % LIB_PATH)
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in PROTOTYPES.items():
            fn = getattr(lib, name)  # AttributeError if the symbol is missing
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib
