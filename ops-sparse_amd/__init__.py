"""ctypes binding of libops_sparse.so (the aclsparse CSR SpMV / SpMM path on MI355X).

The directory name contains a hyphen, so load it with importlib under the module
name ``ops_sparse_amd`` (see ``load_package()`` in tests/conftest.py, bench.py).

This module is host-side plumbing over the C ABI declared in
include/cann_ops_sparse.h and include/ops_sparse_hip.h:

* ``lib()``      the CDLL with argument / result types set; raises if the shared
                 library has not been built — there is no fallback path.
* enum values    ACL_* / ACL_SPARSE_* constants with the header's numbering.
* ``Handle``, ``Csr``, ``DnVec``, ``DnMat``   RAII wrappers in the style of the
                 reference's test/frame/descriptor_manager.h, holding torch
                 tensors (device memory) alive for as long as the descriptor lives.
* ``spmv`` / ``spmm``   the reference call protocol (GetBufferSize -> Preprocess
                 -> compute) in one place for tests and the benchmark.

torch is used for device memory and streams only.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libops_sparse.so")

# ---- aclDataType (include/acl/acl_base_rt.h)
ACL_FLOAT, ACL_FLOAT16, ACL_INT8, ACL_INT32 = 0, 1, 2, 3
ACL_INT64, ACL_DOUBLE, ACL_BF16 = 9, 11, 27
# ---- aclsparseOperation_t
ACL_SPARSE_OP_NON_TRANSPOSE, ACL_SPARSE_OP_TRANSPOSE, ACL_SPARSE_OP_CONJUGATE_TRANSPOSE = 0, 1, 2
# ---- aclsparseOrder_t
ACL_SPARSE_ORDER_ROW, ACL_SPARSE_ORDER_COL = 0, 1
# ---- aclsparseSpMMAlg_t
ACL_SPARSE_SPMM_ALG_DEFAULT, ACL_SPARSE_SPMM_CSR_ALG1, ACL_SPARSE_SPMM_CSR_FP32_HIGH_PRECISION_ALG = 0, 1, 2
# ---- aclsparseSpMVAlg_t
ACL_SPARSE_SPMV_ALG_DEFAULT, ACL_SPARSE_SPMV_COO_ALG1, ACL_SPARSE_SPMV_CSR_ALG1 = 0, 1, 3
ACL_SPARSE_SPMV_CSR_ALG2 = 4
# ---- aclsparseSpMVOpAlg_t
ACL_SPARSE_SPMVOP_ALG_DEFAULT, ACL_SPARSE_SPMVOP_ALG1, ACL_SPARSE_SPMVOP_ALG2 = 0, 1, 2
# ---- aclsparseIndexType_t / aclsparseIndexBase_t / aclsparseFormat_t
ACL_SPARSE_INDEX_32I, ACL_SPARSE_INDEX_64I = 0, 1
ACL_SPARSE_INDEX_BASE_ZERO, ACL_SPARSE_INDEX_BASE_ONE = 0, 1
ACL_SPARSE_FORMAT_COO, ACL_SPARSE_FORMAT_CSR, ACL_SPARSE_FORMAT_CSC = 0, 1, 2
# ---- aclsparsePointerMode_t
ACL_SPARSE_POINTER_MODE_HOST, ACL_SPARSE_POINTER_MODE_DEVICE = 0, 1
# ---- aclsparseStatus_t
(ACL_SPARSE_STATUS_SUCCESS, ACL_SPARSE_STATUS_NOT_INITIALIZED, ACL_SPARSE_STATUS_ALLOC_FAILED,
 ACL_SPARSE_STATUS_INVALID_VALUE, ACL_SPARSE_STATUS_ARCH_MISMATCH, ACL_SPARSE_STATUS_EXECUTION_FAILED,
 ACL_SPARSE_STATUS_INTERNAL_ERROR, ACL_SPARSE_STATUS_MATRIX_TYPE_NOT_SUPPORTED, ACL_SPARSE_STATUS_NOT_SUPPORTED,
 ACL_SPARSE_STATUS_INSUFFICIENT_RESOURCES, ACL_SPARSE_STATUS_HANDLE_IS_NULLPTR) = range(11)

STATUS_NAMES = ["SUCCESS", "NOT_INITIALIZED", "ALLOC_FAILED", "INVALID_VALUE", "ARCH_MISMATCH", "EXECUTION_FAILED",
                "INTERNAL_ERROR", "MATRIX_TYPE_NOT_SUPPORTED", "NOT_SUPPORTED", "INSUFFICIENT_RESOURCES",
                "HANDLE_IS_NULLPTR"]

# ---- raw launch layer (include/ops_sparse_hip.h)
OPSPARSE_F32, OPSPARSE_F16, OPSPARSE_BF16, OPSPARSE_I32, OPSPARSE_I8 = range(5)
(OPSPARSE_SPMV_AUTO, OPSPARSE_SPMV_SCALE_ONLY, OPSPARSE_SPMV_STREAM_ROWS, OPSPARSE_SPMV_VECTOR_ROWS,
 OPSPARSE_SPMV_MERGE_PATH) = range(5)
OPSPARSE_OK, OPSPARSE_E_INVALID, OPSPARSE_E_UNSUPPORTED, OPSPARSE_E_WORKSPACE, OPSPARSE_E_LAUNCH = 0, -1, -2, -3, -4
OPSPARSE_SPMV_COLUMN_PANELS = 5
OPSPARSE_SPMV_BLOCKED_GATHER = 6
OPSPARSE_SPMV_BLOCKED_LIVE = 7
OPSPARSE_SPMV_SCATTER_LIVE = 8
OPSPARSE_BLOCKED_TRANSPOSE, OPSPARSE_BLOCKED_LIVE_VALUES = 1, 2
OPSPARSE_BLOCKED_VALUES_F16, OPSPARSE_BLOCKED_VALUES_BF16, OPSPARSE_BLOCKED_VALUES_I32 = 4, 8, 16
OPSPARSE_SPMM_AUTO, OPSPARSE_SPMM_ROW_SPLIT, OPSPARSE_SPMM_BINNED = range(3)

# Every symbol the two public headers declare; tests check that the library exports all of them.
ACLSPARSE_SYMBOLS = [
    "aclsparseCreate", "aclsparseDestroy", "aclsparseSetStream", "aclsparseGetStream", "aclsparseSetWorkspace",
    "aclsparseGetWorkspace", "aclsparseGetVersion", "aclsparseSetPointerMode", "aclsparseGetPointerMode",
    "aclsparseCreateDnVec", "aclsparseCreateConstDnVec", "aclsparseDestroyDnVec", "aclsparseDnVecGet",
    "aclsparseConstDnVecGet", "aclsparseDnVecGetValues", "aclsparseConstDnVecGetValues", "aclsparseDnVecSetValues",
    "aclsparseCreateCsr", "aclsparseCreateConstCsr", "aclsparseCsrSetPointers", "aclsparseDestroySpMat",
    "aclsparseSpMatGetFormat", "aclsparseSpMatGetValues", "aclsparseConstSpMatGetValues", "aclsparseSpMatSetValues",
    "aclsparseSpMatGetSize", "aclsparseCreateDnMat", "aclsparseCreateConstDnMat", "aclsparseDestroyDnMat",
    "aclsparseDnMatGet", "aclsparseConstDnMatGet", "aclsparseDnMatGetValues", "aclsparseConstDnMatGetValues",
    "aclsparseDnMatSetValues", "aclsparseSpMVGetBufferSize", "aclsparseSpMVPreprocess", "aclsparseSpMV",
    "aclsparseSpMMGetBufferSize", "aclsparseSpMMPreprocess", "aclsparseSpMM",
    "aclsparseSpMVOp_bufferSize", "aclsparseSpMVOp_createDescr", "aclsparseSpMVOp_destroyDescr",
    "aclsparseSpMVOp_createPlan", "aclsparseSpMVOp_destroyPlan", "aclsparseSpMVOp_setGlobalUserData",
    "aclsparseSpMVOp",
    "aclsparseCreateMatDescr", "aclsparseDestroyMatDescr", "aclsparseSetMatType", "aclsparseSetMatIndexBase",
    "aclsparseSetMatDiagType", "aclsparseSetMatFillMode", "aclsparseGetMatType", "aclsparseGetMatIndexBase",
    "aclsparseGetMatDiagType", "aclsparseGetMatFillMode",
    "aclsparseXcoo2csr", "aclsparseXcsr2coo", "aclsparseXcsrsort_bufferSizeExt", "aclsparseXcsrsort",
    "aclsparseXcscsort_bufferSizeExt", "aclsparseXcscsort",
    "aclsparseXcoosort_bufferSizeExt", "aclsparseXcoosortByRow", "aclsparseXcoosortByColumn",
    "aclsparseCsr2cscEx2_bufferSize", "aclsparseCsr2cscEx2",
]
ACL_SPARSE_ACTION_SYMBOLIC, ACL_SPARSE_ACTION_NUMERIC = 0, 1
ACL_SPARSE_CSR2CSC_ALG_DEFAULT, ACL_SPARSE_CSR2CSC_ALG1 = 0, 1
OPSPARSE_SYMBOLS = [
    "opsparse_spmv_csr_workspace_bytes", "opsparse_spmv_csr_analyse", "opsparse_spmv_csr_launch",
    "opsparse_spmv_csr_launch_zy", "opsparse_spmv_csr_indexed_launch",
    "opsparse_spmv_csr_launch_noalloc", "opsparse_spmv_csr_noalloc_max_bytes", "opsparse_rebase_offsets_launch",
    "opsparse_spmv_csr_panels_workspace_bytes", "opsparse_spmv_csr_panels_analyse",
    "opsparse_spmv_csr_blocked_workspace_bytes", "opsparse_spmv_csr_blocked_resident_bytes",
    "opsparse_spmv_csr_blocked_analyse",
    "opsparse_spmv_csr_live_workspace_bytes", "opsparse_spmv_csr_live_resident_bytes", "opsparse_spmv_csr_live_analyse",
    "opsparse_spmv_csr_live_analyse_split", "opsparse_spmv_csr_blocked_analyse_split",
    "opsparse_spmv_csr_scatter_workspace_bytes", "opsparse_spmv_csr_scatter_resident_bytes",
    "opsparse_spmv_csr_scatter_analyse", "opsparse_spmv_csr_scatter_analyse_split",
    "opsparse_spmv_csr_gathers_scattered",
    "opsparse_spmm_csr_workspace_bytes", "opsparse_spmm_csr_analyse", "opsparse_spmm_csr_launch",
    "opsparse_dense_restage",
    "opsparse_spmm_csr_narrow_rows",
    "opsparse_scan_workspace_bytes", "opsparse_coo2csr_launch", "opsparse_csr2coo_launch",
    "opsparse_csrsort_workspace_bytes", "opsparse_csrsort_launch", "opsparse_coosort_workspace_bytes",
    "opsparse_coosort_launch", "opsparse_csr2csc_workspace_bytes",
    "opsparse_csr2csc_launch",
    "opsparse_copy_launch", "opsparse_read_launch", "opsparse_gather_launch",
]

vp = ctypes.c_void_p
i64 = ctypes.c_int64
i32 = ctypes.c_int32
sz = ctypes.c_size_t


class OpsparseScalar(ctypes.Structure):
    _fields_ = [("value", ctypes.c_double), ("devicePtr", vp), ("isInt", i32), ("reserved", i32)]


class OpsparseSpmvPlan(ctypes.Structure):
    _fields_ = [("kernel", i32), ("lanesPerRow", i32), ("rowsPerBlock", i32), ("mergeBlocks", i32),
                ("maxRowNnz", i32), ("partitionReady", i32), ("numPanels", i32),
                ("panelShift", i32), ("numRowBlocks", i32), ("entryWindow", i32), ("transposed", i32),
                ("guardTiles", i32), ("tileRowNnz", i32), ("longRowsBeside", i32), ("liveValues", i32),
                ("numLongRows", i32), ("numDeferredLongRows", i32), ("valueType", i32), ("numEmptyRows", i32), ("streamedBlocks", i32), ("reserved0", i32), ("rows", i64), ("nnz", i64),
                ("partOff", i64),
                ("carryOff", i64), ("headOff", i64), ("bytes", i64), ("panelStart", i64 * 17)]


class OpsparseSpmmPlan(ctypes.Structure):
    _fields_ = [("kernel", i32), ("maxRowNnz", i32), ("longRowNnz", i32), ("numLongRows", i32),
                ("numSegments", i32), ("segmentNnz", i32), ("rows", i64), ("nnz", i64), ("n", i64),
                ("longRowsOff", i64), ("segRowOff", i64), ("segStartOff", i64), ("longFirstSegOff", i64),
                ("partialOff", i64), ("slabStartOff", i64), ("numSlabs", i64), ("bytes", i64)]


_lib = None


def lib():
    """The loaded shared library.  Raises if it is not built: nothing else can compute."""
    global _lib
    if _lib is not None:
        return _lib
    # (OPS_SPARSE_LIBRARY: another build of the same library, e.g. the ones `build.py --asan` / `--coverage` make)
    path = os.environ.get("OPS_SPARSE_LIBRARY") or LIB_PATH
    if not os.path.exists(path):
        raise RuntimeError(
            "libops_sparse.so is not built (%s missing); run `python ops-sparse_amd/build.py`" % path)
    L = ctypes.CDLL(path)
    for name in ACLSPARSE_SYMBOLS:
        getattr(L, name).restype = None if name.startswith("aclsparseSetMat") else ctypes.c_int
    PV = ctypes.POINTER(vp)
    L.aclsparseCreate.argtypes = [PV]
    L.aclsparseDestroy.argtypes = [vp]
    L.aclsparseSetStream.argtypes = [vp, vp]
    L.aclsparseGetStream.argtypes = [vp, PV]
    L.aclsparseSetWorkspace.argtypes = [vp, vp, sz]
    L.aclsparseGetWorkspace.argtypes = [vp, PV, ctypes.POINTER(sz)]
    L.aclsparseGetVersion.argtypes = [vp, ctypes.POINTER(ctypes.c_int)]
    L.aclsparseSetPointerMode.argtypes = [vp, ctypes.c_int]
    L.aclsparseGetPointerMode.argtypes = [vp, ctypes.POINTER(ctypes.c_int)]
    L.aclsparseCreateDnVec.argtypes = [PV, i64, vp, ctypes.c_int]
    L.aclsparseCreateConstDnVec.argtypes = [PV, i64, vp, ctypes.c_int]
    L.aclsparseDestroyDnVec.argtypes = [vp]
    L.aclsparseDnVecGet.argtypes = [vp, ctypes.POINTER(i64), PV, ctypes.POINTER(ctypes.c_int)]
    L.aclsparseConstDnVecGet.argtypes = L.aclsparseDnVecGet.argtypes
    L.aclsparseDnVecGetValues.argtypes = [vp, PV]
    L.aclsparseConstDnVecGetValues.argtypes = [vp, PV]
    L.aclsparseDnVecSetValues.argtypes = [vp, vp]
    csr_args = [PV, i64, i64, i64, vp, vp, vp, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int]
    L.aclsparseCreateCsr.argtypes = csr_args
    L.aclsparseCreateConstCsr.argtypes = csr_args
    L.aclsparseCsrSetPointers.argtypes = [vp, vp, vp, vp]
    L.aclsparseDestroySpMat.argtypes = [vp]
    L.aclsparseSpMatGetFormat.argtypes = [vp, ctypes.POINTER(ctypes.c_int)]
    L.aclsparseSpMatGetValues.argtypes = [vp, PV]
    L.aclsparseConstSpMatGetValues.argtypes = [vp, PV]
    L.aclsparseSpMatSetValues.argtypes = [vp, vp]
    L.aclsparseSpMatGetSize.argtypes = [vp, ctypes.POINTER(i64), ctypes.POINTER(i64), ctypes.POINTER(i64)]
    dn_args = [PV, i64, i64, i64, vp, ctypes.c_int, ctypes.c_int]
    L.aclsparseCreateDnMat.argtypes = dn_args
    L.aclsparseCreateConstDnMat.argtypes = dn_args
    L.aclsparseDestroyDnMat.argtypes = [vp]
    dn_get = [vp, ctypes.POINTER(i64), ctypes.POINTER(i64), ctypes.POINTER(i64), PV, ctypes.POINTER(ctypes.c_int),
              ctypes.POINTER(ctypes.c_int)]
    L.aclsparseDnMatGet.argtypes = dn_get
    L.aclsparseConstDnMatGet.argtypes = dn_get
    L.aclsparseDnMatGetValues.argtypes = [vp, PV]
    L.aclsparseConstDnMatGetValues.argtypes = [vp, PV]
    L.aclsparseDnMatSetValues.argtypes = [vp, vp]
    spmv_common = [vp, ctypes.c_int, vp, vp, vp, vp, vp, ctypes.c_int, ctypes.c_int]
    L.aclsparseSpMVGetBufferSize.argtypes = spmv_common + [ctypes.POINTER(sz)]
    L.aclsparseSpMVPreprocess.argtypes = spmv_common + [vp]
    L.aclsparseSpMV.argtypes = spmv_common + [vp]
    spmm_common = [vp, ctypes.c_int, ctypes.c_int, vp, vp, vp, vp, vp, ctypes.c_int, ctypes.c_int]
    L.aclsparseSpMMGetBufferSize.argtypes = spmm_common + [ctypes.POINTER(sz)]
    L.aclsparseSpMMPreprocess.argtypes = spmm_common + [vp]
    L.aclsparseSpMM.argtypes = spmm_common + [vp]
    spmvop_common = [vp, ctypes.c_int, vp, vp, vp, vp, ctypes.c_int, ctypes.c_int]
    L.aclsparseSpMVOp_bufferSize.argtypes = spmvop_common + [ctypes.POINTER(sz)]
    L.aclsparseSpMVOp_createDescr.argtypes = [vp, PV, ctypes.c_int, vp, vp, vp, vp, ctypes.c_int, ctypes.c_int, vp]
    L.aclsparseSpMVOp_destroyDescr.argtypes = [vp]
    L.aclsparseSpMVOp_createPlan.argtypes = [vp, vp, PV, vp, sz]
    L.aclsparseSpMVOp_destroyPlan.argtypes = [vp]
    L.aclsparseSpMVOp_setGlobalUserData.argtypes = [vp, vp, ctypes.c_char_p, vp, sz]
    L.aclsparseSpMVOp.argtypes = [vp, vp, vp, vp, vp, vp, vp]
    ci = ctypes.c_int
    L.aclsparseCreateMatDescr.argtypes = [PV]
    L.aclsparseDestroyMatDescr.argtypes = [vp]
    for name in ("Type", "IndexBase", "DiagType", "FillMode"):
        getattr(L, "aclsparseSetMat" + name).argtypes = [vp, ci]
        getattr(L, "aclsparseGetMat" + name).argtypes = [vp]
    L.aclsparseXcoo2csr.argtypes = [vp, vp, ci, ci, vp, ci]
    L.aclsparseXcsr2coo.argtypes = [vp, vp, i64, i64, vp, ci]
    L.aclsparseXcsrsort_bufferSizeExt.argtypes = [vp, ci, ci, ci, vp, vp, ctypes.POINTER(sz)]
    L.aclsparseXcsrsort.argtypes = [vp, ci, ci, ci, vp, vp, vp, vp, vp]
    L.aclsparseXcscsort_bufferSizeExt.argtypes = [vp, ci, ci, ci, vp, vp, ctypes.POINTER(sz)]
    L.aclsparseXcscsort.argtypes = [vp, ci, ci, ci, vp, vp, vp, vp, vp]
    L.aclsparseXcoosort_bufferSizeExt.argtypes = [vp, ci, ci, ci, vp, vp, ctypes.POINTER(sz)]
    L.aclsparseXcoosortByRow.argtypes = [vp, ci, ci, ci, vp, vp, vp, vp]
    L.aclsparseXcoosortByColumn.argtypes = [vp, ci, ci, ci, vp, vp, vp, vp]
    csc_common = [vp, ci, ci, ci, vp, vp, vp, vp, vp, vp, ci, ci, ci, ci]
    L.aclsparseCsr2cscEx2_bufferSize.argtypes = csc_common + [ctypes.POINTER(sz)]
    L.aclsparseCsr2cscEx2.argtypes = csc_common + [vp]
    L.opsparse_scan_workspace_bytes.restype = sz
    L.opsparse_scan_workspace_bytes.argtypes = [i64]
    L.opsparse_coo2csr_launch.restype = ci
    L.opsparse_coo2csr_launch.argtypes = [vp, i64, i64, vp, i32, vp, sz, vp]
    L.opsparse_csr2coo_launch.restype = ci
    L.opsparse_csr2coo_launch.argtypes = [vp, i64, i64, vp, i32, vp]
    L.opsparse_csrsort_workspace_bytes.restype = sz
    L.opsparse_csrsort_workspace_bytes.argtypes = [i64, i64]
    L.opsparse_csrsort_launch.restype = ci
    L.opsparse_csrsort_launch.argtypes = [i64, i64, i64, i32, vp, vp, vp, vp, sz, vp]
    L.opsparse_coosort_workspace_bytes.restype = sz
    L.opsparse_coosort_workspace_bytes.argtypes = [i64]
    L.opsparse_coosort_launch.restype = ci
    L.opsparse_coosort_launch.argtypes = [i64, i32, vp, vp, vp, vp, sz, vp]
    L.opsparse_csr2csc_workspace_bytes.restype = sz
    L.opsparse_csr2csc_workspace_bytes.argtypes = [i64, i64, i64]
    L.opsparse_csr2csc_launch.restype = ci
    L.opsparse_csr2csc_launch.argtypes = [i64, i64, i64, vp, vp, vp, vp, vp, vp, i32, i32, vp, sz, vp]

    L.opsparse_spmv_csr_workspace_bytes.restype = sz
    L.opsparse_spmv_csr_workspace_bytes.argtypes = [i64, i64]
    L.opsparse_spmv_csr_analyse.restype = ctypes.c_int
    L.opsparse_spmv_csr_analyse.argtypes = [vp, i64, i64, i64, vp, sz, i32, ctypes.POINTER(OpsparseSpmvPlan), vp]
    L.opsparse_spmv_csr_launch.restype = ctypes.c_int
    L.opsparse_spmv_csr_launch.argtypes = [ctypes.POINTER(OpsparseSpmvPlan), i32, vp, vp, vp, vp, vp, i64, i64, i64,
                                           OpsparseScalar, OpsparseScalar, i32, i32, i32, vp, sz, vp]
    L.opsparse_spmv_csr_launch_zy.restype = ctypes.c_int
    L.opsparse_spmv_csr_launch_zy.argtypes = [ctypes.POINTER(OpsparseSpmvPlan), i32, vp, vp, vp, vp, vp, vp, i64, i64,
                                              i64, OpsparseScalar, OpsparseScalar, i32, i32, i32, vp, sz, vp]
    L.opsparse_spmv_csr_noalloc_max_bytes.restype = sz
    L.opsparse_spmv_csr_noalloc_max_bytes.argtypes = []
    L.opsparse_spmv_csr_launch_noalloc.restype = ctypes.c_int
    L.opsparse_spmv_csr_launch_noalloc.argtypes = [vp, vp, vp, vp, vp, i64, i64, i64, OpsparseScalar, OpsparseScalar,
                                                   i32, i32, i32, vp]
    L.opsparse_spmv_csr_panels_workspace_bytes.restype = sz
    L.opsparse_spmv_csr_panels_workspace_bytes.argtypes = [i64, i64, i64]
    L.opsparse_spmv_csr_gathers_scattered.restype = ctypes.c_int
    L.opsparse_spmv_csr_gathers_scattered.argtypes = [vp, vp, i64, i64, i64, vp, sz, ctypes.POINTER(i32), vp]
    L.opsparse_spmv_csr_blocked_workspace_bytes.restype = sz
    L.opsparse_spmv_csr_blocked_workspace_bytes.argtypes = [i64, i64, i64, i32]
    L.opsparse_spmv_csr_blocked_resident_bytes.restype = sz
    L.opsparse_spmv_csr_blocked_resident_bytes.argtypes = [i64, i64, i64, i32]
    L.opsparse_spmv_csr_live_workspace_bytes.restype = sz
    L.opsparse_spmv_csr_live_workspace_bytes.argtypes = [i64, i64, i64]
    L.opsparse_spmv_csr_live_resident_bytes.restype = sz
    L.opsparse_spmv_csr_live_resident_bytes.argtypes = [i64, i64, i64]
    for name in ("opsparse_spmv_csr_scatter_workspace_bytes", "opsparse_spmv_csr_scatter_resident_bytes"):
        getattr(L, name).restype = sz
        getattr(L, name).argtypes = [i64, i64, i64, i32]
    L.opsparse_spmv_csr_scatter_analyse.restype = ctypes.c_int
    L.opsparse_spmv_csr_scatter_analyse.argtypes = [vp, vp, i64, i64, i64, i32, vp, sz, ctypes.POINTER(OpsparseSpmvPlan), vp]
    L.opsparse_spmv_csr_scatter_analyse_split.restype = ctypes.c_int
    L.opsparse_spmv_csr_scatter_analyse_split.argtypes = [vp, vp, i64, i64, i64, i32, vp, sz, vp, sz,
                                                          ctypes.POINTER(OpsparseSpmvPlan), vp]
    L.opsparse_spmv_csr_live_analyse.restype = ctypes.c_int
    L.opsparse_spmv_csr_live_analyse.argtypes = [vp, vp, vp, i64, i64, i64, i32, vp, sz,
                                                 ctypes.POINTER(OpsparseSpmvPlan), vp]
    for name in ("opsparse_spmv_csr_live_analyse_split", "opsparse_spmv_csr_blocked_analyse_split"):
        getattr(L, name).restype = ctypes.c_int
        getattr(L, name).argtypes = [vp, vp, vp, i64, i64, i64, i32, vp, sz, vp, sz, ctypes.POINTER(OpsparseSpmvPlan), vp]
    L.opsparse_spmv_csr_blocked_analyse.restype = ctypes.c_int
    L.opsparse_spmv_csr_blocked_analyse.argtypes = [vp, vp, vp, i64, i64, i64, i32, vp, sz,
                                                    ctypes.POINTER(OpsparseSpmvPlan), vp]
    L.opsparse_spmv_csr_panels_analyse.restype = ctypes.c_int
    L.opsparse_spmv_csr_panels_analyse.argtypes = [vp, vp, vp, i64, i64, i64, vp, sz, ctypes.POINTER(OpsparseSpmvPlan),
                                                   vp]
    L.opsparse_rebase_offsets_launch.restype = ctypes.c_int
    L.opsparse_rebase_offsets_launch.argtypes = [vp, i32, i32, i64, vp, vp]
    L.opsparse_spmv_csr_indexed_launch.restype = ctypes.c_int
    L.opsparse_spmv_csr_indexed_launch.argtypes = [vp, i32, i32, vp, vp, vp, vp, vp, i64, i64, i64, OpsparseScalar,
                                                   OpsparseScalar, vp]
    L.opsparse_spmm_csr_workspace_bytes.restype = ctypes.c_int
    L.opsparse_spmm_csr_workspace_bytes.argtypes = [vp, i64, i64, i64, vp, ctypes.POINTER(sz)]
    L.opsparse_spmm_csr_analyse.restype = ctypes.c_int
    L.opsparse_spmm_csr_analyse.argtypes = [vp, i64, i64, i64, vp, sz, i32, ctypes.POINTER(OpsparseSpmmPlan), vp]
    L.opsparse_spmm_csr_launch.restype = ctypes.c_int
    L.opsparse_spmm_csr_launch.argtypes = [ctypes.POINTER(OpsparseSpmmPlan), vp, vp, vp, vp, vp, i64, i64, i64, i64,
                                           i64, i64, i32, i32, i32, OpsparseScalar, OpsparseScalar, i32, i32, vp, sz,
                                           vp]
    L.opsparse_spmm_csr_narrow_rows.restype = ctypes.c_int
    L.opsparse_spmm_csr_narrow_rows.argtypes = [ctypes.POINTER(OpsparseSpmmPlan), vp, i64, i64, i32, i32]
    L.opsparse_dense_restage.restype = ctypes.c_int
    L.opsparse_dense_restage.argtypes = [vp, vp, i64, i64, i64, i64, i32, i64, i32, i32, vp]
    L.opsparse_copy_launch.restype = ctypes.c_int
    L.opsparse_copy_launch.argtypes = [vp, vp, sz, vp]
    L.opsparse_read_launch.restype = ctypes.c_int
    L.opsparse_read_launch.argtypes = [vp, sz, vp, vp]
    L.opsparse_gather_launch.restype = ctypes.c_int
    L.opsparse_gather_launch.argtypes = [vp, vp, sz, vp, vp]
    _lib = L
    return L


class AclsparseError(RuntimeError):
    def __init__(self, what, status):
        self.status = status
        name = STATUS_NAMES[status] if 0 <= status < len(STATUS_NAMES) else str(status)
        super().__init__("%s returned ACL_SPARSE_STATUS_%s" % (what, name))


def check(status, what="aclsparse call"):
    if status != ACL_SPARSE_STATUS_SUCCESS:
        raise AclsparseError(what, status)


def _acl_dtype(t):
    import torch
    return {torch.float32: ACL_FLOAT, torch.float16: ACL_FLOAT16, torch.bfloat16: ACL_BF16, torch.int32: ACL_INT32,
            torch.int8: ACL_INT8, torch.float64: ACL_DOUBLE, torch.int64: ACL_INT64}[t.dtype]


def _ptr(t):
    return vp(t.data_ptr()) if t is not None and t.numel() > 0 else vp(None)


class Handle:
    """aclsparseCreate / SetStream / Destroy.  `stream` is a torch.cuda.Stream (or None)."""

    def __init__(self, stream=None):
        self.h = vp(None)
        check(lib().aclsparseCreate(ctypes.byref(self.h)), "aclsparseCreate")
        self.stream = stream
        if stream is not None:
            check(lib().aclsparseSetStream(self.h, vp(stream.cuda_stream)), "aclsparseSetStream")

    def set_pointer_mode(self, mode):
        check(lib().aclsparseSetPointerMode(self.h, mode), "aclsparseSetPointerMode")

    def close(self):
        if self.h:
            lib().aclsparseDestroy(self.h)
            self.h = vp(None)

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Csr:
    """aclsparseCreateCsr over three device tensors (kept alive here)."""

    def __init__(self, rows, cols, rowptr, colind, values, index_base=ACL_SPARSE_INDEX_BASE_ZERO):
        self.rows, self.cols, self.nnz = int(rows), int(cols), int(colind.numel())
        self.rowptr, self.colind, self.values = rowptr, colind, values
        self.d = vp(None)
        it = lambda t: ACL_SPARSE_INDEX_64I if t.dtype.itemsize == 8 else ACL_SPARSE_INDEX_32I
        check(lib().aclsparseCreateCsr(ctypes.byref(self.d), self.rows, self.cols, self.nnz, _ptr(rowptr),
                                       _ptr(colind), _ptr(values), it(rowptr), it(colind), index_base,
                                       _acl_dtype(values)), "aclsparseCreateCsr")

    def close(self):
        if self.d:
            lib().aclsparseDestroySpMat(self.d)
            self.d = vp(None)

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class DnVec:
    def __init__(self, tensor):
        self.t = tensor
        self.d = vp(None)
        check(lib().aclsparseCreateDnVec(ctypes.byref(self.d), tensor.numel(), _ptr(tensor), _acl_dtype(tensor)),
              "aclsparseCreateDnVec")

    def close(self):
        if self.d:
            lib().aclsparseDestroyDnVec(self.d)
            self.d = vp(None)

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class DnMat:
    """aclsparseCreateDnMat over a flat (or 2-D contiguous) device tensor in its storage layout."""

    def __init__(self, rows, cols, ld, tensor, order=ACL_SPARSE_ORDER_ROW):
        self.t = tensor
        self.rows, self.cols, self.ld, self.order = int(rows), int(cols), int(ld), order
        self.d = vp(None)
        check(lib().aclsparseCreateDnMat(ctypes.byref(self.d), self.rows, self.cols, self.ld, _ptr(tensor),
                                         _acl_dtype(tensor), order), "aclsparseCreateDnMat")

    def close(self):
        if self.d:
            lib().aclsparseDestroyDnMat(self.d)
            self.d = vp(None)

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def _scalar_ref(v, compute_type):
    """Host scalar of the compute type, returned as (ctypes object, void pointer)."""
    if v is None:
        return None, vp(None)
    c = ctypes.c_int32(int(v)) if compute_type == ACL_INT32 else ctypes.c_float(float(v))
    return c, ctypes.cast(ctypes.pointer(c), vp)


class SpmvOp:
    """One matrix / vector pair bound for repeated y = alpha*op(A)*x + beta*y calls.

    preprocess=True runs aclsparseSpMVGetBufferSize + aclsparseSpMVPreprocess once
    and passes the buffer to every aclsparseSpMV; preprocess=False passes NULL.
    """

    def __init__(self, handle, A, x, y, op=ACL_SPARSE_OP_NON_TRANSPOSE, compute_type=ACL_FLOAT, preprocess=True,
                 alg=ACL_SPARSE_SPMV_ALG_DEFAULT):
        import torch
        self.handle, self.A, self.x, self.y = handle, A, x, y
        self.op, self.compute_type, self.alg = op, compute_type, alg
        self.buffer = None
        if preprocess:
            n = sz(0)
            check(lib().aclsparseSpMVGetBufferSize(handle.h, op, None, A.d, x.d, None, y.d, compute_type, alg,
                                                   ctypes.byref(n)), "aclsparseSpMVGetBufferSize")
            self.buffer = torch.empty(max(int(n.value), 16), dtype=torch.uint8, device=y.t.device)
            check(lib().aclsparseSpMVPreprocess(handle.h, op, None, A.d, x.d, None, y.d, compute_type, alg,
                                                _ptr(self.buffer)), "aclsparseSpMVPreprocess")

    def __call__(self, alpha=1.0, beta=0.0):
        ka, pa = _scalar_ref(alpha, self.compute_type)
        kb, pb = _scalar_ref(beta, self.compute_type)
        st = lib().aclsparseSpMV(self.handle.h, self.op, pa, self.A.d, self.x.d, pb, self.y.d, self.compute_type,
                                 self.alg, _ptr(self.buffer) if self.buffer is not None else vp(None))
        check(st, "aclsparseSpMV")


class SpmvOpPlan:
    """aclsparseSpMVOp_bufferSize -> createDescr -> createPlan, then z = alpha*A*x + beta*y per call.

    x, y, z are DnVec objects; z may be y.  The descriptor, the plan and (ALG2) the
    buffer live as long as this object.
    """

    def __init__(self, handle, A, x, y, z, alg=ACL_SPARSE_SPMVOP_ALG_DEFAULT):
        import torch
        self.handle, self.A, self.x, self.y, self.z, self.alg = handle, A, x, y, z, alg
        self.descr, self.plan = vp(None), vp(None)
        n = sz(0)
        common = (ACL_SPARSE_OP_NON_TRANSPOSE, A.d, x.d, y.d, z.d, ACL_FLOAT, alg)
        check(lib().aclsparseSpMVOp_bufferSize(handle.h, *common, ctypes.byref(n)), "aclsparseSpMVOp_bufferSize")
        self.buffer_bytes = int(n.value)
        self.buffer = None
        if alg == ACL_SPARSE_SPMVOP_ALG2 or self.buffer_bytes > 0:
            self.buffer = torch.empty(max(self.buffer_bytes, 16), dtype=torch.uint8, device=z.t.device)
        check(lib().aclsparseSpMVOp_createDescr(handle.h, ctypes.byref(self.descr), *common,
                                                _ptr(self.buffer) if self.buffer is not None else vp(None)),
              "aclsparseSpMVOp_createDescr")
        check(lib().aclsparseSpMVOp_createPlan(handle.h, self.descr, ctypes.byref(self.plan), None, 0),
              "aclsparseSpMVOp_createPlan")

    def __call__(self, alpha=1.0, beta=0.0, x=None, y=None, z=None):
        """alpha / beta: Python numbers (HOST pointer mode) or one-element fp32 device tensors (DEVICE mode)."""
        if hasattr(alpha, "data_ptr"):
            pa, pb = vp(alpha.data_ptr()), vp(beta.data_ptr())
        else:
            ka, pa = _scalar_ref(alpha, ACL_FLOAT)
            kb, pb = _scalar_ref(beta, ACL_FLOAT)
        st = lib().aclsparseSpMVOp(self.handle.h, self.plan, pa, pb, (x or self.x).d, (y or self.y).d,
                                   (z or self.z).d)
        check(st, "aclsparseSpMVOp")

    def close(self):
        # plan first: it only borrows the descriptor
        if self.plan:
            lib().aclsparseSpMVOp_destroyPlan(self.plan)
            self.plan = vp(None)
        if self.descr:
            lib().aclsparseSpMVOp_destroyDescr(self.descr)
            self.descr = vp(None)

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class SpmmOp:
    """aclsparseSpMMGetBufferSize -> Preprocess -> SpMM for one (A, B, C) triple."""

    def __init__(self, handle, A, B, C, op_b=ACL_SPARSE_OP_NON_TRANSPOSE, compute_type=ACL_FLOAT,
                 alg=ACL_SPARSE_SPMM_ALG_DEFAULT):
        import torch
        self.handle, self.A, self.B, self.C = handle, A, B, C
        self.op_b, self.compute_type, self.alg = op_b, compute_type, alg
        n = sz(0)
        args = (handle.h, ACL_SPARSE_OP_NON_TRANSPOSE, op_b, None, A.d, B.d, None, C.d, compute_type, alg)
        check(lib().aclsparseSpMMGetBufferSize(*args, ctypes.byref(n)), "aclsparseSpMMGetBufferSize")
        self.buffer_bytes = int(n.value)
        self.buffer = torch.empty(max(self.buffer_bytes, 16), dtype=torch.uint8, device=C.t.device)
        check(lib().aclsparseSpMMPreprocess(*args, _ptr(self.buffer)), "aclsparseSpMMPreprocess")

    def __call__(self, alpha=1.0, beta=0.0):
        ka, pa = _scalar_ref(alpha, self.compute_type)
        kb, pb = _scalar_ref(beta, self.compute_type)
        st = lib().aclsparseSpMM(self.handle.h, ACL_SPARSE_OP_NON_TRANSPOSE, self.op_b, pa, self.A.d, self.B.d, pb,
                                 self.C.d, self.compute_type, self.alg, _ptr(self.buffer))
        check(st, "aclsparseSpMM")
