/* The two public headers must be usable from plain C (the boundary is a C ABI):
 * this file is compiled with `gcc -std=c99 -fsyntax-only` by tests/test_cpp_frame.py.
 * Taking every entry point's address checks that each is declared with C linkage
 * and a complete prototype. */
#include "cann_ops_sparse.h"
#include "ops_sparse_hip.h"

typedef void (*fn)(void);

fn opsparse_abi_table[] = {
    (fn)aclsparseCreate, (fn)aclsparseDestroy, (fn)aclsparseSetStream, (fn)aclsparseGetStream,
    (fn)aclsparseSetWorkspace, (fn)aclsparseGetWorkspace, (fn)aclsparseGetVersion, (fn)aclsparseSetPointerMode,
    (fn)aclsparseGetPointerMode, (fn)aclsparseCreateDnVec, (fn)aclsparseCreateConstDnVec, (fn)aclsparseDestroyDnVec,
    (fn)aclsparseCreateCsr, (fn)aclsparseCreateConstCsr, (fn)aclsparseCsrSetPointers, (fn)aclsparseDestroySpMat,
    (fn)aclsparseCreateDnMat, (fn)aclsparseCreateConstDnMat, (fn)aclsparseDestroyDnMat,
    (fn)aclsparseSpMVGetBufferSize, (fn)aclsparseSpMVPreprocess, (fn)aclsparseSpMV,
    (fn)aclsparseSpMMGetBufferSize, (fn)aclsparseSpMMPreprocess, (fn)aclsparseSpMM,
    (fn)aclsparseSpMVOp_bufferSize, (fn)aclsparseSpMVOp_createDescr, (fn)aclsparseSpMVOp_destroyDescr,
    (fn)aclsparseSpMVOp_createPlan, (fn)aclsparseSpMVOp_destroyPlan, (fn)aclsparseSpMVOp_setGlobalUserData,
    (fn)aclsparseSpMVOp, (fn)aclsparseCreateMatDescr, (fn)aclsparseDestroyMatDescr, (fn)aclsparseSetMatIndexBase,
    (fn)aclsparseGetMatIndexBase, (fn)aclsparseXcoo2csr, (fn)aclsparseXcsr2coo, (fn)aclsparseXcsrsort_bufferSizeExt,
    (fn)aclsparseXcsrsort, (fn)aclsparseCsr2cscEx2_bufferSize, (fn)aclsparseCsr2cscEx2,
    (fn)opsparse_spmv_csr_workspace_bytes, (fn)opsparse_spmv_csr_analyse, (fn)opsparse_spmv_csr_launch,
    (fn)opsparse_spmv_csr_launch_zy, (fn)opsparse_spmv_csr_indexed_launch,
    (fn)opsparse_spmv_csr_panels_workspace_bytes, (fn)opsparse_spmv_csr_panels_analyse,
    (fn)opsparse_spmm_csr_workspace_bytes, (fn)opsparse_spmm_csr_analyse, (fn)opsparse_spmm_csr_launch,
    (fn)opsparse_scan_workspace_bytes, (fn)opsparse_coo2csr_launch, (fn)opsparse_csr2coo_launch,
    (fn)opsparse_csrsort_workspace_bytes, (fn)opsparse_csrsort_launch, (fn)opsparse_csr2csc_workspace_bytes,
    (fn)opsparse_csr2csc_launch, (fn)opsparse_copy_launch, (fn)opsparse_read_launch, (fn)opsparse_gather_launch,
};

OpsparseSpmvPlan opsparse_abi_spmv_plan;
OpsparseSpmmPlan opsparse_abi_spmm_plan;
OpsparseScalar opsparse_abi_scalar;
