// TEST INFRASTRUCTURE ONLY.  C entry points around the reference's own CPU
// goldens of the CSR producers.  This file contains none of their code: it
// includes the golden headers where they lie in the reference tree (the
// REF_*_H macros are set by oracle/Makefile; the headers need only the C++
// standard library and test/frame/fill.h) and forwards to them.  The library
// lives in oracle/_ref/ and is used by tests to check oracle.c's restatements.
#include <cstddef>  // the golden headers use size_t unqualified

#include REF_COO2CSR_H
#include REF_CSR2COO_H
#include REF_CSRSORT_H
#include REF_CSR2CSC_H
#include REF_COOSORT_H
#include REF_CSCSORT_H

#include <cstdint>
#include <cstring>
#include <vector>

extern "C" {

void ref_coo2csr(const int32_t *rowInd, int32_t nnz, int32_t m, int32_t base, int32_t *rowPtr)
{
    const std::vector<int32_t> in(rowInd, rowInd + nnz);
    const std::vector<int32_t> out = sparse_test::Coo2CsrGolden(in, nnz, m, base);
    std::memcpy(rowPtr, out.data(), sizeof(int32_t) * out.size());
}

void ref_csr2coo(const int32_t *rowPtr, int64_t m, int64_t nnz, int32_t base, int32_t *rowInd)
{
    const std::vector<int32_t> in(rowPtr, rowPtr + m + 1);
    const std::vector<int32_t> out = sparse_test::Csr2CooGolden(in, m, nnz, base);
    std::memcpy(rowInd, out.data(), sizeof(int32_t) * out.size());
}

void ref_csrsort(const int32_t *rowPtr, int32_t m, int32_t nnz, int32_t base, int32_t *colInd, int32_t *perm)
{
    const std::vector<int32_t> rp(rowPtr, rowPtr + m + 1), ci(colInd, colInd + nnz), p(perm, perm + nnz);
    const sparse_test::CsrsortGoldenResult r = sparse_test::csrsortGolden(rp, ci, p, m, base);
    std::memcpy(colInd, r.colInd.data(), sizeof(int32_t) * nnz);
    std::memcpy(perm, r.P.data(), sizeof(int32_t) * nnz);
}

// Values as fp32 bit patterns; narrower types are the caller's business (the
// golden moves raw bytes, so one width pins the permutation).
void ref_csr2csc(int32_t m, int32_t n, int32_t nnz, int32_t base, const int32_t *rowPtr, const int32_t *colInd,
                 const float *val, int32_t *colPtr, int32_t *rowInd, float *cscVal)
{
    sparse_test::CsrMatrix csr;
    csr.rows = m;
    csr.cols = n;
    csr.nnz = nnz;
    csr.rowOffsets.assign(rowPtr, rowPtr + m + 1);
    csr.colIndices.assign(colInd, colInd + nnz);
    const std::vector<float> values(val, val + nnz);
    const sparse_test::Csr2CscGoldenResult r = sparse_test::Csr2CscGolden<float>(csr, values, base);
    std::memcpy(colPtr, r.cscColPtr.data(), sizeof(int32_t) * r.cscColPtr.size());
    if (nnz > 0) {
        std::memcpy(rowInd, r.cscRowInd.data(), sizeof(int32_t) * nnz);
        std::memcpy(cscVal, r.cscVal.data(), sizeof(float) * nnz);
    }
}

// P is taken to be 0 .. nnz-1 on entry, as the golden does.
void ref_coosort(const int32_t *rows, const int32_t *cols, int32_t nnz, int32_t byRow, int32_t *outRows,
                 int32_t *outCols, int32_t *outP)
{
    const std::vector<int32_t> r(rows, rows + nnz), c(cols, cols + nnz);
    const sparse_test::CoosortGoldenResult g = sparse_test::coosortGolden(r, c, byRow != 0);
    if (nnz > 0) {
        std::memcpy(outRows, g.rows.data(), sizeof(int32_t) * nnz);
        std::memcpy(outCols, g.cols.data(), sizeof(int32_t) * nnz);
        std::memcpy(outP, g.P.data(), sizeof(int32_t) * nnz);
    }
}

void ref_cscsort(const int32_t *colPtr, int32_t n, int32_t nnz, int32_t base, int32_t *rowInd, int32_t *perm)
{
    const std::vector<int32_t> cp(colPtr, colPtr + n + 1), ri(rowInd, rowInd + nnz), p(perm, perm + nnz);
    const sparse_test::CscsortGoldenResult r = sparse_test::cscsortGolden(cp, ri, p, n, base);
    if (nnz > 0) {
        std::memcpy(rowInd, r.rowInd.data(), sizeof(int32_t) * nnz);
        std::memcpy(perm, r.P.data(), sizeof(int32_t) * nnz);
    }
}

}  // extern "C"
