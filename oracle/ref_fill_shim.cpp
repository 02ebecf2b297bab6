// TEST INFRASTRUCTURE ONLY.  C entry points around the reference's own seeded
// data generator: this file contains no generator code, it includes the
// reference header test/frame/fill.h from the reference tree (REF_FILL_H is
// set by oracle/Makefile) and forwards to it.  The resulting library lives in
// oracle/_ref/ and is used by tests to check oracle.c's restatement of the
// generator and to write the fixtures under tests/golden/.
#include REF_FILL_H

#include <cstdint>
#include <cstring>

extern "C" {

// SparseFillGenerator(seed) with setSparsity / setEmptyRowProb / setValueRange
// then generateCsr(rows, cols, nnzHint).  Arrays are filled up to `capacity`
// entries; the return value is the generated nnz (which may exceed capacity,
// in which case call again with larger arrays).
int64_t ref_fill_csr(uint32_t seed, int64_t rows, int64_t cols, int64_t nnzHint, double sparsity,
                     double emptyRowProb, double lo, double hi, int32_t *rowptr, int32_t *colind, float *val,
                     int64_t capacity)
{
    sparse_test::SparseFillGenerator gen(seed);
    gen.setSparsity(sparsity);
    gen.setEmptyRowProb(emptyRowProb);
    gen.setValueRange(lo, hi);
    const sparse_test::CsrMatrix m = gen.generateCsr(rows, cols, nnzHint);
    std::memcpy(rowptr, m.rowOffsets.data(), sizeof(int32_t) * m.rowOffsets.size());
    const int64_t n = static_cast<int64_t>(m.colIndices.size());
    const int64_t copy = n < capacity ? n : capacity;
    std::memcpy(colind, m.colIndices.data(), sizeof(int32_t) * copy);
    std::memcpy(val, m.values.data(), sizeof(float) * copy);
    return n;
}

// makeDenseFloat(size, lo, hi, seed)
void ref_fill_dense(uint32_t seed, int64_t size, double lo, double hi, float *out)
{
    const std::vector<float> v = sparse_test::makeDenseFloat(size, lo, hi, seed);
    std::memcpy(out, v.data(), sizeof(float) * v.size());
}

}  // extern "C"
