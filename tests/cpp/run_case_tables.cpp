// Runs the reference's CSV case tables (tests/golden/*.csv) against
// libops_sparse.so from C++, the way a caller of the reference would: through
// cann_ops_sparse.h only.  One line per case; exit status 0 iff all passed.
//
//   run_case_tables <directory with the csv files> [table ...]
//
// Tables: spmv_op, coo2csr, csr2coo, csr2csc, csrsort (default: all).  Mirrors
// test/spmv_op/arch35/spmv_op_test.cpp:73-142, test/coo2csr/arch35/coo2csr_test.cpp,
// test/csr2coo/arch35/csr2coo_test.cpp and test/csr2csc_ex2/arch35/csr2csc_ex2_test.cpp of the
// reference, with the frame of tests/cpp/frame.h and the CPU oracle as golden.  csrsort has no
// csv in the reference: its named success cases (test/csrsort/arch35/csrsort_test.cpp:239-420) are
// built here as that program builds them.
#include <cmath>
#include <cstring>

#include "frame.h"

using frame::Check;
using Row = std::map<std::string, std::string>;

namespace {

int64_t I(const Row &r, const char *k) { return std::stoll(r.at(k)); }
double D(const Row &r, const char *k) { return std::stod(r.at(k)); }

frame::CsrHost Matrix(const Row &r, const char *colsKey)
{
    const int64_t m = I(r, "m"), n = I(r, colsKey);
    if (r.at("pattern") == "diag") {
        return frame::DiagCsr(m);
    }
    if (r.at("pattern") == "empty" || m <= 0 || n <= 0 || D(r, "sparsity") >= 1.0) {
        frame::CsrHost a;
        a.rows = m;
        a.cols = n;
        a.rowptr.assign(static_cast<size_t>(m > 0 ? m : 0) + 1, 0);
        return a;
    }
    return frame::FillCsr(m, n, D(r, "sparsity"), D(r, "empty_row_prob"), static_cast<uint32_t>(I(r, "seed")), -5.0f,
                            5.0f);
}

bool SpmvOpCase(const frame::Stream &stream, const frame::Handle &handle, const Row &r)
{
    frame::CsrHost a = Matrix(r, "k");
    const int64_t m = a.rows, k = a.cols, nnz = a.nnz();
    const uint32_t seed = static_cast<uint32_t>(I(r, "seed"));
    if (I(r, "unsorted") != 0) {  // shuffle the entries inside every row
        std::mt19937 rng(seed);
        for (int64_t i = 0; i < m; ++i) {
            for (int32_t p = a.rowptr[i + 1] - 1; p > a.rowptr[i]; --p) {
                const int32_t q = a.rowptr[i] + static_cast<int32_t>(rng() % static_cast<uint32_t>(p - a.rowptr[i] + 1));
                std::swap(a.colind[p], a.colind[q]);
                std::swap(a.val[p], a.val[q]);
            }
        }
    }
    const std::vector<float> x = frame::FillDense(k, -3.0f, 3.0f, seed + 1);
    const std::vector<float> y = frame::FillDense(m, -3.0f, 3.0f, seed + 2);
    const float alpha = static_cast<float>(D(r, "alpha")), beta = static_cast<float>(D(r, "beta"));
    std::vector<float> gold(static_cast<size_t>(m));
    oracle_spmv_f64(m, k, a.rowptr.data(), a.colind.data(), a.val.data(), x.data(), y.data(), alpha, beta, gold.data());

    const bool i64 = r.at("row_offset_type") == "i64", alias = I(r, "alias_z_y") != 0;
    const bool deviceScalars = r.at("pointer_mode") == "DEVICE";
    frame::DeviceArray<int32_t> dPtr32(i64 ? std::vector<int32_t>{} : a.rowptr);
    frame::DeviceArray<int64_t> dPtr64(i64 ? std::vector<int64_t>(a.rowptr.begin(), a.rowptr.end()) : std::vector<int64_t>{});
    frame::DeviceArray<int32_t> dCol(a.colind);
    frame::DeviceArray<float> dVal(a.val), dX(x), dY(y), dZ(static_cast<size_t>(alias ? 0 : m));
    frame::DeviceArray<float> dScal(std::vector<float>{alpha, beta});
    void *rowPtr = i64 ? static_cast<void *>(dPtr64.get()) : static_cast<void *>(dPtr32.get());

    const frame::SpMat ownA = frame::SpMat::createCsr(m, k, nnz, rowPtr, dCol.get(), dVal.get(),
                                                      i64 ? ACL_SPARSE_INDEX_64I : ACL_SPARSE_INDEX_32I);
    const frame::DnVec ownX = frame::DnVec::create(k, dX.get()), ownY = frame::DnVec::create(m, dY.get());
    const frame::DnVec ownZ = alias ? frame::DnVec() : frame::DnVec::create(m, dZ.get());
    const aclsparseSpMatDescr_t matA = ownA.get();
    const aclsparseDnVecDescr_t vx = ownX.get(), vy = ownY.get(), vz = ownZ.get();
    aclsparseDnVecDescr_t out = alias ? vy : vz;
    const std::string algName = r.at("alg");
    const aclsparseSpMVOpAlg_t alg = algName == "ALG2"   ? ACL_SPARSE_SPMVOP_ALG2
                                     : algName == "ALG1" ? ACL_SPARSE_SPMVOP_ALG1
                                                         : ACL_SPARSE_SPMVOP_ALG_DEFAULT;
    size_t bytes = 0;
    Check(aclsparseSpMVOp_bufferSize(handle.get(), ACL_SPARSE_OP_NON_TRANSPOSE, matA, vx, vy, out, ACL_FLOAT, alg, &bytes),
          "aclsparseSpMVOp_bufferSize");
    frame::DeviceArray<unsigned char> buffer(alg == ACL_SPARSE_SPMVOP_ALG2 ? (bytes > 0 ? bytes : 16) : 0);
    aclsparseSpMVOpDescr_t descr = nullptr;
    aclsparseSpMVOpPlan_t plan = nullptr;
    Check(aclsparseSpMVOp_createDescr(handle.get(), &descr, ACL_SPARSE_OP_NON_TRANSPOSE, matA, vx, vy, out, ACL_FLOAT, alg,
                                      buffer.get()), "aclsparseSpMVOp_createDescr");
    Check(aclsparseSpMVOp_createPlan(handle.get(), descr, &plan, nullptr, 0), "aclsparseSpMVOp_createPlan");
    Check(aclsparseSetPointerMode(handle.get(), deviceScalars ? ACL_SPARSE_POINTER_MODE_DEVICE
                                                              : ACL_SPARSE_POINTER_MODE_HOST), "aclsparseSetPointerMode");
    const void *pa = deviceScalars ? static_cast<const void *>(dScal.get()) : &alpha;
    const void *pb = deviceScalars ? static_cast<const void *>(dScal.get() + 1) : &beta;
    const aclsparseStatus_t st = aclsparseSpMVOp(handle.get(), plan, pa, pb, vx, vy, out);
    (void)aclsparseSetPointerMode(handle.get(), ACL_SPARSE_POINTER_MODE_HOST);
    Check(st, "aclsparseSpMVOp");
    stream.sync();
    const std::vector<float> got = alias ? dY.download() : dZ.download();
    (void)aclsparseSpMVOp_destroyPlan(plan);
    (void)aclsparseSpMVOp_destroyDescr(descr);

    // |d| <= 1e-5 |gold| per element, and the table's own MERE / MARE limits
    for (int64_t i = 0; i < m; ++i) {
        const double g = gold[i], d = std::fabs(static_cast<double>(got[i]) - g);
        if (!(d <= 1e-5 * std::fmax(std::fabs(g), 1e-30))) {
            std::printf("    element %lld: got %.9g, golden %.9g\n", static_cast<long long>(i), got[i], gold[i]);
            return false;
        }
    }
    const frame::VerifyReport rep = frame::Verify(
        got.data(), gold.data(), static_cast<size_t>(m), 1,
        frame::VerifyConfig().SetMERE(D(r, "mere_threshold")).SetMARE(D(r, "mare_multiplier")));
    return rep.pass;
}

// ---- csrsort: the named cases of the reference's test program

struct SortCase {
    std::string name;
    int m = 0, n = 0;
    int32_t base = 0;
    std::vector<int32_t> rowPtr, colInd, perm;  // perm empty: the identity
};

std::vector<SortCase> SortCases()
{
    std::vector<SortCase> c;
    c.push_back({"Basic", 3, 3, 0, {0, 3, 6, 9}, {2, 1, 0, 0, 2, 1, 1, 2, 0}, {}});
    c.push_back({"EmptyRows", 4, 5, 0, {0, 0, 2, 2, 4}, {3, 1, 4, 2}, {}});
    c.push_back({"AlreadySorted", 3, 5, 0, {0, 2, 4, 6}, {0, 1, 2, 3, 0, 4}, {}});
    c.push_back({"Reverse", 3, 5, 0, {0, 2, 4, 6}, {4, 0, 3, 2, 4, 1}, {}});
    c.push_back({"DuplicateCols", 1, 5, 0, {0, 5}, {2, 1, 2, 1, 0}, {10, 20, 30, 40, 50}});
    c.push_back({"NonIdentityP", 2, 4, 0, {0, 2, 4}, {3, 1, 0, 2}, {100, 200, 300, 400}});
    c.push_back({"Base1", 2, 4, 1, {1, 3, 5}, {4, 2, 1, 3}, {}});
    c.push_back({"EmptyMatrix", 3, 3, 0, {0, 0, 0, 0}, {}, {}});
    c.push_back({"SingleElemRows", 4, 4, 0, {0, 0, 1, 1, 2}, {3, 1}, {}});
    {  // ManySmallRows: 200 rows of rng() % 4 entries, columns rng() % 10, std::mt19937(99)
        SortCase s{"ManySmallRows", 200, 10, 0, std::vector<int32_t>(201, 0), {}, {}};
        std::mt19937 rng(99);
        for (int i = 0; i < s.m; ++i) {
            const int len = static_cast<int>(rng() % 4);
            for (int j = 0; j < len; ++j) {
                s.colInd.push_back(static_cast<int32_t>(rng() % static_cast<uint32_t>(s.n)));
            }
            s.rowPtr[i + 1] = static_cast<int32_t>(s.colInd.size());
        }
        c.push_back(s);
    }
    {  // MultiCoreSkewedRows: rows of 10000, 2048, 0 and row % 7 entries
        SortCase s{"MultiCoreSkewedRows", 257, 4096, 0, std::vector<int32_t>(258, 0), {}, {}};
        for (int row = 0; row < s.m; ++row) {
            const int len = row % 64 == 0 ? 10000 : (row % 8 == 0 ? 2048 : (row % 5 != 0 ? row % 7 : 0));
            for (int j = 0; j < len; ++j) {
                s.colInd.push_back((row * 131 + len - j) % s.n);
            }
            s.rowPtr[row + 1] = static_cast<int32_t>(s.colInd.size());
        }
        c.push_back(s);
    }
    {  // LongRow: one row, a shuffle of 0 .. 999
        SortCase s{"LongRow", 1, 1000, 0, {0, 1000}, std::vector<int32_t>(1000), {}};
        for (int i = 0; i < 1000; ++i) {
            s.colInd[i] = i;
        }
        std::mt19937 rng(123);
        std::shuffle(s.colInd.begin(), s.colInd.end(), rng);
        c.push_back(s);
    }
    {  // LongRowMultiRun: one row of 32768 entries over 4096 columns, every key eight times
        SortCase s{"LongRowMultiRun", 1, 4096, 0, {0, 32768}, std::vector<int32_t>(32768), {}};
        for (int i = 0; i < 32768; ++i) {
            s.colInd[i] = i % s.n;
        }
        std::mt19937 rng(2026);
        std::shuffle(s.colInd.begin(), s.colInd.end(), rng);
        c.push_back(s);
    }
    {  // SingleHugeRow: a million entries in one row, 4096 distinct keys
        constexpr int nnz = 1024 * 1024;
        SortCase s{"SingleHugeRow", 1, 65536, 0, {0, nnz}, std::vector<int32_t>(nnz), std::vector<int32_t>(nnz)};
        for (int i = 0; i < nnz; ++i) {
            s.colInd[i] = static_cast<int32_t>((static_cast<uint64_t>(i) * 65521U + 7919U) % 4096U);
            s.perm[i] = i;
        }
        c.push_back(s);
    }
    return c;
}

// RunSortAndVerify of the reference (csrsort_test.cpp:118-232): an empty matrix needs no buffer and no arrays;
// otherwise bufferSizeExt must ask for a buffer, and row offsets, sorted columns and P are compared exactly.
bool CsrsortCase(const frame::Stream &stream, const frame::Handle &handle, const SortCase &c)
{
    const int nnz = static_cast<int>(c.colInd.size());
    aclsparseMatDescr_t descr = nullptr;
    Check(aclsparseCreateMatDescr(&descr), "aclsparseCreateMatDescr");
    aclsparseSetMatIndexBase(descr, static_cast<aclsparseIndexBase_t>(c.base));
    bool ok = false;
    if (nnz == 0) {
        size_t bytes = 42;
        Check(aclsparseXcsrsort_bufferSizeExt(handle.get(), c.m, c.n, 0, c.rowPtr.data(), nullptr, &bytes),
              "aclsparseXcsrsort_bufferSizeExt");
        Check(aclsparseXcsrsort(handle.get(), c.m, c.n, 0, descr, c.rowPtr.data(), nullptr, nullptr, nullptr),
              "aclsparseXcsrsort");
        ok = bytes == 0;
    } else {
        std::vector<int32_t> perm = c.perm;
        if (perm.empty()) {
            perm.resize(static_cast<size_t>(nnz));
            for (int i = 0; i < nnz; ++i) {
                perm[i] = i;
            }
        }
        std::vector<int32_t> goldCol = c.colInd, goldPerm = perm;
        oracle_csrsort(c.rowPtr.data(), c.m, c.base, goldCol.data(), goldPerm.data());
        frame::DeviceArray<int32_t> dPtr(c.rowPtr), dCol(c.colInd), dPerm(perm);
        size_t bytes = 0;
        Check(aclsparseXcsrsort_bufferSizeExt(handle.get(), c.m, c.n, nnz, dPtr.get(), dCol.get(), &bytes),
              "aclsparseXcsrsort_bufferSizeExt");
        frame::DeviceArray<unsigned char> buffer(bytes);
        Check(aclsparseXcsrsort(handle.get(), c.m, c.n, nnz, descr, dPtr.get(), dCol.get(), dPerm.get(), buffer.get()),
              "aclsparseXcsrsort");
        stream.sync();
        ok = bytes > 0 && dPtr.download() == c.rowPtr && dCol.download() == goldCol && dPerm.download() == goldPerm;
    }
    (void)aclsparseDestroyMatDescr(descr);
    return ok;
}

// The csrsort cases read as CSC matrices (test/cscsort/arch35/cscsort_test.cpp:245-530 builds the same shapes with
// rows and columns exchanged): c.m columns, row indices below c.n.  The buffer is aligned to 128 bytes, as the
// reference demands of its callers; one that is not must be refused.
bool CscsortCase(const frame::Stream &stream, const frame::Handle &handle, const SortCase &c)
{
    const int nnz = static_cast<int>(c.colInd.size());
    const int rows = c.n, cols = c.m;
    aclsparseMatDescr_t descr = nullptr;
    Check(aclsparseCreateMatDescr(&descr), "aclsparseCreateMatDescr");
    aclsparseSetMatIndexBase(descr, static_cast<aclsparseIndexBase_t>(c.base));
    bool ok = false;
    if (nnz == 0) {
        size_t bytes = 42;
        Check(aclsparseXcscsort_bufferSizeExt(handle.get(), rows, cols, 0, c.rowPtr.data(), nullptr, &bytes),
              "aclsparseXcscsort_bufferSizeExt");
        Check(aclsparseXcscsort(handle.get(), rows, cols, 0, descr, c.rowPtr.data(), nullptr, nullptr, nullptr),
              "aclsparseXcscsort");
        ok = bytes == 0;
    } else {
        std::vector<int32_t> perm = c.perm;
        if (perm.empty()) {
            perm.resize(static_cast<size_t>(nnz));
            for (int i = 0; i < nnz; ++i) {
                perm[i] = 3 * i + 1;  // NonIdentityP
            }
        }
        std::vector<int32_t> goldRow = c.colInd, goldPerm = perm;
        oracle_cscsort(c.rowPtr.data(), cols, c.base, goldRow.data(), goldPerm.data());
        frame::DeviceArray<int32_t> dPtr(c.rowPtr), dRow(c.colInd), dPerm(perm);
        size_t bytes = 0;
        Check(aclsparseXcscsort_bufferSizeExt(handle.get(), rows, cols, nnz, dPtr.get(), dRow.get(), &bytes),
              "aclsparseXcscsort_bufferSizeExt");
        frame::DeviceArray<unsigned char> buffer(bytes + 256);
        auto *aligned = reinterpret_cast<unsigned char *>((reinterpret_cast<uintptr_t>(buffer.get()) + 127) / 128 * 128);
        const bool refused = aclsparseXcscsort(handle.get(), rows, cols, nnz, descr, dPtr.get(), dRow.get(), dPerm.get(),
                                               aligned + 8) == ACL_SPARSE_STATUS_INVALID_VALUE;
        Check(aclsparseXcscsort(handle.get(), rows, cols, nnz, descr, dPtr.get(), dRow.get(), dPerm.get(), aligned),
              "aclsparseXcscsort");
        stream.sync();
        ok = refused && bytes > 0 && dPtr.download() == c.rowPtr && dRow.download() == goldRow &&
             dPerm.download() == goldPerm;
    }
    (void)aclsparseDestroyMatDescr(descr);
    return ok;
}

struct CooCase {
    std::string name;
    int m, n;
    bool byRow;
    std::vector<int32_t> rows, cols;
};

// Inputs of test/coosort/arch35/coosort_test.cpp: the hand-written cases (:233-262), random matrices of 12 .. 388
// entries (:266-352), the sizes of its multi-core cases (:563-680), and indices outside the matrix, which the
// sort compares as signed integers (coosort_golden.h:29).
std::vector<CooCase> CooCases()
{
    std::vector<CooCase> c;
    for (const bool byRow : {true, false}) {
        c.push_back({byRow ? "ByRowBasic" : "ByColumnBasic", 4, 4, byRow, {2, 0, 3, 0, 1, 2}, {1, 3, 2, 1, 0, 3}});
        c.push_back({byRow ? "ByRowStableDuplicateKey" : "ByColumnStableDuplicateKey", 3, 5, byRow, {0, 0, 0, 1, 1, 2},
                     {4, 1, 3, 2, 0, 9}});
        c.push_back({byRow ? "ByRowNnzZero" : "ByColumnNnzZero", 4, 4, byRow, {}, {}});
        int seed = 42;
        for (const int nnz : {12, 49, 103, 215, 388, 4097, 70000, 300001}) {
            std::mt19937 rng(static_cast<uint32_t>(seed++));
            const int m = nnz < 1000 ? 64 : 5000, n = nnz < 1000 ? 48 : 3000;
            CooCase k{(byRow ? "ByRowRandom_" : "ByColumnRandom_") + std::to_string(nnz), m, n, byRow, {}, {}};
            for (int i = 0; i < nnz; ++i) {
                k.rows.push_back(static_cast<int32_t>(rng() % static_cast<uint32_t>(m)));
                k.cols.push_back(static_cast<int32_t>(rng() % static_cast<uint32_t>(n)));
            }
            c.push_back(k);
        }
        CooCase k{byRow ? "ByRowSignedIndices" : "ByColumnSignedIndices", 10, 10, byRow, {}, {}};
        std::mt19937 rng(7);
        for (int i = 0; i < 20000; ++i) {
            k.rows.push_back(static_cast<int32_t>(rng()));  // the whole int32 range
            k.cols.push_back(static_cast<int32_t>(rng() % 9U) - 4);
        }
        c.push_back(k);
    }
    return c;
}

// RunSortAndVerify of the reference (coosort_test.cpp:141-228): P preset to 0 .. nnz-1, bufferSizeExt must ask for
// a buffer when there is something to sort, rows, columns and P compared exactly.
bool CoosortCase(const frame::Stream &stream, const frame::Handle &handle, const CooCase &c)
{
    const int nnz = static_cast<int>(c.rows.size());
    size_t bytes = 42;
    if (nnz == 0) {
        Check(aclsparseXcoosort_bufferSizeExt(handle.get(), c.m, c.n, 0, nullptr, nullptr, &bytes),
              "aclsparseXcoosort_bufferSizeExt");
        Check((c.byRow ? aclsparseXcoosortByRow : aclsparseXcoosortByColumn)(handle.get(), c.m, c.n, 0, nullptr, nullptr,
                                                                             nullptr, nullptr), "aclsparseXcoosort");
        return bytes == 0;
    }
    std::vector<int32_t> perm(static_cast<size_t>(nnz));
    for (int i = 0; i < nnz; ++i) {
        perm[i] = i;
    }
    std::vector<int32_t> goldRows = c.rows, goldCols = c.cols, goldPerm = perm;
    oracle_coosort(nnz, c.byRow ? 1 : 0, goldRows.data(), goldCols.data(), goldPerm.data());
    frame::DeviceArray<int32_t> dRows(c.rows), dCols(c.cols), dPerm(perm);
    Check(aclsparseXcoosort_bufferSizeExt(handle.get(), c.m, c.n, nnz, dRows.get(), dCols.get(), &bytes),
          "aclsparseXcoosort_bufferSizeExt");
    frame::DeviceArray<unsigned char> buffer(bytes);
    Check((c.byRow ? aclsparseXcoosortByRow : aclsparseXcoosortByColumn)(handle.get(), c.m, c.n, nnz, dRows.get(),
                                                                         dCols.get(), dPerm.get(), buffer.get()),
          "aclsparseXcoosort");
    stream.sync();
    return bytes >= static_cast<size_t>(nnz) * 12 && dRows.download() == goldRows && dCols.download() == goldCols &&
           dPerm.download() == goldPerm;
}

bool Coo2CsrCase(const frame::Stream &stream, const frame::Handle &handle, const Row &r)
{
    const int32_t base = static_cast<int32_t>(I(r, "idx_base"));
    const int64_t m = I(r, "m");
    std::vector<int32_t> rows;
    if (r.at("pattern") == "allsame") {
        const int64_t nnz = std::max<int64_t>(static_cast<int64_t>(m * I(r, "n") * (1.0 - D(r, "sparsity"))), 1);
        rows.assign(static_cast<size_t>(nnz), base);
    } else {
        const frame::CsrHost a = Matrix(r, "n");
        rows.resize(static_cast<size_t>(a.nnz()));
        oracle_csr2coo(a.rowptr.data(), a.rows, a.nnz(), 0, rows.data());
        for (auto &v : rows) {
            v += base;
        }
    }
    std::vector<int32_t> gold(static_cast<size_t>(m) + 1);
    oracle_coo2csr(rows.data(), static_cast<int64_t>(rows.size()), m, base, gold.data());
    frame::DeviceArray<int32_t> dRows(rows), dPtr(static_cast<size_t>(m) + 1);
    Check(aclsparseXcoo2csr(handle.get(), dRows.get(), static_cast<int>(rows.size()), static_cast<int>(m), dPtr.get(),
                            static_cast<aclsparseIndexBase_t>(base)), "aclsparseXcoo2csr");
    stream.sync();
    return dPtr.download() == gold;
}

bool Csr2CooCase(const frame::Stream &stream, const frame::Handle &handle, const Row &r)
{
    const int32_t base = static_cast<int32_t>(I(r, "idx_base"));
    Row rr = r;
    if (rr.at("pattern") == "csc") {
        rr["pattern"] = "random";  // any offsets array will do: the operation only sees row offsets
    }
    frame::CsrHost a = Matrix(rr, "n");
    for (auto &v : a.rowptr) {
        v += base;
    }
    std::vector<int32_t> gold(static_cast<size_t>(a.nnz()));
    oracle_csr2coo(a.rowptr.data(), a.rows, a.nnz(), base, gold.data());
    frame::DeviceArray<int32_t> dPtr(a.rowptr), dRows(static_cast<size_t>(a.nnz()));
    Check(aclsparseXcsr2coo(handle.get(), dPtr.get(), a.nnz(), a.rows, dRows.get(), static_cast<aclsparseIndexBase_t>(base)),
          "aclsparseXcsr2coo");
    stream.sync();
    return dRows.download() == gold;
}

bool Csr2CscCase(const frame::Stream &stream, const frame::Handle &handle, const Row &r)
{
    const int32_t base = static_cast<int32_t>(I(r, "idx_base"));
    frame::CsrHost a = Matrix(r, "n");
    const int64_t m = a.rows, n = a.cols, nnz = a.nnz();
    for (auto &v : a.rowptr) v += base;
    for (auto &v : a.colind) v += base;
    const std::string vt = r.at("val_type");
    const aclDataType type = vt == "INT8" ? ACL_INT8 : vt == "FP16" ? ACL_FLOAT16 : vt == "BF16" ? ACL_BF16 : ACL_FLOAT;
    const int32_t width = vt == "INT8" ? 1 : vt == "FP32" ? 4 : 2;
    // values of the requested width: the low bytes of the fp32 patterns (moved as raw bytes anyway)
    std::vector<unsigned char> val(static_cast<size_t>(nnz) * width);
    for (int64_t i = 0; i < nnz; ++i) {
        std::memcpy(val.data() + i * width, reinterpret_cast<const unsigned char *>(&a.val[i]) + (4 - width), width);
    }
    const bool numeric = r.at("copy_values") == "NUMERIC";
    std::vector<int32_t> goldPtr(static_cast<size_t>(n) + 1), goldRow(static_cast<size_t>(nnz));
    std::vector<unsigned char> goldVal(val.size(), 0x55);
    oracle_csr2csc(m, n, nnz, base, a.rowptr.data(), a.colind.data(), val.data(), numeric ? width : 0, goldPtr.data(),
                   goldRow.data(), goldVal.data());
    frame::DeviceArray<int32_t> dPtr(a.rowptr), dCol(a.colind), oPtr(static_cast<size_t>(n) + 1), oRow(static_cast<size_t>(nnz));
    frame::DeviceArray<unsigned char> dVal(val), oVal(std::vector<unsigned char>(val.size(), 0x55));
    const aclsparseAction_t action = numeric ? ACL_SPARSE_ACTION_NUMERIC : ACL_SPARSE_ACTION_SYMBOLIC;
    size_t bytes = 0;
    Check(aclsparseCsr2cscEx2_bufferSize(handle.get(), static_cast<int>(m), static_cast<int>(n), static_cast<int>(nnz),
                                         dVal.get(), dPtr.get(), dCol.get(), oVal.get(), oPtr.get(), oRow.get(), type,
                                         action, static_cast<aclsparseIndexBase_t>(base), ACL_SPARSE_CSR2CSC_ALG_DEFAULT,
                                         &bytes), "aclsparseCsr2cscEx2_bufferSize");
    frame::DeviceArray<unsigned char> buffer(bytes > 0 ? bytes : 16);
    Check(aclsparseCsr2cscEx2(handle.get(), static_cast<int>(m), static_cast<int>(n), static_cast<int>(nnz), dVal.get(),
                              dPtr.get(), dCol.get(), oVal.get(), oPtr.get(), oRow.get(), type, action,
                              static_cast<aclsparseIndexBase_t>(base), ACL_SPARSE_CSR2CSC_ALG_DEFAULT, buffer.get()),
          "aclsparseCsr2cscEx2");
    stream.sync();
    return oPtr.download() == goldPtr && oRow.download() == goldRow && oVal.download() == goldVal;
}

}  // namespace

int main(int argc, char **argv)
{
    if (argc < 2) {
        std::fprintf(stderr, "usage: %s <directory with the csv case tables> [spmv_op|coo2csr|csr2coo|csr2csc|csrsort|cscsort|coosort ...]\n",
                     argv[0]);
        return 2;
    }
    const std::string dir = argv[1];
    std::vector<std::string> tables;
    for (int i = 2; i < argc; ++i) {
        tables.push_back(argv[i]);
    }
    if (tables.empty()) {
        tables = {"spmv_op", "coo2csr", "csr2coo", "csr2csc", "csrsort", "cscsort", "coosort"};
    }
    int failed = 0, total = 0;
    try {
        frame::Stream stream;
        frame::Handle handle(stream);
        for (const std::string &t : tables) {
            if (t == "coosort") {
                for (const CooCase &c : CooCases()) {
                    bool ok = false;
                    std::string error;
                    try {
                        ok = CoosortCase(stream, handle, c);
                    } catch (const std::exception &e) {
                        error = e.what();
                    }
                    ++total;
                    failed += ok ? 0 : 1;
                    std::printf("[%s] %-32s %s %s\n", t.c_str(), c.name.c_str(), ok ? "PASS" : "FAIL", error.c_str());
                    std::fflush(stdout);
                }
                continue;
            }
            if (t == "csrsort" || t == "cscsort") {
                for (const SortCase &c : SortCases()) {
                    bool ok = false;
                    std::string error;
                    try {
                        ok = t == "csrsort" ? CsrsortCase(stream, handle, c) : CscsortCase(stream, handle, c);
                    } catch (const std::exception &e) {
                        error = e.what();
                    }
                    ++total;
                    failed += ok ? 0 : 1;
                    std::printf("[%s] %-32s %s %s\n", t.c_str(), c.name.c_str(), ok ? "PASS" : "FAIL", error.c_str());
                    std::fflush(stdout);
                }
                continue;
            }
            const auto rows = frame::LoadCsv(dir + "/" + t + "_cases.csv");
            for (const Row &r : rows) {
                bool ok = false;
                std::string error;
                try {
                    ok = t == "spmv_op"   ? SpmvOpCase(stream, handle, r)
                         : t == "coo2csr" ? Coo2CsrCase(stream, handle, r)
                         : t == "csr2coo" ? Csr2CooCase(stream, handle, r)
                                          : Csr2CscCase(stream, handle, r);
                } catch (const std::exception &e) {
                    error = e.what();
                }
                ++total;
                failed += ok ? 0 : 1;
                std::printf("[%s] %-32s %s %s\n", t.c_str(), r.at("case_name").c_str(), ok ? "PASS" : "FAIL", error.c_str());
                std::fflush(stdout);
            }
        }
    } catch (const std::exception &e) {
        std::fprintf(stderr, "fatal: %s\n", e.what());
        return 2;
    }
    std::printf("%d cases, %d failed\n", total, failed);
    return failed == 0 ? 0 : 1;
}
