// Runs the reference's CSV case tables (tests/golden/*.csv) against
// libops_sparse.so from C++, the way a caller of the reference would: through
// cann_ops_sparse.h only.  One line per case; exit status 0 iff all passed.
//
//   run_case_tables <directory with the csv files> [table ...]
//
// Tables: spmv_op, coo2csr, csr2coo, csr2csc (default: all).  Mirrors
// test/spmv_op/arch35/spmv_op_test.cpp:73-142, test/coo2csr/arch35/coo2csr_test.cpp,
// test/csr2coo/arch35/csr2coo_test.cpp and test/csr2csc_ex2/arch35/csr2csc_ex2_test.cpp of the
// reference, with the frame of tests/cpp/frame.h and the CPU oracle as golden.
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
    return frame::RandomCsr(m, n, D(r, "sparsity"), D(r, "empty_row_prob"), static_cast<uint32_t>(I(r, "seed")), -5.0f,
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
    const std::vector<float> x = frame::RandomVector(k, -3.0f, 3.0f, seed + 1);
    const std::vector<float> y = frame::RandomVector(m, -3.0f, 3.0f, seed + 2);
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

    aclsparseSpMatDescr_t matA = nullptr;
    aclsparseDnVecDescr_t vx = nullptr, vy = nullptr, vz = nullptr;
    Check(aclsparseCreateCsr(&matA, m, k, nnz, rowPtr, dCol.get(), dVal.get(),
                             i64 ? ACL_SPARSE_INDEX_64I : ACL_SPARSE_INDEX_32I, ACL_SPARSE_INDEX_32I,
                             ACL_SPARSE_INDEX_BASE_ZERO, ACL_FLOAT), "aclsparseCreateCsr");
    Check(aclsparseCreateDnVec(&vx, k, dX.get(), ACL_FLOAT), "aclsparseCreateDnVec x");
    Check(aclsparseCreateDnVec(&vy, m, dY.get(), ACL_FLOAT), "aclsparseCreateDnVec y");
    if (!alias) {
        Check(aclsparseCreateDnVec(&vz, m, dZ.get(), ACL_FLOAT), "aclsparseCreateDnVec z");
    }
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
    (void)aclsparseDestroyDnVec(vx);
    (void)aclsparseDestroyDnVec(vy);
    if (vz != nullptr) {
        (void)aclsparseDestroyDnVec(vz);
    }
    (void)aclsparseDestroySpMat(matA);

    // |d| <= 1e-5 |gold| per element, and the table's own MERE / MARE limits
    for (int64_t i = 0; i < m; ++i) {
        const double g = gold[i], d = std::fabs(static_cast<double>(got[i]) - g);
        if (!(d <= 1e-5 * std::fmax(std::fabs(g), 1e-30))) {
            std::printf("    element %lld: got %.9g, golden %.9g\n", static_cast<long long>(i), got[i], gold[i]);
            return false;
        }
    }
    double res[4] = {0, 0, 0, 0};
    if (m > 0) {
        oracle_mere_mare(got.data(), gold.data(), m, std::ldexp(1.0, -14), res);
    }
    const double mere = D(r, "mere_threshold");
    return res[2] == 0 && res[0] < mere && res[1] < mere * D(r, "mare_multiplier");
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
        std::fprintf(stderr, "usage: %s <directory with the csv case tables> [spmv_op|coo2csr|csr2coo|csr2csc ...]\n", argv[0]);
        return 2;
    }
    const std::string dir = argv[1];
    std::vector<std::string> tables;
    for (int i = 2; i < argc; ++i) {
        tables.push_back(argv[i]);
    }
    if (tables.empty()) {
        tables = {"spmv_op", "coo2csr", "csr2coo", "csr2csc"};
    }
    int failed = 0, total = 0;
    try {
        frame::Stream stream;
        frame::Handle handle(stream);
        for (const std::string &t : tables) {
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
