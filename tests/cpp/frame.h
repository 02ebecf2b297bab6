// Small C++ test frame over HIP for callers written against cann_ops_sparse.h:
// RAII owners for the stream, the aclsparse handle, device arrays and
// descriptors, a CSV case-table loader with typed case parameters, the
// verification rules (absolute, relative, MERE / MARE, exact, integer) and a
// seeded CSR generator.  It plays the role of the reference's test/frame
// (descriptor_manager.h, sparse_test.h, csv_loader.h:125-136, verify.h:28-196,
// types.h:18-60, fill.h) for the case tables kept under tests/golden/, without
// GoogleTest: a test program is a plain main() that prints one line per case.
// Test infrastructure only; links libops_sparse.so and (as the checker)
// oracle/liboracle.so.
#pragma once

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <fstream>
#include <map>
#include <random>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

#include "cann_ops_sparse.h"

// The CPU checker (oracle/oracle.c).
extern "C" {
void oracle_spmv_f64(int64_t rows, int64_t cols, const int32_t *rowptr, const int32_t *colind, const float *val,
                     const float *x, const float *y, float alpha, float beta, float *z);
void oracle_mere_mare(const float *out, const float *gold, int64_t n, double eps, double *result);
void oracle_coo2csr(const int32_t *rowInd, int64_t nnz, int64_t m, int32_t base, int32_t *rowPtr);
void oracle_csr2coo(const int32_t *rowPtr, int64_t m, int64_t nnz, int32_t base, int32_t *rowInd);
void oracle_csr2csc(int64_t m, int64_t n, int64_t nnz, int32_t base, const int32_t *rowPtr, const int32_t *colInd,
                    const void *val, int32_t valBytes, int32_t *colPtr, int32_t *rowInd, void *cscVal);
void oracle_csrsort(const int32_t *rowPtr, int64_t m, int32_t base, int32_t *colInd, int32_t *perm);
void oracle_cscsort(const int32_t *colPtr, int64_t n, int32_t base, int32_t *rowInd, int32_t *perm);
void oracle_coosort(int64_t nnz, int32_t byRow, int32_t *rows, int32_t *cols, int32_t *perm);
uint64_t oracle_fnv1a(const void *data, int64_t bytes);
}

namespace frame {

inline void Check(hipError_t e, const char *what)
{
    if (e != hipSuccess) {
        throw std::runtime_error(std::string(what) + ": " + hipGetErrorString(e));
    }
}
inline void Check(aclsparseStatus_t s, const char *what)
{
    if (s != ACL_SPARSE_STATUS_SUCCESS) {
        throw std::runtime_error(std::string(what) + ": aclsparse status " + std::to_string(static_cast<int>(s)));
    }
}

class Stream {
public:
    Stream() { Check(hipStreamCreate(&s_), "hipStreamCreate"); }
    ~Stream() { (void)hipStreamDestroy(s_); }
    Stream(const Stream &) = delete;
    Stream &operator=(const Stream &) = delete;
    hipStream_t get() const { return s_; }
    void sync() const { Check(hipStreamSynchronize(s_), "hipStreamSynchronize"); }

private:
    hipStream_t s_ = nullptr;
};

class Handle {
public:
    explicit Handle(const Stream &s)
    {
        Check(aclsparseCreate(&h_), "aclsparseCreate");
        Check(aclsparseSetStream(h_, s.get()), "aclsparseSetStream");
    }
    ~Handle() { (void)aclsparseDestroy(h_); }
    Handle(const Handle &) = delete;
    Handle &operator=(const Handle &) = delete;
    aclsparseHandle_t get() const { return h_; }

private:
    aclsparseHandle_t h_ = nullptr;
};

// Device array with upload / download; an empty array has a NULL pointer.
template <typename T>
class DeviceArray {
public:
    DeviceArray() = default;
    explicit DeviceArray(size_t n) { Allocate(n); }
    explicit DeviceArray(const std::vector<T> &host)
    {
        Allocate(host.size());
        if (n_ > 0) {
            Check(hipMemcpy(p_, host.data(), n_ * sizeof(T), hipMemcpyHostToDevice), "hipMemcpy H2D");
        }
    }
    ~DeviceArray() { (void)hipFree(p_); }
    DeviceArray(const DeviceArray &) = delete;
    DeviceArray &operator=(const DeviceArray &) = delete;
    DeviceArray(DeviceArray &&o) noexcept : p_(o.p_), n_(o.n_) { o.p_ = nullptr; o.n_ = 0; }
    T *get() const { return p_; }
    size_t size() const { return n_; }
    std::vector<T> download() const
    {
        std::vector<T> out(n_);
        if (n_ > 0) {
            Check(hipMemcpy(out.data(), p_, n_ * sizeof(T), hipMemcpyDeviceToHost), "hipMemcpy D2H");
        }
        return out;
    }

private:
    void Allocate(size_t n)
    {
        n_ = n;
        if (n_ > 0) {
            Check(hipMalloc(reinterpret_cast<void **>(&p_), n_ * sizeof(T)), "hipMalloc");
        }
    }
    T *p_ = nullptr;
    size_t n_ = 0;
};

// Owners of the API's descriptors, in the shape of the reference's SpMatManager / DnVecManager
// (test/frame/descriptor_manager.h:22-60, :190-): a static creator per format, get(), destroyed with the owner.
class SpMat {
public:
    SpMat() = default;
    static SpMat createCsr(int64_t rows, int64_t cols, int64_t nnz, void *rowOffsets, void *colIndices, void *values,
                           aclsparseIndexType_t rowOffsetType = ACL_SPARSE_INDEX_32I,
                           aclsparseIndexType_t colIdxType = ACL_SPARSE_INDEX_32I,
                           aclsparseIndexBase_t idxBase = ACL_SPARSE_INDEX_BASE_ZERO, aclDataType valueType = ACL_FLOAT)
    {
        SpMat m;
        Check(aclsparseCreateCsr(&m.d_, rows, cols, nnz, rowOffsets, colIndices, values, rowOffsetType, colIdxType,
                                 idxBase, valueType), "aclsparseCreateCsr");
        return m;
    }
    ~SpMat() { if (d_ != nullptr) { (void)aclsparseDestroySpMat(d_); } }
    SpMat(const SpMat &) = delete;
    SpMat &operator=(const SpMat &) = delete;
    SpMat(SpMat &&o) noexcept : d_(o.d_) { o.d_ = nullptr; }
    aclsparseSpMatDescr_t get() const { return d_; }

private:
    aclsparseSpMatDescr_t d_ = nullptr;
};

class DnVec {
public:
    DnVec() = default;
    static DnVec create(int64_t size, void *values, aclDataType valueType = ACL_FLOAT)
    {
        DnVec v;
        Check(aclsparseCreateDnVec(&v.d_, size, values, valueType), "aclsparseCreateDnVec");
        return v;
    }
    ~DnVec() { if (d_ != nullptr) { (void)aclsparseDestroyDnVec(d_); } }
    DnVec(const DnVec &) = delete;
    DnVec &operator=(const DnVec &) = delete;
    DnVec(DnVec &&o) noexcept : d_(o.d_) { o.d_ = nullptr; }
    aclsparseDnVecDescr_t get() const { return d_; }

private:
    aclsparseDnVecDescr_t d_ = nullptr;
};

// ------------------------------------------------------------ verification
// The reference's rules (test/frame/types.h:18-60, verify.h:28-196), one function instead of a strategy
// class per rule.  Elements are read with a stride, as there.  Defaults are the reference's: MERE / MARE with
// threshold 2^-13 and multiplier 10, relative errors over |golden| + 2^-14.
enum class PrecisionMode { ABS, REL, COMBINED, MERE_MARE, EXACT, INTEGER };

struct VerifyConfig {
    PrecisionMode mode = PrecisionMode::MERE_MARE;
    double absTol = 1e-5;
    double relTol = 1e-5;
    double mereThreshold = 0.0001220703125;  // 2^-13
    double mareMultiplier = 10.0;
    double epsilonForRel = 1e-7;
    VerifyConfig &SetMode(PrecisionMode m) { mode = m; return *this; }
    VerifyConfig &SetAbsTol(double t) { absTol = t; return *this; }
    VerifyConfig &SetRelTol(double t) { relTol = t; return *this; }
    VerifyConfig &SetMERE(double t) { mereThreshold = t; return *this; }
    VerifyConfig &SetMARE(double m) { mareMultiplier = m; return *this; }
    VerifyConfig &SetEpsilon(double e) { epsilonForRel = e; return *this; }
};

struct VerifyReport {
    bool pass = false;
    size_t count = 0, skipped = 0, failures = 0, mismatches = 0, outliers = 0;
    double mere = 0.0, mare = 0.0;  // mean and maximum relative error over the elements that were compared
};

inline VerifyReport Verify(const float *output, const float *golden, size_t count, int64_t stride,
                           const VerifyConfig &cfg = VerifyConfig())
{
    constexpr double kMereEpsilon = 0.00006103515625;  // 2^-14 (verify.h:153)
    VerifyReport r;
    r.count = count;
    double sumRel = 0.0;
    const double outlierLimit = cfg.mareMultiplier * cfg.mereThreshold;
    for (size_t i = 0; i < count; ++i) {
        const float o = output[static_cast<int64_t>(i) * stride], g = golden[static_cast<int64_t>(i) * stride];
        const bool oBad = std::isnan(o) || std::isinf(o), gBad = std::isnan(g) || std::isinf(g);
        if (cfg.mode == PrecisionMode::INTEGER) {  // never skips (verify.h:178)
            r.failures += static_cast<int64_t>(o) != static_cast<int64_t>(g) ? 1 : 0;
            continue;
        }
        // equal values and a NaN on both sides are not looked at (verify.h:51-55); MERE / MARE also passes over
        // an infinity or NaN on both sides (:117-123)
        if (o == g || (std::isnan(o) && std::isnan(g)) || (cfg.mode == PrecisionMode::MERE_MARE && oBad && gBad)) {
            r.skipped++;
            continue;
        }
        const double d = std::abs(o - g);  // in float, like the reference
        switch (cfg.mode) {
            case PrecisionMode::ABS:
                r.failures += d > cfg.absTol ? 1 : 0;
                break;
            case PrecisionMode::REL: {
                const double rel = d / (std::abs(g) + cfg.epsilonForRel);
                r.mare = rel > r.mare ? rel : r.mare;
                break;
            }
            case PrecisionMode::COMBINED:
                r.failures += d > cfg.absTol + cfg.relTol * std::abs(g) ? 1 : 0;
                break;
            case PrecisionMode::MERE_MARE: {
                if (oBad || gBad) {
                    r.mismatches++;
                    break;
                }
                const double rel = d / (std::abs(g) + kMereEpsilon);
                sumRel += rel;
                r.mare = rel > r.mare ? rel : r.mare;
                r.outliers += rel > outlierLimit ? 1 : 0;
                break;
            }
            case PrecisionMode::EXACT:
                r.failures++;  // anything that was not skipped as equal
                break;
            default:
                break;
        }
    }
    switch (cfg.mode) {
        case PrecisionMode::REL:
            r.pass = r.mare < cfg.relTol;
            break;
        case PrecisionMode::MERE_MARE: {
            const size_t effective = count - r.skipped - r.mismatches;
            r.mere = effective > 0 ? sumRel / static_cast<double>(effective) : 0.0;
            r.pass = r.mismatches == 0 && r.mere < cfg.mereThreshold && r.mare < outlierLimit;
            break;
        }
        default:
            r.pass = r.failures == 0;
            break;
    }
    return r;
}

struct CsrHost {
    int64_t rows = 0, cols = 0;
    std::vector<int32_t> rowptr{0}, colind;
    std::vector<float> val;
    int64_t nnz() const { return static_cast<int64_t>(colind.size()); }
};

// The reference's seeded matrices (SparseFillGenerator(seed) with setSparsity / setEmptyRowProb / setValueRange, then
// generateCsr(rows, cols, nnzHint): reference test/frame/fill.h:55-111), bit for bit — the same engine, the same
// distributions of the same standard library, drawn from in the same order: per row one uniform float against the
// empty-row probability (only when that is above 0), the row length (Binomial(cols, 1 - sparsity), or nnzHint /
// rows when a hint is given, capped at cols), then columns until that many distinct ones are found or four times
// as many were drawn, and, after sorting, one value per entry.  frame_selftest holds it against fingerprints of
// the reference's own output (tests/golden/fill_generator.json).
inline CsrHost FillCsr(int64_t rows, int64_t cols, double sparsity, double emptyRowProb, uint32_t seed, float lo, float hi,
                       int64_t nnzHint = -1)
{
    CsrHost a;
    a.rows = rows;
    a.cols = cols;
    a.rowptr.assign(static_cast<size_t>(rows > 0 ? rows : 0) + 1, 0);
    if (rows <= 0 || cols <= 0) {
        return a;
    }
    std::mt19937 engine(seed);
    std::uniform_real_distribution<float> chance(0.0f, 1.0f), value(lo, hi);
    // (one object for all rows: it keeps a spare normal deviate between draws)
    std::binomial_distribution<int> length(static_cast<int>(cols), 1.0 - std::min(std::max(sparsity, 0.0), 1.0));
    const float skip = static_cast<float>(std::min(std::max(emptyRowProb, 0.0), 1.0));
    std::vector<int> seenInRow(static_cast<size_t>(cols), -1);
    std::vector<int32_t> picked;
    for (int64_t r = 0; r < rows; ++r) {
        a.rowptr[r] = static_cast<int32_t>(a.colind.size());
        if (skip > 0.0f && chance(engine) < skip) {
            continue;
        }
        int want = nnzHint > 0 ? static_cast<int>(nnzHint / std::max<int64_t>(rows, 1)) : length(engine);
        want = std::min(want, static_cast<int>(cols));
        picked.clear();
        for (int draws = 0; want > 0 && static_cast<int>(picked.size()) < want && draws < 4 * want; ++draws) {
            const int32_t c = std::uniform_int_distribution<int32_t>(0, static_cast<int32_t>(cols) - 1)(engine);
            if (seenInRow[c] != static_cast<int>(r)) {
                seenInRow[c] = static_cast<int>(r);
                picked.push_back(c);
            }
        }
        std::sort(picked.begin(), picked.end());
        for (int32_t c : picked) {
            a.colind.push_back(c);
            a.val.push_back(value(engine));
        }
    }
    a.rowptr[rows] = static_cast<int32_t>(a.colind.size());
    return a;
}

inline CsrHost DiagCsr(int64_t m)
{
    CsrHost a;
    a.rows = a.cols = m;
    a.rowptr.resize(static_cast<size_t>(m) + 1);
    for (int64_t i = 0; i <= m; ++i) {
        a.rowptr[i] = static_cast<int32_t>(i);
    }
    for (int64_t i = 0; i < m; ++i) {
        a.colind.push_back(static_cast<int32_t>(i));
        a.val.push_back(1.0f);
    }
    return a;
}

// makeDenseFloat(n, lo, hi, seed) of the reference (test/frame/fill.h:199-203): n uniform floats from a fresh engine.
inline std::vector<float> FillDense(int64_t n, float lo, float hi, uint32_t seed)
{
    std::mt19937 engine(seed);
    std::uniform_real_distribution<float> value(lo, hi);
    std::vector<float> v(static_cast<size_t>(n > 0 ? n : 0));
    for (auto &e : v) {
        e = value(engine);
    }
    return v;
}

// Rows of a CSV case table keyed by the header names; lines starting with '#' are comments.
using CsvRow = std::map<std::string, std::string>;
inline std::vector<CsvRow> LoadCsv(const std::string &path);

// A test's parameter type fills itself from a row and names its case (the reference's SparseTestParamBase,
// csv_loader.h:112-122); GetCasesFromCsv<ParamType> turns a table into a vector of them (:125-136).
class CaseParamBase {
public:
    virtual ~CaseParamBase() = default;
    virtual void fillCustom(const CsvRow &row) = 0;
    virtual std::string caseId() const = 0;
};

template <typename ParamType>
std::vector<ParamType> GetCasesFromCsv(const std::string &csvPath)
{
    std::vector<ParamType> cases;
    for (const CsvRow &row : LoadCsv(csvPath)) {
        ParamType p;
        p.fillCustom(row);
        cases.push_back(std::move(p));
    }
    return cases;
}

inline std::vector<CsvRow> LoadCsv(const std::string &path)
{
    std::ifstream in(path);
    if (!in) {
        throw std::runtime_error("cannot open " + path);
    }
    auto split = [](const std::string &line) {
        std::vector<std::string> out;
        std::stringstream ss(line);
        std::string cell;
        while (std::getline(ss, cell, ',')) {
            while (!cell.empty() && (cell.back() == '\r' || cell.back() == ' ')) {
                cell.pop_back();
            }
            out.push_back(cell);
        }
        return out;
    };
    std::string line;
    std::vector<std::string> header;
    std::vector<std::map<std::string, std::string>> rows;
    while (std::getline(in, line)) {
        if (line.empty() || line[0] == '#') {
            continue;
        }
        const auto cells = split(line);
        if (header.empty()) {
            header = cells;
            continue;
        }
        std::map<std::string, std::string> row;
        for (size_t i = 0; i < header.size() && i < cells.size(); ++i) {
            row[header[i]] = cells[i];
        }
        rows.push_back(row);
    }
    return rows;
}

}  // namespace frame
