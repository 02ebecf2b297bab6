// CPU-only checks of tests/cpp/frame.h: the verification rules against the C checker's MERE / MARE and against
// values worked out by hand, and the typed CSV loader on one of the committed tables.  No GPU call is made.
//
//   frame_selftest <directory with the csv case tables>
#include <cstdio>
#include <fstream>
#include <sstream>

#include "frame.h"

namespace {

int g_failed = 0;
void Expect(bool ok, const char *what)
{
    std::printf("%-70s %s\n", what, ok ? "ok" : "FAILED");
    g_failed += ok ? 0 : 1;
}

struct SpmvOpParam : frame::CaseParamBase {
    std::string name;
    int64_t m = 0, k = 0;
    double alpha = 0, beta = 0;
    void fillCustom(const frame::CsvRow &row) override
    {
        name = row.at("case_name");
        m = std::stoll(row.at("m"));
        k = std::stoll(row.at("k"));
        alpha = std::stod(row.at("alpha"));
        beta = std::stod(row.at("beta"));
    }
    std::string caseId() const override { return name; }
};

}  // namespace

int main(int argc, char **argv)
{
    using frame::PrecisionMode;
    using frame::Verify;
    using frame::VerifyConfig;
    // MERE / MARE by hand: relative errors over |g| + 2^-14 of (1.001 vs 1), (2 vs 2: skipped), (-3.003 vs -3)
    {
        const float out[3] = {1.001f, 2.0f, -3.003f}, gold[3] = {1.0f, 2.0f, -3.0f};
        const double e0 = std::abs(out[0] - gold[0]) / (1.0 + 0.00006103515625);
        const double e2 = std::abs(out[2] - gold[2]) / (3.0 + 0.00006103515625);
        const auto r = Verify(out, gold, 3, 1, VerifyConfig().SetMERE(0.01));
        Expect(r.skipped == 1 && std::abs(r.mere - (e0 + e2) / 2) < 1e-15 && std::abs(r.mare - std::max(e0, e2)) < 1e-15 &&
                   r.pass, "MERE / MARE of three elements, one equal");
        Expect(!Verify(out, gold, 3, 1, VerifyConfig()).pass, "the same against the default threshold 2^-13 fails");
        Expect(Verify(out, gold, 2, 2, VerifyConfig().SetMERE(0.01)).count == 2, "stride 2 reads elements 0 and 2");
    }
    // against the C checker on a seeded vector, including NaN / infinity on one and on both sides
    {
        std::vector<float> gold = frame::FillDense(5000, -4.0f, 4.0f, 7), out = gold;
        std::mt19937 rng(8);
        for (auto &v : out) {
            v *= 1.0f + 1e-4f * static_cast<float>(static_cast<int>(rng() % 2001) - 1000) / 1000.0f;
        }
        out[10] = gold[10] = NAN;
        out[11] = gold[11] = INFINITY;
        double res[4];
        oracle_mere_mare(out.data(), gold.data(), 5000, 0.00006103515625, res);
        const auto r = Verify(out.data(), gold.data(), 5000, 1);
        Expect(std::abs(r.mere - res[0]) <= 1e-12 * res[0] && r.mare == res[1] && r.mismatches == 0 && res[2] == 0,
               "MERE / MARE equal to oracle_mere_mare on 5000 seeded elements");
        out[12] = NAN;  // abnormal on one side only: a mismatch, and the case fails
        oracle_mere_mare(out.data(), gold.data(), 5000, 0.00006103515625, res);
        const auto bad = Verify(out.data(), gold.data(), 5000, 1);
        Expect(bad.mismatches == 1 && res[2] == 1 && !bad.pass, "a NaN on one side only is a mismatch");
    }
    // the other rules
    {
        const float out[4] = {1.0f, 2.00001f, 3.5f, -7.0f}, gold[4] = {1.0f, 2.0f, 3.0f, -7.0f};
        Expect(Verify(out, gold, 4, 1, VerifyConfig().SetMode(PrecisionMode::ABS).SetAbsTol(1e-4)).failures == 1,
               "ABS: one element off by 0.5");
        Expect(!Verify(out, gold, 4, 1, VerifyConfig().SetMode(PrecisionMode::EXACT)).pass &&
                   Verify(out, gold, 4, 1, VerifyConfig().SetMode(PrecisionMode::EXACT)).failures == 2,
               "EXACT: two elements differ");
        Expect(Verify(out, gold, 4, 1, VerifyConfig().SetMode(PrecisionMode::INTEGER)).pass,
               "INTEGER: equal after truncation");
        const auto rel = Verify(out, gold, 4, 1, VerifyConfig().SetMode(PrecisionMode::REL).SetRelTol(0.2));
        Expect(rel.pass && std::abs(rel.mare - 0.5 / (3.0 + 1e-7)) < 1e-12, "REL: maximum 0.5 / 3");
    }
    if (argc > 1) {
        const auto cases = frame::GetCasesFromCsv<SpmvOpParam>(std::string(argv[1]) + "/spmv_op_cases.csv");
        Expect(cases.size() == 70 && !cases[0].caseId().empty() && cases[0].m >= 0, "GetCasesFromCsv: 70 typed rows");
    }
    if (argc > 1) {
        // The generator against fingerprints of the reference's own output (FNV-1a of the three arrays, written by
        // tests/golden/make_fill_fixture.py): every object of the "csr" and "dense" lists of fill_generator.json.
        std::ifstream in(std::string(argv[1]) + "/fill_generator.json");
        std::stringstream all;
        all << in.rdbuf();
        const std::string text = all.str();
        // (the file is flat enough for this: a field is "name": value up to the next comma, brace or bracket)
        auto field = [&](size_t from, size_t to, const char *name) {
            const std::string key = std::string("\"") + name + "\":";
            const size_t at = text.find(key, from);
            if (at == std::string::npos || at >= to) {
                return std::string();
            }
            size_t b = at + key.size();
            while (b < to && (text[b] == ' ' || text[b] == '"')) {
                ++b;
            }
            size_t e = b;
            while (e < to && text[e] != ',' && text[e] != '"' && text[e] != '}' && text[e] != '\n') {
                ++e;
            }
            return text.substr(b, e - b);
        };
        auto hex = [](uint64_t v) {
            char buf[17];
            std::snprintf(buf, sizeof(buf), "%016llx", static_cast<unsigned long long>(v));
            return std::string(buf);
        };
        const size_t csrAt = text.find("\"csr\":"), denseAt = text.find("\"dense\":");
        int csrCases = 0, csrOk = 0, denseCases = 0, denseOk = 0;
        for (size_t at = text.find('{', csrAt); at != std::string::npos && at < denseAt; at = text.find('{', at + 1)) {
            const size_t end = text.find('}', at);
            const frame::CsrHost a = frame::FillCsr(
                std::stoll(field(at, end, "rows")), std::stoll(field(at, end, "cols")), std::stod(field(at, end, "sparsity")),
                std::stod(field(at, end, "empty_row_prob")), static_cast<uint32_t>(std::stoul(field(at, end, "seed"))),
                std::stof(field(at, end, "lo")), std::stof(field(at, end, "hi")), std::stoll(field(at, end, "nnz_hint")));
            ++csrCases;
            csrOk += (a.nnz() == std::stoll(field(at, end, "nnz")) &&
                      hex(oracle_fnv1a(a.rowptr.data(), 4 * static_cast<int64_t>(a.rowptr.size()))) == field(at, end, "rowptr_fnv1a") &&
                      hex(oracle_fnv1a(a.colind.data(), 4 * a.nnz())) == field(at, end, "colind_fnv1a") &&
                      hex(oracle_fnv1a(a.val.data(), 4 * a.nnz())) == field(at, end, "values_fnv1a"))
                         ? 1 : 0;
        }
        for (size_t at = text.find('{', denseAt); at != std::string::npos; at = text.find('{', at + 1)) {
            const size_t end = text.find('}', at);
            const std::vector<float> v = frame::FillDense(std::stoll(field(at, end, "n")), std::stof(field(at, end, "lo")),
                                                          std::stof(field(at, end, "hi")),
                                                          static_cast<uint32_t>(std::stoul(field(at, end, "seed"))));
            ++denseCases;
            denseOk += hex(oracle_fnv1a(v.data(), 4 * static_cast<int64_t>(v.size()))) == field(at, end, "fnv1a") ? 1 : 0;
        }
        Expect(csrCases >= 8 && csrOk == csrCases, "FillCsr: the reference generator's matrices, bit for bit (hint and binomial)");
        Expect(denseCases >= 2 && denseOk == denseCases, "FillDense: the reference generator's vectors, bit for bit");
    }
    std::printf("%d failed\n", g_failed);
    return g_failed == 0 ? 0 : 1;
}
