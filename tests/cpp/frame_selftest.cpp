// CPU-only checks of tests/cpp/frame.h: the verification rules against the C checker's MERE / MARE and against
// values worked out by hand, and the typed CSV loader on one of the committed tables.  No GPU call is made.
//
//   frame_selftest <directory with the csv case tables>
#include <cstdio>

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
        std::vector<float> gold = frame::RandomVector(5000, -4.0f, 4.0f, 7), out = gold;
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
    std::printf("%d failed\n", g_failed);
    return g_failed == 0 ? 0 : 1;
}
