// Host-side code of the library (encoder, 2:4 split and packing, residual lists, planner, synthetic
// inputs) driven on edge-case inputs in a build with AddressSanitizer and UndefinedBehaviorSanitizer.
// Every result is also checked against a plain restatement here, so the run fails on a wrong answer
// as well as on a bad access.  Exit status 0 = clean.
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "a24_format.h"
#include "launch_plan.h"
#include "tiled_csl_format.h"

namespace {

int failures = 0;
#define CHECK(cond)                                                         \
    do {                                                                    \
        if (!(cond)) {                                                      \
            std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);   \
            failures++;                                                     \
        }                                                                   \
    } while (0)

// Tiled-CSL back to a dense matrix: word = fp16 | (row * 64 + (col ^ ((row % 8) << 3))) << 16
std::vector<uint16_t> decode(const uint32_t* items, const int* offsets, int M, int K)
{
    std::vector<uint16_t> A(static_cast<size_t>(M) * K, 0);
    const int tr = M / tcsl::kTileRows, tc = K / tcsl::kTileCols;
    for (int t = 0; t < tr * tc; t++)
        for (long w = 4L * offsets[t]; w < 4L * offsets[t + 1]; w++) {
            const uint32_t word = items[w];
            const uint16_t v = static_cast<uint16_t>(word & 0xffff);
            if (v == 0)
                continue;  // padding
            const int pos = word >> 16, row = pos / 64, col = (pos % 64) ^ ((row % 8) << 3);
            uint16_t& cell = A[static_cast<size_t>((t / tc) * tcsl::kTileRows + row) * K + (t % tc) * tcsl::kTileCols + col];
            CHECK(cell == 0);  // no position twice
            cell = v;
        }
    return A;
}

void encoder_case(int M, int K, double sparsity, int skew, uint64_t seed, int mode)
{
    std::vector<uint16_t> A(static_cast<size_t>(M) * K);
    if (mode == 0)
        tcsl::synth_weights(A.data(), M, K, sparsity, skew, seed);
    else if (mode == 1)
        tcsl::synth_harness_weights(A.data(), M, K, sparsity, skew, seed);
    else if (mode == 2)
        std::fill(A.begin(), A.end(), 0);
    else if (mode == 3)
        std::fill(A.begin(), A.end(), 0x3c00);  // fully dense
    else {
        std::fill(A.begin(), A.end(), 0);
        A[static_cast<size_t>(M - 1) * K + (K - 1)] = 0xbc00;  // one value, in the last corner
    }
    for (int reorder = 0; reorder < 2; reorder++) {
        uint32_t* items = nullptr;
        int* offsets = nullptr;
        const int n = reorder ? tcsl::encode(A.data(), M, K, &items, &offsets)
                              : tcsl::encode_noreorder(A.data(), M, K, &items, &offsets);
        const int tiles = (M / tcsl::kTileRows) * (K / tcsl::kTileCols);
        CHECK(n >= 0 && items && offsets);
        if (n < 0 || !items || !offsets)
            continue;
        CHECK(offsets[0] == 0 && offsets[tiles] == offsets[tiles + 1]);
        for (int t = 0; t < tiles; t++)
            CHECK(offsets[t] <= offsets[t + 1]);
        std::vector<uint16_t> back = decode(items, offsets, M, K);
        // a stored zero (positive or negative) is not a non-zero of the format
        for (size_t i = 0; i < A.size(); i++)
            if (back[i] != ((A[i] & 0x7fff) ? A[i] : 0)) {
                CHECK(!"round trip");
                break;
            }
        std::free(items);
        std::free(offsets);
    }
}

void rejects()
{
    uint32_t* items = nullptr;
    int* offsets = nullptr;
    std::vector<uint16_t> A(128 * 64, 0);
    CHECK(tcsl::encode(A.data(), 100, 64, &items, &offsets) < 0 && !items && !offsets);
    CHECK(tcsl::encode(A.data(), 128, 60, &items, &offsets) < 0 && !items && !offsets);
    CHECK(tcsl::encode(nullptr, 128, 64, &items, &offsets) < 0);
    CHECK(tcsl::encode(A.data(), 0, 64, &items, &offsets) < 0);
    CHECK(tcsl::encode_file("/nonexistent/dense.bin", 128, 64, "/tmp/a", "/tmp/b", "/tmp/c") < 0);
}

void files(const std::string& dir)
{
    const int M = 256, K = 192;
    std::vector<uint16_t> A(static_cast<size_t>(M) * K);
    tcsl::synth_weights(A.data(), M, K, 0.8, 0, 5);
    const std::string dense = dir + "/dense.bin", nz = dir + "/nz.bin", off = dir + "/off.bin", sizes = dir + "/sizes.bin";
    FILE* f = std::fopen(dense.c_str(), "wb");
    CHECK(f != nullptr);
    if (!f)
        return;
    CHECK(std::fwrite(A.data(), 2, A.size(), f) == A.size());
    std::fclose(f);
    CHECK(tcsl::encode_file(dense.c_str(), M, K, nz.c_str(), off.c_str(), sizes.c_str()) >= 0);
    uint32_t* items = nullptr;
    int* offsets = nullptr;
    const int n = tcsl::encode(A.data(), M, K, &items, &offsets);
    CHECK(n >= 0);
    std::vector<int> from_file(n);
    f = std::fopen(off.c_str(), "rb");
    CHECK(f && std::fread(from_file.data(), 4, n, f) == static_cast<size_t>(n));
    if (f)
        std::fclose(f);
    CHECK(std::memcmp(from_file.data(), offsets, 4 * static_cast<size_t>(n)) == 0);
    std::free(items);
    std::free(offsets);
}

void split_case(int M, int K, double sparsity, int skew, uint64_t seed)
{
    std::vector<uint16_t> A(static_cast<size_t>(M) * K), A1(A.size()), A2(A.size());
    tcsl::synth_weights(A.data(), M, K, sparsity, skew, seed);
    if (!A.empty()) {
        A[0] = 0x7c00;  // infinity, NaN and a negative zero among the values
        A[1] = 0x7e00;
        A[2] = 0x8000;
    }
    a24::decompose(A.data(), A1.data(), A2.data(), static_cast<long>(A.size()));
    for (size_t g = 0; g < A.size(); g += 4) {
        int kept = 0;
        for (int j = 0; j < 4; j++) {
            kept += (A1[g + j] & 0x7fff) != 0;
            CHECK((A1[g + j] & 0x7fff) == 0 || (A2[g + j] & 0x7fff) == 0);  // a value goes to one part
            CHECK(((A1[g + j] & 0x7fff) ? A1[g + j] : A2[g + j]) == ((A[g + j] & 0x7fff) ? A[g + j] : A2[g + j]));
        }
        CHECK(kept <= 2);
    }
    std::vector<uint8_t> packed(static_cast<size_t>(a24::bytes(M, K)));
    CHECK(a24::pack(A1.data(), M, K, packed.data()) == 0);
    CHECK(a24::pack(A.data(), M, K, packed.data()) == a24::kErrNotTwoOfFour || sparsity >= 0.99);
    uint32_t* words = nullptr;
    int* offsets = nullptr;
    int longest = -1;
    const int n = a24::pack_residual(A2.data(), M, K, &words, &offsets, &longest);
    const int lists = (M / a24::kRows) * (K / a24::kUnitCols);
    CHECK(n == lists + 1 && words && offsets && longest >= 0);
    if (n == lists + 1 && words && offsets) {
        long total = 0, nz = 0;
        int seen_longest = 0;
        for (int l = 0; l < lists; l++) {
            const int len = offsets[l + 1] - offsets[l];
            CHECK(len >= 0);
            seen_longest = len > seen_longest ? len : seen_longest;
            total += len;
        }
        for (size_t i = 0; i < A2.size(); i++)
            nz += (A2[i] & 0x7fff) != 0;
        CHECK(total == offsets[lists] && total >= nz && seen_longest == longest);
        for (int i = 0; i < a24::kListPadWords; i++)
            CHECK(words[offsets[lists] + i] == 0);  // the padding a wave may read past the last list
    }
    std::free(words);
    std::free(offsets);
}

void planner()
{
    const int Ns[] = {8, 16, 32, 64};
    const int Ms[] = {128, 256, 1024, 7168, 9216, 21504, 28672, 36864, 49152, 65536, 1 << 20};
    const int Ks[] = {64, 128, 1024, 7168, 9216, 12288, 28672, 49152, 1 << 18};
    for (int N : Ns)
        for (int M : Ms)
            for (int K : Ks) {
                tcsl::LaunchPlan p{};
                const int s = tcsl::suggest_split_k(M, N, K, &p);
                const long nkb = K / 64;
                CHECK(s >= 1 && s <= 32 && s <= nkb);
                CHECK(s == 1 || ((nkb + s - 1) / s) * (s - 1) < nkb);  // no empty batch
                tcsl::LaunchPlan q = p;
                CHECK(tcsl::complete_plan(N, K, s, false, q) && q.lds_bytes <= 160 * 1024);
                for (int split : {1, 2, 3, 7, 32, 4096}) {
                    double cost = 0;
                    const tcsl::LaunchPlan r = tcsl::plan_launch(M, N, K, split, split & 1, &cost);
                    tcsl::LaunchPlan c = r;
                    CHECK(tcsl::complete_plan(N, K, split, split & 1, c));
                    CHECK(cost > 0 && cost < 1e9);
                }
                for (double bytes : {800.0, 3300.0, 6558.0, 9800.0, 32768.0})
                    CHECK(tcsl::suggest_split_k(M, N, K, nullptr, bytes) >= 1);
            }
    tcsl::LaunchPlan bad{0, 9, 0, 0};
    CHECK(!tcsl::complete_plan(16, 1024, 1, false, bad));
    bad = {0, 4, 1, 0};
    CHECK(!tcsl::complete_plan(64, 1024, 1, false, bad));
    bad = {1, 4, 1, 0};
    CHECK(!tcsl::complete_plan(16, 1024, 1, false, bad));
    bad = {0, 4, 0, 0};
    CHECK(!tcsl::complete_plan(24, 1024, 1, false, bad));
}

}  // namespace

int main(int argc, char** argv)
{
    const std::string dir = argc > 1 ? argv[1] : "/tmp";
    const int shapes[][2] = {{128, 64}, {128, 320}, {384, 64}, {256, 192}, {512, 1024}};
    for (const auto& s : shapes) {
        for (int mode = 0; mode < 5; mode++)
            encoder_case(s[0], s[1], 0.8, 0, 11 + mode, mode);
        encoder_case(s[0], s[1], 0.3, 1, 3, 0);
        encoder_case(s[0], s[1], 0.97, 1, 4, 1);
    }
    rejects();
    files(dir);
    const int split_shapes[][2] = {{128, 128}, {256, 384}, {128, 1280}, {640, 256}};
    for (const auto& s : split_shapes)
        for (double sp : {0.0, 0.3, 0.5, 0.8, 0.99})
            split_case(s[0], s[1], sp, sp > 0.2 && sp < 0.9, 17);
    planner();
    std::printf("%s, %d failed checks\n", failures ? "FAILED" : "clean", failures);
    return failures ? 1 : 0;
}
