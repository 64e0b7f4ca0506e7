// Host test of the coarse-bin arithmetic the kernels share (mako_amd/csrc/log_bins.h): the bins of a frame tile the
// units below its maximum, and the counts of a slice's bins move into the frame of a higher maximum exactly.
#include <cstdint>
#include <cstdio>
#include <random>

#include "../../mako_amd/csrc/log_bins.h"

using namespace mako;

static int failures = 0;
#define CHECK(cond, ...)                                                                                             \
    do {                                                                                                             \
        if (!(cond)) {                                                                                               \
            if (failures < 20) {                                                                                     \
                std::printf("FAIL %s:%d: ", __FILE__, __LINE__);                                                     \
                std::printf(__VA_ARGS__);                                                                            \
                std::printf("\n");                                                                                   \
            }                                                                                                        \
            ++failures;                                                                                              \
        }                                                                                                            \
    } while (0)

static const int32_t kUnitsCovered = (int32_t)(kLogFine + ((kLogBins - 1u - kLogFine) << kLogCoarseShift));

static void check_frame(int32_t k_top)
{
    // every unit from the maximum's down to well below the bins: one bin each, never decreasing on the way down
    uint32_t prev = 0;
    int32_t first_uncounted = 0;
    bool seen_uncounted = false;
    for (int32_t k = k_top; k > k_top - kUnitsCovered - 40; --k) {
        const uint32_t b = log_bin_in_frame(k, k_top);
        {
            // the counting form: the bin itself, or a slot from kLogBins - 1 to the end of the spare ones
            const uint32_t spare_end = kLogBins + (uint32_t)(k & 63);
            const uint32_t s = log_slot_in_frame(k, k_top, spare_end);
            CHECK(b == kLogNotCounted ? (s >= kLogBins - 1u && s <= spare_end) : s == b, "top %d unit %d: slot %u, bin %u", k_top, k, s, b);
        }
        if (b == kLogNotCounted) {
            if (!seen_uncounted)
                first_uncounted = k;
            seen_uncounted = true;
            continue;
        }
        CHECK(!seen_uncounted, "top %d: unit %d counted below uncounted unit %d", k_top, k, first_uncounted);
        CHECK(b < kLogBins - 1u, "top %d unit %d: bin %u", k_top, k, b);
        CHECK(b >= prev && b <= prev + 1u, "top %d unit %d: bin %u after %u", k_top, k, b, prev);
        CHECK(b < kLogFine ? (uint32_t)(k_top - k) == b : (uint32_t)(k_top - k) >= kLogFine, "top %d unit %d: bin %u", k_top, k, b);
        prev = b;
    }
    CHECK(seen_uncounted && prev == kLogBins - 2u, "top %d: last bin %u", k_top, prev);
    CHECK(k_top - first_uncounted > kUnitsCovered - (1 << kLogCoarseShift) - 1, "top %d: covers only %d units", k_top, k_top - first_uncounted);
    float middle_before = -1.0f;
    for (uint32_t b = 0; b < kLogBins - 1u; ++b) {
        // a bin's representative unit is in it; everything from its upper edge on lies in earlier bins, the unit below
        // the edge in the bin itself; its middle lies inside it
        const int32_t u = log_bin_unit(b, k_top);
        CHECK(log_bin_in_frame(u, k_top) == b, "top %d bin %u: unit %d is in bin %u", k_top, b, u, log_bin_in_frame(u, k_top));
        if (b >= 1) {
            const int32_t e = log_bin_upper_edge(b, k_top);
            CHECK(log_bin_in_frame(e, k_top) == b - 1u && log_bin_in_frame(e - 1, k_top) == b, "top %d bin %u: edge %d", k_top, b, e);
        }
        const float mid = log_bin_middle(b, k_top);
        CHECK(mid > middle_before, "top %d bin %u: middle %g after %g", k_top, b, mid, middle_before);
        // (distances count from the lower edge of the maximum's unit: unit k spans [k_top - k - 1, k_top - k) + 1)
        const int32_t k_mid = k_top - (int32_t)(mid + 1.0f);
        CHECK(log_bin_in_frame(k_mid, k_top) == b || log_bin_in_frame(k_mid + 1, k_top) == b, "top %d bin %u: middle %g", k_top, b, mid);
        middle_before = mid;
    }
}

static void check_merge(int32_t k_row, int32_t k_slice, std::mt19937& rng)
{
    // every unit the slice counted: its bin there, moved through the bin's representative unit, is the unit's own bin
    // in the row's frame (or both are outside the row's bins)
    std::uniform_int_distribution<int32_t> below(0, kUnitsCovered + 50);
    for (int i = 0; i < 4000; ++i) {
        const int32_t k = k_slice - (i < 600 ? i : below(rng));
        const uint32_t sb = log_bin_in_frame(k, k_slice);
        if (sb == kLogNotCounted)
            continue;
        const uint32_t direct = log_bin_in_frame(k, k_row);
        const uint32_t moved = log_bin_in_frame(log_bin_unit(sb, k_slice), k_row);
        CHECK(direct == moved, "row top %d slice top %d unit %d: slice bin %u -> row bin %u, its own %u", k_row, k_slice, k, sb, moved, direct);
    }
    // the short form of the move, for every bin of the slice's frame
    for (uint32_t b = 0; b < kLogBins - 1u; ++b) {
        const uint32_t composed = log_bin_in_frame(log_bin_unit(b, k_slice), k_row);
        const uint32_t moved = log_bin_moved(b, k_slice, k_row);
        CHECK(composed == moved, "row top %d slice top %d bin %u: moved to %u, composition says %u", k_row, k_slice, b, moved, composed);
    }
}

int main()
{
    std::mt19937 rng(12345);
    std::uniform_int_distribution<int32_t> tops(-2000000, 2000000);
    const int32_t fixed[] = {0, 1, -1, 15, 16, 17, 511, 512, 513, -511, -512, -513, 8191, -8192, 1 << 30, -(1 << 30)};
    for (int32_t t : fixed)
        check_frame(t);
    for (int i = 0; i < 200; ++i)
        check_frame(tops(rng));
    std::uniform_int_distribution<int32_t> gaps(0, 9000);
    for (int i = 0; i < 3000; ++i) {
        const int32_t k_row = i < 16 ? fixed[i] : tops(rng);
        const int32_t gap = i % 5 == 0 ? i % 40 : gaps(rng); // (slices' maxima are usually close to the row's)
        check_merge(k_row, k_row - gap, rng);
    }
    std::printf("log_bins_test: %d failures\n", failures);
    return failures != 0;
}
