/*
 * Per-launch kernel timing with HIP events (see launch.h).  Not thread-safe:
 * one profile at a time, opened and closed by the thread that launches.
 */
#include "blt_hip.h"
#include "launch.h"

#include <cstring>
#include <string>
#include <vector>

namespace {

struct Booking {
    const char *tag;
    hipEvent_t start, stop;
};

bool g_open = false;
std::vector<Booking> g_bookings;

} // namespace

bool blt_profile_is_open() { return g_open; }

void blt_profile_book(const char *tag, hipEvent_t *start, hipEvent_t *stop) {
    Booking b;
    b.tag = tag;
    HIP_CHECK(hipEventCreate(&b.start));
    HIP_CHECK(hipEventCreate(&b.stop));
    g_bookings.push_back(b);
    *start = b.start;
    *stop = b.stop;
}

extern "C" void blt_hip_profile_begin(void) {
    BLT_REQUIRE(!g_open, "blt_hip_profile_begin: a profile is already open");
    g_bookings.clear();
    g_open = true;
}

extern "C" size_t blt_hip_profile_end_list(float *ms_out, size_t capacity) {
    BLT_REQUIRE(g_open, "blt_hip_profile_end_list: no profile is open");
    g_open = false;
    HIP_CHECK(hipDeviceSynchronize());
    size_t at = 0;
    for (const Booking &b : g_bookings) {
        float ms = 0.f;
        HIP_CHECK(hipEventElapsedTime(&ms, b.start, b.stop));
        HIP_CHECK(hipEventDestroy(b.start));
        HIP_CHECK(hipEventDestroy(b.stop));
        if (ms_out && at < capacity) ms_out[at] = ms;
        at++;
    }
    g_bookings.clear();
    return at;
}

extern "C" size_t blt_hip_profile_end(blt_hip_kernel_time *out, size_t capacity) {
    BLT_REQUIRE(g_open, "blt_hip_profile_end: no profile is open");
    g_open = false;
    HIP_CHECK(hipDeviceSynchronize());
    std::vector<blt_hip_kernel_time> rows;
    for (const Booking &b : g_bookings) {
        float ms = 0.f;
        HIP_CHECK(hipEventElapsedTime(&ms, b.start, b.stop));
        HIP_CHECK(hipEventDestroy(b.start));
        HIP_CHECK(hipEventDestroy(b.stop));
        blt_hip_kernel_time *row = nullptr;
        for (blt_hip_kernel_time &r : rows)
            if (std::strcmp(r.name, b.tag) == 0) row = &r;
        if (!row) {
            blt_hip_kernel_time fresh;
            std::memset(&fresh, 0, sizeof(fresh));
            std::strncpy(fresh.name, b.tag, sizeof(fresh.name) - 1);
            fresh.min_ms = 1e30;
            rows.push_back(fresh);
            row = &rows.back();
        }
        row->launches += 1;
        row->total_ms += ms;
        if (ms < row->min_ms) row->min_ms = ms;
        if (ms > row->max_ms) row->max_ms = ms;
    }
    g_bookings.clear();
    const size_t n = rows.size() < capacity ? rows.size() : capacity;
    if (out && n) std::memcpy(out, rows.data(), n * sizeof(blt_hip_kernel_time));
    return rows.size();
}
