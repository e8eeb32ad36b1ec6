// Per-kernel event timing aid of libenatten.so (enatten_profile_* in enatten.h).
//
// Host code only.  While the aid is off a launch reads one atomic flag and nothing
// else.  While it is on, every n-th launch of a kernel is bracketed by two HIP events,
// and a third is recorded straight after the second: the time between those two, with
// nothing launched in between, is what a bracket itself adds on a busy queue (about
// 5 us on MI355X; the sum of the raw brackets of a step otherwise exceeds the step's
// own wall time), and is accumulated beside the raw figure so a reader can subtract
// it.  The ProfScope owns its events until all are recorded; only then are they handed
// to the shared table, under a mutex, so launches from several threads (the caller's
// and the autograd engine's) can be timed at once.  Switching the aid off, switching
// it on again and reading a kernel's figures all wait for the recorded events, add
// their durations to plain numbers and destroy them: no HIP object outlives
// enatten_profile_enable(0).  The table is allocated once and never destroyed, so
// nothing of it runs during static destruction at process exit.
#include <atomic>
#include <mutex>
#include <vector>

#include "na2d_common.h"

namespace enatten {
namespace {

struct ProfRec { hipEvent_t e0, e1, e2; };
struct ProfSlot {
    std::vector<ProfRec> recs;  // recorded, not yet read back
    int calls = 0;              // launches seen since the aid was switched on
    int timed = 0;              // launches read back
    double total_ms = 0.0;      // raw brackets
    double empty_ms = 0.0;      // the empty brackets recorded after them
    const char *name = "";      // string literal of the last launch
};
struct ProfState {
    std::mutex mu;
    ProfSlot slot[ENATTEN_KERNEL_COUNT];
    int period = 1;
    unsigned generation = 0;    // bumped whenever the table is reset
};
constexpr int kProfMax = 8192;  // timed launches kept per kernel between two resets

std::atomic<int> g_on{0};
ProfState &state() {
    static ProfState *p = new ProfState;
    return *p;
}

// Wait for the recorded events of a slot, add their durations, destroy them.
// Caller holds the mutex.  Returns false if an event could not be read.
bool harvest(ProfSlot &ps) {
    bool ok = true;
    for (const ProfRec &r : ps.recs) {
        float ms = 0.f, empty = 0.f;
        if (hipEventSynchronize(r.e2) == hipSuccess &&
            hipEventElapsedTime(&ms, r.e0, r.e1) == hipSuccess &&
            hipEventElapsedTime(&empty, r.e1, r.e2) == hipSuccess) {
            ps.total_ms += ms;
            ps.empty_ms += empty;
            ps.timed++;
        } else {
            ok = false;
        }
        (void)hipEventDestroy(r.e0);
        (void)hipEventDestroy(r.e1);
        (void)hipEventDestroy(r.e2);
    }
    ps.recs.clear();
    return ok;
}

}  // namespace

ProfScope::ProfScope(int kernel_slot, const char *kernel_name, hipStream_t stream)
    : slot(kernel_slot), st(stream), e0(nullptr), e1(nullptr), e2(nullptr), generation(0), armed(false) {
    if (!g_on.load(std::memory_order_acquire)) return;
    ProfState &S = state();
    {
        std::lock_guard<std::mutex> lock(S.mu);
        if (!g_on.load(std::memory_order_relaxed)) return;
        ProfSlot &ps = S.slot[slot];
        ps.name = kernel_name;
        if (ps.calls++ % S.period != 0) return;
        if (ps.timed + (int)ps.recs.size() >= kProfMax) return;
        generation = S.generation;
    }
    if (hipEventCreate(&e0) != hipSuccess) return;
    if (hipEventCreate(&e1) != hipSuccess || hipEventCreate(&e2) != hipSuccess ||
        hipEventRecord(e0, st) != hipSuccess) {
        (void)hipEventDestroy(e0);
        if (e1) (void)hipEventDestroy(e1);
        if (e2) (void)hipEventDestroy(e2);
        return;
    }
    armed = true;
}

ProfScope::~ProfScope() {
    if (!armed) return;
    const bool recorded = hipEventRecord(e1, st) == hipSuccess && hipEventRecord(e2, st) == hipSuccess;
    ProfState &S = state();
    {
        std::lock_guard<std::mutex> lock(S.mu);
        // a reset since the constructor means nobody will read this record
        if (recorded && generation == S.generation && g_on.load(std::memory_order_relaxed)) {
            S.slot[slot].recs.push_back(ProfRec{e0, e1, e2});
            return;
        }
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    (void)hipEventDestroy(e2);
}

}  // namespace enatten

using namespace enatten;

extern "C" {
#pragma GCC visibility push(default)

int enatten_profile_enable(int on) {
    ProfState &S = state();
    std::lock_guard<std::mutex> lock(S.mu);
    const int prev = g_on.load(std::memory_order_relaxed) ? S.period : 0;
    if (on > 0) {
        for (ProfSlot &ps : S.slot) {
            harvest(ps);
            ps.calls = 0;
            ps.timed = 0;
            ps.total_ms = 0.0;
            ps.empty_ms = 0.0;
        }
        S.period = on;
        S.generation++;
        g_on.store(1, std::memory_order_release);
    } else {
        g_on.store(0, std::memory_order_release);
        for (ProfSlot &ps : S.slot) harvest(ps);
        S.generation++;
    }
    return prev;
}

int enatten_profile_read(int kernel, int *launches, double *total_ms) {
    if (kernel < 0 || kernel >= ENATTEN_KERNEL_COUNT || !launches || !total_ms) {
        set_error("enatten_profile_read: bad arguments");
        return ENATTEN_EINVAL;
    }
    ProfState &S = state();
    std::lock_guard<std::mutex> lock(S.mu);
    ProfSlot &ps = S.slot[kernel];
    const bool ok = harvest(ps);
    *launches = ps.timed;
    *total_ms = ps.total_ms;
    if (!ok) {
        set_error("enatten_profile_read: an event could not be read");
        return ENATTEN_ELAUNCH;
    }
    return ENATTEN_OK;
}

int enatten_profile_read_overhead(int kernel, double *total_empty_ms) {
    if (kernel < 0 || kernel >= ENATTEN_KERNEL_COUNT || !total_empty_ms) {
        set_error("enatten_profile_read_overhead: bad arguments");
        return ENATTEN_EINVAL;
    }
    ProfState &S = state();
    std::lock_guard<std::mutex> lock(S.mu);
    ProfSlot &ps = S.slot[kernel];
    const bool ok = harvest(ps);
    *total_empty_ms = ps.empty_ms;
    if (!ok) {
        set_error("enatten_profile_read_overhead: an event could not be read");
        return ENATTEN_ELAUNCH;
    }
    return ENATTEN_OK;
}

const char *enatten_profile_kernel_name(int kernel) {
    if (kernel < 0 || kernel >= ENATTEN_KERNEL_COUNT) return "";
    ProfState &S = state();
    std::lock_guard<std::mutex> lock(S.mu);
    return S.slot[kernel].name;
}

#pragma GCC visibility pop
}  // extern "C"
