// Placed memory: two physical allocations that a timing probe has shown to lie in different regions of HBM, mapped
// side by side in one virtual range, ONE pair per GPU and process.  Contexts take leases from it: rank arenas (half
// the ranks in either allocation) and row blocks (n rows back to back that straddle the junction).
//
// Why: on MI355X the 288 GiB behave as three regions of 96 GiB, and streams written at the same time disturb each
// other less when they lie in different regions (the write-heavy schedules here gain 15 to 25 %).  Where an
// allocation lands physically is the driver's business, so the pair is found by measurement (see find_pair in
// placed_pool.cpp).  The reference has one buffer per GPU and no such choice (allreduce_8GPU.cu:977-990).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace sar {

// What a search needs of the calling context: the probe kernel runs on its stream and times itself on the device's
// wall clock.
struct ProbeEnv { int device; hipStream_t stream; int wall_khz; };

// What the last search for the pair on a GPU saw (reported through sar_stats).
struct SearchRecord {
    int candidates = 0;              // allocations probed against the first one
    float same_ms = 0.f;             // the probe's time for two windows that share a region (the yardstick)
    float pair_ms = 0.f;             // ... and for the pair that was kept (the slower of its two probes)
    uint64_t search_bytes = 0;       // most memory held at a time while looking, the pair included
    uint64_t pool_bytes = 0;         // the pair as it is now: both allocations together (0 = none)
    int users = 0;                   // contexts attached to it
};

// ---- the decisions of the search, as functions of probe times alone (checked against recorded times without a device)
// Yardstick: the probe's time for the two ends of the first allocation (or the median of three neighbouring pairs of
// its windows, should that be faster).  False when the ends probe so much faster than the median neighbouring pair
// that a region boundary must run through the allocation.
bool spread_yardstick(const float neighbours_ms[3], float ends_ms, float* yardstick_ms);
// A single probe against the first allocation says "another region": clearly below the yardstick.
bool spread_is_elsewhere(float yardstick_ms, float probe_ms);
// All candidates' probe times at once: the index of the candidate to take (the fastest) when it is clearly below the
// yardstick and the times fall into two populations -- sorted, they jump by 4 % and more somewhere below the limit --,
// or when every candidate is clearly below the yardstick; else -1: nobody is clearly elsewhere, or the times run on
// without a gap.
int spread_pick(float yardstick_ms, const float* probe_ms, int n);

// ---- the pool ------------------------------------------------------------------------------------------------
// `owner` identifies the context; every call takes the pool's lock.  Reasons are SAR_SPREAD_* codes.
void pool_attach(int device, const void* owner);
// Gives back the owner's leases; when nobody is attached any more the pair is unmapped and released.
void pool_detach(int device, const void* owner);
// lo_bytes for ranks [0, ceil(n/2)), hi_bytes for the rest; *lo and *hi are 2 MiB-aligned device addresses in the two
// allocations.  SAR_SPREAD_FOUND, or why not (nothing is held for the owner then).
int pool_lease_arena(const ProbeEnv& env, const void* owner, uint64_t lo_bytes, uint64_t hi_bytes, char** lo, char** hi);
// One address range of lo_bytes + hi_bytes whose first lo_bytes end where the second allocation begins.
int pool_lease_rows(const ProbeEnv& env, const void* owner, uint64_t lo_bytes, uint64_t hi_bytes, char** base);
// Nothing on the device may still be using the memory (the caller drains the device first).
void pool_release_arena(int device, const void* owner);
void pool_release_rows(int device, const void* owner);
// Unmaps and releases the pair if nobody holds a lease (it may be what keeps a plain allocation from fitting).
bool pool_trim(int device);
// Whether [p, p + 1) lies in a lease the owner holds.
bool pool_leased_by(int device, const void* owner, const char* p);
SearchRecord pool_record(int device);

}  // namespace sar
