// The pair of allocations in different regions of HBM and the leases contexts hold on it (see placed_pool.hpp).
#include "placed_pool.hpp"

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <mutex>
#include <vector>

#include "kernels.hpp"
#include "sar.h"

namespace sar {
namespace {

constexpr int kMaxDevices = 64;
constexpr uint64_t kGranule = 2ull << 20;              // leases start on 2 MiB boundaries (one large-page fragment)
constexpr uint64_t kHeadroom = 16ull << 30;            // memory left alone while looking for the pair
constexpr uint64_t kMinHalf = 4ull << 30;              // per allocation: eight probe windows, the least the yardstick needs
constexpr uint64_t kMaxHalf = 32ull << 30;
constexpr uint64_t kSearch = 96ull << 30;              // candidates held while looking, beyond the pair itself: one region
constexpr uint64_t kProbeStream = 128ull << 20;        // region probe: 8 streams of this size (beyond what the Infinity Cache absorbs)
// What separates the two populations of probe times.  Two windows that share a region take 181-228 us and scatter (which
// banks collide is a matter of the exact addresses); two windows in different regions take 158-167 us whatever the
// addresses.  The yardstick is the probe's time for the two ENDS of the first allocation (181-189 us in every search on
// record), or the median of its three neighbouring pairs should that be faster.  The fastest of all four was tried first
// and drifts: in an allocation pieced together from freed memory one neighbouring pair read 173-175 us, which pulled
// candidates elsewhere at 162-167 us above the limit.  Against the yardstick candidates elsewhere come in at 0.85-0.90
// on an empty device and 0.932 with 80 GiB of other allocations around, candidates of the same region at 0.98 and more.
// The candidates' own times must show the two populations as well: sorted, they jump by kGap and more somewhere below
// the limit (measured 9-18 % between the slowest candidate elsewhere and the fastest of the first allocation's region).
constexpr float kFaster = 0.95f, kGap = 0.04f;
constexpr float kStraddle = 0.86f;                     // the two ends of an allocation against its neighbouring windows: below this a
                                                       // boundary runs through it (measured 0.80 with a boundary, 0.90 to 0.93 without)

struct Lease { const void* owner; bool rows; uint64_t lo_off, lo_len, hi_off, hi_len; };

struct Pool {
    char* va = nullptr;                                // lower allocation at [va, va + half), upper at [va + half, va + 2 * half)
    uint64_t half = 0;
    hipMemGenericAllocationHandle_t lo_h{}, hi_h{};
    std::vector<const void*> users;
    std::vector<Lease> leases;
    SearchRecord rec;
};

std::mutex g_mutex[kMaxDevices];                      // one per GPU: a search on one does not hold up the others
Pool g_pool[kMaxDevices];

uint64_t up(uint64_t v, uint64_t a) { return (v + a - 1) / a * a; }

// A physical allocation mapped read-write at a virtual address of its own.
struct VmBlock { char* va = nullptr; uint64_t bytes = 0; hipMemGenericAllocationHandle_t h{}; };

hipMemAccessDesc vm_access(int device) {
    hipMemAccessDesc acc{};
    acc.location.type = hipMemLocationTypeDevice; acc.location.id = device; acc.flags = hipMemAccessFlagsProtReadWrite;
    return acc;
}

// False when any step fails; nothing is left behind then.
bool vm_block_create(int device, uint64_t bytes, VmBlock* out) {
    hipMemAllocationProp prop{};
    prop.type = hipMemAllocationTypePinned; prop.location.type = hipMemLocationTypeDevice; prop.location.id = device;
    VmBlock b; b.bytes = bytes;
    if (hipMemCreate(&b.h, bytes, &prop, 0) != hipSuccess) { (void)hipGetLastError(); return false; }
    void* va = nullptr;
    if (hipMemAddressReserve(&va, bytes, kGranule, nullptr, 0) != hipSuccess || !va) { (void)hipGetLastError(); (void)hipMemRelease(b.h); return false; }
    if (hipMemMap(va, bytes, 0, b.h, 0) != hipSuccess) { (void)hipGetLastError(); (void)hipMemAddressFree(va, bytes); (void)hipMemRelease(b.h); return false; }
    const hipMemAccessDesc acc = vm_access(device);
    if (hipMemSetAccess(va, bytes, &acc, 1) != hipSuccess) {
        (void)hipGetLastError(); (void)hipMemUnmap(va, bytes); (void)hipMemAddressFree(va, bytes); (void)hipMemRelease(b.h); return false;
    }
    b.va = (char*)va; *out = b;
    return true;
}

void complain(const char* what, hipError_t e) {
    (void)hipGetLastError();
    if (std::getenv("SAR_DEBUG") || std::getenv("SAR_DEBUG_SPREAD")) std::fprintf(stderr, "sar placed memory: %s: %s\n", what, hipGetErrorString(e));
}

// Takes the block out of the address space; the physical allocation goes as well unless the caller keeps its handle.
void vm_block_unmap(VmBlock& b, bool keep_handle) {
    hipError_t e;
    if (b.va) {
        if ((e = hipMemUnmap(b.va, b.bytes)) != hipSuccess) complain("hipMemUnmap", e);
        if ((e = hipMemAddressFree(b.va, b.bytes)) != hipSuccess) complain("hipMemAddressFree", e);
        b.va = nullptr;
    }
    if (!keep_handle && (e = hipMemRelease(b.h)) != hipSuccess) complain("hipMemRelease", e);
}

// Best of `reps` runs of the region probe on two windows of 4 * kProbeStream bytes, in milliseconds as the kernel
// timed itself on the device's wall clock; negative on error.  `stamps`: two 64-bit words of device memory.
float probe_ms(const ProbeEnv& env, unsigned long long* stamps, char* a, char* b, int reps) {
    float best = -1.f;
    for (int i = 0; i < reps; ++i) {
        unsigned long long h[2] = {~0ull, 0ull};
        if (hipMemcpyAsync(stamps, h, sizeof(h), hipMemcpyHostToDevice, env.stream) != hipSuccess ||
            launch_region_probe(env.stream, a, b, kProbeStream, stamps) != hipSuccess ||
            hipMemcpyAsync(h, stamps, sizeof(h), hipMemcpyDeviceToHost, env.stream) != hipSuccess ||
            hipStreamSynchronize(env.stream) != hipSuccess || h[1] <= h[0]) { (void)hipGetLastError(); return -1.f; }
        const float ms = (float)((double)(h[1] - h[0]) / (double)env.wall_khz);
        if (best < 0.f || ms < best) best = ms;
    }
    return best;
}

// Unmaps and releases the pair.  The caller has made sure nothing on the device uses it any more.
void free_pair(Pool& p) {
    if (!p.va) return;
    hipError_t e;
    // two mappings, each taken out with the address and size it was mapped with
    if ((e = hipMemUnmap(p.va, p.half)) != hipSuccess) complain("hipMemUnmap (lower allocation)", e);
    if ((e = hipMemUnmap(p.va + p.half, p.half)) != hipSuccess) complain("hipMemUnmap (upper allocation)", e);
    if ((e = hipMemRelease(p.lo_h)) != hipSuccess) complain("hipMemRelease (lower allocation)", e);
    if ((e = hipMemRelease(p.hi_h)) != hipSuccess) complain("hipMemRelease (upper allocation)", e);
    if ((e = hipMemAddressFree(p.va, 2 * p.half)) != hipSuccess) complain("hipMemAddressFree", e);
    p.va = nullptr; p.half = 0; p.rec.pool_bytes = 0;
}

// Two physical allocations of `half` bytes each that lie in different regions of HBM, mapped side by side into p.
//
// Candidates are allocated one after the other (nothing is assumed about the order in which the driver hands out
// memory) and each is timed against the first with a short probe: eight write streams of 128 MiB, four in either
// allocation.  The yardstick is the probe's own time for windows that do share a region, not a fixed figure: the
// two ends of the first allocation against each other (measured 181-189 us; candidates in the same region 183-228 us,
// elsewhere 158-167 us).  ALL candidates within the budget are probed -- enough of them to cross a region
// boundary from anywhere, one region's worth -- and the verdict is taken on the whole set (spread_pick): the times must
// fall into two populations with a clear gap, one of them clearly below the yardstick, and the candidate taken must
// confirm its time on other windows of both allocations.  Everything else is given back.  A wrong verdict would cost speed, not correctness; without a clear
// one the caller's ranks sit in an ordinary allocation.
int find_pair(const ProbeEnv& env, uint64_t half, Pool& p) {
    const uint64_t window = 4 * kProbeStream;
    p.rec.candidates = 0; p.rec.same_ms = p.rec.pair_ms = 0.f; p.rec.search_bytes = 0;
    if (half < 8 * window) return SAR_SPREAD_NO_PAIR;
    size_t free_b = 0, total_b = 0;
    if (hipMemGetInfo(&free_b, &total_b) != hipSuccess) { (void)hipGetLastError(); return SAR_SPREAD_NO_MEMORY; }
    if (free_b < 4 * half + kHeadroom) return SAR_SPREAD_NO_MEMORY;
    const uint64_t budget = std::min<uint64_t>((uint64_t)free_b - kHeadroom, kSearch + 2 * half);
    const bool debug = std::getenv("SAR_DEBUG_SPREAD") != nullptr;
    unsigned long long* stamps = nullptr;
    if (hipMalloc((void**)&stamps, 2 * sizeof(unsigned long long)) != hipSuccess) { (void)hipGetLastError(); return SAR_SPREAD_NO_MEMORY; }
    std::vector<VmBlock> live;
    std::vector<float> times;                        // times[i]: candidate live[first_cand + i] against the first allocation
    try { live.reserve((size_t)(budget / half) + 4); times.reserve(live.capacity()); }
    catch (const std::bad_alloc&) { (void)hipFree(stamps); return SAR_SPREAD_NO_MEMORY; }
    auto get = [&]() -> char* {
        VmBlock blk;
        if (live.size() == live.capacity() || !vm_block_create(env.device, half, &blk)) return nullptr;
        live.push_back(blk);
        return blk.va;
    };
    auto give_all_back = [&](const char* keep_a, const char* keep_b) {
        for (VmBlock& b : live) if (b.va != keep_a && b.va != keep_b) vm_block_unmap(b, false);
    };
    // The first allocation and the yardstick.  Should a region boundary run through the allocation, its two ends
    // probe like a pair in different regions while its neighbouring windows do not: it then stays held as a spacer
    // and the one behind it takes its place.
    char* lo = nullptr;
    float same = -1.f;
    uint64_t used = 0;
    for (int attempt = 0; attempt < 2 && used + half <= budget; ++attempt) {
        if (!(lo = get())) break;
        used += half;
        float adj[3];
        for (int k = 0; k < 3; ++k) adj[k] = probe_ms(env, stamps, lo + (uint64_t)(2 * k) * window, lo + (uint64_t)(2 * k + 1) * window, 3);
        const float ends = probe_ms(env, stamps, lo, lo + half - window, 3);
        if (adj[0] <= 0.f || adj[1] <= 0.f || adj[2] <= 0.f || ends <= 0.f) { same = -1.f; break; }
        if (debug) std::fprintf(stderr, "sar spread: first allocation %p, neighbouring windows %.1f %.1f %.1f us, ends %.1f us\n", (void*)lo, adj[0] * 1e3, adj[1] * 1e3, adj[2] * 1e3, ends * 1e3);
        const bool whole = spread_yardstick(adj, ends, &same);
        if (!whole && attempt == 0) { lo = nullptr; same = -1.f; continue; }
        break;
    }
    if (!lo || same <= 0.f) {
        give_all_back(nullptr, nullptr); (void)hipFree(stamps);
        p.rec.search_bytes = used;
        return lo ? SAR_SPREAD_NO_PAIR : SAR_SPREAD_NO_MEMORY;
    }
    const size_t first_cand = live.size();
    for (; used + half <= budget; used += half) {
        char* cand = get();
        if (!cand) break;
        const float t = probe_ms(env, stamps, lo, cand, 3);
        times.push_back(t);
        if (debug) std::fprintf(stderr, "sar spread: candidate %zu %p %.1f us (yardstick %.1f us)\n", times.size(), (void*)cand, t * 1e3, same * 1e3);
    }
    p.rec.candidates = (int)times.size();
    p.rec.same_ms = same;
    p.rec.search_bytes = used;
    // the verdict on the whole set; the candidate it names must confirm on other windows, else its time is
    // replaced by the slower one and the set is judged again
    char* hi = nullptr;
    for (int round = 0; round < 4 && !hi; ++round) {
        const int k = times.empty() ? -1 : spread_pick(same, times.data(), (int)times.size());
        if (k < 0) {
            if (debug) std::fprintf(stderr, "sar spread: no verdict on %zu candidates (nobody clearly below the yardstick, or no gap between those and the rest)\n", times.size());
            break;
        }
        char* cand = live[first_cand + (size_t)k].va;
        const float t2 = probe_ms(env, stamps, lo + half - window, cand + half - window, 3);
        if (debug) std::fprintf(stderr, "sar spread: candidate %d picked (%.1f us), other windows %.1f us\n", k + 1, times[(size_t)k] * 1e3, t2 * 1e3);
        if (spread_is_elsewhere(same, t2)) { hi = cand; p.rec.pair_ms = std::max(times[(size_t)k], t2); }
        else times[(size_t)k] = t2 > 0.f ? std::max(times[(size_t)k], t2) : -1.f;
    }
    (void)hipFree(stamps);
    if (!hi) { give_all_back(nullptr, nullptr); return SAR_SPREAD_NO_PAIR; }
    VmBlock blo, bhi;
    for (VmBlock& b : live) { if (b.va == lo) blo = b; else if (b.va == hi) bhi = b; }
    give_all_back(lo, hi);
    // the probes have completed (probe_ms waits for each); the pair moves into one range, lo first
    vm_block_unmap(blo, true); vm_block_unmap(bhi, true);
    void* va = nullptr;
    bool ok = hipMemAddressReserve(&va, 2 * half, kGranule, nullptr, 0) == hipSuccess && va;
    bool m0 = false, m1 = false;
    if (ok) ok = m0 = hipMemMap(va, half, 0, blo.h, 0) == hipSuccess;
    if (ok) ok = m1 = hipMemMap((char*)va + half, half, 0, bhi.h, 0) == hipSuccess;
    if (ok) { const hipMemAccessDesc acc = vm_access(env.device); ok = hipMemSetAccess(va, 2 * half, &acc, 1) == hipSuccess; }
    if (!ok) {
        (void)hipGetLastError();
        if (m0) (void)hipMemUnmap(va, half);
        if (m1) (void)hipMemUnmap((char*)va + half, half);
        if (va) (void)hipMemAddressFree(va, 2 * half);
        (void)hipMemRelease(blo.h); (void)hipMemRelease(bhi.h);
        return SAR_SPREAD_NO_MEMORY;
    }
    p.va = (char*)va; p.half = half; p.lo_h = blo.h; p.hi_h = bhi.h; p.rec.pool_bytes = 2 * half;
    return SAR_SPREAD_FOUND;
}

bool free_in(const Pool& p, bool upper, uint64_t off, uint64_t len) {
    for (const Lease& l : p.leases) {
        const uint64_t o = upper ? l.hi_off : l.lo_off, n = upper ? l.hi_len : l.lo_len;
        if (n && off < o + n && o < off + len) return false;
    }
    return true;
}

// The pair, large enough for `need` bytes per allocation: the one that is there, or a new one when nobody holds a
// lease on the old.
int ensure_pair(const ProbeEnv& env, Pool& p, uint64_t need) {
    if (need > kMaxHalf) return SAR_SPREAD_TOO_LARGE;
    if (p.va && p.half >= need) return SAR_SPREAD_FOUND;
    if (p.va && !p.leases.empty()) return SAR_SPREAD_POOL_BUSY;
    if (p.va) { (void)hipDeviceSynchronize(); free_pair(p); }
    uint64_t half = kMinHalf;
    while (half < need) half <<= 1;
    // room for a second context of the same shape (a step and its predecessor on buffers of their own, two groups of one
    // process) where the largest pair allows it: the pair cannot grow while somebody holds a lease
    const uint64_t least = half;
    if (half < 2 * need && 2 * half <= kMaxHalf) half <<= 1;
    int reason = find_pair(env, half, p);
    // no clear verdict with the larger allocations: the search again with the smaller ones, which the driver cuts from
    // memory differently
    if (reason == SAR_SPREAD_NO_PAIR && half > least) reason = find_pair(env, least, p);
    return reason;
}

// When a context goes, a pair larger than the smallest one is not kept idle for those that stay.
void shrink_if_idle(Pool& p) {
    if (p.va && p.leases.empty() && p.half > kMinHalf) { (void)hipDeviceSynchronize(); free_pair(p); }
}

void release(Pool& p, const void* owner, bool rows) {
    p.leases.erase(std::remove_if(p.leases.begin(), p.leases.end(), [&](const Lease& l) { return l.owner == owner && l.rows == rows; }), p.leases.end());
}

bool valid(int device) { return device >= 0 && device < kMaxDevices; }

}  // namespace

bool spread_yardstick(const float neighbours_ms[3], float ends_ms, float* yardstick_ms) {
    float adj[3] = {neighbours_ms[0], neighbours_ms[1], neighbours_ms[2]};
    std::sort(adj, adj + 3);
    *yardstick_ms = std::min(ends_ms, adj[1]);
    return !(ends_ms < kStraddle * adj[1]);
}

bool spread_is_elsewhere(float yardstick_ms, float probe_ms_value) { return probe_ms_value > 0.f && probe_ms_value < kFaster * yardstick_ms; }

int spread_pick(float yardstick_ms, const float* t, int n) {
    if (!(yardstick_ms > 0.f) || !t || n < 1) return -1;
    std::vector<int> order;
    try { order.reserve((size_t)n); } catch (const std::bad_alloc&) { return -1; }
    for (int i = 0; i < n; ++i) if (t[i] > 0.f) order.push_back(i);           // a failed probe says nothing
    if (order.empty()) return -1;
    std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return t[a] < t[b]; });
    const int best = order.front();
    if (!spread_is_elsewhere(yardstick_ms, t[best])) return -1;               // nobody clearly below the yardstick
    if (spread_is_elsewhere(yardstick_ms, t[order.back()])) return best;      // everybody is: the yardstick has spoken
    // Two populations: somewhere among the times below the limit the sorted list must jump by kGap and more.  (The limit
    // itself does not separate them: with a yardstick of 190 us it lies at 181 us, where candidates of the first
    // allocation's own region have been seen -- 180.7 us in a search whose candidates elsewhere ended at 163 us.)
    float widest = 0.f;
    for (size_t k = 0; k + 1 < order.size(); ++k) {
        const float lo = t[order[k]], hi = t[order[k + 1]];
        if (!spread_is_elsewhere(yardstick_ms, lo)) break;
        widest = std::max(widest, hi / lo - 1.f);
    }
    return widest >= kGap ? best : -1;
}

void pool_attach(int device, const void* owner) {
    if (!valid(device)) return;
    std::lock_guard<std::mutex> lock(g_mutex[device]);
    Pool& p = g_pool[device];
    if (std::find(p.users.begin(), p.users.end(), owner) == p.users.end()) p.users.push_back(owner);
    p.rec.users = (int)p.users.size();
}

void pool_detach(int device, const void* owner) {
    if (!valid(device)) return;
    std::lock_guard<std::mutex> lock(g_mutex[device]);
    Pool& p = g_pool[device];
    p.leases.erase(std::remove_if(p.leases.begin(), p.leases.end(), [&](const Lease& l) { return l.owner == owner; }), p.leases.end());
    p.users.erase(std::remove(p.users.begin(), p.users.end(), owner), p.users.end());
    p.rec.users = (int)p.users.size();
    if (p.va && hipSetDevice(device) != hipSuccess) (void)hipGetLastError();
    if (p.users.empty() && p.va) { (void)hipDeviceSynchronize(); free_pair(p); }
    else shrink_if_idle(p);
}

int pool_lease_arena(const ProbeEnv& env, const void* owner, uint64_t lo_bytes, uint64_t hi_bytes, char** lo, char** hi) {
    if (!valid(env.device) || !lo || !hi) return SAR_SPREAD_NO_MEMORY;
    std::lock_guard<std::mutex> lock(g_mutex[env.device]);
    if (hipSetDevice(env.device) != hipSuccess) { (void)hipGetLastError(); return SAR_SPREAD_NO_MEMORY; }
    Pool& p = g_pool[env.device];
    release(p, owner, false);                                  // an owner holds one arena at a time
    const uint64_t lo_len = up(lo_bytes, kGranule), hi_len = up(hi_bytes, kGranule);
    const int reason = ensure_pair(env, p, std::max(lo_len, hi_len));
    if (reason != SAR_SPREAD_FOUND) return reason;
    // the lower allocation is filled from its start, the upper one from its end: the junction stays free for rows
    uint64_t lo_off = ~0ull, hi_off = ~0ull;
    for (uint64_t off = 0; off + lo_len <= p.half; off += kGranule) if (free_in(p, false, off, lo_len)) { lo_off = off; break; }
    for (uint64_t off = p.half - hi_len;; off -= kGranule) { if (free_in(p, true, off, hi_len)) { hi_off = off; break; } if (off < kGranule) break; }
    if (lo_off == ~0ull || hi_off == ~0ull) return SAR_SPREAD_POOL_BUSY;
    p.leases.push_back({owner, false, lo_off, lo_len, hi_off, hi_len});
    *lo = p.va + lo_off; *hi = p.va + p.half + hi_off;
    return SAR_SPREAD_FOUND;
}

int pool_lease_rows(const ProbeEnv& env, const void* owner, uint64_t lo_bytes, uint64_t hi_bytes, char** base) {
    if (!valid(env.device) || !base) return SAR_SPREAD_NO_MEMORY;
    std::lock_guard<std::mutex> lock(g_mutex[env.device]);
    if (hipSetDevice(env.device) != hipSuccess) { (void)hipGetLastError(); return SAR_SPREAD_NO_MEMORY; }
    Pool& p = g_pool[env.device];
    release(p, owner, true);
    const int reason = ensure_pair(env, p, std::max(lo_bytes, hi_bytes));
    if (reason != SAR_SPREAD_FOUND) return reason;
    if (!free_in(p, false, p.half - lo_bytes, lo_bytes) || !free_in(p, true, 0, hi_bytes)) return SAR_SPREAD_POOL_BUSY;
    p.leases.push_back({owner, true, p.half - lo_bytes, lo_bytes, 0, hi_bytes});
    *base = p.va + p.half - lo_bytes;
    return SAR_SPREAD_FOUND;
}

void pool_release_arena(int device, const void* owner) {
    if (!valid(device)) return;
    std::lock_guard<std::mutex> lock(g_mutex[device]);
    release(g_pool[device], owner, false);
}

void pool_release_rows(int device, const void* owner) {
    if (!valid(device)) return;
    std::lock_guard<std::mutex> lock(g_mutex[device]);
    release(g_pool[device], owner, true);
}

bool pool_trim(int device) {
    if (!valid(device)) return false;
    std::lock_guard<std::mutex> lock(g_mutex[device]);
    Pool& p = g_pool[device];
    if (!p.va || !p.leases.empty()) return false;
    if (hipSetDevice(device) != hipSuccess) { (void)hipGetLastError(); return false; }
    (void)hipDeviceSynchronize();
    free_pair(p);
    return true;
}

bool pool_leased_by(int device, const void* owner, const char* ptr) {
    if (!valid(device)) return false;
    std::lock_guard<std::mutex> lock(g_mutex[device]);
    const Pool& p = g_pool[device];
    if (!p.va || ptr < p.va || ptr >= p.va + 2 * p.half) return false;
    const uint64_t off = (uint64_t)(ptr - p.va);
    for (const Lease& l : p.leases) {
        if (l.owner != owner) continue;
        if ((off >= l.lo_off && off < l.lo_off + l.lo_len) || (off >= p.half + l.hi_off && off < p.half + l.hi_off + l.hi_len)) return true;
    }
    return false;
}

SearchRecord pool_record(int device) {
    if (!valid(device)) return SearchRecord{};
    std::lock_guard<std::mutex> lock(g_mutex[device]);
    return g_pool[device].rec;
}

}  // namespace sar
