// Host executor and C ABI: rank arena in HBM, lowering of a schedule to
// per-round op tables, cache-policy planning, launch / hipGraph replay, timing.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <mutex>
#include <stdexcept>
#include <string>
#include <vector>

#include "column_plan.hpp"
#include "kernels.hpp"
#include "placed_pool.hpp"
#include "sar.h"
#include "schedule.hpp"

namespace {

thread_local std::string g_error;

int set_error(int code, const std::string& msg) { g_error = msg; return code; }

#define SAR_HIP(expr)                                                                                   \
    do {                                                                                                \
        hipError_t e_ = (expr);                                                                         \
        if (e_ != hipSuccess)                                                                           \
            return set_error(SAR_EHIP, std::string(#expr) + ": " + hipGetErrorString(e_));              \
    } while (0)

constexpr uint64_t kArenaAlign = 2ull << 20;   // rank bases on 2 MiB boundaries (one large-page fragment each)
constexpr uint64_t kSpreadMinPayload = 128ull << 20;   // spread arena: from 16 MiB per rank at n = 8 (below, the caches carry the schedule)
constexpr float kMaxDelayMs = 60000.f;

// One kernel launch: the rows of a round that share a kernel (COPY /
// REDUCE_INTO / XREDUCE in one, MREDUCE in the other).
struct Launch {
    uint32_t first_op = 0, nops = 0, total_tiles = 0, tiles_per_op = 0, reverse = 0;
    bool mreduce = false;
    uint64_t algorithmic_bytes = 0;
};

int elem_size_of(int dtype) { return dtype == SAR_F32 ? 4 : 2; }

// Runs the body of an entry point; no exception leaves the C ABI.
template <class F> int guarded(F&& body) {
    try { return body(); }
    catch (const std::bad_alloc&) { return set_error(SAR_ENOMEM, "out of host memory"); }
    catch (const std::exception& e) { return set_error(SAR_EINVAL, e.what()); }
    catch (...) { return set_error(SAR_EINVAL, "unexpected error"); }
}

}  // namespace

// Row tables of sar_run_static: device memory that belongs to the library image, so that entry point never has to
// allocate.  Every GPU the library runs on holds its own copy of the array at its own address for the life of the
// process.  In host code the name is only a handle for hipGetSymbolAddress (static_scratch below); the address it
// returns is what copies and kernels use.
#define SAR_STATIC_SCRATCH_BYTES (1u << 20)
static __device__ __align__(256) unsigned char scratch[SAR_STATIC_SCRATCH_BYTES];

namespace { int static_scratch(int device, char** out); }

// A column plan as it sits on the device.
struct ColumnDevice {
    bool ready = false;
    uint32_t* d_group_begin = nullptr;
    sar::ColumnComp* d_comps = nullptr;
    uint32_t first_op = 0, ncomp = 0, ncols = 0, run = 1, items = 0, grid = 0, block = 512, slots = 0, lane_local = 0, table_rows = 0, table_groups = 0, policy = 0, multi_source = 0, two_vectors = 0;
};

struct sar_ctx {
    int device = 0;
    hipStream_t stream = nullptr, prework_stream = nullptr;
    hipEvent_t ev_start = nullptr, ev_stop = nullptr, ev_join = nullptr;
    std::vector<hipEvent_t> ev_prof;
    int wall_khz = 100000;

    int n = 0, dtype = SAR_F32;
    uint64_t bytes_per_rank = 0, stride = 0;
    char* arena = nullptr;             // ranks [0, split) at arena + r * stride
    char* arena_hi = nullptr;          // ranks [split, n) at arena_hi + (r - split) * stride (spread arena only)
    int split = 0;
    // Placed memory comes from the GPU's pair of allocations in different regions of HBM (placed_pool.hpp), which all
    // contexts of the process share: an arena lease (ranks [0, split) in the lower allocation, the rest in the upper
    // one) and a lease for sar_alloc_rows (n rows back to back across the junction of the two).  Otherwise `arena` and
    // `rows_plain` are ordinary allocations of this context.
    bool pool_attached = false, arena_leased = false, rows_leased = false;
    char* rows_plain = nullptr;
    char* rows_base = nullptr;         // what the caller holds (null: none handed out)
    uint64_t rows_bytes = 0;
    bool spread_capable = false;       // the device is one whose regions are known (MI355X, 288 GiB)
    int spread_reason = SAR_SPREAD_OFF;            // why the ranks sit where they sit (SAR_SPREAD_*)
    char* snapshot = nullptr;
    int* d_flag = nullptr;

    sar_tuning_t tune{256, 1, 0, 2, 2, 0, 0, 2, 0, 0, 1, 0, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 0};

    // prepared plan
    bool prepared = false;
    sar::DevOp* d_ops = nullptr;
    char** d_ptrs = nullptr;
    std::vector<Launch> prework, rounds;
    sar_stats_t stats{};
    hipGraph_t graph = nullptr, graph_fused = nullptr;            // the main schedule; pre-work + main schedule in one launch
    hipGraphExec_t graph_exec = nullptr, graph_fused_exec = nullptr;

    // column plan (tune.executor == 1): the whole main schedule as one launch
    bool column = false;
    ColumnDevice col;                  // the main schedule
    ColumnDevice fused;                // pre-work + main schedule in one launch (used by sar_run with no delay)
    ColumnDevice pre;                  // the pre-work alone as one column launch (runs beside the straggler's delay)
    int cu_count = 0;

    std::vector<char*> adopted;        // caller-owned rank buffers (sar_adopt_ranks); empty when the arena is in use

    bool has_ranks() const { return arena != nullptr || !adopted.empty(); }
    char* rank_base(int r) const {
        if (!adopted.empty()) return adopted[(size_t)r];
        return r < split ? arena + (uint64_t)r * stride : arena_hi + (uint64_t)(r - split) * stride;
    }
    bool spread() const { return adopted.empty() && arena != nullptr && split < n; }
    uint64_t elems() const { return bytes_per_rank / (uint64_t)elem_size_of(dtype); }
    uint64_t snapshot_stride() const { return adopted.empty() ? stride : (bytes_per_rank + 255u) & ~(uint64_t)255u; }
};

namespace {

void drop_plan(sar_ctx* c) {
    if (c->graph_exec) { (void)hipGraphExecDestroy(c->graph_exec); c->graph_exec = nullptr; }
    if (c->graph) { (void)hipGraphDestroy(c->graph); c->graph = nullptr; }
    if (c->graph_fused_exec) { (void)hipGraphExecDestroy(c->graph_fused_exec); c->graph_fused_exec = nullptr; }
    if (c->graph_fused) { (void)hipGraphDestroy(c->graph_fused); c->graph_fused = nullptr; }
    if (c->d_ops) { (void)hipFree(c->d_ops); c->d_ops = nullptr; }
    if (c->d_ptrs) { (void)hipFree(c->d_ptrs); c->d_ptrs = nullptr; }
    for (ColumnDevice* d : {&c->col, &c->fused, &c->pre}) {
        if (d->d_group_begin) (void)hipFree(d->d_group_begin);
        if (d->d_comps) (void)hipFree(d->d_comps);
        *d = ColumnDevice{};
    }
    c->column = false;
    c->prework.clear(); c->rounds.clear(); c->prepared = false;
    c->stats = sar_stats_t{};
}

sar::ProbeEnv probe_env(const sar_ctx* c) { return sar::ProbeEnv{c->device, c->stream, c->wall_khz}; }

void attach_pool(sar_ctx* c) {
    if (!c->pool_attached) { sar::pool_attach(c->device, c); c->pool_attached = true; }
}

// The rank buffers go.  A lease goes back to the pool only once the whole device is idle: a caller's own kernels on
// streams of its own may still be working on addresses it got from sar_rank_pointer.
void drop_ranks(sar_ctx* c) {
    drop_plan(c);
    if (c->arena && c->arena_leased) { (void)hipDeviceSynchronize(); sar::pool_release_arena(c->device, c); }
    else if (c->arena) (void)hipFree(c->arena);
    c->arena = c->arena_hi = nullptr; c->split = 0; c->arena_leased = false;
    if (c->snapshot) { (void)hipFree(c->snapshot); c->snapshot = nullptr; }
    c->adopted.clear();
    c->n = 0; c->bytes_per_rank = 0; c->stride = 0;
}

// ---- rows in one virtual range (sar_alloc_rows) --------------------------------------------------------
// Everything sar_alloc_rows holds.  The whole device is drained first: a caller's kernels on streams of its own (a
// torch tensor over these rows) may still be touching the memory.
void release_rows(sar_ctx* c) {
    if (c->rows_leased || c->rows_plain) (void)hipDeviceSynchronize();
    if (c->rows_leased) sar::pool_release_rows(c->device, c);
    if (c->rows_plain) {
        const hipError_t e = hipFree(c->rows_plain);
        if (e != hipSuccess) { (void)hipGetLastError(); if (std::getenv("SAR_DEBUG")) std::fprintf(stderr, "sar: releasing rows: hipFree: %s\n", hipGetErrorString(e)); }
    }
    c->rows_plain = c->rows_base = nullptr; c->rows_bytes = 0; c->rows_leased = false;
}

bool rows_adopted(const sar_ctx* c) {
    if (!c->rows_base) return false;
    for (const char* p : c->adopted) if (p >= c->rows_base && p < c->rows_base + c->rows_bytes) return true;
    return false;
}

// A byte interval of one rank buffer that a row reads or writes.
struct Touch { int rank; uint64_t lo, hi; };

struct RowAccess {
    std::vector<Touch> reads, writes;   // writes[0] belongs to p0, writes[1] to p1 (XREDUCE)
};

bool overlaps(const Touch& a, const Touch& b) { return a.rank == b.rank && a.lo < b.hi && b.lo < a.hi; }

RowAccess accesses(const sar::Schedule& s, const sar::Op& op, uint64_t elems, int es) {
    sar::Range r = sar::lower_range(s, op, elems);
    RowAccess a;
    uint64_t dlo = r.dst_off * es, slo = r.src_off * es, len = r.len * es;
    switch (op.kind) {
        case SAR_OP_COPY:
            a.reads.push_back({op.src_rank, slo, slo + len});
            a.writes.push_back({op.dst_rank, dlo, dlo + len});
            break;
        case SAR_OP_REDUCE_INTO:
            a.reads.push_back({op.dst_rank, dlo, dlo + len});
            a.reads.push_back({op.src_rank, slo, slo + len});
            a.writes.push_back({op.dst_rank, dlo, dlo + len});
            break;
        case SAR_OP_XREDUCE:
            a.reads.push_back({op.dst_rank, dlo, dlo + len});
            a.reads.push_back({op.src_rank, slo, slo + len});
            a.writes.push_back({op.dst_rank, dlo, dlo + len});
            a.writes.push_back({op.src_rank, slo, slo + len});
            break;
        default:
            for (int q = 0; q < op.group; ++q) a.reads.push_back({q, dlo, dlo + len});
            if (op.bcast) { for (int q = 0; q < op.group; ++q) a.writes.push_back({q, dlo, dlo + len}); }
            else a.writes.push_back({op.dst_rank, dlo, dlo + len});
            break;
    }
    return a;
}

// Lower every round of `s` to device rows appended to `rows` / `ptrs`.
int lower(sar_ctx* c, const sar::Schedule& s, std::vector<sar::DevOp>& rows, std::vector<char*>& ptrs, std::vector<Launch>& out,
          const sar::Schedule* next /* schedule that runs afterwards, for the cache look-ahead */) {
    const int es = elem_size_of(c->dtype);
    const uint64_t elems = c->elems();
    const uint64_t round_tile_bytes = (uint64_t)c->tune.block * (uint64_t)c->tune.unroll * 16u;

    // per-round access lists, including those of the schedule that follows
    std::vector<std::vector<RowAccess>> acc;
    for (const auto& round : s.rounds) {
        std::vector<RowAccess> v;
        for (const auto& op : round) v.push_back(accesses(s, op, elems, es));
        acc.push_back(v);
    }
    const size_t own_rounds = acc.size();
    if (next)
        for (const auto& round : next->rounds) {
            std::vector<RowAccess> v;
            for (const auto& op : round) v.push_back(accesses(*next, op, elems, es));
            acc.push_back(v);
        }
    auto read_soon = [&](size_t round, const Touch& t) {
        size_t last = std::min(acc.size(), round + 1 + (size_t)std::max(0, c->tune.reuse_rounds));
        for (size_t r = round + 1; r < last; ++r)
            for (const auto& ra : acc[r])
                for (const auto& rd : ra.reads)
                    if (overlaps(rd, t)) return true;
        return false;
    };

    // With segments > 1 every row is cut into that many consecutive pieces and the whole schedule is run
    // piece by piece: all rounds on the first piece of every chunk, then all rounds on the second, ...
    // (the work is element-wise, so the pieces are independent); this shrinks what has to stay in the
    // Infinity Cache between a round and the next.
    uint64_t nseg = (uint64_t)std::max(0, c->tune.segments);
    if (nseg == 0) {
        // automatic: keep the bytes the rows of one round cover near the capacity of the 256 MB cache
        // (measured on n=8: 1 piece is best at 38 MB rows, 4 pieces at 153 MB rows)
        uint64_t widest = 0;
        for (const auto& round : s.rounds) {
            uint64_t sum = 0;
            for (const auto& op : round) sum += sar::lower_range(s, op, elems).len * es;
            widest = std::max(widest, sum);
        }
        nseg = std::max<uint64_t>(1, std::min<uint64_t>(256, widest / 300000000ull));
    }
    for (uint64_t seg = 0; seg < nseg; ++seg)
    for (size_t ri = 0; ri < own_rounds; ++ri) {
      const auto& round = s.rounds[ri];
      for (int cls = 0; cls < 2; ++cls) {
        const uint64_t tile_bytes = cls ? sar::mreduce_tile_bytes() : round_tile_bytes;
        Launch L; L.first_op = (uint32_t)rows.size(); L.mreduce = cls != 0;
        uint64_t tiles = 0; bool uniform = true; uint64_t first_tiles = 0;
        for (size_t oi = 0; oi < round.size(); ++oi) {
            const sar::Op& op = round[oi];
            if ((op.kind == SAR_OP_MREDUCE) != (cls != 0)) continue;
            sar::Range rg = sar::lower_range(s, op, elems);
            const uint64_t row_bytes = rg.len * es;
            if (row_bytes == 0) continue;   // buffer shorter than `parts` elements: nothing to move
            const uint64_t row_doff = rg.dst_off * es, row_soff = rg.src_off * es;
            if (row_doff + row_bytes > c->bytes_per_rank || row_soff + row_bytes > c->bytes_per_rank) return set_error(SAR_ESCHED, "row leaves the rank buffer");
            // The part of this row that belongs to piece `seg`.  Pieces partition the offset WITHIN a chunk
            // (rows move whole chunks, so an element only ever meets elements at its own within-chunk
            // offset): a row of several chunks contributes one span per chunk.
            struct Span { uint64_t doff, soff, bytes; };
            std::vector<Span> spans;
            if (nseg == 1) {
                spans.push_back({row_doff, row_soff, row_bytes});
            } else {
                const uint64_t chunk_bytes = (elems / (uint64_t)s.parts) * es;
                const uint64_t piece = ((chunk_bytes + nseg - 1) / nseg + 4095u) & ~(uint64_t)4095u;
                for (int j = 0; j < op.nchunks; ++j) {
                    const uint64_t base = (uint64_t)j * chunk_bytes;
                    const uint64_t len = (j == op.nchunks - 1) ? row_bytes - base : chunk_bytes;   // a to_end row ends with a longer chunk
                    const uint64_t lo = std::min(seg * piece, len);
                    const uint64_t hi = (seg == nseg - 1) ? len : std::min((seg + 1) * piece, len);
                    if (lo < hi) spans.push_back({row_doff + base + lo, row_soff + base + lo, hi - lo});
                }
            }
            for (const Span& sp : spans) {
            const uint64_t doff = sp.doff, soff = sp.soff, bytes = sp.bytes;
            sar::DevOp d{};
            d.kind = (uint32_t)op.kind; d.bytes = bytes;
            bool aligned = true;
            if (op.kind == SAR_OP_MREDUCE) {
                // ring order over the group: x_{r+1}, x_{r+2}, ..., x_{r-1}, x_r (the owner last)
                d.ptr_off = (uint32_t)ptrs.size(); d.nsrc = (uint32_t)op.group;
                for (int j = 1; j <= op.group; ++j) ptrs.push_back(c->rank_base((op.dst_rank + j) % op.group) + doff);
                if (op.bcast) { d.ndst = (uint32_t)op.group; for (int q = 0; q < op.group; ++q) ptrs.push_back(c->rank_base(q) + doff); }
                else { d.ndst = 1; ptrs.push_back(c->rank_base(op.dst_rank) + doff); }
                for (size_t k = d.ptr_off; k < ptrs.size(); ++k) aligned &= ((uintptr_t)ptrs[k] & 15u) == 0;
            } else {
                d.p0 = c->rank_base(op.dst_rank) + doff;
                d.p1 = c->rank_base(op.src_rank) + soff;
                aligned = (((uintptr_t)d.p0 | (uintptr_t)d.p1) & 15u) == 0;
            }
            if (aligned) d.flags |= sar::DEVOP_VEC;
            // cache policy
            const RowAccess& ra = acc[ri][oi];
            if (c->tune.cache_policy == 1) {
                d.flags |= sar::DEVOP_LNT | sar::DEVOP_SNT0 | sar::DEVOP_SNT1;
            } else if (c->tune.cache_policy == 3) {
                d.flags |= sar::DEVOP_LNT;
            } else if (c->tune.cache_policy == 2) {
                bool any_read_again = false;
                for (const auto& rd : ra.reads) any_read_again |= read_soon(ri, rd);
                if (!any_read_again) d.flags |= sar::DEVOP_LNT;
                if (op.kind == SAR_OP_MREDUCE) {
                    bool again = false;
                    for (const auto& w : ra.writes) again |= read_soon(ri, w);
                    if (!again) d.flags |= sar::DEVOP_SNT0;
                } else {
                    if (!read_soon(ri, ra.writes[0])) d.flags |= sar::DEVOP_SNT0;
                    if (ra.writes.size() > 1 && !read_soon(ri, ra.writes[1])) d.flags |= sar::DEVOP_SNT1;
                }
            }
            uint64_t nt = (bytes + tile_bytes - 1) / tile_bytes;
            if (tiles + nt > 0x7fffffffull) return set_error(SAR_EINVAL, "round needs more than 2^31 tiles");
            d.tile_begin = (uint32_t)tiles; d.ntiles = (uint32_t)nt;
            if (L.nops == 0) first_tiles = nt; else uniform &= (nt == first_tiles);
            tiles += nt;
            uint64_t k = 0;
            switch (op.kind) {
                case SAR_OP_COPY: k = 2; break;
                case SAR_OP_REDUCE_INTO: k = 3; break;
                case SAR_OP_XREDUCE: k = 4; break;
                default: k = d.nsrc + d.ndst; break;
            }
            L.algorithmic_bytes += k * bytes;
            rows.push_back(d); L.nops++;
            }
        }
        if (L.nops == 0) continue;
        L.total_tiles = (uint32_t)tiles;
        L.tiles_per_op = uniform ? (uint32_t)first_tiles : 0;
        L.reverse = (c->tune.reverse_odd && (ri & 1)) ? 1u : 0u;
        out.push_back(L);
      }
    }
    return SAR_OK;
}

using sar::ColumnPlan;

sar::ColumnEnv column_env(const sar_ctx* c) {
    sar::ColumnEnv env;
    env.tune = c->tune; env.n = c->n; env.elem_size = elem_size_of(c->dtype); env.elems = c->elems();
    env.bytes_per_rank = c->bytes_per_rank; env.compute_units = c->cu_count;
    for (int r = 0; r < c->n; ++r) env.rank_base.push_back(c->rank_base(r));
    return env;
}

int lower_column(const sar_ctx* c, const std::vector<const sar::Schedule*>& scheds, std::vector<sar::DevOp>& rows, std::vector<char*>& ptrs, ColumnPlan& plan) {
    std::string error;
    const int rc = sar::plan_columns(column_env(c), scheds, rows, ptrs, plan, &error);
    return rc == SAR_OK ? SAR_OK : set_error(rc, error);
}

// Which executor is expected to be faster (executor = 2).  Constants are measurements on MI355X.
// Column kernel, bandwidth regime: without forwarding 7.1 algorithmic TB/s while a work item is up to ~128
// rows long, less for longer items, whose workgroups drift apart and scatter the access streams (6.4 up to
// 256 rows, 5.3 beyond).  With forwarding what counts is the bytes that still go to memory: 5.0 TB/s when
// they are mostly stores (three tenths or more of the operands found in slots), 6.0 otherwise.  A workgroup
// needs about 0.6 us per row of its item while everything stays cache resident, 0.95 us beyond that; with
// the item's rows in LDS (latency plan) 0.32-0.65 us.  One launch per round moves 6.5 TB/s and costs about
// 3 us per launch.
bool column_pays(const sar_ctx* c, const ColumnPlan& cp) {
    const double bytes = (double)c->stats.algorithmic_bytes;
    const double item_rows = (double)cp.max_comp_rows;
    double est_rounds = 0;
    for (const auto& L : c->rounds) if (L.total_tiles) est_rounds += 3.0 + (double)L.algorithmic_bytes / 6.5e6;
    if (cp.staged) {
        const double resident_bytes = (double)c->bytes_per_rank * c->n;
        const double per_row_us = resident_bytes <= 262144.0 ? 0.32 : resident_bytes <= 33554432.0 ? 0.45 : 0.65;
        return 4.0 + std::max(item_rows * per_row_us, bytes / 5.5e6) <= est_rounds;
    }
    const uint64_t cb = cp.column_bytes();
    const double items = (double)((cp.widest_row + cb - 1) / cb) * (double)cp.comps.size();
    double wgs_per_cu = 2048.0 / cp.block;
    if (cp.nslots) wgs_per_cu = std::max(1.0, std::min(wgs_per_cu, std::floor(160.0 * 1024.0 / ((double)cp.nslots * (double)cb))));
    const double resident = (double)std::max(1, c->cu_count) * wgs_per_cu;
    const double per_row_us = (double)c->bytes_per_rank * c->n <= 200e6 ? 0.6 : 0.95;
    const double passes = std::ceil(items / resident);
    double est_stream;
    if (cp.nslots) {
        const double to_memory = std::max(0.0, bytes - (double)cp.forwarded_bytes - (double)cp.elided_bytes);
        est_stream = to_memory / ((double)cp.forwarded_bytes >= 0.3 * bytes ? 5.0e6 : 6.0e6);             // bytes per us
    } else {
        est_stream = bytes / (item_rows <= 128 ? 7.1e6 : item_rows <= 256 ? 6.4e6 : 5.3e6);
    }
    const double est_column = std::max(est_stream, item_rows * per_row_us * passes) + 4.0;
    return est_column <= est_rounds;
}

int launch_column_plan(sar_ctx* c, const ColumnDevice& d, hipStream_t st) {
    sar::ColumnLaunch L{};
    L.ops = c->d_ops + d.first_op; L.group_begin = d.d_group_begin; L.comps = d.d_comps; L.ptrs = c->d_ptrs;
    L.ncomp = d.ncomp; L.nitems = d.items;
    L.table_rows = d.table_rows; L.table_groups = d.table_groups;
    L.lane_local = d.lane_local; L.policy = d.policy; L.multi_source = d.multi_source; L.two_vectors = d.two_vectors;
    L.ncols = d.ncols; L.run = d.run;
    SAR_HIP(sar::launch_column(c->dtype, (int)d.block, d.grid, d.slots, st, L));
    return SAR_OK;
}
int launch_column_plan(sar_ctx* c, const ColumnDevice& d) { return launch_column_plan(c, d, c->stream); }

// Launch shape of a column plan whose rows sit in the row table from `first_op` on (no device work).
int shape_column_plan(const sar_ctx* c, const ColumnPlan& cp, uint32_t first_op, ColumnDevice& d) {
    const uint64_t cb = cp.column_bytes();
    const uint64_t ncols = (cp.widest_row + cb - 1) / cb;
    const uint64_t items = ncols * cp.comps.size();
    if (items > 0x7fffffffull) return set_error(SAR_EINVAL, "schedule needs more than 2^31 work items");
    d.block = (uint32_t)cp.block;
    d.slots = cp.nslots;
    d.lane_local = (cp.lane_local && c->tune.col_light_sync) ? 1u : 0u;
    d.multi_source = cp.multi_source ? 1u : 0u;
    d.table_rows = cp.staged ? cp.max_comp_rows : 0u;
    d.table_groups = cp.staged ? cp.max_comp_groups + 1u : 0u;
    d.policy = cp.policy;
    d.two_vectors = cp.two_vectors ? 1u : 0u;
    d.first_op = first_op; d.ncomp = (uint32_t)cp.comps.size(); d.ncols = (uint32_t)ncols;
    d.run = cp.component_major ? (uint32_t)ncols : 1u;        // d.run divides ncols either way: no padding items
    d.items = (uint32_t)items;
    // Grid: one workgroup per item, so that the workgroups resident at a time work on neighbouring items (a smaller
    // grid whose workgroups stride over the items has them on several distant ranges at once: n = 8, 1 GiB per
    // rank, 2 to 4 % slower for all four algorithms).  A launch of multi-source rows alone is the exception: seven
    // reads per vector run 2 % faster from 64 workgroups per compute unit striding.
    const uint64_t per_cu = c->tune.col_wgs > 0 ? (uint64_t)c->tune.col_wgs : (cp.multi_source && cp.nslots == 0 ? 64u : 4096u);
    d.grid = (uint32_t)std::min<uint64_t>(items, (uint64_t)std::max(1, c->cu_count) * per_cu);
    return SAR_OK;
}

// Copy a column plan's tables to the device (its rows are in d_ops from `first_op` on).
int upload_column_plan(sar_ctx* c, const ColumnPlan& cp, uint32_t first_op, ColumnDevice& d) {
    int rc = shape_column_plan(c, cp, first_op, d); if (rc) return rc;
    SAR_HIP(hipMalloc((void**)&d.d_group_begin, cp.group_begin.size() * sizeof(uint32_t)));
    SAR_HIP(hipMemcpy(d.d_group_begin, cp.group_begin.data(), cp.group_begin.size() * sizeof(uint32_t), hipMemcpyHostToDevice));
    SAR_HIP(hipMalloc((void**)&d.d_comps, cp.comps.size() * sizeof(sar::ColumnComp)));
    SAR_HIP(hipMemcpy(d.d_comps, cp.comps.data(), cp.comps.size() * sizeof(sar::ColumnComp), hipMemcpyHostToDevice));
    d.ready = true;
    return SAR_OK;
}

int launch_one(sar_ctx* c, const Launch& L, hipStream_t st) {
    if (L.total_tiles == 0) return SAR_OK;
    const uint32_t interleave = (uint32_t)(c->tune.order == 1);
    if (L.mreduce)
        SAR_HIP(sar::launch_mreduce(c->dtype, st, c->d_ops + L.first_op, L.nops, c->d_ptrs, L.total_tiles, L.tiles_per_op, interleave, L.reverse));
    else
        SAR_HIP(sar::launch_round(c->dtype, c->tune.unroll, c->tune.block, st, c->d_ops + L.first_op, L.nops,
                                  L.total_tiles, L.tiles_per_op, interleave, L.reverse));
    return SAR_OK;
}
int launch_one(sar_ctx* c, const Launch& L) { return launch_one(c, L, c->stream); }

int launch_all(sar_ctx* c, const std::vector<Launch>& v, hipStream_t st) {
    for (const auto& L : v) { int rc = launch_one(c, L, st); if (rc) return rc; }
    return SAR_OK;
}
int launch_all(sar_ctx* c, const std::vector<Launch>& v) { return launch_all(c, v, c->stream); }

int launch_main(sar_ctx* c) { return c->column ? launch_column_plan(c, c->col) : launch_all(c, c->rounds); }

// The column plans sar_prepare may use, and whether it does.
struct HostPlans {
    ColumnPlan cp, fp, pp;             // the main schedule; pre-work + main schedule in one launch; the pre-work alone
    uint32_t col_first = 0, fused_first = 0, pre_first = 0;      // their first rows in the row table
    bool want_column = false, want_fused = false, want_pre = false;
};

// Everything sar_prepare decides, on the host alone: the rows of both executors, and whether the column executor runs.
int plan_on_host(sar_ctx* c, const sar_schedule* prework, const sar_schedule* main_sched, std::vector<sar::DevOp>& rows,
                 std::vector<char*>& ptrs, HostPlans& hp) {
    int rc;
    hp = HostPlans();
    try {
        if (prework && (rc = lower(c, prework->s, rows, ptrs, c->prework, &main_sched->s)) != SAR_OK) return rc;
        if ((rc = lower(c, main_sched->s, rows, ptrs, c->rounds, nullptr)) != SAR_OK) return rc;
        sar::byte_counts(main_sched->s, c->elems(), elem_size_of(c->dtype), &c->stats.algorithmic_bytes, nullptr);
        bool columnar = c->tune.executor != 0;
        bool multi_source = false;
        for (const auto& L : c->rounds) multi_source |= L.mreduce;
        // a schedule of multi-source rows (the pre-work timed on its own) runs as column launches when col_prework says so
        if (multi_source && !c->tune.col_prework) columnar = false;
        if (columnar) {
            hp.col_first = (uint32_t)rows.size();
            if ((rc = lower_column(c, {&main_sched->s}, rows, ptrs, hp.cp)) != SAR_OK) return rc;
            columnar = rows.size() > hp.col_first && !hp.cp.unsupported;
        }
        // (multi-source rows: measured, the column kernel is the faster one at every size, see mreduce_kernel)
        if (columnar && c->tune.executor == 2 && !multi_source) columnar = column_pays(c, hp.cp);
        hp.want_column = columnar;
        // Pre-work and main schedule as ONE launch, for runs in which nobody is late (the pre-work then simply
        // precedes the schedule): its result for a chunk is handed to the exchange of that chunk in a value slot.
        if (columnar && prework && c->tune.col_fuse_prework) {
            hp.fused_first = (uint32_t)rows.size();
            // A schedule of whole-buffer rows (direct) behind a pre-work that is cut into chunks: the same rows,
            // written over the pre-work's chunks (the last one takes the elements past the last chunk boundary
            // along, as the pre-work's last row does).
            sar::Schedule recut;
            const sar::Schedule* second = &main_sched->s;
            if (second->parts == 1 && prework->s.parts > 1) {
                recut = *second;
                recut.parts = prework->s.parts;
                bool whole = true;
                for (auto& round : recut.rounds)
                    for (auto& op : round) {
                        whole = whole && op.kind != SAR_OP_MREDUCE && op.dst_chunk == 0 && op.src_chunk == 0 && op.nchunks == 1;
                        op.nchunks = recut.parts; op.to_end = 1;
                    }
                if (whole) second = &recut;
            }
            if ((rc = lower_column(c, {&prework->s, second}, rows, ptrs, hp.fp)) != SAR_OK) return rc;
            hp.want_fused = rows.size() > hp.fused_first && !hp.fp.unsupported;
        }
        // The pre-work alone as one column launch, for runs in which it overlaps the straggler's delay (and for
        // runs without a delay when there is no single launch for both).
        if (prework && c->tune.executor != 0 && c->tune.col_prework) {
            hp.pre_first = (uint32_t)rows.size();
            if ((rc = lower_column(c, {&prework->s}, rows, ptrs, hp.pp)) != SAR_OK) return rc;
            hp.want_pre = rows.size() > hp.pre_first && !hp.pp.unsupported;
        }
    } catch (const std::bad_alloc&) { return set_error(SAR_ENOMEM, "out of host memory"); }
    return SAR_OK;
}

sar_stats_t plan_stats(const sar_ctx* c, const sar_schedule* prework, const sar_schedule* main_sched, const ColumnPlan& cp, bool column, bool fused, bool pre_column,
                       const ColumnPlan* fp = nullptr) {
    sar_stats_t st{};
    sar::byte_counts(main_sched->s, c->elems(), elem_size_of(c->dtype), &st.algorithmic_bytes, &st.reference_op_bytes);
    if (prework) sar::byte_counts(prework->s, c->elems(), elem_size_of(c->dtype), &st.prework_bytes, nullptr);
    st.rounds = (int)main_sched->s.rounds.size();
    for (const auto& r : main_sched->s.rounds) st.ops += (int)r.size();
    if (column) st.main_launches = 1;
    else for (const auto& L : c->rounds) st.main_launches += L.total_tiles ? 1 : 0;
    if (pre_column) st.prework_launches = 1;
    else for (const auto& L : c->prework) st.prework_launches += L.total_tiles ? 1 : 0;
    st.launches = st.main_launches + st.prework_launches;
    st.executor = column ? 1 : 0;
    st.col_block = column ? (int32_t)cp.block : 0;
    st.col_slots = column ? (int32_t)cp.nslots : 0;
    st.col_components = column ? (int32_t)cp.comps.size() : 0;
    st.forwarded_bytes = column ? cp.forwarded_bytes : 0;
    st.elided_store_bytes = column ? cp.elided_bytes : 0;
    st.fused_prework = fused ? 1 : 0;
    if (fused && fp) { st.fused_forwarded_bytes = fp->forwarded_bytes; st.fused_elided_store_bytes = fp->elided_bytes; }
    st.arena_spread = c->spread() ? 1 : 0;
    st.spread_reason = c->spread_reason;
    if (c->pool_attached) {
        const sar::SearchRecord rec = sar::pool_record(c->device);
        st.spread_candidates = rec.candidates; st.spread_same_ms = rec.same_ms; st.spread_pair_ms = rec.pair_ms;
        st.spread_search_bytes = rec.search_bytes; st.placed_pool_bytes = rec.pool_bytes; st.placed_pool_contexts = rec.users;
    }
    return st;
}

bool valid_tuning(const sar_tuning_t& t) {
    return (t.block == 256 || t.block == 512) && (t.unroll == 1 || t.unroll == 2 || t.unroll == 4 || t.unroll == 8) &&
           (t.order == 0 || t.order == 1) && t.cache_policy >= 0 && t.cache_policy <= 3 && t.reuse_rounds >= 0 && t.reuse_rounds <= 64 &&
           (t.reverse_odd == 0 || t.reverse_odd == 1) && t.segments >= 0 && t.segments <= 256 &&
           (t.executor >= 0 && t.executor <= 2) && t.col_wgs >= 0 && t.col_wgs <= 4096 &&
           (t.col_block == 0 || t.col_block == 256 || t.col_block == 512 || t.col_block == 1024) &&
           (t.col_forward == 0 || t.col_forward == 1) && t.col_slots >= 0 && t.col_slots <= 255 &&
           (t.col_light_sync == 0 || t.col_light_sync == 1) && t.col_latency_plan >= 0 && t.col_latency_plan <= 2 &&
           (t.col_split == 0 || t.col_split == 1) && (t.col_fuse_prework == 0 || t.col_fuse_prework == 1) &&
           (t.col_elide_stores == 0 || t.col_elide_stores == 1) && t.col_fuse_chains >= 0 && t.col_fuse_chains <= 2 && t.col_fuse_copies >= 0 && t.col_fuse_copies <= 2 &&
           (t.arena_spread == 0 || t.arena_spread == 1) && (t.col_prework == 0 || t.col_prework == 1) && (t.col_depth_first == 0 || t.col_depth_first == 1) && t.col_vectors >= 0 && t.col_vectors <= 2;
}

// sar_plan / sar_plan_rows: a context that never touches the device, with the rank buffers at made-up, suitably
// aligned addresses (only ever used for arithmetic), and everything sar_prepare would decide for it.
struct HostPlan {
    sar_ctx c;
    uint64_t stride = 0;
    std::vector<sar::DevOp> rows; std::vector<char*> ptrs;
    HostPlans hp;

    int make(const sar_schedule* prework, const sar_schedule* main_sched, int n, uint64_t bytes_per_rank, int dtype,
             const sar_tuning_t* tuning, int compute_units) {
        if (!main_sched) return set_error(SAR_EINVAL, "null argument");
        if (n < 2 || n > SAR_MAX_RANKS) return set_error(SAR_EINVAL, "n out of range");
        if (dtype != SAR_F32 && dtype != SAR_F16 && dtype != SAR_BF16) return set_error(SAR_EINVAL, "unknown dtype");
        if (bytes_per_rank == 0 || bytes_per_rank % (uint64_t)elem_size_of(dtype)) return set_error(SAR_EINVAL, "bytes_per_rank must be a positive multiple of the element size");
    if (bytes_per_rank > SAR_MAX_RANK_BYTES) return set_error(SAR_EINVAL, "bytes_per_rank is larger than SAR_MAX_RANK_BYTES");
        if (tuning && !valid_tuning(*tuning)) return set_error(SAR_EINVAL, "tuning value out of range");
        for (const sar_schedule* s : {prework, main_sched}) {
            if (!s) continue;
            if (s->s.n != n) return set_error(SAR_EINVAL, "schedule and rank count disagree");
            std::string why = sar::validate(s->s);
            if (!why.empty()) return set_error(SAR_ESCHED, why);
        }
        c.n = n; c.dtype = dtype; c.bytes_per_rank = bytes_per_rank;
        c.cu_count = compute_units > 0 ? compute_units : 256;
        if (tuning) c.tune = *tuning;
        stride = (bytes_per_rank + (2u << 20) - 1) & ~(uint64_t)((2u << 20) - 1);
        for (int r = 0; r < n; ++r) c.adopted.push_back(reinterpret_cast<char*>((uintptr_t)1 << 40) + (uint64_t)r * stride);
        return plan_on_host(&c, prework, main_sched, rows, ptrs, hp);
    }
};

}  // namespace

extern "C" {

int sar_version(void) { return SAR_VERSION; }
const char* sar_last_error(void) { return g_error.c_str(); }

int sar_device_count(int* count) {
    if (!count) return set_error(SAR_EINVAL, "count is null");
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess) { *count = 0; (void)hipGetLastError(); return set_error(SAR_ENODEV, std::string("hipGetDeviceCount: ") + hipGetErrorString(e)); }
    *count = n;
    return SAR_OK;
}

uint64_t sar_pad_bytes(uint64_t bytes, int n) { return sar::pad_bytes(bytes, n); }

// ---- schedules ---------------------------------------------------------------

int sar_schedule_parse(const char* text, size_t len, int n, sar_schedule** out) {
    if (!out) return set_error(SAR_EINVAL, "out is null");
    *out = nullptr;
    try {
        sar_schedule* s = new sar_schedule{sar::parse_table(text, len, n)};
        *out = s; return SAR_OK;
    } catch (const std::bad_alloc&) { return set_error(SAR_ENOMEM, "out of host memory");
    } catch (const std::exception& e) { return set_error(SAR_EPARSE, e.what()); }
}

int sar_schedule_builtin(const char* alg, int n, sar_schedule** out) {
    if (!out || !alg) return set_error(SAR_EINVAL, "null argument");
    *out = nullptr;
    try {
        sar_schedule* s = new sar_schedule{sar::builtin(alg, n)};
        *out = s; return SAR_OK;
    } catch (const std::bad_alloc&) { return set_error(SAR_ENOMEM, "out of host memory");
    } catch (const std::exception& e) { return set_error(SAR_EINVAL, e.what()); }
}

static int schedule_validate_body(const sar_schedule* s, char* msg, size_t cap) {
    if (!s) return set_error(SAR_EINVAL, "schedule is null");
    std::string why;
    try { why = sar::validate(s->s); } catch (const std::exception& e) { why = e.what(); }
    if (msg && cap) { std::snprintf(msg, cap, "%s", why.c_str()); }
    if (!why.empty()) return set_error(SAR_ESCHED, why);
    return SAR_OK;
}

int sar_schedule_validate(const sar_schedule* s, char* msg, size_t cap) {
    return guarded([&] { return schedule_validate_body(s, msg, cap); });
}

int sar_schedule_ranks(const sar_schedule* s) { return s ? s->s.n : SAR_EINVAL; }
int sar_schedule_parts(const sar_schedule* s) { return s ? s->s.parts : SAR_EINVAL; }
int sar_schedule_rounds(const sar_schedule* s) { return s ? (int)s->s.rounds.size() : SAR_EINVAL; }
int sar_schedule_round_ops(const sar_schedule* s, int round) {
    if (!s || round < 0 || round >= (int)s->s.rounds.size()) return set_error(SAR_EINVAL, "round out of range");
    return (int)s->s.rounds[round].size();
}
int sar_schedule_op(const sar_schedule* s, int round, int index, sar_op_info* out) {
    if (!s || !out || round < 0 || round >= (int)s->s.rounds.size()) return set_error(SAR_EINVAL, "round out of range");
    const auto& r = s->s.rounds[round];
    if (index < 0 || index >= (int)r.size()) return set_error(SAR_EINVAL, "row out of range");
    const sar::Op& o = r[index];
    out->kind = o.kind; out->dst_rank = o.dst_rank; out->src_rank = o.src_rank; out->dst_chunk = o.dst_chunk;
    out->src_chunk = o.src_chunk; out->nchunks = o.nchunks; out->group = o.group; out->bcast = o.bcast; out->to_end = o.to_end;
    return SAR_OK;
}

int sar_schedule_bytes(const sar_schedule* s, uint64_t elems, int elem_size, uint64_t* algorithmic, uint64_t* reference_op) {
    if (!s || elem_size < 1) return set_error(SAR_EINVAL, "bad argument");
    sar::byte_counts(s->s, elems, elem_size, algorithmic, reference_op);
    return SAR_OK;
}

void sar_schedule_free(sar_schedule* s) { delete s; }

// ---- context -------------------------------------------------------------------

int sar_create(int device, sar_ctx** out) {
    if (!out) return set_error(SAR_EINVAL, "out is null");
    *out = nullptr;
    int count = 0;
    int rc = sar_device_count(&count);
    if (rc) return rc;
    if (count < 1) return set_error(SAR_ENODEV, "no HIP device: this library has no CPU path");
    if (device < 0 || device >= count) return set_error(SAR_EINVAL, "device index out of range");
    SAR_HIP(hipSetDevice(device));
    sar_ctx* c = new (std::nothrow) sar_ctx();
    if (!c) return set_error(SAR_ENOMEM, "out of host memory");
    c->device = device;
    hipError_t e;
    if ((e = hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking)) != hipSuccess ||
        (e = hipStreamCreateWithFlags(&c->prework_stream, hipStreamNonBlocking)) != hipSuccess ||
        (e = hipEventCreate(&c->ev_start)) != hipSuccess || (e = hipEventCreate(&c->ev_stop)) != hipSuccess ||
        (e = hipEventCreateWithFlags(&c->ev_join, hipEventDisableTiming)) != hipSuccess ||
        (e = hipMalloc((void**)&c->d_flag, sizeof(int))) != hipSuccess) {
        sar_destroy(c);
        return set_error(SAR_EHIP, std::string("context setup: ") + hipGetErrorString(e));
    }
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) == hipSuccess && cus > 0) c->cu_count = cus;
    {
        // three regions of 96 GiB (see find_pair in placed_pool.cpp); only known for the 288 GiB of MI355X
        size_t free_b = 0, total_b = 0;
        if (hipMemGetInfo(&free_b, &total_b) == hipSuccess && total_b >= (280ull << 30) && total_b <= (290ull << 30)) c->spread_capable = true;
        else (void)hipGetLastError();
    }
    int khz = 0;
    if (hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, device) == hipSuccess && khz > 0) c->wall_khz = khz;
    // this GPU's address of the static row table (sar_run_static), resolved here once, with the device current
    char* static_base = nullptr;
    if (int rc2 = static_scratch(device, &static_base)) { sar_destroy(c); return rc2; }
    *out = c;
    return SAR_OK;
}

void sar_destroy(sar_ctx* c) {
    if (!c) return;
    (void)hipSetDevice(c->device);
    if (c->stream) (void)hipStreamSynchronize(c->stream);
    if (c->prework_stream) (void)hipStreamSynchronize(c->prework_stream);
    drop_ranks(c);
    release_rows(c);
    if (c->pool_attached) sar::pool_detach(c->device, c);        // the last context to go takes the pair along
    for (auto e : c->ev_prof) (void)hipEventDestroy(e);
    if (c->d_flag) (void)hipFree(c->d_flag);
    if (c->ev_start) (void)hipEventDestroy(c->ev_start);
    if (c->ev_stop) (void)hipEventDestroy(c->ev_stop);
    if (c->ev_join) (void)hipEventDestroy(c->ev_join);
    if (c->stream) (void)hipStreamDestroy(c->stream);
    if (c->prework_stream) (void)hipStreamDestroy(c->prework_stream);
    delete c;
}

static int alloc_ranks_body(sar_ctx* c, int n, uint64_t bytes_per_rank, int dtype) {
    if (!c) return set_error(SAR_EINVAL, "context is null");
    if (n < 2 || n > SAR_MAX_RANKS) return set_error(SAR_EINVAL, "n out of range");
    if (dtype != SAR_F32 && dtype != SAR_F16 && dtype != SAR_BF16) return set_error(SAR_EINVAL, "unknown dtype");
    if (bytes_per_rank == 0 || bytes_per_rank % (uint64_t)elem_size_of(dtype)) return set_error(SAR_EINVAL, "bytes_per_rank must be a positive multiple of the element size");
    if (bytes_per_rank > SAR_MAX_RANK_BYTES) return set_error(SAR_EINVAL, "bytes_per_rank is larger than SAR_MAX_RANK_BYTES");
    SAR_HIP(hipSetDevice(c->device));
    SAR_HIP(hipStreamSynchronize(c->stream));
    drop_ranks(c);
    uint64_t stride = (bytes_per_rank + kArenaAlign - 1) / kArenaAlign * kArenaAlign;
    // Spread arena: half the ranks in the other of the GPU's two allocations that were found to lie in different
    // regions of HBM (placed_pool.hpp).  Only for payloads that are bound by memory, and only when the device has the
    // room to look for such a pair; otherwise the ranks sit back to back in an allocation of this context's own.
    const int half = (n + 1) / 2;
    const uint64_t payload = stride * (uint64_t)n;
    int reason = !c->tune.arena_spread ? SAR_SPREAD_OFF : !c->spread_capable ? SAR_SPREAD_UNKNOWN_DEVICE :
                 payload < kSpreadMinPayload ? SAR_SPREAD_SMALL_PAYLOAD : SAR_SPREAD_FOUND;
    if (reason == SAR_SPREAD_FOUND) {
        attach_pool(c);
        reason = sar::pool_lease_arena(probe_env(c), c, stride * (uint64_t)half, stride * (uint64_t)(n - half), &c->arena, &c->arena_hi);
    }
    c->spread_reason = reason;
    if (reason == SAR_SPREAD_FOUND) {
        c->split = half; c->arena_leased = true;
    } else {
        hipError_t e = hipMalloc((void**)&c->arena, payload);
        if (e != hipSuccess && sar::pool_trim(c->device)) {       // the idle pair may be what is in the way
            (void)hipGetLastError();
            e = hipMalloc((void**)&c->arena, payload);
        }
        if (e != hipSuccess) { (void)hipGetLastError(); c->arena = nullptr; return set_error(SAR_ENOMEM, std::string("rank arena: ") + hipGetErrorString(e)); }
        c->arena_hi = nullptr; c->split = n; c->arena_leased = false;
    }
    c->n = n; c->dtype = dtype; c->bytes_per_rank = bytes_per_rank; c->stride = stride;
    return SAR_OK;
}

int sar_alloc_ranks(sar_ctx* c, int n, uint64_t bytes_per_rank, int dtype) {
    return guarded([&] { return alloc_ranks_body(c, n, bytes_per_rank, dtype); });
}

// Caller-owned rank buffers: n device pointers on GPU `device`, element-aligned, each with bytes_per_rank bytes of
// its allocation in front of it, no two overlapping.  Host checks only; nothing is launched or allocated.
static int check_rank_pointers(int device, int n, void* const* device_ptrs, uint64_t bytes_per_rank, int dtype) {
    if (n < 2 || n > SAR_MAX_RANKS) return set_error(SAR_EINVAL, "n out of range");
    if (!device_ptrs) return set_error(SAR_EINVAL, "pointer list is null");
    if (dtype != SAR_F32 && dtype != SAR_F16 && dtype != SAR_BF16) return set_error(SAR_EINVAL, "unknown dtype");
    if (bytes_per_rank == 0 || bytes_per_rank % (uint64_t)elem_size_of(dtype)) return set_error(SAR_EINVAL, "bytes_per_rank must be a positive multiple of the element size");
    if (bytes_per_rank > SAR_MAX_RANK_BYTES) return set_error(SAR_EINVAL, "bytes_per_rank is larger than SAR_MAX_RANK_BYTES");
    for (int r = 0; r < n; ++r) {
        if (!device_ptrs[r]) return set_error(SAR_EINVAL, "a rank pointer is null");
        if ((uintptr_t)device_ptrs[r] % (uintptr_t)elem_size_of(dtype)) return set_error(SAR_EINVAL, "a rank pointer is not aligned to the element size");
        hipPointerAttribute_t at{};
        if (hipPointerGetAttributes(&at, device_ptrs[r]) != hipSuccess || at.type != hipMemoryTypeDevice || at.device != device) {
            (void)hipGetLastError();
            return set_error(SAR_EINVAL, "a rank pointer is not device memory of this context's GPU");
        }
        // the whole of [ptr, ptr + bytes_per_rank) must lie inside the allocation the pointer belongs to: a kernel
        // that writes past it faults the device instead of returning an error
        hipDeviceptr_t base = nullptr; size_t span = 0;
        if (hipMemGetAddressRange(&base, &span, (hipDeviceptr_t)device_ptrs[r]) != hipSuccess) {
            (void)hipGetLastError();
            return set_error(SAR_EINVAL, "a rank pointer does not belong to a device allocation");
        }
        const uint64_t into = (uint64_t)((const char*)device_ptrs[r] - (const char*)base);
        if (into > span || bytes_per_rank > span - into) return set_error(SAR_EINVAL, "a rank buffer is shorter than bytes_per_rank");
        for (int q = 0; q < r; ++q) {
            const char* a = (const char*)device_ptrs[q]; const char* b = (const char*)device_ptrs[r];
            if (a < b + bytes_per_rank && b < a + bytes_per_rank) return set_error(SAR_EINVAL, "rank buffers overlap");
        }
    }
    return SAR_OK;
}

static int adopt_ranks_body(sar_ctx* c, int n, void* const* device_ptrs, uint64_t bytes_per_rank, int dtype) {
    if (!c) return set_error(SAR_EINVAL, "context is null");
    SAR_HIP(hipSetDevice(c->device));
    int rc = check_rank_pointers(c->device, n, device_ptrs, bytes_per_rank, dtype); if (rc) return rc;
    // the context's own arena is given back below: pointers into it would be left dangling
    if (c->arena) {
        const uint64_t lo_span = c->stride * (uint64_t)(c->arena_leased ? c->split : c->n), hi_span = c->stride * (uint64_t)(c->n - c->split);
        for (int r = 0; r < n; ++r) {
            const char* p = (const char*)device_ptrs[r];
            if ((p >= c->arena && p < c->arena + lo_span) || (c->arena_hi && p >= c->arena_hi && p < c->arena_hi + hi_span))
                return set_error(SAR_EINVAL, "a rank pointer lies in this context's own rank arena, which adoption gives back");
        }
    }
    SAR_HIP(hipStreamSynchronize(c->stream));
    drop_ranks(c);
    for (int r = 0; r < n; ++r) c->adopted.push_back((char*)device_ptrs[r]);
    c->n = n; c->dtype = dtype; c->bytes_per_rank = bytes_per_rank; c->stride = 0;
    c->spread_reason = SAR_SPREAD_ADOPTED;
    return SAR_OK;
}

int sar_adopt_ranks(sar_ctx* c, int n, void* const* device_ptrs, uint64_t bytes_per_rank, int dtype) {
    return guarded([&] { return adopt_ranks_body(c, n, device_ptrs, bytes_per_rank, dtype); });
}

// n rows of bytes_per_row bytes back to back in one virtual range; see sar.h.
static int alloc_rows_body(sar_ctx* c, int n, uint64_t bytes_per_row, void** base, int* placed, int* reason_out) {
    if (!c || !base) return set_error(SAR_EINVAL, "null argument");
    *base = nullptr;
    if (placed) *placed = 0;
    if (n < 2 || n > SAR_MAX_RANKS) return set_error(SAR_EINVAL, "n out of range");
    if (bytes_per_row == 0 || bytes_per_row > SAR_MAX_RANK_BYTES) return set_error(SAR_EINVAL, "bytes_per_row out of range");
    SAR_HIP(hipSetDevice(c->device));
    SAR_HIP(hipStreamSynchronize(c->stream));
    SAR_HIP(hipStreamSynchronize(c->prework_stream));
    if (rows_adopted(c)) drop_ranks(c);                       // the rows those rank buffers were go away
    release_rows(c);
    const uint64_t total = (uint64_t)n * bytes_per_row, lo_bytes = (uint64_t)((n + 1) / 2) * bytes_per_row;
    int reason = !c->tune.arena_spread ? SAR_SPREAD_OFF : !c->spread_capable ? SAR_SPREAD_UNKNOWN_DEVICE :
                 total < kSpreadMinPayload ? SAR_SPREAD_SMALL_PAYLOAD : SAR_SPREAD_FOUND;
    if (reason == SAR_SPREAD_FOUND) {
        // rows [0, ceil(n/2)) end where the second allocation begins
        attach_pool(c);
        reason = sar::pool_lease_rows(probe_env(c), c, lo_bytes, total - lo_bytes, &c->rows_base);
    }
    if (reason == SAR_SPREAD_FOUND) {
        c->rows_leased = true;
    } else {
        hipError_t e = hipMalloc((void**)&c->rows_plain, total);
        if (e != hipSuccess && sar::pool_trim(c->device)) { (void)hipGetLastError(); e = hipMalloc((void**)&c->rows_plain, total); }
        if (e != hipSuccess) { (void)hipGetLastError(); c->rows_plain = nullptr; return set_error(SAR_ENOMEM, std::string("rows: ") + hipGetErrorString(e)); }
        c->rows_base = c->rows_plain;
    }
    c->rows_bytes = total;
    *base = c->rows_base;
    if (placed) *placed = reason == SAR_SPREAD_FOUND ? 1 : 0;
    if (reason_out) *reason_out = reason;
    return SAR_OK;
}

int sar_alloc_rows(sar_ctx* c, int n, uint64_t bytes_per_row, void** base, int* placed, int* reason) {
    return guarded([&] { return alloc_rows_body(c, n, bytes_per_row, base, placed, reason); });
}

int sar_free_rows(sar_ctx* c) {
    if (!c) return set_error(SAR_EINVAL, "context is null");
    SAR_HIP(hipSetDevice(c->device));
    SAR_HIP(hipStreamSynchronize(c->stream));
    SAR_HIP(hipStreamSynchronize(c->prework_stream));
    if (rows_adopted(c)) drop_ranks(c);
    release_rows(c);                                          // (the GPU's pair itself stays for the next call)
    return SAR_OK;
}

static int check_rank_range(sar_ctx* c, int rank, uint64_t off, uint64_t bytes) {
    if (!c || !c->has_ranks()) return set_error(SAR_ESTATE, "no rank buffers allocated");
    if (rank < 0 || rank >= c->n) return set_error(SAR_EINVAL, "rank out of range");
    if (off > c->bytes_per_rank || bytes > c->bytes_per_rank - off) return set_error(SAR_EINVAL, "range leaves the rank buffer");
    return SAR_OK;
}

int sar_rank_pointer(sar_ctx* c, int rank, void** device_ptr) {
    int rc = check_rank_range(c, rank, 0, 0); if (rc) return rc;
    if (!device_ptr) return set_error(SAR_EINVAL, "null argument");
    *device_ptr = c->rank_base(rank);
    return SAR_OK;
}

int sar_upload(sar_ctx* c, int rank, uint64_t byte_off, const void* host, uint64_t bytes) {
    int rc = check_rank_range(c, rank, byte_off, bytes); if (rc) return rc;
    if (!host && bytes) return set_error(SAR_EINVAL, "host pointer is null");
    SAR_HIP(hipSetDevice(c->device));
    SAR_HIP(hipStreamSynchronize(c->stream));
    if (bytes) SAR_HIP(hipMemcpy(c->rank_base(rank) + byte_off, host, bytes, hipMemcpyHostToDevice));
    return SAR_OK;
}

int sar_download(sar_ctx* c, int rank, uint64_t byte_off, void* host, uint64_t bytes) {
    int rc = check_rank_range(c, rank, byte_off, bytes); if (rc) return rc;
    if (!host && bytes) return set_error(SAR_EINVAL, "host pointer is null");
    SAR_HIP(hipSetDevice(c->device));
    SAR_HIP(hipStreamSynchronize(c->stream));
    if (bytes) SAR_HIP(hipMemcpy(host, c->rank_base(rank) + byte_off, bytes, hipMemcpyDeviceToHost));
    return SAR_OK;
}

int sar_fill_const(sar_ctx* c, int rank, uint64_t elem_off, uint64_t elems, double value) {
    if (!c || !c->has_ranks()) return set_error(SAR_ESTATE, "no rank buffers allocated");
    const uint64_t es = elem_size_of(c->dtype);
    if (elem_off > c->elems() || elems > c->elems() - elem_off) return set_error(SAR_EINVAL, "range leaves the rank buffer");
    int rc = check_rank_range(c, rank, elem_off * es, elems * es); if (rc) return rc;
    SAR_HIP(hipSetDevice(c->device));
    SAR_HIP(sar::launch_fill_const(c->stream, c->rank_base(rank) + elem_off * es, elems, (float)value, c->dtype));
    SAR_HIP(hipStreamSynchronize(c->stream));
    return SAR_OK;
}

static int fill_reference_pattern_body(sar_ctx* c, const char* alg, float delay_ms, int base) {
    if (!c || !c->has_ranks()) return set_error(SAR_ESTATE, "no rank buffers allocated");
    if (!alg) return set_error(SAR_EINVAL, "alg is null");
    const std::string a(alg);
    if (a != "stragglar" && a != "ring" && a != "rhd" && a != "direct") return set_error(SAR_EINVAL, "unknown algorithm");
    const int n = c->n; const uint64_t elems = c->elems(), es = elem_size_of(c->dtype);
    float presum = 0.f;
    for (int i = 0; i < n - 1; ++i) presum += (float)(i + base);
    const uint64_t chunk = elems / (uint64_t)(n - 1);
    SAR_HIP(hipSetDevice(c->device));
    for (int i = 0; i < n; ++i) {
        float v = (delay_ms < 0 && a == "direct" && i < n - 1) ? presum : (float)(i + base);
        SAR_HIP(sar::launch_fill_const(c->stream, c->rank_base(i), elems, v, c->dtype));
        if (delay_ms < 0 && a == "stragglar" && i < n - 1)
            SAR_HIP(sar::launch_fill_const(c->stream, c->rank_base(i) + (uint64_t)i * chunk * es, chunk, presum, c->dtype));
    }
    SAR_HIP(hipStreamSynchronize(c->stream));
    return SAR_OK;
}

int sar_fill_reference_pattern(sar_ctx* c, const char* alg, float delay_ms, int base) {
    return guarded([&] { return fill_reference_pattern_body(c, alg, delay_ms, base); });
}

static int fill_random(sar_ctx* c, int rank, uint64_t seed, double a, double b, int mode) {
    int rc = check_rank_range(c, rank, 0, 0); if (rc) return rc;
    SAR_HIP(hipSetDevice(c->device));
    uint64_t key = seed * 0xD1B54A32D192ED03ull + (uint64_t)(rank + 1) * 0x8CB92BA72F3D8DD7ull;
    SAR_HIP(sar::launch_fill_random(c->stream, c->rank_base(rank), c->elems(), key, a, b, mode, c->dtype));
    SAR_HIP(hipStreamSynchronize(c->stream));
    return SAR_OK;
}

int sar_fill_uniform(sar_ctx* c, int rank, uint64_t seed, double lo, double hi) { return fill_random(c, rank, seed, lo, hi - lo, 0); }
int sar_fill_normal(sar_ctx* c, int rank, uint64_t seed, double mean, double std) { return fill_random(c, rank, seed, mean, std, 1); }

int sar_snapshot(sar_ctx* c) {
    if (!c || !c->has_ranks()) return set_error(SAR_ESTATE, "no rank buffers allocated");
    SAR_HIP(hipSetDevice(c->device));
    const uint64_t stride = c->snapshot_stride();
    if (!c->snapshot) {
        hipError_t e = hipMalloc((void**)&c->snapshot, stride * (uint64_t)c->n);
        if (e != hipSuccess) { (void)hipGetLastError(); c->snapshot = nullptr; return set_error(SAR_ENOMEM, std::string("snapshot: ") + hipGetErrorString(e)); }
    }
    if (c->adopted.empty() && !c->spread()) {
        SAR_HIP(hipMemcpyAsync(c->snapshot, c->arena, stride * (uint64_t)c->n, hipMemcpyDeviceToDevice, c->stream));
    } else {
        for (int r = 0; r < c->n; ++r)
            SAR_HIP(hipMemcpyAsync(c->snapshot + (uint64_t)r * stride, c->rank_base(r), c->bytes_per_rank, hipMemcpyDeviceToDevice, c->stream));
    }
    SAR_HIP(hipStreamSynchronize(c->stream));
    return SAR_OK;
}

int sar_restore(sar_ctx* c) {
    if (!c || !c->has_ranks() || !c->snapshot) return set_error(SAR_ESTATE, "no snapshot taken");
    SAR_HIP(hipSetDevice(c->device));
    const uint64_t stride = c->snapshot_stride();
    // (a copy kernel of the library's own, with streaming stores: the runtime's copy leaves up to a cache's worth of
    // modified lines in the Infinity Cache, which the timed run that follows would have to push out -- 4 us of a 400 us
    // step at n = 8, 256 MiB per rank)
    for (int r = 0; r < c->n; ++r)
        SAR_HIP(sar::launch_copy(c->stream, c->rank_base(r), c->snapshot + (uint64_t)r * stride, c->bytes_per_rank));
    SAR_HIP(hipStreamSynchronize(c->stream));
    return SAR_OK;
}

int sar_ranks_identical(sar_ctx* c, uint64_t elems, int* identical) {
    if (!c || !c->has_ranks()) return set_error(SAR_ESTATE, "no rank buffers allocated");
    if (!identical || elems > c->elems()) return set_error(SAR_EINVAL, "bad argument");
    SAR_HIP(hipSetDevice(c->device));
    int zero = 0;
    SAR_HIP(hipMemcpyAsync(c->d_flag, &zero, sizeof(int), hipMemcpyHostToDevice, c->stream));
    for (int r = 1; r < c->n; ++r)
        SAR_HIP(sar::launch_compare(c->stream, c->rank_base(0), c->rank_base(r), elems * (uint64_t)elem_size_of(c->dtype), c->d_flag));
    int flag = 0;
    SAR_HIP(hipMemcpyAsync(&flag, c->d_flag, sizeof(int), hipMemcpyDeviceToHost, c->stream));
    SAR_HIP(hipStreamSynchronize(c->stream));
    *identical = flag ? 0 : 1;
    return SAR_OK;
}

int sar_get_tuning(sar_ctx* c, sar_tuning_t* out) {
    if (!c || !out) return set_error(SAR_EINVAL, "null argument");
    *out = c->tune; return SAR_OK;
}

int sar_set_tuning(sar_ctx* c, const sar_tuning_t* in) {
    if (!c || !in) return set_error(SAR_EINVAL, "null argument");
    if (!valid_tuning(*in)) return set_error(SAR_EINVAL, "tuning value out of range");
    // A prepared plan was lowered for the old values (tile counts, launch shapes, a captured graph): it goes, and
    // sar_run reports SAR_ESTATE until the next sar_prepare.
    if (c->prepared) {
        SAR_HIP(hipSetDevice(c->device));
        SAR_HIP(hipStreamSynchronize(c->stream));
        drop_plan(c);
    }
    c->tune = *in; return SAR_OK;
}

static int prepare_body(sar_ctx* c, const sar_schedule* prework, const sar_schedule* main_sched, int use_graph) {
    if (!c || !c->has_ranks()) return set_error(SAR_ESTATE, "no rank buffers allocated");
    if (!main_sched) return set_error(SAR_EINVAL, "main schedule is null");
    for (const sar_schedule* s : {prework, main_sched}) {
        if (!s) continue;
        if (s->s.n != c->n) return set_error(SAR_EINVAL, "schedule and context disagree on the rank count");
        std::string why = sar::validate(s->s);
        if (!why.empty()) return set_error(SAR_ESCHED, why);
    }
    SAR_HIP(hipSetDevice(c->device));
    SAR_HIP(hipStreamSynchronize(c->stream));
    drop_plan(c);
    std::vector<sar::DevOp> rows; std::vector<char*> ptrs;
    HostPlans hp;
    int rc = plan_on_host(c, prework, main_sched, rows, ptrs, hp);
    if (rc != SAR_OK) { drop_plan(c); return rc; }
    if (!rows.empty()) {
        SAR_HIP(hipMalloc((void**)&c->d_ops, rows.size() * sizeof(sar::DevOp)));
        SAR_HIP(hipMemcpy(c->d_ops, rows.data(), rows.size() * sizeof(sar::DevOp), hipMemcpyHostToDevice));
    }
    SAR_HIP(hipMalloc((void**)&c->d_ptrs, (ptrs.size() + 1) * sizeof(char*)));
    if (!ptrs.empty()) SAR_HIP(hipMemcpy(c->d_ptrs, ptrs.data(), ptrs.size() * sizeof(char*), hipMemcpyHostToDevice));

    if (hp.want_column) {
        if ((rc = upload_column_plan(c, hp.cp, hp.col_first, c->col)) != SAR_OK) { drop_plan(c); return rc; }
        c->column = true;
        if (hp.want_fused && (rc = upload_column_plan(c, hp.fp, hp.fused_first, c->fused)) != SAR_OK) { drop_plan(c); return rc; }
    }
    if (hp.want_pre && (rc = upload_column_plan(c, hp.pp, hp.pre_first, c->pre)) != SAR_OK) { drop_plan(c); return rc; }

    sar_stats_t st = plan_stats(c, prework, main_sched, hp.cp, c->column, c->fused.ready, c->pre.ready, &hp.fp);
    if (use_graph) {
        // the main rounds as one graph, and the single launch of pre-work + schedule (what sar_run with delay 0
        // runs) as another: kernel nodes only (no memset nodes)
        for (int which = 0; which < (c->fused.ready ? 2 : 1); ++which) {
            hipGraph_t* g = which ? &c->graph_fused : &c->graph;
            hipGraphExec_t* ge = which ? &c->graph_fused_exec : &c->graph_exec;
            hipError_t e = hipStreamBeginCapture(c->stream, hipStreamCaptureModeThreadLocal);
            if (e != hipSuccess) { drop_plan(c); return set_error(SAR_EHIP, std::string("hipStreamBeginCapture: ") + hipGetErrorString(e)); }
            rc = which ? launch_column_plan(c, c->fused) : launch_main(c);
            e = hipStreamEndCapture(c->stream, g);
            if (rc != SAR_OK) { drop_plan(c); return rc; }
            if (e != hipSuccess) { drop_plan(c); return set_error(SAR_EHIP, std::string("hipStreamEndCapture: ") + hipGetErrorString(e)); }
            e = hipGraphInstantiate(ge, *g, nullptr, nullptr, 0);
            if (e != hipSuccess) { drop_plan(c); return set_error(SAR_EHIP, std::string("hipGraphInstantiate: ") + hipGetErrorString(e)); }
        }
        st.uses_graph = 1;
    }
    c->stats = st;
    c->prepared = true;
    return SAR_OK;
}

int sar_prepare(sar_ctx* c, const sar_schedule* prework, const sar_schedule* main_sched, int use_graph) {
    return guarded([&] { return prepare_body(c, prework, main_sched, use_graph); });
}

int sar_run(sar_ctx* c, float delay_ms, float* elapsed_ms) {
    if (!c || !c->prepared) return set_error(SAR_ESTATE, "sar_prepare has not succeeded");
    if (!(delay_ms <= kMaxDelayMs)) return set_error(SAR_EINVAL, "delay out of range");
    SAR_HIP(hipSetDevice(c->device));
    SAR_HIP(hipEventRecord(c->ev_start, c->stream));
    bool main_done = false;
    if (delay_ms == 0 && c->fused.ready) {
        // nobody is late: pre-work and schedule as the one launch planned for this case
        if (c->graph_fused_exec) SAR_HIP(hipGraphLaunch(c->graph_fused_exec, c->stream));
        else { int rc = launch_column_plan(c, c->fused); if (rc) return rc; }
        main_done = true;
    } else if (delay_ms == 0) {
        // nobody is late: pre-work, then the schedule, on one stream
        int rc = c->pre.ready ? launch_column_plan(c, c->pre) : launch_all(c, c->prework); if (rc) return rc;
    } else if (delay_ms > 0) {
        // The straggler is busy for delay_ms (gpu_sleep_kernel on its stream, allreduce_8GPU.cu:876-889) while the
        // others do their pre-work.  Here the wait sits on the stream that goes on to run the schedule and the
        // pre-work on the second one: a pre-work that hides behind the delay has signalled its event long before
        // the sleep ends, and the schedule starts right behind the sleep kernel (about 5 us sooner after the
        // straggler's arrival than with the join of the two streams on the critical path).
        const uint64_t ticks = (uint64_t)((double)delay_ms * (double)c->wall_khz);
        SAR_HIP(hipStreamWaitEvent(c->prework_stream, c->ev_start, 0));
        int rc = c->pre.ready ? launch_column_plan(c, c->pre, c->prework_stream) : launch_all(c, c->prework, c->prework_stream); if (rc) return rc;
        SAR_HIP(hipEventRecord(c->ev_join, c->prework_stream));
        SAR_HIP(sar::launch_sleep(c->stream, ticks));
        SAR_HIP(hipStreamWaitEvent(c->stream, c->ev_join, 0));
    }
    if (main_done) {}
    else if (c->graph_exec) SAR_HIP(hipGraphLaunch(c->graph_exec, c->stream));
    else { int rc = launch_main(c); if (rc) return rc; }
    SAR_HIP(hipEventRecord(c->ev_stop, c->stream));
    SAR_HIP(hipEventSynchronize(c->ev_stop));
    if (delay_ms > 0) SAR_HIP(hipStreamSynchronize(c->prework_stream));
    float ms = 0.f;
    SAR_HIP(hipEventElapsedTime(&ms, c->ev_start, c->ev_stop));
    if (elapsed_ms) *elapsed_ms = ms;
    return SAR_OK;
}

static int run_profiled_body(sar_ctx* c, float* ms, int cap, int* count) {
    if (!c || !c->prepared) return set_error(SAR_ESTATE, "sar_prepare has not succeeded");
    if (cap < 0 || (cap > 0 && !ms)) return set_error(SAR_EINVAL, "bad argument");
    SAR_HIP(hipSetDevice(c->device));
    if (c->column) {
        while (c->ev_prof.size() < 2) { hipEvent_t e; SAR_HIP(hipEventCreate(&e)); c->ev_prof.push_back(e); }
        SAR_HIP(hipEventRecord(c->ev_prof[0], c->stream));
        int rc = launch_column_plan(c, c->col); if (rc) return rc;
        SAR_HIP(hipEventRecord(c->ev_prof[1], c->stream));
        SAR_HIP(hipStreamSynchronize(c->stream));
        if (cap > 0) SAR_HIP(hipEventElapsedTime(&ms[0], c->ev_prof[0], c->ev_prof[1]));
        if (count) *count = 1;
        return SAR_OK;
    }
    std::vector<const Launch*> ls;
    for (const auto& L : c->rounds) if (L.total_tiles) ls.push_back(&L);
    while (c->ev_prof.size() < ls.size() + 1) {
        hipEvent_t e; SAR_HIP(hipEventCreate(&e)); c->ev_prof.push_back(e);
    }
    SAR_HIP(hipEventRecord(c->ev_prof[0], c->stream));
    for (size_t i = 0; i < ls.size(); ++i) {
        int rc = launch_one(c, *ls[i]); if (rc) return rc;
        SAR_HIP(hipEventRecord(c->ev_prof[i + 1], c->stream));
    }
    SAR_HIP(hipStreamSynchronize(c->stream));
    for (size_t i = 0; i < ls.size() && (int)i < cap; ++i) SAR_HIP(hipEventElapsedTime(&ms[i], c->ev_prof[i], c->ev_prof[i + 1]));
    if (count) *count = (int)ls.size();
    return SAR_OK;
}

int sar_run_profiled(sar_ctx* c, float* ms, int cap, int* count) {
    return guarded([&] { return run_profiled_body(c, ms, cap, count); });
}

int sar_launch_bytes(sar_ctx* c, uint64_t* bytes, int cap, int* count) {
    if (!c || !c->prepared) return set_error(SAR_ESTATE, "sar_prepare has not succeeded");
    if (cap < 0 || (cap > 0 && !bytes)) return set_error(SAR_EINVAL, "bad argument");
    int k = 0;
    if (c->column) {
        if (cap > 0) bytes[0] = c->stats.algorithmic_bytes;
        if (count) *count = 1;
        return SAR_OK;
    }
    for (const auto& L : c->rounds) {
        if (!L.total_tiles) continue;
        if (k < cap) bytes[k] = L.algorithmic_bytes;
        ++k;
    }
    if (count) *count = k;
    return SAR_OK;
}

static int probe_streams_body(sar_ctx* c, int njobs, const sar_probe_job* jobs, uint64_t bytes, int reps, sar_probe_result* out) {
    if (!c || !c->has_ranks()) return set_error(SAR_ESTATE, "no rank buffers allocated");
    if (!jobs || !out || njobs < 1 || njobs > 8 || reps < 1 || reps > 1000) return set_error(SAR_EINVAL, "bad argument");
    if (bytes < 16 || (bytes & 15u)) return set_error(SAR_EINVAL, "bytes must be a positive multiple of 16");
    sar::ProbeJobs J{};
    J.njobs = (uint32_t)njobs; J.bytes = bytes;
    uint64_t moved = 0;
    for (int j = 0; j < njobs; ++j) {
        const sar_probe_job& b = jobs[j];
        if (b.nread < 0 || b.nread > 8 || b.nwrite < 0 || b.nwrite > 8 || b.nread + b.nwrite == 0 || b.nread != jobs[0].nread)
            return set_error(SAR_EINVAL, "a job has 0 to 8 read and 0 to 8 written streams, and all jobs read equally many");
        if (b.byte_off > c->bytes_per_rank || bytes > c->bytes_per_rank - b.byte_off) return set_error(SAR_EINVAL, "a job leaves the rank buffer");
        J.nread[j] = (uint32_t)b.nread; J.nwrite[j] = (uint32_t)b.nwrite;
        for (int k = 0; k < b.nread + b.nwrite; ++k) {
            const int rank = k < b.nread ? b.read_rank[k] : b.write_rank[k - b.nread];
            if (rank < 0 || rank >= c->n) return set_error(SAR_EINVAL, "rank out of range");
            char* p = c->rank_base(rank) + b.byte_off;
            if ((uintptr_t)p & 15u) return set_error(SAR_EINVAL, "a stream does not start on a 16-byte boundary");
            if (k < b.nread) J.rd[j][k] = p; else J.wr[j][k - b.nread] = p;
        }
        moved += (uint64_t)(b.nread + b.nwrite) * bytes;
    }
    SAR_HIP(hipSetDevice(c->device));
    while (c->ev_prof.size() < 2) { hipEvent_t e; SAR_HIP(hipEventCreate(&e)); c->ev_prof.push_back(e); }
    *out = sar_probe_result{};
    out->bytes_moved = moved;
    for (int block : {256, 512, 1024})
        for (int unroll : {1, 2, 4})
            for (int nt = 0; nt < 3; ++nt)
                for (int persistent = 0; persistent < 2; ++persistent)
                    for (int interleave = 0; interleave < (njobs > 1 ? 2 : 1); ++interleave) {
                        float best = -1.f;
                        for (int r = 0; r <= reps; ++r) {                   // the first run warms up and is not counted
                            SAR_HIP(hipEventRecord(c->ev_prof[0], c->stream));
                            SAR_HIP(sar::launch_stream_probe(c->stream, J, block, unroll, nt, persistent != 0, interleave != 0, c->cu_count));
                            SAR_HIP(hipEventRecord(c->ev_prof[1], c->stream));
                            SAR_HIP(hipEventSynchronize(c->ev_prof[1]));
                            float ms = 0.f;
                            SAR_HIP(hipEventElapsedTime(&ms, c->ev_prof[0], c->ev_prof[1]));
                            if (r > 0 && (best < 0.f || ms < best)) best = ms;
                        }
                        if (out->variants < 108) out->variant_ms[out->variants] = best;
                        out->variants += 1;
                        if (out->best_ms <= 0.f || best < out->best_ms) {
                            out->best_ms = best; out->block = block; out->unroll = unroll; out->nontemporal = nt;
                            out->persistent = persistent; out->interleave = interleave;
                        }
                        if (best > out->worst_ms) out->worst_ms = best;
                    }
    return SAR_OK;
}

int sar_spread_yardstick(const float* neighbours_ms, float ends_ms, float* yardstick_ms) {
    if (!neighbours_ms || !yardstick_ms) return set_error(SAR_EINVAL, "null argument");
    if (!(neighbours_ms[0] > 0.f && neighbours_ms[1] > 0.f && neighbours_ms[2] > 0.f && ends_ms > 0.f)) return set_error(SAR_EINVAL, "probe times must be positive");
    return sar::spread_yardstick(neighbours_ms, ends_ms, yardstick_ms) ? 0 : 1;
}

int sar_spread_is_elsewhere(float yardstick_ms, float probe_ms_value) {
    if (!(yardstick_ms > 0.f)) return set_error(SAR_EINVAL, "the yardstick must be positive");
    return sar::spread_is_elsewhere(yardstick_ms, probe_ms_value) ? 1 : 0;
}

int sar_spread_pick(float yardstick_ms, const float* probe_ms, int n, int* pick) {
    if (!(yardstick_ms > 0.f) || !probe_ms || n < 0 || !pick) return set_error(SAR_EINVAL, "bad argument");
    *pick = n ? sar::spread_pick(yardstick_ms, probe_ms, n) : -1;
    return *pick >= 0 ? 1 : 0;
}

int sar_probe_streams(sar_ctx* c, int njobs, const sar_probe_job* jobs, uint64_t bytes, int reps, sar_probe_result* out) {
    return guarded([&] { return probe_streams_body(c, njobs, jobs, bytes, reps, out); });
}

int sar_sleep_ticks(sar_ctx* c, float delay_ms, int64_t* ticks) {
    if (!c || !ticks) return set_error(SAR_EINVAL, "null argument");
    if (!(delay_ms >= 0) || !(delay_ms <= kMaxDelayMs)) return set_error(SAR_EINVAL, "delay out of range");
    *ticks = (int64_t)((double)delay_ms * (double)c->wall_khz);
    return SAR_OK;
}

int sar_stats(sar_ctx* c, sar_stats_t* out) {
    if (!c || !out) return set_error(SAR_EINVAL, "null argument");
    if (!c->prepared) return set_error(SAR_ESTATE, "sar_prepare has not succeeded");
    *out = c->stats; return SAR_OK;
}

int sar_default_tuning(sar_tuning_t* out) {
    if (!out) return set_error(SAR_EINVAL, "null argument");
    *out = sar_ctx().tune; return SAR_OK;
}

static int plan_body(const sar_schedule* prework, const sar_schedule* main_sched, int n, uint64_t bytes_per_rank, int dtype,
             const sar_tuning_t* tuning, int compute_units, sar_stats_t* out) {
    if (!out) return set_error(SAR_EINVAL, "null argument");
    HostPlan hp;
    const int rc = hp.make(prework, main_sched, n, bytes_per_rank, dtype, tuning, compute_units);
    if (rc != SAR_OK) return rc;
    *out = plan_stats(&hp.c, prework, main_sched, hp.hp.cp, hp.hp.want_column, hp.hp.want_column && hp.hp.want_fused, hp.hp.want_pre, &hp.hp.fp);
    return SAR_OK;
}

int sar_plan(const sar_schedule* prework, const sar_schedule* main_sched, int n, uint64_t bytes_per_rank, int dtype,
             const sar_tuning_t* tuning, int compute_units, sar_stats_t* out) {
    return guarded([&] { return plan_body(prework, main_sched, n, bytes_per_rank, dtype, tuning, compute_units, out); });
}

static int plan_rows_body(const sar_schedule* prework, const sar_schedule* main_sched, int n, uint64_t bytes_per_rank, int dtype,
                  const sar_tuning_t* tuning, int compute_units, int same_launch,
                  sar_plan_row* out_rows, int row_cap, int* nrows, sar_plan_ptr* out_ptrs, int ptr_cap, int* nptrs) {
    if (!nrows || !nptrs || (row_cap > 0 && !out_rows) || (ptr_cap > 0 && !out_ptrs) || row_cap < 0 || ptr_cap < 0)
        return set_error(SAR_EINVAL, "null argument");
    HostPlan hp;
    const int rc = hp.make(prework, main_sched, n, bytes_per_rank, dtype, tuning, compute_units);
    if (rc != SAR_OK) return rc;
    const ColumnPlan& cp = same_launch == 2 ? hp.hp.pp : same_launch ? hp.hp.fp : hp.hp.cp;
    const size_t first = same_launch == 2 ? hp.hp.pre_first : same_launch ? hp.hp.fused_first : hp.hp.col_first;
    const size_t count = cp.group_begin.empty() ? 0 : cp.group_begin.back();
    if (cp.unsupported || count == 0 || first + count > hp.rows.size())
        return set_error(SAR_ESTATE, same_launch == 2 ? "no column plan for the pre-work alone" : same_launch ? "no plan for pre-work and schedule in one launch" : "no column plan for this schedule and tuning");
    auto locate = [&](const char* p, int32_t* rank, uint64_t* off) {
        const uint64_t d = (uint64_t)(p - hp.c.adopted[0]);
        *rank = (int32_t)(d / hp.stride); *off = d % hp.stride;
    };
    *nrows = (int)count; *nptrs = (int)hp.ptrs.size();
    for (size_t k = 0; k < hp.ptrs.size() && k < (size_t)ptr_cap; ++k) { out_ptrs[k] = sar_plan_ptr{}; locate(hp.ptrs[k], &out_ptrs[k].rank, &out_ptrs[k].off); }
    for (size_t comp = 0; comp < cp.comps.size(); ++comp) {
        for (uint32_t g = cp.comps[comp].group_first; g < cp.comps[comp].group_end; ++g) {
            for (uint32_t i = cp.group_begin[g]; i < cp.group_begin[g + 1] && i < (uint32_t)row_cap; ++i) {
                const sar::DevOp& d = hp.rows[first + i];
                sar_plan_row r{};
                r.kind = (int32_t)d.kind; r.component = (int32_t)comp; r.group = (int32_t)(g - cp.comps[comp].group_first);
                r.vector = (d.flags & sar::DEVOP_VEC) ? 1 : 0;
                r.bytes = d.bytes; r.head_bytes = (int32_t)(d.flags >> sar::DEVOP_HEAD_SHIFT & 15u);
                r.get0_slot = (d.flags & sar::DEVOP_GET0) ? (int32_t)(d.slots & 0xffu) : -1;
                r.get1_slot = (d.flags & sar::DEVOP_GET1) ? (int32_t)(d.slots >> 8 & 0xffu) : -1;
                r.put_slot = (d.flags & sar::DEVOP_PUT) ? (int32_t)(d.slots >> 16 & 0xffu) : -1;
                r.dead0 = (d.flags & sar::DEVOP_DEAD0) ? 1 : 0; r.dead1 = (d.flags & sar::DEVOP_DEAD1) ? 1 : 0;
                r.joins = (d.flags & sar::DEVOP_JOIN) ? 1 : 0;
                if (d.kind == SAR_OP_MREDUCE) {
                    r.dst_rank = r.src_rank = -1;
                    r.nsrc = (int32_t)d.nsrc; r.ndst = (int32_t)d.ndst; r.first_ptr = (int32_t)d.ptr_off;
                } else {
                    locate(d.p0, &r.dst_rank, &r.dst_off);
                    locate(d.p1, &r.src_rank, &r.src_off);
                    r.ndst = (int32_t)d.ndst; r.first_ptr = (int32_t)d.ptr_off;      // extra destinations
                }
                out_rows[i] = r;
            }
        }
    }
    return SAR_OK;
}

int sar_plan_rows(const sar_schedule* prework, const sar_schedule* main_sched, int n, uint64_t bytes_per_rank, int dtype,
                  const sar_tuning_t* tuning, int compute_units, int same_launch,
                  sar_plan_row* out_rows, int row_cap, int* nrows, sar_plan_ptr* out_ptrs, int ptr_cap, int* nptrs) {
    return guarded([&] { return plan_rows_body(prework, main_sched, n, bytes_per_rank, dtype, tuning, compute_units, same_launch, out_rows, row_cap, nrows, out_ptrs, ptr_cap, nptrs); });
}

}  // extern "C"

// ---- an entry point that allocates nothing ---------------------------------------------------------------

namespace {

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
char* g_scratch_ptr[kMaxDevices] = {};      // device address of `scratch` on every GPU it was resolved on
std::mutex g_static_run_mutex[kMaxDevices]; // one sar_run_static at a time per GPU: they all write the one array

// The address of this GPU's copy of `scratch`, resolved once per device with that device current.
int static_scratch(int device, char** out) {
    if (device < 0 || device >= kMaxDevices) return set_error(SAR_EINVAL, "device index out of range");
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[device]) {
        SAR_HIP(hipSetDevice(device));
        void* p = nullptr;
        SAR_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (!p) return set_error(SAR_EHIP, "hipGetSymbolAddress returned no address for the static row table");
        g_scratch_ptr[device] = (char*)p;
    }
    *out = g_scratch_ptr[device];
    return SAR_OK;
}

int run_static_body(int device, void* stream, const sar_schedule* prework, const sar_schedule* main_sched, int n,
                    void* const* device_ptrs, uint64_t bytes_per_rank, int dtype) {
    if (!main_sched) return set_error(SAR_EINVAL, "main schedule is null");
    int count = 0;
    int rc = sar_device_count(&count); if (rc) return rc;
    if (device < 0 || device >= count) return set_error(SAR_EINVAL, "device index out of range");
    SAR_HIP(hipSetDevice(device));
    if ((rc = check_rank_pointers(device, n, device_ptrs, bytes_per_rank, dtype)) != SAR_OK) return rc;
    for (const sar_schedule* s : {prework, main_sched}) {
        if (!s) continue;
        if (s->s.n != n) return set_error(SAR_EINVAL, "schedule and rank count disagree");
        std::string why = sar::validate(s->s);
        if (!why.empty()) return set_error(SAR_ESCHED, why);
    }
    char* base = nullptr;
    if ((rc = static_scratch(device, &base)) != SAR_OK) return rc;

    // a context that lives on the host only: the caller's buffers and stream, the default tuning, no device objects
    sar_ctx c;
    c.device = device; c.stream = (hipStream_t)stream;
    c.n = n; c.dtype = dtype; c.bytes_per_rank = bytes_per_rank;
    for (int r = 0; r < n; ++r) c.adopted.push_back((char*)device_ptrs[r]);
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) == hipSuccess && cus > 0) c.cu_count = cus;
    else { (void)hipGetLastError(); c.cu_count = 256; }

    std::vector<sar::DevOp> rows; std::vector<char*> ptrs;
    HostPlans hp;
    if ((rc = plan_on_host(&c, prework, main_sched, rows, ptrs, hp)) != SAR_OK) return rc;
    const ColumnPlan& cp = hp.cp; const ColumnPlan& fp = hp.fp;
    const uint32_t col_first = hp.col_first, fused_first = hp.fused_first;
    const bool want_column = hp.want_column, want_fused = hp.want_fused;

    // what runs: pre-work and schedule in one launch, or the pre-work's launches followed by the schedule's (one
    // column launch, or one launch per round)
    const bool one_launch = want_column && want_fused;
    const ColumnPlan* col = one_launch ? &fp : want_column ? &cp : nullptr;
    const uint32_t col_rows_first = one_launch ? fused_first : col_first;
    std::vector<Launch> per_round;
    if (!one_launch) per_round = c.prework;
    if (!want_column) per_round.insert(per_round.end(), c.rounds.begin(), c.rounds.end());

    // the part of the row table that these launches read
    uint64_t lo = rows.size(), hi = 0;
    for (const Launch& L : per_round) if (L.total_tiles) { lo = std::min<uint64_t>(lo, L.first_op); hi = std::max<uint64_t>(hi, (uint64_t)L.first_op + L.nops); }
    if (col) { lo = std::min<uint64_t>(lo, col_rows_first); hi = std::max<uint64_t>(hi, (uint64_t)col_rows_first + col->group_begin.back()); }
    if (hi <= lo) return SAR_OK;                // buffers shorter than `parts` elements: nothing moves

    // layout in the static array: [rows][pointer lists][group boundaries][components], each on a 256-byte boundary
    auto up = [](uint64_t v) { return (v + 255u) & ~(uint64_t)255u; };
    const uint64_t rows_b = (hi - lo) * sizeof(sar::DevOp), ptrs_b = ptrs.size() * sizeof(char*);
    const uint64_t grp_b = col ? col->group_begin.size() * sizeof(uint32_t) : 0, comp_b = col ? col->comps.size() * sizeof(sar::ColumnComp) : 0;
    const uint64_t ptrs_at = up(rows_b), grp_at = ptrs_at + up(ptrs_b), comp_at = grp_at + up(grp_b), need = comp_at + up(comp_b);
    if (need > SAR_STATIC_SCRATCH_BYTES)
        return set_error(SAR_EINVAL, "the schedule's row tables take " + std::to_string(need) + " bytes, the static array of sar_run_static holds " +
                                         std::to_string((uint64_t)SAR_STATIC_SCRATCH_BYTES) + " (use sar_prepare / sar_run)");
    hipStream_t st = c.stream;
    c.d_ops = (sar::DevOp*)base; c.d_ptrs = (char**)(base + ptrs_at);
    for (Launch& L : per_round) L.first_op -= (uint32_t)lo;
    // Copies and launches on the caller's stream.  Whatever happens, the stream is drained before the host copies of
    // the tables go out of scope; the result is complete when it has.  Every call on this GPU writes the same array
    // and its kernels read it until the stream has drained, so the calls take turns: the lock is held from the first
    // copy until the drain (a second thread's call waits here; nothing is lost, the call blocks on its stream anyway).
    std::lock_guard<std::mutex> turn(g_static_run_mutex[device]);
    auto enqueue = [&]() -> int {
        SAR_HIP(hipMemcpyAsync(base, rows.data() + lo, rows_b, hipMemcpyHostToDevice, st));
        if (ptrs_b) SAR_HIP(hipMemcpyAsync(base + ptrs_at, ptrs.data(), ptrs_b, hipMemcpyHostToDevice, st));
        int e = launch_all(&c, per_round, st); if (e) return e;
        if (col) {
            SAR_HIP(hipMemcpyAsync(base + grp_at, col->group_begin.data(), grp_b, hipMemcpyHostToDevice, st));
            SAR_HIP(hipMemcpyAsync(base + comp_at, col->comps.data(), comp_b, hipMemcpyHostToDevice, st));
            ColumnDevice d;
            if ((e = shape_column_plan(&c, *col, col_rows_first - (uint32_t)lo, d)) != SAR_OK) return e;
            d.d_group_begin = (uint32_t*)(base + grp_at); d.d_comps = (sar::ColumnComp*)(base + comp_at);
            if ((e = launch_column_plan(&c, d)) != SAR_OK) return e;
        }
        return SAR_OK;
    };
    // The caller may have a stream capture open in this thread, or another thread one in global mode: both refuse
    // "potentially unsafe" calls, hipStreamSynchronize among them, also on streams that are not being captured.
    // Nothing here touches a capturing stream (`st` must not be one), so the thread takes relaxed mode for the call.
    hipStreamCaptureMode mode = hipStreamCaptureModeRelaxed;
    const bool relaxed = hipThreadExchangeStreamCaptureMode(&mode) == hipSuccess;
    if (!relaxed) (void)hipGetLastError();
    rc = enqueue();
    const hipError_t drained = hipStreamSynchronize(st);
    if (relaxed) (void)hipThreadExchangeStreamCaptureMode(&mode);
    if (rc != SAR_OK) return rc;
    if (drained != hipSuccess) return set_error(SAR_EHIP, std::string("hipStreamSynchronize: ") + hipGetErrorString(drained));
    return SAR_OK;
}

}  // namespace

extern "C" int sar_run_static(int device, void* stream, const sar_schedule* prework, const sar_schedule* main_sched, int n,
                              void* const* device_ptrs, uint64_t bytes_per_rank, int dtype) {
    return guarded([&] { return run_static_body(device, stream, prework, main_sched, n, device_ptrs, bytes_per_rank, dtype); });
}

extern "C" uint64_t sar_static_scratch_bytes(void) { return SAR_STATIC_SCRATCH_BYTES; }
