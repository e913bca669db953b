// Host-side planner of the column executor: turns schedules into the row table, components, value-slot
// flags and launch shape that column_kernel runs.  Pure host code: it needs addresses, not a device.
#pragma once
#include <stdint.h>

#include <string>
#include <vector>

#include "kernels.hpp"
#include "sar.h"
#include "schedule.hpp"

namespace sar {

// What the planner needs to know of a context.
struct ColumnEnv {
    sar_tuning_t tune;
    int n = 0;
    int elem_size = 4;
    uint64_t elems = 0;               // per rank
    uint64_t bytes_per_rank = 0;
    int compute_units = 1;
    std::vector<char*> rank_base;     // device address of every rank's buffer
};

// Column plan: every row of the schedules, cut into single-chunk rows (all rows then share one within-chunk
// offset space), sorted into components and, within a component, into groups of one round each.
//
// Value forwarding.  A lane of the column kernel meets the same (rank, chunk) cells again and again: what
// round r writes, later rounds read back.  The kernel can keep up to `nslots` such values per lane in LDS,
// and which read finds its operand there is decided here, on the host, by running the slot bookkeeping over
// the rows once: a slot stands for one value and the set of cells that currently equal it (a COPY from a
// held value adds its destination to the set at no cost; a write to a cell takes it out of its old set).
// When all slots are busy the value whose next use is furthest away gives way, which is known exactly
// because the whole schedule is.  Rows get DEVOP_GET0 / GET1 / PUT and their slot numbers, and DEVOP_DEAD0 /
// DEAD1 where a stored value is overwritten before anybody loads it.
struct ColumnPlan {
    std::vector<uint32_t> group_begin;       // first row of every group (rows of one component and one round), plus the end
    std::vector<ColumnComp> comps;
    uint32_t max_comp_rows = 0, max_comp_groups = 0;
    uint64_t widest_row = 0;
    int block = 512;
    uint32_t nslots = 0;
    uint64_t forwarded_bytes = 0;    // operand bytes taken from value slots instead of memory, per run
    uint64_t elided_bytes = 0;       // result bytes not stored because they are overwritten unread, per run
    bool lane_local = false;         // every row 16-byte aligned and a whole number of vectors long
    bool staged = false;             // latency plan: a workgroup copies the rows of its component into LDS first
    uint32_t policy = 0;             // cache policy of the launch: 0 cached, 1 streaming loads, 2 streaming loads and stores
    bool unsupported = false;        // the rows cannot all run in the column kernel
    bool multi_source = false;       // some rows are MREDUCE rows
    bool component_major = false;    // dispatch order of the items: all columns of a component, then the next component
    bool two_vectors = false;        // with value slots, outside the latency plan: a lane moves two vectors per row (else one)
    uint64_t column_bytes() const { return sar::column_bytes(block, two_vectors); }
};

// `scheds`: the schedules to run back to back in the one launch (the main schedule, or pre-work + main); they
// share `parts`.  Multi-source rows (pre-work) are only taken when every pointer is 16-byte aligned and the row
// is a whole number of vectors long; otherwise plan.unsupported is set and the caller keeps the pre-work as
// launches of its own.  The rows are appended to `rows`, the pointer lists of multi-source rows to `ptrs`.
// Returns SAR_OK, or an error code with its message in *error.
int plan_columns(const ColumnEnv& env, const std::vector<const Schedule*>& scheds, std::vector<DevOp>& rows,
                 std::vector<char*>& ptrs, ColumnPlan& plan, std::string* error);

}  // namespace sar
