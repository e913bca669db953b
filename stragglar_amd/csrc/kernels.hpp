// Interface between the host executor and the gfx950 device code.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "sar.h"

namespace sar {

enum : uint32_t {
    // cache policy per row, honoured by the round and multi-source kernels (the column kernel has one policy per launch)
    DEVOP_LNT = 1u,    // loads are streaming (nontemporal)
    DEVOP_SNT0 = 2u,   // stores to p0 (or to every MREDUCE destination) are streaming
    DEVOP_SNT1 = 4u,   // stores to p1 are streaming (XREDUCE only)
    DEVOP_VEC = 8u,    // every pointer of the row is 16-byte aligned
    DEVOP_GET0 = 16u,  // column executor: p0's current value is in value slot (slots & 0xff)
    DEVOP_GET1 = 32u,  // column executor: p1's current value is in value slot (slots >> 8 & 0xff)
    DEVOP_PUT = 64u,   // column executor: keep the row's result in value slot (slots >> 16 & 0xff)
    DEVOP_DEAD0 = 128u,    // column executor: the whole vectors stored to p0 (MREDUCE: to every destination) are
                           // overwritten before anybody loads them (every reader in between takes the value from
                           // a slot): not stored
    DEVOP_DEAD1 = 4096u,   // the same for p1 (XREDUCE)
    DEVOP_JOIN = 8192u,    // column executor, plan for few work items: the row takes its operands together with the
                           // row before it (same group; it needs neither that row's result nor that of any row
                           // the one before joined), and the sums and stores follow in row order
    DEVOP_HEAD_SHIFT = 8u  // column executor: flags >> 8 & 15 = bytes of the row that lie before p0 and p1 (both moved
                           // up to the next 16-byte boundary; `bytes` counts from there)
};

// One lowered row of a round, read by the kernel through scalar loads.
struct DevOp {
    char* p0;             // COPY/REDUCE_INTO: destination; XREDUCE: first side; MREDUCE: unused
    char* p1;             // COPY/REDUCE_INTO: source; XREDUCE: second side; MREDUCE: unused
    uint64_t bytes;       // length of the row
    uint32_t kind;        // SAR_OP_*
    uint32_t flags;       // DEVOP_*
    uint32_t tile_begin;  // first tile of this row within its round
    uint32_t ntiles;
    uint32_t nsrc;        // MREDUCE: sources, in add order
    uint32_t ndst;        // MREDUCE: destinations
    uint32_t ptr_off;     // MREDUCE: index of srcs[0] in the pointer list; dsts follow the srcs
    uint32_t slots;       // column executor: value slots of DEVOP_GET0 / GET1 / PUT, one byte each
    uint64_t reserved1;
};
static_assert(sizeof(DevOp) == 64, "DevOp is read as one 64-byte scalar load");

// COPY / REDUCE_INTO / XREDUCE rows: tiles of block*unroll 16-byte vectors
hipError_t launch_round(int dtype, int unroll, int block, hipStream_t st, const DevOp* ops, uint32_t nops,
                        uint32_t total_tiles, uint32_t tiles_per_op, uint32_t interleave, uint32_t reverse);
// MREDUCE rows: tiles of mreduce_tile_bytes()
uint64_t mreduce_tile_bytes();
hipError_t launch_mreduce(int dtype, hipStream_t st, const DevOp* ops, uint32_t nops, char* const* ptrs,
                          uint32_t total_tiles, uint32_t tiles_per_op, uint32_t interleave, uint32_t reverse);
// column executor: all rounds of COPY / REDUCE_INTO / XREDUCE rows (each exactly one chunk long) in one
// launch.  The rows are sorted into components (sets of rows that share rank-chunk cells with each other and
// with no other row); a work item is one component for one column of column_bytes(block, two_vectors) bytes: one
// 16-byte vector per lane and row, or two (with forwarding, nslots > 0, outside the latency plan, where the plan says so).
struct ColumnComp {
    uint32_t group_first, group_end;   // the component's groups (rows of one round each) in group_begin[]
    uint32_t row_first, row_end;       // = group_begin[group_first], group_begin[group_end]
};
struct ColumnLaunch {
    const DevOp* ops;            // the rows, component by component, in round order within a component
    const uint32_t* group_begin; // rows of group g are ops[group_begin[g] .. group_begin[g+1])
    const ColumnComp* comps;
    char* const* ptrs;           // pointer lists of MREDUCE rows (srcs, then dsts, from the row's ptr_off)
    uint32_t ncomp, ncols, run;  // items in dispatch order: `run` neighbouring columns of component 0, the same columns of
    uint32_t nitems;             // component 1, ...; then the next `run` columns.  nitems = ceil(ncols / run) * run * ncomp
    uint32_t table_rows;         // 0, or the most rows of a component: latency plan, the workgroup copies the rows and
    uint32_t table_groups;       // group boundaries (at most table_groups) of its component into LDS first (block =
                                 // column_latency_block())
    uint32_t multi_source;       // != 0: some rows are MREDUCE rows (a kernel variant of its own: their loads cost registers)
    uint32_t lane_local;         // != 0 promises that no lane reads bytes another lane wrote (all rows 16-byte
                                 // aligned, no partial vectors): groups are then separated by an execution barrier only
    uint32_t policy;             // whole launch: 0 = cached accesses, 1 = streaming loads, 2 = streaming loads and stores
    uint32_t two_vectors;        // with value slots and without a staged table: != 0 = a lane moves two 16-byte vectors per row
};
// With nslots > 0 a workgroup keeps up to nslots values per lane in LDS (nslots vectors per lane and vector of the row) and
// rows flagged DEVOP_GET* take their operands from there instead of memory.  Slots plus the staged table
// (column_table_bytes) must fit column_lds_budget().
uint64_t column_bytes(int block, bool two_vectors);
uint64_t column_lds_budget();
uint64_t column_table_bytes(uint32_t rows, uint32_t groups);
int column_latency_block();
hipError_t launch_column(int dtype, int block, uint32_t grid, uint32_t nslots, hipStream_t st, const ColumnLaunch& L);

hipError_t launch_fill_const(hipStream_t st, char* dst, uint64_t elems, float value, int dtype);
hipError_t launch_fill_random(hipStream_t st, char* dst, uint64_t elems, uint64_t key, double a, double b, int mode, int dtype);
// device-to-device copy with streaming accesses (hipMemcpyAsync when a pointer is not 16-byte aligned)
hipError_t launch_copy(hipStream_t st, char* dst, const char* src, uint64_t bytes);
hipError_t launch_compare(hipStream_t st, const char* a, const char* b, uint64_t bytes, int* differs);
// writes 4 * stream_bytes to each of the two windows; stamps[0] / stamps[1] (preset to ~0 / 0) receive the wall-clock
// ticks of the earliest start and the latest end
hipError_t launch_region_probe(hipStream_t st, char* a, char* b, uint64_t stream_bytes, unsigned long long* stamps);
// stream probe (see stream_probe_kernel): up to 8 jobs of up to 8 read and 8 written streams of `bytes` bytes each
struct ProbeJobs {
    char* rd[8][8];
    char* wr[8][8];
    uint32_t nread[8], nwrite[8];
    uint32_t njobs, reserved;
    uint64_t bytes;
};
// policy: 0 = cached accesses, 1 = streaming loads and cached stores, 2 = streaming loads and stores
hipError_t launch_stream_probe(hipStream_t st, const ProbeJobs& J, int block, int unroll, int policy, bool persistent, bool interleave, int compute_units);
hipError_t launch_sleep(hipStream_t st, uint64_t ticks);

}  // namespace sar
