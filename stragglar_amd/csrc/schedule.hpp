// Schedule representation of an emulated n-rank AllReduce: rounds of rows,
// each row a chunk move or reduce between rank buffers.  Host-only code.
#pragma once
#include <cstddef>
#include <cstdint>
#include <string>
#include <vector>

#include "sar.h"

namespace sar {

struct Op {
    int kind = SAR_OP_COPY;
    int dst_rank = 0;    // XREDUCE: first side
    int src_rank = 0;    // XREDUCE: second side; MREDUCE: unused (-1)
    int dst_chunk = 0;
    int src_chunk = 0;
    int nchunks = 1;
    int group = 0;       // MREDUCE: ranks 0..group-1
    int bcast = 0;       // MREDUCE: result goes to every group member
    int to_end = 0;      // range also covers the elements past parts*chunk
};

struct Schedule {
    int n = 0;
    int parts = 1;               // chunks per rank buffer
    bool stragglar_rules = false; // validate with the synthesizers' own per-round rules
    std::string name;
    std::vector<std::vector<Op>> rounds;
};

// Element range of a row for a buffer of `elems` elements.
struct Range { uint64_t dst_off, src_off, len; };
Range lower_range(const Schedule& s, const Op& op, uint64_t elems);

// text format of the reference synthesizers, or a row list (first line 'sar-rows <ranks> <parts>') -> schedule;
// throws std::runtime_error
Schedule parse_table(const char* text, size_t len, int n);
Schedule builtin(const std::string& alg, int n);
// empty string = valid, else the reason
std::string validate(const Schedule& s);
void byte_counts(const Schedule& s, uint64_t elems, int elem_size, uint64_t* algorithmic, uint64_t* reference_op);
uint64_t pad_bytes(uint64_t bytes, int n);

}  // namespace sar

struct sar_schedule { sar::Schedule s; };
