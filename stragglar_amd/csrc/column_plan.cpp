// Planner of the column executor (see column_plan.hpp).  The steps, in order:
//   rows         every schedule row cut into single-chunk rows with the (rank, chunk) cells they touch
//   components   rows that share cells, transitively; within a component, groups of one round each
//   heads        components whose chunks start off the 16-byte boundary are moved up to it
//   shape        column width, latency plan
//   forwarding   which operands come from value slots, how many slots
//   dead stores  which stored values nobody loads
//   launch       cache policy, dispatch order of the items, kind of barrier
#include "column_plan.hpp"

#include <algorithm>

namespace sar {
namespace {

constexpr uint32_t kNever = 0xffffffffu;

struct ColRow {
    DevOp d;
    int c0, c1;                        // cells of p0 and p1
    uint32_t round;
    std::vector<int> mreads, mwrites;  // cells of a multi-source row; mwrites of any other row: its extra destinations
};

struct Ev { uint32_t row; bool reads, writes; };   // a row touching a cell; a reducing row reads and writes its cell

// result of one pass of the slot bookkeeping
struct Forwarding {
    std::vector<uint32_t> flags, slots;      // per row: DEVOP_GET0 | GET1 | PUT (| DEAD0 | DEAD1) and the packed slot numbers
    uint32_t nslots = 0;
    uint64_t bytes = 0;                      // operand bytes found in slots
};

class Planner {
public:
    Planner(const ColumnEnv& env, const std::vector<const Schedule*>& scheds, std::vector<char*>& ptrs, ColumnPlan& plan)
        : env_(env), scheds_(scheds), s_(*scheds.back()), ptrs_(ptrs), plan_(plan),
          chunk_bytes_((env.elems / (uint64_t)s_.parts) * (uint64_t)env.elem_size),
          cells_per_rank_(s_.parts + 1), ncells_(env.n * (s_.parts + 1)) {}

    int run(std::vector<DevOp>& rows, std::string* error) {
        plan_ = ColumnPlan();
        const int rc = make_rows(error);
        if (rc != SAR_OK || plan_.unsupported) return rc;
        split_components();
        align_heads();
        choose_shape();
        if (env_.tune.col_depth_first && !plan_.staged) order_depth_first();
        index_cells();
        Forwarding fwd = choose_forwarding();
        const Shape before = shape();
        if (fwd.nslots && env_.tune.col_elide_stores) {
            mark_dead_stores(fwd);
            // (in the bandwidth regime the chain is bound by memory either way: measured equal to 2 % slower)
            if (env_.tune.col_fuse_chains == 2 || (env_.tune.col_fuse_chains == 1 && plan_.staged)) fuse_chains(fwd);
        }
        const bool pays = !plan_.staged || env_.tune.col_slots != 0 || !fwd.nslots || slots_pay_when_staged(fwd);
        const uint32_t rows_before = (uint32_t)before.cr.size();
        if (fwd.nslots && (env_.tune.col_fuse_copies == 2 || (env_.tune.col_fuse_copies == 1 && copies_pay(fwd)))) fuse_copies(fwd);
        // (latency plan) ... or when taking the copies of held values into the rows that produce them shortens the
        // items by a quarter or more (halving-doubling: the doubling half disappears, 11.4 -> 10.2 us at n = 8)
        if (!pays && nrows() * 4u > rows_before * 3u) {
            restore(before);
            fwd = forward(0); all_found_ = false;
        }
        plan_.nslots = fwd.nslots; plan_.forwarded_bytes = fwd.bytes;
        for (uint32_t i = 0; i < nrows(); ++i) { cr_[i].d.flags |= fwd.flags[i]; cr_[i].d.slots = fwd.slots[i]; }
        if (plan_.staged) mark_joins();
        choose_vectors();
        choose_launch();
        for (const auto& r : cr_) { rows.push_back(r.d); plan_.multi_source |= r.d.kind == SAR_OP_MREDUCE; }
        return SAR_OK;
    }

private:
    uint32_t nrows() const { return (uint32_t)cr_.size(); }
    int cell_of(int rank, uint64_t byte_off) const {
        return rank * cells_per_rank_ + (int)(chunk_bytes_ ? std::min<uint64_t>(byte_off / chunk_bytes_, (uint64_t)s_.parts) : 0);
    }

    int make_rows(std::string* error) {
        const uint64_t es = (uint64_t)env_.elem_size;
        uint32_t round_no = 0;
        for (const Schedule* sp : scheds_) {
            if (sp->parts != s_.parts) { plan_.unsupported = true; return SAR_OK; }
            for (size_t ri = 0; ri < sp->rounds.size(); ++ri, ++round_no) {
                for (const Op& op : sp->rounds[ri]) {
                    const Range rg = lower_range(*sp, op, env_.elems);
                    const uint64_t row_bytes = rg.len * es;
                    if (row_bytes == 0) continue;
                    const uint64_t row_doff = rg.dst_off * es, row_soff = rg.src_off * es;
                    if (row_doff + row_bytes > env_.bytes_per_rank || row_soff + row_bytes > env_.bytes_per_rank) {
                        if (error) *error = "row leaves the rank buffer";
                        return SAR_ESCHED;
                    }
                    for (int j = 0; j < op.nchunks; ++j) {
                        const uint64_t base = (uint64_t)j * chunk_bytes_;
                        ColRow r{};
                        r.d.kind = (uint32_t)op.kind;
                        r.d.bytes = (j == op.nchunks - 1) ? row_bytes - base : chunk_bytes_;     // a to_end row ends with a longer chunk
                        r.round = round_no;
                        if (op.kind == SAR_OP_MREDUCE) {
                            if (!multi_source_row(op, row_doff + base, r)) { plan_.unsupported = true; return SAR_OK; }
                        } else {
                            r.d.p0 = env_.rank_base[(size_t)op.dst_rank] + row_doff + base;
                            r.d.p1 = env_.rank_base[(size_t)op.src_rank] + row_soff + base;
                            r.d.flags = ((((uintptr_t)r.d.p0 | (uintptr_t)r.d.p1) & 15u) == 0) ? DEVOP_VEC : 0u;
                            r.c0 = cell_of(op.dst_rank, row_doff + base);
                            r.c1 = cell_of(op.src_rank, row_soff + base);
                        }
                        cr_.push_back(r);
                    }
                }
            }
        }
        if (cr_.size() > 0x7ffffff0ull) { if (error) *error = "schedule has too many rows"; return SAR_EINVAL; }
        return SAR_OK;
    }

    // ring order over the group: x_{r+1}, x_{r+2}, ..., x_{r-1}, x_r (the owner last), as one launch per round has it
    bool multi_source_row(const Op& op, uint64_t off, ColRow& r) {
        r.d.ptr_off = (uint32_t)ptrs_.size(); r.d.nsrc = (uint32_t)op.group;
        for (int q = 1; q <= op.group; ++q) {
            const int rank = (op.dst_rank + q) % op.group;
            ptrs_.push_back(env_.rank_base[(size_t)rank] + off); r.mreads.push_back(cell_of(rank, off));
        }
        if (op.bcast) {
            r.d.ndst = (uint32_t)op.group;
            for (int q = 0; q < op.group; ++q) { ptrs_.push_back(env_.rank_base[(size_t)q] + off); r.mwrites.push_back(cell_of(q, off)); }
        } else {
            r.d.ndst = 1; ptrs_.push_back(env_.rank_base[(size_t)op.dst_rank] + off); r.mwrites.push_back(cell_of(op.dst_rank, off));
        }
        bool aligned = (r.d.bytes & 15u) == 0;
        for (size_t k = r.d.ptr_off; k < ptrs_.size(); ++k) aligned &= ((uintptr_t)ptrs_[k] & 15u) == 0;
        if (!aligned) return false;
        r.d.flags = DEVOP_VEC;
        r.d.p0 = ptrs_[r.d.ptr_off + r.d.nsrc]; r.d.p1 = ptrs_[r.d.ptr_off];
        r.c0 = r.mwrites[0]; r.c1 = r.mreads[0];
        return true;
    }

    // Components: rows that (transitively) share a cell.  Rows of different components touch disjoint bytes in
    // every column, so no order is needed between them; within a component the round order is kept.  For the
    // four algorithms every row moves a chunk to the same chunk index, and the components are the chunk indices.
    void split_components() {
        const bool split = env_.tune.col_split != 0;
        std::vector<int> parent((size_t)ncells_);
        for (int i = 0; i < ncells_; ++i) parent[(size_t)i] = i;
        auto find = [&](int x) { while (parent[(size_t)x] != x) { parent[(size_t)x] = parent[(size_t)parent[(size_t)x]]; x = parent[(size_t)x]; } return x; };
        auto unite = [&](int x, int y) { const int a = find(x), b = find(y); if (a != b) parent[(size_t)b] = a; };
        if (split) for (const auto& r : cr_) {
            unite(r.c0, r.c1);
            for (int cell : r.mreads) unite(r.c0, cell);
            for (int cell : r.mwrites) unite(r.c0, cell);
        }
        std::vector<int> comp_of_root((size_t)ncells_, -1);
        std::vector<std::vector<uint32_t>> members;
        for (uint32_t i = 0; i < nrows(); ++i) {
            const int root = split ? find(cr_[i].c0) : 0;
            if (comp_of_root[(size_t)root] < 0) { comp_of_root[(size_t)root] = (int)members.size(); members.emplace_back(); }
            members[(size_t)comp_of_root[(size_t)root]].push_back(i);
        }
        std::vector<ColRow> sorted; sorted.reserve(nrows());
        for (const auto& m : members) {
            ColumnComp cc{};
            cc.group_first = (uint32_t)plan_.group_begin.size(); cc.row_first = (uint32_t)sorted.size();
            uint32_t last_round = kNever;
            for (uint32_t i : m) {
                if (cr_[i].round != last_round) { plan_.group_begin.push_back((uint32_t)sorted.size()); last_round = cr_[i].round; }
                sorted.push_back(cr_[i]);
            }
            cc.group_end = (uint32_t)plan_.group_begin.size(); cc.row_end = (uint32_t)sorted.size();
            plan_.max_comp_rows = std::max(plan_.max_comp_rows, cc.row_end - cc.row_first);
            plan_.max_comp_groups = std::max(plan_.max_comp_groups, cc.group_end - cc.group_first);
            plan_.comps.push_back(cc);
        }
        plan_.group_begin.push_back((uint32_t)sorted.size());
        cr_.swap(sorted);
    }

    // Chunks that do not start on a 16-byte boundary (a buffer cut into a number of parts that its size was not
    // padded for).  When all rows of a component start the same distance h in front of a boundary, on both sides,
    // they are moved up to it and run as vectors; the h bytes in front are done element by element in the first
    // column.  All rows of a component must move together: a column has to mean the same offsets in each of them.
    void align_heads() {
        for (const auto& cc : plan_.comps) {
            const uint32_t phase = (uint32_t)((uintptr_t)cr_[cc.row_first].d.p0 & 15u), h = 16u - phase;
            bool same = phase != 0 && phase % (uint32_t)env_.elem_size == 0;
            for (uint32_t i = cc.row_first; i < cc.row_end && same; ++i) {
                const DevOp& d = cr_[i].d;
                same = d.kind != SAR_OP_MREDUCE && ((uintptr_t)d.p0 & 15u) == phase && ((uintptr_t)d.p1 & 15u) == phase && d.bytes > h;
            }
            if (!same) continue;
            for (uint32_t i = cc.row_first; i < cc.row_end; ++i) {
                DevOp& d = cr_[i].d;
                d.p0 += h; d.p1 += h; d.bytes -= h;
                d.flags |= DEVOP_VEC | (h << DEVOP_HEAD_SHIFT);
            }
        }
        plan_.widest_row = 0;
        for (const auto& r : cr_) plan_.widest_row = std::max(plan_.widest_row, r.d.bytes);
    }

    void choose_shape() {
        // column width: 512 vectors when that still leaves enough columns to fill the chip, else 256
        plan_.block = env_.tune.col_block ? env_.tune.col_block : (plan_.widest_row / column_bytes(512, false) >= 2048 ? 512 : 256);

        // Latency plan: when the work items are so few that they are all resident at once, time goes into dependent
        // round trips, not bandwidth, and nobody warms the scalar cache: a row read through scalar loads is a trip to
        // L2.  A workgroup then copies the rows of its component into LDS first, and a lane moves one vector per row
        // (few items are better spread over more workgroups).  Forwarding is kept only where it takes the loads out of
        // most rows (see choose_forwarding).
        const int lb = column_latency_block();
        const uint64_t lcols = (plan_.widest_row + column_bytes(lb, false) - 1) / column_bytes(lb, false);
        const uint64_t items = lcols * plan_.comps.size();
        const bool few = env_.tune.col_latency_plan == 2 || (env_.tune.col_latency_plan == 1 && items <= 8u * (uint64_t)std::max(1, env_.compute_units));
        if (few && (env_.tune.col_block == 0 || env_.tune.col_block == lb) &&
            column_table_bytes(plan_.max_comp_rows, plan_.max_comp_groups + 1) <= column_lds_budget()) {
            plan_.staged = true;
            plan_.block = lb;
        }
    }

    // The cells a row reads and writes.
    void touches(const ColRow& r, std::vector<int>& reads, std::vector<int>& writes) const {
        reads.clear(); writes.clear();
        if (r.d.kind == SAR_OP_MREDUCE) { reads = r.mreads; writes = r.mwrites; return; }
        reads.push_back(r.c1);
        if (r.d.kind != SAR_OP_COPY) reads.push_back(r.c0);
        writes.push_back(r.c0);
        if (r.d.kind == SAR_OP_XREDUCE) writes.push_back(r.c1);
        for (int cell : r.mwrites) writes.push_back(cell);
    }

    // Bandwidth plan: the order of a component's rows decides how many values are alive at a time, and with it the
    // value slots a lane needs and the workgroups a compute unit holds.  Round order runs a reduce tree level by
    // level (halving-doubling: n/2 partial sums alive after the first round); taking a row as soon as the values it
    // consumes exist walks the tree depth first instead (log2 n alive: 3 slots instead of 4 at n = 8, 4 instead of
    // 8 at n = 16).  Rows that touch a common cell, one of them writing it, keep their order; nothing else about a
    // round is binding, since every lane meets only its own column.  Among the rows that may run next, one that
    // reads a cell written by a row already placed goes first, else the earliest in round order.  Groups are cut
    // anew: a row joins the open group unless it conflicts with a row in it.  Tables whose rows already come in
    // this order (the StragglAR tables, ring, direct) are left as they are.
    void order_depth_first() {
        std::vector<ColRow> out; out.reserve(nrows());
        std::vector<uint32_t> group_begin;
        std::vector<ColumnComp> comps;
        uint32_t max_groups = 0;
        std::vector<int> rd, wr, rd2, wr2;
        for (const auto& cc : plan_.comps) {
            const uint32_t m = cc.row_end - cc.row_first;
            // predecessors by conflict
            std::vector<std::vector<uint32_t>> preds(m);
            std::vector<std::vector<int>> reads(m), writes(m);
            for (uint32_t j = 0; j < m; ++j) touches(cr_[cc.row_first + j], reads[j], writes[j]);
            auto hits = [](const std::vector<int>& a, const std::vector<int>& b) {
                for (int x : a) for (int y : b) if (x == y) return true;
                return false;
            };
            for (uint32_t j = 0; j < m; ++j)
                for (uint32_t i = 0; i < j; ++i)
                    if (hits(writes[i], reads[j]) || hits(writes[i], writes[j]) || hits(reads[i], writes[j])) preds[j].push_back(i);
            std::vector<char> placed(m, 0);
            std::vector<uint32_t> order; order.reserve(m);
            for (uint32_t step = 0; step < m; ++step) {
                int pick = -1;
                for (uint32_t j = 0; j < m && pick < 0; ++j) {          // a consumer of a value that exists already
                    if (placed[j]) continue;
                    bool ready = true, consumes = false;
                    for (uint32_t i : preds[j]) { ready = ready && placed[i]; consumes = consumes || (placed[i] && hits(writes[i], reads[j])); }
                    if (ready && consumes) pick = (int)j;
                }
                for (uint32_t j = 0; j < m && pick < 0; ++j) {          // else the earliest row whose turn it can be
                    if (placed[j]) continue;
                    bool ready = true;
                    for (uint32_t i : preds[j]) ready = ready && placed[i];
                    if (ready) pick = (int)j;
                }
                placed[(size_t)pick] = 1; order.push_back((uint32_t)pick);
            }
            ColumnComp nc{};
            nc.group_first = (uint32_t)group_begin.size(); nc.row_first = (uint32_t)out.size();
            uint32_t open = 0;                                          // first row (index into order) of the open group
            for (uint32_t k = 0; k < m; ++k) {
                bool conflict = k == 0;
                for (uint32_t q = open; q < k && !conflict; ++q)
                    conflict = std::find(preds[order[k]].begin(), preds[order[k]].end(), order[q]) != preds[order[k]].end() ||
                               std::find(preds[order[q]].begin(), preds[order[q]].end(), order[k]) != preds[order[q]].end();
                if (conflict) { group_begin.push_back((uint32_t)out.size()); open = k; }
                out.push_back(cr_[cc.row_first + order[k]]);
            }
            nc.group_end = (uint32_t)group_begin.size(); nc.row_end = (uint32_t)out.size();
            max_groups = std::max(max_groups, nc.group_end - nc.group_first);
            comps.push_back(nc);
        }
        group_begin.push_back((uint32_t)out.size());
        cr_.swap(out); plan_.group_begin.swap(group_begin); plan_.comps.swap(comps);
        plan_.max_comp_groups = max_groups;
    }

    // per cell, the rows that touch it, in order
    void index_cells() {
        ev_.assign((size_t)ncells_, {});
        for (uint32_t i = 0; i < nrows(); ++i) {
            const ColRow& r = cr_[i];
            if (r.d.kind == SAR_OP_MREDUCE) {
                for (int cell : r.mreads)
                    ev_[(size_t)cell].push_back({i, true, std::find(r.mwrites.begin(), r.mwrites.end(), cell) != r.mwrites.end()});
                for (int cell : r.mwrites)
                    if (std::find(r.mreads.begin(), r.mreads.end(), cell) == r.mreads.end()) ev_[(size_t)cell].push_back({i, false, true});
                continue;
            }
            const bool reduce = r.d.kind != SAR_OP_COPY, both = r.d.kind == SAR_OP_XREDUCE;
            ev_[(size_t)r.c0].push_back({i, reduce, true});
            if (r.c1 != r.c0) ev_[(size_t)r.c1].push_back({i, true, both});
            for (int cell : r.mwrites) ev_[(size_t)cell].push_back({i, false, true});
        }
    }
    std::vector<Ev>::const_iterator first_after(int cell, uint32_t i) const {
        const auto& v = ev_[(size_t)cell];
        return std::upper_bound(v.begin(), v.end(), i, [](uint32_t x, const Ev& e) { return x < e.row; });
    }
    // the next row after `i` that reads the cell's present value (never: it is overwritten first, or not read again)
    uint32_t next_read(int cell, uint32_t i) const {
        const auto it = first_after(cell, i);
        return (it != ev_[(size_t)cell].end() && it->reads) ? it->row : kNever;
    }

    // one pass of the slot bookkeeping with at most `max_slots` slots
    Forwarding forward(uint32_t max_slots) const {
        Forwarding f;
        f.flags.assign(nrows(), 0); f.slots.assign(nrows(), 0);
        if (max_slots == 0) return f;
        struct Slot { std::vector<int> cells; uint64_t bytes = 0; };
        std::vector<Slot> slot(max_slots);
        std::vector<int> cell_slot((size_t)ncells_, -1);
        auto drop_cell = [&](int cell) {
            const int k = cell_slot[(size_t)cell];
            if (k < 0) return;
            auto& v = slot[(size_t)k].cells;
            v.erase(std::remove(v.begin(), v.end(), cell), v.end());
            cell_slot[(size_t)cell] = -1;
        };
        auto clear_slot = [&](int k) {
            for (int cell : slot[(size_t)k].cells) cell_slot[(size_t)cell] = -1;
            slot[(size_t)k].cells.clear();
        };
        auto slot_next_use = [&](int k, uint32_t i) {
            uint32_t m = kNever;
            for (int cell : slot[(size_t)k].cells) m = std::min(m, next_read(cell, i));
            return m;
        };
        // a slot for a value next used at row `nu`: a free one, else the one whose own next use is furthest (and later than nu)
        auto take_slot = [&](uint32_t nu, uint32_t i) {
            int far = -1; uint32_t far_use = 0;
            for (int k = 0; k < (int)max_slots; ++k) {
                if (slot[(size_t)k].cells.empty()) return k;
                const uint32_t u = slot_next_use(k, i);
                if (u == kNever) { clear_slot(k); return k; }
                if (u > far_use) { far_use = u; far = k; }
            }
            if (far >= 0 && far_use > nu) { clear_slot(far); return far; }
            return -1;
        };
        auto uses = [&](int k) { f.nslots = std::max(f.nslots, (uint32_t)k + 1); };
        for (uint32_t i = 0; i < nrows(); ++i) {
            const DevOp& d = cr_[i].d;
            if (d.kind == SAR_OP_MREDUCE) {
                // all operands come from memory (they are inputs nobody has touched); the result is a new value
                uint32_t nu = kNever;
                for (int cell : cr_[i].mwrites) { drop_cell(cell); nu = std::min(nu, next_read(cell, i)); }
                const int k = nu == kNever ? -1 : take_slot(nu, i);
                if (k >= 0) {
                    slot[(size_t)k].bytes = d.bytes;
                    for (int cell : cr_[i].mwrites) { slot[(size_t)k].cells.push_back(cell); cell_slot[(size_t)cell] = k; }
                    f.flags[i] |= DEVOP_PUT; f.slots[i] |= (uint32_t)k << 16; uses(k);
                }
                continue;
            }
            const int c0 = cr_[i].c0, c1 = cr_[i].c1;
            const bool reduce = d.kind != SAR_OP_COPY;
            const bool can = (d.flags & DEVOP_VEC) && c0 != c1;
            int k0 = (can && reduce) ? cell_slot[(size_t)c0] : -1, k1 = can ? cell_slot[(size_t)c1] : -1;
            if (k0 >= 0 && slot[(size_t)k0].bytes != d.bytes) k0 = -1;
            if (k1 >= 0 && slot[(size_t)k1].bytes != d.bytes) k1 = -1;
            if (k0 >= 0) { f.flags[i] |= DEVOP_GET0; f.slots[i] |= (uint32_t)k0; f.bytes += d.bytes & ~(uint64_t)15u; uses(k0); }
            if (k1 >= 0) { f.flags[i] |= DEVOP_GET1; f.slots[i] |= (uint32_t)k1 << 8; f.bytes += d.bytes & ~(uint64_t)15u; uses(k1); }
            // the row's result replaces what its destination cells held
            drop_cell(c0);
            if (d.kind == SAR_OP_XREDUCE) drop_cell(c1);
            if (d.kind == SAR_OP_COPY && k1 >= 0) {
                slot[(size_t)k1].cells.push_back(c0); cell_slot[(size_t)c0] = k1;          // the held value now lives in c0 too
            } else if (can) {
                uint32_t nu = next_read(c0, i);
                if (d.kind != SAR_OP_REDUCE_INTO) nu = std::min(nu, next_read(c1, i));      // COPY: source and destination hold the value
                const int k = nu == kNever ? -1 : take_slot(nu, i);
                if (k >= 0) {
                    if (d.kind == SAR_OP_COPY) drop_cell(c1);
                    slot[(size_t)k].bytes = d.bytes;
                    slot[(size_t)k].cells.push_back(c0); cell_slot[(size_t)c0] = k;
                    if (d.kind != SAR_OP_REDUCE_INTO) { slot[(size_t)k].cells.push_back(c1); cell_slot[(size_t)c1] = k; }
                    f.flags[i] |= DEVOP_PUT; f.slots[i] |= (uint32_t)k << 16; uses(k);
                }
            }
        }
        if (f.bytes == 0) { f.flags.assign(nrows(), 0); f.slots.assign(nrows(), 0); f.nslots = 0; }    // nothing found: no slots at all
        return f;
    }

    Forwarding choose_forwarding() {
        Forwarding fwd = forward(0);
        all_found_ = false;
        no_reuse_ = forward(255u).bytes == 0;
        // Nothing is read twice and every row is a pairwise row (the exchanges of a table on their own): nothing to keep in
        // slots, two cold loads and one or two stores per vector, and the narrower column runs ahead (n = 8, in a sequence
        // of steps: 256 MiB per rank 172.8 against 175.0 us, 1 GiB 681 against 698).  A plan of multi-source rows alone
        // (a pre-work) stays at 512: 1024 threads gain 1.7 % at 1 GiB fp32 per rank, nothing in bf16 and lose 2.5 % at 256 MiB.
        if (no_reuse_ && !env_.tune.col_block && !plan_.staged && plan_.block == 512) {
            bool pairwise = !cr_.empty();
            for (const auto& r : cr_) pairwise = pairwise && r.d.kind != SAR_OP_MREDUCE;
            if (pairwise) plan_.block = 256;
        }
        if (!env_.tune.col_forward) return fwd;
        const uint64_t table = plan_.staged ? column_table_bytes(plan_.max_comp_rows, plan_.max_comp_groups + 1) : 0u;
        const uint32_t fit = (uint32_t)std::min<uint64_t>(255u, (column_lds_budget() - table) / column_bytes(plan_.block, !plan_.staged));
        if (env_.tune.col_slots > 0) {
            fwd = forward(std::min<uint32_t>(fit, (uint32_t)env_.tune.col_slots));
            all_found_ = fwd.nslots && fwd.bytes == forward(255u).bytes;
            return fwd;
        }
        // How many slots.  LDS per compute unit is what they cost: up to 5 per lane all 2048 lanes of a compute
        // unit stay resident, up to 10 half of them.  Measured on MI355X, half occupancy pays when every re-read
        // is then found in a slot (what still goes to memory is the cold inputs and the stores), but not for a
        // part of them; and a plan that finds less than a tenth of the bytes the rows move is not worth the
        // longer row loop.  (Component by component few values are alive at a time: one for the StragglAR
        // tables and ring, four for halving-doubling at n = 8.)
        const uint64_t all = forward(255u).bytes;
        fwd = forward(std::min<uint32_t>(fit, 10u));
        if (fwd.bytes != all) fwd = forward(std::min<uint32_t>(fit, 5u));
        all_found_ = fwd.nslots && fwd.bytes == all;
        uint64_t moved = 0;                  // algorithmic bytes of the rows
        for (const auto& r : cr_) moved += r.d.bytes * (r.d.kind == SAR_OP_COPY ? 2u : r.d.kind == SAR_OP_XREDUCE ? 4u : r.d.kind == SAR_OP_MREDUCE ? r.d.nsrc + r.d.ndst : 3u);
        if (fwd.bytes * 10u < moved) { fwd = forward(0); all_found_ = false; }
        return fwd;
    }

    // Latency plan: the buffers sit in L2 and an operand from there arrives about as fast as one from a slot.
    // What forwarding buys is rows that load nothing at all (copies of a held value: no round trip in the
    // chain).  Keep it when two thirds of the rows are such (the broadcast trees of the StragglAR tables and of
    // direct: n = 32 at 1 MiB per rank 17.8 us against 21.8 us; ring once its reduce-scatter chain is one row),
    // not for rows that mostly still load (halving-doubling: 12.9 against 11.7 us at n = 8).
    // Copies stored by the row that produced their value (col_fuse_copies = 1): always in the latency plan.  In the
    // bandwidth plan the traffic is the same either way and what is saved is rows, which counts while a good part of
    // the payload stays in the 256 MB Infinity Cache (n = 8: 3 to 9 % faster at 8 to 64 MiB per rank, equal to 3 %
    // slower at 256 MiB, where eight stores in one burst suit the memory less than stores spread over the rounds),
    // and where the value slots leave a CU fewer workgroups than its thread limit allows, so that the rows of an item
    // have less company to hide behind (halving-doubling, 4 or 5 slots: 3 % faster at every size).
    bool copies_pay(const Forwarding& fwd) const {
        if (plan_.staged) return true;
        if (env_.bytes_per_rank * (uint64_t)env_.n <= (768ull << 20)) return true;
        const uint64_t wgs_by_threads = 2048u / (uint32_t)plan_.block;
        return (uint64_t)fwd.nslots * column_bytes(plan_.block, true) * wgs_by_threads > column_lds_budget();
    }

    bool slots_pay_when_staged(const Forwarding& fwd) const {
        uint32_t free_rows = 0;
        for (uint32_t i = 0; i < nrows(); ++i) free_rows += cr_[i].d.kind == SAR_OP_COPY && (fwd.flags[i] & DEVOP_GET1);
        return free_rows * 3u >= nrows() * 2u;
    }

    // what fuse_chains changes, to be able to take it back
    struct Shape {
        std::vector<ColRow> cr; std::vector<uint32_t> group_begin; std::vector<ColumnComp> comps;
        uint32_t max_comp_rows, max_comp_groups; size_t nptrs; uint64_t elided;
    };
    Shape shape() const { return {cr_, plan_.group_begin, plan_.comps, plan_.max_comp_rows, plan_.max_comp_groups, ptrs_.size(), plan_.elided_bytes}; }
    void restore(const Shape& sh) {
        cr_ = sh.cr; plan_.group_begin = sh.group_begin; plan_.comps = sh.comps;
        plan_.max_comp_rows = sh.max_comp_rows; plan_.max_comp_groups = sh.max_comp_groups;
        ptrs_.resize(sh.nptrs); plan_.elided_bytes = sh.elided;
    }

    // Chains of one-sided reduces.  `b += a; c += b; d += c; ...` where every partial sum has the next row as its
    // only reader, comes to it in a slot and is never stored (the reduce-scatter half of a ring) is one
    // multi-source row: a + b, then + c, + d in the same order, with all cold operands loaded together instead of
    // one round trip per row.  It takes the place of the chain's last row; the loads it moves there from earlier
    // rounds read cells that nobody writes in between (the rows' own stores were dead).
    void fuse_chains(Forwarding& fwd) {
        auto plain = [&](uint32_t i) {
            const DevOp& d = cr_[i].d;
            return d.kind == SAR_OP_REDUCE_INTO && (d.flags & DEVOP_VEC) && !(d.flags >> DEVOP_HEAD_SHIFT & 15u) && !(d.bytes & 15u) && cr_[i].c0 != cr_[i].c1;
        };
        auto written_between = [&](int cell, uint32_t after, uint32_t upto) {      // a row in (after, upto] writes the cell
            for (auto it = first_after(cell, after); it != ev_[(size_t)cell].end() && it->row <= upto; ++it) if (it->writes) return true;
            return false;
        };
        std::vector<char> removed(nrows(), 0), taken(nrows(), 0);
        std::vector<std::pair<uint32_t, ColRow>> fused;          // (row replaced, the multi-source row)
        for (uint32_t i = 0; i < nrows(); ++i) {
            if (taken[i] || !plain(i) || (fwd.flags[i] & (DEVOP_GET0 | DEVOP_GET1))) continue;
            std::vector<uint32_t> chain{i};
            for (uint32_t cur = i;;) {
                const uint32_t want = DEVOP_PUT | DEVOP_DEAD0;
                if ((fwd.flags[cur] & want) != want) break;
                const int cell = cr_[cur].c0;
                const uint32_t j = next_read(cell, cur);
                if (j == kNever || taken[j] || !plain(j) || cr_[j].c1 != cell || cr_[j].d.bytes != cr_[cur].d.bytes) break;
                if ((fwd.flags[j] & (DEVOP_GET0 | DEVOP_GET1)) != DEVOP_GET1 || (fwd.slots[j] >> 8 & 0xffu) != (fwd.slots[cur] >> 16 & 0xffu)) break;
                if (next_read(cell, j) != kNever) break;                            // somebody else reads the partial sum too
                chain.push_back(j); cur = j;
            }
            if (chain.size() < 2) continue;
            const uint32_t last = chain.back();
            bool safe = !written_between(cr_[chain[0]].c1, chain[0], last);
            for (size_t k = 0; k + 1 < chain.size() && safe; ++k) safe = !written_between(cr_[chain[k]].c0, chain[k], last);
            if (!safe) continue;
            ColRow f = cr_[last];
            f.d.kind = SAR_OP_MREDUCE;
            f.d.ptr_off = (uint32_t)ptrs_.size(); f.d.nsrc = (uint32_t)chain.size() + 1u; f.d.ndst = 1;
            ptrs_.push_back(cr_[chain[0]].d.p1); f.mreads.push_back(cr_[chain[0]].c1);
            for (uint32_t r : chain) { ptrs_.push_back(cr_[r].d.p0); f.mreads.push_back(cr_[r].c0); }
            ptrs_.push_back(cr_[last].d.p0); f.mwrites.push_back(cr_[last].c0);
            f.d.p1 = cr_[chain[0]].d.p1; f.c1 = cr_[chain[0]].c1;
            for (uint32_t r : chain) taken[r] = 1;
            for (size_t k = 0; k + 1 < chain.size(); ++k) removed[chain[k]] = 1;
            fused.emplace_back(last, f);
        }
        if (fused.empty()) return;
        for (const auto& fr : fused) {
            cr_[fr.first] = fr.second;
            fwd.flags[fr.first] &= DEVOP_PUT | DEVOP_DEAD0; fwd.slots[fr.first] &= 0xff0000u;
        }
        remove_rows(removed, fwd);
    }

    // Takes rows out of the plan: same components, groups that became empty disappear; the cell index is rebuilt.
    void remove_rows(const std::vector<char>& removed, Forwarding& fwd) {
        std::vector<ColRow> cr; std::vector<uint32_t> flags, slots, group_begin; std::vector<ColumnComp> comps;
        uint32_t max_rows = 0, max_groups = 0;
        for (const auto& cc : plan_.comps) {
            ColumnComp nc{};
            nc.group_first = (uint32_t)group_begin.size(); nc.row_first = (uint32_t)cr.size();
            for (uint32_t g = cc.group_first; g < cc.group_end; ++g) {
                bool open = false;
                for (uint32_t i = plan_.group_begin[g]; i < plan_.group_begin[g + 1]; ++i) {
                    if (removed[i]) continue;
                    if (!open) { group_begin.push_back((uint32_t)cr.size()); open = true; }
                    cr.push_back(cr_[i]); flags.push_back(fwd.flags[i]); slots.push_back(fwd.slots[i]);
                }
            }
            nc.group_end = (uint32_t)group_begin.size(); nc.row_end = (uint32_t)cr.size();
            max_rows = std::max(max_rows, nc.row_end - nc.row_first); max_groups = std::max(max_groups, nc.group_end - nc.group_first);
            comps.push_back(nc);
        }
        group_begin.push_back((uint32_t)cr.size());
        cr_.swap(cr); fwd.flags.swap(flags); fwd.slots.swap(slots);
        plan_.group_begin.swap(group_begin); plan_.comps.swap(comps);
        plan_.max_comp_rows = max_rows; plan_.max_comp_groups = max_groups;
        index_cells();                          // row numbers have changed
    }

    // Copies of a held value.  A row that keeps its result in a slot is often followed, rounds later, by copies of
    // that very value to other ranks (the broadcast tree of a StragglAR exchange, a ring's all-gather): rows that
    // load nothing and store one vector.  When nobody touches a copy's destination between the producing row and
    // the copy, the store can just as well be issued by the producing row: the copy row goes away (with its round
    // boundary, when it was alone in it) and the producing row gets one more destination.  Only for plans made of
    // whole vectors; a copy whose store was dead simply disappears.
    void fuse_copies(Forwarding& fwd) {
        for (const auto& r : cr_)
            if (!(r.d.flags & DEVOP_VEC) || (r.d.bytes & 15u) || (r.d.flags >> DEVOP_HEAD_SHIFT & 15u)) return;
        std::vector<char> removed(nrows(), 0);
        bool any = false;
        for (const auto& cc : plan_.comps) {
            for (uint32_t p = cc.row_first; p < cc.row_end; ++p) {
                if (removed[p] || !(fwd.flags[p] & DEVOP_PUT)) continue;
                const uint32_t k = fwd.slots[p] >> 16 & 0xffu;
                std::vector<uint32_t> extra;
                for (uint32_t q = p + 1; q < cc.row_end; ++q) {
                    if (removed[q]) continue;
                    if ((fwd.flags[q] & DEVOP_PUT) && (fwd.slots[q] >> 16 & 0xffu) == k) break;       // the slot gets another value
                    const ColRow& c = cr_[q];
                    if (c.d.kind != SAR_OP_COPY || !(fwd.flags[q] & DEVOP_GET1) || (fwd.slots[q] >> 8 & 0xffu) != k || c.d.bytes != cr_[p].d.bytes) continue;
                    bool clean = true;                    // nobody touches the destination between the two rows
                    for (auto it = first_after(c.c0, p); it != ev_[(size_t)c.c0].end() && it->row < q; ++it) clean = false;
                    if (!clean) continue;
                    removed[q] = 1; any = true;
                    if (!(fwd.flags[q] & DEVOP_DEAD0)) extra.push_back(q);
                }
                if (extra.empty()) continue;
                ColRow& pr = cr_[p];
                const uint32_t first = (uint32_t)ptrs_.size();
                if (pr.d.kind == SAR_OP_MREDUCE) {        // its list again, with the new destinations behind the old
                    if (fwd.flags[p] & DEVOP_DEAD0) {     // ... which go when their store was dead: the flag covers the whole list
                        pr.d.ndst = 0; pr.mwrites.clear(); fwd.flags[p] &= ~(uint32_t)DEVOP_DEAD0;
                    }
                    for (uint32_t i = 0; i < pr.d.nsrc + pr.d.ndst; ++i) { char* const t = ptrs_[pr.d.ptr_off + i]; ptrs_.push_back(t); }
                } else if (pr.d.ndst) {
                    for (uint32_t i = 0; i < pr.d.ndst; ++i) { char* const t = ptrs_[pr.d.ptr_off + i]; ptrs_.push_back(t); }
                }
                for (uint32_t q : extra) { ptrs_.push_back(cr_[q].d.p0); pr.mwrites.push_back(cr_[q].c0); }
                pr.d.ptr_off = first; pr.d.ndst += (uint32_t)extra.size();
            }
        }
        if (any) remove_rows(removed, fwd);
    }

    // Stores nobody needs.  A row's result for a cell is dead when a later row overwrites the cell and every row
    // that reads it before then (the overwriting row included, if it reads) takes it from a slot: the partial
    // sums of ring and halving-doubling, the pre-work's result ahead of the exchange in a same-launch run.  Only
    // the whole vectors are left out; the bytes in front of the first and behind the last one always go through
    // memory.  What the rank buffers hold after the launch does not change.
    void mark_dead_stores(Forwarding& fwd) {
        auto from_slot = [&](uint32_t j, int cell) {            // does row j take the cell's value from a slot?
            const ColRow& r = cr_[j];
            if (r.d.kind == SAR_OP_MREDUCE || r.c0 == r.c1) return false;
            if (cell == r.c1) return (fwd.flags[j] & DEVOP_GET1) != 0;
            return cell == r.c0 && r.d.kind != SAR_OP_COPY && (fwd.flags[j] & DEVOP_GET0) != 0;
        };
        auto dead = [&](uint32_t i, int cell) {
            if (!(cr_[i].d.flags & DEVOP_VEC)) return false;
            for (auto it = first_after(cell, i); it != ev_[(size_t)cell].end(); ++it) {
                if (it->reads && !from_slot(it->row, cell)) return false;
                if (it->writes) return (cr_[it->row].d.flags & DEVOP_VEC) && cr_[it->row].d.bytes == cr_[i].d.bytes;
            }
            return false;                                       // never overwritten: part of the result
        };
        for (uint32_t i = 0; i < nrows(); ++i) {
            const ColRow& r = cr_[i];
            const uint64_t vec_bytes = r.d.bytes & ~(uint64_t)15u;
            if (r.d.kind == SAR_OP_MREDUCE) {
                bool all = true;
                for (int cell : r.mwrites) all = all && dead(i, cell);
                if (all) { fwd.flags[i] |= DEVOP_DEAD0; plan_.elided_bytes += vec_bytes * r.d.ndst; }
                continue;
            }
            if (r.c0 == r.c1) continue;
            if (dead(i, r.c0)) { fwd.flags[i] |= DEVOP_DEAD0; plan_.elided_bytes += vec_bytes; }
            if (r.d.kind == SAR_OP_XREDUCE && dead(i, r.c1)) { fwd.flags[i] |= DEVOP_DEAD1; plan_.elided_bytes += vec_bytes; }
        }
    }

    // Plan for few work items: nothing covers a row's round trip to memory there, and the rows of a group do not
    // depend on each other through memory.  Runs of up to four whole-vector rows of a group take their operands
    // together (DEVOP_JOIN on every row of a run but the first).  Two rows of a group can still meet in a value
    // slot -- both read the same cell and the first one keeps it for the second -- so a row that takes a slot which
    // a row of the run fills starts a run of its own.
    void mark_joins() {
        constexpr uint32_t kRun = 4;
        for (size_t g = 0; g + 1 < plan_.group_begin.size(); ++g) {
            uint32_t start = plan_.group_begin[g];
            bool start_plain = false;
            for (uint32_t i = plan_.group_begin[g]; i < plan_.group_begin[g + 1]; ++i) {
                DevOp& d = cr_[i].d;
                const bool plain = (d.flags & DEVOP_VEC) && d.kind != SAR_OP_MREDUCE;
                bool join = i > plan_.group_begin[g] && plain && start_plain && i - start < kRun;
                for (uint32_t p = start; p < i && join; ++p) {
                    const DevOp& e = cr_[p].d;
                    if (!(e.flags & DEVOP_PUT)) continue;
                    const uint32_t k = e.slots >> 16 & 0xffu;
                    if (((d.flags & DEVOP_GET0) && (d.slots & 0xffu) == k) || ((d.flags & DEVOP_GET1) && (d.slots >> 8 & 0xffu) == k)) join = false;
                }
                if (join) d.flags |= DEVOP_JOIN;
                else { start = i; start_plain = plain; }
            }
        }
    }

    // Vectors per lane and row where values are forwarded (bandwidth plan).  Two as a rule: what a row still loads
    // is little and far between, and two loads in flight per lane pay (ring at 16 and 32 ranks: 4 to 5 %).  One for a
    // plan that mostly stores -- the StragglAR tables and direct send two chunks' worth of cold reads and n chunks'
    // worth of stores to memory -- once the payload is far beyond the Infinity Cache: more and smaller work items with
    // streaming stores (see choose_launch) are the shape in which a kernel that does nothing else moves this mix
    // fastest, and the schedule gains the same 2 to 3 % (n = 8, 256 MiB per rank: 416 -> 404 us; 1 GiB: 1658 -> 1628).
    void choose_vectors() {
        plan_.two_vectors = false; store_heavy_ = false;
        if (!plan_.nslots || plan_.staged) return;
        uint64_t reads = 0, writes = 0;
        for (const auto& r : cr_) {
            const DevOp& d = r.d;
            const uint64_t b = d.bytes;
            if (d.kind == SAR_OP_MREDUCE) { reads += b * d.nsrc; writes += (d.flags & DEVOP_DEAD0) ? 0 : b * d.ndst; continue; }
            if (!(d.flags & DEVOP_GET1)) reads += b;
            if (d.kind != SAR_OP_COPY && !(d.flags & DEVOP_GET0)) reads += b;
            if (!(d.flags & DEVOP_DEAD0)) writes += b;
            if (d.kind == SAR_OP_XREDUCE && !(d.flags & DEVOP_DEAD1)) writes += b;
            writes += b * d.ndst;
        }
        store_heavy_ = all_found_ && writes >= 3 * reads && plan_.block >= 512 &&
                       env_.bytes_per_rank * (uint64_t)env_.n >= (1ull << 30);
        // Three value slots and more (halving-doubling) on payloads of 1 GiB and more: the slots of two vectors per lane are what limits the workgroups
        // resident on a compute unit, and one vector per lane runs level or ahead (n = 8, 1 GiB per rank: 2816 -> 2763 us;
        // n = 32 and 64, 2 GiB over all ranks: -2 and -3 %; n = 8 and 16 at 2 GiB: level).
        const bool slot_bound = plan_.nslots >= 3 && env_.bytes_per_rank * (uint64_t)env_.n >= (1ull << 30);
        plan_.two_vectors = env_.tune.col_vectors ? env_.tune.col_vectors == 2 : !store_heavy_ && !slot_bound;
    }

    void choose_launch() {
        // Cache policy of the launch (the column kernel takes one for all its rows).  Planned (2): when every re-read is
        // forwarded, what is still loaded is read exactly once: streaming loads (+1.5 % for the StragglAR table);
        // otherwise the re-reads are meant to find their data in the caches and nothing streams (streaming loads cost
        // 4-10 % there).
        // A launch in which no row reads what another wrote or read (the exchanges of a table on their own, a pre-work
        // on its own) has nothing to find in the caches either: streaming loads.  When all its rows are multi-source
        // rows, streaming stores as well: seven reads and one write per vector run 3 % faster with them (358 against
        // 369 us), and a pre-work that runs beside the straggler's delay then leaves no modified lines in the Infinity
        // Cache for the schedule to push out (n = 8, 1 GiB per rank: the schedule took 65 us longer behind a pre-work
        // with cached stores).
        // Streaming stores for every such plan once the payload is twice the Infinity Cache and more: a cached store
        // is fast while the cache takes it and is paid for when the line is pushed out, by this launch or the next.
        // Timed behind a restore that leaves the cache clean, cached stores look 3 to 12 % faster than they are (the
        // last 256 MB of the launch never reach memory inside the timed span); timed in a sequence of steps, each
        // inheriting what the one before left, streaming stores win: n = 8, 256 MiB per rank, ring 680 against 703 us,
        // halving-doubling 694 against 714, the exchanges alone 175 against 177 (1 GiB: 698 against 722); 64 MiB per
        // rank: ring 174 against 180, StragglAR 106.5 against 108.5.  Up to 32 MiB per rank (everything fits the
        // cache and the next step finds it there) cached stores stay ahead by 1 to 5 %.
        const int cp = env_.tune.cache_policy;
        bool only_multi_source = !cr_.empty();
        for (const auto& r : cr_) only_multi_source = only_multi_source && r.d.kind == SAR_OP_MREDUCE;
        const bool beyond_cache = env_.bytes_per_rank * (uint64_t)env_.n >= (512ull << 20);
        // (A plan that mostly stores, one vector per lane, payload far beyond the cache -- choose_vectors -- streamed its
        // stores before this rule and still does.)
        const uint32_t planned = all_found_ ? (beyond_cache || (store_heavy_ && !plan_.two_vectors) ? 2u : 1u)
                                            : no_reuse_ ? (only_multi_source || beyond_cache ? 2u : 1u) : 0u;
        plan_.policy = cp == 0 ? 0u : cp == 1 ? 2u : cp == 3 ? 1u : planned;

        // Dispatch order of the items.  All columns of one component before the next component keeps the resident
        // workgroups on few (rank, chunk) streams at a time (+3 to +5 % for the StragglAR tables, +2 % for ring at 64 MiB
        // per rank and more).  It only matters, and only pays, when the items outnumber the resident workgroups
        // severalfold and every row is vector-aligned; and it does not pay where a component reduces several pairs of
        // ranks in the same round (halving-doubling: -4 to -15 %).  Otherwise the items of one column, all components,
        // are dispatched together.
        uint32_t most = 0;
        bool aligned = true;
        for (size_t g = 0; g + 1 < plan_.group_begin.size(); ++g) {
            uint32_t reducing = 0;
            for (uint32_t i = plan_.group_begin[g]; i < plan_.group_begin[g + 1]; ++i) {
                reducing += cr_[i].d.kind != SAR_OP_COPY;
                aligned &= (cr_[i].d.flags & DEVOP_VEC) != 0;
            }
            most = std::max(most, reducing);
        }
        const uint64_t cbytes = plan_.column_bytes();
        const uint64_t items = (plan_.widest_row + cbytes - 1) / cbytes * plan_.comps.size();
        const uint64_t resident = (uint64_t)std::max(1, env_.compute_units) * (2048u / (uint32_t)plan_.block);
        plan_.component_major = most <= 1 && aligned && !plan_.staged && items >= 2 * resident;

        // Between rounds the waves of a workgroup only have to meet (no wait for their stores) when every lane
        // re-reads nothing but bytes it wrote itself: all rows whole vectors on vector boundaries.
        plan_.lane_local = true;
        for (const auto& r : cr_)
            if (!(r.d.flags & DEVOP_VEC) || (r.d.bytes & 15u) || (r.d.flags >> DEVOP_HEAD_SHIFT & 15u)) plan_.lane_local = false;
    }

    const ColumnEnv& env_;
    const std::vector<const Schedule*>& scheds_;
    const Schedule& s_;                 // the last schedule gives the chunking
    std::vector<char*>& ptrs_;
    ColumnPlan& plan_;
    const uint64_t chunk_bytes_;
    const int cells_per_rank_, ncells_;
    std::vector<ColRow> cr_;
    std::vector<std::vector<Ev>> ev_;
    bool all_found_ = false;            // every re-read of a column finds its operand in a slot
    bool no_reuse_ = false;             // no row reads a cell that an earlier row read or wrote
    bool store_heavy_ = false;          // every re-read forwarded, three times as many bytes stored as loaded, a large payload
};

}  // namespace

int plan_columns(const ColumnEnv& env, const std::vector<const Schedule*>& scheds, std::vector<DevOp>& rows,
                 std::vector<char*>& ptrs, ColumnPlan& plan, std::string* error) {
    return Planner(env, scheds, ptrs, plan).run(rows, error);
}

}  // namespace sar
