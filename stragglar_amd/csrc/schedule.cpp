// Host-side schedule layer: table parser, built-in comparators, validator and
// byte accounting.  The reference keeps none of this as data: every algorithm
// is an unrolled list of ncclSend/ncclRecv/reduce_add calls.  The builders
// below derive the same moves from index formulas and express each "receive
// into temp + reduce_add" as one fused row.
#include "schedule.hpp"

#include <algorithm>
#include <cctype>
#include <cstring>
#include <set>
#include <sstream>
#include <stdexcept>

namespace sar {

namespace {

Op copy_op(int src, int dst, int src_chunk, int dst_chunk, int nchunks = 1) {
    Op o; o.kind = SAR_OP_COPY; o.src_rank = src; o.dst_rank = dst;
    o.src_chunk = src_chunk; o.dst_chunk = dst_chunk; o.nchunks = nchunks; return o;
}
Op xreduce_op(int a, int b, int chunk, int nchunks = 1) {
    Op o; o.kind = SAR_OP_XREDUCE; o.dst_rank = a; o.src_rank = b;
    o.dst_chunk = chunk; o.src_chunk = chunk; o.nchunks = nchunks; return o;
}
Op reduce_into_op(int src, int dst, int src_chunk, int dst_chunk, int nchunks = 1) {
    Op o; o.kind = SAR_OP_REDUCE_INTO; o.src_rank = src; o.dst_rank = dst;
    o.src_chunk = src_chunk; o.dst_chunk = dst_chunk; o.nchunks = nchunks; return o;
}
Op mreduce_op(int owner, int chunk, int group, int bcast, int to_end) {
    Op o; o.kind = SAR_OP_MREDUCE; o.dst_rank = owner; o.src_rank = -1;
    o.dst_chunk = chunk; o.src_chunk = chunk; o.nchunks = 1; o.group = group; o.bcast = bcast; o.to_end = to_end; return o;
}

int mod(int a, int n) { return ((a % n) + n) % n; }

// ---- tiny scanner for the synthesizer text -------------------------------
struct Scanner {
    const char* p; const char* end;
    void ws() { while (p < end && (*p == ' ' || *p == '\t')) ++p; }
    bool lit(const char* s) {
        ws();
        size_t l = std::strlen(s);
        if ((size_t)(end - p) >= l && std::memcmp(p, s, l) == 0) { p += l; return true; }
        return false;
    }
    bool num(int* out) {
        ws();
        if (p >= end || !std::isdigit((unsigned char)*p)) return false;
        long v = 0;
        while (p < end && std::isdigit((unsigned char)*p)) { v = v * 10 + (*p - '0'); if (v > 1000000) return false; ++p; }
        *out = (int)v; return true;
    }
};

[[noreturn]] void fail(const std::string& m) { throw std::runtime_error(m); }

// One matching string, e.g. "TwoWayMatching: 4 -> 0, chunk_id: 1; 0 -> 4, chunk_id: 0".
void parse_matching(const char* b, const char* e, int round, std::vector<Op>& out) {
    Scanner s{b, e};
    int a, c, d, c2, a2, d2;
    if (s.lit("StragglerMatching:")) {
        if (!(s.num(&a) && s.lit("<->") && s.num(&d) && s.lit(",") && s.lit("chunk_id:") && s.num(&c)))
            fail("round " + std::to_string(round) + ": malformed StragglerMatching");
        out.push_back(xreduce_op(a, d, c));
    } else if (s.lit("OneWayMatching:")) {
        if (!(s.num(&a) && s.lit("->") && s.num(&d) && s.lit(",") && s.lit("chunk_id:") && s.num(&c)))
            fail("round " + std::to_string(round) + ": malformed OneWayMatching");
        out.push_back(copy_op(a, d, c, c));
    } else if (s.lit("TwoWayMatching:")) {
        if (!(s.num(&a) && s.lit("->") && s.num(&d) && s.lit(",") && s.lit("chunk_id:") && s.num(&c) && s.lit(";") &&
              s.num(&a2) && s.lit("->") && s.num(&d2) && s.lit(",") && s.lit("chunk_id:") && s.num(&c2)))
            fail("round " + std::to_string(round) + ": malformed TwoWayMatching");
        if (a2 != d || d2 != a) fail("round " + std::to_string(round) + ": TwoWayMatching names two different pairs");
        out.push_back(copy_op(a, d, c, c));
        out.push_back(copy_op(a2, d2, c2, c2));
    } else {
        fail("round " + std::to_string(round) + ": unknown matching '" + std::string(b, e) + "'");
    }
    s.ws();
    if (s.p != s.end) fail("round " + std::to_string(round) + ": trailing text in matching '" + std::string(b, e) + "'");
}

// Row list: any schedule of chunk moves, one row per line.
//   sar-rows <ranks> <parts>
//   round
//   copy <src_rank> <dst_rank> <src_chunk> <dst_chunk> [<nchunks>]
//   reduce <src_rank> <dst_rank> <src_chunk> <dst_chunk> [<nchunks>]     dst += src
//   xreduce <rank_a> <rank_b> <chunk> [<nchunks>]                         both sides get a + b
// '#' starts a comment.  The buffer is cut into <parts> chunks of size/parts elements.
Schedule parse_rows(const char* text, size_t len, int n) {
    Schedule sch; sch.name = "rows";
    const char* p = text; const char* end = text + len;
    bool header = false;
    int line_no = 0;
    while (p < end) {
        const char* eol = (const char*)std::memchr(p, '\n', (size_t)(end - p));
        if (!eol) eol = end;
        ++line_no;
        const char* b = p; const char* e = eol;
        if (const char* hash = (const char*)std::memchr(b, '#', (size_t)(e - b))) e = hash;
        while (b < e && std::isspace((unsigned char)*b)) ++b;
        while (e > b && std::isspace((unsigned char)e[-1])) --e;
        p = eol < end ? eol + 1 : end;
        if (b == e) continue;
        Scanner s{b, e};
        auto bad = [&](const std::string& why) { fail("line " + std::to_string(line_no) + ": " + why); };
        auto done = [&]() { s.ws(); if (s.p != s.end) bad("trailing text"); };
        if (!header) {
            if (!(s.lit("sar-rows") && s.num(&sch.n) && s.num(&sch.parts))) bad("expected 'sar-rows <ranks> <parts>'");
            done();
            if (sch.n != n) bad("the table is for " + std::to_string(sch.n) + " ranks, not " + std::to_string(n));
            if (sch.parts < 1) bad("parts must be positive");
            header = true;
            continue;
        }
        if (s.lit("round")) { done(); sch.rounds.emplace_back(); continue; }
        if (sch.rounds.empty()) bad("a row before the first 'round' line");
        int a = 0, d = 0, sc = 0, dc = 0, nch = 1;
        if (s.lit("xreduce")) {
            if (!(s.num(&a) && s.num(&d) && s.num(&sc))) bad("expected 'xreduce <rank_a> <rank_b> <chunk> [<nchunks>]'");
            s.ws(); if (s.p != s.end && !s.num(&nch)) bad("malformed chunk count");
            done();
            sch.rounds.back().push_back(xreduce_op(a, d, sc, nch));
            continue;
        }
        const bool is_copy = s.lit("copy");
        if (!is_copy && !s.lit("reduce")) bad("unknown row '" + std::string(b, e) + "'");
        if (!(s.num(&a) && s.num(&d) && s.num(&sc) && s.num(&dc))) bad("expected '<src_rank> <dst_rank> <src_chunk> <dst_chunk> [<nchunks>]'");
        s.ws(); if (s.p != s.end && !s.num(&nch)) bad("malformed chunk count");
        done();
        sch.rounds.back().push_back(is_copy ? copy_op(a, d, sc, dc, nch) : reduce_into_op(a, d, sc, dc, nch));
    }
    if (!header) fail("no 'sar-rows' line");
    if (sch.rounds.empty()) fail("no rounds found");
    return sch;
}

}  // namespace

Schedule parse_table(const char* text, size_t len, int n) {
    if (!text) fail("no text");
    {
        const char* b = text; const char* e = text + len;
        while (b < e && std::isspace((unsigned char)*b)) ++b;
        if ((size_t)(e - b) >= 8 && std::memcmp(b, "sar-rows", 8) == 0) {
            if (n < 2 || n > SAR_MAX_RANKS) fail("n must be in [2, " + std::to_string(SAR_MAX_RANKS) + "]");
            return parse_rows(text, len, n);
        }
    }
    if (n < 3 || n > SAR_MAX_RANKS) fail("n must be in [3, " + std::to_string(SAR_MAX_RANKS) + "]");
    Schedule sch; sch.n = n; sch.parts = n - 1; sch.stragglar_rules = true; sch.name = "stragglar";
    const char* p = text; const char* end = text + len;
    bool expect_list = false;
    while (p < end) {
        const char* eol = (const char*)std::memchr(p, '\n', (size_t)(end - p));
        if (!eol) eol = end;
        const char* b = p; const char* e = eol;
        while (b < e && std::isspace((unsigned char)*b)) ++b;
        while (e > b && std::isspace((unsigned char)e[-1])) --e;
        if (expect_list) {
            expect_list = false;
            Scanner s{b, e};
            int count;
            if (!s.num(&count)) fail("round " + std::to_string(sch.rounds.size()) + ": expected '<count> [...]'");
            std::vector<Op> ops; int found = 0;
            const char* q = s.p;
            while (q < e) {
                const char* q0 = (const char*)std::memchr(q, '\'', (size_t)(e - q));
                if (!q0) break;
                const char* q1 = (const char*)std::memchr(q0 + 1, '\'', (size_t)(e - q0 - 1));
                if (!q1) fail("round " + std::to_string(sch.rounds.size()) + ": unterminated quote");
                parse_matching(q0 + 1, q1, (int)sch.rounds.size(), ops);
                ++found; q = q1 + 1;
            }
            if (found != count)
                fail("round " + std::to_string(sch.rounds.size()) + " announces " + std::to_string(count) +
                     " matchings, " + std::to_string(found) + " found");
            sch.rounds.push_back(ops);
        } else if ((size_t)(e - b) > 6 && std::memcmp(b, "Round ", 6) == 0) {
            Scanner s{b + 6, e};
            int k;
            if (!s.num(&k) || k != (int)sch.rounds.size()) fail("rounds must be numbered 0,1,2,... in order");
            expect_list = true;
        }
        p = eol < end ? eol + 1 : end;
    }
    if (expect_list) fail("text ends after a 'Round' line");
    if (sch.rounds.empty()) fail("no rounds found");
    return sch;
}

// ---- built-in tables ----------------------------------------------------

namespace {

// allreduce_8GPU.cu:555-874 and allreduce_4GPU.cu:299-368, as text in the
// synthesizers' own format so that they go through the same parser.
const char* kStragglar8 =
    "Round 0\n1 ['StragglerMatching: 0 <-> 7, chunk_id: 0']\n"
    "Round 1\n2 ['StragglerMatching: 1 <-> 7, chunk_id: 1', 'OneWayMatching: 0 -> 3, chunk_id: 0']\n"
    "Round 2\n4 ['StragglerMatching: 2 <-> 7, chunk_id: 2', 'OneWayMatching: 1 -> 4, chunk_id: 1', "
    "'OneWayMatching: 0 -> 5, chunk_id: 0', 'OneWayMatching: 3 -> 6, chunk_id: 0']\n"
    "Round 3\n4 ['StragglerMatching: 3 <-> 7, chunk_id: 3', 'TwoWayMatching: 0 -> 2, chunk_id: 0; 2 -> 0, chunk_id: 2', "
    "'TwoWayMatching: 1 -> 5, chunk_id: 1; 5 -> 1, chunk_id: 0', 'TwoWayMatching: 4 -> 6, chunk_id: 1; 6 -> 4, chunk_id: 0']\n"
    "Round 4\n4 ['StragglerMatching: 4 <-> 7, chunk_id: 4', 'TwoWayMatching: 1 -> 3, chunk_id: 1; 3 -> 1, chunk_id: 3', "
    "'TwoWayMatching: 0 -> 5, chunk_id: 2; 5 -> 0, chunk_id: 1', 'TwoWayMatching: 2 -> 6, chunk_id: 2; 6 -> 2, chunk_id: 1']\n"
    "Round 5\n4 ['StragglerMatching: 5 <-> 7, chunk_id: 5', 'TwoWayMatching: 2 -> 4, chunk_id: 2; 4 -> 2, chunk_id: 4', "
    "'TwoWayMatching: 0 -> 3, chunk_id: 2; 3 -> 0, chunk_id: 3', 'TwoWayMatching: 1 -> 6, chunk_id: 3; 6 -> 1, chunk_id: 2']\n"
    "Round 6\n4 ['StragglerMatching: 6 <-> 7, chunk_id: 6', 'TwoWayMatching: 3 -> 5, chunk_id: 3; 5 -> 3, chunk_id: 5', "
    "'TwoWayMatching: 0 -> 2, chunk_id: 3; 2 -> 0, chunk_id: 4', 'TwoWayMatching: 1 -> 4, chunk_id: 3; 4 -> 1, chunk_id: 4']\n"
    "Round 7\n4 ['TwoWayMatching: 4 -> 6, chunk_id: 4; 6 -> 4, chunk_id: 6', 'TwoWayMatching: 0 -> 3, chunk_id: 4; 3 -> 0, chunk_id: 5', "
    "'TwoWayMatching: 1 -> 5, chunk_id: 4; 5 -> 1, chunk_id: 5', 'OneWayMatching: 7 -> 2, chunk_id: 6']\n"
    "Round 8\n4 ['TwoWayMatching: 0 -> 2, chunk_id: 5; 2 -> 0, chunk_id: 6', 'TwoWayMatching: 1 -> 4, chunk_id: 5; 4 -> 1, chunk_id: 6', "
    "'TwoWayMatching: 3 -> 6, chunk_id: 5; 6 -> 3, chunk_id: 6', 'OneWayMatching: 7 -> 5, chunk_id: 6']\n";

const char* kStragglar4 =
    "Round 0\n1 ['StragglerMatching: 0 <-> 3, chunk_id: 0']\n"
    "Round 1\n2 ['StragglerMatching: 1 <-> 3, chunk_id: 1', 'OneWayMatching: 0 -> 2, chunk_id: 0']\n"
    "Round 2\n2 ['StragglerMatching: 2 <-> 3, chunk_id: 2', 'TwoWayMatching: 0 -> 1, chunk_id: 0; 1 -> 0, chunk_id: 1']\n"
    "Round 3\n2 ['OneWayMatching: 3 -> 1, chunk_id: 2', 'TwoWayMatching: 0 -> 2, chunk_id: 1; 2 -> 0, chunk_id: 2']\n";

// ring_allreduce_helper, allreduce_8GPU.cu:146-198.  In step `step` of the
// reduce-scatter rank r receives chunk (r-step-1) from r-1 and adds it; in
// step `step` of the all-gather it receives chunk (r-step-1) in place.
Schedule build_ring(int n) {
    Schedule s; s.n = n; s.parts = n; s.name = "ring";
    for (int step = 1; step < n; ++step) {
        std::vector<Op> ops;
        for (int r = 0; r < n; ++r) {
            int from = mod(r - 1, n), c = mod(r - step - 1, n);
            ops.push_back(reduce_into_op(from, r, c, c));
        }
        s.rounds.push_back(ops);
    }
    for (int step = 0; step < n - 1; ++step) {
        std::vector<Op> ops;
        for (int r = 0; r < n; ++r) {
            int from = mod(r - 1, n), c = mod(r - step - 1, n);
            ops.push_back(copy_op(from, r, c, c));
        }
        s.rounds.push_back(ops);
    }
    return s;
}

// rhd_allreduce_helper, allreduce_8GPU.cu:221-532 / allreduce_4GPU.cu:196-278.
// Halving step k pairs r with r^(1<<k) over a block of n>>(k+1) chunks; a
// rank keeps the upper half of its block iff bit k of r is set.
Schedule build_rhd(int n) {
    Schedule s; s.n = n; s.parts = n; s.name = "rhd";
    int logn = 0; while ((1 << logn) < n) ++logn;
    std::vector<int> start(n, 0);
    for (int k = 0; k < logn; ++k) {
        int half = n >> (k + 1);
        std::vector<Op> ops;
        for (int r = 0; r < n; ++r) {
            int peer = r ^ (1 << k);
            int keep = start[r] + (((r >> k) & 1) ? half : 0);
            ops.push_back(reduce_into_op(peer, r, keep, keep, half));   // peer sends exactly the half r keeps
        }
        for (int r = 0; r < n; ++r) start[r] += ((r >> k) & 1) ? half : 0;
        s.rounds.push_back(ops);
    }
    for (int k = logn - 1; k >= 0; --k) {
        int half = n >> (k + 1);
        std::vector<Op> ops;
        for (int r = 0; r < n; ++r) {
            int peer = r ^ (1 << k);
            ops.push_back(copy_op(r, peer, start[r], start[r], half));
        }
        for (int r = 0; r < n; ++r) if ((r >> k) & 1) start[r] -= half;
        s.rounds.push_back(ops);
    }
    return s;
}

// direct_allreduce_helper, allreduce_8GPU.cu:60-113 / allreduce_4GPU.cu:56-92.
Schedule build_direct(int n) {
    Schedule s; s.n = n; s.parts = 1; s.name = "direct";
    s.rounds.push_back({xreduce_op(0, n - 1, 0)});
    int side = n / 2;
    for (int k = 1; k < side; k *= 2) {
        std::vector<Op> ops;
        for (int i = 0; i < k; ++i) {
            if (i + k < side) {
                ops.push_back(copy_op(i, i + k, 0, 0));
                ops.push_back(copy_op(n - 1 - i, n - 1 - i - k, 0, 0));
            }
        }
        if (!ops.empty()) s.rounds.push_back(ops);
    }
    for (auto& r : s.rounds) for (auto& o : r) o.to_end = 1;
    return s;
}

// The reference hands these two to NCCL on an (n-1)-rank sub-communicator
// (allreduce_8GPU.cu:890-895 and :129-134).  Here each becomes one round of
// multi-source reduces whose association is the ring order over the group.
Schedule build_prework(int n, bool allreduce) {
    Schedule s; s.n = n; s.parts = n - 1; s.name = allreduce ? "prework_ar" : "prework_rs";
    std::vector<Op> ops;
    for (int r = 0; r < n - 1; ++r) ops.push_back(mreduce_op(r, r, n - 1, allreduce ? 1 : 0, (allreduce && r == n - 2) ? 1 : 0));
    s.rounds.push_back(ops);
    return s;
}

}  // namespace

Schedule builtin(const std::string& alg, int n) {
    if (n < 2 || n > SAR_MAX_RANKS) fail("n must be in [2, " + std::to_string(SAR_MAX_RANKS) + "]");
    if (alg == "stragglar") {
        if (n == 8) return parse_table(kStragglar8, std::strlen(kStragglar8), 8);
        if (n == 4) return parse_table(kStragglar4, std::strlen(kStragglar4), 4);
        fail("the reference hard-codes StragglAR tables for n=4 and n=8 only; pass a synthesized table for n=" + std::to_string(n));
    }
    if (alg == "ring") return build_ring(n);
    if (alg == "rhd") {
        if (n & (n - 1)) fail("rhd needs a power-of-two n");
        return build_rhd(n);
    }
    if (alg == "direct") {
        if (n & 1) fail("direct needs an even n");
        return build_direct(n);
    }
    if (alg == "prework_rs" || alg == "prework_ar") {
        if (n < 3) fail("pre-work needs n >= 3");
        return build_prework(n, alg == "prework_ar");
    }
    fail("unknown algorithm '" + alg + "'");
}

// ---- lowering / accounting ------------------------------------------------

Range lower_range(const Schedule& s, const Op& op, uint64_t elems) {
    uint64_t chunk = elems / (uint64_t)s.parts;
    Range r;
    r.dst_off = (uint64_t)op.dst_chunk * chunk;
    r.src_off = (uint64_t)op.src_chunk * chunk;
    r.len = (uint64_t)op.nchunks * chunk;
    if (op.to_end) r.len = elems - r.dst_off;
    return r;
}

void byte_counts(const Schedule& s, uint64_t elems, int elem_size, uint64_t* algorithmic, uint64_t* reference_op) {
    uint64_t alg = 0, ref = 0;
    for (const auto& round : s.rounds) {
        for (const auto& op : round) {
            uint64_t b = lower_range(s, op, elems).len * (uint64_t)elem_size;
            switch (op.kind) {
                case SAR_OP_COPY: alg += 2 * b; ref += 2 * b; break;
                case SAR_OP_REDUCE_INTO: alg += 3 * b; ref += 5 * b; break;      // recv-to-temp 2 + reduce_add 3
                case SAR_OP_XREDUCE: alg += 4 * b; ref += 10 * b; break;         // both sides
                case SAR_OP_MREDUCE: {
                    uint64_t m = (uint64_t)op.group;
                    alg += (m + (op.bcast ? m : 1)) * b;
                    // ring over m ranks for this chunk: m-1 hops of (2 + 3), plus m-1 forwarding copies when all-gathered
                    ref += (m - 1) * 5 * b + (op.bcast ? (m - 1) * 2 * b : 0);
                    break;
                }
                default: break;
            }
        }
    }
    if (algorithmic) *algorithmic = alg;
    if (reference_op) *reference_op = ref;
}

uint64_t pad_bytes(uint64_t bytes, int n) {
    if (n < 2) return bytes;
    uint64_t raw = bytes / (uint64_t)(n - 1);
    uint64_t chunk = (raw / 1024 + 1) * 1024;
    return chunk * (uint64_t)(n - 1);
}

// ---- validation -------------------------------------------------------------

namespace {

struct Access { int rank; int lo, hi; bool write; int row; bool to_end; };   // chunk interval [lo, hi)

bool overlap(const Access& a, const Access& b, int parts) {
    if (a.rank != b.rank) return false;
    int ahi = a.to_end ? parts + 1 : a.hi, bhi = b.to_end ? parts + 1 : b.hi;
    return a.lo < bhi && b.lo < ahi;
}

}  // namespace

std::string validate(const Schedule& s) {
    std::ostringstream err;
    if (s.n < 2 || s.n > SAR_MAX_RANKS) return "rank count out of range";
    if (s.parts < 1) return "parts must be positive";
    const int n = s.n;
    std::vector<std::vector<char>> holds;   // StragglAR rules: rank x chunk -> holds the fully reduced chunk
    if (s.stragglar_rules) holds.assign(n, std::vector<char>(s.parts, 0));
    for (size_t ri = 0; ri < s.rounds.size(); ++ri) {
        const auto& round = s.rounds[ri];
        std::vector<Access> acc;
        std::vector<int> sends(n, 0), recvs(n, 0);
        auto newly = holds;
        for (size_t oi = 0; oi < round.size(); ++oi) {
            const Op& o = round[oi];
            auto bad = [&](const char* why) { err << "round " << ri << " row " << oi << ": " << why; return err.str(); };
            if (o.kind < SAR_OP_COPY || o.kind > SAR_OP_MREDUCE) return bad("unknown kind");
            if (o.dst_rank < 0 || o.dst_rank >= n) return bad("destination rank out of range");
            if (o.nchunks < 1) return bad("empty range");
            if (o.dst_chunk < 0 || o.dst_chunk + o.nchunks > s.parts) return bad("destination chunk out of range");
            if (o.kind == SAR_OP_MREDUCE) {
                if (o.group < 2 || o.group > n) return bad("group out of range");
                if (o.dst_rank >= o.group) return bad("owner outside its group");
                if (o.src_chunk != o.dst_chunk) return bad("multi-source reduce must keep the chunk index");
                for (int q = 0; q < o.group; ++q) {
                    acc.push_back({q, o.dst_chunk, o.dst_chunk + o.nchunks, false, (int)oi, o.to_end != 0});
                    if (o.bcast || q == o.dst_rank) acc.push_back({q, o.dst_chunk, o.dst_chunk + o.nchunks, true, (int)oi, o.to_end != 0});
                }
                continue;
            }
            if (o.src_rank < 0 || o.src_rank >= n) return bad("source rank out of range");
            if (o.src_rank == o.dst_rank) return bad("a rank cannot exchange with itself");
            if (o.src_chunk < 0 || o.src_chunk + o.nchunks > s.parts) return bad("source chunk out of range");
            if (o.kind == SAR_OP_XREDUCE && o.src_chunk != o.dst_chunk) return bad("exchange must use one chunk index");
            bool rmw = (o.kind == SAR_OP_XREDUCE || o.kind == SAR_OP_REDUCE_INTO);
            acc.push_back({o.dst_rank, o.dst_chunk, o.dst_chunk + o.nchunks, true, (int)oi, o.to_end != 0});
            if (rmw) acc.push_back({o.dst_rank, o.dst_chunk, o.dst_chunk + o.nchunks, false, (int)oi, o.to_end != 0});
            acc.push_back({o.src_rank, o.src_chunk, o.src_chunk + o.nchunks, false, (int)oi, o.to_end != 0});
            if (o.kind == SAR_OP_XREDUCE) acc.push_back({o.src_rank, o.src_chunk, o.src_chunk + o.nchunks, true, (int)oi, o.to_end != 0});
            if (s.stragglar_rules) {
                if (o.kind == SAR_OP_REDUCE_INTO) return bad("a StragglAR table has no one-sided reduce");
                if (o.nchunks != 1 || o.src_chunk != o.dst_chunk) return bad("a StragglAR table moves single chunks in place");
                if (o.kind == SAR_OP_XREDUCE) {
                    // synthesizer_pow2.py:217-220: round r pairs rank r with the straggler on chunk r
                    if (!((o.dst_rank == n - 1) ^ (o.src_rank == n - 1))) return bad("a StragglerMatching pairs one rank with rank n-1");
                    int other = o.dst_rank == n - 1 ? o.src_rank : o.dst_rank;
                    if (other != o.dst_chunk) return bad("rank r exchanges chunk r with the straggler");
                    if (holds[other][o.dst_chunk] || holds[n - 1][o.dst_chunk]) return bad("chunk exchanged with the straggler twice");
                    sends[o.dst_rank]++; sends[o.src_rank]++; recvs[o.dst_rank]++; recvs[o.src_rank]++;
                    newly[o.dst_rank][o.dst_chunk] = 1; newly[o.src_rank][o.dst_chunk] = 1;
                } else {
                    if (!holds[o.src_rank][o.src_chunk]) return bad("sender does not hold the fully reduced chunk it sends");
                    if (holds[o.dst_rank][o.dst_chunk]) return bad("receiver already holds that chunk");
                    sends[o.src_rank]++; recvs[o.dst_rank]++;
                    newly[o.dst_rank][o.dst_chunk] = 1;
                }
            }
        }
        for (size_t i = 0; i < acc.size(); ++i)
            for (size_t j = i + 1; j < acc.size(); ++j) {
                if (acc[i].row == acc[j].row) continue;
                if (!(acc[i].write || acc[j].write)) continue;
                if (overlap(acc[i], acc[j], s.parts)) {
                    err << "round " << ri << ": rows " << acc[i].row << " and " << acc[j].row
                        << " touch rank " << acc[i].rank << " on overlapping chunks and one of them writes";
                    return err.str();
                }
            }
        if (s.stragglar_rules) {
            for (int r = 0; r < n; ++r) {
                if (sends[r] > 1) { err << "round " << ri << ": rank " << r << " sends twice"; return err.str(); }
                if (recvs[r] > 1) { err << "round " << ri << ": rank " << r << " receives twice"; return err.str(); }
            }
            holds = newly;
        }
    }
    if (s.stragglar_rules) {
        if (s.parts != n - 1) return "a StragglAR table cuts the buffer into n-1 chunks";
        for (int r = 0; r < n; ++r)
            for (int c = 0; c < s.parts; ++c)
                if (!holds[r][c]) { err << "rank " << r << " never receives chunk " << c; return err.str(); }
    }
    return "";
}

}  // namespace sar
