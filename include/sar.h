/*
 * sar.h -- C ABI of the MI355X (gfx950) executor for emulated n-rank
 * AllReduce schedules (StragglAR, ring, recursive halving/doubling, direct).
 *
 * All emulated ranks live in one GPU's HBM; a schedule round becomes one
 * batched kernel launch of fused chunk moves and reduces.  The reference has
 * no library boundary for this path: its executors are functions inside a
 * single benchmark translation unit.  Each entry point below therefore names
 * the reference function (file:line under the reference checkout) whose role
 * it takes over.
 *
 * Conventions: every function returns 0 on success or a negative SAR_E*
 * code; sar_last_error() gives a thread-local message for the last failure on
 * the calling thread.  No exceptions cross the boundary.  A context is used
 * by one host thread at a time.  The caller owns host memory, the context
 * owns device memory.  There is no CPU fallback: without a usable HIP device
 * sar_create() fails.
 */
#ifndef SAR_H
#define SAR_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SAR_VERSION 100

enum {
    SAR_OK = 0,
    SAR_EINVAL = -1,      /* bad argument */
    SAR_ENODEV = -2,      /* no usable HIP device */
    SAR_ENOMEM = -3,      /* host or device allocation failed */
    SAR_EHIP = -4,        /* a HIP runtime call failed */
    SAR_EPARSE = -5,      /* schedule text not understood */
    SAR_ESCHED = -6,      /* schedule is not valid */
    SAR_ESTATE = -7       /* call made in the wrong state (e.g. run before prepare) */
};

enum { SAR_F32 = 0, SAR_F16 = 1, SAR_BF16 = 2 };

/* operation kinds of the schedule representation (one row of a round) */
enum {
    SAR_OP_COPY = 0,        /* dst chunk <- src chunk                       (a plain ncclSend/ncclRecv pair)        */
    SAR_OP_XREDUCE = 1,     /* s = a + b; a <- s; b <- s                    (exchange into temp + reduce_add twice) */
    SAR_OP_REDUCE_INTO = 2, /* dst += src                                   (recv into temp + reduce_add)           */
    SAR_OP_MREDUCE = 3      /* dst(s) <- ring-ordered sum over a rank group (the NCCL pre-work collectives)         */
};

/* why the rank buffers sit where they sit (sar_stats_t.spread_reason) */
enum {
    SAR_SPREAD_FOUND = 0,          /* two allocations in different regions of HBM were found: arena_spread = 1 */
    SAR_SPREAD_OFF = 1,            /* tuning.arena_spread is 0 */
    SAR_SPREAD_SMALL_PAYLOAD = 2,  /* less than 128 MiB over all ranks: the caches carry the schedule */
    SAR_SPREAD_UNKNOWN_DEVICE = 3, /* not a 288 GiB MI355X: the regions of this device are not known */
    SAR_SPREAD_NO_MEMORY = 4,      /* too little free device memory to look for a pair */
    SAR_SPREAD_NO_PAIR = 5,        /* the probe times of the candidates did not fall into two populations with a clear gap */
    SAR_SPREAD_TOO_LARGE = 6,      /* half the ranks take more than 32 GiB */
    SAR_SPREAD_ADOPTED = 7,        /* caller-owned buffers (sar_adopt_ranks) are taken where they are */
    SAR_SPREAD_POOL_BUSY = 8       /* the GPU's pair of allocations has no room left beside the leases other contexts hold */
};

#define SAR_MAX_RANKS 64
#define SAR_MAX_RANK_BYTES (1ull << 40)   /* largest bytes_per_rank any call accepts */

typedef struct sar_ctx sar_ctx;
typedef struct sar_schedule sar_schedule;

/* one lowered schedule row, as reported by sar_schedule_op() */
typedef struct sar_op_info {
    int32_t kind;        /* SAR_OP_*                                                        */
    int32_t dst_rank;    /* COPY/REDUCE_INTO/MREDUCE: destination; XREDUCE: first side      */
    int32_t src_rank;    /* COPY/REDUCE_INTO: source; XREDUCE: second side; MREDUCE: -1     */
    int32_t dst_chunk;   /* first chunk written, in units of the schedule's `parts`         */
    int32_t src_chunk;   /* first chunk read                                                */
    int32_t nchunks;     /* consecutive chunks moved                                        */
    int32_t group;       /* MREDUCE: ranks 0..group-1 take part                             */
    int32_t bcast;       /* MREDUCE: 1 = every group member receives the result             */
    int32_t to_end;      /* 1 = the range also takes the elements past parts*chunk          */
} sar_op_info;

typedef struct sar_stats_t {
    uint64_t algorithmic_bytes;    /* minimum bytes the prepared main schedule must move (see sar_schedule_bytes) */
    uint64_t reference_op_bytes;   /* bytes of the reference's own op sequence (temp staging + reduce_add)        */
    uint64_t prework_bytes;        /* algorithmic bytes of the prepared pre-work schedule, 0 if none              */
    int32_t rounds;                /* rounds of the main schedule                                                 */
    int32_t launches;              /* kernel launches per sar_run (main + pre-work, sleep excluded)               */
    int32_t ops;                   /* rows of the main schedule                                                   */
    int32_t uses_graph;            /* 1 if sar_run replays a hipGraph                                             */
    int32_t executor;              /* executor the main schedule was lowered for: 0 per round, 1 column           */
    int32_t col_block;             /* column executor: threads per workgroup in use (0 otherwise)                 */
    int32_t col_slots;             /* column executor: value slots per lane in use (0 = no forwarding)            */
    int32_t col_components;        /* column executor: independent row components (work items per column)        */
    uint64_t forwarded_bytes;      /* part of algorithmic_bytes that the column executor takes from value slots   */
                                   /* in LDS instead of loading it again from the rank buffers                    */
    int32_t fused_prework;         /* 1 if sar_run(delay 0) runs pre-work + main schedule as a single launch      */
    int32_t arena_spread;          /* 1 if the two halves of the rank buffers lie in different regions of HBM    */
    uint64_t elided_store_bytes;   /* part of algorithmic_bytes that the column executor does not store because a */
                                   /* later row overwrites it and every reader in between takes it from a slot    */
    int32_t spread_reason;         /* SAR_SPREAD_*: why arena_spread is what it is                                */
    int32_t spread_candidates;     /* the search for the two allocations (last one this context ran): candidates  */
    float spread_same_ms;          /* probed, the region probe's time for two windows in one region (the fastest  */
    float spread_pair_ms;          /* of four pairs) and for the pair that was kept (the slower of its two probes), and */
    uint64_t spread_search_bytes;  /* the most device memory held at a time while looking, the pair included      */
                                   /* (the search is the GPU's, shared: whichever context ran it last)            */
    uint64_t fused_forwarded_bytes;    /* the same two figures for the single launch of pre-work + main schedule  */
    uint64_t fused_elided_store_bytes; /* (fused_prework = 1), out of algorithmic_bytes + prework_bytes           */
    uint64_t placed_pool_bytes;    /* the GPU's pair of allocations in different regions of HBM, shared by all     */
    int32_t placed_pool_contexts;  /* contexts of the process: its size (both together) and the contexts attached  */
    int32_t main_launches;         /* `launches` split: kernel launches of the main schedule ...                  */
    int32_t prework_launches;      /* ... and of the pre-work when it runs on its own (beside a delay, or in front */
                                   /* of the schedule when there is no single launch for both)                    */
} sar_stats_t;

/* run-time tunables of the executors; sar_get_tuning() reports the defaults */
typedef struct sar_tuning_t {
    int32_t block;        /* threads per workgroup: 256 or 512                                       */
    int32_t unroll;       /* 16-byte vectors per thread and stream: 1, 2, 4 or 8                     */
    int32_t order;        /* 0 = tiles op by op, 1 = tiles of a round's ops interleaved              */
    int32_t cache_policy; /* 0 = all accesses cached, 1 = all streaming (nontemporal), 3 = streaming */
                          /*     loads and cached stores, 2 = planned (default).  One launch per     */
                          /*     round plans per row: streaming unless the data is read again within */
                          /*     `reuse_rounds`.  The column executor has one policy per launch: it  */
                          /*     plans streaming loads when every re-read is forwarded (else all     */
                          /*     cached), and streaming stores as well once the rank buffers add up  */
                          /*     to 512 MiB and more: a cached store is only paid for when the line  */
                          /*     is pushed out of the 256 MB Infinity Cache, by this launch or the   */
                          /*     next, and in a sequence of steps streaming stores are 1 - 3 % ahead */
    int32_t reuse_rounds; /* look-ahead of policy 2, in rounds                                       */
    int32_t reverse_odd;  /* 1 = odd rounds walk their tiles backwards (keeps the cache tail warm)   */
    int32_t segments;     /* >1: cut every row into this many pieces and run the whole schedule      */
                          /*     piece by piece (smaller cache footprint between rounds); 0 = choose */
                          /*     from the size of the widest round                                    */
    int32_t executor;     /* 0 = one launch per round; 1 = column executor: one launch for the whole */
                          /*     main schedule, each workgroup walking all rounds for its own range  */
                          /*     of within-chunk offsets (schedules with MREDUCE rows fall back to   */
                          /*     0); 2 = whichever a small cost model expects to be faster (default) */
    int32_t col_wgs;      /* column executor: most workgroups per compute unit in the grid (they stride over */
                          /*     the work items); 0 = chosen by the library (default)                       */
    int32_t col_block;    /* column executor: threads per workgroup = 16-byte vectors per column     */
                          /*     (256, 512 or 1024; 0 = chosen from the number of columns)           */
    int32_t col_forward;  /* column executor: 1 = a value a lane wrote in an earlier round and needs  */
                          /*     again is kept in LDS and not loaded again (same bits);              */
                          /*     0 = every operand is loaded from its rank buffer                    */
    int32_t col_slots;    /* column executor: most values kept per lane (0 = chosen by the planner)  */
    int32_t col_light_sync; /* column executor: 1 = between rounds the waves of a workgroup only meet   */
                          /*     (no wait for their stores) whenever no lane reads bytes another lane */
                          /*     wrote; 0 = always a full barrier                                     */
    int32_t col_latency_plan; /* column executor: the plan for few work items (a workgroup copies the */
                          /*     rows of its item into LDS first, one vector per lane): 0 = never, 1 = */
                          /*     when there are at most eight work items per compute unit, 2 = always */
    int32_t col_split;    /* column executor: 1 = rows that share no rank-chunk cell (for the four   */
                          /*     algorithms: rows of different chunk indices) form work items of     */
                          /*     their own, one per component and column; 0 = one item per column   */
                          /*     walks all rows in round order                                       */
    int32_t col_fuse_prework; /* column executor: 1 = sar_run with delay 0 runs pre-work and main     */
                          /*     schedule as one launch (the pre-work's result for a chunk goes to   */
                          /*     that chunk's exchange in a value slot); with a delay the pre-work   */
                          /*     stays a launch of its own, overlapping the straggler's absence      */
    int32_t col_elide_stores; /* column executor: 1 = a forwarded value whose stored copy nobody loads  */
                          /*     before a later row overwrites it (partial sums of ring and halving- */
                          /*     doubling, the pre-work's result in a same-launch run) is not stored;*/
                          /*     the buffers after sar_run are the same either way                  */
    int32_t col_fuse_chains; /* column executor: 1 = a chain of one-sided reduces whose partial sums are  */
                          /*     neither stored nor read by anyone else (a ring's reduce-scatter)   */
                          /*     runs as one multi-source row, all its cold operands loaded together */
                          /*     (in the plan for few work items, where the round trips are the cost;  */
                          /*     2 = in every plan: measured 1 to 7 % slower where memory is the bound)      */
    int32_t col_fuse_copies; /* column executor: 1 = copies of a value that an earlier row of the work   */
                          /*     item still holds are issued by that row as extra stores, and the    */
                          /*     copy rows (with their round boundaries) go away, where that was     */
                          /*     measured to pay: the plan for few work items, payloads up to 768    */
                          /*     MiB, plans whose value slots limit the workgroups per CU;           */
                          /*     2 = in every plan; 0 = never                                        */
    int32_t arena_spread; /* sar_alloc_ranks: 1 = for payloads of 128 MiB and more, half the ranks go   */
                          /*     into an allocation that a short timing probe has shown to lie in    */
                          /*     another region of HBM than the first half's (MI355X: buffers in     */
                          /*     different thirds of the 288 GiB disturb each other less).  The two  */
                          /*     allocations are ONE pair per GPU and process, shared by all contexts */
                          /*     and released with the last context that used it; ranks back to back */
                          /*     when no such pair is found or the device lacks the room; 0 = never  */
    int32_t col_prework;  /* 1 = multi-source rows run in the column kernel as well: the pre-work that      */
                          /*     overlaps the straggler's delay is one column launch on the second stream,  */
                          /*     and so is a schedule that consists of such rows (the pre-work timed on its */
                          /*     own); 0 = they run in the multi-source kernel, one launch per round.       */
                          /*     Rows that are not whole 16-byte vectors on vector boundaries always do     */
    int32_t col_depth_first; /* column executor, outside the plan for few work items: 1 = a work item takes a  */
                          /*     row as soon as the values it consumes exist (a reduce tree is walked depth   */
                          /*     first: log2 n values alive at a time instead of n/2, so fewer value slots    */
                          /*     and more workgroups per compute unit); rows that touch a common chunk of a   */
                          /*     rank keep their order, so the bits are the same; 0 = round order             */
    int32_t col_vectors;  /* column executor with value slots, outside the plan for few work items: 16-byte     */
                          /*     vectors a lane moves per row, 1 or 2; 0 = chosen by the planner (two, except    */
                          /*     for plans that mostly store, on payloads of 1 GiB and more)                     */
} sar_tuning_t;

/* ---- library ------------------------------------------------------- */
int sar_version(void);
const char* sar_last_error(void);

/* Number of HIP devices.  Replaces cudaGetDeviceCount + "Need at least %d
 * GPUs" (allreduce_8GPU.cu:932-937): one device is enough here. */
int sar_device_count(int* count);

/* pad_buffers.py:31-48: chunk = (bytes/(n-1)/1024 + 1)*1024, padded =
 * chunk*(n-1).  Always grows, also when bytes is already divisible. */
uint64_t sar_pad_bytes(uint64_t bytes, int n);

/* ---- schedules (host only; usable without a GPU) -------------------- */

/* Parse a table in the text format the reference synthesizers print
 * (synthesizer_pow2.py:241-247, matching strings :54,:71,:84).  Closes the
 * reference's manual step "translate the output into ncclSend/ncclRecv by
 * hand" (README.md:35).
 * A text whose first line is "sar-rows <ranks> <parts>" is read as a row list
 * instead, for schedules the matching strings cannot express: after a line
 * "round", one row per line,
 *   copy    <src_rank> <dst_rank> <src_chunk> <dst_chunk> [<nchunks>]
 *   reduce  <src_rank> <dst_rank> <src_chunk> <dst_chunk> [<nchunks>]   (dst += src)
 *   xreduce <rank_a> <rank_b> <chunk> [<nchunks>]                        (both get a + b)
 * with '#' comments; chunks are size/parts elements.  Such a table is checked
 * for ranges and for rows of one round that touch the same chunk of a rank
 * with one of them writing, not for being an AllReduce. */
int sar_schedule_parse(const char* text, size_t len, int n, sar_schedule** out);

/* Built-in tables.  alg is one of
 *   "stragglar"   the table hard-coded in stragglar_allreduce_helper
 *                 (allreduce_8GPU.cu:555-874 for n=8, allreduce_4GPU.cu:299-368 for n=4)
 *   "ring"        ring_allreduce_helper  (allreduce_8GPU.cu:146-198), any n >= 2
 *   "rhd"         rhd_allreduce_helper   (allreduce_8GPU.cu:221-532, allreduce_4GPU.cu:196-278), n a power of two
 *   "direct"      direct_allreduce_helper (allreduce_8GPU.cu:60-113, allreduce_4GPU.cu:56-92), even n
 *   "prework_rs"  the (n-1)-rank in-place ncclReduceScatter (allreduce_8GPU.cu:890-895, reducescatter.cu:103-108)
 *   "prework_ar"  the (n-1)-rank ncclAllReduce before `direct` in delay mode (allreduce_8GPU.cu:129-134) */
int sar_schedule_builtin(const char* alg, int n, sar_schedule** out);

/* Structural checks: rank/chunk bounds; no row of a round writes a range that
 * another row of the same round reads or writes; for StragglAR tables also the
 * synthesizers' own rules (valid_round, synthesizer_pow2.py:86-103: one send
 * and one receive per rank and round; senders hold what they send, :47,:58-59;
 * termination with every rank holding every chunk, :213).  On failure the
 * reason is copied into msg (if cap > 0) and SAR_ESCHED is returned. */
int sar_schedule_validate(const sar_schedule* s, char* msg, size_t cap);

int sar_schedule_ranks(const sar_schedule* s);
int sar_schedule_parts(const sar_schedule* s);   /* chunks per rank buffer: n-1 (stragglar), n (ring, rhd), 1 (direct) */
int sar_schedule_rounds(const sar_schedule* s);
int sar_schedule_round_ops(const sar_schedule* s, int round);
int sar_schedule_op(const sar_schedule* s, int round, int index, sar_op_info* out);

/* Bytes one execution moves for `elems` elements of `elem_size` bytes per
 * rank.  algorithmic: COPY 2NE, REDUCE_INTO 3NE, XREDUCE 4NE, MREDUCE
 * (sources + destinations)NE.  reference_op: the reference's own sequence for
 * the same rows (recv-to-temp 2NE + reduce_add 3NE per receiving side). */
int sar_schedule_bytes(const sar_schedule* s, uint64_t elems, int elem_size,
                       uint64_t* algorithmic, uint64_t* reference_op);

void sar_schedule_free(sar_schedule* s);

/* ---- device context -------------------------------------------------- */

/* Replaces the per-process setup of main() (allreduce_8GPU.cu:939-963): one
 * device, one stream for the schedule (and the straggler's wait in front of it)
 * and one for the pre-work of the ranks that are on time. */
int sar_create(int device, sar_ctx** out);
void sar_destroy(sar_ctx* ctx);

/* Rank buffers, replacing cudaMallocAsync(d_buffers[i]) (allreduce_8GPU.cu
 * :977-990).  No temp buffers exist: exchanges are fused.  All ranks share one
 * arena; rank r starts at r*stride, stride = bytes rounded up to 2 MiB (with
 * tuning.arena_spread the upper half of the ranks starts over in the second
 * of the GPU's two placed allocations).  bytes_per_rank: a positive multiple of the element size, at
 * most SAR_MAX_RANK_BYTES. */
int sar_alloc_ranks(sar_ctx* ctx, int n, uint64_t bytes_per_rank, int dtype);

/* Use caller-owned device buffers as the rank buffers instead of the arena: device_ptrs[r] is rank r's
 * buffer of bytes_per_rank bytes on the context's GPU; the buffers must not overlap and stay valid until
 * the next sar_alloc_ranks / sar_adopt_ranks / sar_destroy; the context never frees them.  This is what
 * a caller holding one flat gradient tensor per emulated rank needs (the role of tensors[0].data_ptr() in
 * allreduce_stragglar, implementation/custom_backend/src/dummy.cpp:256-271).  The caller orders its own
 * work on those buffers against sar_run (which blocks until the result is complete). */
int sar_adopt_ranks(sar_ctx* ctx, int n, void* const* device_ptrs, uint64_t bytes_per_rank, int dtype);

/* Device address of rank r's buffer (d_buffers[r] of allreduce_8GPU.cu:977-990), for callers that run their own
 * kernels on the rank buffers or hand them on; valid until the ranks are allocated or adopted anew. */
int sar_rank_pointer(sar_ctx* ctx, int rank, void** device_ptr);

/* n rows of bytes_per_row bytes back to back in ONE virtual address range, row r at *base + r * bytes_per_row: memory
 * for a caller that keeps the emulated ranks as the rows of one [n, numel] tensor, as the one-process counterpart of
 * the reference's backend does (the tensor handed to dist.all_reduce, implementation/custom_backend/example.py:21-29),
 * and then passes the row addresses to sar_adopt_ranks.  With the tuning's arena_spread on, a 288 GiB device and 128 MiB
 * or more in all, rows [0, ceil(n/2)) and the rest lie in two physical allocations that were found to sit in
 * different regions of HBM (the search sar_alloc_ranks uses) and are mapped next to each other, which rows of an
 * ordinary allocation cannot have; *placed says whether (may be null), *reason why not (SAR_SPREAD_*, may be null).
 * Otherwise a plain allocation.  The rows belong to the context: valid until the next sar_alloc_rows, sar_free_rows
 * or sar_destroy; rank buffers adopted from them are dropped with them.  The two allocations are the GPU's one pair
 * that all contexts of the process share (see sar_alloc_ranks); the rows take the place across its junction, which
 * one block of rows can hold at a time (a second one is a plain allocation, reason SAR_SPREAD_POOL_BUSY). */
int sar_alloc_rows(sar_ctx* ctx, int n, uint64_t bytes_per_row, void** base, int* placed, int* reason);
int sar_free_rows(sar_ctx* ctx);

int sar_upload(sar_ctx* ctx, int rank, uint64_t byte_off, const void* host, uint64_t bytes);
int sar_download(sar_ctx* ctx, int rank, uint64_t byte_off, void* host, uint64_t bytes);

/* fill_pattern (allreduce_8GPU.cu:41-45) on elements [elem_off, elem_off+elems) of one rank. */
int sar_fill_const(sar_ctx* ctx, int rank, uint64_t elem_off, uint64_t elems, double value);

/* The reference's per-iteration self-check fill (allreduce_8GPU.cu:1011-1021,
 * allreduce_4GPU.cu:535-545): rank i <- i+base; with delay < 0 `direct`
 * pre-fills ranks < n-1, and `stragglar` chunk i of rank i < n-1, with the sum
 * of the first n-1 constants. */
int sar_fill_reference_pattern(sar_ctx* ctx, const char* alg, float delay_ms, int base);

/* Seeded synthetic inputs generated on the device, counter-based so that the
 * value of (seed, rank, element) does not depend on launch shape.
 * uniform: lo + (hi-lo)*k/2^24 with k the top 24 bits of a 64-bit mix.
 * normal:  mean + std*(sum of 12 such uniforms - 6)  (Irwin-Hall). */
int sar_fill_uniform(sar_ctx* ctx, int rank, uint64_t seed, double lo, double hi);
int sar_fill_normal(sar_ctx* ctx, int rank, uint64_t seed, double mean, double std);

/* Keep / bring back a device-side copy of all rank buffers (the reference
 * re-fills before every iteration, allreduce_8GPU.cu:1009-1026).  sar_restore
 * copies with streaming stores, as the fills store: a run that follows starts
 * with nothing of its inputs in the caches and no modified lines of the copy
 * in the Infinity Cache to push out. */
int sar_snapshot(sar_ctx* ctx);
int sar_restore(sar_ctx* ctx);

/* 1 if every rank buffer holds the same bits over its first parts*chunk elements. */
int sar_ranks_identical(sar_ctx* ctx, uint64_t elems, int* identical);

int sar_get_tuning(sar_ctx* ctx, sar_tuning_t* out);
/* Takes effect at the next sar_prepare.  A plan prepared under the old values is dropped: sar_run, sar_stats
 * and the other calls that need a plan return SAR_ESTATE until sar_prepare has run again. */
int sar_set_tuning(sar_ctx* ctx, const sar_tuning_t* in);

/* Lower `main` (and the optional pre-work run before it in delay mode) onto
 * the allocated ranks: row tables in device memory for the executor the
 * tuning selects (see sar_tuning_t), launch shapes, and with use_graph != 0 a
 * captured hipGraph of the main schedule.  Replaces the unrolled bodies of
 * the *_allreduce_helper functions. */
int sar_prepare(sar_ctx* ctx, const sar_schedule* prework, const sar_schedule* main_sched, int use_graph);

/* One timed execution = one call of stragglar_allreduce / ring_allreduce /
 * ... (delay < 0, allreduce_8GPU.cu:900-905) or of their *_delay variants
 * (delay >= 0, :876-898): start event, the straggler's stream sleeps
 * delay_ms while the pre-work runs, then the rounds, stop event, block on
 * stop.  elapsed_ms is stop - start as in the reference (:1052). */
int sar_run(sar_ctx* ctx, float delay_ms, float* elapsed_ms);

/* sar_adopt_ranks + sar_prepare + sar_run(delay 0, or < 0 without pre-work) in one call that allocates nothing on the
 * device.  No counterpart in the reference; it is for callers that cannot allocate: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  The row tables that sar_prepare would put in
 * memory of its own go into an array that is part of the library image, sar_static_scratch_bytes() (1 MiB) per
 * GPU, held until the process ends; a schedule whose tables need more is refused with SAR_EINVAL (the n = 8
 * tables take a few KiB, a 64-rank ring about half a MiB).  `stream` is the caller's hipStream_t (NULL = the
 * null stream): the tables are copied and the kernels launched on it, and the call returns when it has drained
 * and the result is complete (so `stream` itself must not be capturing: the call is for a process that has a
 * capture open elsewhere, or may not allocate for other reasons; the calling thread runs in relaxed capture mode
 * for the duration of the call, since thread-local and global mode refuse hipStreamSynchronize on any stream; the
 * table copies are hipMemcpyAsync from ordinary host memory, staged by the runtime).  device_ptrs as for sar_adopt_ranks (checked the same way); the default tuning
 * applies.  No context is needed or touched.  All calls on one GPU share the one array, which keeps the last
 * call's tables; the library lets them take turns (a per-GPU lock held from the first table copy until the stream
 * has drained), so calls from several threads are safe and run one after the other. */
int sar_run_static(int device, void* stream, const sar_schedule* prework, const sar_schedule* main_sched, int n,
                   void* const* device_ptrs, uint64_t bytes_per_rank, int dtype);
uint64_t sar_static_scratch_bytes(void);

/* Same as sar_run with delay < 0 and no graph, with an event pair around
 * every launch: ms[i] is the duration of launch i (at most cap written,
 * *count = launches). */
int sar_run_profiled(sar_ctx* ctx, float* ms, int cap, int* count);

/* Algorithmic bytes of each launch of the prepared main schedule, in launch
 * order (the denominator-free half of a per-kernel roofline figure). */
int sar_launch_bytes(sar_ctx* ctx, uint64_t* bytes, int cap, int* count);

/* What the memory system delivers for a mix of read and written streams laid over the rank buffers where they
 * are: the yardstick for the data kernels (no counterpart in the reference, which is bound by its links).  A job
 * is nread streams read and nwrite streams written, each `bytes` long, starting byte_off into the named ranks'
 * buffers; every 16-byte vector written is the fp32 sum of the job's read streams.  A rank named on both sides is
 * updated in place, as the two sides of an exchange are (allreduce_8GPU.cu:564-578 followed by reduce_add :29-34).
 * All jobs of a call run in one launch of a kernel that does nothing else, in 54 (one job) or 108 shapes --
 * 256/512/1024 threads x 1/2/4 vectors per thread x cached / streaming loads with cached stores / streaming loads and stores x one tile per workgroup or a
 * resident grid x jobs one after the other or taking turns --, each timed `reps` times with events after one
 * warm-up launch; the result names the fastest shape.  THE RANK BUFFERS ARE OVERWRITTEN. */
typedef struct sar_probe_job {
    int32_t nread, nwrite;            /* 0..8 each, not both 0; all jobs of a call have the same nread */
    int32_t read_rank[8], write_rank[8];
    uint64_t byte_off;                /* into each named rank buffer; the streams must start on 16-byte boundaries */
} sar_probe_job;
typedef struct sar_probe_result {
    float best_ms, worst_ms;          /* fastest and slowest shape (each the minimum over its reps) */
    int32_t block, unroll, nontemporal, persistent, interleave;      /* the fastest shape; nontemporal: 0 = cached accesses, */
                                      /* 1 = streaming loads and cached stores, 2 = streaming loads and stores */
    int32_t variants;                 /* shapes tried */
    uint64_t bytes_moved;             /* (nread + nwrite) * bytes summed over the jobs */
    float variant_ms[108];            /* every shape's time, in the order they are tried: threads 256, 512, 1024 (slowest     */
                                      /* index) x vectors 1, 2, 4 x the three cache modes x tile per workgroup, resident grid x */
                                      /* jobs one after the other, taking turns (fastest index; one job: this level is absent) */
} sar_probe_result;
int sar_probe_streams(sar_ctx* ctx, int njobs, const sar_probe_job* jobs, uint64_t bytes, int reps, sar_probe_result* out);

/* The two decisions sar_alloc_ranks takes when it looks for a second allocation in another region of HBM (tuning
 * arena_spread), as functions of the region probe's times alone -- no device is touched; tests feed them recorded
 * times.  No counterpart in the reference (one buffer per GPU: allreduce_8GPU.cu:977-990).
 * sar_spread_yardstick: neighbours_ms = the probe's time for three pairs of neighbouring windows of the first
 * allocation, ends_ms = for its first and last window.  *yardstick_ms = ends_ms, the time of two distant windows that
 * share a region (or the median neighbouring pair, should that be faster).  Returns 0, or 1 when the ends are so much
 * faster than the median neighbouring pair that a region boundary must run through the allocation (the search then
 * sets it aside and starts from the next one).
 * sar_spread_is_elsewhere: 1 when a candidate's probe time against the first allocation says "another region"
 * (clearly below the yardstick), else 0.  Negative = SAR_EINVAL. */
int sar_spread_yardstick(const float* neighbours_ms, float ends_ms, float* yardstick_ms);
int sar_spread_is_elsewhere(float yardstick_ms, float probe_ms);
/* The verdict on a whole search: probe_ms[0..n) are the candidates' times against the first allocation.  Returns 1 and
 * *pick = the candidate to take (the fastest) when it is clearly below the yardstick and the times fall into two
 * populations -- sorted, they jump by 4 % and more somewhere below the limit -- or all lie clearly below the yardstick;
 * else 0 and *pick = -1: the ranks then sit in one ordinary allocation (SAR_SPREAD_NO_PAIR).  Times <= 0 are failed
 * probes and say nothing. */
int sar_spread_pick(float yardstick_ms, const float* probe_ms, int n, int* pick);

/* Ticks of the device's constant-rate wall clock that delay_ms lasts: the
 * figure the CLI prints as "Sleep cycles" (calculate_sleep_cycles,
 * allreduce_8GPU.cu:47-58, uses ms * clockRate_kHz of the shader clock). */
int sar_sleep_ticks(sar_ctx* ctx, float delay_ms, int64_t* ticks);

/* What sar_prepare planned (launches, executor, column width, components, value slots, forwarded bytes). */
int sar_stats(sar_ctx* ctx, sar_stats_t* out);

/* The tuning a new context starts with (no device needed). */
int sar_default_tuning(sar_tuning_t* out);

/* What sar_prepare would decide for `n` rank buffers of `bytes_per_rank` bytes, worked out on the host alone:
 * no device, no context, nothing is allocated.  `tuning` NULL = the defaults; `compute_units` 0 = 256 (MI355X).
 * No counterpart in the reference, whose executors are fixed code (allreduce_8GPU.cu:555-874); meant for tools
 * and tests that inspect a plan. */
int sar_plan(const sar_schedule* prework, const sar_schedule* main_schedule, int n, uint64_t bytes_per_rank, int dtype,
             const sar_tuning_t* tuning, int compute_units, sar_stats_t* out);

/* One row of the column executor's plan, as sar_plan_rows() reports it.  A work item of the kernel is one
 * component for one column (a range of within-chunk offsets); it walks the component's rows in this order. */
typedef struct sar_plan_row {
    int32_t kind;        /* SAR_OP_*                                                                           */
    int32_t component;   /* rows of different components never touch the same chunk of a rank                   */
    int32_t group;       /* rows of one component and round; the workgroup meets at a barrier after each group  */
    int32_t vector;      /* 1 = runs as 16-byte vectors, 0 = element by element                                 */
    int32_t dst_rank;    /* rank of p0 (COPY/REDUCE_INTO: destination; XREDUCE: first side; MREDUCE: -1)        */
    int32_t src_rank;    /* rank of p1 (source / second side; MREDUCE: -1)                                      */
    uint64_t dst_off;    /* byte offset in dst_rank's buffer of the row's first whole vector                    */
    uint64_t src_off;    /* the same for src_rank                                                               */
    uint64_t bytes;      /* length from there                                                                   */
    int32_t head_bytes;  /* bytes of the row in front of dst_off / src_off (a chunk that starts off the 16-byte */
                         /* boundary): done element by element in the first column                              */
    int32_t get0_slot;   /* value slot the operand at p0 is taken from instead of being loaded, -1 = loaded     */
    int32_t get1_slot;   /* the same for the operand at p1                                                      */
    int32_t put_slot;    /* value slot the result is kept in, -1 = not kept                                     */
    int32_t dead0;       /* 1 = the whole vectors of the result are not stored to p0 (MREDUCE: to any           */
                         /* destination): a later row overwrites them before anybody loads them                 */
    int32_t dead1;       /* the same for p1 (XREDUCE)                                                           */
    int32_t nsrc;        /* MREDUCE: sources, in add order ...                                                  */
    int32_t ndst;        /* ... and destinations: entries [first_ptr, first_ptr + nsrc + ndst) of the pointer   */
    int32_t first_ptr;   /* list.  Other kinds: nsrc = 0 and ndst further destinations of the result (copies    */
                         /* of it that later rows would have made), entries [first_ptr, first_ptr + ndst)       */
    int32_t joins;       /* 1 = (plan for few work items) the row takes its operands together with the row      */
                         /* before it, ahead of that row's sum and stores                                       */
} sar_plan_row;

typedef struct sar_plan_ptr { int32_t rank; int32_t reserved; uint64_t off; } sar_plan_ptr;

/* The rows behind sar_plan(): the column executor's plan for the main schedule (same_launch 0), for pre-work
 * and main schedule in one launch (same_launch 1) or for the pre-work alone (same_launch 2), whether or not
 * the cost model would pick that executor.
 * Writes at most row_cap rows and ptr_cap pointer-list entries; *nrows and *nptrs are the full counts.
 * SAR_ESTATE when there is no such plan (executor 0, rows the column kernel cannot run, no pre-work).
 * Host only; for tools and for tests that check the plan row by row. */
int sar_plan_rows(const sar_schedule* prework, const sar_schedule* main_schedule, int n, uint64_t bytes_per_rank, int dtype,
                  const sar_tuning_t* tuning, int compute_units, int same_launch,
                  sar_plan_row* rows, int row_cap, int* nrows, sar_plan_ptr* ptrs, int ptr_cap, int* nptrs);

#ifdef __cplusplus
}
#endif
#endif /* SAR_H */
