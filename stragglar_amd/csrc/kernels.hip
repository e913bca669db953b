// gfx950 device code of the schedule executor: the column kernel (a whole
// schedule in one launch), the round kernel (all rows of one round per
// launch), the multi-source reduce of the pre-work, and the small fill /
// compare / sleep kernels.
//
// The data kernels replace the reference's "ncclSend/ncclRecv into a temp
// buffer, then reduce_add<<<ceil(count/256),256>>>" (allreduce_8GPU.cu:29-34
// and every call site in :60-874).  They are pure streaming work bound by HBM
// bandwidth: 16-byte accesses per lane, every wavefront touching 1 KiB of
// consecutive memory per instruction.  Round kernel: U independent vectors in
// flight per lane and stream, one tile per workgroup so that the hardware
// dispatcher balances rows of different cost.  Column kernel: see its section.
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include <algorithm>

#include "kernels.hpp"

namespace sar {

typedef float f4 __attribute__((ext_vector_type(4)));
typedef uint32_t u4 __attribute__((ext_vector_type(4)));
typedef _Float16 h8 __attribute__((ext_vector_type(8)));

// ---- cache-policy aware 16-byte accesses --------------------------------
// Rank buffers are device memory: saying so (address space 1) keeps these global_load / global_store
// instructions also where the pointer was rebuilt from integers (a flat access would tie up the LDS
// counter as well and serialise against the LDS traffic of the column kernel).
typedef __attribute__((address_space(1))) f4 gf4;
template <bool NT>
__device__ __forceinline__ f4 ld16(const char* p) {
    const gf4* q = (const gf4*)p;
    if (NT) return __builtin_nontemporal_load(q);
    return *q;
}
template <bool NT>
__device__ __forceinline__ void st16(char* p, f4 v) {
    gf4* q = (gf4*)p;
    if (NT) __builtin_nontemporal_store(v, q);
    else *q = v;
}

// One value to `n` destinations whose addresses are a list in memory: the addresses four at a time (one scalar
// load), so that a long list is not one round trip to the scalar cache per store.
template <bool NT>
__device__ __forceinline__ void st16_to_all(char* const* __restrict__ list, uint32_t n, uint64_t o, f4 v) {
    uint32_t d = 0;
    for (; d + 4u <= n; d += 4u) {
        char* const q0 = list[d];
        char* const q1 = list[d + 1u];
        char* const q2 = list[d + 2u];
        char* const q3 = list[d + 3u];
        st16<NT>(q0 + o, v); st16<NT>(q1 + o, v); st16<NT>(q2 + o, v); st16<NT>(q3 + o, v);
    }
    for (; d < n; ++d) st16<NT>(list[d] + o, v);
}

// Marks a loaded value as used here, on every path.  A load that some path never uses stays pending in the
// compiler's bookkeeping, and the next write to its registers -- a slot read, the row table -- then waits for
// everything in flight, stores included (the memory counter runs in order).
__device__ __forceinline__ void consume(f4 v) { asm volatile("" : : "v"(v)); }

// ---- element arithmetic ---------------------------------------------------
// fp32: IEEE add.  fp16: correctly rounded add (same bits as widening to
// fp32, adding, and narrowing with round-to-nearest-even).  bf16: widen by a
// shift, fp32 add, round-to-nearest-even narrow by gfx950's v_cvt_pk_bf16_f32
// (two results per instruction; the integer sequence it replaces cost 18 VALU
// operations per pair against 7 and showed in schedules that add a lot).  A NaN
// stays a NaN; which NaN is the hardware's choice.
typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
typedef float f2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t bf16x2_add(uint32_t a, uint32_t b) {
    f2 s;
    s.x = __uint_as_float(a << 16) + __uint_as_float(b << 16);
    s.y = __uint_as_float(a & 0xffff0000u) + __uint_as_float(b & 0xffff0000u);
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(s, bf2));
}

template <int DT>
__device__ __forceinline__ f4 add16(f4 a, f4 b) {
    if (DT == SAR_F32) {
        return a + b;
    } else if (DT == SAR_F16) {
        h8 x = __builtin_bit_cast(h8, a), y = __builtin_bit_cast(h8, b);
        return __builtin_bit_cast(f4, x + y);
    } else {
        u4 x = __builtin_bit_cast(u4, a), y = __builtin_bit_cast(u4, b), r;
        r.x = bf16x2_add(x.x, y.x); r.y = bf16x2_add(x.y, y.y);
        r.z = bf16x2_add(x.z, y.z); r.w = bf16x2_add(x.w, y.w);
        return __builtin_bit_cast(f4, r);
    }
}

template <int DT> struct Elem;
template <> struct Elem<SAR_F32> { typedef float T; };
template <> struct Elem<SAR_F16> { typedef _Float16 T; };
template <> struct Elem<SAR_BF16> { typedef uint16_t T; };

template <int DT>
__device__ __forceinline__ typename Elem<DT>::T add1(typename Elem<DT>::T a, typename Elem<DT>::T b) {
    if constexpr (DT == SAR_BF16) {
        return (uint16_t)bf16x2_add(a, b);
    } else {
        return a + b;
    }
}

// ---- one tile of one row ---------------------------------------------------
// `len` bytes starting at byte `off` of the row, len <= BLOCK*U*16.
// Full 16-byte vectors are spread over the lanes with a stride of BLOCK
// vectors; the < 16 trailing bytes of a row are finished element by element.

template <int DT, int U, int BLOCK, bool LNT, bool SNT>
__device__ __forceinline__ void tile_copy(char* __restrict__ dst, const char* __restrict__ src, uint64_t off, uint32_t len) {
    const uint32_t nvec = len >> 4;
    f4 v[U];
    if (nvec == BLOCK * U) {
#pragma unroll
        for (int u = 0; u < U; ++u) v[u] = ld16<LNT>(src + off + ((uint64_t)(threadIdx.x + u * BLOCK) << 4));
#pragma unroll
        for (int u = 0; u < U; ++u) st16<SNT>(dst + off + ((uint64_t)(threadIdx.x + u * BLOCK) << 4), v[u]);
        return;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
        uint32_t i = threadIdx.x + u * BLOCK;
        if (i < nvec) v[u] = ld16<LNT>(src + off + ((uint64_t)i << 4));
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
        uint32_t i = threadIdx.x + u * BLOCK;
        if (i < nvec) st16<SNT>(dst + off + ((uint64_t)i << 4), v[u]);
    }
    typedef typename Elem<DT>::T T;
    const uint32_t tail = (len & 15u) / sizeof(T);
    if (threadIdx.x < tail) {
        uint64_t o = off + ((uint64_t)nvec << 4) + threadIdx.x * sizeof(T);
        *reinterpret_cast<T*>(dst + o) = *reinterpret_cast<const T*>(src + o);
    }
}

// dst += src  (TWO = false)   or   s = a + b; a <- s; b <- s  (TWO = true; dst = a, src = b)
template <int DT, int U, int BLOCK, bool TWO, bool LNT, bool SNT0, bool SNT1>
__device__ __forceinline__ void tile_reduce(char* __restrict__ dst, char* __restrict__ src, uint64_t off, uint32_t len) {
    const uint32_t nvec = len >> 4;
    f4 a[U], b[U];
    if (nvec == BLOCK * U) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            uint64_t o = off + ((uint64_t)(threadIdx.x + u * BLOCK) << 4);
            a[u] = ld16<LNT>(dst + o);
            b[u] = ld16<LNT>(src + o);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            uint64_t o = off + ((uint64_t)(threadIdx.x + u * BLOCK) << 4);
            f4 s = add16<DT>(a[u], b[u]);
            st16<SNT0>(dst + o, s);
            if (TWO) st16<SNT1>(src + o, s);
        }
        return;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
        uint32_t i = threadIdx.x + u * BLOCK;
        if (i < nvec) { a[u] = ld16<LNT>(dst + off + ((uint64_t)i << 4)); b[u] = ld16<LNT>(src + off + ((uint64_t)i << 4)); }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
        uint32_t i = threadIdx.x + u * BLOCK;
        if (i < nvec) {
            f4 s = add16<DT>(a[u], b[u]);
            st16<SNT0>(dst + off + ((uint64_t)i << 4), s);
            if (TWO) st16<SNT1>(src + off + ((uint64_t)i << 4), s);
        }
    }
    typedef typename Elem<DT>::T T;
    const uint32_t tail = (len & 15u) / sizeof(T);
    if (threadIdx.x < tail) {
        uint64_t o = off + ((uint64_t)nvec << 4) + threadIdx.x * sizeof(T);
        T s = add1<DT>(*reinterpret_cast<T*>(dst + o), *reinterpret_cast<T*>(src + o));
        *reinterpret_cast<T*>(dst + o) = s;
        if (TWO) *reinterpret_cast<T*>(src + o) = s;
    }
}

// Ring-ordered multi-source reduce.  srcs[0..nsrc) are in the order the ring
// adds them: acc = srcs[0]; acc = srcs[k] + acc for k = 1..nsrc-1 (the owner's
// own data comes last).  The result goes to every dsts[0..ndst).
template <int DT, int U, int BLOCK, bool LNT, bool SNT>
__device__ __forceinline__ void tile_mreduce(char* const* __restrict__ srcs, uint32_t nsrc, char* const* __restrict__ dsts, uint32_t ndst,
                                             uint64_t off, uint32_t len) {
    const uint32_t nvec = len >> 4;
#pragma unroll
    for (int u = 0; u < U; ++u) {
        uint32_t i = threadIdx.x + u * BLOCK;
        if (i >= nvec) continue;
        uint64_t o = off + ((uint64_t)i << 4);
        // (sources in variables of their own and marked used on every path: kept in an array, or left pending on a
        // path that skips them, they make later register writes wait for everything in flight -- the stores to the
        // destinations then went out one at a time)
        f4 acc = ld16<LNT>(srcs[0] + o);
        for (uint32_t k0 = 1; k0 < nsrc; k0 += 8) {
            const f4 z = f4{0.f, 0.f, 0.f, 0.f};
            f4 v0 = ld16<LNT>(srcs[k0] + o), v1 = z, v2 = z, v3 = z, v4 = z, v5 = z, v6 = z, v7 = z;
            if (k0 + 1 < nsrc) v1 = ld16<LNT>(srcs[k0 + 1] + o);
            if (k0 + 2 < nsrc) v2 = ld16<LNT>(srcs[k0 + 2] + o);
            if (k0 + 3 < nsrc) v3 = ld16<LNT>(srcs[k0 + 3] + o);
            if (k0 + 4 < nsrc) v4 = ld16<LNT>(srcs[k0 + 4] + o);
            if (k0 + 5 < nsrc) v5 = ld16<LNT>(srcs[k0 + 5] + o);
            if (k0 + 6 < nsrc) v6 = ld16<LNT>(srcs[k0 + 6] + o);
            if (k0 + 7 < nsrc) v7 = ld16<LNT>(srcs[k0 + 7] + o);
            consume(acc); consume(v0); consume(v1); consume(v2); consume(v3); consume(v4); consume(v5); consume(v6); consume(v7);
            acc = add16<DT>(v0, acc);
            if (k0 + 1 < nsrc) acc = add16<DT>(v1, acc);
            if (k0 + 2 < nsrc) acc = add16<DT>(v2, acc);
            if (k0 + 3 < nsrc) acc = add16<DT>(v3, acc);
            if (k0 + 4 < nsrc) acc = add16<DT>(v4, acc);
            if (k0 + 5 < nsrc) acc = add16<DT>(v5, acc);
            if (k0 + 6 < nsrc) acc = add16<DT>(v6, acc);
            if (k0 + 7 < nsrc) acc = add16<DT>(v7, acc);
        }
        st16_to_all<SNT>(dsts, ndst, o, acc);
    }
    typedef typename Elem<DT>::T T;
    const uint32_t tail = (len & 15u) / sizeof(T);
    if (threadIdx.x < tail) {
        uint64_t o = off + ((uint64_t)nvec << 4) + threadIdx.x * sizeof(T);
        T acc = *reinterpret_cast<const T*>(srcs[0] + o);
        for (uint32_t k = 1; k < nsrc; ++k) acc = add1<DT>(*reinterpret_cast<const T*>(srcs[k] + o), acc);
        for (uint32_t d = 0; d < ndst; ++d) *reinterpret_cast<T*>(dsts[d] + o) = acc;
    }
}

// Rows whose pointers are not all 16-byte aligned (unpadded buffer sizes):
// element by element, still coalesced across the wavefront.
template <int DT, int BLOCK>
__device__ __forceinline__ void tile_scalar(uint32_t kind, char* p0, char* p1, uint64_t off, uint32_t len) {
    typedef typename Elem<DT>::T T;
    const uint32_t n = len / sizeof(T);
    for (uint32_t e = threadIdx.x; e < n; e += BLOCK) {
        uint64_t o = off + (uint64_t)e * sizeof(T);
        if (kind == SAR_OP_COPY) {
            *reinterpret_cast<T*>(p0 + o) = *reinterpret_cast<const T*>(p1 + o);
        } else {
            T s = add1<DT>(*reinterpret_cast<T*>(p0 + o), *reinterpret_cast<T*>(p1 + o));
            *reinterpret_cast<T*>(p0 + o) = s;
            if (kind == SAR_OP_XREDUCE) *reinterpret_cast<T*>(p1 + o) = s;
        }
    }
}

// Which row and which tile of it a workgroup owns.
__device__ __forceinline__ void locate(const DevOp* __restrict__ ops, uint32_t nops, uint32_t total_tiles, uint32_t tiles_per_op,
                                       uint32_t interleave, uint32_t reverse, uint32_t* row, uint32_t* t) {
    uint32_t tile = reverse ? total_tiles - 1u - blockIdx.x : blockIdx.x;
    if (tiles_per_op) {                       // every row of the launch has the same length
        if (interleave) { *row = tile % nops; *t = tile / nops; }
        else { *row = tile / tiles_per_op; *t = tile - *row * tiles_per_op; }
    } else {                                  // rows of different length: find the row by its first tile
        uint32_t lo = 0, hi = nops;
        while (hi - lo > 1) { uint32_t mid = (lo + hi) >> 1; if (ops[mid].tile_begin <= tile) lo = mid; else hi = mid; }
        *row = lo; *t = tile - ops[lo].tile_begin;
    }
}

// COPY / REDUCE_INTO / XREDUCE rows of one round; one tile of BLOCK*U vectors per workgroup.
template <int DT, int U, int BLOCK>
__global__ __launch_bounds__(BLOCK) void round_kernel(const DevOp* __restrict__ ops, uint32_t nops, uint32_t total_tiles,
                                                       uint32_t tiles_per_op, uint32_t interleave, uint32_t reverse) {
    uint32_t j, t;
    locate(ops, nops, total_tiles, tiles_per_op, interleave, reverse, &j, &t);
    char* const p0 = ops[j].p0;
    char* const p1 = ops[j].p1;
    const uint64_t bytes = ops[j].bytes;
    const uint32_t kind = ops[j].kind, flags = ops[j].flags;
    constexpr uint64_t tile_bytes = (uint64_t)BLOCK * U * 16u;
    const uint64_t off = (uint64_t)t * tile_bytes;
    if (off >= bytes) return;
    const uint64_t rem = bytes - off;
    const uint32_t len = rem < tile_bytes ? (uint32_t)rem : (uint32_t)tile_bytes;

    if (!(flags & DEVOP_VEC)) { tile_scalar<DT, BLOCK>(kind, p0, p1, off, len); return; }
    const bool lnt = flags & DEVOP_LNT, s0 = flags & DEVOP_SNT0, s1 = flags & DEVOP_SNT1;
    if (kind == SAR_OP_COPY) {
        if (lnt) { if (s0) tile_copy<DT, U, BLOCK, true, true>(p0, p1, off, len); else tile_copy<DT, U, BLOCK, true, false>(p0, p1, off, len); }
        else     { if (s0) tile_copy<DT, U, BLOCK, false, true>(p0, p1, off, len); else tile_copy<DT, U, BLOCK, false, false>(p0, p1, off, len); }
    } else if (kind == SAR_OP_REDUCE_INTO) {
        if (lnt) { if (s0) tile_reduce<DT, U, BLOCK, false, true, true, true>(p0, p1, off, len); else tile_reduce<DT, U, BLOCK, false, true, false, false>(p0, p1, off, len); }
        else     { if (s0) tile_reduce<DT, U, BLOCK, false, false, true, true>(p0, p1, off, len); else tile_reduce<DT, U, BLOCK, false, false, false, false>(p0, p1, off, len); }
    } else {
        if (lnt) {
            if (s0) { if (s1) tile_reduce<DT, U, BLOCK, true, true, true, true>(p0, p1, off, len); else tile_reduce<DT, U, BLOCK, true, true, true, false>(p0, p1, off, len); }
            else    { if (s1) tile_reduce<DT, U, BLOCK, true, true, false, true>(p0, p1, off, len); else tile_reduce<DT, U, BLOCK, true, true, false, false>(p0, p1, off, len); }
        } else {
            if (s0) { if (s1) tile_reduce<DT, U, BLOCK, true, false, true, true>(p0, p1, off, len); else tile_reduce<DT, U, BLOCK, true, false, true, false>(p0, p1, off, len); }
            else    { if (s1) tile_reduce<DT, U, BLOCK, true, false, false, true>(p0, p1, off, len); else tile_reduce<DT, U, BLOCK, true, false, false, false>(p0, p1, off, len); }
        }
    }
}

// MREDUCE rows (the pre-work collectives): the sources themselves provide the
// memory-level parallelism, so a tile is BLOCK*MR_U vectors with a small MR_U.
constexpr int MR_U = 1;        // measured: 4 KiB tiles 5.8-5.9 TB/s, 8 KiB 5.5-5.7, 16 KiB 5.4
constexpr int MR_BLOCK = 256;

template <int DT>
__global__ __launch_bounds__(MR_BLOCK) void mreduce_kernel(const DevOp* __restrict__ ops, uint32_t nops, char* const* __restrict__ ptrs,
                                                            uint32_t total_tiles, uint32_t tiles_per_op, uint32_t interleave, uint32_t reverse) {
    uint32_t j, t;
    locate(ops, nops, total_tiles, tiles_per_op, interleave, reverse, &j, &t);
    const uint64_t bytes = ops[j].bytes;
    const uint32_t flags = ops[j].flags, nsrc = ops[j].nsrc, ndst = ops[j].ndst;
    char* const* srcs = ptrs + ops[j].ptr_off;
    char* const* dsts = srcs + nsrc;
    constexpr uint64_t tile_bytes = (uint64_t)MR_BLOCK * MR_U * 16u;
    const uint64_t off = (uint64_t)t * tile_bytes;
    if (off >= bytes) return;
    const uint64_t rem = bytes - off;
    const uint32_t len = rem < tile_bytes ? (uint32_t)rem : (uint32_t)tile_bytes;
    if (!(flags & DEVOP_VEC)) {
        typedef typename Elem<DT>::T T;
        const uint32_t n = len / sizeof(T);
        for (uint32_t e = threadIdx.x; e < n; e += MR_BLOCK) {
            uint64_t o = off + (uint64_t)e * sizeof(T);
            T acc = *reinterpret_cast<const T*>(srcs[0] + o);
            for (uint32_t k = 1; k < nsrc; ++k) acc = add1<DT>(*reinterpret_cast<const T*>(srcs[k] + o), acc);
            for (uint32_t d = 0; d < ndst; ++d) *reinterpret_cast<T*>(dsts[d] + o) = acc;
        }
        return;
    }
    const bool lnt = flags & DEVOP_LNT, s0 = flags & DEVOP_SNT0;
    if (lnt) { if (s0) tile_mreduce<DT, MR_U, MR_BLOCK, true, true>(srcs, nsrc, dsts, ndst, off, len); else tile_mreduce<DT, MR_U, MR_BLOCK, true, false>(srcs, nsrc, dsts, ndst, off, len); }
    else     { if (s0) tile_mreduce<DT, MR_U, MR_BLOCK, false, true>(srcs, nsrc, dsts, ndst, off, len); else tile_mreduce<DT, MR_U, MR_BLOCK, false, false>(srcs, nsrc, dsts, ndst, off, len); }
}

#define SAR_LAUNCH_ROUND(DT, U, B) \
    hipLaunchKernelGGL((round_kernel<DT, U, B>), grid, dim3(B), 0, st, ops, nops, total_tiles, tiles_per_op, interleave, reverse)

template <int DT>
static hipError_t launch_round_dt(int unroll, int block, dim3 grid, hipStream_t st, const DevOp* ops, uint32_t nops,
                                  uint32_t total_tiles, uint32_t tiles_per_op, uint32_t interleave, uint32_t reverse) {
    switch (unroll * 1024 + block) {
        case 1 * 1024 + 256: SAR_LAUNCH_ROUND(DT, 1, 256); break;
        case 2 * 1024 + 256: SAR_LAUNCH_ROUND(DT, 2, 256); break;
        case 4 * 1024 + 256: SAR_LAUNCH_ROUND(DT, 4, 256); break;
        case 8 * 1024 + 256: SAR_LAUNCH_ROUND(DT, 8, 256); break;
        case 1 * 1024 + 512: SAR_LAUNCH_ROUND(DT, 1, 512); break;
        case 2 * 1024 + 512: SAR_LAUNCH_ROUND(DT, 2, 512); break;
        case 4 * 1024 + 512: SAR_LAUNCH_ROUND(DT, 4, 512); break;
        case 8 * 1024 + 512: SAR_LAUNCH_ROUND(DT, 8, 512); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_round(int dtype, int unroll, int block, hipStream_t st, const DevOp* ops, uint32_t nops,
                        uint32_t total_tiles, uint32_t tiles_per_op, uint32_t interleave, uint32_t reverse) {
    if (total_tiles == 0) return hipSuccess;
    dim3 g(total_tiles);
    switch (dtype) {
        case SAR_F32: return launch_round_dt<SAR_F32>(unroll, block, g, st, ops, nops, total_tiles, tiles_per_op, interleave, reverse);
        case SAR_F16: return launch_round_dt<SAR_F16>(unroll, block, g, st, ops, nops, total_tiles, tiles_per_op, interleave, reverse);
        case SAR_BF16: return launch_round_dt<SAR_BF16>(unroll, block, g, st, ops, nops, total_tiles, tiles_per_op, interleave, reverse);
        default: return hipErrorInvalidValue;
    }
}

uint64_t mreduce_tile_bytes() { return (uint64_t)MR_BLOCK * MR_U * 16u; }

hipError_t launch_mreduce(int dtype, hipStream_t st, const DevOp* ops, uint32_t nops, char* const* ptrs,
                          uint32_t total_tiles, uint32_t tiles_per_op, uint32_t interleave, uint32_t reverse) {
    if (total_tiles == 0) return hipSuccess;
    dim3 g(total_tiles), b(MR_BLOCK);
    switch (dtype) {
        case SAR_F32: hipLaunchKernelGGL((mreduce_kernel<SAR_F32>), g, b, 0, st, ops, nops, ptrs, total_tiles, tiles_per_op, interleave, reverse); break;
        case SAR_F16: hipLaunchKernelGGL((mreduce_kernel<SAR_F16>), g, b, 0, st, ops, nops, ptrs, total_tiles, tiles_per_op, interleave, reverse); break;
        case SAR_BF16: hipLaunchKernelGGL((mreduce_kernel<SAR_BF16>), g, b, 0, st, ops, nops, ptrs, total_tiles, tiles_per_op, interleave, reverse); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

// ---- column executor: the whole schedule in one launch, no waiting between workgroups -----------
// Rows move whole chunks, so an element only ever meets the elements at its own offset within a
// chunk: the schedule falls apart into independent "columns" (one range of within-chunk offsets each).
// A workgroup owns a column of BLOCK 16-byte vectors and walks ALL rounds for it, row after row, with
// nothing but a workgroup barrier between rounds.  What a later round re-reads was written by the same
// lane moments ago: without forwarding it comes back from L2 / Infinity Cache instead of HBM; with
// forwarding (FWD) the lane kept it in an LDS value slot that the host assigned when it lowered the
// schedule, and the load is not issued at all.  Every row stores its result to the rank buffers, in
// schedule order for each element, except where the host found that a later row overwrites the value
// before anybody loads it (DEVOP_DEAD0 / DEAD1).
// One row at a time turned out best (24 VGPRs without forwarding, 38 with: eight waves per SIMD
// resident, the other workgroups of the compute unit cover a row's latency; batching the loads of
// several rows cost occupancy and was slower: 6.8 against 7.1 TB/s).

// One row as the column kernel uses it, every field wave-uniform (SGPRs).
struct ColRow { char* p0; char* p1; uint64_t bytes; uint32_t kind, flags, slots, nsrc, ndst, ptr_off; };

__device__ __forceinline__ uint32_t uniform32(uint32_t v) { return (uint32_t)__builtin_amdgcn_readfirstlane((int)v); }

// Row j of the launch: from the copy of the row table in LDS when there is one (a broadcast read, made
// uniform again with readfirstlane), else through scalar loads from memory.
template <bool STAGED>
__device__ __forceinline__ ColRow column_row(const DevOp* __restrict__ ops, const u4* table, uint32_t j) {
    ColRow r;
    if (STAGED) {
        const u4 q0 = table[j * 4u], q1 = table[j * 4u + 1u], q2 = table[j * 4u + 2u], q3 = table[j * 4u + 3u];
        r.p0 = reinterpret_cast<char*>((uint64_t)uniform32(q0.x) | ((uint64_t)uniform32(q0.y) << 32));
        r.p1 = reinterpret_cast<char*>((uint64_t)uniform32(q0.z) | ((uint64_t)uniform32(q0.w) << 32));
        r.bytes = (uint64_t)uniform32(q1.x) | ((uint64_t)uniform32(q1.y) << 32);
        r.kind = uniform32(q1.z); r.flags = uniform32(q1.w); r.slots = uniform32(q3.y);
        r.nsrc = uniform32(q2.z); r.ndst = uniform32(q2.w); r.ptr_off = uniform32(q3.x);
    } else {
        r.p0 = ops[j].p0; r.p1 = ops[j].p1; r.bytes = ops[j].bytes;
        r.kind = ops[j].kind; r.flags = ops[j].flags; r.slots = ops[j].slots;
        r.nsrc = ops[j].nsrc; r.ndst = ops[j].ndst; r.ptr_off = ops[j].ptr_off;
    }
    return r;
}
static_assert(offsetof(DevOp, p1) == 8 && offsetof(DevOp, bytes) == 16 && offsetof(DevOp, kind) == 24 &&
              offsetof(DevOp, flags) == 28 && offsetof(DevOp, nsrc) == 40 && offsetof(DevOp, ndst) == 44 &&
              offsetof(DevOp, ptr_off) == 48 && offsetof(DevOp, slots) == 52, "column_row reads DevOp by position");

// The sum (or the copied value) of one vector of a row: to the rank buffers, to a value slot, to the further
// destinations the host attached.  `v`: which of the lane's V vectors.
template <int DT, int BLOCK, bool FWD, bool SNT, uint32_t V>
__device__ __forceinline__ void column_row_store(const ColRow& row, uint64_t o, uint32_t v, f4 a, f4 b, bool live0, bool live1, f4* mine,
                                                 char* const* __restrict__ ptrs) {
    const f4 s = row.kind == SAR_OP_COPY ? b : add16<DT>(a, b);
    if (live0) st16<SNT>(row.p0 + o, s);
    if (row.kind == SAR_OP_XREDUCE && live1) st16<SNT>(row.p1 + o, s);
    if (FWD && (row.flags & DEVOP_PUT)) mine[((row.slots >> 16 & 0xffu) * V + v) * BLOCK] = s;
    // copies of the result that later rows would have made (taken over by the host)
    if (FWD && row.ndst) st16_to_all<SNT>(ptrs + row.ptr_off, row.ndst, o, s);
}

// Latency plan (one vector per lane and row), a row of whole vectors in two steps, so that the loads of several
// rows of a group can be in flight together: the rows of a group never depend on each other.
template <int BLOCK, bool FWD, bool LNT>
__device__ __forceinline__ void lat_row_load(const ColRow& row, uint64_t voff, const f4* mine, f4& a, f4& b) {
    a = f4{0.f, 0.f, 0.f, 0.f}; b = a;
    if (voff + 16u > row.bytes) return;
    const uint32_t slots = FWD ? row.slots : 0u;
    if (FWD && (row.flags & DEVOP_GET1)) b = mine[(slots >> 8 & 0xffu) * BLOCK]; else b = ld16<LNT>(row.p1 + voff);
    if (row.kind != SAR_OP_COPY) { if (FWD && (row.flags & DEVOP_GET0)) a = mine[(slots & 0xffu) * BLOCK]; else a = ld16<LNT>(row.p0 + voff); }
}

template <int DT, int BLOCK, bool FWD, bool SNT>
__device__ __forceinline__ void lat_row_finish(const ColRow& row, uint64_t off, uint64_t voff, f4* mine, char* const* __restrict__ ptrs, f4 a, f4 b) {
    typedef typename Elem<DT>::T T;
    const uint32_t flags = row.flags, kind = row.kind;
    char* const p0 = row.p0;
    char* const p1 = row.p1;
    if (voff + 16u <= row.bytes) {
        const f4 s = kind == SAR_OP_COPY ? b : add16<DT>(a, b);
        if (!(FWD && (flags & DEVOP_DEAD0))) st16<SNT>(p0 + voff, s);
        if (kind == SAR_OP_XREDUCE && !(FWD && (flags & DEVOP_DEAD1))) st16<SNT>(p1 + voff, s);
        if (FWD && (flags & DEVOP_PUT)) mine[(row.slots >> 16 & 0xffu) * BLOCK] = s;
        if (FWD && row.ndst) st16_to_all<SNT>(ptrs + row.ptr_off, row.ndst, voff, s);
    }
    // the bytes behind the last whole vector and in front of the first one, as in the one-row path
    const uint64_t tail_at = row.bytes & ~(uint64_t)15u;
    const uint32_t tail = (uint32_t)(row.bytes & 15u) / sizeof(T);
    if (tail && tail_at >= off && tail_at < off + (uint64_t)BLOCK * 16u && threadIdx.x < tail) {
        const uint64_t o = tail_at + threadIdx.x * sizeof(T);
        T s = *reinterpret_cast<const T*>(p1 + o);
        if (kind != SAR_OP_COPY) s = add1<DT>(*reinterpret_cast<const T*>(p0 + o), s);
        *reinterpret_cast<T*>(p0 + o) = s;
        if (kind == SAR_OP_XREDUCE) *reinterpret_cast<T*>(p1 + o) = s;
    }
    const uint32_t head = (flags >> DEVOP_HEAD_SHIFT & 15u) / (uint32_t)sizeof(T);
    if (head && off == 0 && threadIdx.x < head) {
        const int64_t o = ((int64_t)threadIdx.x - (int64_t)head) * (int64_t)sizeof(T);
        T s = *reinterpret_cast<const T*>(p1 + o);
        if (kind != SAR_OP_COPY) s = add1<DT>(*reinterpret_cast<const T*>(p0 + o), s);
        *reinterpret_cast<T*>(p0 + o) = s;
        if (kind == SAR_OP_XREDUCE) *reinterpret_cast<T*>(p1 + o) = s;
    }
}

// Rows that share no (rank, chunk) cell never depend on each other, whatever round they sit in.  The host
// therefore splits the rows into connected components (for all four algorithms: one per chunk index) and a
// work item is one component for one column: its rows, in round order, cut into groups at the round
// boundaries (a barrier follows each group).  Items are independent of each other.
//
// FWD: value slots in LDS (rows flagged DEVOP_GET* / DEVOP_PUT).  LAT: the plan for few items -- the rows and
// groups of the item's component are copied into LDS first.  POL: cache policy of the whole launch, 0 = all
// accesses cached, 1 = streaming (nontemporal) loads and cached stores, 2 = streaming loads and stores.  The
// policy is a template argument because a flavour picked per row at run time does not survive compilation:
// the two otherwise identical accesses are folded into one and the nontemporal hint is dropped.  MR: the
// launch has multi-source rows (a pre-work collective in the same launch); their batched loads take more
// registers and a longer row loop, so launches without such rows run a variant without that path.
template <int DT, int BLOCK, bool FWD, bool LAT, int POL, bool MR, bool TWO>
__global__ __launch_bounds__(BLOCK) void column_kernel(const DevOp* __restrict__ ops, const uint32_t* __restrict__ group_begin,
                                                        const ColumnComp* __restrict__ comps, char* const* __restrict__ ptrs, ColumnLaunch L) {
    typedef typename Elem<DT>::T T;
    // Vectors per lane and row (TWO, only with FWD and without LAT): two when values are forwarded in the bandwidth
    // regime and the rows still load a good part of their operands (the loads that remain are few and far between,
    // and two in flight per lane pay: ring at 16 and 32 ranks +4 to +5 %), one otherwise: every row loads and
    // occupancy covers the latency; few items are better spread over more workgroups; and a plan that mostly
    // stores (the StragglAR tables, direct) runs 2 to 3 % faster with more, smaller work items.
    constexpr uint32_t V = (FWD && !LAT && TWO) ? 2u : 1u;
    constexpr uint64_t col_bytes = (uint64_t)BLOCK * 16u * V;
    constexpr bool LNT = POL >= 1, SNT = POL == 2;
    // LDS: LAT: [the component's rows: table_rows x 64 B][its group boundaries: table_groups x 4 B, padded to
    // 16 B]; then FWD: the value slots, slot k of lane t at vector k*BLOCK + t.  A lane only ever touches its
    // own slot vectors, so the slots need no synchronisation of their own.  (With V vectors per lane slot k, vector v
    // of lane t sits at (k*V + v)*BLOCK + t.)
    // (the tables come as kernel arguments of their own: only a __restrict__ const parameter lets the compiler
    // read them through scalar loads)
    extern __shared__ __align__(16) char lds_raw[];
    const uint32_t table_vecs = LAT ? L.table_rows * 4u : 0u, group_vecs = LAT ? (L.table_groups + 3u) / 4u : 0u;
    const u4* const table = reinterpret_cast<const u4*>(lds_raw);
    uint32_t* const lgroups = reinterpret_cast<uint32_t*>(lds_raw) + table_vecs * 4u;
    f4* const mine = reinterpret_cast<f4*>(lds_raw) + table_vecs + group_vecs + threadIdx.x;
    bool first_item = true;
    for (uint32_t item = blockIdx.x; item < L.nitems; item += gridDim.x) {
        // items in dispatch order: `run` neighbouring columns of one component, then the same columns of the next
        // component, ...; then the next `run` columns
        const uint32_t per_block = L.run * L.ncomp, blk = item / per_block, within = item - blk * per_block;
        const uint32_t comp = within / L.run, col = blk * L.run + within % L.run;
        if (col >= L.ncols) continue;
        const ColumnComp C = comps[comp];
        if (LAT) {
            // Few workgroups, nobody to warm the scalar cache: a row read through scalar loads costs a trip to
            // L2 (about half a microsecond) and the rows come one after the other.  Fetch them all at once.
            if (!first_item) __syncthreads();                    // the previous item is done with the table
            first_item = false;
            u4* dst = reinterpret_cast<u4*>(lds_raw);
            const u4* src = reinterpret_cast<const u4*>(ops + C.row_first);
            const uint32_t nvec = (C.row_end - C.row_first) * 4u, ngrp = C.group_end - C.group_first + 1u;
            for (uint32_t i = threadIdx.x; i < nvec; i += BLOCK) dst[i] = src[i];
            for (uint32_t i = threadIdx.x; i < ngrp; i += BLOCK) lgroups[i] = group_begin[C.group_first + i];
            __syncthreads();
        }
        const uint64_t off = (uint64_t)col * col_bytes;
        const uint64_t voff = off + ((uint64_t)threadIdx.x << 4);       // this lane's vector within every row
        for (uint32_t g = C.group_first; g < C.group_end; ++g) {
            uint32_t rb, re;
            if (LAT) { rb = uniform32(lgroups[g - C.group_first]) - C.row_first; re = uniform32(lgroups[g - C.group_first + 1u]) - C.row_first; }
            else { rb = group_begin[g]; re = group_begin[g + 1u]; }
            for (uint32_t j = rb; j < re; ++j) {
                const ColRow row = column_row<LAT>(ops, table, j);
                if (LAT && j + 1u < re) {
                    // Few items: nothing covers a row's round trip to memory.  Rows that the host flagged DEVOP_JOIN
                    // (up to three behind a row of whole vectors, none needing another's result) go together: all
                    // their loads and slot reads first, then the sums and stores in row order.
                    // (rows and operands in variables of their own, not arrays: see the one-row path below)
                    ColRow r1 = row, r2 = row, r3 = row;
                    uint32_t nb = 1;
                    r1 = column_row<true>(ops, table, j + 1u);
                    if (r1.flags & DEVOP_JOIN) {
                        nb = 2;
                        if (j + 2u < re) {
                            r2 = column_row<true>(ops, table, j + 2u);
                            if (r2.flags & DEVOP_JOIN) {
                                nb = 3;
                                if (j + 3u < re) { r3 = column_row<true>(ops, table, j + 3u); if (r3.flags & DEVOP_JOIN) nb = 4; }
                            }
                        }
                    }
                    if (nb > 1u) {
                        f4 a0, b0, a1, b1, a2 = f4{0.f, 0.f, 0.f, 0.f}, b2 = a2, a3 = a2, b3 = a2;
                        lat_row_load<BLOCK, FWD, LNT>(row, voff, mine, a0, b0);
                        lat_row_load<BLOCK, FWD, LNT>(r1, voff, mine, a1, b1);
                        if (nb > 2u) lat_row_load<BLOCK, FWD, LNT>(r2, voff, mine, a2, b2);
                        if (nb > 3u) lat_row_load<BLOCK, FWD, LNT>(r3, voff, mine, a3, b3);
                        consume(a0); consume(b0); consume(a1); consume(b1); consume(a2); consume(b2); consume(a3); consume(b3);
                        lat_row_finish<DT, BLOCK, FWD, SNT>(row, off, voff, mine, ptrs, a0, b0);
                        lat_row_finish<DT, BLOCK, FWD, SNT>(r1, off, voff, mine, ptrs, a1, b1);
                        if (nb > 2u) lat_row_finish<DT, BLOCK, FWD, SNT>(r2, off, voff, mine, ptrs, a2, b2);
                        if (nb > 3u) lat_row_finish<DT, BLOCK, FWD, SNT>(r3, off, voff, mine, ptrs, a3, b3);
                        j += nb - 1u;
                        continue;
                    }
                }
                const uint32_t flags = row.flags, kind = row.kind;
                const uint64_t bytes = row.bytes;
                char* const p0 = row.p0;
                char* const p1 = row.p1;
                if (MR && kind == SAR_OP_MREDUCE) {
                    // Multi-source row (a pre-work collective lowered into the same launch; the host only does that
                    // when all its pointers are 16-byte aligned and the row is a whole number of vectors long):
                    // acc = srcs[0]; acc = srcs[k] + acc, the owner's own data last; the result goes to every dst
                    // and, flagged PUT, into a slot for the exchange that follows.
                    char* const* const srcs = ptrs + row.ptr_off;
                    char* const* const dsts = srcs + row.nsrc;
                    constexpr uint64_t vstep = (uint64_t)BLOCK * 16u;
#pragma unroll
                    for (uint32_t v = 0; v < V; ++v) {
                        const uint64_t o = voff + v * vstep;
                        if (o + 16u <= bytes) {
                            f4 acc = ld16<LNT>(srcs[0] + o);
                            for (uint32_t k0 = 1; k0 < row.nsrc; k0 += 4u) {
                                const f4 z = f4{0.f, 0.f, 0.f, 0.f};
                                f4 t0 = ld16<LNT>(srcs[k0] + o), t1 = z, t2 = z, t3 = z;
                                if (k0 + 1u < row.nsrc) t1 = ld16<LNT>(srcs[k0 + 1u] + o);
                                if (k0 + 2u < row.nsrc) t2 = ld16<LNT>(srcs[k0 + 2u] + o);
                                if (k0 + 3u < row.nsrc) t3 = ld16<LNT>(srcs[k0 + 3u] + o);
                                consume(acc); consume(t0); consume(t1); consume(t2); consume(t3);
                                acc = add16<DT>(t0, acc);
                                if (k0 + 1u < row.nsrc) acc = add16<DT>(t1, acc);
                                if (k0 + 2u < row.nsrc) acc = add16<DT>(t2, acc);
                                if (k0 + 3u < row.nsrc) acc = add16<DT>(t3, acc);
                            }
                            if (!(FWD && (flags & DEVOP_DEAD0))) st16_to_all<SNT>(dsts, row.ndst, o, acc);
                            if (FWD && (flags & DEVOP_PUT)) mine[((row.slots >> 16 & 0xffu) * V + v) * BLOCK] = acc;
                        }
                    }
                } else if (flags & DEVOP_VEC) {
                    if (voff + 16u <= bytes) {
                        const uint32_t slots = FWD ? row.slots : 0u;
                        const bool get0 = FWD && (flags & DEVOP_GET0), get1 = FWD && (flags & DEVOP_GET1);
                        constexpr uint64_t vstep = (uint64_t)BLOCK * 16u;
                        const bool live0 = !(FWD && (flags & DEVOP_DEAD0)), live1 = !(FWD && (flags & DEVOP_DEAD1));
                        if (FWD && kind == SAR_OP_COPY && get1) {
                            // A copy of a held value is a store and nothing else.  It has a path of its own so
                            // that it does not pass the wait for loaded operands below: the memory counter
                            // runs in order, and that wait would also sit out the stores of the rows before.
#pragma unroll
                            for (uint32_t v = 0; v < V; ++v)
                                if (live0 && voff + v * vstep + 16u <= bytes) st16<SNT>(p0 + voff + v * vstep, mine[((slots >> 8 & 0xffu) * V + v) * BLOCK]);
                        } else {
                            // (Every operand in a variable of its own: an array of vectors is kept as one wide value,
                            // and a load into it is waited for on the spot in order to copy it in, which serialises
                            // the loads of a row.)
                            const uint64_t o1 = voff + vstep;
                            const bool in1 = V > 1u && o1 + 16u <= bytes;
                            const uint64_t oc1 = in1 ? o1 : voff;                  // past the end: reload the first vector, keep nothing
                            const uint32_t g0 = (slots & 0xffu) * V, g1 = (slots >> 8 & 0xffu) * V;
                            // Slot reads before loads: a slot read that follows a load of the same row in the code is
                            // made to wait for that load (both may end up in the same registers), and the loads of
                            // the row would again go out one at a time.
                            f4 a0 = f4{0.f, 0.f, 0.f, 0.f}, a1 = a0, b0 = a0, b1 = a0;
                            const bool load_a = kind != SAR_OP_COPY && !get0;
                            if (get1) { b0 = mine[g1 * BLOCK]; if (V > 1u) b1 = mine[(g1 + 1u) * BLOCK]; }
                            if (get0 && kind != SAR_OP_COPY) { a0 = mine[g0 * BLOCK]; if (V > 1u) a1 = mine[(g0 + 1u) * BLOCK]; }
                            if (!get1) { b0 = ld16<LNT>(p1 + voff); if (V > 1u) b1 = ld16<LNT>(p1 + oc1); }
                            if (load_a) { a0 = ld16<LNT>(p0 + voff); if (V > 1u) a1 = ld16<LNT>(p0 + oc1); }
                            // (all operands of the row at once, before its first store: a wait placed behind stores
                            // waits for the stores as well)
                            consume(a0); consume(b0);
                            if (V > 1u) { consume(a1); consume(b1); }              // also where the second vector lies past the end
                            column_row_store<DT, BLOCK, FWD, SNT, V>(row, voff, 0u, a0, b0, live0, live1, mine, ptrs);
                            if (V > 1u && in1) column_row_store<DT, BLOCK, FWD, SNT, V>(row, o1, 1u, a1, b1, live0, live1, mine, ptrs);
                        }
                    }
                    // the < 16 bytes behind the last whole vector of the row, in the column that holds them
                    // (always through memory: every forwarded value has been stored as well)
                    const uint64_t tail_at = bytes & ~(uint64_t)15u;
                    const uint32_t tail = (uint32_t)(bytes & 15u) / sizeof(T);
                    if (tail && tail_at >= off && tail_at < off + col_bytes && threadIdx.x < tail) {
                        const uint64_t o = tail_at + threadIdx.x * sizeof(T);
                        T s = *reinterpret_cast<const T*>(p1 + o);
                        if (kind != SAR_OP_COPY) s = add1<DT>(*reinterpret_cast<const T*>(p0 + o), s);
                        *reinterpret_cast<T*>(p0 + o) = s;
                        if (kind == SAR_OP_XREDUCE) *reinterpret_cast<T*>(p1 + o) = s;
                    }
                    // the < 16 bytes in front of p0 and p1 of a row that was moved up to a 16-byte boundary, in
                    // the first column (through memory as well)
                    const uint32_t head = (flags >> DEVOP_HEAD_SHIFT & 15u) / (uint32_t)sizeof(T);
                    if (head && off == 0 && threadIdx.x < head) {
                        const int64_t o = ((int64_t)threadIdx.x - (int64_t)head) * (int64_t)sizeof(T);
                        T s = *reinterpret_cast<const T*>(p1 + o);
                        if (kind != SAR_OP_COPY) s = add1<DT>(*reinterpret_cast<const T*>(p0 + o), s);
                        *reinterpret_cast<T*>(p0 + o) = s;
                        if (kind == SAR_OP_XREDUCE) *reinterpret_cast<T*>(p1 + o) = s;
                    }
                } else if (off < bytes) {                               // row not 16-byte aligned: element by element
                    const uint64_t rem = bytes - off;
                    const uint32_t len = rem < col_bytes ? (uint32_t)rem : (uint32_t)col_bytes;
                    tile_scalar<DT, BLOCK>(kind, p0, p1, off, len);
                }
            }
            // This group's stores are complete before this workgroup's loads of the next one.  (Lanes mostly
            // re-read what they wrote themselves, but elements change lanes between aligned and unaligned
            // rows and at partial vectors; measured, the barrier also pays for itself by keeping the waves
            // of a workgroup on the same rows.)  When the host has found that every lane only re-reads bytes
            // it wrote itself (lane_local), program order already covers that and the waves only meet,
            // without waiting for their stores to drain.
            if (L.lane_local) __builtin_amdgcn_s_barrier(); else __syncthreads();
        }
    }
}

uint64_t column_bytes(int block, bool two_vectors) { return (uint64_t)block * 16u * (two_vectors ? 2u : 1u); }
uint64_t column_lds_budget() { return 65536u; }
uint64_t column_table_bytes(uint32_t rows, uint32_t groups) { return (uint64_t)rows * sizeof(DevOp) + (((uint64_t)groups + 3u) / 4u) * 16u; }
int column_latency_block() { return 256; }

template <int DT, bool FWD, int POL, bool MR, bool TWO>
static hipError_t launch_column_block(int block, uint32_t grid, uint32_t lds, hipStream_t st, const ColumnLaunch& L) {
    switch (block) {
        case 256: hipLaunchKernelGGL((column_kernel<DT, 256, FWD, false, POL, MR, TWO>), dim3(grid), dim3(256), lds, st, L.ops, L.group_begin, L.comps, L.ptrs, L); break;
        case 512: hipLaunchKernelGGL((column_kernel<DT, 512, FWD, false, POL, MR, TWO>), dim3(grid), dim3(512), lds, st, L.ops, L.group_begin, L.comps, L.ptrs, L); break;
        case 1024: hipLaunchKernelGGL((column_kernel<DT, 1024, FWD, false, POL, MR, TWO>), dim3(grid), dim3(1024), lds, st, L.ops, L.group_begin, L.comps, L.ptrs, L); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

template <int DT, int POL, bool MR>
static hipError_t launch_column_policy(int block, uint32_t grid, uint32_t lds, bool fwd, hipStream_t st, const ColumnLaunch& L) {
    if (L.table_rows) {
        if (fwd) hipLaunchKernelGGL((column_kernel<DT, 256, true, true, POL, MR, false>), dim3(grid), dim3(256), lds, st, L.ops, L.group_begin, L.comps, L.ptrs, L);
        else hipLaunchKernelGGL((column_kernel<DT, 256, false, true, POL, MR, false>), dim3(grid), dim3(256), lds, st, L.ops, L.group_begin, L.comps, L.ptrs, L);
        return hipGetLastError();
    }
    if (!fwd) return launch_column_block<DT, false, POL, MR, false>(block, grid, lds, st, L);
    return L.two_vectors ? launch_column_block<DT, true, POL, MR, true>(block, grid, lds, st, L) : launch_column_block<DT, true, POL, MR, false>(block, grid, lds, st, L);
}

template <int DT>
static hipError_t launch_column_dt(int block, uint32_t grid, uint32_t lds, bool fwd, hipStream_t st, const ColumnLaunch& L) {
    switch (L.policy) {
        case 0: return L.multi_source ? launch_column_policy<DT, 0, true>(block, grid, lds, fwd, st, L) : launch_column_policy<DT, 0, false>(block, grid, lds, fwd, st, L);
        case 1: return L.multi_source ? launch_column_policy<DT, 1, true>(block, grid, lds, fwd, st, L) : launch_column_policy<DT, 1, false>(block, grid, lds, fwd, st, L);
        case 2: return L.multi_source ? launch_column_policy<DT, 2, true>(block, grid, lds, fwd, st, L) : launch_column_policy<DT, 2, false>(block, grid, lds, fwd, st, L);
        default: return hipErrorInvalidValue;
    }
}

hipError_t launch_column(int dtype, int block, uint32_t grid, uint32_t nslots, hipStream_t st, const ColumnLaunch& L) {
    if (L.nitems == 0 || grid == 0 || L.ncomp == 0) return hipSuccess;
    const bool lat = L.table_rows != 0;
    const uint64_t lds = (lat ? column_table_bytes(L.table_rows, L.table_groups) : 0u) + (uint64_t)nslots * column_bytes(block, nslots != 0 && !lat && L.two_vectors);
    if (nslots > 255u || lds > column_lds_budget() || (lat && block != column_latency_block())) return hipErrorInvalidValue;
    switch (dtype) {
        case SAR_F32: return launch_column_dt<SAR_F32>(block, grid, (uint32_t)lds, nslots != 0, st, L);
        case SAR_F16: return launch_column_dt<SAR_F16>(block, grid, (uint32_t)lds, nslots != 0, st, L);
        case SAR_BF16: return launch_column_dt<SAR_BF16>(block, grid, (uint32_t)lds, nslots != 0, st, L);
        default: return hipErrorInvalidValue;
    }
}

// ---- fills -------------------------------------------------------------------

// fp32 -> bf16, round to nearest even, NaN quieted (fills are not hot: plain integer code)
__device__ __forceinline__ uint32_t bf16_round(float f) {
    uint32_t x = __float_as_uint(f);
    uint32_t r = (x + 0x7fffu + ((x >> 16) & 1u)) >> 16;
    uint32_t q = (x >> 16) | 0x40u;
    return ((x & 0x7fffffffu) > 0x7f800000u) ? q : r;
}

__device__ __forceinline__ uint16_t narrow16(float f, int dtype) {
    if (dtype == SAR_F16) { _Float16 h = (_Float16)f; return __builtin_bit_cast(uint16_t, h); }
    return (uint16_t)bf16_round(f);
}

// fill_pattern, allreduce_8GPU.cu:41-45
__global__ void fill_const_kernel(char* dst, uint64_t elems, float value, int dtype) {
    uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x, stride = (uint64_t)gridDim.x * blockDim.x;
    // (streaming stores, here and in fill_random_kernel: a fill in front of a timed run must not leave a cache's worth
    // of modified lines in the Infinity Cache for that run to push out)
    if (dtype == SAR_F32) { float* d = reinterpret_cast<float*>(dst); for (; i < elems; i += stride) __builtin_nontemporal_store(value, d + i); }
    else { uint16_t h = narrow16(value, dtype); uint16_t* d = reinterpret_cast<uint16_t*>(dst); for (; i < elems; i += stride) __builtin_nontemporal_store(h, d + i); }
}

__device__ __forceinline__ uint64_t mix64(uint64_t z) {
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

// mode 0: a + b*k/2^24;  mode 1: a + b*(sum of 12 such k/2^24 - 6)
__global__ void fill_random_kernel(char* dst, uint64_t elems, uint64_t key, double a, double b, int mode, int dtype) {
    uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x, stride = (uint64_t)gridDim.x * blockDim.x;
    for (; i < elems; i += stride) {
        double v;
        if (mode == 0) {
            uint64_t k = mix64(key + (i + 1) * 0x9E3779B97F4A7C15ull) >> 40;
            v = a + b * ((double)k * 0x1p-24);
        } else {
            uint64_t sum = 0;
            for (uint64_t j = 0; j < 12; ++j) sum += mix64(key + (i * 12 + j + 1) * 0x9E3779B97F4A7C15ull) >> 40;
            v = a + b * (((double)sum - 6.0 * 0x1p24) * 0x1p-24);
        }
        float f = (float)v;
        if (dtype == SAR_F32) __builtin_nontemporal_store(f, reinterpret_cast<float*>(dst) + i);
        else __builtin_nontemporal_store(narrow16(f, dtype), reinterpret_cast<uint16_t*>(dst) + i);
    }
}

// *differs is raised when rank buffers a and b differ anywhere in their first `bytes` bytes (bytes a multiple of 2)
__global__ void compare_kernel(const char* a, const char* b, uint64_t bytes, int* differs) {
    uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x, stride = (uint64_t)gridDim.x * blockDim.x;
    const uint16_t* x = reinterpret_cast<const uint16_t*>(a);
    const uint16_t* y = reinterpret_cast<const uint16_t*>(b);
    bool bad = false;
    for (uint64_t n = bytes >> 1; i < n; i += stride) bad |= (x[i] != y[i]);
    if (bad) atomicOr(differs, 1);
}

// dst <- src, 16 bytes per lane with streaming loads and stores (the < 16 bytes behind the last whole vector byte by
// byte): the copy that puts the inputs back before a timed run.  Streaming stores do not allocate in the 256 MB
// Infinity Cache, so the copy leaves no modified lines there for the run that follows to push out, and no part of
// the inputs in the caches either: the run starts cold.  Both pointers 16-byte aligned.
__global__ __launch_bounds__(256) void copy_kernel(char* __restrict__ dst, const char* __restrict__ src, uint64_t bytes) {
    const uint64_t nvec = bytes >> 4, step = (uint64_t)gridDim.x * blockDim.x;
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < nvec; i += step) st16<true>(dst + (i << 4), ld16<true>(src + (i << 4)));
    if (blockIdx.x == 0 && threadIdx.x < (uint32_t)(bytes & 15u)) dst[(nvec << 4) + threadIdx.x] = src[(nvec << 4) + threadIdx.x];
}

// gpu_sleep_kernel, allreduce_8GPU.cu:36-39: one lane spins until `ticks` of
// the constant-rate wall clock have passed.  The clock is monotonic, so the
// loop always ends; the host bounds `ticks`.
__global__ void sleep_kernel(uint64_t ticks) {
    uint64_t start = wall_clock64();
    while (wall_clock64() - start < ticks) __builtin_amdgcn_s_sleep(64);
}

hipError_t launch_fill_const(hipStream_t st, char* dst, uint64_t elems, float value, int dtype) {
    if (elems == 0) return hipSuccess;
    uint64_t blocks = (elems + 255) / 256; if (blocks > 8192) blocks = 8192;
    hipLaunchKernelGGL(fill_const_kernel, dim3((uint32_t)blocks), dim3(256), 0, st, dst, elems, value, dtype);
    return hipGetLastError();
}
hipError_t launch_fill_random(hipStream_t st, char* dst, uint64_t elems, uint64_t key, double a, double b, int mode, int dtype) {
    if (elems == 0) return hipSuccess;
    uint64_t blocks = (elems + 255) / 256; if (blocks > 16384) blocks = 16384;
    hipLaunchKernelGGL(fill_random_kernel, dim3((uint32_t)blocks), dim3(256), 0, st, dst, elems, key, a, b, mode, dtype);
    return hipGetLastError();
}
hipError_t launch_copy(hipStream_t st, char* dst, const char* src, uint64_t bytes) {
    if (bytes == 0) return hipSuccess;
    if ((((uintptr_t)dst | (uintptr_t)src) & 15u) != 0) return hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, st);
    uint64_t blocks = ((bytes >> 4) + 255) / 256;
    if (blocks < 1) blocks = 1;
    if (blocks > 16384) blocks = 16384;
    hipLaunchKernelGGL(copy_kernel, dim3((uint32_t)blocks), dim3(256), 0, st, dst, src, bytes);
    return hipGetLastError();
}
hipError_t launch_compare(hipStream_t st, const char* a, const char* b, uint64_t bytes, int* differs) {
    if (bytes < 2) return hipSuccess;
    uint64_t blocks = (bytes / 2 + 255) / 256; if (blocks > 8192) blocks = 8192;
    hipLaunchKernelGGL(compare_kernel, dim3((uint32_t)blocks), dim3(256), 0, st, a, b, bytes, differs);
    return hipGetLastError();
}
// Region probe: four write streams in window a and four in window b, stream_bytes each, all running at once.
// How long it takes tells whether the two windows lie in the same region of HBM (see find_pair in
// placed_pool.cpp).  The kernel times itself on the device's constant-rate wall clock -- stamps[0] = earliest start,
// stamps[1] = latest end with all stores acknowledged, preset by the host to ~0 and 0 -- so that neither launch
// overhead nor a profiler's bookkeeping enters the figure.
__global__ __launch_bounds__(256) void region_probe_kernel(char* a, char* b, uint64_t stream_bytes, unsigned long long* stamps) {
    if (threadIdx.x == 0) atomicMin(&stamps[0], (unsigned long long)wall_clock64());
    const uint64_t nvec = stream_bytes >> 4, step = (uint64_t)gridDim.x * blockDim.x;
    const f4 v = {1.f, 2.f, 3.f, 4.f};
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < nvec; i += step) {
#pragma unroll
        for (uint32_t k = 0; k < 4u; ++k) {
            st16<false>(a + k * stream_bytes + (i << 4), v);
            st16<false>(b + k * stream_bytes + (i << 4), v);
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");       // this wave's stores acknowledged (no cache write-back)
    __syncthreads();
    if (threadIdx.x == 0) atomicMax(&stamps[1], (unsigned long long)wall_clock64());
}
hipError_t launch_region_probe(hipStream_t st, char* a, char* b, uint64_t stream_bytes, unsigned long long* stamps) {
    hipLaunchKernelGGL(region_probe_kernel, dim3(2048), dim3(256), 0, st, a, b, stream_bytes, stamps);
    return hipGetLastError();
}
// Stream probe: what the memory system delivers for a given mix of read and written streams, by a kernel that has
// nothing else to do.  A job is up to 8 streams read and up to 8 written, all `bytes` long; every 16-byte vector
// of a job is the fp32 sum of its read streams (a constant when there is none), stored to each of its written
// streams.  A stream that is both read and written is updated in place, as an exchange does.  Tiles of BLOCK * U
// vectors, one per workgroup (PERSIST = false: the dispatcher hands them out) or a grid of 8 workgroups per CU
// striding over them; tiles job by job or, `interleave`, the jobs taking turns.  POL as for the column kernel: 0 = cached
// accesses, 1 = streaming loads and cached stores, 2 = streaming loads and stores.
template <int R, int U, int POL, bool PERSIST>
__global__ __launch_bounds__(1024) void stream_probe_kernel(ProbeJobs J, uint32_t tiles_per_job, uint32_t interleave) {
    constexpr bool LNT = POL >= 1, SNT = POL == 2;
    const uint32_t ntiles = tiles_per_job * J.njobs;
    const uint64_t nvec = J.bytes >> 4;
    for (uint32_t tile = blockIdx.x; tile < ntiles; tile += PERSIST ? gridDim.x : ntiles) {
        const uint32_t job = interleave ? tile % J.njobs : tile / tiles_per_job;
        const uint32_t t = interleave ? tile / J.njobs : tile - job * tiles_per_job;
        const uint32_t nw = J.nwrite[job];
        const uint64_t first = (uint64_t)t * U * blockDim.x + threadIdx.x;
        const bool whole = ((uint64_t)t + 1u) * U * blockDim.x <= nvec;       // all loads of a whole tile go out together
        f4 v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint64_t i = first + (uint64_t)u * blockDim.x;
            v[u] = R ? f4{0.f, 0.f, 0.f, 0.f} : f4{1.f, 2.f, 3.f, 4.f};
            if (whole || i < nvec) {
#pragma unroll
                for (int k = 0; k < R; ++k) v[u] += ld16<LNT>(J.rd[job][k] + (i << 4));
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint64_t i = first + (uint64_t)u * blockDim.x;
            if (whole || i < nvec)
                for (uint32_t w = 0; w < nw; ++w) st16<SNT>(J.wr[job][w] + (i << 4), v[u]);
        }
    }
}

template <int R>
static hipError_t launch_stream_probe_r(hipStream_t st, const ProbeJobs& J, uint32_t grid, int block, uint32_t tiles_per_job, int unroll, int policy, bool persistent, uint32_t il) {
#define SAR_PROBE(U, POL, P) hipLaunchKernelGGL((stream_probe_kernel<R, U, POL, P>), dim3(grid), dim3(block), 0, st, J, tiles_per_job, il)
#define SAR_PROBE_U(U)                                                                        \
    switch (policy * 2 + (persistent ? 1 : 0)) {                                              \
        case 0: SAR_PROBE(U, 0, false); break; case 1: SAR_PROBE(U, 0, true); break;          \
        case 2: SAR_PROBE(U, 1, false); break; case 3: SAR_PROBE(U, 1, true); break;          \
        case 4: SAR_PROBE(U, 2, false); break; case 5: SAR_PROBE(U, 2, true); break;          \
        default: return hipErrorInvalidValue;                                                 \
    }
    switch (unroll) {
        case 1: SAR_PROBE_U(1) break;
        case 2: SAR_PROBE_U(2) break;
        case 4: SAR_PROBE_U(4) break;
        default: return hipErrorInvalidValue;
    }
#undef SAR_PROBE_U
#undef SAR_PROBE
    return hipGetLastError();
}

// All jobs of a launch read the same number of streams (J.nread[0]); the written streams may differ in number.
hipError_t launch_stream_probe(hipStream_t st, const ProbeJobs& J, int block, int unroll, int policy, bool persistent, bool interleave, int compute_units) {
    if (policy < 0 || policy > 2) return hipErrorInvalidValue;
    if (J.njobs == 0 || J.njobs > 8 || J.bytes < 16 || (block != 256 && block != 512 && block != 1024)) return hipErrorInvalidValue;
    for (uint32_t j = 0; j < J.njobs; ++j) if (J.nread[j] != J.nread[0] || J.nread[j] > 8 || J.nwrite[j] > 8) return hipErrorInvalidValue;
    const uint64_t tile_vecs = (uint64_t)block * (uint64_t)unroll;
    const uint64_t tiles_per_job = ((J.bytes >> 4) + tile_vecs - 1) / tile_vecs;
    if (tiles_per_job * J.njobs > 0x7fffffffull) return hipErrorInvalidValue;
    const uint32_t ntiles = (uint32_t)(tiles_per_job * J.njobs), tpj = (uint32_t)tiles_per_job;
    const uint32_t grid = persistent ? (uint32_t)std::min<uint64_t>(ntiles, (uint64_t)std::max(1, compute_units) * 8u) : ntiles;
    const uint32_t il = interleave ? 1u : 0u;
    switch (J.nread[0]) {
        case 0: return launch_stream_probe_r<0>(st, J, grid, block, tpj, unroll, policy, persistent, il);
        case 1: return launch_stream_probe_r<1>(st, J, grid, block, tpj, unroll, policy, persistent, il);
        case 2: return launch_stream_probe_r<2>(st, J, grid, block, tpj, unroll, policy, persistent, il);
        case 3: return launch_stream_probe_r<3>(st, J, grid, block, tpj, unroll, policy, persistent, il);
        case 4: return launch_stream_probe_r<4>(st, J, grid, block, tpj, unroll, policy, persistent, il);
        case 5: return launch_stream_probe_r<5>(st, J, grid, block, tpj, unroll, policy, persistent, il);
        case 6: return launch_stream_probe_r<6>(st, J, grid, block, tpj, unroll, policy, persistent, il);
        case 7: return launch_stream_probe_r<7>(st, J, grid, block, tpj, unroll, policy, persistent, il);
        default: return launch_stream_probe_r<8>(st, J, grid, block, tpj, unroll, policy, persistent, il);
    }
}

hipError_t launch_sleep(hipStream_t st, uint64_t ticks) {
    hipLaunchKernelGGL(sleep_kernel, dim3(1), dim3(1), 0, st, ticks);
    return hipGetLastError();
}

}  // namespace sar
