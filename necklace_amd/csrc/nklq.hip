// nklq.hip — 2-bit gradient quantizer for MI355X (gfx950, CDNA4): kernels + C-ABI.
//
// Semantics follow necklace/cuda/quantize.py:16-51 (quantize) and :56-87
// (dequantize); the layout of the code words is the one of :34-51.  Nothing
// here is GEMM-shaped: every kernel is a single streaming pass bounded by HBM
// bandwidth, so the design is about memory access only:
//
//   * a flat vector is cut into chunks of 256 elements (1 KiB of fp32, 16 code
//     words).  A wave moves a chunk with one global_load_dwordx4 per array: 64
//     lanes x 16 B of contiguous memory;
//   * chunks are dealt to workgroups so that neighbouring chunks run on
//     different XCDs at about the same time (see chunk_of): the 8 XCDs then
//     sweep the arrays as one narrow front instead of eight distant ones, which
//     measures 5-8 % faster on HBM than handing each workgroup a contiguous
//     piece;
//   * a lane's 4 elements give one byte of codes; the 4 lanes of a quad are OR-ed
//     together with two DPP quad permutes (no LDS, no memory) to form the word of
//     16 codes;
//   * the residual is written back in the same pass (one read of g and r, one
//     write of r and of the codes: 12.25 bytes per element); the fp32 streams
//     use non-temporal loads and stores (touched once), the code words ordinary
//     ones (two chunks share a 128 B line of them);
//   * the last partial chunk goes through a bounds-checked one-element-per-lane
//     path in one extra workgroup of the same launch (codes combined across the
//     16 lanes of a DPP row);
//   * 64-bit element indices throughout (vectors of more than 2^31 elements);
//   * a cache line shared by two waves must be completed inside ONE XCD's L2 or it reaches memory
//     as two partial-line writes: views that start off a 128-byte line, and matrices whose rows
//     do, get workgroup -> work maps that keep neighbours on one XCD, and the decodes move
//     their grids onto lines (quant_flat_offline_kernel, deq_flat_shift_kernel, tile_of);
//   * the sum over K payloads (acc_flat_kernel), the matrix forms (quant_tiles_kernel for
//     wide matrices, quant_bands_kernel for up to 384 columns) and the many-vectors form
//     (quant_multi_kernel) are described at their kernels.
//
// fp32 arithmetic is IEEE: no fast-math, no contraction, denormals kept.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <algorithm>
#include <atomic>
#include <tuple>
#include <utility>
#include <vector>

#include "nklq.h"
#if defined(NKLQ_TUNING_BUILD) && NKLQ_TUNING_BUILD
#include "nklq_tuning.h"
#endif

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
// Same vector with only element alignment promised: gradient views cut out of a
// flat buffer (torch.narrow) start at any element.  gfx950 global memory
// instructions need dword alignment only, so these still move 16 bytes per lane.
typedef f32x4 f32x4_a4 __attribute__((aligned(4)));
typedef u32x4 u32x4_a4 __attribute__((aligned(4)));

// The product library carries one launch geometry (one chunk per wave, 256-thread workgroups) and the
// non-temporal forms only.  Built with -DNKLQ_TUNING_BUILD=1 the same source also carries the other
// geometries and the cached forms that nklq_tune can switch to, a plain copy kernel and the sum over
// interleaved payloads (include/nklq_tuning.h): what the launch-geometry sweeps and the knob tests need.
#ifndef NKLQ_TUNING_BUILD
#define NKLQ_TUNING_BUILD 0
#endif
#if NKLQ_TUNING_BUILD
#define NKLQ_NT(nt) (nt)
#else
#define NKLQ_NT(nt) true
#endif

constexpr int kWave = 64;
constexpr int kChunk = 256;          // elements per chunk: one dwordx4 per lane
constexpr int kWordsPerChunk = 16;

// Kernel arguments are fetched with scalar loads where the compiler first needs them; behind an early
// exit that is a second round trip to memory before the kernel's first vector load can be issued, and
// a short-lived workgroup lives about as long as its chain of round trips.  Naming the pointers here
// makes the compiler fetch them at the top, together with the other arguments.
template <typename P>
__device__ __forceinline__ void fetch_argument_now(P ptr)
{
    asm volatile("" : : "s"(ptr));
}
template <typename... P>
__device__ __forceinline__ void fetch_arguments_now(P... ptrs)
{
    (fetch_argument_now(ptrs), ...);
}

// ---------------------------------------------------------------- per element

// necklace/cuda/quantize.py:41-49.  `a >= t` is tested first; NaN fails both
// tests and is passed through with code 0.
__device__ __forceinline__ uint32_t quant_one(float a, float t, float& r)
{
    // Both candidates are computed and then selected (v_cndmask), so a wave
    // never branches on data.  The untouched case must be a copy, not a + 0.0f:
    // that would turn -0.0 into +0.0.
    const bool ge = a >= t;
    const bool le = a <= -t;
    const float up = a - t;
    const float dn = a + t;
    r = ge ? up : (le ? dn : a);
    return ge ? 1u : (le ? 2u : 0u);
}

// necklace/cuda/quantize.py:80-87: 01 -> +t, 10 -> -t, 00 and 11 -> +0.0
__device__ __forceinline__ float deq_code(uint32_t c2, float t)
{
    return (c2 == 1u) ? t : ((c2 == 2u) ? -t : 0.0f);
}

__device__ __forceinline__ f32x4 deq_byte(uint32_t b, float t)
{
    f32x4 v;
    v.x = deq_code(b & 3u, t);
    v.y = deq_code((b >> 2) & 3u, t);
    v.z = deq_code((b >> 4) & 3u, t);
    v.w = deq_code((b >> 6) & 3u, t);
    return v;
}

// ---------------------------------------------------------------- lane exchange

// OR over the 4 lanes of a quad; every lane gets the result.
__device__ __forceinline__ uint32_t quad_or(uint32_t v)
{
    // quad_perm [1,0,3,2] = 0xB1, [2,3,0,1] = 0x4E
    v |= (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0xB1, 0xF, 0xF, true);
    v |= (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0x4E, 0xF, 0xF, true);
    return v;
}

// OR over the 16 lanes of a DPP row; every lane gets the result.
__device__ __forceinline__ uint32_t row_or(uint32_t v)
{
    v = quad_or(v);
    // row_ror:4 = 0x124, row_ror:8 = 0x128
    v |= (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0x124, 0xF, 0xF, true);
    v |= (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0x128, 0xF, 0xF, true);
    return v;
}

// ---------------------------------------------------------------- memory access

template <bool ALIGNED, bool NT>
__device__ __forceinline__ f32x4 ld4(const float* p)
{
    if constexpr (ALIGNED) {
        const f32x4* q = reinterpret_cast<const f32x4*>(p);
        if constexpr (NT) return __builtin_nontemporal_load(q);
        else return *q;
    } else {
        const f32x4_a4* q = reinterpret_cast<const f32x4_a4*>(p);
        if constexpr (NT) return __builtin_nontemporal_load(q);
        else return *q;
    }
}

template <bool ALIGNED, bool NT>
__device__ __forceinline__ void st4(float* p, f32x4 v)
{
    if constexpr (ALIGNED) {
        f32x4* q = reinterpret_cast<f32x4*>(p);
        if constexpr (NT) __builtin_nontemporal_store(v, q);
        else *q = v;
    } else {
        f32x4_a4* q = reinterpret_cast<f32x4_a4*>(p);
        if constexpr (NT) __builtin_nontemporal_store(v, q);
        else *q = v;
    }
}

// ---------------------------------------------------------------- chunk -> workgroup map

// Workgroups are handed to the XCDs round-robin by workgroup id.  With
// X = 2^xs, workgroup b belongs to group b / X and has the slot k = b % X in
// it; a group covers X * WPB * U consecutive chunks and the workgroup takes
// those whose index is k modulo X: chunk j of wave w is
//     group * (X*WPB*U) + (j*WPB + w) * X + k.
// xs = 0 gives every workgroup one contiguous piece.
template <int U, int BLOCK>
__device__ __forceinline__ uint64_t chunk_of(uint32_t b, uint32_t w, int j, uint32_t xs)
{
    constexpr uint32_t WPB = BLOCK / kWave;
    const uint64_t group = b >> xs;
    const uint32_t k = b & ((1u << xs) - 1u);
    return group * ((uint64_t)(WPB * U) << xs) + ((uint64_t)(j * WPB + w) << xs) + k;
}

// ---------------------------------------------------------------- flat quantize

// Tail of a flat vector: elements [base, n), base a multiple of 256, fewer than
// 256 of them.  One element per lane; lane l of a DPP row owns code position l
// of the word.  All lanes of a wave reach the row_or.
template <bool ADD, int BLOCK>
__device__ __forceinline__ void quant_tail(const float* g, const float* rin, float* rout,
                                           uint32_t* c, uint64_t base, uint64_t n, float t)
{
    const int tid = threadIdx.x;
    for (int first = 0; first < kChunk; first += BLOCK) {
        const uint64_t e = base + (uint64_t)(first + tid);
        const bool live = (first + tid) < kChunk && e < n;
        uint32_t code = 0;
        if (live) {
            float a = g[e];
            if constexpr (ADD) a = a + rin[e];
            float r;
            code = quant_one(a, t, r);
            rout[e] = r;
        }
        const uint32_t word = row_or(code << (2 * (tid & 15)));
        if (live && (tid & 15) == 0) c[e >> 4] = word;
    }
}

// One launch quantizes the whole flat vector: gridDim.x - has_tail workgroups
// share the n_chunks full chunks, the last workgroup takes the tail.
template <int U, int BLOCK, bool ALIGNED, bool ADD, bool NT>
__global__ __launch_bounds__(BLOCK) void quant_flat_kernel(
    const float* g, const float* rin, float* rout, uint32_t* __restrict__ c, uint64_t n,
    uint64_t n_chunks, uint32_t has_tail, uint32_t xs, float t)
{
    if (has_tail && blockIdx.x == gridDim.x - 1) {
        quant_tail<ADD, BLOCK>(g, rin, rout, c, n_chunks * kChunk, n, t);
        return;
    }
    const int lane = threadIdx.x & (kWave - 1);
    const uint32_t w = threadIdx.x >> 6;
    uint64_t ch[U];
    f32x4 a[U];
    f32x4 r[U];
#pragma unroll
    for (int j = 0; j < U; ++j) ch[j] = chunk_of<U, BLOCK>(blockIdx.x, w, j, xs);
#pragma unroll
    for (int j = 0; j < U; ++j)
        if (ch[j] < n_chunks) a[j] = ld4<ALIGNED, NT>(g + ch[j] * kChunk + lane * 4);
    if constexpr (ADD) {
#pragma unroll
        for (int j = 0; j < U; ++j)
            if (ch[j] < n_chunks) r[j] = ld4<ALIGNED, NT>(rin + ch[j] * kChunk + lane * 4);
    }
#pragma unroll
    for (int j = 0; j < U; ++j) {
        if (ch[j] < n_chunks) {
            f32x4 v = a[j];
            if constexpr (ADD) v = v + r[j];
            float o0, o1, o2, o3;
            uint32_t b = quant_one(v.x, t, o0);
            b |= quant_one(v.y, t, o1) << 2;
            b |= quant_one(v.z, t, o2) << 4;
            b |= quant_one(v.w, t, o3) << 6;
            f32x4 o;
            o.x = o0; o.y = o1; o.z = o2; o.w = o3;
            st4<ALIGNED, NT>(rout + ch[j] * kChunk + lane * 4, o);
            // byte lane%4 of word lane/4; after the quad OR all 4 lanes hold the word
            const uint32_t word = quad_or(b << (8 * (lane & 3)));
            // plain store: the 64 B of a chunk's words share a cache line with the
            // next chunk's, and a non-temporal partial-line store measures slower
            if ((lane & 3) == 0) c[ch[j] * kWordsPerChunk + (lane >> 2)] = word;
        }
    }
}

// The same pass for a residual that does not start on a 128-byte line (a view cut out of a larger
// buffer at any element): every chunk's first and last line is then shared with the neighbouring
// chunk, and written from two XCDs the two parts reach memory as two partial-line writes.  Here
// chunks are dealt to the XCDs in runs of 16 (workgroup b runs on XCD b % 8; a run of 16 chunks = 4
// consecutive workgroups of ONE XCD, the next run goes to the next XCD), so that all but one
// boundary in 16 lies inside one XCD's L2, where the parts merge.  One chunk per wave, 256-thread
// workgroups.
constexpr uint32_t kRunChunks = 16;

template <bool ALIGNED, bool ADD, bool NT>
__global__ __launch_bounds__(256) void quant_flat_offline_kernel(
    const float* g, const float* rin, float* rout, uint32_t* __restrict__ c, uint64_t n,
    uint64_t n_chunks, uint32_t has_tail, float t)
{
    if (has_tail && blockIdx.x == gridDim.x - 1) {
        quant_tail<ADD, 256>(g, rin, rout, c, n_chunks * kChunk, n, t);
        return;
    }
    const int lane = threadIdx.x & (kWave - 1);
    const uint32_t w = threadIdx.x >> 6;
    const uint32_t xcd = blockIdx.x & 7u;
    const uint32_t j = blockIdx.x >> 3;
    const uint64_t run = (uint64_t)(j >> 2) * 8 + xcd;
    const uint64_t ch = run * kRunChunks + (j & 3u) * 4 + w;
    if (ch >= n_chunks) return;
    f32x4 v = ld4<ALIGNED, NT>(g + ch * kChunk + lane * 4);
    if constexpr (ADD) v = v + ld4<ALIGNED, NT>(rin + ch * kChunk + lane * 4);
    float o0, o1, o2, o3;
    uint32_t b = quant_one(v.x, t, o0);
    b |= quant_one(v.y, t, o1) << 2;
    b |= quant_one(v.z, t, o2) << 4;
    b |= quant_one(v.w, t, o3) << 6;
    f32x4 o;
    o.x = o0; o.y = o1; o.z = o2; o.w = o3;
    st4<ALIGNED, NT>(rout + ch * kChunk + lane * 4, o);
    const uint32_t word = quad_or(b << (8 * (lane & 3)));
    if ((lane & 3) == 0) c[ch * kWordsPerChunk + (lane >> 2)] = word;
}

// ---------------------------------------------------------------- flat dequantize

// out[j] = decode(c)[j]  (the reference dequantize, flat).  The 4 lanes of a quad read the
// same code word (one 64 B request per wave) and each takes its byte.  Code words are read
// with ordinary (cached) loads: two chunks share a 128 B line, and non-temporal loads of half
// lines measure 20-35 % slower here.  The target starts on a 128-byte line (any other start takes
// deq_flat_shift_kernel), so every store is a whole aligned 16 bytes.
//
// A workgroup here lives about as long as its one read of code words takes, and the chip holds a
// fixed number of them: when the words come from HBM instead of the memory-side cache (they were
// not written or read just before, or there are more of them than the cache holds) the read takes
// 2-3 times as long and the whole decode runs at 0.6 of the HBM peak instead of 0.95.  pf_lead > 0
// (xs = 0 only) adds 8 prefetch workgroups, one per XCD, behind every 256 working ones: each reads
// one word of every 128-byte line of code words that the workgroups pf_lead blocks of 256 further
// on will need, which brings the lines into the memory-side cache: 0.88 with words from HBM.  The
// second trip of the words over the fabric costs their share of the bytes, 6 %, when they were in the
// cache anyway (0.89 against 0.95), so the host side asks for it only where they cannot be.
constexpr uint32_t kPrefetchBlock = 256;  // working workgroups per block; 8 prefetching ones follow
template <int U, int BLOCK, bool NT>
__global__ __launch_bounds__(BLOCK) void deq_flat_kernel(
    float* out, const uint32_t* __restrict__ c, uint64_t n, uint64_t n_chunks, uint32_t has_tail,
    uint32_t xs, float t, uint32_t pf_lead)
{
    if (has_tail && blockIdx.x == gridDim.x - 1) {
        // tail: one element per lane, bounds-checked
        for (int first = 0; first < kChunk; first += BLOCK) {
            const uint64_t e = n_chunks * kChunk + (uint64_t)(first + threadIdx.x);
            if ((first + (int)threadIdx.x) < kChunk && e < n)
                out[e] = deq_code((c[e >> 4] >> (2 * (uint32_t)(e & 15))) & 3u, t);
        }
        return;
    }
    uint32_t b = blockIdx.x;
    if (pf_lead) {
        // working workgroup p of the vector stays on XCD p % 8, as without prefetching
        const uint32_t q = b / (kPrefetchBlock + 8), r = b - q * (kPrefetchBlock + 8);
        if (r >= kPrefetchBlock) {
            constexpr uint32_t words = (kPrefetchBlock / 8) * (BLOCK / kWave) * U * kWordsPerChunk;  // an eighth of a block's
            const uint64_t first = ((uint64_t)(q + pf_lead) * 8 + (r - kPrefetchBlock)) * words;
            uint32_t bits = 0;
            for (uint32_t i = threadIdx.x; i < words / 32; i += BLOCK) {
                const uint64_t wi = first + 32ull * i;
                if (wi < n_chunks * kWordsPerChunk) bits ^= c[wi];
            }
            asm volatile("" : : "v"(bits));  // (the loads have to be issued and waited for; their values are not used)
            return;
        }
        b = q * kPrefetchBlock + r;
    }
    const int lane = threadIdx.x & (kWave - 1);
    const uint32_t w = threadIdx.x >> 6;
    const uint32_t sh = 8 * (lane & 3);
#pragma unroll
    for (int j = 0; j < U; ++j) {
        const uint64_t ch = chunk_of<U, BLOCK>(b, w, j, xs);
        if (ch >= n_chunks) continue;
        const uint32_t word = c[ch * kWordsPerChunk + (lane >> 2)];
        st4<true, NT>(out + ch * kChunk + lane * 4, deq_byte((word >> sh) & 0xFFu, t));
    }
}

// Decode into a vector that does not start on a 128-byte line: the chunk grid is moved left by the
// d = 0..31 elements the vector's start lies past a line, so that every wave still writes whole,
// aligned lines: chunk j covers elements [256 j - d, 256 j - d + 256), clipped to the vector.  A
// lane's 4 elements then start at any code position, possibly across two words: the 8 bits are
// cut out of the 64-bit pair.  Only the first and the last quad can be partial (element by element).
template <bool NT>
__global__ __launch_bounds__(256) void deq_flat_shift_kernel(float* out, const uint32_t* __restrict__ c,
                                                             uint64_t n, uint64_t n_chunks, uint32_t d, float t)
{
    const int lane = threadIdx.x & (kWave - 1);
    const uint64_t ch = (uint64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (ch >= n_chunks) return;
    const int64_t e = (int64_t)(ch * kChunk) - (int64_t)d + lane * 4;
    if (e >= (int64_t)n || e + 4 <= 0) return;
    if (e >= 0 && e + 4 <= (int64_t)n) {
        const uint64_t wi = (uint64_t)e >> 4;
        const uint32_t sh = 2 * (uint32_t)(e & 15);
        uint64_t bits = c[wi];
        if (sh > 24) bits |= (uint64_t)c[wi + 1] << 32;  // the quad reaches into the next word (e + 3 < n: it exists)
        st4<true, NT>(out + e, deq_byte((uint32_t)(bits >> sh) & 0xFFu, t));
    } else {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int64_t ek = e + k;
            if (ek >= 0 && ek < (int64_t)n) out[ek] = deq_code((c[ek >> 4] >> (2 * (uint32_t)(ek & 15))) & 3u, t);
        }
    }
}

// ---------------------------------------------------------------- flat accumulate over payloads

struct PayloadPtrs {
    const uint32_t* p[NKLQ_MAX_PAYLOADS_PER_LAUNCH];
};

typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

constexpr int kTile = 1024;          // elements per wave in the accumulate kernels: 64 code words
constexpr int kAccBlock = 256;       // 4 waves, 4 tiles per workgroup
constexpr int kAccLdsPerWave = 1024; // LDS floats per wave: the 4 KiB of a tile's transpose
// Extra (unused) LDS given to every workgroup of a launch with at least kAccThrottleTiles tiles: it
// keeps a CU at 20 resident waves instead of 32, which measures 1-3 % faster on long vectors.  The
// kernel is bound by how HBM copes with K thin read streams next to one wide write stream, and
// fewer requests in flight serve it better; short vectors (one round of resident waves) want all
// 32 slots instead.
constexpr uint32_t kAccThrottleLdsBytes = 16384;
constexpr uint64_t kAccThrottleTiles = 1u << 16;

// Position in a wave's LDS area of 16-byte slot q (0..3) of row `row` (0..63; a row is the 16 sums
// one lane owns).  Rows are 16 floats apart; the slot index is XOR-ed with bits of the row so that
// both access patterns of the transpose are bank-conflict free for b128: a lane writing slot q of
// its own row (8 consecutive lanes: rows r..r+7) and a lane reading slot lane&3 of row lane>>2 + 16j
// (8 consecutive lanes: two rows, all four slots) each cover all 32 banks once.
__device__ __forceinline__ int lds_slot(int row, int q) { return 16 * row + 4 * (q ^ ((row >> 1) & 3)); }

// 2-bit codes -> 2 + b0 - b1 per field, all 16 fields of a word at once: 01 -> 11, 10 -> 01,
// 00 and 11 -> 10.  Per field the value is 1..3, so the subtraction never borrows across fields.
// Read as (sign, top exponent bit) of an IEEE half whose other bits are 0 these are -2, +2 and -0.
__device__ __forceinline__ uint32_t codes_to_half_tops(uint32_t w)
{
    return ((w & 0x55555555u) | 0xAAAAAAAAu) - ((w >> 1) & 0x55555555u);
}

// acc[j] = ((start + d_0[j]) + d_1[j]) + ... strictly in payload order, start = accumulate ?
// acc[j] : +0.0f, for one tile of 1024 elements.  A lane OWNS one code word of each payload (16
// elements): a wave fetches a payload's 64 words with one coalesced 256 B load, every shift is an
// immediate, and nothing moves between lanes during the sum.  The 16 running sums of a lane are
// 64 B apart in memory from its neighbour's, so the tile goes through LDS once on the way out (and
// once on the way in when accumulating) to become 1 KiB-contiguous stores.
//
// K > 0: exactly K payloads (loop fully unrolled, no dead registers); K == 0: k_payloads of them,
// at most NKLQ_MAX_PAYLOADS_PER_LAUNCH.
//
// MIX: for a finite t >= +0 whose half is exact, (+t, -t, +0) = h * th with th = -t/2 and h in
// {-2, +2, -0} exactly, and fma(h, th, s) rounds s + h*th once: the same bits as s + decode.  h
// is built as a half (the word's recoded field shifted to the top two bits of a 16-bit lane, two
// elements per register) and consumed by the mixed-precision fma, which converts it for free:
// one shift + one mask per TWO elements and one fma per element, against extract + convert + fma
// per element for an integer multiplier, or two compares + two selects + add for the plain form.
// Any other t (negative, NaN, infinite, below 2^-125) takes the plain form.
// PARTIAL: the last, shorter tile of a vector (rem = 1..1023 elements): the same pass with the words,
// loads and stores past the end masked (a quad cut by the end goes element by element); the codes of
// the last word past the end give sums that are never stored.
template <int K, bool ALIGNED, bool MIX, bool PARTIAL>
__device__ __forceinline__ void acc_tile(float* o, const PayloadPtrs& pl, int k_payloads, uint64_t word0,
                                         float t, float th, int accumulate, float divisor, float recip,
                                         float* my, int lane, uint32_t rem = kTile)
{
    constexpr int KMAX = K > 0 ? K : NKLQ_MAX_PAYLOADS_PER_LAUNCH;
    // every payload's word for this lane, all loads in flight together
    uint32_t wd[KMAX];
#pragma unroll
    for (int p = 0; p < KMAX; ++p)
        if (K > 0 || p < k_payloads) wd[p] = (!PARTIAL || (uint32_t)lane * 16 < rem) ? pl.p[p][word0 + lane] : 0u;

    float s[16];
    if (accumulate) {
        // coalesced read of the running sums, through LDS into the one-word-per-lane layout
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            f32x4 v;
            const uint32_t e = j * 256 + lane * 4;
            if (!PARTIAL || e + 4 <= rem) {
                v = ld4<ALIGNED, true>(o + e);
            } else {
                v.x = e < rem ? o[e] : 0.0f;
                v.y = e + 1 < rem ? o[e + 1] : 0.0f;
                v.z = e + 2 < rem ? o[e + 2] : 0.0f;
                v.w = 0.0f;
            }
            *reinterpret_cast<f32x4*>(my + lds_slot(16 * j + (lane >> 2), lane & 3)) = v;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const f32x4 v = *reinterpret_cast<const f32x4*>(my + lds_slot(lane, q));
            s[4 * q] = v.x; s[4 * q + 1] = v.y; s[4 * q + 2] = v.z; s[4 * q + 3] = v.w;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    } else {
#pragma unroll
        for (int i = 0; i < 16; ++i) s[i] = 0.0f;
    }

#pragma unroll
    for (int p = 0; p < KMAX; ++p) {
        if (K > 0 || p < k_payloads) {
            if constexpr (MIX) {
                const uint32_t m = codes_to_half_tops(wd[p]);
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    // elements i (low half) and i + 8 (high half) of the word
                    const f16x2 h = __builtin_bit_cast(f16x2, (m << (14 - 2 * i)) & 0xC000C000u);
                    s[i] = __builtin_fmaf((float)h.x, th, s[i]);
                    s[i + 8] = __builtin_fmaf((float)h.y, th, s[i + 8]);
                }
            } else {
#pragma unroll
                for (int i = 0; i < 16; ++i) s[i] = s[i] + deq_code((wd[p] >> (2 * i)) & 3u, t);
            }
        }
    }
    if (recip != 0.0f) {
        // the divisor is a power of two: its reciprocal is exact, so the product is the same real
        // number as the quotient and rounds to the same bits (one multiply instead of ~10 instructions)
#pragma unroll
        for (int i = 0; i < 16; ++i) s[i] = s[i] * recip;
    } else if (divisor != 1.0f) {  // IEEE division, correctly rounded
#pragma unroll
        for (int i = 0; i < 16; ++i) s[i] = s[i] / divisor;
    }

    // one-word-per-lane layout -> LDS -> 1 KiB-contiguous stores
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        f32x4 v;
        v.x = s[4 * q]; v.y = s[4 * q + 1]; v.z = s[4 * q + 2]; v.w = s[4 * q + 3];
        *reinterpret_cast<f32x4*>(my + lds_slot(lane, q)) = v;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const f32x4 v = *reinterpret_cast<const f32x4*>(my + lds_slot(16 * j + (lane >> 2), lane & 3));
        const uint32_t e = j * 256 + lane * 4;
        if (!PARTIAL || e + 4 <= rem) {
            st4<ALIGNED, true>(o + e, v);
        } else {
            if (e < rem) o[e] = v.x;
            if (e + 1 < rem) o[e + 1] = v.y;
            if (e + 2 < rem) o[e + 2] = v.z;
        }
    }
}

// RUNS (measurement builds only): the payloads are not k separate arrays but ONE array in which they
// alternate in runs of 2^run_shift words (payload p's j-th run starts at word (j * k + p) << run_shift
// of the array pl.p[0] points to; pl.p[p] = pl.p[0] + (p << run_shift)).  Same words, same bytes,
// same arithmetic; only how far apart in memory the k reads of one tile are changes.
template <int K, bool ALIGNED, bool MIX, bool RUNS = false>
__global__ __launch_bounds__(kAccBlock) void acc_flat_kernel(
    float* acc, PayloadPtrs pl, int k_payloads, uint64_t n, uint64_t n_tiles, uint32_t has_tail,
    uint32_t xs, float t, float th, int accumulate, uint32_t run_shift)
{
    __shared__ __attribute__((aligned(16))) float lds[kAccBlock / kWave][kAccLdsPerWave];
    const int lane = threadIdx.x & (kWave - 1);
    const uint32_t w = threadIdx.x >> 6;
    if (has_tail && blockIdx.x == gridDim.x - 1) {
        // the vector's last, shorter tile: one wave of the extra workgroup
        if (w == 0)
            acc_tile<K, ALIGNED, MIX, true>(acc + n_tiles * kTile, pl, k_payloads, n_tiles * (kTile / 16), t, th,
                                            accumulate, 1.0f, 0.0f, lds[0], lane, (uint32_t)(n - n_tiles * kTile));
        return;
    }
    const uint64_t tile = chunk_of<1, kAccBlock>(blockIdx.x, w, 0, xs);
    if (tile >= n_tiles) return;
    uint64_t word0 = tile * (kTile / 16);
    if constexpr (RUNS) word0 += ((word0 >> run_shift) * (uint64_t)((K > 0 ? K : k_payloads) - 1)) << run_shift;
    acc_tile<K, ALIGNED, MIX, false>(acc + tile * kTile, pl, k_payloads, word0, t, th, accumulate,
                                     1.0f, 0.0f, lds[w], lane);
}

// ---------------------------------------------------------------- matrix (n, k) kernels

// Word (x, y) packs rows 16x .. 16x+15 of column y (quantize.py:35-51), so the 16 codes of a
// word are k floats apart in memory: the 16 rows behind one row of words are a "band".  Which
// kernel a matrix takes depends on its number of columns k:
//   quantize  k <= kBandsMaxColumns: quant_bands_kernel (bands streamed as flat memory)
//             wider: quant_tiles_kernel (tiles of 16 rows x 128 or 256 columns)
//   decode    k <= 96: deq_bands_kernel (LDS image of whole bands)
//             97 .. 8192: deq_stream_kernel (no LDS; 4 KiB pieces of a band)
//             wider, or from 4096 with every row on a 128-byte line: deq_2d_rows_kernel (16 waves,
//             wave i = row i of a tile of 16 rows x 256 columns, one dwordx4 per lane)
// Rows may start at any element (k not a multiple of 4, bases only 4-byte aligned): the same
// 16-byte requests are issued with dword alignment, and quads cut by a row end are masked.
constexpr int kRowsBlock = 16 * kWave;  // 1024 threads

// Workgroup -> tile (band x, column tile T) of the tile decode.  Workgroups go to the 8 XCDs
// round-robin by id; pinned = 1: the tiles of one band are given to ONE XCD, in column order, and 8
// neighbouring bands run side by side on the 8 XCDs; pinned = 0: plain row-major order.  Returns
// false for the padding workgroups of the last group of bands.
__device__ __forceinline__ bool rows_tile_of(uint32_t b, uint32_t col_tiles, uint64_t m, uint64_t* x,
                                             uint32_t* T, uint32_t pinned = 1)
{
    if (!pinned) {
        *x = b / col_tiles;
        *T = b % col_tiles;
        return *x < m;
    }
    const uint32_t e = b & 7u;
    const uint32_t j = b >> 3;
    *x = (uint64_t)(j / col_tiles) * 8 + e;
    *T = j % col_tiles;
    return *x < m;
}

// ---- quantize by tiles of 16 rows x 128 columns (more than kBandsMaxColumns columns)
//
// A workgroup of 8 waves takes a tile; a wave moves two rows' pieces of 512 bytes, lane = 4
// columns.  The 16 codes of a word come from 16 different lanes of 8 waves: every lane writes its 4
// codes as 4 bytes into an image of the tile in LDS (row-major like the tile, no zeroing, no
// atomics), and after ONE barrier 128 lanes gather the 16 bytes of their column into a word.
// (Measured against the form it replaced, 16 waves x one row of 256 columns OR-ing codes into
// zeroed LDS words between two barriers: 8192 x 8192 fused 0.81 -> 0.85 of the HBM peak,
// 100000 x 1000 0.77 -> 0.81; 4 waves x 4 rows of 64 columns 0.76-0.80.)
//
// Rows that do not start on 128-byte lines make neighbouring tiles of a row share a line at their
// common edge; written from two XCDs (two L2s) it reaches memory as two partial-line writes.
//   * EDGES: the tiles of one band are given to ONE XCD (TileMap), so that a line both tiles read is
//     fetched once: 8191 x 8191 0.59 in plain order, 0.77 pinned.  The two halves of a shared line
//     are still written separately: 4-6 % more 64-byte write requests than the bytes need.
//   * SHIFT: each row's window is moved left by the s = 0..31 elements the row's start lies past a
//     line: columns [128 T - s, 128 T + 128 - s), so every store is whole lines.  The tile still owns
//     the words of columns [128 T, 128 T + 128): the s elements its window misses at the right end are
//     loaded a second time (8 lanes per row, one line, an L2 hit as the neighbour runs on the same
//     XCD) for their codes only; their residual belongs to the neighbour.  That is a second reader
//     of elements another workgroup updates, so this form is ONLY for calls whose residual output
//     aliases neither input (the reference's own kernel, quantize.py:41-49, with R apart from A; the
//     fused step with three buffers): in place, the neighbour may already have replaced r by r'.
//     8191 x 8191 0.80, 16384 x 16383 0.81 against 0.77 / 0.76 with EDGES; write requests then equal
//     the bytes.  Used from 4096 columns on: below, the re-read fringe costs more than it saves.

// Workgroup -> (band x, column tile T).  Workgroups go to the 8 XCDs round-robin by id.  Plain order
// (pinned = 0) when every row starts on a line.  Pinned: bands are dealt to the XCDs in groups of
// 8, the tiles of a band run on one XCD in column order.  The last group may have fewer than 8
// bands: its bands are then cut into 2^seg_shift segments of `seg_tiles` consecutive tiles, one XCD
// each, so that no XCD stays idle.
// Plain order with runs (pinned = 0, run_shift > 0), for matrices of a few bands with rows off
// lines: tiles in row-major order, but every XCD takes 2^run_shift NEIGHBOURING tiles of each group
// of 8 * 2^run_shift, so that most lines shared between tiles are fetched by one XCD only while all
// XCDs still work on the same few megabytes (16 x 4,000,001 in place: 0.62 of the HBM peak in plain
// order, 0.67 / 0.70 / 0.69 with runs of 2 / 4 / 8; with whole bands or long segments per XCD 0.15-0.58).
struct TileMap {
    uint64_t inv_tiles;    // floor(2^64 / col_tiles) + 1
    uint32_t col_tiles;
    uint32_t full_blocks;  // pinned: workgroups of the full groups of 8 bands; runs: workgroups in whole groups
    uint32_t last_bands;   // bands of the last, smaller group (0: none)
    uint64_t last_first;   // and the first of them
    uint32_t seg_shift, seg_tiles;
    uint32_t pinned;
    uint32_t run_shift;
};

__device__ __forceinline__ bool tile_of(const TileMap& tm, uint32_t b, uint64_t* x, uint32_t* T)
{
    if (!tm.pinned) {
        if (tm.run_shift && b < tm.full_blocks) {
            // within its group of 8 << run_shift workgroups: XCD (b & 7) takes tiles (b & 7) << run_shift ...
            const uint32_t group = 8u << tm.run_shift, o = b & (group - 1);
            b = (b - o) + ((o & 7u) << tm.run_shift) + (o >> 3);
        }
        const uint32_t q = tm.col_tiles == 1 ? b : (uint32_t)__umul64hi((uint64_t)b, tm.inv_tiles);
        *x = q;
        *T = b - q * tm.col_tiles;
        return true;
    }
    if (b < tm.full_blocks) {
        const uint32_t e = b & 7u, j = b >> 3;
        const uint32_t q = tm.col_tiles == 1 ? j : (uint32_t)__umul64hi((uint64_t)j, tm.inv_tiles);
        *x = (uint64_t)q * 8 + e;
        *T = j - q * tm.col_tiles;
        return true;
    }
    const uint32_t bl = b - tm.full_blocks, e = bl & 7u, j = bl >> 3;
    const uint32_t band = e >> tm.seg_shift, seg = e & ((1u << tm.seg_shift) - 1u);
    *x = tm.last_first + band;
    *T = seg * tm.seg_tiles + j;
    return band < tm.last_bands && *T < tm.col_tiles;
}

// Elements [y, y + 4) of a row of k >= 4 elements; those outside the row read as 0.  ONE 16-byte load
// for every lane, whole quad or not: a quad cut by an end of the row loads the four elements at that
// end instead (address clamped into the row) and moves them into place.  (Loading the elements of a
// cut quad one by one, in a branch of its own, made the compiler wait for the other lanes' loads
// first: a second round trip to memory for every wave with a row end in it.)
template <bool NT>
__device__ __forceinline__ f32x4 ld4_row(const float* rowp, int64_t y, int64_t k)
{
    const int64_t yc = y < 0 ? 0 : (y + 4 > k ? k - 4 : y);
    f32x4 w = ld4<false, NT>(rowp + yc);  // (dword alignment: the same global_load_dwordx4)
    const int d = (int)(y - yc);          // -3 .. 3; element j of the quad is w[j + d]
    if (d != 0) {
        const float e[4] = {w.x, w.y, w.z, w.w};
        float o[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float v = 0.0f;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (i - j == d) v = e[i];   // (i - j ranges over -3 .. 3: at most one i per j matches)
            o[j] = v;
        }
        w.x = o[0]; w.y = o[1]; w.z = o[2]; w.w = o[3];
    }
    return w;
}

// 4 codes as 4 bytes and the 4 residuals of a quad; the codes of elements outside the row are 0
template <bool ADD>
__device__ __forceinline__ uint32_t quant_quad(f32x4 va, f32x4 vr, float t, int64_t y, int64_t k, f32x4* o)
{
    f32x4 v = va;
    if constexpr (ADD) v = v + vr;
    float o0, o1, o2, o3;
    uint32_t codes = quant_one(v.x, t, o0) | (quant_one(v.y, t, o1) << 8) | (quant_one(v.z, t, o2) << 16) |
                     (quant_one(v.w, t, o3) << 24);
    o->x = o0; o->y = o1; o->z = o2; o->w = o3;
    if (!(y >= 0 && y + 4 <= k)) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (!(y + j >= 0 && y + j < k)) codes &= ~(0xFFu << (8 * j));
    }
    return codes;
}

// W columns per tile, Q quads per lane (4 W / Q threads): 128 x 1 when no line is shared between
// tiles (rows on lines, or SHIFT), 256 x 1 with EDGES and long rows (half as many shared lines:
// 16384 x 16383 in place 0.74 with 128 columns, 0.78 with 256; but 150000 x 401 0.75 / 0.64; the
// host side has the rule) and for matrices of a few bands.  More quads per lane (1024 columns per
// tile) measured no better anywhere.
template <int W, int Q, bool ADD, bool NT, bool SHIFT>
__global__ __launch_bounds__(4 * W / Q) void quant_tiles_kernel(
    const float* g, const float* rin, float* rout, uint32_t* __restrict__ c, uint64_t n, uint64_t k, TileMap tm,
    float t)
{
    constexpr int BLOCK = 4 * W / Q;           // 16 rows x (W / 4) quads / Q quads per lane
    constexpr int TPR = W / 4 / Q;             // lanes per row
    constexpr int ROWB = SHIFT ? W + 32 : W;   // image bytes per row: the window, and the 32 elements after it
    static_assert(BLOCK == 16 * TPR && BLOCK <= 1024 && TPR >= 8, "tile geometry");
    __shared__ __attribute__((aligned(16))) uint8_t image[16 * ROWB];
    fetch_arguments_now(g, rin, rout, c);
    uint64_t x;
    uint32_t T;
    if (!tile_of(tm, blockIdx.x, &x, &T)) return;
    if (x * 16 >= n) return;  // padding workgroups of the last group of 8 bands
    const uint32_t i = threadIdx.x / TPR;  // row within the tile = code position within the word
    const uint32_t l = threadIdx.x % TPR;  // lane within the row
    const uint64_t row = x * 16 + i;
    const int64_t kk = (int64_t)k;
    uint32_t codes[Q], codes_after = 0;
#pragma unroll
    for (int q = 0; q < Q; ++q) codes[q] = 0;
    if (row < n) {
        const float* grow = g + row * k;
        const float* rrow = rin + row * k;
        float* orow = rout + row * k;
        const int64_t s = SHIFT ? (int64_t)((reinterpret_cast<uintptr_t>(orow) >> 2) & 31u) : 0;
        const int64_t y0 = (int64_t)T * W - s + 4 * l;      // this lane's first quad; the next ones 4 TPR columns on
        const int64_t ya = y0 + W;                          // for the first lanes: the quad one window on
        const bool on_after = SHIFT && 4 * (int64_t)l < s && ya < kk;
        f32x4 va[Q], vr[Q], wa = {0.0f, 0.0f, 0.0f, 0.0f}, wr = wa;
#pragma unroll
        for (int q = 0; q < Q; ++q) {
            const int64_t y = y0 + 4 * TPR * q;
            va[q] = wa;
            vr[q] = wa;
            if (y + 4 > 0 && y < kk) {
                va[q] = ld4_row<NT>(grow, y, kk);
                if constexpr (ADD) vr[q] = ld4_row<NT>(rrow, y, kk);
            }
        }
        if (on_after) {
            wa = ld4_row<NT>(grow, ya, kk);
            if constexpr (ADD) wr = ld4_row<NT>(rrow, ya, kk);
        }
#pragma unroll
        for (int q = 0; q < Q; ++q) {
            const int64_t y = y0 + 4 * TPR * q;
            if (y + 4 > 0 && y < kk) {
                f32x4 o;
                codes[q] = quant_quad<ADD>(va[q], vr[q], t, y, kk, &o);
                if (y >= 0 && y + 4 <= kk) {
                    st4<false, NT>(orow + y, o);  // (dword alignment: the same global_store_dwordx4)
                } else {
                    const float oe[4] = {o.x, o.y, o.z, o.w};
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        if (y + j >= 0 && y + j < kk) orow[y + j] = oe[j];
                }
            }
        }
        if (on_after) {
            f32x4 o;
            codes_after = quant_quad<ADD>(wa, wr, t, ya, kk, &o);
        }
    }
    // image[i][p] = code of column W T - s_i + p of row i
#pragma unroll
    for (int q = 0; q < Q; ++q) *reinterpret_cast<uint32_t*>(&image[i * ROWB + 4 * (l + TPR * q)]) = codes[q];
    if (SHIFT && l < 8) *reinterpret_cast<uint32_t*>(&image[i * ROWB + W + 4 * l]) = codes_after;
    __syncthreads();
    for (uint32_t cc = threadIdx.x; cc < (uint32_t)W; cc += BLOCK) {
        const uint64_t col = (uint64_t)T * W + cc;
        if (col < k) {
            uint32_t s = SHIFT ? (uint32_t)((reinterpret_cast<uintptr_t>(rout + x * 16 * k) >> 2) & 31u) : 0u;
            const uint32_t k32 = (uint32_t)(k & 31u);
            uint32_t word = 0;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                word |= (uint32_t)image[r * ROWB + cc + s] << (2 * r);
                if constexpr (SHIFT) s = (s + k32) & 31u;  // the next row starts k elements on
            }
            c[x * k + col] = word;
        }
    }
}

// Decode of a tile.  SHIFT = false: every row starts on a 128-byte line (k a multiple of 32, base
// on a line) and wave i writes columns [256 T, 256 T + 256) of its row.  SHIFT = true: each row's
// window is moved left by the s = 0..31 elements its start lies past a line, so that a wave still
// writes whole, aligned lines: columns [256 T - s, 256 T + 256 - s), clipped to the row (one more
// column tile covers the rows' ends).  Nothing is shared between rows here, so the windows of the
// 16 rows need not coincide; only the first and last line of a row are partial.  All 16 waves
// read the tile's words (cache hits after the first).
template <bool NT, bool SHIFT>
__global__ __launch_bounds__(kRowsBlock) void deq_2d_rows_kernel(
    float* out, const uint32_t* __restrict__ c, uint64_t n, uint64_t k, uint32_t col_tiles, float t, uint32_t pinned)
{
    const int lane = threadIdx.x & (kWave - 1);
    const uint32_t i = threadIdx.x >> 6;
    uint64_t x;
    uint32_t T;
    if (!rows_tile_of(blockIdx.x, col_tiles, (n + 15) / 16, &x, &T, pinned)) return;
    const uint64_t row = x * 16 + i;
    if (row >= n) return;
    float* orow = out + row * k;
    const int64_t s = SHIFT ? (int64_t)((reinterpret_cast<uintptr_t>(orow) >> 2) & 31u) : 0;
    const int64_t y = (int64_t)T * 256 - s + lane * 4;  // first of this lane's 4 columns
    if (y >= (int64_t)k || y + 4 <= 0) return;
    const uint32_t sh = 2 * i;
    const uint32_t* cw = c + x * k;
    if (y >= 0 && y + 4 <= (int64_t)k) {
        uint32_t w0, w1, w2, w3;
        if constexpr (SHIFT) {
            const u32x4_a4 w = *reinterpret_cast<const u32x4_a4*>(cw + y);
            w0 = w.x; w1 = w.y; w2 = w.z; w3 = w.w;
        } else {
            const u32x4 w = *reinterpret_cast<const u32x4*>(cw + y);
            w0 = w.x; w1 = w.y; w2 = w.z; w3 = w.w;
        }
        f32x4 v;
        v.x = deq_code((w0 >> sh) & 3u, t);
        v.y = deq_code((w1 >> sh) & 3u, t);
        v.z = deq_code((w2 >> sh) & 3u, t);
        v.w = deq_code((w3 >> sh) & 3u, t);
        st4<true, NT>(orow + y, v);  // 16-byte aligned in both forms
    } else {
        // a quad cut by an end of the row: its words are requested together (column clamped into the
        // row) and then stored one by one; load - store - load - store would be four memory round
        // trips in a row, and a wave lives about as long as its round trips take
        uint32_t w[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int64_t yj = y + j < 0 ? 0 : (y + j < (int64_t)k ? y + j : (int64_t)k - 1);
            w[j] = cw[yj];
        }
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (y + j >= 0 && y + j < (int64_t)k) orow[y + j] = deq_code((w[j] >> sh) & 3u, t);
    }
}

// ---- matrices of up to kBandsMaxColumns columns
//
// The 16 rows behind one row of code words ("a band") are 16 k CONTIGUOUS floats in memory and
// give k contiguous words.  With few columns a 256-column tile would leave most lanes idle, and
// walking down a column touches one float per row; instead a workgroup takes whole bands as a
// flat stream: `bands_per_wg` bands when a band is short (so that the range is 2048-4096
// elements), one band otherwise.  The range is read and written 16 bytes per lane like a flat vector
// (quads laid out from a 16-byte boundary of the residual, so only the first and last quad of a range
// can be partial and go element by element), each element finds its (row, column) by one
// multiply-high with a precomputed reciprocal of k, and its code is OR-ed into the band's words in
// LDS; after a barrier the words are stored, contiguous.
constexpr int kBandsBlock = 256;
constexpr uint64_t kBandsMaxColumns = 384;  // LDS words per workgroup; wider matrices take the row tiles (measured crossover: 300-500 columns)
constexpr uint64_t kBandsRangeQuant = 2048;      // elements per workgroup when bands are short: quantize
constexpr uint64_t kBandsDecodeElems = 960;      // decode: elements per workgroup, at least (about one quad per lane)
constexpr uint64_t kBandsDecodeWholeMax = 1536;  // decode: bands up to this many elements (96 columns) go through the LDS image
// words of a workgroup of whole bands: k of one band of at least kBandsDecodeElems elements, or fewer than
// 2 * kBandsDecodeElems / 16 of several shorter ones
static_assert(kBandsDecodeWholeMax / 16 <= (uint64_t)kBandsBlock && 2 * (kBandsDecodeElems / 16) <= (uint64_t)kBandsBlock,
              "words of whole bands: one per lane");

// (row within the workgroup's range, column) of local element index li; inv = floor(2^32 / k) + 1,
// exact for li * k < 2^32 (li < 16384, k <= 1024 here).
__device__ __forceinline__ void band_row_col(uint32_t li, uint32_t k, uint32_t inv, uint32_t* row, uint32_t* col)
{
    const uint32_t q = __umulhi(li, inv);
    *row = q;
    *col = li - q * k;
}

// Workgroup -> range.  A range rarely starts on a 128-byte line, so neighbouring ranges share one:
// ranges are dealt to the XCDs in runs of kBandRun (workgroup b runs on XCD b % 8), so that all but
// one shared line in kBandRun is completed inside one XCD's L2.
constexpr uint32_t kBandRun = 8;
__device__ __forceinline__ uint64_t band_range_of(uint32_t b)
{
    const uint32_t xcd = b & 7u, j = b >> 3;
    return ((uint64_t)(j / kBandRun) * 8 + xcd) * kBandRun + (j % kBandRun);
}

template <bool ADD, bool NT, bool ALIGNED>
__global__ __launch_bounds__(kBandsBlock) void quant_bands_kernel(
    const float* g, const float* rin, float* rout, uint32_t* __restrict__ c, uint64_t n, uint32_t k,
    uint32_t bands_per_wg, uint32_t inv, float t)
{
    __shared__ uint32_t words[kBandsMaxColumns];
    const uint64_t m = (n + 15) / 16;
    const uint64_t x0 = band_range_of(blockIdx.x) * bands_per_wg;
    if (x0 >= m) return;  // padding workgroups of the last group of runs
    const uint64_t x1 = (x0 + bands_per_wg < m) ? x0 + bands_per_wg : m;
    const uint64_t e0 = x0 * 16 * k;
    const uint64_t e1 = (x1 * 16 < n ? x1 * 16 : n) * k;
    const uint32_t n_words = (uint32_t)(x1 - x0) * k;
    const uint32_t len = (uint32_t)(e1 - e0);
    for (uint32_t w = threadIdx.x; w < n_words; w += kBandsBlock) words[w] = 0;
    __syncthreads();
    // quads start `a` elements before the range, on a 16-byte boundary of rout
    const uint32_t a = (uint32_t)((reinterpret_cast<uintptr_t>(rout + e0) >> 2) & 3u);
    const float* gq = g + e0;
    const float* rq = rin + e0;
    float* oq = rout + e0;
    // local index of a quad's first element, relative to e0: -a + 4 * quad (negative only for quad 0)
    constexpr int U = 4;  // quads per lane whose loads are issued together
    for (int32_t base = -(int32_t)a + 4 * (int32_t)threadIdx.x; base < (int32_t)len; base += U * 4 * kBandsBlock) {
        f32x4 va[U], vr[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int32_t li = base + u * 4 * kBandsBlock;
            if (li >= 0 && li + 4 <= (int32_t)len) {
                va[u] = ld4<ALIGNED, NT>(gq + li);
                if constexpr (ADD) vr[u] = ld4<ALIGNED, NT>(rq + li);
            } else {
                float xa[4] = {0.0f, 0.0f, 0.0f, 0.0f}, xr[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if (li + j >= 0 && li + j < (int32_t)len) {
                        xa[j] = gq[li + j];
                        if constexpr (ADD) xr[j] = rq[li + j];
                    }
                }
                va[u].x = xa[0]; va[u].y = xa[1]; va[u].z = xa[2]; va[u].w = xa[3];
                if constexpr (ADD) { vr[u].x = xr[0]; vr[u].y = xr[1]; vr[u].z = xr[2]; vr[u].w = xr[3]; }
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int32_t li = base + u * 4 * kBandsBlock;
            if (li >= (int32_t)len) break;
            f32x4 v = va[u];
            if constexpr (ADD) v = v + vr[u];
            float in[4] = {v.x, v.y, v.z, v.w};
            float o[4];
            uint32_t code[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) code[j] = quant_one(in[j], t, o[j]);
            const bool full = li >= 0 && li + 4 <= (int32_t)len;
            if (full) {
                f32x4 vo;
                vo.x = o[0]; vo.y = o[1]; vo.z = o[2]; vo.w = o[3];
                st4<true, NT>(oq + li, vo);
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    if (li + j >= 0 && li + j < (int32_t)len) oq[li + j] = o[j];
            }
            uint32_t row, col;
            band_row_col((uint32_t)(li < 0 ? 0 : li), k, inv, &row, &col);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (li + j >= 0 && li + j < (int32_t)len) {
                    // word of (row, col): band row / 16 of this range, bits of row % 16
                    if (code[j]) atomicOr(&words[(row >> 4) * k + col], code[j] << (2 * (row & 15u)));
                    if (++col == k) { col = 0; ++row; }
                }
            }
        }
    }
    __syncthreads();
    uint32_t* cq = c + x0 * k;
    for (uint32_t w = threadIdx.x; w < n_words; w += kBandsBlock) cq[w] = words[w];
}

// Decode of bands.  What the write stream to HBM wants decided the shape (all measured):
//   * a workgroup writes a little over 4 KiB and ends, and workgroup i writes the i-th piece: the
//     chip then sweeps the matrix as one narrow front, like the flat decode.  With 2, 4, 8 stores
//     per lane (8 to 32 KiB per workgroup) the same stores ran at 0.81, 0.80, 0.75 of the HBM peak
//     where one store per lane runs at 0.89;
//   * with so little to do a workgroup lives about as long as its chain of dependent steps takes
//     (arguments, code words, LDS, barrier, store), and the rate is the bytes of the resident
//     workgroups over that time: every step added to the chain shows (a second round trip to memory
//     behind the first cost 20 %, a few dozen scalar instructions of index arithmetic 5-15 %).  So
//     the code words are requested at once, one per lane, and everything that can be worked out on
//     the host is.
// A workgroup's elements are whole rows, contiguous in memory: `bands_per_wg` whole bands;
// for longer bands see deq_stream_kernel.
//
// A lane decodes the rows of ITS word with immediate shifts (no row or column arithmetic per
// element) and writes the floats into the range's image in LDS, `k` floats apart; lanes with
// neighbouring words write neighbouring floats, so the writes are free of bank conflicts.  After a
// barrier the image leaves as 16-byte quads laid out from a 16-byte boundary of `out` (LDS reads of
// 16 bytes per lane, stores of 1 KiB per wave); only the first and the last quad of a range can be
// partial.
//
// MIX: (+t, -t, +0) = h * th with th = -t/2 and h in {-2, +2, -0} taken from the recoded word as IEEE
// halves, two elements per shift-and-mask (see acc_tile); the addend -0 keeps every result exact,
// also -t = -0 for t = +0.  Any other t takes compare-and-select.
template <bool NT>
__device__ __forceinline__ void band_image_out(const float* band_image, float* oq, uint32_t a, uint32_t len)
{
    for (int32_t li = -(int32_t)a + 4 * (int32_t)threadIdx.x; li < (int32_t)len; li += 4 * kBandsBlock) {
        f32x4 v = *reinterpret_cast<const f32x4*>(band_image + (li + (int32_t)a));
        asm volatile("" : "+v"(v));  // keeps the load one 16-byte LDS read (element uses below would split it)
        if (li >= 0 && li + 4 <= (int32_t)len) {
            st4<true, NT>(oq + li, v);
        } else {
            const float e[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (li + j >= 0 && li + j < (int32_t)len) oq[li + j] = e[j];
        }
    }
}

template <bool NT, bool MIX>
__global__ __launch_bounds__(kBandsBlock) void deq_bands_kernel(
    float* out, const uint32_t* __restrict__ c, uint64_t n, uint32_t k, uint32_t bands_per_wg, uint32_t inv,
    float t, float th)
{
    extern __shared__ __attribute__((aligned(16))) float band_image_base[];  // 4 + bands_per_wg * 16 * k floats
    float* band_image = static_cast<float*>(__builtin_assume_aligned(band_image_base, 16));
    const uint64_t m = (n + 15) / 16;
    const uint64_t x0 = (uint64_t)blockIdx.x * bands_per_wg;
    const uint64_t x1 = (x0 + bands_per_wg < m) ? x0 + bands_per_wg : m;
    const uint64_t e0 = x0 * 16 * k;
    const uint64_t e1 = (x1 * 16 < n ? x1 * 16 : n) * k;
    const uint32_t n_words = (uint32_t)(x1 - x0) * k;  // at most kBandsBlock: one per lane
    float* oq = out + e0;
    // element li of the range lives at band_image[a + li]: quads that start on a 16-byte boundary of
    // `out` then start on one of the image
    const uint32_t a = (uint32_t)((reinterpret_cast<uintptr_t>(oq) >> 2) & 3u);
    const uint32_t w = threadIdx.x;
    if (w < n_words) {
        uint32_t b = 0, y = w;
        if (bands_per_wg > 1) band_row_col(w, k, inv, &b, &y);  // band within the range, column
        const uint32_t word = c[x0 * k + w];
        float* col = band_image + a + b * 16 * k + y;
        if constexpr (MIX) {
            const uint32_t tops = codes_to_half_tops(word);
#pragma unroll
            for (int s = 0; s < 8; ++s) {
                const f16x2 h = __builtin_bit_cast(f16x2, (tops << (14 - 2 * s)) & 0xC000C000u);
                col[s * k] = __builtin_fmaf((float)h.x, th, -0.0f);
                col[(s + 8) * k] = __builtin_fmaf((float)h.y, th, -0.0f);
            }
        } else {
#pragma unroll
            for (int s = 0; s < 16; ++s) col[s * k] = deq_code((word >> (2 * s)) & 3u, t);
        }
    }
    __syncthreads();
    band_image_out<NT>(band_image, oq, a, (uint32_t)(e1 - e0));
}

// Bands longer than that: no LDS and no barrier at all.  A band (16 rows of the matrix, 16 k contiguous
// floats, k code words) is cut on a grid of 4 KiB pieces that starts at the 128-byte line at or
// before the band: workgroup (band, piece) writes one piece, a wave 1 KiB of whole lines, a lane one
// quad, exactly like the flat decode.  The lane finds (row, column) of its quad by one multiply-high
// and fetches the four words of columns col .. col+3 with ONE 16-byte load at word alignment;
// neighbouring lanes read neighbouring 16 bytes, so a wave reads 1 KiB of contiguous words.  A quad
// that runs over the end of its row takes its last elements from the first words of the band (the
// next row's), which every lane loads from the same address; the four words are picked out of the
// seven without a branch.  Each word is read by the 16 waves that write its 16 rows: the workgroups
// of a band run on ONE XCD (workgroups go to the XCDs round-robin by id; bands are dealt to the XCDs
// in groups of 8), so it comes from memory once and from that XCD's L2 fifteen times (measured at 401
// columns: 0.83 of the HBM peak with the bands pinned, 0.70 in plain order).
// Measured against what it replaced (band kernels with the words staged in LDS up to 800 columns,
// tiles of 16 rows x 256 columns above): 0.83 against 0.68 at 401 columns, 0.88 / 0.70 at 201,
// 0.95 / 0.80 at 255, 0.79 / 0.65 at 799, 0.85 / 0.67 at 1001, 0.96 / 0.89 at 8191.
// For 97 to 8192 columns (the 32-bit multiply-high is exact while 17 k^2 + 1024 k < 2^32); wider matrices
// keep the tiles of 16 rows x 256 columns.
constexpr uint64_t kStreamMaxColumns = 8192;

template <bool NT>
__global__ __launch_bounds__(256) void deq_stream_kernel(
    float* out, const uint32_t* __restrict__ c, uint64_t n, uint32_t k, uint32_t pieces, uint64_t inv_pieces,
    uint32_t inv_k, float t, uint32_t pinned)
{
    // pinned: bands dealt to the XCDs in groups of 8; else plain order (a matrix of a few bands: all XCDs busy,
    // the words then come from the memory-side cache more than once)
    const uint32_t xcd = pinned ? blockIdx.x & 7u : 0u, j = pinned ? blockIdx.x >> 3 : blockIdx.x;
    const uint32_t jb = (uint32_t)__umul64hi((uint64_t)j, inv_pieces);  // j / pieces
    const uint32_t q = j - jb * pieces;                                 // piece within the band
    const uint64_t x = pinned ? (uint64_t)jb * 8 + xcd : (uint64_t)jb;  // band
    if (x * 16 >= n) return;  // padding workgroups of the last group of 8 bands
    const uint32_t rows = n - x * 16 < 16 ? (uint32_t)(n - x * 16) : 16u;
    const int32_t blen = (int32_t)(rows * k);
    float* ob = out + x * 16 * k;
    const uint32_t* cq = c + x * k;
    const int32_t d = (int32_t)((reinterpret_cast<uintptr_t>(ob) >> 2) & 31u);
    const int32_t li = 1024 * (int32_t)q - d + 4 * (int32_t)threadIdx.x;  // first element of the quad, within the band
    if (li + 4 <= 0 || li >= blen) return;
    // (row, col), counted from one row before the band so that a first quad that starts before it
    // needs no case of its own: its elements inside the band are "the next row's"
    const uint32_t v = (uint32_t)(li + (int32_t)k);
    const uint32_t row1 = __umulhi(v, inv_k);
    const uint32_t col = v - row1 * k;
    const uint32_t sh = 2 * row1 - 2;               // bit position of this row's codes (of no use for row1 = 0: never stored)
    const uint32_t nf = k - col;                    // elements of the quad that lie in this row (4 or more: all)
    const uint32_t col_a = nf >= 4 ? col : k - 4;   // the load stays inside the band's words
    const u32x4_a4 wa = *reinterpret_cast<const u32x4_a4*>(cq + col_a);
    const u32x4_a4 wb = *reinterpret_cast<const u32x4_a4*>(cq);
    const uint32_t first = nf >= 4 ? 0u : 4u - nf;  // the quad's words are v[first .. first + 3]
    const uint32_t sa = sh & 31u, sb = (sh + 2) & 31u;
    const uint32_t v0 = wa.x >> sa, v1 = wa.y >> sa, v2 = wa.z >> sa, v3 = wa.w >> sa;
    const uint32_t v4 = wb.x >> sb, v5 = wb.y >> sb, v6 = wb.z >> sb;
    const bool f1 = first & 1u, f2 = first & 2u;
    const uint32_t y0 = f1 ? v1 : v0, y1 = f1 ? v2 : v1, y2 = f1 ? v3 : v2, y3 = f1 ? v4 : v3, y4 = f1 ? v5 : v4,
                   y5 = f1 ? v6 : v5;
    f32x4 vo;
    vo.x = deq_code((f2 ? y2 : y0) & 3u, t);
    vo.y = deq_code((f2 ? y3 : y1) & 3u, t);
    vo.z = deq_code((f2 ? y4 : y2) & 3u, t);
    vo.w = deq_code((f2 ? y5 : y3) & 3u, t);
    if (li >= 0 && li + 4 <= blen) {
        st4<true, NT>(ob + li, vo);
    } else {
        const float o[4] = {vo.x, vo.y, vo.z, vo.w};
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (li + e >= 0 && li + e < blen) ob[li + e] = o[e];
    }
}

// ---------------------------------------------------------------- many vectors in one launch

// A model's gradients are many separate vectors (161 for ResNet-50, most of them small); one
// launch per vector costs more in launch latency than the data takes to stream.  These kernels
// take a table of up to kMaxSegments (96) vectors in their arguments and treat the chunks (or tiles)
// of all of them as one index space; a wave finds its vector in the table (find_segment).

constexpr int kMaxSegments = 96;  // 96 x 36 B of table stays under the 4 KiB kernel-argument limit

struct QuantSegments {
    const float* g[kMaxSegments];
    float* r[kMaxSegments];
    uint32_t* c[kMaxSegments];
    uint64_t n[kMaxSegments];
    uint32_t first[kMaxSegments + 1];  // first[s] = index of segment s's first chunk; first[count] = total
    int count;
};

// Largest s with first[s] <= q, for q < first[count]; the host fills first[count..96] with the total,
// so the answer is the number of entries first[1..96) that are <= q.  Counted in two rounds of
// independent scalar loads (7 pivots 12 entries apart, then the 11 entries behind the pivot) instead
// of the 7 dependent loads of a binary search: a wave starts its memory traffic that much earlier.
static_assert(kMaxSegments == 8 * 12, "find_segment splits the table into 8 blocks of 12");
__device__ __forceinline__ int find_segment(const uint32_t* first, uint32_t q)
{
    int block = 0;
#pragma unroll
    for (int p = 1; p < 8; ++p) block += first[12 * p] <= q ? 1 : 0;
    int s = 12 * block;
#pragma unroll
    for (int j = 1; j < 12; ++j) s += first[12 * block + j] <= q ? 1 : 0;
    return s;
}

template <bool ALIGNED, bool ADD, bool NT>
__global__ __launch_bounds__(256) void quant_multi_kernel(QuantSegments seg, uint32_t xs, float t)
{
    const int lane = threadIdx.x & (kWave - 1);
    const uint32_t w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint64_t q64 = chunk_of<1, 256>(blockIdx.x, w, 0, xs);
    if (q64 >= seg.first[seg.count]) return;
    const uint32_t q = (uint32_t)q64;
    const int sidx = find_segment(seg.first, q);
    const float* g = seg.g[sidx];
    float* r = seg.r[sidx];
    uint32_t* c = seg.c[sidx];
    const uint64_t n = seg.n[sidx];
    const uint64_t e0 = (uint64_t)(q - seg.first[sidx]) * kChunk;
    if (e0 + kChunk <= n) {
        const uint64_t e = e0 + lane * 4;
        f32x4 v = ld4<ALIGNED, NT>(g + e);
        if constexpr (ADD) v = v + ld4<ALIGNED, NT>(r + e);
        float o0, o1, o2, o3;
        uint32_t b = quant_one(v.x, t, o0);
        b |= quant_one(v.y, t, o1) << 2;
        b |= quant_one(v.z, t, o2) << 4;
        b |= quant_one(v.w, t, o3) << 6;
        f32x4 o;
        o.x = o0; o.y = o1; o.z = o2; o.w = o3;
        st4<ALIGNED, NT>(r + e, o);
        const uint32_t word = quad_or(b << (8 * (lane & 3)));
        if ((lane & 3) == 0) c[(e0 >> 4) + (lane >> 2)] = word;
    } else {
        // last, shorter chunk of the vector (rem = 1..255 elements): the same pass with the lanes past
        // the end idle and the quad the end cuts going element by element; codes past the end are 0
        const uint32_t rem = (uint32_t)(n - e0);
        const uint32_t le = (uint32_t)lane * 4;
        const float* gp = g + e0 + le;
        float* rp = r + e0 + le;
        uint32_t b = 0;
        if (le + 4 <= rem) {
            f32x4 v = ld4<ALIGNED, NT>(gp);
            if constexpr (ADD) v = v + ld4<ALIGNED, NT>(rp);
            float o0, o1, o2, o3;
            b = quant_one(v.x, t, o0);
            b |= quant_one(v.y, t, o1) << 2;
            b |= quant_one(v.z, t, o2) << 4;
            b |= quant_one(v.w, t, o3) << 6;
            f32x4 o;
            o.x = o0; o.y = o1; o.z = o2; o.w = o3;
            st4<ALIGNED, NT>(rp, o);
        } else if (le < rem) {
            for (uint32_t i = 0; i < rem - le; ++i) {
                float a = gp[i];
                if constexpr (ADD) a = a + rp[i];
                float res;
                b |= quant_one(a, t, res) << (2 * i);
                rp[i] = res;
            }
        }
        const uint32_t word = quad_or(b << (8 * (lane & 3)));
        if ((lane & 3) == 0 && le < rem) c[(e0 >> 4) + (lane >> 2)] = word;
    }
}

struct AccSegments {
    float* acc[kMaxSegments];
    uint64_t n[kMaxSegments];
    uint64_t word_offset[kMaxSegments];  // of the vector's first code word inside every payload
    uint32_t first[kMaxSegments + 1];    // in tiles of 1024 elements
    int count;
};

template <int K, bool ALIGNED, bool MIX>
__global__ __launch_bounds__(kAccBlock) void acc_multi_kernel(AccSegments seg, PayloadPtrs pl, int k_payloads,
                                                              uint32_t xs, float t, float th, int accumulate,
                                                              float divisor, float recip)
{
    __shared__ __attribute__((aligned(16))) float lds[kAccBlock / kWave][kAccLdsPerWave];
    const int lane = threadIdx.x & (kWave - 1);
    const uint32_t w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint64_t q64 = chunk_of<1, kAccBlock>(blockIdx.x, w, 0, xs);
    if (q64 >= seg.first[seg.count]) return;
    const uint32_t q = (uint32_t)q64;
    const int sidx = find_segment(seg.first, q);
    const uint64_t n = seg.n[sidx];
    const uint64_t e0 = (uint64_t)(q - seg.first[sidx]) * kTile;
    if (e0 + kTile > n) {
        // last, shorter tile of the vector
        acc_tile<K, ALIGNED, MIX, true>(seg.acc[sidx] + e0, pl, k_payloads, seg.word_offset[sidx] + (e0 >> 4), t,
                                        th, accumulate, divisor, recip, lds[w], lane, (uint32_t)(n - e0));
        return;
    }
    acc_tile<K, ALIGNED, MIX, false>(seg.acc[sidx] + e0, pl, k_payloads, seg.word_offset[sidx] + (e0 >> 4), t, th,
                                     accumulate, divisor, recip, lds[w], lane);
}

// ---------------------------------------------------------------- copy (measurement aid)

#if NKLQ_TUNING_BUILD
template <int U, int BLOCK, bool NT>
__global__ __launch_bounds__(BLOCK) void copy_kernel(float* dst, const float* src, uint64_t n,
                                                      uint64_t n_chunks, uint32_t has_tail,
                                                      uint32_t xs)
{
    if (has_tail && blockIdx.x == gridDim.x - 1) {
        for (uint64_t e = n_chunks * kChunk + threadIdx.x; e < n; e += BLOCK) dst[e] = src[e];
        return;
    }
    const int lane = threadIdx.x & (kWave - 1);
    const uint32_t w = threadIdx.x >> 6;
    uint64_t ch[U];
    f32x4 a[U];
#pragma unroll
    for (int j = 0; j < U; ++j) ch[j] = chunk_of<U, BLOCK>(blockIdx.x, w, j, xs);
#pragma unroll
    for (int j = 0; j < U; ++j)
        if (ch[j] < n_chunks) a[j] = ld4<true, NT>(src + ch[j] * kChunk + lane * 4);
#pragma unroll
    for (int j = 0; j < U; ++j)
        if (ch[j] < n_chunks) st4<true, NT>(dst + ch[j] * kChunk + lane * 4, a[j]);
}
#endif

// ---------------------------------------------------------------- host side

// Launch-geometry knobs (results never depend on them); defaults from a sweep on MI355X.  They
// are process-wide and may be changed by one host thread while others launch: every entry point
// takes one snapshot of them when it is called and uses only that.
struct Knobs {
    int chunks_per_wave;  // 1, 2 or 4
    int block;            // 64, 128, 256, 512 or 1024 threads
    int nontemporal;
    int xcd_shift;        // quantize/copy: chunks interleaved over 2^xcd_shift workgroups
    int xcd_shift_decode; // the same for dequantize (write-dominated: contiguous wins)
    int xcd_shift_acc;    // the same for the sum over payloads (tiles of 1024 elements over all 8 XCDs)
    int decode_prefetch;  // flat decode: 0 = prefetch the code words when they cannot all be in the memory-side cache, 1 = always, 2 = never
};
constexpr int kKnobCount = 7;
std::atomic<int> g_knobs[kKnobCount] = {{1}, {256}, {1}, {2}, {0}, {3}, {0}};

thread_local Knobs tk;  // the calling thread's snapshot, taken on entry to an entry point

inline void snapshot_knobs()
{
    tk.chunks_per_wave = g_knobs[NKLQ_TUNE_CHUNKS_PER_WAVE].load(std::memory_order_relaxed);
    tk.block = g_knobs[NKLQ_TUNE_WORKGROUP_SIZE].load(std::memory_order_relaxed);
    tk.nontemporal = g_knobs[NKLQ_TUNE_NONTEMPORAL].load(std::memory_order_relaxed);
    tk.xcd_shift = g_knobs[NKLQ_TUNE_XCD_INTERLEAVE_LOG2].load(std::memory_order_relaxed);
    tk.xcd_shift_decode = g_knobs[NKLQ_TUNE_XCD_INTERLEAVE_LOG2_DECODE].load(std::memory_order_relaxed);
    tk.xcd_shift_acc = g_knobs[NKLQ_TUNE_XCD_INTERLEAVE_LOG2_ACCUMULATE].load(std::memory_order_relaxed);
    tk.decode_prefetch = g_knobs[NKLQ_TUNE_DECODE_PREFETCH].load(std::memory_order_relaxed);
}

// ---- kernel launch with the launch's own status
//
// hipLaunchKernel returns what THIS launch did; the runtime's "last error" is left alone unless the
// launch failed (then it is cleared, since the failure is reported through the return value).
thread_local int t_launch_status = NKLQ_OK;

template <typename Tuple, size_t... I>
inline void arg_pointers(Tuple& vals, void** out, std::index_sequence<I...>)
{
    ((out[I] = static_cast<void*>(&std::get<I>(vals))), ...);
}

template <typename... KArgs, typename... Args>
inline void launch_kernel(void (*kernel)(KArgs...), dim3 grid, dim3 block, uint32_t lds_bytes, hipStream_t s,
                          Args... args)
{
    static_assert(sizeof...(KArgs) == sizeof...(Args), "kernel argument count");
    std::tuple<KArgs...> vals(static_cast<KArgs>(args)...);
    void* ptrs[sizeof...(KArgs)];
    arg_pointers(vals, ptrs, std::index_sequence_for<KArgs...>{});
    const hipError_t e = hipLaunchKernel(reinterpret_cast<const void*>(kernel), grid, block, ptrs, lds_bytes, s);
    if (e != hipSuccess) (void)hipGetLastError();
    t_launch_status = e == hipSuccess ? NKLQ_OK : (int)e;
}

inline int launch_status() { return t_launch_status; }

// ---- overlap checks
//
// Byte ranges of the buffers of a call.  An output may coincide EXACTLY with an input that is named
// as its in-place partner (r_out == r_in, r_out == g: each element is read and then written by the
// same lane); any other overlap that involves an output is refused, also an exact coincidence with
// an input that is not its partner (the code words on top of a one-row gradient, say).
struct Span {
    uintptr_t lo, hi;
    bool out;
    int tag;  // an output: its own id; an input: the id of the output it may coincide with, or -1
};

inline Span span_of(const void* p, uint64_t bytes, bool out, int tag = -1)
{
    const uintptr_t lo = reinterpret_cast<uintptr_t>(p);
    return Span{lo, lo + (uintptr_t)bytes, out, tag};
}

bool spans_conflict(std::vector<Span>& v)
{
    std::sort(v.begin(), v.end(), [](const Span& a, const Span& b) {
        if (a.lo != b.lo) return a.lo < b.lo;
        if (a.hi != b.hi) return a.hi < b.hi;
        return a.out > b.out;  // of identical ranges the output comes first
    });
    uintptr_t end_out = 0, end_any = 0;  // furthest end among the outputs / all ranges seen so far
    uintptr_t out_lo = 0, out_hi = 0;    // the latest output
    int out_tag = -1;
    for (size_t i = 0; i < v.size(); ++i) {
        if (v[i].lo == v[i].hi) continue;
        // inputs identical to the output sorted just before them, and named as its partner, are in place
        const bool partner = !v[i].out && out_hi != 0 && v[i].lo == out_lo && v[i].hi == out_hi &&
                             v[i].tag >= 0 && v[i].tag == out_tag;
        if (v[i].out) { out_lo = v[i].lo; out_hi = v[i].hi; out_tag = v[i].tag; }
        if (!partner) {
            if (v[i].out ? v[i].lo < end_any : v[i].lo < end_out) return true;
        }
        if (v[i].out && v[i].hi > end_out) end_out = v[i].hi;
        if (v[i].hi > end_any) end_any = v[i].hi;
    }
    return false;
}

// The overlap check of a many-vectors call sorts a few hundred ranges; its answer depends on the
// addresses and sizes alone.  A training loop passes the same tables step after step, so each host
// thread remembers the last set it has checked and found free of overlaps, and a call with exactly
// that set again (compared value by value, not by a hash) skips the sort.
struct CheckedTables {
    std::vector<uint64_t> seen;
    std::vector<uint64_t> now;
    void begin() { now.clear(); }
    void add(const void* table, size_t entries)
    {
        const uint64_t* p = static_cast<const uint64_t*>(table);  // tables of pointers or of uint64_t
        now.insert(now.end(), p, p + entries);
    }
    void add(uint64_t v) { now.push_back(v); }
    bool known() const { return now == seen; }
    void remember() { seen.swap(now); }
};
static_assert(sizeof(void*) == sizeof(uint64_t), "pointer tables are compared as 64-bit words");

struct FlatGrid {
    uint64_t n_chunks;
    uint32_t has_tail;
    uint32_t blocks;  // 0: the vector is too long for one launch
    uint32_t xs;
};

// Work split of a flat vector of n elements for workgroups of `block` threads, U chunks per wave.
FlatGrid flat_grid(uint64_t n, int U, int block, int xcd_shift)
{
    FlatGrid fg;
    fg.xs = (uint32_t)xcd_shift;
    fg.n_chunks = n / kChunk;
    fg.has_tail = (fg.n_chunks * kChunk < n) ? 1u : 0u;
    const uint64_t per_group = ((uint64_t)(block / kWave) * (uint64_t)U) << fg.xs;
    const uint64_t work = ((fg.n_chunks + per_group - 1) / per_group) << fg.xs;
    fg.blocks = (work + fg.has_tail > 0x7FFFFFFFull) ? 0u : (uint32_t)work + fg.has_tail;
    return fg;
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline bool aligned4(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 3u) == 0; }

// ---- flat quantize dispatch: (U, BLOCK) -> (ALIGNED, ADD, NT)

template <int U, int BLOCK>
int launch_quant_flat(const float* g, const float* rin, float* rout, uint32_t* c, uint64_t n, float t,
                      bool add, bool al, hipStream_t s)
{
    const FlatGrid fg = flat_grid(n, U, BLOCK, tk.xcd_shift);
    if (fg.blocks == 0) return NKLQ_ERANGE;
    const bool nt = tk.nontemporal != 0;
#define NKLQ_Q(AL, ADD, NT)                                                                       \
    launch_kernel((quant_flat_kernel<U, BLOCK, AL, ADD, NKLQ_NT(NT)>), dim3(fg.blocks), dim3(BLOCK), 0, \
                       s, g, rin, rout, c, n, fg.n_chunks, fg.has_tail, fg.xs, t)
    const int sel = (al ? 4 : 0) | (add ? 2 : 0) | (nt ? 1 : 0);
    switch (sel) {
        case 7: NKLQ_Q(true, true, true); break;
        case 6: NKLQ_Q(true, true, false); break;
        case 5: NKLQ_Q(true, false, true); break;
        case 4: NKLQ_Q(true, false, false); break;
        case 3: NKLQ_Q(false, true, true); break;
        case 2: NKLQ_Q(false, true, false); break;
        case 1: NKLQ_Q(false, false, true); break;
        default: NKLQ_Q(false, false, false); break;
    }
#undef NKLQ_Q
    return launch_status();
}

constexpr uint32_t kPrefetchLead = 16;                     // blocks of kPrefetchBlock workgroups (16 MiB of output) ahead
constexpr uint64_t kPrefetchFromElements = 1ull << 30;     // 256 MiB of code words

template <int U, int BLOCK>
int launch_deq_flat(float* out, const uint32_t* c, uint64_t n, float t, hipStream_t s)
{
    FlatGrid fg = flat_grid(n, U, BLOCK, tk.xcd_shift_decode);
    if (fg.blocks == 0) return NKLQ_ERANGE;
    // Prefetch workgroups (see the kernel) when the code words cannot all be in the 256 MB memory-side cache
    // (from 2^30 elements: 1.0e9 elements still decode at 0.94 of the HBM peak without, 1.1e9 at 0.77, 1.4e9 at
    // 0.61), or when the caller says they are not there; never for vectors of a few blocks
    uint32_t pf_lead = 0;
    const uint64_t work = fg.blocks - fg.has_tail;
    const bool wanted = tk.decode_prefetch == 1 || (tk.decode_prefetch == 0 && n >= kPrefetchFromElements);
    if (wanted && fg.xs == 0 && work >= 2 * kPrefetchLead * kPrefetchBlock) {
        const uint64_t with = (work + kPrefetchBlock - 1) / kPrefetchBlock * (kPrefetchBlock + 8) + fg.has_tail;
        if (with <= 0x7FFFFFFFull) {
            fg.blocks = (uint32_t)with;
            pf_lead = kPrefetchLead;
        }
    }
    if (tk.nontemporal)
        launch_kernel((deq_flat_kernel<U, BLOCK, true>), dim3(fg.blocks), dim3(BLOCK), 0, s, out, c, n,
                      fg.n_chunks, fg.has_tail, fg.xs, t, pf_lead);
    else
        launch_kernel((deq_flat_kernel<U, BLOCK, NKLQ_NT(false)>), dim3(fg.blocks), dim3(BLOCK), 0, s, out, c, n,
                      fg.n_chunks, fg.has_tail, fg.xs, t, pf_lead);
    return launch_status();
}

// The fast form of the sum needs 0 * t = +0, an exact t/2 and exact products: finite t >= +0 with
// a biased exponent of at least 2 (or t = +0).
inline bool mix_ok(float t)
{
    const uint32_t b = __builtin_bit_cast(uint32_t, t);
    const uint32_t ex = (b >> 23) & 0xFFu;
    return (b >> 31) == 0 && ex != 0xFFu && (ex >= 2 || b == 0);
}

// 1 / d when d is a power of two (other than 1) whose reciprocal is a normal number: then x * (1/d)
// and x / d are the same real number and round to the same bits.  Else 0.
inline float exact_reciprocal(float d)
{
    const uint32_t b = __builtin_bit_cast(uint32_t, d);
    const uint32_t ex = (b >> 23) & 0xFFu;
    if ((b & 0x007FFFFFu) != 0 || ex < 1 || ex > 253 || d == 1.0f) return 0.0f;
    return __builtin_bit_cast(float, (b & 0x80000000u) | ((254u - ex) << 23));
}

// Instantiates BODY(K, AL, MIX) for the payload count k: K = k up to 8 (unrolled), else K = 0 (the
// runtime-count form); the plain (non-MIX) form only exists with K = 0.
#define NKLQ_ACC_DISPATCH(BODY, k, al, mix)                                          \
    do {                                                                             \
        if (!(mix)) {                                                                \
            if (al) BODY(0, true, false); else BODY(0, false, false);                \
        } else {                                                                     \
            switch ((k) <= 8 ? (k) : 0) {                                            \
                case 1: if (al) BODY(1, true, true); else BODY(1, false, true); break; \
                case 2: if (al) BODY(2, true, true); else BODY(2, false, true); break; \
                case 3: if (al) BODY(3, true, true); else BODY(3, false, true); break; \
                case 4: if (al) BODY(4, true, true); else BODY(4, false, true); break; \
                case 5: if (al) BODY(5, true, true); else BODY(5, false, true); break; \
                case 6: if (al) BODY(6, true, true); else BODY(6, false, true); break; \
                case 7: if (al) BODY(7, true, true); else BODY(7, false, true); break; \
                case 8: if (al) BODY(8, true, true); else BODY(8, false, true); break; \
                default: if (al) BODY(0, true, true); else BODY(0, false, true); break; \
            }                                                                        \
        }                                                                            \
    } while (0)

// The accumulate kernels work on tiles of 1024 elements, one per wave, 256-thread workgroups.
int launch_acc_flat(float* acc, const PayloadPtrs& pl, int k, uint64_t n, float t, int accumulate,
                    hipStream_t s)
{
    const uint64_t n_tiles = n / kTile;
    const uint32_t has_tail = (n_tiles * kTile < n) ? 1u : 0u;
    const uint32_t xs = (uint32_t)tk.xcd_shift_acc;
    const uint64_t per_group = (uint64_t)(kAccBlock / kWave) << xs;
    const uint64_t work = ((n_tiles + per_group - 1) / per_group) << xs;
    if (work + has_tail > 0x7FFFFFFFull) return NKLQ_ERANGE;
    const uint32_t blocks = (uint32_t)work + has_tail;
    const bool al = aligned16(acc);
    const bool mix = mix_ok(t);
    const float th = -0.5f * t;
    const uint32_t pad = n_tiles >= kAccThrottleTiles ? kAccThrottleLdsBytes : 0u;
#define NKLQ_ACC(K, AL, MIX)                                                                        \
    launch_kernel((acc_flat_kernel<K, AL, MIX>), dim3(blocks), dim3(kAccBlock), pad, s, acc, pl, k, n, \
                       n_tiles, has_tail, xs, t, th, accumulate, 0u)
    NKLQ_ACC_DISPATCH(NKLQ_ACC, k, al, mix);
#undef NKLQ_ACC
    return launch_status();
}

// Expands to the call of FN<U, BLOCK, ...> for the current knob values.
#if NKLQ_TUNING_BUILD
#define NKLQ_FOR_GEOMETRY(CALL)                                  \
    switch (tk.chunks_per_wave * 10000 + tk.block) {               \
        case 10064: return CALL(1, 64);                          \
        case 10128: return CALL(1, 128);                         \
        case 10256: return CALL(1, 256);                         \
        case 10512: return CALL(1, 512);                         \
        case 11024: return CALL(1, 1024);                        \
        case 20064: return CALL(2, 64);                          \
        case 20128: return CALL(2, 128);                         \
        case 20256: return CALL(2, 256);                         \
        case 20512: return CALL(2, 512);                         \
        case 21024: return CALL(2, 1024);                        \
        case 40064: return CALL(4, 64);                          \
        case 40128: return CALL(4, 128);                         \
        case 40256: return CALL(4, 256);                         \
        case 40512: return CALL(4, 512);                         \
        case 41024: return CALL(4, 1024);                        \
        default: return NKLQ_ERANGE;                             \
    }
#else
#define NKLQ_FOR_GEOMETRY(CALL) return CALL(1, 256);
#endif

// Residual views that do not start on a 128-byte line take the kernel that keeps shared lines whole.
int launch_quant_flat_offline(const float* g, const float* rin, float* rout, uint32_t* c, uint64_t n, float t,
                              bool add, bool al, hipStream_t s)
{
    const uint64_t n_chunks = n / kChunk;
    const uint32_t has_tail = (n_chunks * kChunk < n) ? 1u : 0u;
    const uint64_t runs8 = ((n_chunks + kRunChunks - 1) / kRunChunks + 7) / 8 * 8;  // runs, in groups of 8 XCDs
    const uint64_t work = runs8 * (kRunChunks / 4);
    if (work + has_tail > 0x7FFFFFFFull) return NKLQ_ERANGE;
    const dim3 grid((uint32_t)work + has_tail), block(256);
    const bool nt = tk.nontemporal != 0;
#define NKLQ_QO(AL, ADD, NT) \
    launch_kernel((quant_flat_offline_kernel<AL, ADD, NKLQ_NT(NT)>), grid, block, 0, s, g, rin, rout, c, n, n_chunks, has_tail, t)
    switch ((al ? 4 : 0) | (add ? 2 : 0) | (nt ? 1 : 0)) {
        case 7: NKLQ_QO(true, true, true); break;
        case 6: NKLQ_QO(true, true, false); break;
        case 5: NKLQ_QO(true, false, true); break;
        case 4: NKLQ_QO(true, false, false); break;
        case 3: NKLQ_QO(false, true, true); break;
        case 2: NKLQ_QO(false, true, false); break;
        case 1: NKLQ_QO(false, false, true); break;
        default: NKLQ_QO(false, false, false); break;
    }
#undef NKLQ_QO
    return launch_status();
}

int dispatch_quant_flat(const float* g, const float* rin, float* rout, uint32_t* c, uint64_t n,
                        float t, bool add, bool al, hipStream_t s)
{
    if ((reinterpret_cast<uintptr_t>(rout) & 127u) != 0 && n >= kChunk)
        return launch_quant_flat_offline(g, rin, rout, c, n, t, add, al, s);
#define NKLQ_CALL(U, B) launch_quant_flat<U, B>(g, rin, rout, c, n, t, add, al, s)
    NKLQ_FOR_GEOMETRY(NKLQ_CALL)
#undef NKLQ_CALL
}

int dispatch_deq_flat(float* out, const uint32_t* c, uint64_t n, float t, hipStream_t s)
{
    const uint32_t d = (uint32_t)((reinterpret_cast<uintptr_t>(out) >> 2) & 31u);  // elements past a 128-byte line
    if (d != 0) {
        const uint64_t n_chunks = (n + d + kChunk - 1) / kChunk;
        const uint64_t blocks = (n_chunks + 3) / 4;
        if (blocks > 0x7FFFFFFFull) return NKLQ_ERANGE;
        if (tk.nontemporal)
            launch_kernel((deq_flat_shift_kernel<true>), dim3((uint32_t)blocks), dim3(256), 0, s, out, c, n, n_chunks, d, t);
        else
            launch_kernel((deq_flat_shift_kernel<NKLQ_NT(false)>), dim3((uint32_t)blocks), dim3(256), 0, s, out, c, n, n_chunks, d, t);
        return launch_status();
    }
#define NKLQ_CALL(U, B) launch_deq_flat<U, B>(out, c, n, t, s)
    NKLQ_FOR_GEOMETRY(NKLQ_CALL)
#undef NKLQ_CALL
}

#if NKLQ_TUNING_BUILD
template <int U, int BLOCK>
int launch_copy(float* dst, const float* src, uint64_t n, hipStream_t s)
{
    const FlatGrid fg = flat_grid(n, U, BLOCK, tk.xcd_shift);
    if (fg.blocks == 0) return NKLQ_ERANGE;
    if (tk.nontemporal)
        launch_kernel((copy_kernel<U, BLOCK, true>), dim3(fg.blocks), dim3(BLOCK), 0, s, dst, src,
                           n, fg.n_chunks, fg.has_tail, fg.xs);
    else
        launch_kernel((copy_kernel<U, BLOCK, false>), dim3(fg.blocks), dim3(BLOCK), 0, s, dst,
                           src, n, fg.n_chunks, fg.has_tail, fg.xs);
    return launch_status();
}

int dispatch_copy(float* dst, const float* src, uint64_t n, hipStream_t s)
{
#define NKLQ_CALL(U, B) launch_copy<U, B>(dst, src, n, s)
    NKLQ_FOR_GEOMETRY(NKLQ_CALL)
#undef NKLQ_CALL
}
#endif

// Workgroups for `total` wave items (chunks or tiles), 4 waves per workgroup, dealt over 2^xs.
bool multi_grid(uint64_t total, uint32_t xs, uint32_t* blocks)
{
    const uint64_t per_group = (uint64_t)4 << xs;
    const uint64_t work = ((total + per_group - 1) / per_group) << xs;
    if (work > 0x7FFFFFFFull) return false;
    *blocks = (uint32_t)work;
    return true;
}

int launch_quant_multi(const QuantSegments& seg, bool al, bool add, float t, hipStream_t s)
{
    uint32_t blocks;
    const uint32_t xs = (uint32_t)tk.xcd_shift;
    if (!multi_grid(seg.first[seg.count], xs, &blocks)) return NKLQ_ERANGE;
    if (blocks == 0) return NKLQ_OK;
    const bool nt = tk.nontemporal != 0;
#define NKLQ_QM(AL, ADD, NT) \
    launch_kernel((quant_multi_kernel<AL, ADD, NKLQ_NT(NT)>), dim3(blocks), dim3(256), 0, s, seg, xs, t)
    switch ((al ? 4 : 0) | (add ? 2 : 0) | (nt ? 1 : 0)) {
        case 7: NKLQ_QM(true, true, true); break;
        case 6: NKLQ_QM(true, true, false); break;
        case 5: NKLQ_QM(true, false, true); break;
        case 4: NKLQ_QM(true, false, false); break;
        case 3: NKLQ_QM(false, true, true); break;
        case 2: NKLQ_QM(false, true, false); break;
        case 1: NKLQ_QM(false, false, true); break;
        default: NKLQ_QM(false, false, false); break;
    }
#undef NKLQ_QM
    return launch_status();
}

int launch_acc_multi(const AccSegments& seg, const PayloadPtrs& pl, int k, bool al, float t,
                     int accumulate, float divisor, hipStream_t s)
{
    uint32_t blocks;
    const uint32_t xs = (uint32_t)tk.xcd_shift_acc;
    if (!multi_grid(seg.first[seg.count], xs, &blocks)) return NKLQ_ERANGE;
    if (blocks == 0) return NKLQ_OK;
    const bool mix = mix_ok(t);
    const float th = -0.5f * t;
    const uint32_t pad = seg.first[seg.count] >= kAccThrottleTiles ? kAccThrottleLdsBytes : 0u;
    const float recip = exact_reciprocal(divisor);
#define NKLQ_AM(K, AL, MIX)                                                                           \
    launch_kernel((acc_multi_kernel<K, AL, MIX>), dim3(blocks), dim3(kAccBlock), pad, s, seg, pl, k, xs, \
                       t, th, accumulate, divisor, recip)
    NKLQ_ACC_DISPATCH(NKLQ_AM, k, al, mix);
#undef NKLQ_AM
    return launch_status();
}

// Bands per workgroup of the band kernels, and the launch's workgroup count (0: out of range).
uint32_t bands_grid(uint64_t n_rows, uint64_t n_cols, uint64_t range, bool runs, uint32_t* bands_per_wg)
{
    const uint64_t m = n_rows / 16 + (n_rows % 16 ? 1 : 0);
    const uint64_t per = range / (16 * n_cols);
    *bands_per_wg = (uint32_t)(per ? per : 1);
    const uint64_t ranges = (m + *bands_per_wg - 1) / *bands_per_wg;
    const uint64_t blocks = runs ? (ranges + 8 * kBandRun - 1) / (8 * kBandRun) * (8 * kBandRun) : ranges;  // whole groups of runs
    return blocks > 0x7FFFFFFFull ? 0u : (uint32_t)blocks;
}

// n_rows * n_cols with overflow check
bool mul_ok(uint64_t a, uint64_t b, uint64_t* out)
{
    if (a != 0 && b > UINT64_MAX / a) return false;
    *out = a * b;
    return true;
}

// One word of every 128-byte line of `words` code words is read (and dropped): the lines are then in
// the memory-side cache for the decode that follows on the same stream.
__global__ __launch_bounds__(256) void touch_words_kernel(const uint32_t* __restrict__ c, uint64_t words)
{
    const uint64_t wi = ((uint64_t)blockIdx.x * 256 + threadIdx.x) * 32;
    if (wi < words) {
        const uint32_t bits = c[wi];
        asm volatile("" : : "v"(bits));
    }
}
constexpr uint64_t kTouchRangeWords = 1ull << 24;      // 64 MiB of code words per range: a quarter of the memory-side cache
constexpr uint64_t kTouchFromElements = 1ull << 24;    // smaller matrices are decoded as they are

int decode_matrix(float* out, const uint32_t* c, uint64_t n_rows, uint64_t n_cols, float thrd, hipStream_t s);

}  // namespace

// ---------------------------------------------------------------- C-ABI

extern "C" {

int nklq_version(void) { return NKLQ_VERSION; }

uint64_t nklq_packed_words(uint64_t n_rows, uint64_t n_cols)
{
    return (n_rows / 16 + (n_rows % 16 ? 1 : 0)) * n_cols;
}

const char* nklq_strerror(int code)
{
    switch (code) {
        case NKLQ_OK: return "success";
        case NKLQ_ENULL: return "nklq: a required pointer is NULL";
        case NKLQ_EALIGN: return "nklq: a pointer is not 4-byte aligned";
        case NKLQ_ERANGE: return "nklq: a size or count is out of range";
        case NKLQ_EALIAS: return "nklq: output buffers overlap";
        default: break;
    }
    if (code > 0) return hipGetErrorString((hipError_t)code);
    return "nklq: unknown error";
}

int nklq_tune(int which, int value)
{
    if (which < 0 || which >= kKnobCount) return NKLQ_ERANGE;
    if (value < 0) return g_knobs[which].load(std::memory_order_relaxed);
    switch (which) {
#if NKLQ_TUNING_BUILD
        case NKLQ_TUNE_CHUNKS_PER_WAVE:
            if (value != 1 && value != 2 && value != 4) return NKLQ_ERANGE;
            break;
        case NKLQ_TUNE_WORKGROUP_SIZE:
            if (value != 64 && value != 128 && value != 256 && value != 512 && value != 1024)
                return NKLQ_ERANGE;
            break;
        case NKLQ_TUNE_NONTEMPORAL:
            value = value ? 1 : 0;
            break;
#else
        // the product library carries one form of each: only that value is accepted
        case NKLQ_TUNE_CHUNKS_PER_WAVE:
            if (value != 1) return NKLQ_ERANGE;
            break;
        case NKLQ_TUNE_WORKGROUP_SIZE:
            if (value != 256) return NKLQ_ERANGE;
            break;
        case NKLQ_TUNE_NONTEMPORAL:
            if (value != 1) return NKLQ_ERANGE;
            break;
#endif
        case NKLQ_TUNE_DECODE_PREFETCH:
            if (value > 2) return NKLQ_ERANGE;
            break;
        default:
            if (value > 6) return NKLQ_ERANGE;
            break;
    }
    return g_knobs[which].exchange(value, std::memory_order_relaxed);
}

int nklq_quantize_f32(const float* g, const float* r_in, float* r_out, uint32_t* c,
                      uint64_t n_rows, uint64_t n_cols, float thrd, int add_residual, void* stream)
{
    uint64_t total;
    if (!mul_ok(n_rows, n_cols, &total)) return NKLQ_ERANGE;
    if (total == 0) return NKLQ_OK;
    if (!g || !r_out || !c || (add_residual && !r_in)) return NKLQ_ENULL;
    if (!aligned4(g) || !aligned4(r_out) || !aligned4(c) || (add_residual && !aligned4(r_in)))
        return NKLQ_EALIGN;
    const bool add = add_residual != 0;
    {
        std::vector<Span> spans = {span_of(r_out, 4 * total, true, 0),
                                   span_of(c, 4 * nklq_packed_words(n_rows, n_cols), true, 1),
                                   span_of(g, 4 * total, false, 0)};
        if (add) spans.push_back(span_of(r_in, 4 * total, false, 0));
        if (spans_conflict(spans)) return NKLQ_EALIAS;
    }
    snapshot_knobs();
    hipStream_t s = (hipStream_t)stream;
    if (!add) r_in = g;  // never read; keeps the argument a valid address

    if (n_cols == 1) {
        const bool al = aligned16(g) && aligned16(r_out) && (!add || aligned16(r_in));
        return dispatch_quant_flat(g, r_in, r_out, c, total, thrd, add, al, s);
    }
    const uint64_t m = n_rows / 16 + (n_rows % 16 ? 1 : 0);
    if (n_cols <= kBandsMaxColumns) {
        uint32_t per;
        const uint32_t grid = bands_grid(n_rows, n_cols, kBandsRangeQuant, true, &per);
        if (grid == 0) return NKLQ_ERANGE;
        const uint32_t k32 = (uint32_t)n_cols;
        const uint32_t inv = (uint32_t)(0x100000000ull / k32) + 1u;
        // quads are laid out from a 16-byte boundary of r_out; g and r_in load as aligned vectors when
        // they sit at the same offset from one
        const uintptr_t ph = reinterpret_cast<uintptr_t>(r_out) & 15u;
        const bool same = (reinterpret_cast<uintptr_t>(g) & 15u) == ph &&
                          (!add || (reinterpret_cast<uintptr_t>(r_in) & 15u) == ph);
#define NKLQ_QB(ADD, NT, AL)                                                                          \
    launch_kernel((quant_bands_kernel<ADD, NKLQ_NT(NT), AL>), dim3(grid), dim3(kBandsBlock), 0, s, g, r_in, r_out, \
                       c, n_rows, k32, per, inv, thrd)
        switch ((add ? 4 : 0) | (tk.nontemporal ? 2 : 0) | (same ? 1 : 0)) {
            case 7: NKLQ_QB(true, true, true); break;
            case 6: NKLQ_QB(true, true, false); break;
            case 5: NKLQ_QB(true, false, true); break;
            case 4: NKLQ_QB(true, false, false); break;
            case 3: NKLQ_QB(false, true, true); break;
            case 2: NKLQ_QB(false, true, false); break;
            case 1: NKLQ_QB(false, false, true); break;
            default: NKLQ_QB(false, false, false); break;
        }
#undef NKLQ_QB
        return launch_status();
    }
    // tiles of 16 rows x 128 columns; which form (see quant_tiles_kernel):
    const bool on_lines = (n_cols % 32 == 0) && (reinterpret_cast<uintptr_t>(r_out) & 127u) == 0;
    const uintptr_t o_lo = reinterpret_cast<uintptr_t>(r_out), o_hi = o_lo + 4 * total;
    const auto clear_of = [&](const float* p) {
        const uintptr_t lo = reinterpret_cast<uintptr_t>(p);
        return lo + 4 * total <= o_lo || o_hi <= lo;
    };
    // r_out aliases no input, and rows long enough for the re-read right fringe (up to 31 elements per tile and
    // row) to pay: 16384 x 16383 537 -> 514 us, 8191 x 8191 132 -> 128 us, but 100000 x 1000 188 -> 191 us and
    // 150000 x 401 125 -> 170 us
    const bool shift = !on_lines && n_cols >= 4096 && clear_of(g) && (!add || clear_of(r_in));
    // tile width: 128 columns; 256 for matrices of a few bands and when tiles share lines and rows are long: from
    // 4096 columns, and from 1000 when rows do not even start on 16-byte boundaries (every quad of 3 rows in 4 is
    // then split over two 16-byte pieces: 60000 x 1023 0.68 -> 0.74, 30000 x 2047 0.75 -> 0.78; below 1000
    // columns the narrow tile stays ahead, 120000 x 513 0.73 against 0.67)
    const bool few_bands = m < 32;
    const bool long_rows = n_cols >= 4096 || (n_cols % 4 != 0 && n_cols >= 1000);
    uint64_t tile_cols = few_bands || (!on_lines && !shift && long_rows) ? 256 : 128;
    TileMap tm = {};
    const uint64_t col_tiles = ((shift ? n_cols + 31 : n_cols) + tile_cols - 1) / tile_cols;
    if (col_tiles > 0x7FFFFFFFull) return NKLQ_ERANGE;
    tm.col_tiles = (uint32_t)col_tiles;
    tm.inv_tiles = col_tiles > 1 ? ~0ull / col_tiles + 1 : 0;  // floor(2^64 / col_tiles) + 1; with one tile per band it is not used
    // Plain order when no line is shared between tiles, and (with short runs per XCD, see TileMap) for a few
    // bands: there pinning leaves XCDs idle or with a short band (100 x 1,000,003 in place 0.61 of the HBM peak in
    // plain order, 0.56-0.58 pinned with the bands cut into segments, 0.70 with runs of 4; the tile width, 128 to
    // 1024 columns, made no difference)
    tm.pinned = on_lines || few_bands ? 0u : 1u;
    uint64_t blocks;
    if (!tm.pinned) {
        blocks = m * col_tiles;
        if (!on_lines) {  // (a few bands, rows off lines)
            tm.run_shift = 2;
            tm.full_blocks = (uint32_t)((blocks >> (3 + tm.run_shift) << (3 + tm.run_shift)) & 0x7FFFFFFFull);
        }
    } else {
        const uint64_t full = (m / 8) * 8 * col_tiles;
        tm.last_bands = (uint32_t)(m % 8);
        tm.last_first = (m / 8) * 8;
        blocks = full;
        if (tm.last_bands) {
            // 1 band -> 8 segments, 2 -> 4, 3 or 4 -> 2, more -> 1
            tm.seg_shift = tm.last_bands == 1 ? 3u : (tm.last_bands == 2 ? 2u : (tm.last_bands <= 4 ? 1u : 0u));
            tm.seg_tiles = (uint32_t)((col_tiles + (1u << tm.seg_shift) - 1) >> tm.seg_shift);
            blocks += 8ull * tm.seg_tiles;
        }
        if (full > 0x7FFFFFFFull) return NKLQ_ERANGE;
        tm.full_blocks = (uint32_t)full;
    }
    if (blocks > 0x7FFFFFFFull) return NKLQ_ERANGE;
    const dim3 grid((uint32_t)blocks);
#define NKLQ_QT(W, Q, ADD, NT, SHIFT)                                                                      \
    launch_kernel((quant_tiles_kernel<W, Q, ADD, NKLQ_NT(NT), SHIFT>), grid, dim3(4 * W / Q), 0, s, g, r_in, r_out, c, \
                  n_rows, n_cols, tm, thrd)
#define NKLQ_QT_W(ADD, NT, SHIFT)                                  \
    do {                                                           \
        if (tile_cols == 128) NKLQ_QT(128, 1, ADD, NT, SHIFT);     \
        else NKLQ_QT(256, 1, ADD, NT, SHIFT);                      \
    } while (0)
#define NKLQ_QT_FORM(ADD, NT)                  \
    do {                                       \
        if (shift) NKLQ_QT_W(ADD, NT, true);   \
        else NKLQ_QT_W(ADD, NT, false);        \
    } while (0)
    switch ((add ? 2 : 0) | (tk.nontemporal ? 1 : 0)) {
        case 3: NKLQ_QT_FORM(true, true); break;
        case 2: NKLQ_QT_FORM(true, false); break;
        case 1: NKLQ_QT_FORM(false, true); break;
        default: NKLQ_QT_FORM(false, false); break;
    }
#undef NKLQ_QT_FORM
#undef NKLQ_QT_W
#undef NKLQ_QT
    return launch_status();
}

int nklq_dequantize_f32(float* out, const uint32_t* c, uint64_t n_rows, uint64_t n_cols, float thrd,
                        void* stream)
{
    uint64_t total;
    if (!mul_ok(n_rows, n_cols, &total)) return NKLQ_ERANGE;
    if (total == 0) return NKLQ_OK;
    if (!out || !c) return NKLQ_ENULL;
    if (!aligned4(out) || !aligned4(c)) return NKLQ_EALIGN;
    {
        std::vector<Span> spans = {span_of(out, 4 * total, true, 0),
                                   span_of(c, 4 * nklq_packed_words(n_rows, n_cols), false)};
        if (spans_conflict(spans)) return NKLQ_EALIAS;
    }
    snapshot_knobs();
    hipStream_t s = (hipStream_t)stream;
    if (n_cols == 1) {
        return dispatch_deq_flat(out, c, total, thrd, s);
    }
    // The matrix decodes are as sensitive to where their code words come from as the flat one (see
    // deq_flat_kernel): 16384 x 16383 runs at 0.92 of the HBM peak with the words in the memory-side cache and
    // at 0.58 with the words in HBM.  When they cannot all be in that cache, or the caller says they are not, the
    // matrix is decoded in ranges of bands of at most 64 MiB of words, each right after a pass that reads one
    // word of every line of the range's words (touch_words_kernel): that pass costs the words' share of the bytes.
    const bool touch = tk.decode_prefetch == 1 || (tk.decode_prefetch == 0 && total >= kPrefetchFromElements);
    if (touch && total >= kTouchFromElements) {
        uint64_t bands = kTouchRangeWords / n_cols / 8 * 8;   // whole groups of 8 bands (the tile maps deal bands in eights)
        if (bands < 8) bands = 8;
        const uint64_t rows = bands * 16;
        for (uint64_t r0 = 0; r0 < n_rows; r0 += rows) {
            const uint64_t nr = n_rows - r0 < rows ? n_rows - r0 : rows;
            const uint32_t* cr = c + (r0 / 16) * n_cols;
            const uint64_t words = nklq_packed_words(nr, n_cols);
            const uint64_t lines = (words + 31) / 32;
            const uint64_t tb = (lines + 255) / 256;
            if (tb > 0x7FFFFFFFull) return NKLQ_ERANGE;
            launch_kernel(touch_words_kernel, dim3((uint32_t)tb), dim3(256), 0, s, cr, words);
            if (launch_status() != NKLQ_OK) return launch_status();
            const int st = decode_matrix(out + r0 * n_cols, cr, nr, n_cols, thrd, s);
            if (st != NKLQ_OK) return st;
        }
        return NKLQ_OK;
    }
    return decode_matrix(out, c, n_rows, n_cols, thrd, s);
}

}  // extern "C"

namespace {

int decode_matrix(float* out, const uint32_t* c, uint64_t n_rows, uint64_t n_cols, float thrd, hipStream_t s)
{
    const uint64_t m = n_rows / 16 + (n_rows % 16 ? 1 : 0);
    if (16 * n_cols <= kBandsDecodeWholeMax) {
        // short bands: the fewest whole bands that give every lane of the workgroup a quad
        const uint32_t k32 = (uint32_t)n_cols;
        const bool mix = mix_ok(thrd);
        const float th = -0.5f * thrd;
        const uint32_t inv = (uint32_t)(0x100000000ull / k32) + 1u;
        const uint32_t per = (uint32_t)((kBandsDecodeElems + 16 * n_cols - 1) / (16 * n_cols));
        const uint64_t blocks = (m + per - 1) / per;
        if (blocks > 0x7FFFFFFFull) return NKLQ_ERANGE;
        const uint32_t lds = 4u * (4u + 16u * per * k32);
#define NKLQ_DB(NT, MIX)                                                                                      \
    launch_kernel((deq_bands_kernel<NKLQ_NT(NT), MIX>), dim3((uint32_t)blocks), dim3(kBandsBlock), lds, s, out, c, n_rows, \
                  k32, per, inv, thrd, th)
        if (tk.nontemporal && mix) NKLQ_DB(true, true);
        else if (tk.nontemporal) NKLQ_DB(true, false);
        else if (mix) NKLQ_DB(false, true);
        else NKLQ_DB(false, false);
#undef NKLQ_DB
        return launch_status();
    }
    // Tiles of 16 rows x 256 columns for more than 8192 columns (0.93 of the HBM peak against 0.86 for the band
    // stream at 16384 x 16383) and from 4096 columns when every row starts on a 128-byte line (0.89 against 0.85
    // at 8192 x 8192 in one process; the band stream is ahead at 1024 and 2048 columns, and at 8191: 0.96 / 0.89)
    const bool plain = (n_cols % 32 == 0) && (reinterpret_cast<uintptr_t>(out) & 127u) == 0 && aligned16(c);
    if (n_cols > kStreamMaxColumns || (n_cols >= 4096 && plain)) {
        const uint64_t col_tiles = ((plain ? n_cols : n_cols + 31) + 255) / 256;
        // No line is shared between tiles here and a tile's words are read by its own 16 waves: bands
        // need not stay on one XCD.  They are still dealt to the XCDs in groups of 8 when there are many
        // (each XCD sweeps one band: 0.93 against 0.91 at 16384 x 16383), in plain order when there are
        // few (a 16 x 4,000,001 matrix would otherwise run on one XCD of eight)
        const uint32_t pinned = m >= 32 ? 1u : 0u;
        const uint64_t m8 = pinned ? (m + 7) / 8 * 8 : m;
        if (col_tiles > 0x7FFFFFFFull || m8 > 0x7FFFFFFFull / col_tiles) return NKLQ_ERANGE;
        const dim3 grid((uint32_t)(m8 * col_tiles)), block(kRowsBlock);
#define NKLQ_D2(NT, SHIFT)                                                                        \
    launch_kernel((deq_2d_rows_kernel<NKLQ_NT(NT), SHIFT>), grid, block, 0, s, out, c, n_rows, n_cols, \
                       (uint32_t)col_tiles, thrd, pinned)
        if (tk.nontemporal && plain) NKLQ_D2(true, false);
        else if (tk.nontemporal) NKLQ_D2(true, true);
        else if (plain) NKLQ_D2(false, false);
        else NKLQ_D2(false, true);
#undef NKLQ_D2
        return launch_status();
    }
    // everything else (97 .. 8192 columns): the band stream
    const uint64_t pieces = (16 * n_cols + 31 + 1023) / 1024;  // 4 KiB pieces of a band, on a grid that starts up to 31 elements before it
    const uint32_t pinned = m >= 32 ? 1u : 0u;
    const uint64_t m8 = pinned ? (m + 7) / 8 * 8 : m;
    if (m8 > 0x7FFFFFFFull / pieces) return NKLQ_ERANGE;
    const uint32_t blocks = (uint32_t)(m8 * pieces);
    const uint64_t inv_pieces = ~0ull / pieces + 1;  // floor(2^64 / pieces) + 1 (pieces >= 2): exact quotients for j * pieces < 2^64
    const uint32_t inv_k = (uint32_t)(0x100000000ull / n_cols) + 1u;
    if (tk.nontemporal)
        launch_kernel((deq_stream_kernel<true>), dim3(blocks), dim3(256), 0, s, out, c, n_rows, (uint32_t)n_cols,
                      (uint32_t)pieces, inv_pieces, inv_k, thrd, pinned);
    else
        launch_kernel((deq_stream_kernel<NKLQ_NT(false)>), dim3(blocks), dim3(256), 0, s, out, c, n_rows, (uint32_t)n_cols,
                      (uint32_t)pieces, inv_pieces, inv_k, thrd, pinned);
    return launch_status();
}

}  // namespace

extern "C" {

int nklq_dequant_accumulate_f32(float* acc, const uint32_t* const* payloads, int k_payloads,
                                uint64_t n, float thrd, int accumulate, void* stream)
{
    if (k_payloads < 1) return NKLQ_ERANGE;
    if (n == 0) return NKLQ_OK;
    if (!acc || !payloads) return NKLQ_ENULL;
    if (!aligned4(acc)) return NKLQ_EALIGN;
    {
        std::vector<Span> spans = {span_of(acc, 4 * n, true, 0)};
        for (int p = 0; p < k_payloads; ++p) {
            if (!payloads[p]) return NKLQ_ENULL;
            if (!aligned4(payloads[p])) return NKLQ_EALIGN;
            spans.push_back(span_of(payloads[p], 4 * nklq_packed_words(n, 1), false));
        }
        if (spans_conflict(spans)) return NKLQ_EALIAS;
    }
    snapshot_knobs();
    hipStream_t s = (hipStream_t)stream;
    if (k_payloads == 1 && !accumulate && (__builtin_bit_cast(uint32_t, thrd) & 0x7FFFFFFFu) != 0) {
        // +0.0 + d is d for d in {+t, -t, +0.0} unless t is a zero (then -t = -0.0 would become
        // +0.0): a single payload into a fresh buffer is the plain decode, which is faster
        return dispatch_deq_flat(acc, payloads[0], n, thrd, s);
    }
    int acc_flag = accumulate ? 1 : 0;
    for (int first = 0; first < k_payloads; first += NKLQ_MAX_PAYLOADS_PER_LAUNCH) {
        PayloadPtrs pl = {};
        int k = k_payloads - first;
        if (k > NKLQ_MAX_PAYLOADS_PER_LAUNCH) k = NKLQ_MAX_PAYLOADS_PER_LAUNCH;
        for (int p = 0; p < k; ++p) pl.p[p] = payloads[first + p];
        for (int p = k; p < NKLQ_MAX_PAYLOADS_PER_LAUNCH; ++p) pl.p[p] = payloads[first];
        const int st = launch_acc_flat(acc, pl, k, n, thrd, acc_flag, s);
        if (st != NKLQ_OK) return st;
        acc_flag = 1;  // later launches continue the running sum held in acc
    }
    return NKLQ_OK;
}

int nklq_quantize_multi_f32(int count, const float* const* g, float* const* r, uint32_t* const* c,
                            const uint64_t* n, float thrd, int add_residual, void* stream)
{
    if (count < 0) return NKLQ_ERANGE;
    if (count == 0) return NKLQ_OK;
    if (!g || !r || !c || !n) return NKLQ_ENULL;
    for (int i = 0; i < count; ++i) {
        if (n[i] == 0) continue;
        if (!g[i] || !r[i] || !c[i]) return NKLQ_ENULL;
        if (!aligned4(g[i]) || !aligned4(r[i]) || !aligned4(c[i])) return NKLQ_EALIGN;
        if (n[i] / kChunk + 1 > 0x7FFFFFFFull) return NKLQ_ERANGE;
    }
    thread_local CheckedTables checked;
    checked.begin();
    checked.add(g, (size_t)count);
    checked.add(r, (size_t)count);
    checked.add(c, (size_t)count);
    checked.add(n, (size_t)count);
    if (!checked.known()) {
        std::vector<Span> spans;
        spans.reserve(3 * (size_t)count);
        for (int i = 0; i < count; ++i) {
            if (n[i] == 0) continue;
            spans.push_back(span_of(r[i], 4 * n[i], true, 2 * i));  // r[i] is its own input: in place
            spans.push_back(span_of(c[i], 4 * nklq_packed_words(n[i], 1), true, 2 * i + 1));
            spans.push_back(span_of(g[i], 4 * n[i], false, 2 * i));
        }
        if (spans_conflict(spans)) return NKLQ_EALIAS;
        checked.remember();
    }
    snapshot_knobs();
    hipStream_t s = (hipStream_t)stream;
    int i = 0;
    while (i < count) {
        QuantSegments seg = {};
        bool al = true;
        uint64_t chunks = 0;
        int m = 0;
        for (; i < count && m < kMaxSegments; ++i) {
            if (n[i] == 0) continue;
            const uint64_t mine = n[i] / kChunk + (n[i] % kChunk ? 1 : 0);
            if (chunks + mine > 0x7FFFFFFFull) break;  // next launch
            seg.g[m] = g[i];
            seg.r[m] = r[i];
            seg.c[m] = c[i];
            seg.n[m] = n[i];
            seg.first[m] = (uint32_t)chunks;
            chunks += mine;
            al = al && aligned16(g[i]) && aligned16(r[i]);
            ++m;
        }
        seg.count = m;
        for (int k = m; k <= kMaxSegments; ++k) seg.first[k] = (uint32_t)chunks;
        if (m == 0) {
            if (i < count) return NKLQ_ERANGE;  // a single vector that does not fit one launch
            break;
        }
        const int st = launch_quant_multi(seg, al, add_residual != 0, thrd, s);
        if (st != NKLQ_OK) return st;
    }
    return NKLQ_OK;
}

int nklq_dequant_accumulate_multi_f32(int count, float* const* acc, const uint64_t* n,
                                      const uint64_t* word_offset,
                                      const uint32_t* const* payload_base, int k_payloads,
                                      float thrd, int accumulate, float divisor, void* stream)
{
    if (count < 0 || k_payloads < 1) return NKLQ_ERANGE;
    if (count == 0) return NKLQ_OK;
    if (!acc || !n || !word_offset || !payload_base) return NKLQ_ENULL;
    for (int p = 0; p < k_payloads; ++p) {
        if (!payload_base[p]) return NKLQ_ENULL;
        if (!aligned4(payload_base[p])) return NKLQ_EALIGN;
    }
    for (int i = 0; i < count; ++i) {
        if (n[i] == 0) continue;
        if (!acc[i]) return NKLQ_ENULL;
        if (!aligned4(acc[i])) return NKLQ_EALIGN;
        if (n[i] / kTile + 1 > 0x7FFFFFFFull) return NKLQ_ERANGE;
    }
    thread_local CheckedTables checked;
    checked.begin();
    checked.add(acc, (size_t)count);
    checked.add(n, (size_t)count);
    checked.add(word_offset, (size_t)count);
    checked.add(payload_base, (size_t)k_payloads);
    checked.add((uint64_t)count);  // (where the first three tables end)
    if (!checked.known()) {
        // every payload is read between its lowest and highest word any vector uses
        uint64_t w_lo = UINT64_MAX, w_hi = 0;
        std::vector<Span> spans;
        spans.reserve((size_t)count + (size_t)k_payloads);
        for (int i = 0; i < count; ++i) {
            if (n[i] == 0) continue;
            spans.push_back(span_of(acc[i], 4 * n[i], true, i));
            if (word_offset[i] < w_lo) w_lo = word_offset[i];
            const uint64_t end = word_offset[i] + nklq_packed_words(n[i], 1);
            if (end > w_hi) w_hi = end;
        }
        if (w_lo < w_hi)
            for (int p = 0; p < k_payloads; ++p)
                spans.push_back(span_of(payload_base[p] + w_lo, 4 * (w_hi - w_lo), false));
        if (spans_conflict(spans)) return NKLQ_EALIAS;
        checked.remember();
    }
    snapshot_knobs();
    hipStream_t s = (hipStream_t)stream;
    int acc_flag = accumulate ? 1 : 0;
    for (int first_p = 0; first_p < k_payloads; first_p += NKLQ_MAX_PAYLOADS_PER_LAUNCH) {
        PayloadPtrs pl = {};
        int k = k_payloads - first_p;
        if (k > NKLQ_MAX_PAYLOADS_PER_LAUNCH) k = NKLQ_MAX_PAYLOADS_PER_LAUNCH;
        for (int p = 0; p < k; ++p) pl.p[p] = payload_base[first_p + p];
        for (int p = k; p < NKLQ_MAX_PAYLOADS_PER_LAUNCH; ++p) pl.p[p] = payload_base[first_p];
        int i = 0;
        while (i < count) {
            AccSegments seg = {};
            bool al = true;
            uint64_t tiles = 0;
            int m = 0;
            for (; i < count && m < kMaxSegments; ++i) {
                if (n[i] == 0) continue;
                const uint64_t mine = n[i] / kTile + (n[i] % kTile ? 1 : 0);
                if (tiles + mine > 0x7FFFFFFFull) break;
                seg.acc[m] = acc[i];
                seg.n[m] = n[i];
                seg.word_offset[m] = word_offset[i];
                seg.first[m] = (uint32_t)tiles;
                tiles += mine;
                al = al && aligned16(acc[i]);
                ++m;
            }
            seg.count = m;
            for (int j = m; j <= kMaxSegments; ++j) seg.first[j] = (uint32_t)tiles;
            if (m == 0) {
                if (i < count) return NKLQ_ERANGE;
                break;
            }
            // the division belongs to the last group of payloads only
            const bool last = first_p + NKLQ_MAX_PAYLOADS_PER_LAUNCH >= k_payloads;
            const int st = launch_acc_multi(seg, pl, k, al, thrd, acc_flag, last ? divisor : 1.0f, s);
            if (st != NKLQ_OK) return st;
        }
        acc_flag = 1;
    }
    return NKLQ_OK;
}

#if NKLQ_TUNING_BUILD
int nklq_copy_f32(float* dst, const float* src, uint64_t n, void* stream)
{
    if (n == 0) return NKLQ_OK;
    if (!dst || !src) return NKLQ_ENULL;
    if (!aligned16(dst) || !aligned16(src)) return NKLQ_EALIGN;
    {
        std::vector<Span> spans = {span_of(dst, 4 * n, true, 0), span_of(src, 4 * n, false)};
        if (spans_conflict(spans)) return NKLQ_EALIAS;
    }
    snapshot_knobs();
    return dispatch_copy(dst, src, n, (hipStream_t)stream);
}

int nklq_tuning_sum_interleaved_f32(float* acc, const uint32_t* words, int k_payloads, uint64_t n,
                                    int run_words_log2, float thrd, void* stream)
{
    if (k_payloads < 1 || k_payloads > NKLQ_MAX_PAYLOADS_PER_LAUNCH) return NKLQ_ERANGE;
    if (run_words_log2 < 6 || run_words_log2 > 40 || n % kTile != 0) return NKLQ_ERANGE;
    if (n == 0) return NKLQ_OK;
    if (!acc || !words) return NKLQ_ENULL;
    if (!aligned16(acc) || !aligned4(words)) return NKLQ_EALIGN;
    const uint64_t run = 1ull << run_words_log2;
    const uint64_t runs = (n / 16 + run - 1) / run;
    if (runs > (UINT64_MAX >> run_words_log2) / (uint64_t)k_payloads) return NKLQ_ERANGE;
    {
        std::vector<Span> spans = {span_of(acc, 4 * n, true, 0),
                                   span_of(words, 4 * runs * (uint64_t)k_payloads * run, false)};
        if (spans_conflict(spans)) return NKLQ_EALIAS;
    }
    snapshot_knobs();
    if (!mix_ok(thrd)) return NKLQ_ERANGE;
    PayloadPtrs pl = {};
    for (int p = 0; p < NKLQ_MAX_PAYLOADS_PER_LAUNCH; ++p) pl.p[p] = words + ((uint64_t)(p < k_payloads ? p : 0) << run_words_log2);
    const uint64_t n_tiles = n / kTile;
    const uint32_t xs = (uint32_t)tk.xcd_shift_acc;
    const uint64_t per_group = (uint64_t)(kAccBlock / kWave) << xs;
    const uint64_t work = ((n_tiles + per_group - 1) / per_group) << xs;
    if (work > 0x7FFFFFFFull) return NKLQ_ERANGE;
    const uint32_t pad = n_tiles >= kAccThrottleTiles ? kAccThrottleLdsBytes : 0u;
    const float th = -0.5f * thrd;
    hipStream_t s = (hipStream_t)stream;
#define NKLQ_ACC_RUNS(K, AL, MIX)                                                                              \
    launch_kernel((acc_flat_kernel<K, true, true, true>), dim3((uint32_t)work), dim3(kAccBlock), pad, s, acc, pl, \
                  k_payloads, n, n_tiles, 0u, xs, thrd, th, 0, (uint32_t)run_words_log2)
    NKLQ_ACC_DISPATCH(NKLQ_ACC_RUNS, k_payloads, true, true);
#undef NKLQ_ACC_RUNS
    return launch_status();
}
#endif

}  // extern "C"
