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
//   * the sum over K payloads (acc_flat_kernel), the matrix form (quant_2d_rows_kernel) and
//     the many-vectors form (quant_multi_kernel) are described at their kernels.
//
// fp32 arithmetic is IEEE: no fast-math, no contraction, denormals kept.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "nklq.h"

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
// Same vector with only element alignment promised: gradient views cut out of a
// flat buffer (torch.narrow) start at any element.  gfx950 global memory
// instructions need dword alignment only, so these still move 16 bytes per lane.
typedef f32x4 f32x4_a4 __attribute__((aligned(4)));
typedef u32x4 u32x4_a4 __attribute__((aligned(4)));

constexpr int kWave = 64;
constexpr int kChunk = 256;          // elements per chunk: one dwordx4 per lane
constexpr int kWordsPerChunk = 16;

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

// ---------------------------------------------------------------- flat dequantize

// out[j] = decode(c)[j]  (the reference dequantize, flat).  The 4 lanes of a quad read the
// same code word (one 64 B request per wave) and each takes its byte.  Code words are read
// with ordinary (cached) loads: two chunks share a 128 B line, and non-temporal loads of half
// lines measure 20-35 % slower here.
template <int U, int BLOCK, bool ALIGNED, bool NT>
__global__ __launch_bounds__(BLOCK) void deq_flat_kernel(
    float* out, const uint32_t* __restrict__ c, uint64_t n, uint64_t n_chunks, uint32_t has_tail,
    uint32_t xs, float t)
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
    const int lane = threadIdx.x & (kWave - 1);
    const uint32_t w = threadIdx.x >> 6;
    const uint32_t sh = 8 * (lane & 3);
#pragma unroll
    for (int j = 0; j < U; ++j) {
        const uint64_t ch = chunk_of<U, BLOCK>(blockIdx.x, w, j, xs);
        if (ch >= n_chunks) continue;
        const uint32_t word = c[ch * kWordsPerChunk + (lane >> 2)];
        st4<ALIGNED, NT>(out + ch * kChunk + lane * 4, deq_byte((word >> sh) & 0xFFu, t));
    }
}

// ---------------------------------------------------------------- flat accumulate over payloads

struct PayloadPtrs {
    const uint32_t* p[NKLQ_MAX_PAYLOADS_PER_LAUNCH];
};

constexpr int kTile = 1024;        // elements per wave in the accumulate kernel: 64 code words
constexpr int kLdsLaneStride = 20; // floats per lane in LDS (16 used): keeps b128 accesses off shared banks

// Position in a wave's LDS area of element `idx` (0..1023) of the tile.
__device__ __forceinline__ int lds_pos(int idx) { return kLdsLaneStride * (idx >> 4) + (idx & 15); }

// 2-bit codes -> 2-bit two's complement multipliers, all 16 fields of a word at once:
// 00 -> 00 (0), 01 -> 01 (+1), 10 -> 11 (-1), 11 -> 00 (0).  Per field (2 + b0 - b1) is 1..3,
// so the subtraction never borrows across fields; xor 10 then gives the table above.
__device__ __forceinline__ uint32_t codes_to_multipliers(uint32_t w)
{
    const uint32_t e = (w & 0x55555555u) | 0xAAAAAAAAu;
    const uint32_t o = (w >> 1) & 0x55555555u;
    return (e - o) ^ 0xAAAAAAAAu;
}

// acc[j] = ((start + d_0[j]) + d_1[j]) + ... strictly in payload order, start = accumulate ?
// acc[j] : +0.0f.  With K payloads the sum costs K decodes and K adds per element, so the
// layout is chosen for the arithmetic: a lane OWNS one code word of each payload (16 elements),
// so a wave fetches a payload's 64 words with one coalesced 256 B load, every shift is an
// immediate, and nothing moves between lanes during the sum.  The 16 running sums of a lane are
// 64 B apart in memory from its neighbour's, so the tile goes through LDS once on the way out
// (and once on the way in when accumulating) to turn that into 1 KiB-contiguous stores.
//
// FMA: when t is finite and not negative, (+t, -t, 0) is k * t with k in {+1, -1, 0} exactly and
// fma(k, t, s) rounds s + k*t once, i.e. gives the same bits as s + decode: 3 VALU ops per
// element and payload instead of 6 with compares and selects (which the K = 8 sum would be bound
// by).  For any other t (negative, NaN, infinite: 0 * t would not be +0) the select form is used.
template <int BLOCK, bool ALIGNED, bool NT, bool FMA>
__global__ __launch_bounds__(BLOCK) void acc_flat_kernel(
    float* acc, PayloadPtrs pl, int k_payloads, uint64_t n, uint64_t n_tiles, uint32_t has_tail,
    uint32_t xs, float t, int accumulate)
{
    constexpr int WPB = BLOCK / kWave;
    __shared__ __attribute__((aligned(16))) float lds[WPB][kWave * kLdsLaneStride];
    if (has_tail && blockIdx.x == gridDim.x - 1) {
        // tail: fewer than 1024 elements, one per lane and round, bounds-checked
        for (uint64_t e = n_tiles * kTile + threadIdx.x; e < n; e += BLOCK) {
            const uint32_t sh = 2 * (uint32_t)(e & 15);
            float s = accumulate ? acc[e] : 0.0f;
            for (int p = 0; p < k_payloads; ++p) s = s + deq_code((pl.p[p][e >> 4] >> sh) & 3u, t);
            acc[e] = s;
        }
        return;
    }
    const int lane = threadIdx.x & (kWave - 1);
    const uint32_t w = threadIdx.x >> 6;
    const uint64_t tile = chunk_of<1, BLOCK>(blockIdx.x, w, 0, xs);
    if (tile >= n_tiles) return;
    float* my = lds[w];
    float* o = acc + tile * kTile;

    // every payload's word for this lane, all loads in flight together
    uint32_t wd[NKLQ_MAX_PAYLOADS_PER_LAUNCH];
#pragma unroll
    for (int p = 0; p < NKLQ_MAX_PAYLOADS_PER_LAUNCH; ++p)
        if (p < k_payloads) wd[p] = pl.p[p][tile * (kTile / 16) + lane];

    float s[16];
    if (accumulate) {
        // coalesced read of the running sums, through LDS into the one-word-per-lane layout
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const f32x4 v = ld4<ALIGNED, NT>(o + j * 256 + lane * 4);
            *reinterpret_cast<f32x4*>(my + lds_pos(j * 256 + lane * 4)) = v;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const f32x4 v = *reinterpret_cast<const f32x4*>(my + kLdsLaneStride * lane + 4 * q);
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
    for (int p = 0; p < NKLQ_MAX_PAYLOADS_PER_LAUNCH; ++p) {
        if (p < k_payloads) {
            if constexpr (FMA) {
                const int m = (int)codes_to_multipliers(wd[p]);
#pragma unroll
                for (int i = 0; i < 16; ++i)
                    s[i] = __builtin_fmaf((float)(int)__builtin_amdgcn_sbfe(m, 2 * i, 2), t, s[i]);
            } else {
#pragma unroll
                for (int i = 0; i < 16; ++i) s[i] = s[i] + deq_code((wd[p] >> (2 * i)) & 3u, t);
            }
        }
    }

    // one-word-per-lane layout -> LDS -> 1 KiB-contiguous stores
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        f32x4 v;
        v.x = s[4 * q]; v.y = s[4 * q + 1]; v.z = s[4 * q + 2]; v.w = s[4 * q + 3];
        *reinterpret_cast<f32x4*>(my + kLdsLaneStride * lane + 4 * q) = v;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const f32x4 v = *reinterpret_cast<const f32x4*>(my + lds_pos(j * 256 + lane * 4));
        st4<ALIGNED, NT>(o + j * 256 + lane * 4, v);
    }
}

// ---------------------------------------------------------------- matrix (n, k) kernels

// Word (x, y) packs rows 16x .. 16x+15 of column y (quantize.py:35-51), so the 16 codes of a
// word are k floats apart in memory.  A workgroup of 16 waves takes a tile of 16 rows x 256
// columns: wave i moves row 16x+i of the tile with one dwordx4 per lane (1 KiB contiguous, like
// a flat chunk), so neighbouring workgroups (on different XCDs) touch neighbouring 1 KiB pieces
// of the same rows.  The 16 codes of a word come from 16 different waves: each wave ORs its
// code, shifted to its bit position, into the tile's 256 words in LDS; after a barrier 256
// threads store the 1 KiB of words.  When k is not a multiple of 4 (or a base is not 16-byte
// aligned) rows start at any element: ALIGNED = false issues the same loads with dword
// alignment, and the last 1-3 columns of a row are moved one by one.
constexpr int kRowsBlock = 16 * kWave;  // 1024 threads
constexpr uint64_t kNarrowColumns = 64; // below this many columns the one-lane-per-word kernels run

template <bool ADD, bool NT, bool ALIGNED>
__global__ __launch_bounds__(kRowsBlock) void quant_2d_rows_kernel(
    const float* g, const float* rin, float* rout, uint32_t* __restrict__ c, uint64_t n,
    uint64_t k, uint32_t col_tiles, float t)
{
    __shared__ uint32_t words[256];
    const int lane = threadIdx.x & (kWave - 1);
    const uint32_t i = threadIdx.x >> 6;  // row inside the tile = code position inside the word
    const uint64_t x = blockIdx.x / col_tiles;
    const uint64_t y0 = (uint64_t)(blockIdx.x % col_tiles) * 256;
    const uint64_t y = y0 + (uint64_t)lane * 4;
    const uint64_t row = x * 16 + i;
    // columns this lane owns: 4, or fewer at the right edge, or none
    // (with ALIGNED, k is a multiple of 4: it is 4 or none)
    const int cnt = (row < n && y < k) ? ((ALIGNED || k - y >= 4) ? 4 : (int)(k - y)) : 0;
    const uint64_t off = row * k + y;
    float a[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    float r[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (cnt == 4) {
        const f32x4 va = ld4<ALIGNED, NT>(g + off);
        a[0] = va.x; a[1] = va.y; a[2] = va.z; a[3] = va.w;
        if constexpr (ADD) {
            const f32x4 vr = ld4<ALIGNED, NT>(rin + off);
            r[0] = vr.x; r[1] = vr.y; r[2] = vr.z; r[3] = vr.w;
        }
    } else {
#pragma unroll
        for (int j = 0; j < 3; ++j) {
            if (j < cnt) {
                a[j] = g[off + j];
                if constexpr (ADD) r[j] = rin[off + j];
            }
        }
    }
    if (threadIdx.x < 256) words[threadIdx.x] = 0;
    __syncthreads();
    if (cnt > 0) {
        float o[4];
        uint32_t code[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float v = a[j];
            if constexpr (ADD) v = v + r[j];
            code[j] = quant_one(v, t, o[j]);
        }
        if (cnt == 4) {
            f32x4 vo;
            vo.x = o[0]; vo.y = o[1]; vo.z = o[2]; vo.w = o[3];
            st4<ALIGNED, NT>(rout + off, vo);
        } else {
#pragma unroll
            for (int j = 0; j < 3; ++j)
                if (j < cnt) rout[off + j] = o[j];
        }
        const uint32_t sh = 2 * i;
        // column 4*lane + j lives at words[64*j + lane]: consecutive lanes, consecutive banks
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (j < cnt && code[j]) atomicOr(&words[64 * j + lane], code[j] << sh);
    }
    __syncthreads();
    if (threadIdx.x < 256 && y0 + threadIdx.x < k)
        c[x * k + y0 + threadIdx.x] = words[64 * (threadIdx.x & 3) + (threadIdx.x >> 2)];
}

template <bool NT, bool ALIGNED>
__global__ __launch_bounds__(kRowsBlock) void deq_2d_rows_kernel(
    float* out, const uint32_t* __restrict__ c, uint64_t n, uint64_t k, uint32_t col_tiles, float t)
{
    const int lane = threadIdx.x & (kWave - 1);
    const uint32_t i = threadIdx.x >> 6;
    const uint64_t x = blockIdx.x / col_tiles;
    const uint64_t y = (uint64_t)(blockIdx.x % col_tiles) * 256 + (uint64_t)lane * 4;
    const uint64_t row = x * 16 + i;
    if (row >= n || y >= k) return;
    // with ALIGNED, k is a multiple of 4 and every lane inside the matrix owns 4 columns
    const int cnt = ALIGNED ? 4 : ((k - y < 4) ? (int)(k - y) : 4);
    const uint32_t sh = 2 * i;
    const uint32_t* cw = c + x * k + y;
    float* o = out + row * k + y;
    // all 16 waves read the tile's 1 KiB of words (cache hits after the first)
    if (cnt == 4) {
        uint32_t w0, w1, w2, w3;
        if constexpr (ALIGNED) {
            const u32x4 w = *reinterpret_cast<const u32x4*>(cw);
            w0 = w.x; w1 = w.y; w2 = w.z; w3 = w.w;
        } else {
            const u32x4_a4 w = *reinterpret_cast<const u32x4_a4*>(cw);
            w0 = w.x; w1 = w.y; w2 = w.z; w3 = w.w;
        }
        f32x4 v;
        v.x = deq_code((w0 >> sh) & 3u, t);
        v.y = deq_code((w1 >> sh) & 3u, t);
        v.z = deq_code((w2 >> sh) & 3u, t);
        v.w = deq_code((w3 >> sh) & 3u, t);
        st4<ALIGNED, NT>(o, v);
    } else {
        for (int j = 0; j < cnt; ++j) o[j] = deq_code((cw[j] >> sh) & 3u, t);
    }
}

constexpr int kBlock2D = 256;  // workgroup size of the narrow-matrix kernels

// Narrow matrices (k < 64 columns): a 256-column tile would leave most lanes idle, so one lane
// takes one word and lanes walk along the flattened (x, y) index.
template <bool ADD>
__global__ __launch_bounds__(kBlock2D) void quant_2d_kernel(
    const float* g, const float* rin, float* rout, uint32_t* __restrict__ c, uint64_t n,
    uint64_t k, uint64_t items, float t)
{
    for (uint64_t it = (uint64_t)blockIdx.x * kBlock2D + threadIdx.x; it < items;
         it += (uint64_t)gridDim.x * kBlock2D) {
        const uint64_t x = it / k;
        const uint64_t y = it - x * k;
        uint32_t word = 0;
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            float a[8];
            float r[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const uint64_t xm = x * 16 + half * 8 + i;
                if (xm < n) {
                    a[i] = g[xm * k + y];
                    if constexpr (ADD) r[i] = rin[xm * k + y];
                }
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const uint64_t xm = x * 16 + half * 8 + i;
                if (xm < n) {
                    float val = a[i];
                    if constexpr (ADD) val = val + r[i];
                    float o;
                    word |= quant_one(val, t, o) << (2 * (half * 8 + i));
                    rout[xm * k + y] = o;
                }
            }
        }
        c[x * k + y] = word;
    }
}

__global__ __launch_bounds__(kBlock2D) void deq_2d_kernel(float* out, const uint32_t* __restrict__ c,
                                                           uint64_t n, uint64_t k, uint64_t items,
                                                           float t)
{
    for (uint64_t it = (uint64_t)blockIdx.x * kBlock2D + threadIdx.x; it < items;
         it += (uint64_t)gridDim.x * kBlock2D) {
        const uint64_t x = it / k;
        const uint64_t y = it - x * k;
        const uint32_t word = c[x * k + y];
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const uint64_t xm = x * 16 + i;
            if (xm < n) out[xm * k + y] = deq_code((word >> (2 * i)) & 3u, t);
        }
    }
}

// ---------------------------------------------------------------- many vectors in one launch

// A model's gradients are many separate vectors (161 for ResNet-50, most of them small); one
// launch per vector costs more in launch latency than the data takes to stream.  These kernels
// take a table of up to kMaxSegments (96) vectors in their arguments and treat the chunks (or tiles)
// of all of them as one index space; a wave finds its vector by binary search in the table.

constexpr int kMaxSegments = 96;  // 96 x 36 B of table stays under the 4 KiB kernel-argument limit

struct QuantSegments {
    const float* g[kMaxSegments];
    float* r[kMaxSegments];
    uint32_t* c[kMaxSegments];
    uint64_t n[kMaxSegments];
    uint32_t first[kMaxSegments + 1];  // first[s] = index of segment s's first chunk; first[count] = total
    int count;
};

// Largest s with first[s] <= q (q < first[count]).
__device__ __forceinline__ int find_segment(const uint32_t* first, int count, uint32_t q)
{
    int lo = 0, hi = count;  // invariant: first[lo] <= q < first[hi]
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (first[mid] <= q) lo = mid;
        else hi = mid;
    }
    return lo;
}

template <bool ALIGNED, bool ADD, bool NT>
__global__ __launch_bounds__(256) void quant_multi_kernel(QuantSegments seg, uint32_t xs, float t)
{
    const int lane = threadIdx.x & (kWave - 1);
    const uint32_t w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint64_t q64 = chunk_of<1, 256>(blockIdx.x, w, 0, xs);
    if (q64 >= seg.first[seg.count]) return;
    const uint32_t q = (uint32_t)q64;
    const int sidx = find_segment(seg.first, seg.count, q);
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
        // last, partial chunk of the vector: one element per lane, 4 rounds, all lanes reach row_or
#pragma unroll
        for (int first = 0; first < kChunk; first += kWave) {
            const uint64_t e = e0 + (uint64_t)(first + lane);
            const bool live = e < n;
            uint32_t code = 0;
            if (live) {
                float a = g[e];
                if constexpr (ADD) a = a + r[e];
                float res;
                code = quant_one(a, t, res);
                r[e] = res;
            }
            const uint32_t word = row_or(code << (2 * (lane & 15)));
            if (live && (lane & 15) == 0) c[e >> 4] = word;
        }
    }
}

struct AccSegments {
    float* acc[kMaxSegments];
    uint64_t n[kMaxSegments];
    uint64_t word_offset[kMaxSegments];  // of the vector's first code word inside every payload
    uint32_t first[kMaxSegments + 1];    // in tiles of 1024 elements
    int count;
};

template <bool ALIGNED, bool NT, bool FMA>
__global__ __launch_bounds__(256) void acc_multi_kernel(AccSegments seg, PayloadPtrs pl, int k_payloads,
                                                        uint32_t xs, float t, int accumulate,
                                                        float divisor)
{
    const bool divide = divisor != 1.0f;  // IEEE division, correctly rounded (not a reciprocal)
    __shared__ __attribute__((aligned(16))) float lds[4][kWave * kLdsLaneStride];
    const int lane = threadIdx.x & (kWave - 1);
    const uint32_t w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint64_t q64 = chunk_of<1, 256>(blockIdx.x, w, 0, xs);
    if (q64 >= seg.first[seg.count]) return;
    const uint32_t q = (uint32_t)q64;
    const int sidx = find_segment(seg.first, seg.count, q);
    const uint64_t n = seg.n[sidx];
    const uint64_t e0 = (uint64_t)(q - seg.first[sidx]) * kTile;
    float* o = seg.acc[sidx] + e0;
    const uint64_t w0 = seg.word_offset[sidx] + (e0 >> 4);
    if (e0 + kTile > n) {
        // last, partial tile of the vector: one element per lane and round, bounds-checked
        for (uint64_t e = e0 + lane; e < n; e += kWave) {
            const uint32_t sh = 2 * (uint32_t)(e & 15);
            float s = accumulate ? seg.acc[sidx][e] : 0.0f;
            for (int p = 0; p < k_payloads; ++p)
                s = s + deq_code((pl.p[p][seg.word_offset[sidx] + (e >> 4)] >> sh) & 3u, t);
            seg.acc[sidx][e] = divide ? s / divisor : s;
        }
        return;
    }
    float* my = lds[w];
    uint32_t wd[NKLQ_MAX_PAYLOADS_PER_LAUNCH];
#pragma unroll
    for (int p = 0; p < NKLQ_MAX_PAYLOADS_PER_LAUNCH; ++p)
        if (p < k_payloads) wd[p] = pl.p[p][w0 + lane];
    float s[16];
    if (accumulate) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const f32x4 v = ld4<ALIGNED, NT>(o + j * 256 + lane * 4);
            *reinterpret_cast<f32x4*>(my + lds_pos(j * 256 + lane * 4)) = v;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int qd = 0; qd < 4; ++qd) {
            const f32x4 v = *reinterpret_cast<const f32x4*>(my + kLdsLaneStride * lane + 4 * qd);
            s[4 * qd] = v.x; s[4 * qd + 1] = v.y; s[4 * qd + 2] = v.z; s[4 * qd + 3] = v.w;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    } else {
#pragma unroll
        for (int i = 0; i < 16; ++i) s[i] = 0.0f;
    }
#pragma unroll
    for (int p = 0; p < NKLQ_MAX_PAYLOADS_PER_LAUNCH; ++p) {
        if (p < k_payloads) {
            if constexpr (FMA) {
                const int m = (int)codes_to_multipliers(wd[p]);
#pragma unroll
                for (int i = 0; i < 16; ++i)
                    s[i] = __builtin_fmaf((float)(int)__builtin_amdgcn_sbfe(m, 2 * i, 2), t, s[i]);
            } else {
#pragma unroll
                for (int i = 0; i < 16; ++i) s[i] = s[i] + deq_code((wd[p] >> (2 * i)) & 3u, t);
            }
        }
    }
    if (divide) {
#pragma unroll
        for (int i = 0; i < 16; ++i) s[i] = s[i] / divisor;
    }
#pragma unroll
    for (int qd = 0; qd < 4; ++qd) {
        f32x4 v;
        v.x = s[4 * qd]; v.y = s[4 * qd + 1]; v.z = s[4 * qd + 2]; v.w = s[4 * qd + 3];
        *reinterpret_cast<f32x4*>(my + kLdsLaneStride * lane + 4 * qd) = v;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const f32x4 v = *reinterpret_cast<const f32x4*>(my + lds_pos(j * 256 + lane * 4));
        st4<ALIGNED, NT>(o + j * 256 + lane * 4, v);
    }
}

// ---------------------------------------------------------------- copy (measurement aid)

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

// ---------------------------------------------------------------- host side

// Launch-geometry knobs (results never depend on them); defaults from a sweep on MI355X.
int g_chunks_per_wave = 1;  // 1, 2 or 4
int g_block = 256;          // 64, 128, 256, 512 or 1024 threads
int g_nontemporal = 1;
int g_xcd_shift = 2;        // quantize/copy: chunks interleaved over 2^g_xcd_shift workgroups
int g_xcd_shift_decode = 0; // the same for dequantize and accumulate (write-dominated: contiguous wins)

int compute_units()
{
    static int cached[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    if (cached[dev] == 0) {
        int cu = 0;
        if (hipDeviceGetAttribute(&cu, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
            cu <= 0)
            cu = 256;
        cached[dev] = cu;
    }
    return cached[dev];
}

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

inline int launch_status()
{
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? NKLQ_OK : (int)e;
}

// ---- flat quantize dispatch: (U, BLOCK) -> (ALIGNED, ADD, NT)

template <int U, int BLOCK>
int launch_quant_flat(const float* g, const float* rin, float* rout, uint32_t* c, uint64_t n, float t,
                      bool add, bool al, hipStream_t s)
{
    const FlatGrid fg = flat_grid(n, U, BLOCK, g_xcd_shift);
    if (fg.blocks == 0) return NKLQ_ERANGE;
    const bool nt = g_nontemporal != 0;
#define NKLQ_Q(AL, ADD, NT)                                                                       \
    hipLaunchKernelGGL((quant_flat_kernel<U, BLOCK, AL, ADD, NT>), dim3(fg.blocks), dim3(BLOCK), 0, \
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

template <int U, int BLOCK>
int launch_deq_flat(float* out, const uint32_t* c, uint64_t n, float t, hipStream_t s)
{
    const FlatGrid fg = flat_grid(n, U, BLOCK, g_xcd_shift_decode);
    if (fg.blocks == 0) return NKLQ_ERANGE;
    const bool al = aligned16(out);
    const bool nt = g_nontemporal != 0;
#define NKLQ_DEQ(AL, NT)                                                                        \
    hipLaunchKernelGGL((deq_flat_kernel<U, BLOCK, AL, NT>), dim3(fg.blocks), dim3(BLOCK), 0, s, out, \
                       c, n, fg.n_chunks, fg.has_tail, fg.xs, t)
    if (al && nt) NKLQ_DEQ(true, true);
    else if (al) NKLQ_DEQ(true, false);
    else if (nt) NKLQ_DEQ(false, true);
    else NKLQ_DEQ(false, false);
#undef NKLQ_DEQ
    return launch_status();
}

// The accumulate kernel works on tiles of 1024 elements, one per wave, 256-thread workgroups.
int launch_acc_flat(float* acc, const PayloadPtrs& pl, int k, uint64_t n, float t, int accumulate,
                    hipStream_t s)
{
    constexpr int BLOCK = 256;
    const uint32_t xs = (uint32_t)g_xcd_shift_decode;
    const uint64_t n_tiles = n / kTile;
    const uint32_t has_tail = (n_tiles * kTile < n) ? 1u : 0u;
    const uint64_t per_group = (uint64_t)(BLOCK / kWave) << xs;
    const uint64_t work = ((n_tiles + per_group - 1) / per_group) << xs;
    if (work + has_tail > 0x7FFFFFFFull) return NKLQ_ERANGE;
    const uint32_t blocks = (uint32_t)work + has_tail;
    const bool al = aligned16(acc);
    const bool nt = g_nontemporal != 0;
    // fma(k, t, s) reproduces s + decode only when 0 * t is +0 and k * t is exact: finite t >= +0
    const uint32_t tbits = __builtin_bit_cast(uint32_t, t);
    const bool fma_ok = (tbits >> 31) == 0 && (tbits & 0x7F800000u) != 0x7F800000u;
#define NKLQ_ACC(AL, NT, FMA)                                                                     \
    hipLaunchKernelGGL((acc_flat_kernel<BLOCK, AL, NT, FMA>), dim3(blocks), dim3(BLOCK), 0, s, acc, \
                       pl, k, n, n_tiles, has_tail, xs, t, accumulate)
    const int sel = (al ? 4 : 0) | (nt ? 2 : 0) | (fma_ok ? 1 : 0);
    switch (sel) {
        case 7: NKLQ_ACC(true, true, true); break;
        case 6: NKLQ_ACC(true, true, false); break;
        case 5: NKLQ_ACC(true, false, true); break;
        case 4: NKLQ_ACC(true, false, false); break;
        case 3: NKLQ_ACC(false, true, true); break;
        case 2: NKLQ_ACC(false, true, false); break;
        case 1: NKLQ_ACC(false, false, true); break;
        default: NKLQ_ACC(false, false, false); break;
    }
#undef NKLQ_ACC
    return launch_status();
}

// Expands to the call of FN<U, BLOCK, ...> for the current knob values.
#define NKLQ_FOR_GEOMETRY(CALL)                                  \
    switch (g_chunks_per_wave * 10000 + g_block) {               \
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

int dispatch_quant_flat(const float* g, const float* rin, float* rout, uint32_t* c, uint64_t n,
                        float t, bool add, bool al, hipStream_t s)
{
#define NKLQ_CALL(U, B) launch_quant_flat<U, B>(g, rin, rout, c, n, t, add, al, s)
    NKLQ_FOR_GEOMETRY(NKLQ_CALL)
#undef NKLQ_CALL
}

int dispatch_deq_flat(float* out, const uint32_t* c, uint64_t n, float t, hipStream_t s)
{
#define NKLQ_CALL(U, B) launch_deq_flat<U, B>(out, c, n, t, s)
    NKLQ_FOR_GEOMETRY(NKLQ_CALL)
#undef NKLQ_CALL
}

template <int U, int BLOCK>
int launch_copy(float* dst, const float* src, uint64_t n, hipStream_t s)
{
    const FlatGrid fg = flat_grid(n, U, BLOCK, g_xcd_shift);
    if (fg.blocks == 0) return NKLQ_ERANGE;
    if (g_nontemporal)
        hipLaunchKernelGGL((copy_kernel<U, BLOCK, true>), dim3(fg.blocks), dim3(BLOCK), 0, s, dst, src,
                           n, fg.n_chunks, fg.has_tail, fg.xs);
    else
        hipLaunchKernelGGL((copy_kernel<U, BLOCK, false>), dim3(fg.blocks), dim3(BLOCK), 0, s, dst,
                           src, n, fg.n_chunks, fg.has_tail, fg.xs);
    return launch_status();
}

int dispatch_copy(float* dst, const float* src, uint64_t n, hipStream_t s)
{
#define NKLQ_CALL(U, B) launch_copy<U, B>(dst, src, n, s)
    NKLQ_FOR_GEOMETRY(NKLQ_CALL)
#undef NKLQ_CALL
}

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
    const uint32_t xs = (uint32_t)g_xcd_shift;
    if (!multi_grid(seg.first[seg.count], xs, &blocks)) return NKLQ_ERANGE;
    if (blocks == 0) return NKLQ_OK;
    const bool nt = g_nontemporal != 0;
#define NKLQ_QM(AL, ADD, NT) \
    hipLaunchKernelGGL((quant_multi_kernel<AL, ADD, NT>), dim3(blocks), dim3(256), 0, s, seg, xs, t)
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
    const uint32_t xs = (uint32_t)g_xcd_shift_decode;
    if (!multi_grid(seg.first[seg.count], xs, &blocks)) return NKLQ_ERANGE;
    if (blocks == 0) return NKLQ_OK;
    const bool nt = g_nontemporal != 0;
    const uint32_t tbits = __builtin_bit_cast(uint32_t, t);
    const bool fma_ok = (tbits >> 31) == 0 && (tbits & 0x7F800000u) != 0x7F800000u;
#define NKLQ_AM(AL, NT, FMA)                                                                      \
    hipLaunchKernelGGL((acc_multi_kernel<AL, NT, FMA>), dim3(blocks), dim3(256), 0, s, seg, pl, k, xs, \
                       t, accumulate, divisor)
    switch ((al ? 4 : 0) | (nt ? 2 : 0) | (fma_ok ? 1 : 0)) {
        case 7: NKLQ_AM(true, true, true); break;
        case 6: NKLQ_AM(true, true, false); break;
        case 5: NKLQ_AM(true, false, true); break;
        case 4: NKLQ_AM(true, false, false); break;
        case 3: NKLQ_AM(false, true, true); break;
        case 2: NKLQ_AM(false, true, false); break;
        case 1: NKLQ_AM(false, false, true); break;
        default: NKLQ_AM(false, false, false); break;
    }
#undef NKLQ_AM
    return launch_status();
}

uint32_t grid_for_items(uint64_t items)
{
    uint64_t blocks = (items + kBlock2D - 1) / kBlock2D;
    const uint64_t cap = (uint64_t)compute_units() * 64;
    if (blocks > cap) blocks = cap;
    return (uint32_t)(blocks ? blocks : 1);
}

// n_rows * n_cols with overflow check
bool mul_ok(uint64_t a, uint64_t b, uint64_t* out)
{
    if (a != 0 && b > UINT64_MAX / a) return false;
    *out = a * b;
    return true;
}

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
    int* slot = nullptr;
    switch (which) {
        case NKLQ_TUNE_CHUNKS_PER_WAVE: slot = &g_chunks_per_wave; break;
        case NKLQ_TUNE_WORKGROUP_SIZE: slot = &g_block; break;
        case NKLQ_TUNE_NONTEMPORAL: slot = &g_nontemporal; break;
        case NKLQ_TUNE_XCD_INTERLEAVE_LOG2: slot = &g_xcd_shift; break;
        case NKLQ_TUNE_XCD_INTERLEAVE_LOG2_DECODE: slot = &g_xcd_shift_decode; break;
        default: return NKLQ_ERANGE;
    }
    const int prev = *slot;
    if (value < 0) return prev;
    switch (which) {
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
        default:
            if (value > 6) return NKLQ_ERANGE;
            break;
    }
    *slot = value;
    return prev;
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
    if ((const void*)c == (const void*)g || (const void*)c == (const void*)r_out) return NKLQ_EALIAS;
    hipStream_t s = (hipStream_t)stream;
    const bool add = add_residual != 0;
    if (!add) r_in = g;  // never read; keeps the argument a valid address

    if (n_cols == 1) {
        const bool al = aligned16(g) && aligned16(r_out) && (!add || aligned16(r_in));
        return dispatch_quant_flat(g, r_in, r_out, c, total, thrd, add, al, s);
    }
    const uint64_t m = n_rows / 16 + (n_rows % 16 ? 1 : 0);
    if (n_cols < kNarrowColumns) {
        const uint64_t items = m * n_cols;
        const uint32_t grid = grid_for_items(items);
        if (add)
            hipLaunchKernelGGL((quant_2d_kernel<true>), dim3(grid), dim3(kBlock2D), 0, s, g, r_in,
                               r_out, c, n_rows, n_cols, items, thrd);
        else
            hipLaunchKernelGGL((quant_2d_kernel<false>), dim3(grid), dim3(kBlock2D), 0, s, g, r_in,
                               r_out, c, n_rows, n_cols, items, thrd);
        return launch_status();
    }
    const bool al = (n_cols % 4 == 0) && aligned16(g) && aligned16(r_out) && (!add || aligned16(r_in));
    const uint64_t col_tiles = (n_cols + 255) / 256;
    if (col_tiles > 0x7FFFFFFFull || m > 0x7FFFFFFFull / col_tiles) return NKLQ_ERANGE;
    const dim3 grid((uint32_t)(m * col_tiles)), block(kRowsBlock);
#define NKLQ_Q2(ADD, NT, AL)                                                                         \
    hipLaunchKernelGGL((quant_2d_rows_kernel<ADD, NT, AL>), grid, block, 0, s, g, r_in, r_out, c, n_rows, \
                       n_cols, (uint32_t)col_tiles, thrd)
    switch ((add ? 4 : 0) | (g_nontemporal ? 2 : 0) | (al ? 1 : 0)) {
        case 7: NKLQ_Q2(true, true, true); break;
        case 6: NKLQ_Q2(true, true, false); break;
        case 5: NKLQ_Q2(true, false, true); break;
        case 4: NKLQ_Q2(true, false, false); break;
        case 3: NKLQ_Q2(false, true, true); break;
        case 2: NKLQ_Q2(false, true, false); break;
        case 1: NKLQ_Q2(false, false, true); break;
        default: NKLQ_Q2(false, false, false); break;
    }
#undef NKLQ_Q2
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
    if ((const void*)c == (const void*)out) return NKLQ_EALIAS;
    hipStream_t s = (hipStream_t)stream;
    if (n_cols == 1) {
        return dispatch_deq_flat(out, c, total, thrd, s);
    }
    const uint64_t m = n_rows / 16 + (n_rows % 16 ? 1 : 0);
    if (n_cols < kNarrowColumns) {
        const uint64_t items = m * n_cols;
        hipLaunchKernelGGL((deq_2d_kernel), dim3(grid_for_items(items)), dim3(kBlock2D), 0, s, out, c,
                           n_rows, n_cols, items, thrd);
        return launch_status();
    }
    const bool al = (n_cols % 4 == 0) && aligned16(out) && aligned16(c);
    const uint64_t col_tiles = (n_cols + 255) / 256;
    if (col_tiles > 0x7FFFFFFFull || m > 0x7FFFFFFFull / col_tiles) return NKLQ_ERANGE;
    const dim3 grid((uint32_t)(m * col_tiles)), block(kRowsBlock);
#define NKLQ_D2(NT, AL)                                                                            \
    hipLaunchKernelGGL((deq_2d_rows_kernel<NT, AL>), grid, block, 0, s, out, c, n_rows, n_cols, \
                       (uint32_t)col_tiles, thrd)
    if (g_nontemporal && al) NKLQ_D2(true, true);
    else if (g_nontemporal) NKLQ_D2(true, false);
    else if (al) NKLQ_D2(false, true);
    else NKLQ_D2(false, false);
#undef NKLQ_D2
    return launch_status();
}

int nklq_dequant_accumulate_f32(float* acc, const uint32_t* const* payloads, int k_payloads,
                                uint64_t n, float thrd, int accumulate, void* stream)
{
    if (k_payloads < 1) return NKLQ_ERANGE;
    if (n == 0) return NKLQ_OK;
    if (!acc || !payloads) return NKLQ_ENULL;
    if (!aligned4(acc)) return NKLQ_EALIGN;
    for (int p = 0; p < k_payloads; ++p) {
        if (!payloads[p]) return NKLQ_ENULL;
        if (!aligned4(payloads[p])) return NKLQ_EALIGN;
        if ((const void*)payloads[p] == (const void*)acc) return NKLQ_EALIAS;
    }
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
        if ((const void*)c[i] == (const void*)g[i] || (const void*)c[i] == (const void*)r[i])
            return NKLQ_EALIAS;
        if (n[i] / kChunk + 1 > 0x7FFFFFFFull) return NKLQ_ERANGE;
    }
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

int nklq_copy_f32(float* dst, const float* src, uint64_t n, void* stream)
{
    if (n == 0) return NKLQ_OK;
    if (!dst || !src) return NKLQ_ENULL;
    if (!aligned16(dst) || !aligned16(src)) return NKLQ_EALIGN;
    return dispatch_copy(dst, src, n, (hipStream_t)stream);
}

}  // extern "C"
