// nklq.hip — 2-bit gradient quantizer for MI355X (gfx950, CDNA4): kernels + C-ABI.
//
// Semantics follow necklace/cuda/quantize.py:16-51 (quantize) and :56-87
// (dequantize); the layout of the code words is the one of :34-51.  Nothing
// here is GEMM-shaped: every kernel is a single streaming pass bounded by HBM
// bandwidth, so the design is about memory access only:
//
//   * a flat vector is cut into wave tiles of U*256 elements; load j of a
//     wave reads 64 lanes x 16 B = 1 KiB of contiguous memory
//     (global_load_dwordx4), all U loads of g and of the residual are issued
//     before the first use, so a wave keeps 2*U KiB in flight;
//   * a lane's 4 elements give one byte of codes; the 4 lanes of a quad are OR-ed
//     together with two DPP quad permutes (no LDS, no memory) to form the word of
//     16 codes, and for U == 4 every lane ends up storing exactly one word, so a
//     wave writes its 64 words as one 256 B store;
//   * the residual is written back in the same pass (one read of g and r, one
//     write of r and of the codes: 12.25 bytes per element);
//   * lengths that are not a multiple of the tile, and the last partial word,
//     go through a bounds-checked one-element-per-lane path in one extra
//     workgroup of the same launch (codes combined across the 16 lanes of a
//     DPP row);
//   * 64-bit element indices throughout (vectors of more than 2^31 elements).
//
// fp32 arithmetic is IEEE: no fast-math, no contraction, denormals kept.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "nklq.h"

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
// Same vectors with only element alignment promised: gradient views cut out of a
// flat buffer (torch.narrow) start at any element.  gfx950 global memory
// instructions need dword alignment only, so these still move 16 bytes per lane.
typedef f32x4 f32x4_a4 __attribute__((aligned(4)));
typedef u32x4 u32x4_a4 __attribute__((aligned(4)));

constexpr int kWave = 64;
constexpr int kBlock = 256;
constexpr int kWavesPerBlock = kBlock / kWave;

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

// Value of `v` held by lane `src` (0..63) of this wave.
__device__ __forceinline__ uint32_t lane_read(uint32_t v, int src)
{
    return (uint32_t)__builtin_amdgcn_ds_bpermute(src << 2, (int)v);
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

template <bool NT>
__device__ __forceinline__ void st1(uint32_t* p, uint32_t v)
{
    if constexpr (NT) __builtin_nontemporal_store(v, p);
    else *p = v;
}

// ---------------------------------------------------------------- flat quantize

// Tail of a flat vector: elements [base, n), base a multiple of 16, fewer than
// kBlock*ROUNDS of them.  One element per lane per round; lane l of a DPP row
// owns code position l of the word.
template <bool ADD, int ROUNDS>
__device__ __forceinline__ void quant_tail(const float* g, const float* rin, float* rout,
                                           uint32_t* c, uint64_t base, uint64_t n, float t)
{
    const int tid = threadIdx.x;
#pragma unroll 4
    for (int it = 0; it < ROUNDS; ++it) {
        const uint64_t e = base + (uint64_t)it * kBlock + tid;
        const bool live = e < n;
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

// One launch quantizes the whole flat vector.  Waves stride over the
// `n_tiles` full wave tiles; the workgroup with blockIdx.x == gridDim.x - 1 is
// reserved for the tail when `tail_base < n`.
template <int U, bool ALIGNED, bool ADD, bool NT>
__global__ __launch_bounds__(kBlock) void quant_flat_kernel(
    const float* g, const float* rin, float* rout, uint32_t* __restrict__ c, uint64_t n,
    uint64_t n_tiles, uint32_t has_tail, float t)
{
    constexpr uint64_t kTile = (uint64_t)U * 256;  // elements per wave tile
    const uint32_t n_work_blocks = gridDim.x - has_tail;
    if (blockIdx.x >= n_work_blocks) {
        quant_tail<ADD, U>(g, rin, rout, c, n_tiles * kTile, n, t);
        return;
    }
    const int lane = threadIdx.x & (kWave - 1);
    const uint64_t wave = (uint64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
    const uint64_t n_waves = (uint64_t)n_work_blocks * kWavesPerBlock;

    for (uint64_t tile = wave; tile < n_tiles; tile += n_waves) {
        const uint64_t e0 = tile * kTile + (uint64_t)lane * 4;
        f32x4 a[U];
        f32x4 r[U];
#pragma unroll
        for (int j = 0; j < U; ++j) a[j] = ld4<ALIGNED, NT>(g + e0 + j * 256);
        if constexpr (ADD) {
#pragma unroll
            for (int j = 0; j < U; ++j) r[j] = ld4<ALIGNED, NT>(rin + e0 + j * 256);
        }
        uint32_t w[U];
#pragma unroll
        for (int j = 0; j < U; ++j) {
            f32x4 v = a[j];
            if constexpr (ADD) v = v + r[j];
            float o0, o1, o2, o3;
            uint32_t b = quant_one(v.x, t, o0);
            b |= quant_one(v.y, t, o1) << 2;
            b |= quant_one(v.z, t, o2) << 4;
            b |= quant_one(v.w, t, o3) << 6;
            f32x4 o;
            o.x = o0; o.y = o1; o.z = o2; o.w = o3;
            st4<ALIGNED, NT>(rout + e0 + j * 256, o);
            w[j] = quad_or(b << (8 * (lane & 3)));
        }
        // Word 16*j + lane/4 of the tile is now in all 4 lanes of quad lane/4
        // (for each j).  Lane l stores the word of j == l%4 (+4 per extra pass).
        uint32_t* cw = c + tile * (kTile / 16);
#pragma unroll
        for (int s = 0; s < (U + 3) / 4; ++s) {
            const int j = 4 * s + (lane & 3);
            uint32_t mine = w[4 * s];
#pragma unroll
            for (int q = 1; q < 4; ++q)
                if (4 * s + q < U && (lane & 3) == q) mine = w[4 * s + q];
            if (j < U) st1<NT>(cw + 16 * j + (lane >> 2), mine);
        }
    }
}

// ---------------------------------------------------------------- flat dequantize / accumulate

struct PayloadPtrs {
    const uint32_t* p[NKLQ_MAX_PAYLOADS_PER_LAUNCH];
};

// OVERWRITE: out[j] = decode(payload 0)[j]  (the reference dequantize, flat).
// otherwise: out[j] = ((start + d_0[j]) + d_1[j]) + ... strictly in payload
// order, start = accumulate ? out[j] : +0.0f.  A wave fetches the tile's U*16
// words of a payload with one load (one word per lane) and hands each lane its
// byte through the LDS crossbar (ds_bpermute, no LDS memory involved).
template <int U, bool ALIGNED, bool NT, bool OVERWRITE>
__global__ __launch_bounds__(kBlock) void deq_flat_kernel(
    float* out, PayloadPtrs pl, int k_payloads, uint64_t n, uint64_t n_tiles, uint32_t has_tail,
    float t, int accumulate)
{
    constexpr uint64_t kTile = (uint64_t)U * 256;
    constexpr int kWordsPerTile = U * 16;
    const uint32_t n_work_blocks = gridDim.x - has_tail;
    if (blockIdx.x >= n_work_blocks) {
        // tail: one element per lane per round, bounds-checked
        const uint64_t base = n_tiles * kTile;
        for (int it = 0; it < U; ++it) {
            const uint64_t e = base + (uint64_t)it * kBlock + threadIdx.x;
            if (e < n) {
                const uint32_t sh = 2 * (uint32_t)(e & 15);
                if constexpr (OVERWRITE) {
                    out[e] = deq_code((pl.p[0][e >> 4] >> sh) & 3u, t);
                } else {
                    float s = accumulate ? out[e] : 0.0f;
                    for (int p = 0; p < k_payloads; ++p)
                        s = s + deq_code((pl.p[p][e >> 4] >> sh) & 3u, t);
                    out[e] = s;
                }
            }
        }
        return;
    }
    const int lane = threadIdx.x & (kWave - 1);
    const uint64_t wave = (uint64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
    const uint64_t n_waves = (uint64_t)n_work_blocks * kWavesPerBlock;

    for (uint64_t tile = wave; tile < n_tiles; tile += n_waves) {
        const uint64_t e0 = tile * kTile + (uint64_t)lane * 4;
        const uint64_t w0 = tile * kWordsPerTile;
        f32x4 s[U];
        if constexpr (!OVERWRITE) {
            if (accumulate) {
#pragma unroll
                for (int j = 0; j < U; ++j) s[j] = ld4<ALIGNED, NT>(out + e0 + j * 256);
            } else {
#pragma unroll
                for (int j = 0; j < U; ++j) s[j] = (f32x4)(0.0f);
            }
        }
        for (int p = 0; p < (OVERWRITE ? 1 : k_payloads); ++p) {
            // the tile's U*16 words sit in lanes 0 .. U*16-1
            uint32_t word = 0;
            if (lane < kWordsPerTile) {
                if constexpr (NT) word = __builtin_nontemporal_load(pl.p[p] + w0 + lane);
                else word = pl.p[p][w0 + lane];
            }
#pragma unroll
            for (int j = 0; j < U; ++j) {
                // elements e0 + 256 j .. +3 are byte lane%4 of word 16 j + lane/4
                const uint32_t wj = lane_read(word, 16 * j + (lane >> 2));
                const f32x4 d = deq_byte((wj >> (8 * (lane & 3))) & 0xFFu, t);
                if constexpr (OVERWRITE) s[j] = d;
                else s[j] = s[j] + d;
            }
        }
#pragma unroll
        for (int j = 0; j < U; ++j) st4<ALIGNED, NT>(out + e0 + j * 256, s[j]);
    }
}

// ---------------------------------------------------------------- matrix (n, k) kernels

// Word (x, y) packs rows 16x .. 16x+15 of column y (quantize.py:35-51).  Lanes
// walk along y, the contiguous dimension; VEC columns per lane.
template <int VEC, bool ADD>
__global__ __launch_bounds__(kBlock) void quant_2d_kernel(
    const float* g, const float* rin, float* rout, uint32_t* __restrict__ c, uint64_t n,
    uint64_t k, uint64_t items, float t)
{
    const uint64_t kv = k / VEC;  // lanes per row of words
    for (uint64_t it = (uint64_t)blockIdx.x * kBlock + threadIdx.x; it < items;
         it += (uint64_t)gridDim.x * kBlock) {
        const uint64_t x = it / kv;
        const uint64_t y = (it - x * kv) * VEC;
        uint32_t w[VEC];
#pragma unroll
        for (int v = 0; v < VEC; ++v) w[v] = 0;
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            float a[8][VEC];
            float r[8][VEC];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const uint64_t xm = x * 16 + half * 8 + i;
                if (xm < n) {
                    const uint64_t off = xm * k + y;
                    if constexpr (VEC == 4) {
                        const f32x4 q = *reinterpret_cast<const f32x4*>(g + off);
                        a[i][0] = q.x; a[i][1] = q.y; a[i][2] = q.z; a[i][3] = q.w;
                        if constexpr (ADD) {
                            const f32x4 p = *reinterpret_cast<const f32x4*>(rin + off);
                            r[i][0] = p.x; r[i][1] = p.y; r[i][2] = p.z; r[i][3] = p.w;
                        }
                    } else {
                        a[i][0] = g[off];
                        if constexpr (ADD) r[i][0] = rin[off];
                    }
                }
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const uint64_t xm = x * 16 + half * 8 + i;
                if (xm < n) {
                    const uint64_t off = xm * k + y;
                    float o[VEC];
#pragma unroll
                    for (int v = 0; v < VEC; ++v) {
                        float val = a[i][v];
                        if constexpr (ADD) val = val + r[i][v];
                        w[v] |= quant_one(val, t, o[v]) << (2 * (half * 8 + i));
                    }
                    if constexpr (VEC == 4) {
                        f32x4 q;
                        q.x = o[0]; q.y = o[1]; q.z = o[2]; q.w = o[3];
                        *reinterpret_cast<f32x4*>(rout + off) = q;
                    } else {
                        rout[off] = o[0];
                    }
                }
            }
        }
        if constexpr (VEC == 4) {
            u32x4 q;
            q.x = w[0]; q.y = w[1]; q.z = w[2]; q.w = w[3];
            *reinterpret_cast<u32x4*>(c + x * k + y) = q;
        } else {
            c[x * k + y] = w[0];
        }
    }
}

template <int VEC>
__global__ __launch_bounds__(kBlock) void deq_2d_kernel(float* out, const uint32_t* __restrict__ c,
                                                         uint64_t n, uint64_t k, uint64_t items,
                                                         float t)
{
    const uint64_t kv = k / VEC;
    for (uint64_t it = (uint64_t)blockIdx.x * kBlock + threadIdx.x; it < items;
         it += (uint64_t)gridDim.x * kBlock) {
        const uint64_t x = it / kv;
        const uint64_t y = (it - x * kv) * VEC;
        uint32_t w[VEC];
        if constexpr (VEC == 4) {
            const u32x4 q = *reinterpret_cast<const u32x4*>(c + x * k + y);
            w[0] = q.x; w[1] = q.y; w[2] = q.z; w[3] = q.w;
        } else {
            w[0] = c[x * k + y];
        }
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const uint64_t xm = x * 16 + i;
            if (xm < n) {
                const uint64_t off = xm * k + y;
                if constexpr (VEC == 4) {
                    f32x4 q;
                    q.x = deq_code((w[0] >> (2 * i)) & 3u, t);
                    q.y = deq_code((w[1] >> (2 * i)) & 3u, t);
                    q.z = deq_code((w[2] >> (2 * i)) & 3u, t);
                    q.w = deq_code((w[3] >> (2 * i)) & 3u, t);
                    *reinterpret_cast<f32x4*>(out + off) = q;
                } else {
                    out[off] = deq_code((w[0] >> (2 * i)) & 3u, t);
                }
            }
        }
    }
}

// ---------------------------------------------------------------- copy (measurement aid)

template <int U, bool NT>
__global__ __launch_bounds__(kBlock) void copy_kernel(float* dst, const float* src, uint64_t n,
                                                       uint64_t n_tiles, uint32_t has_tail)
{
    constexpr uint64_t kTile = (uint64_t)U * 256;
    const uint32_t n_work_blocks = gridDim.x - has_tail;
    if (blockIdx.x >= n_work_blocks) {
        for (uint64_t e = n_tiles * kTile + threadIdx.x; e < n; e += kBlock) dst[e] = src[e];
        return;
    }
    const int lane = threadIdx.x & (kWave - 1);
    const uint64_t wave = (uint64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
    const uint64_t n_waves = (uint64_t)n_work_blocks * kWavesPerBlock;
    for (uint64_t tile = wave; tile < n_tiles; tile += n_waves) {
        const uint64_t e0 = tile * kTile + (uint64_t)lane * 4;
        f32x4 a[U];
#pragma unroll
        for (int j = 0; j < U; ++j) a[j] = ld4<true, NT>(src + e0 + j * 256);
#pragma unroll
        for (int j = 0; j < U; ++j) st4<true, NT>(dst + e0 + j * 256, a[j]);
    }
}

// ---------------------------------------------------------------- host side

// knobs (results never depend on them)
int g_unroll = 4;      // float4 loads per lane per array in flight: 1, 2 or 4
int g_wg_per_cu = 0;   // 0: one workgroup per 4 wave tiles; > 0: grid-stride with this many per CU
int g_nontemporal = 1;

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
    uint64_t n_tiles;
    uint32_t has_tail;
    uint32_t blocks;
};

// Work split of a flat vector of n elements in wave tiles of U*256.
FlatGrid flat_grid(uint64_t n, int U)
{
    FlatGrid fg;
    const uint64_t tile = (uint64_t)U * 256;
    fg.n_tiles = n / tile;
    fg.has_tail = (fg.n_tiles * tile < n) ? 1u : 0u;
    uint64_t work = (fg.n_tiles + kWavesPerBlock - 1) / kWavesPerBlock;
    if (g_wg_per_cu > 0) {
        const uint64_t cap = (uint64_t)compute_units() * (uint64_t)g_wg_per_cu;
        if (work > cap) work = cap;
    }
    // gridDim.x is 32-bit; 2^31 workgroups of 4 tiles cover far more than any HBM holds,
    // the grid-stride loop takes whatever is left.
    if (work > 0x7FFFFFF0ull) work = 0x7FFFFFF0ull;
    fg.blocks = (uint32_t)work + fg.has_tail;
    return fg;
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline bool aligned4(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 3u) == 0; }

inline int launch_status()
{
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? NKLQ_OK : (int)e;
}

template <int U, bool ALIGNED, bool ADD>
void launch_quant_flat_nt(const float* g, const float* rin, float* rout, uint32_t* c, uint64_t n,
                          float t, hipStream_t s)
{
    const FlatGrid fg = flat_grid(n, U);
    if (g_nontemporal)
        hipLaunchKernelGGL((quant_flat_kernel<U, ALIGNED, ADD, true>), dim3(fg.blocks), dim3(kBlock),
                           0, s, g, rin, rout, c, n, fg.n_tiles, fg.has_tail, t);
    else
        hipLaunchKernelGGL((quant_flat_kernel<U, ALIGNED, ADD, false>), dim3(fg.blocks),
                           dim3(kBlock), 0, s, g, rin, rout, c, n, fg.n_tiles, fg.has_tail, t);
}

template <int U>
void launch_quant_flat(const float* g, const float* rin, float* rout, uint32_t* c, uint64_t n,
                       float t, bool add, bool aligned, hipStream_t s)
{
    if (aligned) {
        if (add) launch_quant_flat_nt<U, true, true>(g, rin, rout, c, n, t, s);
        else launch_quant_flat_nt<U, true, false>(g, rin, rout, c, n, t, s);
    } else {
        if (add) launch_quant_flat_nt<U, false, true>(g, rin, rout, c, n, t, s);
        else launch_quant_flat_nt<U, false, false>(g, rin, rout, c, n, t, s);
    }
}

template <int U, bool OVERWRITE>
void launch_deq_flat(float* out, const PayloadPtrs& pl, int k, uint64_t n, float t, int accumulate,
                     hipStream_t s)
{
    const FlatGrid fg = flat_grid(n, U);
    const bool al = aligned16(out);
    const bool nt = g_nontemporal != 0;
#define NKLQ_DEQ(AL, NT)                                                                         \
    hipLaunchKernelGGL((deq_flat_kernel<U, AL, NT, OVERWRITE>), dim3(fg.blocks), dim3(kBlock), 0, \
                       s, out, pl, k, n, fg.n_tiles, fg.has_tail, t, accumulate)
    if (al && nt) NKLQ_DEQ(true, true);
    else if (al) NKLQ_DEQ(true, false);
    else if (nt) NKLQ_DEQ(false, true);
    else NKLQ_DEQ(false, false);
#undef NKLQ_DEQ
}

uint32_t grid_for_items(uint64_t items)
{
    uint64_t blocks = (items + kBlock - 1) / kBlock;
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
    int* slot = which == 0 ? &g_unroll : which == 1 ? &g_wg_per_cu : which == 2 ? &g_nontemporal : nullptr;
    if (!slot) return NKLQ_ERANGE;
    int prev = *slot;
    if (which == 0) prev *= 4;
    if (value < 0) return prev;
    if (which == 0) {
        if (value != 4 && value != 8 && value != 16) return NKLQ_ERANGE;
        *slot = value / 4;
    } else if (which == 1) {
        if (value > 4096) return NKLQ_ERANGE;
        *slot = value;
    } else {
        *slot = value ? 1 : 0;
    }
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
        switch (g_unroll) {
            case 1: launch_quant_flat<1>(g, r_in, r_out, c, total, thrd, add, al, s); break;
            case 2: launch_quant_flat<2>(g, r_in, r_out, c, total, thrd, add, al, s); break;
            default: launch_quant_flat<4>(g, r_in, r_out, c, total, thrd, add, al, s); break;
        }
        return launch_status();
    }
    const uint64_t m = n_rows / 16 + (n_rows % 16 ? 1 : 0);
    const bool vec = (n_cols % 4 == 0) && aligned16(g) && aligned16(r_out) && aligned16(c) &&
                     (!add || aligned16(r_in));
    if (vec) {
        const uint64_t items = m * (n_cols / 4);
        const uint32_t grid = grid_for_items(items);
        if (add)
            hipLaunchKernelGGL((quant_2d_kernel<4, true>), dim3(grid), dim3(kBlock), 0, s, g, r_in,
                               r_out, c, n_rows, n_cols, items, thrd);
        else
            hipLaunchKernelGGL((quant_2d_kernel<4, false>), dim3(grid), dim3(kBlock), 0, s, g, r_in,
                               r_out, c, n_rows, n_cols, items, thrd);
    } else {
        const uint64_t items = m * n_cols;
        const uint32_t grid = grid_for_items(items);
        if (add)
            hipLaunchKernelGGL((quant_2d_kernel<1, true>), dim3(grid), dim3(kBlock), 0, s, g, r_in,
                               r_out, c, n_rows, n_cols, items, thrd);
        else
            hipLaunchKernelGGL((quant_2d_kernel<1, false>), dim3(grid), dim3(kBlock), 0, s, g, r_in,
                               r_out, c, n_rows, n_cols, items, thrd);
    }
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
        PayloadPtrs pl = {};
        pl.p[0] = c;
        switch (g_unroll) {
            case 1: launch_deq_flat<1, true>(out, pl, 1, total, thrd, 0, s); break;
            case 2: launch_deq_flat<2, true>(out, pl, 1, total, thrd, 0, s); break;
            default: launch_deq_flat<4, true>(out, pl, 1, total, thrd, 0, s); break;
        }
        return launch_status();
    }
    const uint64_t m = n_rows / 16 + (n_rows % 16 ? 1 : 0);
    if ((n_cols % 4 == 0) && aligned16(out) && aligned16(c)) {
        const uint64_t items = m * (n_cols / 4);
        hipLaunchKernelGGL((deq_2d_kernel<4>), dim3(grid_for_items(items)), dim3(kBlock), 0, s, out,
                           c, n_rows, n_cols, items, thrd);
    } else {
        const uint64_t items = m * n_cols;
        hipLaunchKernelGGL((deq_2d_kernel<1>), dim3(grid_for_items(items)), dim3(kBlock), 0, s, out,
                           c, n_rows, n_cols, items, thrd);
    }
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
    int acc_flag = accumulate ? 1 : 0;
    for (int first = 0; first < k_payloads; first += NKLQ_MAX_PAYLOADS_PER_LAUNCH) {
        PayloadPtrs pl = {};
        int k = k_payloads - first;
        if (k > NKLQ_MAX_PAYLOADS_PER_LAUNCH) k = NKLQ_MAX_PAYLOADS_PER_LAUNCH;
        for (int p = 0; p < k; ++p) pl.p[p] = payloads[first + p];
        for (int p = k; p < NKLQ_MAX_PAYLOADS_PER_LAUNCH; ++p) pl.p[p] = payloads[first];
        switch (g_unroll) {
            case 1: launch_deq_flat<1, false>(acc, pl, k, n, thrd, acc_flag, s); break;
            case 2: launch_deq_flat<2, false>(acc, pl, k, n, thrd, acc_flag, s); break;
            default: launch_deq_flat<4, false>(acc, pl, k, n, thrd, acc_flag, s); break;
        }
        const int st = launch_status();
        if (st != NKLQ_OK) return st;
        acc_flag = 1;  // later launches continue the running sum held in acc
    }
    return NKLQ_OK;
}

int nklq_copy_f32(float* dst, const float* src, uint64_t n, void* stream)
{
    if (n == 0) return NKLQ_OK;
    if (!dst || !src) return NKLQ_ENULL;
    if (!aligned16(dst) || !aligned16(src)) return NKLQ_EALIGN;
    hipStream_t s = (hipStream_t)stream;
    const FlatGrid fg = flat_grid(n, 4);
    if (g_nontemporal)
        hipLaunchKernelGGL((copy_kernel<4, true>), dim3(fg.blocks), dim3(kBlock), 0, s, dst, src, n,
                           fg.n_tiles, fg.has_tail);
    else
        hipLaunchKernelGGL((copy_kernel<4, false>), dim3(fg.blocks), dim3(kBlock), 0, s, dst, src, n,
                           fg.n_tiles, fg.has_tail);
    return launch_status();
}

}  // extern "C"
