// Mixed INT4 / FP6-e3m2 weight-only GEMM for gfx950 (MI355X):  C[m,n] = A[m,k] . deq(B)[k,n] * s
//
// Replaces the device kernel and host dispatcher of liuchuan22/FP6-Marlin
// (fp6_marlin/fp6_marlin_cuda_kernel.cu:288-951).  Same packed operands, a different machine mapping:
//
//  * One wavefront (64 lanes) owns a 128-column tile (two 64-column groups of the packed layout) and a
//    contiguous range of k.  It streams the packed words with linear, fully coalesced 16-byte-per-lane
//    loads (1 KiB per k-block and tile), turns them through a wave-private LDS slab so that the
//    fragment owner's k-pair index becomes the high lane bits, dequantises in registers and feeds
//    v_mfma_f32_16x16x32_f16 with the *weights as the 16-row operand* (C^T = W^T A^T), so a single
//    MFMA covers 16 columns x 32 k for up to 16 rows of A.  No workgroup barrier in the main loop.
//  * A workgroup is four such waves splitting k; they are summed through LDS.  `ksplit` workgroups may
//    share a tile; each writes its fp32 partial tile to a per-device scratch, and the workgroup that
//    arrives last (one atomic counter per tile in `workspace`) sums the partials in a fixed order,
//    applies the scales and writes fp16 C.  Nobody spins, so there is nothing to deadlock on, and the
//    counters are zero again when the launch drains.
//  * INT4 and FP6 tiles are entries of one tile list handled by the same launch.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <mutex>

#include "fp6m.h"
#include "fp6m_layout.h"

namespace fp6m {

typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef uint32_t u4 __attribute__((ext_vector_type(4)));
typedef uint32_t u2 __attribute__((ext_vector_type(2)));

constexpr int kWaves = 4;
constexpr int kTileN = 128;          // columns per tile
constexpr int kRedStride = kTileN + 4;                       // floats per row of the reduction slab
constexpr size_t kScratchBytes = size_t(64) << 20;           // per-device partial-sum scratch
constexpr size_t kPackTempBytes = size_t(1) << 20;           // + the packer's flag and per-column maxima

struct GemmArgs {
    const uint16_t* A;
    const uint32_t* b_int4;   // INT4 words
    const uint32_t* b_fp6_2;  // FP6 2-bit plane
    const uint32_t* b_fp6_4;  // FP6 4-bit plane
    uint16_t* C;
    const uint16_t* s_int4;   // per-column (permuted order) or [k/128][n4] group scales
    const uint16_t* s_fp6;    // per-column (permuted order)
    float* scratch;
    int* counters;
    int m, n, k;
    int n4, qc;               // columns in the INT4 / FP6 region
    int tiles6;               // FP6 tiles come first in the tile list
    int tiles;                // all tiles
    int ksplit;               // workgroups per (tile, m-tile)
    // m <= 16 kernel: the FP6 and the INT4 region are covered by separate ranges of workgroups
    int ks6, ks4;             // k parts (workgroups) per tile group, per region
    int groups6, groups4;     // tile groups (WN adjacent tiles) per region
    // row mix (fp6m_mul_rows): rows [0, k4) of every column are INT4 with group scales, rows [k4, k) FP6.  The
    // k slices of a tile (parts x waves) are numbered INT4 first: slices [0, slices4) cover the INT4 rows.
    int k4, slices4;          // 0 = column mix
    // weight planes in the gfx950 order (fp6m_repack_gfx950): [tile][k-block][MFMA lane] instead of the reference's
    // [k-block][64-column group][fragment owner]
    int native;
    // optional epilogue work (fp6m_mul_fused); `fused` is set when any of the three is
    const int32_t* c_cols;    // column of C that packed column j goes to
    const uint16_t* bias;     // fp16 [n], indexed by C column
    const uint16_t* residual; // fp16 [m, n], same rows as C
    int fused;
#ifdef FP6M_TIMELINE
    unsigned long long* timeline;   // 8 realtime-clock stamps per workgroup (performance debugging builds only)
#endif
};

#ifdef FP6M_TIMELINE
#define FP6M_MARK(p, i)                                                                            \
    do {                                                                                           \
        if (__builtin_amdgcn_readfirstlane(threadIdx.x >> 6) == 0 && (p).timeline) /* uniform branch */ \
            (p).timeline[(size_t)(blockIdx.y * gridDim.x + blockIdx.x) * 8 + (i)] = __builtin_amdgcn_s_memrealtime(); \
    } while (0)
#else
#define FP6M_MARK(p, i) do { } while (0)
#endif

// ------------------------------------------------------------------------------------------------ bit tricks

__device__ __forceinline__ h2 as_h2(uint32_t v) { return __builtin_bit_cast(h2, v); }

__device__ __forceinline__ h8 join(h2 a, h2 b, h2 c, h2 d)
{
    h8 v;
    v[0] = a[0]; v[1] = a[1]; v[2] = b[0]; v[3] = b[1];
    v[4] = c[0]; v[5] = c[1]; v[6] = d[0]; v[7] = d[1];
    return v;
}

// Workgroup b of a 1-D grid runs on XCD b % 8.  Renumber so that every XCD sees a contiguous range of
// logical ids: workgroups that share a tile (adjacent logical ids) then share an L2.
__device__ __forceinline__ int xcd_contiguous_id(int b, int total)
{
    const int q = total >> 3, r = total & 7, x = b & 7;
    return x * q + (x < r ? x : r) + (b >> 3);
}

// Epilogue of fp6m_mul_fused for two adjacent packed columns of one row: C[row, c_cols[col]] =
// fp16(v + bias[c_cols[col]] + residual[row, c_cols[col]]), everything added in fp32 and rounded once.
// Map entries are clamped to the row so that a bad map cannot write outside C.
__device__ __forceinline__ void store_fused(const GemmArgs& p, size_t row, int col, float v0, float v1)
{
    int c0 = col, c1 = col + 1;
    if (p.c_cols) {
        c0 = p.c_cols[col];
        c1 = p.c_cols[col + 1];
        c0 = c0 < 0 ? 0 : (c0 >= p.n ? p.n - 1 : c0);
        c1 = c1 < 0 ? 0 : (c1 >= p.n ? p.n - 1 : c1);
    }
    if (p.bias) {
        v0 += (float)__builtin_bit_cast(_Float16, p.bias[c0]);
        v1 += (float)__builtin_bit_cast(_Float16, p.bias[c1]);
    }
    const size_t r = row * (size_t)p.n;
    if (p.residual) {
        v0 += (float)__builtin_bit_cast(_Float16, p.residual[r + c0]);
        v1 += (float)__builtin_bit_cast(_Float16, p.residual[r + c1]);
    }
    p.C[r + c0] = __builtin_bit_cast(uint16_t, (_Float16)v0);
    p.C[r + c1] = __builtin_bit_cast(uint16_t, (_Float16)v1);
}

// ------------------------------------------------------------------------------------------------ tile bookkeeping

struct TileInfo {
    int tile, part, mtile;   // tile in the [FP6 | INT4] tile list, k partner index, m-tile
    bool fp6;
    int tcol;                // tile index inside its region
    int region_n;            // columns of the region
    int col0;                // first column of the tile in C
    int a_step0;             // k step of A that step 0 of the wave's weight segment multiplies (row mix: k4 / 32)
};

// Row mix: slice `sl` of the `nsl` slices of a tile -> its segment (ti.fp6, ti.a_step0) and its steps there.
__device__ __forceinline__ void row_mix_slice(const GemmArgs& p, int sl, int nsl, TileInfo& ti, int& begin, int& end)
{
    ti.fp6 = sl >= p.slices4;
    if (!ti.fp6) {
        const int units = p.k4 / 128;
        begin = (int)((long long)units * sl / p.slices4) * 4;
        end = (int)((long long)units * (sl + 1) / p.slices4) * 4;
        ti.a_step0 = 0;
    } else {
        const int units = (p.k - p.k4) / 64, s6 = sl - p.slices4, n6 = nsl - p.slices4;
        begin = (int)((long long)units * s6 / n6) * 2;
        end = (int)((long long)units * (s6 + 1) / n6) * 2;
        ti.a_step0 = p.k4 / 32;
    }
}

// Where a tile's packed words sit.  Reference order: a k-block (16 rows of k) is one row of region_n * 8 bytes
// (4-bit plane / INT4; half that for the 2-bit plane) in which the tile owns 1 KiB (512 B), lane granules in
// fragment-owner order.  gfx950 order: the tile's k-blocks follow each other, lane granules in MFMA lane order.
struct PlaneGeometry {
    size_t row4, row2;       // bytes from one k-block of the tile to the next
    size_t tile4, tile2;     // byte offset of the tile's first k-block
};
__device__ __forceinline__ PlaneGeometry plane_geometry(const GemmArgs& p, const TileInfo& ti)
{
    PlaneGeometry g;
    if (p.native) {
        const size_t kblocks = (size_t)(p.k4 ? (ti.fp6 ? p.k - p.k4 : p.k4) : p.k) / 16;
        g.row4 = 1024;
        g.row2 = 512;
        g.tile4 = (size_t)ti.tcol * kblocks * 1024;
        g.tile2 = (size_t)ti.tcol * kblocks * 512;
    } else {
        g.row4 = (size_t)ti.region_n * 8;
        g.row2 = (size_t)ti.region_n * 4;
        g.tile4 = (size_t)ti.tcol * 1024;
        g.tile2 = (size_t)ti.tcol * 512;
    }
    return g;
}

__device__ __forceinline__ TileInfo locate_tile(const GemmArgs& p)
{
    TileInfo t;
    const int logical = xcd_contiguous_id(blockIdx.x, gridDim.x);
    t.tile = logical / p.ksplit;
    t.part = logical - t.tile * p.ksplit;
    t.mtile = blockIdx.y;
    t.fp6 = t.tile < p.tiles6;
    t.tcol = t.fp6 ? t.tile : t.tile - p.tiles6;
    t.region_n = t.fp6 ? p.qc : p.n4;
    t.col0 = (t.fp6 ? p.n4 : 0) + t.tcol * kTileN;
    t.a_step0 = 0;
    return t;
}

// k range of one wave in steps of 32 (two k-blocks).  Units of two steps (four with group scales) keep
// every wave's step count even and group-aligned.
template <bool G128, int WK = kWaves>
__device__ __forceinline__ void wave_k_range(const GemmArgs& p, int part, int wave, int& begin, int& end)
{
    constexpr int unit_steps = G128 ? 4 : 2;
    const int units = p.k / (32 * unit_steps);
    const int nwaves = p.ksplit * WK;
    const int wv = part * WK + wave;
    begin = (int)((long long)units * wv / nwaves) * unit_steps;
    end = (int)((long long)units * (wv + 1) / nwaves) * unit_steps;
}

// ------------------------------------------------------------------------------------------------ m <= 16: LDS-ring kernel
//
// Every wave keeps a private ring of DEPTH slots in LDS.  A slot is one k step (32 rows of k) of its
// tile: the packed words (2 x 1 KiB 4-bit/INT4, + 2 x 512 B FP6 2-bit) and the 16 x 32 fp16 activation
// block (1 KiB).  Slots are filled by direct-to-LDS global loads (no VGPR staging): lane L's data lands
// at slot + 16 L, so the *global* granule each lane fetches is permuted (inside aligned 64-byte quads,
// which keeps the loads coalesced) to obtain a layout that the permuted reads hit without bank
// conflicts.  The loads of step s + DEPTH - 1 are issued before step s is consumed; `s_waitcnt vmcnt`
// with a constant count is the only synchronisation in the loop.  LDS reads are inline asm so that
// the compiler does not serialise them behind every outstanding direct-to-LDS load.

#define FP6M_AS1 __attribute__((address_space(1)))
#define FP6M_AS3 __attribute__((address_space(3)))

__device__ __forceinline__ void dma16(const void* gsrc, unsigned char* lds_dst)
{
    __builtin_amdgcn_global_load_lds((const FP6M_AS1 void*)gsrc, (FP6M_AS3 void*)lds_dst, 16, 0, 0);
}
// Same, with the non-temporal hint: for the packed words, which are read exactly once.
__device__ __forceinline__ void dma16_stream(const void* gsrc, unsigned char* lds_dst)
{
    __builtin_amdgcn_global_load_lds((const FP6M_AS1 void*)gsrc, (FP6M_AS3 void*)lds_dst, 16, 0, 2);
}
__device__ __forceinline__ void dma4(const void* gsrc, unsigned char* lds_dst)
{
    __builtin_amdgcn_global_load_lds((const FP6M_AS1 void*)gsrc, (FP6M_AS3 void*)lds_dst, 4, 0, 0);
}
__device__ __forceinline__ uint32_t lds_addr(const void* ptr) { return (uint32_t)(uintptr_t)(const FP6M_AS3 void*)ptr; }

// Direct-to-LDS loads in their scalar-base form: global address = sbase + voff + OFF, LDS address =
// M0 + OFF + 16 * lane.  The immediate moves both sides, so loads whose LDS targets lie within 4 KiB of
// each other share one M0 value (the global side is compensated in voff or sbase) and no vector address
// arithmetic is left in the loop.  One wait state separates the M0 write from its first use.
// The "s" operands below must live in SGPRs: values are made wave-uniform explicitly where they are
// created (a no-op when the compiler already knows it).
__device__ __forceinline__ uint32_t uniform32(uint32_t v) { return __builtin_amdgcn_readfirstlane(v); }
template <typename T>
__device__ __forceinline__ const T* uniform_ptr(const T* ptr)
{
    const uint64_t v = reinterpret_cast<uint64_t>(ptr);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return reinterpret_cast<const T*>(((uint64_t)hi << 32) | lo);
}
__device__ __forceinline__ void set_m0(uint32_t lds_base)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0" : : "s"(lds_base) : "memory");
}
template <int OFF, bool STREAM>
__device__ __forceinline__ void dma16_m0(const void* sbase, uint32_t voff)
{
    static_assert(OFF >= 0 && OFF < 4096, "13-bit signed immediate");
    if constexpr (STREAM)
        asm volatile("global_load_lds_dwordx4 %0, %1 offset:%2 nt" : : "v"(voff), "s"(sbase), "n"(OFF) : "memory");
    else
        asm volatile("global_load_lds_dwordx4 %0, %1 offset:%2" : : "v"(voff), "s"(sbase), "n"(OFF) : "memory");
}
__device__ __forceinline__ void dma4_m0(const void* sbase, uint32_t voff)
{
    asm volatile("global_load_lds_dword %0, %1" : : "v"(voff), "s"(sbase) : "memory");
}
template <int MB, int A_OFF, int I = 0>
__device__ __forceinline__ void dma_a_blocks(uint32_t slot_lds, const void* sbase_a, const uint32_t (&voff)[MB])
{
    if constexpr (I < MB) {
        constexpr int lds_off = A_OFF + 1024 * I;
        if constexpr (lds_off % 4096 == 0) set_m0(slot_lds + lds_off);
        dma16_m0<lds_off % 4096, false>(sbase_a, voff[I]);
        dma_a_blocks<MB, A_OFF, I + 1>(slot_lds, sbase_a, voff);
    }
}

// s_waitcnt immediate that waits for vmcnt <= n only (gfx9 encoding: vmcnt = [3:0] and [15:14]).
constexpr int vmcnt_only(int n) { return (n & 15) | ((n >> 4) << 14) | (7 << 4) | (15 << 8); }

// A value the optimiser must treat as an unknown VGPR: keeps bit masks in registers so that
// (x & mask) | magic selects the three-operand v_and_or_b32 (VOP3 cannot take literals on gfx9).
__device__ __forceinline__ uint32_t vgpr_const(uint32_t v)
{
    asm volatile("" : "+v"(v));
    return v;
}

struct DequantConsts {
    uint32_t lo, hi, ex;          // INT4 nibble masks and the 1024.0 magic
    uint32_t top2, exp_man;       // FP6 plane mask and the s00eeemm field mask
};

__device__ __forceinline__ void dequant_int4_fast(uint32_t q, const DequantConsts& k, h2 (&r)[4])
{
    const h2 bias_lo = {(_Float16)1032.0f, (_Float16)1032.0f};
    const h2 mul_hi = {(_Float16)0.0625f, (_Float16)0.0625f};
    const h2 bias_hi = {(_Float16)-72.0f, (_Float16)-72.0f};
    const uint32_t q8 = q >> 8;
    r[0] = as_h2((q & k.lo) | k.ex) - bias_lo;
    r[1] = __builtin_elementwise_fma(as_h2((q & k.hi) | k.ex), mul_hi, bias_hi);
    r[2] = as_h2((q8 & k.lo) | k.ex) - bias_lo;
    r[3] = __builtin_elementwise_fma(as_h2((q8 & k.hi) | k.ex), mul_hi, bias_hi);
}

typedef short s2 __attribute__((ext_vector_type(2)));

// FP6 without the multiply by 4096 (the MFMA keeps fp16 sub-normal inputs; 4096 goes into the epilogue
// scale).  p holds four bytes `s eee mm xx`, MSB first e1 e3 e0 e2; an arithmetic shift right by two of
// each 16-bit half moves eee mm under the sign and the mask 0x9f00 clears the sign copies and the low byte.
__device__ __forceinline__ void dequant_fp6_fast(uint32_t q2, uint32_t q4, const DequantConsts& k, h2 (&r)[4])
{
    const s2 two = {2, 2};
#pragma unroll
    for (int half = 0; half < 2; half++) {
        const uint32_t lo = half == 0 ? (q4 >> 2) : (q4 << 2);
        const uint32_t hi = half == 0 ? q2 : (q2 << 2);
        const uint32_t p = (hi & k.top2) | (lo & ~k.top2);                       // v_bfi_b32
        const uint32_t p8 = p << 8;
        r[2 * half + 0] = as_h2(__builtin_bit_cast(uint32_t, __builtin_bit_cast(s2, p) >> two) & k.exp_man);
        r[2 * half + 1] = as_h2(__builtin_bit_cast(uint32_t, __builtin_bit_cast(s2, p8) >> two) & k.exp_man);
    }
}

// s_waitcnt immediate that waits for lgkmcnt <= n only.
constexpr int lgkmcnt_only(int n) { return 15 | (3 << 14) | (7 << 4) | ((n & 15) << 8); }

struct StepRegs {
    u4 q0, q1;          // 4-bit plane / INT4 words of the two k-blocks
    u2 t0, t1;          // FP6 2-bit plane
    uint32_t a[4];      // activations in MFMA operand order
};

// AROWS = rows of A a slot holds (4 or 16): 64 bytes per row and step.
template <bool FP6, bool G128, int DEPTH, int AROWS>
__device__ __forceinline__ void stream_tile(const GemmArgs& p, const TileInfo& ti, unsigned char* ring,
                                            int step_begin, int step_end, f4 (&acc)[1][8])
{
    static_assert(DEPTH >= 3, "needs two steps of look-ahead");
    constexpr bool kGroup = G128 && !FP6;                 // group scales apply to INT4 tiles only
    constexpr int kAOff = FP6 ? 3072 : 2048;
    constexpr int kSlot = kAOff + AROWS * 64;
    constexpr int kOps = FP6 ? 4 : 3;                     // direct-to-LDS loads per step
    constexpr int kReads = FP6 ? 8 : 6;                   // LDS reads per step
    constexpr int kUnroll = kGroup ? 4 : 2;               // steps per loop trip (step counts are multiples of it)
    const int lane = threadIdx.x & 63;
    const int i = lane >> 4, c = lane & 15, sigma = c >> 3, l = c & 7;

    DequantConsts kc;
    kc.lo = vgpr_const(0x000f000fu);
    kc.hi = vgpr_const(0x00f000f0u);
    kc.ex = vgpr_const(0x64006400u);
    kc.top2 = vgpr_const(0xc0c0c0c0u);
    kc.exp_man = vgpr_const(0x9f009f00u);

    // ---- fetch side (lane = position in the slot).  Uniform 64-bit bases advance on the scalar unit;
    // each lane only contributes a constant 32-bit offset.
    const uint32_t v4 = (lane ^ ((lane >> 4) & 3)) * 16;
    const PlaneGeometry geo = plane_geometry(p, ti);
    const size_t row4 = geo.row4, row2 = geo.row2;
    const unsigned char* base4 = reinterpret_cast<const unsigned char*>(FP6 ? p.b_fp6_4 : p.b_int4) +
                                 geo.tile4 + (size_t)(2 * step_begin) * row4;
    const int lg = lane & 31;
    const uint32_t v2 = (uint32_t)((lane >> 5) * row2) + (lg ^ (lg >> 4)) * 16;
    const unsigned char* base2 = reinterpret_cast<const unsigned char*>(p.b_fp6_2) + geo.tile2 +
                                 (size_t)(2 * step_begin) * row2;
    const int a_m = lane >> 2;
    const bool a_active = a_m < AROWS && ti.mtile * 16 + a_m < p.m;
    const uint32_t va = (uint32_t)(a_active ? a_m : 0) * (uint32_t)p.k * 2 + 16 * ((lane & 3) ^ ((a_m >> 2) & 3));
    const unsigned char* base_a = reinterpret_cast<const unsigned char*>(p.A + (size_t)ti.mtile * 16 * p.k) +
                                  (size_t)(ti.a_step0 + step_begin) * 64;
    const unsigned char* base_gs = reinterpret_cast<const unsigned char*>(p.s_int4 + (size_t)ti.tcol * kTileN);
    const uint32_t vgs = 4 * lane;
    constexpr int kScaleMask = DEPTH <= 5 ? 1 : 3;        // 256-byte slabs of group scales: 2 suffice up to depth 5
    unsigned char* gs_ring = ring + DEPTH * kSlot;

    int issued = step_begin;                              // next step to fetch (clamped at the last one)
    const int last = step_end - 1;
    auto issue = [&](int slot) {
        unsigned char* dst = ring + slot * kSlot;
        dma16_stream(base4 + v4, dst);
        dma16_stream(base4 + row4 + v4, dst + 1024);
        if (FP6) dma16_stream(base2 + v2, dst + 2048);
        if (a_active) dma16(base_a + va, dst + kAOff);
        if (kGroup && (issued & 3) == 0)
            dma4(base_gs + (size_t)(issued >> 2) * p.n4 * 2 + vgs, gs_ring + ((issued >> 2) & kScaleMask) * 256);
        if (issued < last) {                              // uniform: pointers move on the scalar unit
            issued++;
            base4 += 2 * row4;
            base2 += 2 * row2;
            base_a += 64;
        }
    };

    // ---- read side (lane = MFMA identity)
    const int owner = p.native ? lane : 32 * sigma + 4 * l + i;   // whose granule of the k-block this lane needs
    const uint32_t ring_lds = lds_addr(ring);
    const uint32_t rd4 = ring_lds + (owner ^ ((owner >> 4) & 3)) * 16;
    const int gr2 = owner >> 1;
    const uint32_t rd2 = ring_lds + 2048 + (gr2 ^ (gr2 >> 4)) * 16 + (owner & 1) * 8;
    const int ar = c & (AROWS - 1);                       // rows beyond AROWS re-read a valid row; their sums are never stored
    uint32_t rda[4];
#pragma unroll
    for (int d = 0; d < 4; d++) rda[d] = ring_lds + kAOff + (4 * ar + (d ^ ((ar >> 2) & 3))) * 16 + 4 * i;
    const int q = i;                                      // result side: quarter of the column slots
    const uint32_t rdgs = lds_addr(gs_ring) + (64 * (q >> 1) + 4 * (q & 1)) * 2;

    // kReads LDS reads of one step, not waited for.
    auto fetch = [&](StepRegs& r, int slot) {
        const uint32_t so = slot * kSlot;
        if (FP6) {
            asm volatile(
                "ds_read_b128 %0, %4\n\tds_read_b128 %1, %4 offset:1024\n\t"
                "ds_read_b64 %2, %5\n\tds_read_b64 %3, %5 offset:512"
                : "=&v"(r.q0), "=&v"(r.q1), "=&v"(r.t0), "=&v"(r.t1) : "v"(rd4 + so), "v"(rd2 + so) : "memory");
        } else {
            asm volatile("ds_read_b128 %0, %2\n\tds_read_b128 %1, %2 offset:1024"
                         : "=&v"(r.q0), "=&v"(r.q1) : "v"(rd4 + so) : "memory");
        }
        asm volatile("ds_read_b32 %0, %4\n\tds_read_b32 %1, %5\n\tds_read_b32 %2, %6\n\tds_read_b32 %3, %7"
                     : "=&v"(r.a[0]), "=&v"(r.a[1]), "=&v"(r.a[2]), "=&v"(r.a[3])
                     : "v"(rda[0] + so), "v"(rda[1] + so), "v"(rda[2] + so), "v"(rda[3] + so) : "memory");
    };
    // After the counter wait, the registers of `r` hold their data: make every later use depend on it.
    auto settle = [&](StepRegs& r) {
        asm volatile("" : "+v"(r.q0), "+v"(r.q1), "+v"(r.a[0]), "+v"(r.a[1]), "+v"(r.a[2]), "+v"(r.a[3]));
        if (FP6) asm volatile("" : "+v"(r.t0), "+v"(r.t1));
    };
    auto compute = [&](const StepRegs& r, f4 (&dst)[8], bool fresh) {
        const h8 av = __builtin_bit_cast(h8, u4{r.a[0], r.a[1], r.a[2], r.a[3]});
        const f4 zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < 4; j++) {
            h2 r0[4], r1[4];
            if (FP6) {
                dequant_fp6_fast(r.t0[j >> 1] << (4 * (j & 1)), r.q0[j], kc, r0);
                dequant_fp6_fast(r.t1[j >> 1] << (4 * (j & 1)), r.q1[j], kc, r1);
            } else {
                dequant_int4_fast(r.q0[j], kc, r0);
                dequant_int4_fast(r.q1[j], kc, r1);
            }
            const h8 w_lo = join(r0[0], r0[1], r1[0], r1[1]);  // columns 16j + l
            const h8 w_hi = join(r0[2], r0[3], r1[2], r1[3]);  // columns 16j + 8 + l
            dst[2 * j + 0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(w_lo, av, fresh ? zero : dst[2 * j + 0], 0, 0, 0);
            dst[2 * j + 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(w_hi, av, fresh ? zero : dst[2 * j + 1], 0, 0, 0);
        }
    };

    // Pipeline: while step s is being computed, the LDS reads of step s+1 are in flight and the
    // direct-to-LDS loads of steps s+2 .. s+DEPTH-1 are outstanding.
    int slot_in = 0;
#pragma unroll 1
    for (int d = 0; d < DEPTH - 1; d++) {
        issue(slot_in);
        slot_in = slot_in + 1 == DEPTH ? 0 : slot_in + 1;
    }
    StepRegs regs[2];
    __builtin_amdgcn_s_waitcnt(vmcnt_only(kOps * (DEPTH - 2)));
    FP6M_MARK(p, 1);
    fetch(regs[0], 0);
    int slot_rd = 1;                                      // slot of the step whose LDS reads come next
    f4 grp[8];
#pragma unroll 1
    for (int s = step_begin; s < step_end; s += kUnroll) {
#pragma unroll
        for (int u = 0; u < kUnroll; u++) {
            issue(slot_in);
            slot_in = slot_in + 1 == DEPTH ? 0 : slot_in + 1;
            __builtin_amdgcn_s_waitcnt(vmcnt_only(kOps * (DEPTH - 2)));   // step s+u+1 has landed
            fetch(regs[(u + 1) & 1], slot_rd);
            slot_rd = slot_rd + 1 == DEPTH ? 0 : slot_rd + 1;
            __builtin_amdgcn_s_waitcnt(lgkmcnt_only(kReads));             // reads of step s+u (older) are done
            settle(regs[u & 1]);
            if (kGroup)
                compute(regs[u & 1], grp, u == 0);
            else
                compute(regs[u & 1], acc[0], false);
        }
        if (kGroup) {
            // end of a 128-row group: fold it into the running sum with its scales (fp32)
            const uint32_t ga = rdgs + ((s >> 2) & kScaleMask) * 256;
            u2 sv[8];
            asm volatile(
                "ds_read_b64 %0, %8\n\tds_read_b64 %1, %8 offset:16\n\tds_read_b64 %2, %8 offset:32\n\t"
                "ds_read_b64 %3, %8 offset:48\n\tds_read_b64 %4, %8 offset:64\n\tds_read_b64 %5, %8 offset:80\n\t"
                "ds_read_b64 %6, %8 offset:96\n\tds_read_b64 %7, %8 offset:112\n\ts_waitcnt lgkmcnt(0)"
                : "=&v"(sv[0]), "=&v"(sv[1]), "=&v"(sv[2]), "=&v"(sv[3]), "=&v"(sv[4]), "=&v"(sv[5]), "=&v"(sv[6]),
                  "=&v"(sv[7])
                : "v"(ga) : "memory");
            settle(regs[0]);                              // lgkmcnt(0) also completed the look-ahead reads
#pragma unroll
            for (int t = 0; t < 8; t++) {
                const h2 lo = as_h2(sv[t][0]), hi = as_h2(sv[t][1]);
                acc[0][t][0] += (float)lo[0] * grp[t][0];
                acc[0][t][1] += (float)lo[1] * grp[t][1];
                acc[0][t][2] += (float)hi[0] * grp[t][2];
                acc[0][t][3] += (float)hi[1] * grp[t][3];
            }
        }
    }
    // Redundant tail prefetches and look-ahead reads may still be in flight; the epilogue reuses the ring.
    __builtin_amdgcn_s_waitcnt(vmcnt_only(0) & lgkmcnt_only(0));
    settle(regs[0]);
    if (FP6) {
#pragma unroll
        for (int t = 0; t < 8; t++) acc[0][t] *= 4096.0f;  // the deferred e3m2 exponent re-bias
    }
}

// LDS per wave: the larger of an INT4 ring (D4 slots + the group-scale slabs) and an FP6 ring (D6
// slots), and at least the 16 x 128 fp32 row slab of the epilogue.
constexpr int scale_slab_bytes(int depth) { return depth <= 5 ? 512 : 1024; }
constexpr int max3(int a, int b, int c) { return a > b ? (a > c ? a : c) : (b > c ? b : c); }
constexpr int wave_lds_bytes(int d4, int d6, int arows)
{
    return max3(d4 * (2048 + arows * 64) + scale_slab_bytes(d4), d6 * (3072 + arows * 64), 16 * kRedStride * 4);
}

// The m <= 16 kernel.
//
// A workgroup is WN x WK waves: WN adjacent 128-column tiles (one per wave column, so the workgroup
// reads WN KiB contiguous runs of every k-block row) times WK consecutive slices of the workgroup's
// k range.  Waves never synchronise in the main loop.  Epilogue: every wave turns its MFMA fragments
// into fp32 rows in its own drained ring, one barrier, then wave (wn, wk) sums rows wk, wk+WK, ... of
// tile wn over the WK slices (fixed order) with lane L owning columns 2L, 2L+1.  With one k part per
// tile group it scales and writes C; otherwise it publishes the rows with agent-scope stores, the
// workgroup bumps the group's counter, and the workgroup that arrives last sums all parts in part order.
template <int WN, int WK>
__device__ __forceinline__ void wg_finish(const GemmArgs& p, const TileInfo& ti, bool tile_valid, int wn, int wk,
                                          int ks, int slot_base, int* counter, f4 (&acc)[1][8],
                                          bool per_column_scale, unsigned char* smem, int wave_lds, int* flag,
                                          int first_fp6 = WK)
{
    // first_fp6: row mix only -- k slices first_fp6 .. WK-1 of this workgroup hold FP6 rows, whose sums take the
    // FP6 column scale here (the INT4 slices are already scaled by their group scales)
    constexpr int RMAX = (16 + WK - 1) / WK;                             // rows one wave finishes
    constexpr int PCHUNK = 32 / RMAX;                                    // parts whose loads are in flight together
    typedef float f2 __attribute__((ext_vector_type(2)));
    const int lane = threadIdx.x & 63;
    const int c = lane & 15, q = lane >> 4;
    const int wave = wk * WN + wn;
    if (tile_valid) {
        float* mine = reinterpret_cast<float*>(smem + wave * wave_lds) + c * kRedStride + 64 * (q >> 1) + 4 * (q & 1);
#pragma unroll
        for (int t = 0; t < 8; t++) *reinterpret_cast<f4*>(mine + 16 * (t >> 1) + 8 * (t & 1)) = acc[0][t];
    }
    __syncthreads();
    FP6M_MARK(p, 3);

    const int nrows = p.m < 16 ? p.m : 16;
    float s0 = 1.0f, s1 = 1.0f;
    if (tile_valid && per_column_scale) {
        const uint16_t* sp = ti.fp6 ? p.s_fp6 : p.s_int4;
        const int nr = ti.tcol * kTileN + 2 * lane;                      // even column inside the region
        const h2 sv = *reinterpret_cast<const h2*>(sp + (nr & ~31) + scale_slot(nr & 31));
        s0 = (float)sv[0];
        s1 = (float)sv[1];
    }
    float x0 = 1.0f, x1 = 1.0f;                                          // FP6 column scales of a row mix
    if (tile_valid && first_fp6 < WK) {
        const int nr = ti.tcol * kTileN + 2 * lane;
        const h2 sv = *reinterpret_cast<const h2*>(p.s_fp6 + (nr & ~31) + scale_slot(nr & 31));
        x0 = (float)sv[0];
        x1 = (float)sv[1];
    }
    uint16_t* c_out = p.C + ti.col0 + 2 * lane;
    auto store_row = [&](int m, float v0, float v1) {
        if (p.fused) {
            store_fused(p, (size_t)m, ti.col0 + 2 * lane, v0 * s0, v1 * s1);
            return;
        }
        h2 o = {(_Float16)(v0 * s0), (_Float16)(v1 * s1)};
        *reinterpret_cast<h2*>(c_out + (size_t)m * p.n) = o;
    };

    // Sum of the WK slices of my rows.
    float v0[RMAX], v1[RMAX];
#pragma unroll
    for (int r = 0; r < RMAX; r++) {
        v0[r] = 0.f;
        v1[r] = 0.f;
        const int m = wk + r * WK;
        if (tile_valid && m < nrows) {
#pragma unroll
            for (int j = 0; j < WK; j++) {
                const f2 v = *reinterpret_cast<const f2*>(reinterpret_cast<const float*>(smem + (j * WN + wn) * wave_lds) +
                                                          m * kRedStride + 2 * lane);
                v0[r] += j >= first_fp6 ? v[0] * x0 : v[0];
                v1[r] += j >= first_fp6 ? v[1] * x1 : v[1];
            }
        }
    }
    if (ks == 1) {
#pragma unroll
        for (int r = 0; r < RMAX; r++)
            if (tile_valid && wk + r * WK < nrows) store_row(wk + r * WK, v0[r], v1[r]);
        return;
    }

    // Publish.  A slot holds [WN tiles][16 rows][128 columns] fp32; 8-byte agent-scope accesses.
    constexpr size_t kSlotU64 = (size_t)WN * 16 * kTileN / 2;
    unsigned long long* slot0 = reinterpret_cast<unsigned long long*>(p.scratch) + (size_t)slot_base * kSlotU64 +
                                (size_t)wn * (16 * kTileN / 2) + lane;
    unsigned long long* my = slot0 + (size_t)ti.part * kSlotU64;
#pragma unroll
    for (int r = 0; r < RMAX; r++) {
        const int m = wk + r * WK;
        if (tile_valid && m < nrows) {
            const f2 v = {v0[r], v1[r]};
            __hip_atomic_store(my + m * (kTileN / 2), __builtin_bit_cast(unsigned long long, v), __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");               // my stores have completed
    __syncthreads();
    FP6M_MARK(p, 4);
    if (threadIdx.x == 0) {
        const int seen = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        *flag = (seen == ks - 1);
    }
    __syncthreads();
    FP6M_MARK(p, 5);
    if (!*flag) return;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
#pragma unroll
    for (int r = 0; r < RMAX; r++) {
        v0[r] = 0.f;
        v1[r] = 0.f;
    }
    for (int pp = 0; pp < ks; pp += PCHUNK) {
        unsigned long long t[PCHUNK][RMAX];
#pragma unroll
        for (int u = 0; u < PCHUNK; u++)
#pragma unroll
            for (int r = 0; r < RMAX; r++) {
                const int m = wk + r * WK;
                t[u][r] = 0;
                if (tile_valid && m < nrows && pp + u < ks)
                    t[u][r] = __hip_atomic_load(slot0 + (size_t)(pp + u) * kSlotU64 + m * (kTileN / 2), __ATOMIC_RELAXED,
                                                __HIP_MEMORY_SCOPE_AGENT);
            }
#pragma unroll
        for (int u = 0; u < PCHUNK; u++)
#pragma unroll
            for (int r = 0; r < RMAX; r++) {
                const f2 v = __builtin_bit_cast(f2, t[u][r]);
                v0[r] += v[0];
                v1[r] += v[1];
            }
    }
#pragma unroll
    for (int r = 0; r < RMAX; r++)
        if (tile_valid && wk + r * WK < nrows) store_row(wk + r * WK, v0[r], v1[r]);
    FP6M_MARK(p, 6);
    if (threadIdx.x == 0) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <bool G128, int AROWS, int WN, int WK, int D4, int D6>
// second launch-bound argument = waves per SIMD the register budget must allow (HIP semantics)
__global__ __launch_bounds__(64 * WN * WK, 3) void gemm_m16_kernel(const GemmArgs p)
{
    constexpr int NW = WN * WK;
    constexpr int kWaveLds = wave_lds_bytes(D4, D6, AROWS);
    __shared__ __attribute__((aligned(16))) unsigned char smem[NW * kWaveLds + 16];

    FP6M_MARK(p, 0);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // scalar: addresses stay on the SALU
    const int wn = wave % WN, wk = wave / WN;
    const int logical = xcd_contiguous_id(blockIdx.x, gridDim.x);
    const int wgs6 = p.groups6 * p.ks6;                                  // the FP6 region's workgroups come first
    TileInfo ti;
    ti.fp6 = logical < wgs6;
    const int local = ti.fp6 ? logical : logical - wgs6;
    const int groups = ti.fp6 ? p.groups6 : p.groups4;
    const int ks = ti.fp6 ? p.ks6 : p.ks4;
    ti.part = local / groups;                                            // part-major: neighbours share k, adjoin in n
    const int group = local - ti.part * groups;
    ti.tcol = group * WN + wn;
    ti.region_n = ti.fp6 ? p.qc : p.n4;
    const bool tile_valid = ti.tcol * kTileN < ti.region_n;
    ti.tile = ti.fp6 ? ti.tcol : p.tiles6 + ti.tcol;
    ti.mtile = 0;
    ti.col0 = (ti.fp6 ? p.n4 : 0) + ti.tcol * kTileN;

    constexpr int unit_steps = G128 ? 4 : 2;
    const int units = p.k / (32 * unit_steps);
    const int kp = ti.part * WK + wk, kparts = ks * WK;
    int step_begin = (int)((long long)units * kp / kparts) * unit_steps;
    int step_end = (int)((long long)units * (kp + 1) / kparts) * unit_steps;
    ti.a_step0 = 0;
    const bool region6 = ti.fp6;                                         // the workgroup's column region
    if (p.k4) row_mix_slice(p, kp, kparts, ti, step_begin, step_end);    // per wave: INT4 or FP6 rows of the tile

    f4 acc[1][8];
#pragma unroll
    for (int t = 0; t < 8; t++) acc[0][t] = f4{0.f, 0.f, 0.f, 0.f};
    unsigned char* ring = smem + wave * kWaveLds;
    if (tile_valid && step_begin < step_end) {
        if (ti.fp6)
            stream_tile<true, G128, D6, AROWS>(p, ti, ring, step_begin, step_end, acc);
        else
            stream_tile<false, G128, D4, AROWS>(p, ti, ring, step_begin, step_end, acc);
    }
    FP6M_MARK(p, 2);
    // scratch slots: FP6 groups first (groups6 * ks6 slots), then INT4 groups; counters likewise
    const int slot_base = region6 ? group * p.ks6 : p.groups6 * p.ks6 + group * p.ks4;
    int* counter = p.counters + (region6 ? group : p.groups6 + group);
    wg_finish<WN, WK>(p, ti, tile_valid, wn, wk, ks, slot_base, counter, acc, !p.k4 && (ti.fp6 || !G128), smem, kWaveLds,
                      reinterpret_cast<int*>(smem + NW * kWaveLds), p.k4 ? p.slices4 - ti.part * WK : WK);
    FP6M_MARK(p, 7);
}

// ------------------------------------------------------------------------------------------------ 16 < m: ring kernel with MB row blocks
//
// Same ring and lane routing as the m <= 16 kernel, but a slot carries MB blocks of 16 rows of A (1 KiB
// each) and every dequantised weight fragment feeds 2*MB MFMAs, so the packed words are read once per
// 16*MB rows.  A workgroup is one tile x four k slices; blockIdx.y walks the row tiles.  Group scales are
// applied to the dequantised weights (fp16) because per-group fp32 accumulators would need MB*32 more
// registers.  Rows beyond m are clamped to the last row on the fetch side (every lane always loads, so
// the number of direct-to-LDS loads per step is constant) and never stored.

struct WeightRegs {
    u4 q0, q1;
};

template <int N>
struct Int {
    static constexpr int value = N;
};

template <int OFF>
__device__ __forceinline__ void lds_read_a4(uint32_t (&a)[4], const uint32_t (&addr)[4])
{
    asm volatile(
        "ds_read_b32 %0, %4 offset:%8\n\tds_read_b32 %1, %5 offset:%8\n\t"
        "ds_read_b32 %2, %6 offset:%8\n\tds_read_b32 %3, %7 offset:%8"
        : "=&v"(a[0]), "=&v"(a[1]), "=&v"(a[2]), "=&v"(a[3])
        : "v"(addr[0]), "v"(addr[1]), "v"(addr[2]), "v"(addr[3]), "n"(OFF) : "memory");
}

// acc += w (16 columns x 32 k) * a (16 rows x 32 k), in place.  Written as asm so that the accumulator
// stays in one VGPR quad for the whole loop (the builtin let the allocator rotate the accumulators
// through copies) and the MFMAs keep their place between the LDS reads.  The hazards the compiler would pad for are handled
// here: an MFMA must not read a VGPR in the two wait states after a VALU wrote it (register copies the
// allocator places in front of the asm count), hence the s_nop; the loop never reads an accumulator
// except as the addend of the same MFMA a full step later; the wait states before the first VALU read
// of a result follow the loop.
template <bool FIRST>
__device__ __forceinline__ void mfma_acc(f4& acc, const h8& w, const h8& a)
{
    if constexpr (FIRST)
        asm volatile("s_nop 1\n\tv_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(acc) : "v"(w), "v"(a));
    else
        asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(acc) : "v"(w), "v"(a));
}

// Two of the four h2 a packed word expands to (half 0: fragment columns +0, half 1: columns +8).
template <bool FP6>
__device__ __forceinline__ void dequant_half(uint32_t q2, uint32_t q4, int half, const DequantConsts& k, h2& r0, h2& r1)
{
    if constexpr (FP6) {
        const s2 two = {2, 2};
        const uint32_t lo = half == 0 ? (q4 >> 2) : (q4 << 2);
        const uint32_t hi = half == 0 ? q2 : (q2 << 2);
        const uint32_t p = (hi & k.top2) | (lo & ~k.top2);
        const uint32_t p8 = p << 8;
        r0 = as_h2(__builtin_bit_cast(uint32_t, __builtin_bit_cast(s2, p) >> two) & k.exp_man);
        r1 = as_h2(__builtin_bit_cast(uint32_t, __builtin_bit_cast(s2, p8) >> two) & k.exp_man);
    } else {
        const h2 bias_lo = {(_Float16)1032.0f, (_Float16)1032.0f};
        const h2 mul_hi = {(_Float16)0.0625f, (_Float16)0.0625f};
        const h2 bias_hi = {(_Float16)-72.0f, (_Float16)-72.0f};
        const uint32_t q = half == 0 ? q4 : (q4 >> 8);
        r0 = as_h2((q & k.lo) | k.ex) - bias_lo;
        r1 = __builtin_elementwise_fma(as_h2((q & k.hi) | k.ex), mul_hi, bias_hi);
    }
}

struct MbCtx {
    uint32_t abuf[4][4];
    uint32_t addr_cur[4], addr_next[4];
};

// One step of the MB loop, fully static in BLK: block by block the 16 rows of A are multiplied into
// the step's eight weight fragments.  Activations travel through a ring of four register buffers,
// fetched from LDS two blocks ahead of their use (the latency hides behind 16 MFMAs); the s_waitcnt
// immediates follow from the fixed issue order: [A(0), A(1)] from the previous step, the next step's
// weight words (kExtra reads), then A(2), A(3), ...  After every MFMA `hook(block, t)` runs: the caller
// uses it to dequantise the next step's fragments a few VALU instructions at a time.
template <int MB, int kExtra, int BLK = 0>
struct MbBlocks {
    template <int phase, typename Hook>
    static __device__ __forceinline__ void run(MbCtx& cx, const h8 (&frag)[8], f4 (&acc)[MB][8], Hook&& hook)
    {
        if constexpr (BLK < MB) {
            constexpr int nb = BLK + 2;
            uint32_t (&dst)[4] = cx.abuf[(phase + nb) & 3];
            if constexpr (nb < MB)
                lds_read_a4<nb * 1024>(dst, cx.addr_cur);
            else
                lds_read_a4<(nb - MB) * 1024>(dst, cx.addr_next);
            // block 0 needs A(0): A(1), the extra reads and A(2) may be outstanding; from block 1 on the
            // extra reads must be complete as well
            constexpr int allow = BLK == 0 ? (8 + kExtra < 15 ? 8 + kExtra : 15) : 8;
            __builtin_amdgcn_s_waitcnt(lgkmcnt_only(allow));
            uint32_t (&src)[4] = cx.abuf[(phase + BLK) & 3];
            asm volatile("" : "+v"(src[0]), "+v"(src[1]), "+v"(src[2]), "+v"(src[3]));
            const h8 av = __builtin_bit_cast(h8, u4{src[0], src[1], src[2], src[3]});
            mfma_acc<true>(acc[BLK][0], frag[0], av); hook(Int<BLK>{}, Int<0>{});
            mfma_acc<false>(acc[BLK][1], frag[1], av); hook(Int<BLK>{}, Int<1>{});
            mfma_acc<false>(acc[BLK][2], frag[2], av); hook(Int<BLK>{}, Int<2>{});
            mfma_acc<false>(acc[BLK][3], frag[3], av); hook(Int<BLK>{}, Int<3>{});
            mfma_acc<false>(acc[BLK][4], frag[4], av); hook(Int<BLK>{}, Int<4>{});
            mfma_acc<false>(acc[BLK][5], frag[5], av); hook(Int<BLK>{}, Int<5>{});
            mfma_acc<false>(acc[BLK][6], frag[6], av); hook(Int<BLK>{}, Int<6>{});
            mfma_acc<false>(acc[BLK][7], frag[7], av); hook(Int<BLK>{}, Int<7>{});
            MbBlocks<MB, kExtra, BLK + 1>::template run<phase>(cx, frag, acc, hook);
        }
    }
};

template <bool FP6, bool G128, int DEPTH, int MB>
__device__ __forceinline__ void stream_tile_mb(const GemmArgs& p, const TileInfo& ti, unsigned char* ring,
                                               int step_begin, int step_end, f4 (&acc)[MB][8])
{
    static_assert(DEPTH >= 3, "needs two steps of look-ahead");
    static_assert(MB == 2 || MB == 4, "the A register ring assumes MB | 4; 128 accumulator VGPRs at most");
    constexpr bool kGroup = G128 && !FP6;
    static_assert(!FP6 || DEPTH == 3, "the 2-bit plane alternates between two register sets");
    constexpr int kAOff = 2048;
    constexpr int kSlot = kAOff + MB * 1024;
    constexpr int kOps = 2 + MB + (FP6 ? 2 : 0);          // vector-memory loads per step
    constexpr int kUnroll = kGroup ? 4 : 2;
    constexpr int kW = 2;                                 // LDS reads of one step's weight words
    static_assert(kOps * (DEPTH - 2) <= 63, "vmcnt is a 6-bit counter");
    const int lane = threadIdx.x & 63;
    const int i = lane >> 4, c = lane & 15, sigma = c >> 3, l = c & 7;

    DequantConsts kc;
    kc.lo = vgpr_const(0x000f000fu);
    kc.hi = vgpr_const(0x00f000f0u);
    kc.ex = vgpr_const(0x64006400u);
    kc.top2 = vgpr_const(0xc0c0c0c0u);
    kc.exp_man = vgpr_const(0x9f009f00u);

    // ---- fetch side: uniform 64-bit bases on the scalar unit, per-lane 32-bit offsets that never change.
    // The offsets carry the compensation for the immediates (see dma16_m0): the second k-block of the
    // words sits 1 KiB further in LDS and one row further in memory; the A blocks get theirs on the
    // scalar base, so that the lane offsets stay non-negative.  The FP6 2-bit plane (8 bytes per lane and
    // k-block, already in owner order in memory) skips LDS: it is loaded into registers two steps ahead,
    // alternating between two register sets, which keeps an FP6 slot as small as an INT4 one.
    const PlaneGeometry geo = plane_geometry(p, ti);
    const size_t row4 = geo.row4, row2 = geo.row2;
    const int owner = p.native ? lane : 32 * sigma + 4 * l + i;      // whose granule of the k-block this lane needs
    const uint32_t v4 = (lane ^ ((lane >> 4) & 3)) * 16;
    const uint32_t v4b = v4 + (uint32_t)row4 - 1024;
    const unsigned char* base4 = uniform_ptr(reinterpret_cast<const unsigned char*>(FP6 ? p.b_fp6_4 : p.b_int4) +
                                             geo.tile4 + (size_t)(2 * step_begin) * row4);
    const uint32_t v2 = (uint32_t)owner * 8, v2b = v2 + (uint32_t)row2;
    const unsigned char* base2 = uniform_ptr(reinterpret_cast<const unsigned char*>(p.b_fp6_2) +
                                             geo.tile2 + (size_t)(2 * step_begin) * row2);
    u2 tq[2][2];                                          // [register set][k-block]
    const int a_m = lane >> 2;
    const int tile_row0 = ti.mtile * 16 * MB;
    uint32_t va[MB];
#pragma unroll
    for (int mb = 0; mb < MB; mb++) {
        int row = tile_row0 + 16 * mb + a_m;
        row = row < p.m ? row : p.m - 1;
        va[mb] = (uint32_t)(row - tile_row0) * (uint32_t)p.k * 2 + 16 * ((lane & 3) ^ ((a_m >> 2) & 3)) + 4096 -
                 (kAOff + 1024 * mb) % 4096;
    }
    const unsigned char* base_a = uniform_ptr(reinterpret_cast<const unsigned char*>(p.A + (size_t)tile_row0 * p.k) +
                                              (size_t)(ti.a_step0 + step_begin) * 64 - 4096);
    const unsigned char* base_gs =
        uniform_ptr(reinterpret_cast<const unsigned char*>(p.s_int4 + (size_t)ti.tcol * kTileN));
    const uint32_t vgs = 4 * lane;
    constexpr int kScaleMask = DEPTH <= 5 ? 1 : 3;
    unsigned char* gs_ring = ring + DEPTH * kSlot;
    const uint32_t ring_lds = uniform32(lds_addr(ring));
    const uint32_t gs_lds = uniform32(lds_addr(gs_ring));

    int issued = step_begin;
    const int last = step_end - 1;
    auto issue = [&](int slot, int set) {
        const uint32_t dst = ring_lds + slot * kSlot;
        set_m0(dst);
        dma16_m0<0, true>(base4, v4);
        dma16_m0<1024, true>(base4, v4b);
        dma_a_blocks<MB, kAOff>(dst, base_a, va);
        if (FP6) {
            asm volatile("global_load_dwordx2 %0, %2, %4 nt\n\tglobal_load_dwordx2 %1, %3, %4 nt"
                         : "=&v"(tq[set][0]), "=&v"(tq[set][1]) : "v"(v2), "v"(v2b), "s"(base2) : "memory");
        }
        if (kGroup && (issued & 3) == 0) {
            set_m0(gs_lds + ((issued >> 2) & kScaleMask) * 256);
            dma4_m0(base_gs + (size_t)(issued >> 2) * (size_t)uniform32(p.n4) * 2, vgs);
        }
        if (issued < last) {
            issued++;
            base4 += 2 * row4;
            base2 += 2 * row2;
            base_a += 64;
        }
    };

    // ---- read side
    const uint32_t rd4 = ring_lds + (owner ^ ((owner >> 4) & 3)) * 16;
    uint32_t rda[4];
#pragma unroll
    for (int d = 0; d < 4; d++) rda[d] = ring_lds + kAOff + (4 * c + (d ^ ((c >> 2) & 3))) * 16 + 4 * i;
    const uint32_t rdgs = gs_lds + (64 * sigma + l) * 2;    // weight side: column (j, half) at +32j +16half

    uint32_t gs_next[8];
    h2 gs_cur[8];
    MbCtx cx;
    WeightRegs w;
    auto fetch_w = [&](int slot) {
        const uint32_t so = slot * kSlot;
        asm volatile("ds_read_b128 %0, %2\n\tds_read_b128 %1, %2 offset:1024"
                     : "=&v"(w.q0), "=&v"(w.q1) : "v"(rd4 + so) : "memory");
    };
    auto fetch_scales = [&](int group) {
        const uint32_t ga = rdgs + (group & kScaleMask) * 256;
        asm volatile(
            "ds_read_u16 %0, %8\n\tds_read_u16 %1, %8 offset:16\n\tds_read_u16 %2, %8 offset:32\n\t"
            "ds_read_u16 %3, %8 offset:48\n\tds_read_u16 %4, %8 offset:64\n\tds_read_u16 %5, %8 offset:80\n\t"
            "ds_read_u16 %6, %8 offset:96\n\tds_read_u16 %7, %8 offset:112"
            : "=&v"(gs_next[0]), "=&v"(gs_next[1]), "=&v"(gs_next[2]), "=&v"(gs_next[3]), "=&v"(gs_next[4]),
              "=&v"(gs_next[5]), "=&v"(gs_next[6]), "=&v"(gs_next[7])
            : "v"(ga) : "memory");
    };
    auto settle_scales = [&]() {
#pragma unroll
        for (int t = 0; t < 8; t++) {
            asm volatile("" : "+v"(gs_next[t]));
            gs_cur[t] = as_h2((gs_next[t] & 0xffffu) | (gs_next[t] << 16));
        }
    };
    // A quarter of one j group (a "chunk": 4..8 VALU instructions): chunk = 4j + 2*half + word.  The
    // word is tied to this point of the program first, the results after, so the instructions stay
    // between the two MFMAs the chunk was placed between.
    h2 part[2];
    auto chunk = [&](int ck, int set, h8 (&frag)[8]) {
        const int j = ck >> 2, half = (ck >> 1) & 1, word = ck & 1;
        uint32_t q4 = word ? w.q1[j] : w.q0[j];
        uint32_t q2 = 0;
        asm volatile("" : "+v"(q4));
        if (word) w.q1[j] = q4; else w.q0[j] = q4;
        if (FP6) {
            uint32_t t = tq[set][word][j >> 1];
            asm volatile("" : "+v"(t));
            tq[set][word][j >> 1] = t;
            q2 = t << (4 * (j & 1));
        }
        h2 r0, r1;
        dequant_half<FP6>(q2, q4, half, kc, r0, r1);
        if (kGroup) {
            r0 = r0 * gs_cur[2 * j + half];
            r1 = r1 * gs_cur[2 * j + half];
        }
        if (word == 0) {
            part[0] = r0;
            part[1] = r1;
            asm volatile("" : "+v"(part[0]), "+v"(part[1]));
        } else {
            frag[2 * j + half] = join(part[0], part[1], r0, r1);
            asm volatile("" : "+v"(frag[2 * j + half]));
        }
    };
    auto slot_addrs = [&](uint32_t (&addr)[4], int slot) {
        const uint32_t so = slot * kSlot;
#pragma unroll
        for (int d = 0; d < 4; d++) addr[d] = rda[d] + so;
    };

    int slot_in = 0;
#pragma unroll
    for (int d = 0; d < DEPTH - 1; d++) {
        issue(slot_in, d & 1);
        slot_in = slot_in + 1 == DEPTH ? 0 : slot_in + 1;
    }
    h8 frag[2][8];
    __builtin_amdgcn_s_waitcnt(vmcnt_only(kOps * (DEPTH - 2)));
    slot_addrs(cx.addr_next, 0);
    fetch_w(0);
    lds_read_a4<0>(cx.abuf[0], cx.addr_next);
    lds_read_a4<1024>(cx.abuf[1], cx.addr_next);
    if (kGroup) fetch_scales(step_begin >> 2);
    __builtin_amdgcn_s_waitcnt(lgkmcnt_only(0));
    if (kGroup) settle_scales();
#pragma unroll
    for (int ck = 0; ck < 16; ck++) chunk(ck, 0, frag[0]);
    int slot_rd = 1;
#pragma unroll 1
    for (int s = step_begin; s < step_end; s += kUnroll) {
#pragma unroll
        for (int u = 0; u < kUnroll; u++) {
            issue(slot_in, u & 1);                                    // step s+u+2 (FP6: DEPTH is 3)
            slot_in = slot_in + 1 == DEPTH ? 0 : slot_in + 1;
#pragma unroll
            for (int d = 0; d < 4; d++) cx.addr_cur[d] = cx.addr_next[d];
            slot_addrs(cx.addr_next, slot_rd);
            __builtin_amdgcn_s_waitcnt(vmcnt_only(kOps * (DEPTH - 2)));
            // step s+u+1 (and its group scales) has landed: read its words now, dequantise them
            // between this step's MFMAs
            fetch_w(slot_rd);
            const bool next_group = kGroup && u == kUnroll - 1;       // step s+u+1 starts a 128-row group
            if (next_group) fetch_scales((s + u + 1) >> 2);
            slot_rd = slot_rd + 1 == DEPTH ? 0 : slot_rd + 1;
            h8 (&cur)[8] = frag[u & 1];
            h8 (&nxt)[8] = frag[(u + 1) & 1];
            auto hook = [&](auto blk, auto t) {
                constexpr int mslot = decltype(blk)::value * 8 + decltype(t)::value;   // MFMA just issued
                constexpr int avail = 8 * MB - 8;                     // chunks go after the MFMAs of blocks >= 1
                if constexpr (mslot == 8) {
                    if (next_group) settle_scales();
                }
                if constexpr (mslot >= 8) {
                    constexpr int c0 = (mslot - 8) * 16 / avail, c1 = (mslot - 7) * 16 / avail;
#pragma unroll
                    for (int ck = c0; ck < c1; ck++) chunk(ck, (u + 1) & 1, nxt);
                }
            };
            constexpr int kExtraMax = kW + (kGroup ? 8 : 0);
            if ((u & 1) == 0)                                          // buffer of block 0: (u * MB) mod 4
                MbBlocks<MB, kExtraMax>::template run<0>(cx, cur, acc, hook);
            else
                MbBlocks<MB, kExtraMax>::template run<(MB & 3)>(cx, cur, acc, hook);
        }
    }
    __builtin_amdgcn_s_waitcnt(vmcnt_only(0) & lgkmcnt_only(0));
    // MFMA results -> VALU reads: the wait states, then every accumulator is passed through an (empty)
    // asm so that no read of it can be scheduled above them.
    asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 7");
#pragma unroll
    for (int mb = 0; mb < MB; mb++)
#pragma unroll
        for (int t = 0; t < 8; t++) {
            asm volatile("" : "+v"(acc[mb][t]));
        }
    if (FP6) {
#pragma unroll
        for (int mb = 0; mb < MB; mb++)
#pragma unroll
            for (int t = 0; t < 8; t++) acc[mb][t] *= 4096.0f;
    }
}

// Epilogue of the MB kernel: block by block, the four k slices are summed through LDS (wave wk finishes
// rows wk, wk+4, ... of the block, lane L owns columns 2L, 2L+1); then C is written, or the rows are
// published and the last-arriving workgroup of the (tile, row tile) gathers all parts in part order.
// `smem`, `flag` and `valid` belong to the WK waves that share a tile and a row tile (the whole workgroup in
// gemm_mb_kernel, one of WM groups in gemm_wm_kernel); a group without rows goes through the barriers
// without touching memory.
template <int MB, int WK = kWaves>
__device__ __forceinline__ void wg_finish_mb(const GemmArgs& p, const TileInfo& ti, int wk, int ks, f4 (&acc)[MB][8],
                                             bool per_column_scale, unsigned char* smem, int wave_lds, int* flag,
                                             bool valid = true, int first_fp6 = WK)
{
    constexpr int RMAX = 16 / WK, PCHUNK = 32 / RMAX;                // parts whose loads are in flight together
    typedef float f2 __attribute__((ext_vector_type(2)));
    const int lane = threadIdx.x & 63;
    const bool leader = lane == 0 && wk == 0;
    const int c = lane & 15, q = lane >> 4;
    const int row0 = ti.mtile * 16 * MB;
    const int nrows = !valid ? 0 : (p.m - row0 < 16 * MB ? p.m - row0 : 16 * MB);
    float s0 = 1.0f, s1 = 1.0f;
    if (per_column_scale) {
        const uint16_t* sp = ti.fp6 ? p.s_fp6 : p.s_int4;
        const int nr = ti.tcol * kTileN + 2 * lane;
        const h2 sv = *reinterpret_cast<const h2*>(sp + (nr & ~31) + scale_slot(nr & 31));
        s0 = (float)sv[0];
        s1 = (float)sv[1];
    }
    float x0 = 1.0f, x1 = 1.0f;                                      // row mix: FP6 column scales of slices >= first_fp6
    if (first_fp6 < WK) {
        const int nr = ti.tcol * kTileN + 2 * lane;
        const h2 sv = *reinterpret_cast<const h2*>(p.s_fp6 + (nr & ~31) + scale_slot(nr & 31));
        x0 = (float)sv[0];
        x1 = (float)sv[1];
    }
    uint16_t* c_out = p.C + (size_t)row0 * p.n + ti.col0 + 2 * lane;
    auto store_row = [&](int row, float v0, float v1) {
        if (p.fused) {
            store_fused(p, (size_t)(row0 + row), ti.col0 + 2 * lane, v0 * s0, v1 * s1);
            return;
        }
        h2 o = {(_Float16)(v0 * s0), (_Float16)(v1 * s1)};
        *reinterpret_cast<h2*>(c_out + (size_t)row * p.n) = o;
    };
    constexpr size_t kSlotU64 = (size_t)MB * 16 * kTileN / 2;
    unsigned long long* slot0 = reinterpret_cast<unsigned long long*>(p.scratch) +
                                (size_t)(ti.mtile * p.tiles + ti.tile) * ks * kSlotU64 + lane;
    unsigned long long* my = slot0 + (size_t)ti.part * kSlotU64;

#pragma unroll
    for (int mb = 0; mb < MB; mb++) {
        __syncthreads();
        float* mine = reinterpret_cast<float*>(smem + wk * wave_lds) + c * kRedStride + 64 * (q >> 1) + 4 * (q & 1);
#pragma unroll
        for (int t = 0; t < 8; t++) *reinterpret_cast<f4*>(mine + 16 * (t >> 1) + 8 * (t & 1)) = acc[mb][t];
        __syncthreads();
#pragma unroll
        for (int r = 0; r < RMAX; r++) {
            const int m = wk + r * WK, row = 16 * mb + m;
            if (row < nrows) {
                float v0 = 0.f, v1 = 0.f;
#pragma unroll
                for (int j = 0; j < WK; j++) {
                    const f2 v = *reinterpret_cast<const f2*>(reinterpret_cast<const float*>(smem + j * wave_lds) +
                                                              m * kRedStride + 2 * lane);
                    v0 += j >= first_fp6 ? v[0] * x0 : v[0];
                    v1 += j >= first_fp6 ? v[1] * x1 : v[1];
                }
                if (ks == 1) {
                    store_row(row, v0, v1);
                } else {
                    const f2 v = {v0, v1};
                    __hip_atomic_store(my + (size_t)row * (kTileN / 2), __builtin_bit_cast(unsigned long long, v),
                                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            }
        }
    }
    if (ks == 1) return;

    FP6M_MARK(p, 3);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __syncthreads();
    int* counter = p.counters + ti.mtile * p.tiles + ti.tile;
    if (leader) {
        int last = 0;
        if (valid) last = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == ks - 1;
        *flag = last;
    }
    __syncthreads();
    if (!*flag) return;
    FP6M_MARK(p, 5);
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
#pragma unroll 1
    for (int mb = 0; mb < MB; mb++) {
        float v0[RMAX], v1[RMAX];
#pragma unroll
        for (int r = 0; r < RMAX; r++) {
            v0[r] = 0.f;
            v1[r] = 0.f;
        }
        for (int pp = 0; pp < ks; pp += PCHUNK) {
            unsigned long long t[PCHUNK][RMAX];
#pragma unroll
            for (int u = 0; u < PCHUNK; u++)
#pragma unroll
                for (int r = 0; r < RMAX; r++) {
                    const int row = 16 * mb + wk + r * WK;
                    t[u][r] = 0;
                    if (row < nrows && pp + u < ks)
                        t[u][r] = __hip_atomic_load(slot0 + (size_t)(pp + u) * kSlotU64 + (size_t)row * (kTileN / 2),
                                                    __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
#pragma unroll
            for (int u = 0; u < PCHUNK; u++)
#pragma unroll
                for (int r = 0; r < RMAX; r++) {
                    const f2 v = __builtin_bit_cast(f2, t[u][r]);
                    v0[r] += v[0];
                    v1[r] += v[1];
                }
        }
#pragma unroll
        for (int r = 0; r < RMAX; r++) {
            const int row = 16 * mb + wk + r * WK;
            if (row < nrows) store_row(row, v0[r], v1[r]);
        }
    }
    // the counter is next touched by a later launch on the stream: the reset needs no ordering here
    if (leader) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

constexpr int mb_wave_lds(int mb, int d4, int d6)
{
    return max3(d4 * (2048 + mb * 1024) + scale_slab_bytes(d4), d6 * (2048 + mb * 1024), 16 * kRedStride * 4);
}

// WK = k slices (waves) per workgroup: four, or eight (one workgroup per CU, two waves per SIMD) for grids that
// would otherwise leave every SIMD a single wave.
template <bool G128, int MB, int D4, int D6, int WK>
__global__ __launch_bounds__(64 * WK, WK == 4 ? 2 : 1) void gemm_mb_kernel(const GemmArgs p)
{
    constexpr int kWaveLds = mb_wave_lds(MB, D4, D6);
    static_assert(WK * kWaveLds + 16 <= 160 * 1024, "LDS of one CU");
    __shared__ __attribute__((aligned(16))) unsigned char smem[WK * kWaveLds + 16];

    FP6M_MARK(p, 0);
    TileInfo ti = locate_tile(p);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    int step_begin, step_end;
    wave_k_range<G128, WK>(p, ti.part, wave, step_begin, step_end);
    if (p.k4) row_mix_slice(p, ti.part * WK + wave, p.ksplit * WK, ti, step_begin, step_end);

    f4 acc[MB][8];
#pragma unroll
    for (int mb = 0; mb < MB; mb++)
#pragma unroll
        for (int t = 0; t < 8; t++) acc[mb][t] = f4{0.f, 0.f, 0.f, 0.f};
    unsigned char* ring = smem + wave * kWaveLds;
    if (step_begin < step_end) {
        if (ti.fp6)
            stream_tile_mb<true, G128, D6, MB>(p, ti, ring, step_begin, step_end, acc);
        else
            stream_tile_mb<false, G128, D4, MB>(p, ti, ring, step_begin, step_end, acc);
    }
    FP6M_MARK(p, 2);
    wg_finish_mb<MB, WK>(p, ti, wave, p.ksplit, acc, !p.k4 && (ti.fp6 || !G128), smem, kWaveLds,
                         reinterpret_cast<int*>(smem + WK * kWaveLds), true, p.k4 ? p.slices4 - ti.part * WK : WK);
    FP6M_MARK(p, 7);
}

// ------------------------------------------------------------------------------------------------ 128 < m: fragments shared by four row tiles
//
// The m > 16 kernel spends more issue slots on dequantisation than on MFMAs (a SIMD issues both from one
// pipe), and every row tile repeats that work.  Here a workgroup is eight waves = four row tiles (64 rows
// each) x two k slices of ONE tile: the four waves of a k slice fetch the tile's words once, each
// dequantises a quarter of a step's operand fragments (one 16-column group) into LDS, and all four multiply
// from there.  One workgroup barrier per step publishes the fragments and hands ring slots back to the
// fetches; A stays private to its wave.  LDS per k slice: three slots (words [+ 2-bit plane], four 4 KiB A
// slabs), two 8 KiB fragment buffers, two rows of group scales.

constexpr int kWmRows = 4;                                           // row tiles per workgroup
// WN adjacent tiles x (2 / WN) k slices: with WN = 2 the two tiles' waves also share the A slabs.
template <int WN> constexpr int wm_slot_max() { return WN * 3072 + kWmRows * 4096; }
template <int WN> constexpr int wm_frag_off() { return 3 * wm_slot_max<WN>(); }
template <int WN> constexpr int wm_scale_off() { return wm_frag_off<WN>() + WN * 2 * 8192; }
template <int WN> constexpr int wm_slice_lds() { return wm_scale_off<WN>() + WN * 512; }
constexpr int kWmRegion = 16 * kRedStride * 4;                       // one wave's 16-row block in the epilogue
template <int WN> constexpr int wm_lds() { return max3((2 / WN) * wm_slice_lds<WN>(), 8 * kWmRegion, 0) + 64; }
static_assert(wm_lds<1>() <= 160 * 1024 && wm_lds<2>() <= 160 * 1024, "LDS of one CU");

struct WmState {
    uint32_t abuf[4][4];
    uint32_t addr_cur[4], addr_next[4];
    h8 cur[8];
};

// One step: block by block the 16 rows of A meet the eight fragments.  LDS issue order of a step: the raw
// words of this wave's share (and group scales), the eight fragment reads, then A(2), A(3) and the first
// two blocks of the next step; block 0 waits fragment by fragment.
template <int BLK = 0>
struct WmBlocks {
    template <int phase, typename Hook>
    static __device__ __forceinline__ void run(WmState& st, f4 (&acc)[4][8], Hook&& hook)
    {
        if constexpr (BLK < 4) {
            constexpr int nb = BLK + 2;
            uint32_t (&dst)[4] = st.abuf[(phase + nb) & 3];
            if constexpr (nb < 4)
                lds_read_a4<nb * 1024>(dst, st.addr_cur);
            else
                lds_read_a4<(nb - 4) * 1024>(dst, st.addr_next);
            if constexpr (BLK > 0) __builtin_amdgcn_s_waitcnt(lgkmcnt_only(8));
            uint32_t (&src)[4] = st.abuf[(phase + BLK) & 3];
            asm volatile("" : "+v"(src[0]), "+v"(src[1]), "+v"(src[2]), "+v"(src[3]));
            const h8 av = __builtin_bit_cast(h8, u4{src[0], src[1], src[2], src[3]});
            step<0>(st, acc, av, hook);
            WmBlocks<BLK + 1>::template run<phase>(st, acc, hook);
        }
    }
    template <int T, typename Hook>
    static __device__ __forceinline__ void step(WmState& st, f4 (&acc)[4][8], const h8& av, Hook&& hook)
    {
        if constexpr (T < 8) {
            if constexpr (BLK == 0) {
                // fragments T+1 .. 7 and the four reads of A(2) may still be in flight
                __builtin_amdgcn_s_waitcnt(lgkmcnt_only(11 - T));
                asm volatile("" : "+v"(st.cur[T]));
            }
            mfma_acc<(T == 0 || BLK == 0)>(acc[BLK][T], st.cur[T], av);
            hook(Int<BLK>{}, Int<T>{});
            step<T + 1>(st, acc, av, hook);
        }
    }
};

template <bool FP6, bool G128, int WN>
__device__ __forceinline__ void stream_tile_wm(const GemmArgs& p, const TileInfo& ti, unsigned char* slice, int wm, int wn,
                                               int step_begin, int step_end, int loop_end, f4 (&acc)[4][8])
{
    constexpr int MB = 4, WM = kWmRows, DEPTH = 3;
    constexpr bool kGroup = G128 && !FP6;
    constexpr int kWBytes = FP6 ? 3072 : 2048;
    constexpr int kSlot = WN * kWBytes + WM * 4096;
    constexpr int kUnroll = kGroup ? 4 : 2;
    const int lane = threadIdx.x & 63;
    const int i = lane >> 4, c = lane & 15, sigma = c >> 3, l = c & 7;
    const int j = wm;                                                // this wave dequantises column group j of every step

    DequantConsts kc;
    kc.lo = vgpr_const(0x000f000fu);
    kc.hi = vgpr_const(0x00f000f0u);
    kc.ex = vgpr_const(0x64006400u);
    kc.top2 = vgpr_const(0xc0c0c0c0u);
    kc.exp_man = vgpr_const(0x9f009f00u);

    // ---- fetch side: wave 0 and 1 of the slice fetch the two k-blocks of the words, wave 2 the 2-bit plane,
    // wave 3 the group scales; every wave its own four blocks of A
    const PlaneGeometry geo = plane_geometry(p, ti);
    const size_t row4 = geo.row4, row2 = geo.row2;
    const uint32_t v4 = (lane ^ ((lane >> 4) & 3)) * 16;
    const uint32_t v4b = v4 + (uint32_t)row4 - 1024;
    const unsigned char* base4 = uniform_ptr(reinterpret_cast<const unsigned char*>(FP6 ? p.b_fp6_4 : p.b_int4) +
                                             geo.tile4 + (size_t)(2 * step_begin) * row4);
    const int lg = lane & 31;
    const uint32_t v2 = (uint32_t)((lane >> 5) * row2) + (lg ^ (lg >> 4)) * 16;
    const unsigned char* base2 = uniform_ptr(reinterpret_cast<const unsigned char*>(p.b_fp6_2) +
                                             geo.tile2 + (size_t)(2 * step_begin) * row2);
    const int a_m = lane >> 2;
    const int tile_row0 = ti.mtile * 16 * MB;
    uint32_t va[MB];
#pragma unroll
    for (int mb = 0; mb < MB; mb++) {
        int row = tile_row0 + 16 * mb + a_m;
        row = row < p.m ? row : p.m - 1;
        va[mb] = (uint32_t)(row - tile_row0) * (uint32_t)p.k * 2 + 16 * ((lane & 3) ^ ((a_m >> 2) & 3)) + 4096 - 1024 * mb;
    }
    const unsigned char* base_a = uniform_ptr(reinterpret_cast<const unsigned char*>(p.A + (size_t)tile_row0 * p.k) +
                                              (size_t)(ti.a_step0 + step_begin) * 64 - 4096);
    const unsigned char* base_gs =
        uniform_ptr(reinterpret_cast<const unsigned char*>(p.s_int4 + (size_t)ti.tcol * kTileN));
    const uint32_t vgs = 4 * lane;
    const uint32_t slice_lds = uniform32(lds_addr(slice));
    const uint32_t gs_lds = slice_lds + wm_scale_off<WN>() + uniform32(wn * 512);
    const uint32_t w_off = uniform32(wn * kWBytes);                   // this tile's words inside a slot
    const uint32_t a_off = uniform32(WN * kWBytes + wm * 4096);       // this row tile's slab (shared by the WN tiles)

    int issued = step_begin;
    const int last = step_end - 1;
    auto issue = [&](int slot) {
        const uint32_t dst = slice_lds + slot * kSlot;
        if (wm == 0) {
            set_m0(dst + w_off);
            dma16_m0<0, true>(base4, v4);
        }
        if (wm == 1) {
            set_m0(dst + w_off);
            dma16_m0<1024, true>(base4, v4b);
        }
        if (FP6 && wm == 2) {
            set_m0(dst + w_off + 2048);
            dma16_m0<0, true>(base2, v2);
        }
        if (kGroup && wm == 3 && (issued & 3) == 0) {
            set_m0(gs_lds + ((issued >> 2) & 1) * 256);
            dma4_m0(base_gs + (size_t)(issued >> 2) * (size_t)uniform32(p.n4) * 2, vgs);
        }
        set_m0(dst + a_off);
        if (WN == 1 || wn == 0) {                                     // with two tiles, each loads half of the slab
            dma16_m0<0, false>(base_a, va[0]);
            dma16_m0<1024, false>(base_a, va[1]);
        }
        if (WN == 1 || wn == 1) {
            dma16_m0<2048, false>(base_a, va[2]);
            dma16_m0<3072, false>(base_a, va[3]);
        }
        if (issued < last) {
            issued++;
            base4 += 2 * row4;
            base2 += 2 * row2;
            base_a += 64;
        }
    };

    // ---- read side
    const int owner = p.native ? lane : 32 * sigma + 4 * l + i;      // whose granule of the k-block this lane needs
    const uint32_t rd4 = slice_lds + w_off + (owner ^ ((owner >> 4) & 3)) * 16 + 4 * j;
    const int gr2 = owner >> 1;
    const uint32_t rd2 = slice_lds + w_off + 2048 + (gr2 ^ (gr2 >> 4)) * 16 + (owner & 1) * 8 + 4 * (j >> 1);
    const uint32_t t_shift = 4 * (j & 1);
    uint32_t rda[4];
#pragma unroll
    for (int d = 0; d < 4; d++) rda[d] = slice_lds + a_off + (4 * c + (d ^ ((c >> 2) & 3))) * 16 + 4 * i;
    const uint32_t rdgs = gs_lds + (64 * sigma + l) * 2 + 32 * j;     // columns (j, half 0) and, 16 bytes on, (j, half 1)
    const uint32_t frag_rd = slice_lds + wm_frag_off<WN>() + uniform32(wn * 2 * 8192) + lane * 16;
    const uint32_t frag_wr = frag_rd + 2 * j * 1024;

    WmState st;
    uint32_t q0 = 0, q1 = 0, t0 = 0, t1 = 0, gs_next[2] = {0, 0};
    h2 gs_cur[2], part[2];
    h8 mine[2];
    auto fetch_raw = [&](int slot) {
        const uint32_t so = slot * kSlot;
        asm volatile("ds_read_b32 %0, %2\n\tds_read_b32 %1, %2 offset:1024" : "=&v"(q0), "=&v"(q1) : "v"(rd4 + so) : "memory");
        if (FP6)
            asm volatile("ds_read_b32 %0, %2\n\tds_read_b32 %1, %2 offset:512" : "=&v"(t0), "=&v"(t1) : "v"(rd2 + so) : "memory");
    };
    auto fetch_scales = [&](int group) {
        asm volatile("ds_read_u16 %0, %2\n\tds_read_u16 %1, %2 offset:16"
                     : "=&v"(gs_next[0]), "=&v"(gs_next[1]) : "v"(rdgs + (group & 1) * 256) : "memory");
    };
    auto settle_scales = [&]() {
#pragma unroll
        for (int h = 0; h < 2; h++) {
            asm volatile("" : "+v"(gs_next[h]));
            gs_cur[h] = as_h2((gs_next[h] & 0xffffu) | (gs_next[h] << 16));
        }
    };
    auto fetch_frags = [&](int buf) {
        const uint32_t a = frag_rd + buf * 8192;
        asm volatile(
            "ds_read_b128 %0, %8\n\tds_read_b128 %1, %8 offset:1024\n\tds_read_b128 %2, %8 offset:2048\n\t"
            "ds_read_b128 %3, %8 offset:3072\n\tds_read_b128 %4, %8 offset:4096\n\tds_read_b128 %5, %8 offset:5120\n\t"
            "ds_read_b128 %6, %8 offset:6144\n\tds_read_b128 %7, %8 offset:7168"
            : "=&v"(st.cur[0]), "=&v"(st.cur[1]), "=&v"(st.cur[2]), "=&v"(st.cur[3]), "=&v"(st.cur[4]), "=&v"(st.cur[5]),
              "=&v"(st.cur[6]), "=&v"(st.cur[7])
            : "v"(a) : "memory");
    };
    // chunk ck = 2 * half + word of this wave's column group: two h2 of one packed word
    auto chunk = [&](int ck) {
        const int half = ck >> 1, word = ck & 1;
        uint32_t q4 = word ? q1 : q0, q2 = 0;
        asm volatile("" : "+v"(q4));
        if (word) q1 = q4; else q0 = q4;
        if (FP6) {
            uint32_t t = word ? t1 : t0;
            asm volatile("" : "+v"(t));
            if (word) t1 = t; else t0 = t;
            q2 = t << t_shift;
        }
        h2 r0, r1;
        dequant_half<FP6>(q2, q4, half, kc, r0, r1);
        if (kGroup) {
            r0 = r0 * gs_cur[half];
            r1 = r1 * gs_cur[half];
        }
        if (word == 0) {
            part[0] = r0;
            part[1] = r1;
            asm volatile("" : "+v"(part[0]), "+v"(part[1]));
        } else {
            mine[half] = join(part[0], part[1], r0, r1);
            asm volatile("" : "+v"(mine[half]));
        }
    };
    auto publish = [&](int buf) {
        asm volatile("ds_write_b128 %0, %1\n\tds_write_b128 %0, %2 offset:1024"
                     : : "v"(frag_wr + buf * 8192), "v"(mine[0]), "v"(mine[1]) : "memory");
    };
    auto slot_addrs = [&](uint32_t (&addr)[4], int slot) {
        const uint32_t so = slot * kSlot;
#pragma unroll
        for (int d = 0; d < 4; d++) addr[d] = rda[d] + so;
    };

    issue(0);
    issue(1);
    __builtin_amdgcn_s_waitcnt(vmcnt_only(0));                        // steps 0 and 1: this wave's loads ...
    __builtin_amdgcn_s_barrier();                                     // ... and everybody else's
    slot_addrs(st.addr_next, 0);
    fetch_raw(0);
    lds_read_a4<0>(st.abuf[0], st.addr_next);
    lds_read_a4<1024>(st.abuf[1], st.addr_next);
    if (kGroup) fetch_scales(step_begin >> 2);
    __builtin_amdgcn_s_waitcnt(lgkmcnt_only(0));
    if (kGroup) settle_scales();
#pragma unroll
    for (int ck = 0; ck < 4; ck++) chunk(ck);
    publish(0);                                                       // step_begin is even
    int slot_in = 2, slot_rd = 1;
#pragma unroll 1
    for (int s = step_begin; s < loop_end; s += kUnroll) {
#pragma unroll
        for (int u = 0; u < kUnroll; u++) {
            // step s+u+1 has landed and the fragments of step s+u are written, for everybody; everybody has
            // left step s+u-1, whose slot the loads of step s+u+2 overwrite and whose fragment buffer this
            // step's dequantisation refills
            __builtin_amdgcn_s_waitcnt(vmcnt_only(0) & lgkmcnt_only(0));
            __builtin_amdgcn_s_barrier();
            issue(slot_in);
            slot_in = slot_in + 1 == DEPTH ? 0 : slot_in + 1;
            if (s >= step_end) continue;                              // (uniform) only keeping step with the others
#pragma unroll
            for (int d = 0; d < 4; d++) st.addr_cur[d] = st.addr_next[d];
            slot_addrs(st.addr_next, slot_rd);
            fetch_raw(slot_rd);
            const bool next_group = kGroup && u == kUnroll - 1;       // step s+u+1 starts a 128-row group
            if (next_group) fetch_scales((s + u + 1) >> 2);
            slot_rd = slot_rd + 1 == DEPTH ? 0 : slot_rd + 1;
            fetch_frags(u & 1);
            auto hook = [&](auto blk, auto t) {
                constexpr int mslot = decltype(blk)::value * 8 + decltype(t)::value;   // MFMA just issued
                if constexpr (mslot == 8) {
                    if (next_group) settle_scales();
                }
                if constexpr (mslot >= 8 && mslot < 24 && (mslot & 3) == 0) chunk((mslot - 8) >> 2);
                if constexpr (mslot == 31) publish((u + 1) & 1);
            };
            if ((u & 1) == 0)
                WmBlocks<>::template run<0>(st, acc, hook);
            else
                WmBlocks<>::template run<0>(st, acc, hook);
        }
    }
    __builtin_amdgcn_s_waitcnt(vmcnt_only(0) & lgkmcnt_only(0));
    asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 7");
#pragma unroll
    for (int mb = 0; mb < MB; mb++)
#pragma unroll
        for (int t = 0; t < 8; t++) asm volatile("" : "+v"(acc[mb][t]));
    if (FP6) {
#pragma unroll
        for (int mb = 0; mb < MB; mb++)
#pragma unroll
            for (int t = 0; t < 8; t++) acc[mb][t] *= 4096.0f;
    }
}

template <bool G128, int WN>
__global__ __launch_bounds__(512, 2) void gemm_wm_kernel(const GemmArgs p)
{
    constexpr int MB = 4, WM = kWmRows, WK = 2 / WN;
    __shared__ __attribute__((aligned(16))) unsigned char smem[wm_lds<WN>()];

    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wm = wave % WM, wn = WN == 2 ? wave / WM : 0, wk = WN == 2 ? 0 : wave / WM;
    const int logical = xcd_contiguous_id(blockIdx.x, gridDim.x);
    const int group = logical / p.ksplit;                            // WN adjacent tiles of one region
    TileInfo ti;
    ti.part = logical - group * p.ksplit;
    ti.fp6 = group < p.groups6;
    ti.region_n = ti.fp6 ? p.qc : p.n4;
    const int region_tiles = ti.region_n / kTileN;
    int tcol = (ti.fp6 ? group : group - p.groups6) * WN + wn;
    ti.mtile = blockIdx.y * WM + wm;
    const bool valid = tcol < region_tiles && ti.mtile * 16 * MB < p.m;
    // a wave without a tile or without rows still fetches and dequantises its share for the others: it
    // repeats the last tile / row tile (all its addresses stay inside the operands) and stores nothing
    if (tcol >= region_tiles) tcol = region_tiles - 1;
    if (ti.mtile * 16 * MB >= p.m) ti.mtile = (p.m - 1) / (16 * MB);
    ti.tcol = tcol;
    ti.tile = ti.fp6 ? tcol : p.tiles6 + tcol;
    ti.col0 = (ti.fp6 ? p.n4 : 0) + tcol * kTileN;
    ti.a_step0 = 0;

    // k slices: part-major, then wk; every wave of the workgroup runs the longest slice's step count
    constexpr int unit_steps = G128 ? 4 : 2;
    const int units = p.k / (32 * unit_steps);
    const int nslices = p.ksplit * WK;
    int step_begin = 0, step_end = 0, longest = 0;
#pragma unroll
    for (int q = 0; q < WK; q++) {
        const int sl = ti.part * WK + q;
        const int b = (int)((long long)units * sl / nslices) * unit_steps;
        const int e = (int)((long long)units * (sl + 1) / nslices) * unit_steps;
        if (q == wk) {
            step_begin = b;
            step_end = e;
        }
        longest = e - b > longest ? e - b : longest;
    }

    f4 acc[MB][8];
#pragma unroll
    for (int mb = 0; mb < MB; mb++)
#pragma unroll
        for (int t = 0; t < 8; t++) acc[mb][t] = f4{0.f, 0.f, 0.f, 0.f};
    unsigned char* slice = smem + wk * wm_slice_lds<WN>();
    if (ti.fp6)
        stream_tile_wm<true, G128, WN>(p, ti, slice, wm, wn, step_begin, step_end, step_begin + longest, acc);
    else
        stream_tile_wm<false, G128, WN>(p, ti, slice, wm, wn, step_begin, step_end, step_begin + longest, acc);
    const int grp = wn * WM + wm;                                    // the WK waves that share a tile and a row tile
    wg_finish_mb<MB, WK>(p, ti, wk, p.ksplit, acc, ti.fp6 || !G128, smem + grp * WK * kWmRegion, kWmRegion,
                         reinterpret_cast<int*>(smem + wm_lds<WN>() - 64) + grp, valid);
}

// Activation gather of fp6m_mul_fused: out[r, kk] = A[r, a_cols[kk]] (map entries clamped to the row).  One
// thread per pair of output elements; the m x k result is what the GEMM kernels then stream as their A.
__global__ __launch_bounds__(256) void gather_a_kernel(const uint16_t* __restrict__ A, int lda,
                                                      const int32_t* __restrict__ a_cols, uint16_t* __restrict__ out,
                                                      int k)
{
    const int kk = 2 * (blockIdx.x * 256 + threadIdx.x);
    if (kk >= k) return;
    const size_t row = blockIdx.y;
    int c0 = a_cols[kk], c1 = a_cols[kk + 1];
    c0 = c0 < 0 ? 0 : (c0 >= lda ? lda - 1 : c0);
    c1 = c1 < 0 ? 0 : (c1 >= lda ? lda - 1 : c1);
    const uint32_t v = (uint32_t)A[row * lda + c0] | ((uint32_t)A[row * lda + c1] << 16);
    *reinterpret_cast<uint32_t*>(out + row * k + kk) = v;
}

// ------------------------------------------------------------------------------------------------ host

thread_local int g_last_hip_error = 0;

struct DeviceScratch {
    float* ptr = nullptr;
    int cus = 0;
    uint16_t* gathered = nullptr;   // gathered activations of fp6m_mul_fused (kGatherBytes, on first use)
};
constexpr size_t kGatherBytes = size_t(64) << 20;
constexpr int kMaxDevices = 64;
DeviceScratch g_scratch[kMaxDevices];
std::mutex g_scratch_mutex;

int hip_fail(hipError_t e)
{
    g_last_hip_error = (int)e;
    return FP6M_ERR_HIP;
}

int ensure_scratch(int dev, DeviceScratch** out)
{
    if (dev < 0 || dev >= kMaxDevices) return FP6M_ERR_ARG;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    DeviceScratch& d = g_scratch[dev];
    if (!d.ptr) {
        int prev = 0;
        hipError_t e = hipGetDevice(&prev);
        if (e != hipSuccess) return hip_fail(e);
        if (prev != dev && (e = hipSetDevice(dev)) != hipSuccess) return hip_fail(e);
        void* mem = nullptr;
        e = hipMalloc(&mem, kScratchBytes + kPackTempBytes);          // partial tiles, then the packer's scratch
        int cus = 0;
        if (e == hipSuccess) e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
        if (prev != dev) (void)hipSetDevice(prev);
        if (e != hipSuccess) return hip_fail(e);
        d.ptr = static_cast<float*>(mem);
        d.cus = cus > 0 ? cus : 256;
    }
    *out = &d;
    return FP6M_OK;
}

// The buffer the gathered activations of fp6m_mul_fused go through: allocated on the first call that gathers.
int ensure_gather_buffer(int dev, DeviceScratch* d)
{
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (d->gathered) return FP6M_OK;
    int prev = 0;
    hipError_t e = hipGetDevice(&prev);
    if (e != hipSuccess) return hip_fail(e);
    if (prev != dev && (e = hipSetDevice(dev)) != hipSuccess) return hip_fail(e);
    void* mem = nullptr;
    e = hipMalloc(&mem, kGatherBytes);
    if (prev != dev) (void)hipSetDevice(prev);
    if (e != hipSuccess) return hip_fail(e);
    d->gathered = static_cast<uint16_t*>(mem);
    return FP6M_OK;
}

// Scratch of the on-GPU packer (fp6m_pack.hip): kPackTempBytes behind the partial-sum tiles.
int pack_temp(int dev, void** ptr)
{
    DeviceScratch* d = nullptr;
    const int rc = ensure_scratch(dev, &d);
    if (rc != FP6M_OK) return rc;
    *ptr = reinterpret_cast<unsigned char*>(d->ptr) + kScratchBytes;
    return FP6M_OK;
}

// m <= 16 configurations: rows of A per ring slot, WN x WK waves, ring depths of INT4 / FP6 tiles.
//   0: rows <= 4,  one tile x four k slices per workgroup, four ring slots (three for FP6 tiles)
//   1: rows <= 16, same shape, 1 KiB of A per slot
// Workgroups of several adjacent tiles (WN > 1) were measured and were never faster on MI355X; the
// kernel keeps the template parameter, only WN = 1 is instantiated.
template <int AROWS, int WN, int WK, int D4, int D6>
void launch_m16(const GemmArgs& a, bool g128, dim3 grid, hipStream_t stream)
{
    if (g128)
        hipLaunchKernelGGL((gemm_m16_kernel<true, AROWS, WN, WK, D4, D6>), grid, dim3(64 * WN * WK), 0, stream, a);
    else
        hipLaunchKernelGGL((gemm_m16_kernel<false, AROWS, WN, WK, D4, D6>), grid, dim3(64 * WN * WK), 0, stream, a);
}

struct M16Config {
    int id, wn, wk;
};

inline M16Config m16_config(int m)
{
    return m <= 4 ? M16Config{0, 1, 4} : M16Config{1, 1, 4};
}

inline void launch_m16_any(const M16Config& cfg, const GemmArgs& a, bool g128, dim3 grid, hipStream_t stream)
{
    if (cfg.id == 0)
        launch_m16<4, 1, 4, 4, 3>(a, g128, grid, stream);
    else
        launch_m16<16, 1, 4, 4, 3>(a, g128, grid, stream);
}

template <int MB, int D4, int D6>
void launch_mb(const GemmArgs& a, bool g128, int wk, dim3 grid, hipStream_t stream)
{
    if (wk == 8) {
        if (g128)
            hipLaunchKernelGGL((gemm_mb_kernel<true, MB, D4, D6, 8>), grid, dim3(512), 0, stream, a);
        else
            hipLaunchKernelGGL((gemm_mb_kernel<false, MB, D4, D6, 8>), grid, dim3(512), 0, stream, a);
    } else {
        if (g128)
            hipLaunchKernelGGL((gemm_mb_kernel<true, MB, D4, D6, 4>), grid, dim3(256), 0, stream, a);
        else
            hipLaunchKernelGGL((gemm_mb_kernel<false, MB, D4, D6, 4>), grid, dim3(256), 0, stream, a);
    }
}

void launch_wm(const GemmArgs& a, bool g128, int wn, dim3 grid, hipStream_t stream)
{
    if (wn == 2) {
        if (g128)
            hipLaunchKernelGGL((gemm_wm_kernel<true, 2>), grid, dim3(512), 0, stream, a);
        else
            hipLaunchKernelGGL((gemm_wm_kernel<false, 2>), grid, dim3(512), 0, stream, a);
    } else {
        if (g128)
            hipLaunchKernelGGL((gemm_wm_kernel<true, 1>), grid, dim3(512), 0, stream, a);
        else
            hipLaunchKernelGGL((gemm_wm_kernel<false, 1>), grid, dim3(512), 0, stream, a);
    }
}

}  // namespace fp6m

extern "C" {

int fp6m_last_hip_error(void) { return fp6m::g_last_hip_error; }

int fp6m_init(int dev)
{
    fp6m::DeviceScratch* d = nullptr;
    return fp6m::ensure_scratch(dev, &d);
}

}  // extern "C"

namespace fp6m {

// Optional work around the GEMM (fp6m_mul_fused); all null / zero for fp6m_mul.
struct Fusion {
    const int32_t* a_cols = nullptr;
    int lda = 0;
    const int32_t* c_cols = nullptr;
    const uint16_t* bias = nullptr;
    const uint16_t* residual = nullptr;
    int quant_rows = 0;              // > 0: row mix (fp6m_mul_rows), the last quant_rows rows of k are FP6
    bool native = false;             // weight planes in the gfx950 order (FP6M_LAYOUT_GFX950)
};

int mul_common(const void* A, const void* B, void* C, const void* s, int prob_m, int prob_n, int prob_k,
               void* workspace, int dev, void* stream, int thread_k, int thread_n, int sms, int max_par,
               int quant_cols, int group_size, const Fusion& fu)
{
    if (prob_m < 0 || prob_n < 0 || prob_k < 0) return FP6M_ERR_ARG;

    // Tile-shape arguments are validated the way the reference does it
    // (fp6_marlin_cuda_kernel.cu:890-905, 933-944) even though they do not pick a kernel here.
    if (fu.quant_rows > 0) {
        // the row mix is no reference path: its own rule is whole 128-column tiles (and, below, whole k units)
        if (prob_n % kTileN) return FP6M_ERR_PROB_SHAPE;
        if (prob_m == 0 || prob_n == 0) return FP6M_OK;
    } else {
        if (thread_k == -1 || thread_n == -1) {
            thread_k = prob_m <= 16 ? 128 : 64;
            thread_n = prob_m <= 16 ? 128 : 256;
        }
        if (thread_k <= 0 || thread_n <= 0) return FP6M_ERR_KERN_SHAPE;
        if (prob_n % thread_n != 0 || prob_k % thread_k != 0) return FP6M_ERR_PROB_SHAPE;
        if (prob_m == 0 || prob_n == 0 || prob_k == 0) return FP6M_OK;
        const bool small_tile = thread_k == 128 && thread_n == 128;
        const bool large_tile = thread_k == 64 && thread_n == 256;
        if (!(large_tile || (small_tile && prob_m <= 16))) return FP6M_ERR_KERN_SHAPE;
    }

    if (!A || !B || !C || !s || !workspace) return FP6M_ERR_ARG;
    if (max_par <= 0) return FP6M_ERR_ARG;
    int qc = quant_cols <= 0 ? 0 : quant_cols;
    if (quant_cols < -1 || qc > prob_n) return FP6M_ERR_ARG;
    const int n4 = prob_n - qc;
    if (n4 % kTileN || qc % kTileN) return FP6M_ERR_PROB_SHAPE;
    if (group_size != -1 && group_size != 128) return FP6M_ERR_ARG;
    const bool row_mix = fu.quant_rows > 0;
    const int k4 = prob_k - fu.quant_rows;                            // row mix: INT4 rows
    if (row_mix) {
        if (qc != 0 || group_size != 128 || fu.quant_rows >= prob_k) return FP6M_ERR_ARG;
        if (k4 % 128 || fu.quant_rows % 64) return FP6M_ERR_PROB_SHAPE;
    }
    const bool g128 = group_size == 128 && n4 > 0;
    if (g128 && prob_k % 128 && !row_mix) return FP6M_ERR_PROB_SHAPE;

    DeviceScratch* scratch = nullptr;
    if (int rc = ensure_scratch(dev, &scratch)) return rc;

    GemmArgs a;
    a.b_int4 = static_cast<const uint32_t*>(B);
    a.b_fp6_2 = a.b_int4 + (size_t)prob_k * n4 / 8;
    a.b_fp6_4 = a.b_fp6_2 + (size_t)prob_k * qc / 16;
    a.s_int4 = static_cast<const uint16_t*>(s);
    a.s_fp6 = a.s_int4 + (g128 ? (size_t)(prob_k / 128) * n4 : (size_t)n4);
    a.scratch = scratch->ptr;
    a.counters = static_cast<int*>(workspace);
    a.n = prob_n;
    a.k = prob_k;
    a.n4 = n4;
    a.qc = qc;
    a.tiles6 = qc / kTileN;
    a.tiles = prob_n / kTileN;
    a.k4 = 0;
    a.slices4 = 0;
    if (row_mix) {
        // every tile spans all n columns of both segments: INT4 words of rows [0, k4), then the FP6 planes of the rest
        a.b_fp6_2 = a.b_int4 + (size_t)k4 * prob_n / 8;
        a.b_fp6_4 = a.b_fp6_2 + (size_t)fu.quant_rows * prob_n / 16;
        a.s_fp6 = a.s_int4 + (size_t)(k4 / 128) * prob_n;
        a.qc = prob_n;
        a.k4 = k4;
    }
    a.native = fu.native;
    a.c_cols = fu.c_cols;
    a.bias = fu.bias;
    a.residual = nullptr;
    a.fused = fu.c_cols || fu.bias || fu.residual;
#ifdef FP6M_TIMELINE
    a.timeline = nullptr;
    if (const char* e = getenv("FP6M_TIMELINE_PTR")) a.timeline = reinterpret_cast<unsigned long long*>(strtoull(e, nullptr, 0));
#endif

    // Row blocks per workgroup pass: 32 rows up to m = 32, 64 rows (accumulators in 128 VGPRs, two
    // workgroups per CU) beyond.  128-row blocks (accumulators in AGPRs, one wave per SIMD) measured 10-15 %
    // faster for m >= 512 but left the register allocator no slack, and were dropped.
    int mb = prob_m <= 16 ? 1 : (prob_m <= 32 ? 2 : 4);
    if (const char* e = getenv("FP6M_MB")) {   // tuning/testing override
        const int v = atoi(e);
        if (prob_m > 16 && (v == 2 || v == 4)) mb = v;
    }
    // Launches of 1024 rows on large weights: four 64-row tiles share the dequantised fragments of a tile
    // (gemm_wm_kernel).  Measured on MI355X it beats the private-fragment kernel by 13-20 % there and loses
    // below (m = 512: 102 vs 96 us on 8192 x 8192), where its 256-row workgroups leave CUs idle.
    const long long rows_per_launch = prob_m < 64LL * max_par ? prob_m : 64LL * max_par;
    const long long weights = (long long)prob_n * prob_k;
    bool shared_frags = rows_per_launch >= 1024 && weights >= (64LL << 20);
    if (const char* e = getenv("FP6M_WM")) shared_frags = prob_m > 16 && atoi(e) != 0;   // tuning/testing override
    if (row_mix) shared_frags = false;                                // its waves run in lock step on one segment
    // Row mix: the kWaves * ks slices of a tile are dealt to the two segments in proportion to their cost (an FP6
    // step costs about two INT4 steps), at least one each.
    auto deal_slices = [&](int total) {
        const long long c4 = k4 / 32, c6 = 2LL * (fu.quant_rows / 32);
        long long n6 = (total * c6 + (c4 + c6) / 2) / (c4 + c6);
        if (n6 > fu.quant_rows / 64) n6 = fu.quant_rows / 64;
        if (n6 > total - 1) n6 = total - 1;
        if (n6 < 1) n6 = 1;
        return (int)(total - n6);
    };
    if (shared_frags) mb = 4;
    const int rows_per_tile = 16 * mb;
    const int mtiles_total = (prob_m + rows_per_tile - 1) / rows_per_tile;
    const int units = g128 ? prob_k / 128 : prob_k / 64;

    hipStream_t st = static_cast<hipStream_t>(stream);
    if (fu.a_cols) {
        const long long launch_rows = prob_m < (long long)rows_per_tile * max_par ? prob_m : (long long)rows_per_tile * max_par;
        if ((size_t)launch_rows * prob_k * sizeof(uint16_t) > kGatherBytes) return FP6M_ERR_ARG;
        if (int rc = ensure_gather_buffer(dev, scratch)) return rc;
    }
    for (int mt0 = 0; mt0 < mtiles_total; mt0 += max_par) {
        const int mtiles = mtiles_total - mt0 < max_par ? mtiles_total - mt0 : max_par;
        const int rows0 = mt0 * rows_per_tile;
        a.C = static_cast<uint16_t*>(C) + (size_t)rows0 * prob_n;
        a.residual = fu.residual ? fu.residual + (size_t)rows0 * prob_n : nullptr;
        a.m = prob_m - rows0 < mtiles * rows_per_tile ? prob_m - rows0 : mtiles * rows_per_tile;
        if (fu.a_cols) {
            // the launch's rows of A, gathered into the per-device buffer (stream order keeps the launches apart)
            dim3 ggrid((unsigned)((prob_k / 2 + 255) / 256), (unsigned)a.m);
            hipLaunchKernelGGL(gather_a_kernel, ggrid, dim3(256), 0, st,
                               static_cast<const uint16_t*>(A) + (size_t)rows0 * fu.lda, fu.lda, fu.a_cols,
                               scratch->gathered, prob_k);
            a.A = scratch->gathered;
        } else {
            a.A = static_cast<const uint16_t*>(A) + (size_t)rows0 * prob_k;
        }

        const size_t tile_bytes = (size_t)mb * 16 * kTileN * sizeof(float);
        const long long traffic_cap = (long long)prob_k / (64LL * a.m) > 0 ? (long long)prob_k / (64LL * a.m) : 1;
        long long env_ks = 0;
        if (const char* e = getenv("FP6M_KSPLIT")) env_ks = atoi(e);   // tuning/testing override
        if (shared_frags) {
            // two tiles per workgroup also share the A slabs: pays once the weights are large enough that
            // halving the grid still fills the chip (measured: 8192 x 16384 and up)
            int wn = weights >= (128LL << 20) ? 2 : 1;
            if (const char* e = getenv("FP6M_WN")) wn = atoi(e) == 2 ? 2 : 1;   // tuning/testing override
            const int wk = 2 / wn;
            a.groups6 = (a.tiles6 + wn - 1) / wn;
            a.groups4 = (a.tiles - a.tiles6 + wn - 1) / wn;
            const int groups_m = (mtiles + fp6m::kWmRows - 1) / fp6m::kWmRows;
            const long long base = (long long)(a.groups6 + a.groups4) * groups_m;
            long long ks = scratch->cus / base;
            const long long ks_k = units / (wk * 2) > 0 ? units / (wk * 2) : 1;
            const long long cap = (long long)prob_k / (16LL * rows_per_tile) > 0 ? (long long)prob_k / (16LL * rows_per_tile) : 1;
            if (ks > ks_k) ks = ks_k;
            if (ks > cap) ks = cap;
            if (sms > 0 && ks > sms) ks = sms;
            if (env_ks >= 1) ks = env_ks;
            if (ks < 1) ks = 1;
            while (ks > 1 && (size_t)a.tiles * mtiles * ks * tile_bytes > kScratchBytes) ks--;
            a.ksplit = (int)ks;
            dim3 grid((unsigned)((a.groups6 + a.groups4) * a.ksplit), (unsigned)groups_m);
            if (getenv("FP6M_VERBOSE"))
                fprintf(stderr, "fp6m_mul m=%d n=%d k=%d: shared fragments, %d tile(s) x %d k slice(s), row tiles %d ks=%d grid=%ux%u\n",
                        a.m, prob_n, prob_k, wn, wk, mtiles, a.ksplit, grid.x, grid.y);
            fp6m::launch_wm(a, g128, wn, grid, st);
        } else if (mb == 1) {
            // m <= 16.  Each region (FP6, INT4) has its own number of k parts (workgroups) per tile group;
            // FP6 steps cost about twice an INT4 step, so the FP6 region is split twice as finely.  The
            // split is bounded so that every wave keeps at least one k unit, partial-sum traffic stays
            // well below the weight stream and the partial tiles fit the scratch.
            const M16Config cfg = m16_config(a.m);
            a.groups6 = (a.tiles6 + cfg.wn - 1) / cfg.wn;
            a.groups4 = (a.tiles - a.tiles6 + cfg.wn - 1) / cfg.wn;
            const long long groups = a.groups6 + a.groups4;
            const long long ks_k = units / cfg.wk > 0 ? units / cfg.wk : 1;   // at least one k unit per wave
            // Measured on MI355X: the kernel is fastest with about one and a half workgroups per CU
            // (more concurrent k fronts cost DRAM efficiency, fewer leave CUs idle), as long as every
            // wave keeps at least four k steps.
            const long long target_wgs = (long long)scratch->cus * 3 / 2;
            long long ks = (target_wgs + groups / 2) / groups;
            const long long ks_steps = prob_k / 32 / (4 * cfg.wk) > 0 ? prob_k / 32 / (4 * cfg.wk) : 1;
            if (ks > ks_steps) ks = ks_steps;
            if (ks > ks_k) ks = ks_k;
            if (ks > traffic_cap) ks = traffic_cap;
            if (sms > 0 && ks > sms) ks = sms;
            if (env_ks >= 1) ks = env_ks;
            if (ks < 1) ks = 1;
            const size_t slot_bytes = (size_t)cfg.wn * 16 * kTileN * sizeof(float);
            while (ks > 1 && (size_t)(a.groups4 + 2 * a.groups6) * ks * slot_bytes > kScratchBytes) ks--;
            a.ks4 = (int)ks;
            a.ks6 = (int)(2 * ks <= ks_k ? 2 * ks : (ks > ks_k ? ks : ks_k));
            if (sms > 0 && a.ks6 > sms) a.ks6 = sms;
            a.ksplit = a.ks4;
            if (row_mix) {
                a.ks6 = 0;                                            // no FP6 column region: groups6 is 0
                a.slices4 = deal_slices(a.ks4 * cfg.wk);
            }
            dim3 grid((unsigned)(a.groups6 * a.ks6 + a.groups4 * a.ks4), 1);
            if (getenv("FP6M_VERBOSE"))
                fprintf(stderr, "fp6m_mul m=%d n=%d k=%d: cfg %d (%dx%d waves) groups %d+%d ks4=%d ks6=%d grid=%u\n", a.m, prob_n,
                        prob_k, cfg.id, cfg.wn, cfg.wk, a.groups6, a.groups4, a.ks4, a.ks6, grid.x);
            launch_m16_any(cfg, a, g128, grid, st);
        } else {
            // m > 16: a task is one workgroup (one tile x four k slices) on one row tile and k part.
            // Split k only as far as needed to give every CU a workgroup; partial tiles are 16*MB rows
            // of fp32, so the split is also capped by their traffic relative to the weight stream.
            const long long base = (long long)a.tiles * mtiles;
            long long ks = scratch->cus / base;
            const long long ks_k = units / (kWaves * 2) > 0 ? units / (kWaves * 2) : 1;
            const long long cap = (long long)prob_k / (16LL * rows_per_tile) > 0 ? (long long)prob_k / (16LL * rows_per_tile) : 1;
            if (ks > ks_k) ks = ks_k;
            if (ks > cap) ks = cap;
            if (sms > 0 && ks > sms) ks = sms;
            if (env_ks >= 1) ks = env_ks;
            if (ks < 1) ks = 1;
            while (ks > 1 && (size_t)base * ks * tile_bytes > kScratchBytes) ks--;
            a.ksplit = (int)ks;
            // A grid of at most one workgroup per CU would leave every SIMD a single wave: give the workgroup eight
            // k slices instead of four (same partial-sum traffic, two waves per SIMD) when k is long enough.
            int wk = base * ks <= scratch->cus && units / 16 >= ks ? 8 : kWaves;
            if (const char* e = getenv("FP6M_WK")) wk = atoi(e) == 8 ? 8 : kWaves;   // tuning/testing override
            if (row_mix) a.slices4 = deal_slices(a.ksplit * wk);
            dim3 grid((unsigned)(a.tiles * a.ksplit), (unsigned)mtiles);
            if (getenv("FP6M_VERBOSE"))
                fprintf(stderr, "fp6m_mul m=%d n=%d k=%d: MB=%d row tiles %d ks=%d k slices %d grid=%ux%u\n", a.m, prob_n, prob_k,
                        mb, mtiles, a.ksplit, wk, grid.x, grid.y);
            if (mb == 2) launch_mb<2, 4, 3>(a, g128, wk, grid, st);
            else launch_mb<4, 3, 3>(a, g128, wk, grid, st);
        }
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return hip_fail(e);
    }
    return FP6M_OK;
}

}  // namespace fp6m

extern "C" {

int fp6m_mul(const void* A, const void* B, void* C, const void* s, int prob_m, int prob_n, int prob_k,
             void* workspace, int dev, void* stream, int thread_k, int thread_n, int sms, int max_par,
             int quant_cols, int group_size)
{
    return fp6m::mul_common(A, B, C, s, prob_m, prob_n, prob_k, workspace, dev, stream, thread_k, thread_n, sms, max_par,
                            quant_cols, group_size, fp6m::Fusion{});
}

int fp6m_mul_fused(const void* A, int lda, const void* B, void* C, const void* s, int prob_m, int prob_n, int prob_k,
                   void* workspace, int dev, void* stream, int sms, int max_par, int quant_cols, int group_size,
                   const int32_t* a_cols, const int32_t* c_cols, const void* bias, const void* residual, int flags)
{
    fp6m::Fusion fu;
    if (flags & ~FP6M_LAYOUT_GFX950) return FP6M_ERR_ARG;
    fu.native = (flags & FP6M_LAYOUT_GFX950) != 0;
    fu.a_cols = a_cols;
    fu.lda = lda;
    fu.c_cols = c_cols;
    fu.bias = static_cast<const uint16_t*>(bias);
    fu.residual = static_cast<const uint16_t*>(residual);
    if (a_cols ? lda <= 0 : lda != prob_k) return FP6M_ERR_ARG;
    return fp6m::mul_common(A, B, C, s, prob_m, prob_n, prob_k, workspace, dev, stream, -1, -1, sms, max_par, quant_cols,
                            group_size, fu);
}

int fp6m_mul_rows(const void* A, int lda, const void* B, void* C, const void* s, int prob_m, int prob_n, int prob_k,
                  void* workspace, int dev, void* stream, int sms, int max_par, int quant_rows, const int32_t* a_cols,
                  const int32_t* c_cols, const void* bias, const void* residual, int flags)
{
    fp6m::Fusion fu;
    if (flags & ~FP6M_LAYOUT_GFX950) return FP6M_ERR_ARG;
    fu.native = (flags & FP6M_LAYOUT_GFX950) != 0;
    fu.a_cols = a_cols;
    fu.lda = lda;
    fu.c_cols = c_cols;
    fu.bias = static_cast<const uint16_t*>(bias);
    fu.residual = static_cast<const uint16_t*>(residual);
    fu.quant_rows = quant_rows;
    if (quant_rows <= 0) return FP6M_ERR_ARG;
    if (a_cols ? lda <= 0 : lda != prob_k) return FP6M_ERR_ARG;
    return fp6m::mul_common(A, B, C, s, prob_m, prob_n, prob_k, workspace, dev, stream, -1, -1, sms, max_par, -1, 128, fu);
}

}  // extern "C"
