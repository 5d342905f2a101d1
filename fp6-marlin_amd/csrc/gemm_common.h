// Shared pieces of the GEMM kernels (fp6m_gemm.hip): argument block, tile bookkeeping, the fused store, direct-to-LDS
// load and s_waitcnt helpers, and the register-level dequantisers.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

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
constexpr size_t kScratchBytes = size_t(16) << 20;           // partial-sum scratch of one workspace
constexpr size_t kPackTempBytes = size_t(1) << 20;           // the packer's flag and per-column maxima

// Slice i of a tile's k range, in units (two k steps; four with group scales): the first `first_long` slices hold q
// units, the others q + 1, so that inside a workgroup the longer slices come last (the lock-step kernel lets every
// wave run the longest slice's step count from its own begin, which must stay inside k).
struct SliceRule {
    int q, first_long;
};
__host__ __device__ inline int slice_begin(const SliceRule& r, int i)
{
    const int extra = i - r.first_long;
    return i * r.q + (extra > 0 ? extra : 0);
}

// The k slices of a tile by wave, in units.  A workgroup of eight waves puts two on every SIMD, and the SIMD serves
// the one that arrived first (waves 0-3) ahead of the other (waves 4-7): with equal slices the second wave of every
// SIMD leaves its loop a third later than the first (8192 x 8192 at 128 rows: 14.3 against 19.6 us), and the
// workgroup's reduction waits for it.  So a part (workgroup) of a tile gives its first four waves `lo` units each and
// the others `ly` <= lo; what does not divide goes, a unit each, to the first `eo` older waves in (part, wave) order,
// then to the first `ey` younger ones.  Four-wave workgroups have older waves only.  Slices follow each other along
// k in (part, wave) order.
struct WaveRule {
    int lo, ly, eo, ey;
};
__host__ __device__ inline int wave_rule_begin(const WaveRule& r, int wk, int part, int wave)
{
    const int no = 4, ny = wk - 4;
    const int eo_before = r.eo < no * part ? r.eo : no * part, ey_before = r.ey < ny * part ? r.ey : ny * part;
    int eo_here = r.eo - no * part, ey_here = r.ey - ny * part;
    eo_here = eo_here < 0 ? 0 : (eo_here > no ? no : eo_here);
    ey_here = ey_here < 0 ? 0 : (ey_here > ny ? ny : ey_here);
    const int base = part * (no * r.lo + ny * r.ly) + eo_before + ey_before;
    if (wave < no) return base + wave * r.lo + (wave < eo_here ? wave : eo_here);
    const int y = wave - no;                               // (wave == wk: the begin of the next part)
    return base + no * r.lo + eo_here + y * r.ly + (y < ey_here ? y : ey_here);
}

// n / d for n, d < 65536 as the high half of n * ceil(2^32 / d) (exact in that range: the error term n * e / 2^32 stays
// below 1 / d); magic 0 stands for a plain division (d = 1, or operands out of range).
struct FastDiv {
    uint32_t d, magic;
};
__device__ __forceinline__ int fast_div(const FastDiv& f, int n)
{
    if (f.magic) return (int)__umulhi((uint32_t)n, f.magic);
    return f.d == 1 ? n : n / (int)f.d;
}

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
    // Division-free bookkeeping, prepared by the host (a 64-bit division costs a wave hundreds of scalar
    // instructions before its first load):
    SliceRule rule[2];        // k slices of a tile (row mix): [0] INT4 tiles / INT4 rows, [1] FP6
    WaveRule wrule[2];        // ... (everything else): [0] INT4 tiles, [1] FP6 tiles
    FastDiv div[2];           // m <= 16: by groups4 / groups6;  m > 16: by ks4 / ks6
    // weight planes in the gfx950 order (fp6m_repack_gfx950): [tile][k-block][MFMA lane] instead of the reference's
    // [k-block][64-column group][fragment owner]
    int native;
    // optional epilogue work (fp6m_mul_fused); `fused` is set when any of the three is
    const int32_t* c_cols;    // column of C that packed column j goes to
    const uint16_t* bias;     // fp16 [n], indexed by C column
    const uint16_t* residual; // fp16 [m, n], same rows as C
    int fused;
    unsigned long long* cells;   // m <= 16: the shared tiles' parts meet here instead of in `scratch` (null: they do not)
    // Workgroups that share a tile placed on one XCD (xcd_tile_of): their partial tiles then meet in that XCD's L2.
    // xm4_lo / xm4_hi: 2^32 / (INT4 tiles per XCD, rounded down / up); xm6_*: the same for the FP6 tiles.  (Separate
    // fields, selected by value: an indexed table makes the compiler copy the argument block to scratch memory.)
    int xcd_local;
    uint32_t xm4_lo, xm4_hi, xm6_lo, xm6_hi;
    // m <= 16, two classes of INT4 tiles: the first groups4 tiles in ks4 parts each (their workgroups, with the FP6
    // region's, are the first of the grid: one per CU), the other groups4b tiles in ks4b finer parts (the later
    // workgroups, which share those CUs).  groups4b == 0: one class.
    int groups4b, ks4b;
    WaveRule wrule_b;
    FastDiv div_b;            // by groups4b
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

// Kernel arguments are fetched with scalar loads that the compiler otherwise issues where each field is first used:
// three or four dependent round trips (0.2-0.4 us each on a cold kernarg buffer) before a wave's first weight load.
// Naming the fields in one asm statement at the top makes them one batch behind a single wait.
// (Only the fields the kernel uses: all of them at once would not fit the scalar registers, and the compiler would
// fall back to two batches with spills in between.)  LARGE_M: the m > 16 kernel, which has no use for the m <= 16
// kernel's tile groups, cells and XCD placement.
template <bool LARGE_M, bool CLASSES = true>
__device__ __forceinline__ void preload_args(const GemmArgs& p)
{
    if constexpr (LARGE_M && !CLASSES) {
        // (the build with the row mix and the fused epilogue: the statements its schedule was tuned with)
        asm volatile("" : : "s"(p.A), "s"(p.b_int4), "s"(p.b_fp6_2), "s"(p.b_fp6_4), "s"(p.C), "s"(p.s_int4), "s"(p.s_fp6),
                            "s"(p.scratch), "s"(p.counters), "s"(p.cells), "s"(gridDim.x));
        asm volatile("" : : "s"(p.m), "s"(p.n), "s"(p.k), "s"(p.n4), "s"(p.qc), "s"(p.tiles6), "s"(p.tiles), "s"(p.ksplit),
                            "s"(p.ks6), "s"(p.ks4), "s"(p.groups6), "s"(p.groups4), "s"(p.k4), "s"(p.slices4), "s"(p.native));
        asm volatile("" : : "s"(p.rule[0].q), "s"(p.rule[0].first_long), "s"(p.rule[1].q), "s"(p.rule[1].first_long),
                            "s"(p.div[0].d), "s"(p.div[0].magic), "s"(p.div[1].d), "s"(p.div[1].magic), "s"(p.fused));
        asm volatile("" : : "s"(p.xcd_local), "s"(p.xm4_lo), "s"(p.xm4_hi), "s"(p.xm6_lo), "s"(p.xm6_hi));
        asm volatile("" : : "s"(p.wrule[0].lo), "s"(p.wrule[0].ly), "s"(p.wrule[0].eo), "s"(p.wrule[0].ey), "s"(p.wrule[1].lo),
                            "s"(p.wrule[1].ly), "s"(p.wrule[1].eo), "s"(p.wrule[1].ey));
        return;
    }
    // (The wait for the batch stands in front of the first statement, and the compiler issues the loads that only later
    // statements name behind it: the first statement therefore names the fields at the far end of the block as well.)
    if constexpr (CLASSES)
        asm volatile("" : : "s"(p.A), "s"(p.b_int4), "s"(p.b_fp6_2), "s"(p.b_fp6_4), "s"(p.C), "s"(p.s_int4), "s"(p.s_fp6),
                            "s"(p.scratch), "s"(p.counters), "s"(gridDim.x), "s"(p.groups4b), "s"(p.ks4b), "s"(p.wrule_b.lo),
                            "s"(p.wrule_b.ly), "s"(p.wrule_b.eo), "s"(p.wrule_b.ey), "s"(p.div_b.d), "s"(p.div_b.magic));
    else
        asm volatile("" : : "s"(p.A), "s"(p.b_int4), "s"(p.b_fp6_2), "s"(p.b_fp6_4), "s"(p.C), "s"(p.s_int4), "s"(p.s_fp6),
                            "s"(p.scratch), "s"(p.counters), "s"(gridDim.x));
    asm volatile("" : : "s"(p.m), "s"(p.n), "s"(p.k), "s"(p.n4), "s"(p.qc), "s"(p.tiles6), "s"(p.tiles), "s"(p.ksplit),
                        "s"(p.ks6), "s"(p.ks4), "s"(p.k4), "s"(p.slices4), "s"(p.native));
    asm volatile("" : : "s"(p.rule[0].q), "s"(p.rule[0].first_long), "s"(p.rule[1].q), "s"(p.rule[1].first_long),
                        "s"(p.div[0].d), "s"(p.div[0].magic), "s"(p.div[1].d), "s"(p.div[1].magic), "s"(p.fused));
    asm volatile("" : : "s"(p.wrule[0].lo), "s"(p.wrule[0].ly), "s"(p.wrule[0].eo), "s"(p.wrule[0].ey), "s"(p.wrule[1].lo),
                        "s"(p.wrule[1].ly), "s"(p.wrule[1].eo), "s"(p.wrule[1].ey));
    if constexpr (!LARGE_M) {
        asm volatile("" : : "s"(p.cells), "s"(p.groups6), "s"(p.groups4));
        asm volatile("" : : "s"(p.xcd_local), "s"(p.xm4_lo), "s"(p.xm4_hi), "s"(p.xm6_lo), "s"(p.xm6_hi));
    }
}

// The XCD (accelerator die: 32 CUs with an L2 of their own) this wave runs on.
__device__ __forceinline__ int xcc_id()
{
    int v;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(v));
    return v & 15;
}

// Placement of a 1-D grid's workgroups so that all k parts of a tile run on one XCD.  The hardware deals the workgroups
// of a dispatch to the XCDs round robin, starting at an XCD that depends on the queue: workgroups 8i .. 8i + 7 run on
// eight different XCDs, but which of them runs where is only known to the workgroup itself (XCC_ID).  So a workgroup is
// identified by (x = the XCD it finds itself on, i = index / 8).  The tile list [FP6 tiles | INT4 tiles] is dealt to
// the XCDs round robin; XCD x's workgroups, in the order of i, walk its FP6 tiles part-major (ks6 parts each), then
// its INT4 tiles part-major (ks4 parts each).  The grid is 8 x the largest per-XCD count, so some workgroups are idle.
// (fp6m_init checks the eight-different-XCDs property on the device before the dispatcher uses this; the reduction
// itself notices a (tile, part) that arrives twice, see wg_finish.)
struct XcdPlace {
    bool valid, fp6;
    int group, part;         // tile index inside its region, k part
};
__device__ __forceinline__ XcdPlace xcd_place(const GemmArgs& p, int b, int tiles6, int tiles4)
{
    XcdPlace r;
    const int x = xcc_id() & 7, i = b >> 3;
    const int c6 = (tiles6 + 7 - x) >> 3;                   // FP6 tiles f with f % 8 == x
    const int g0 = (x - tiles6) & 7;                        // first INT4 tile of this XCD
    const int c4 = (tiles4 + 7 - g0) >> 3;
    const int w6 = c6 * p.ks6;
    r.fp6 = i < w6;
    const int li = r.fp6 ? i : i - w6;
    const int c = r.fp6 ? c6 : c4;
    const int lo = (r.fp6 ? tiles6 : tiles4) >> 3;
    const uint32_t magic_lo = r.fp6 ? p.xm6_lo : p.xm4_lo, magic_hi = r.fp6 ? p.xm6_hi : p.xm4_hi;
    const uint32_t magic = c == lo ? magic_lo : magic_hi;
    r.part = c <= 1 ? li : (int)__umulhi((uint32_t)li, magic);
    const int j = li - r.part * c;
    r.group = (r.fp6 ? x : g0) + 8 * j;
    r.valid = c > 0 && r.part < (r.fp6 ? p.ks6 : p.ks4);
    return r;
}
// Epilogue of fp6m_mul_fused for the two adjacent packed columns a lane owns: C[row, c_cols[col]] =
// fp16(v + bias[c_cols[col]] + residual[row, c_cols[col]]), everything added in fp32 and rounded once.
// The lane's destination columns and bias are looked up once (FusedCols), the rows then only add and store.
// Map entries are clamped to the row so that a bad map cannot write outside C.
struct FusedCols {
    int c0, c1;
    float b0, b1;
};
template <typename Args>
__device__ __forceinline__ FusedCols fused_cols(const Args& p, int col)
{
    FusedCols f;
    f.c0 = col;
    f.c1 = col + 1;
    f.b0 = f.b1 = 0.f;
    if (!p.fused) return f;
    if (p.c_cols) {
        f.c0 = p.c_cols[col];
        f.c1 = p.c_cols[col + 1];
        f.c0 = f.c0 < 0 ? 0 : (f.c0 >= p.n ? p.n - 1 : f.c0);
        f.c1 = f.c1 < 0 ? 0 : (f.c1 >= p.n ? p.n - 1 : f.c1);
    }
    if (p.bias) {
        f.b0 = (float)__builtin_bit_cast(_Float16, p.bias[f.c0]);
        f.b1 = (float)__builtin_bit_cast(_Float16, p.bias[f.c1]);
    }
    return f;
}
template <typename Args>
__device__ __forceinline__ void store_fused(const Args& p, const FusedCols& f, size_t row, float v0, float v1)
{
    v0 += f.b0;
    v1 += f.b1;
    const size_t r = row * (size_t)p.n;
    if (p.residual) {
        v0 += (float)__builtin_bit_cast(_Float16, p.residual[r + f.c0]);
        v1 += (float)__builtin_bit_cast(_Float16, p.residual[r + f.c1]);
    }
    p.C[r + f.c0] = __builtin_bit_cast(uint16_t, (_Float16)v0);
    p.C[r + f.c1] = __builtin_bit_cast(uint16_t, (_Float16)v1);
}

// One of the two: element e (0 / 1) of the lane's column pair.
template <typename Args>
__device__ __forceinline__ void store_fused_one(const Args& p, const FusedCols& f, size_t row, int e, float v)
{
    const int col = e ? f.c1 : f.c0;
    v += e ? f.b1 : f.b0;
    const size_t at = row * (size_t)p.n + col;
    if (p.residual) v += (float)__builtin_bit_cast(_Float16, p.residual[at]);
    p.C[at] = __builtin_bit_cast(uint16_t, (_Float16)v);
}

// ------------------------------------------------------------------------------------------------ cells
// One 64-bit cell per output element of a tile that several waves or workgroups share: every part adds
//         2^56  +  2^47  +  round(value * 2^29)            (count | biased fixed-point value, |value| < 2^17)
// with one returning agent-scope atomic; whoever reads back count == parts - 1 holds the complete sum.
constexpr int kCellFracBits = 29;
constexpr unsigned long long kCellBias = 1ull << 47;        // makes every part's contribution positive
constexpr unsigned long long kCellOne = 1ull << 56;         // the arrival count sits above the sum
constexpr unsigned long long kCellSumMask = kCellOne - 1;
constexpr int kMaxParts = 255;                              // 255 * (2^47 + 2^46) < 2^56
constexpr size_t kCellBytes = size_t(8) << 20;              // cells of one workspace: n * m * 8 bytes at most


__device__ __forceinline__ unsigned long long cell_contribution(float x)
{
    const float lim = 131071.0f;
    float y = x < lim ? x : lim;                            // (NaN compares false: it saturates high)
    y = y > -lim ? y : -lim;
    const long long f = (long long)(y * (float)(1ll << kCellFracBits));
    return kCellOne + kCellBias + (unsigned long long)f;
}

// The complete sum as a float: `old` is what the atomic returned, `mine` what this wave added.
__device__ __forceinline__ float cell_total(unsigned long long old, unsigned long long mine, int parts)
{
    const unsigned long long sum = ((old + mine) & kCellSumMask) - (unsigned long long)parts * kCellBias;
    return (float)(long long)sum * (1.0f / (float)(1ll << kCellFracBits));
}


// ------------------------------------------------------------------------------------------------ tile bookkeeping

struct TileInfo {
    int tile, part, mtile;   // tile in the [FP6 | INT4] tile list, k partner index, m-tile
    bool fp6;
    int tcol;                // tile index inside its region
    int region_n;            // columns of the region
    int col0;                // first column of the tile in C
    int a_step0;             // k step of A that step 0 of the wave's weight segment multiplies (row mix: k4 / 32)
    bool later;              // m > 16: an INT4 tile of the second class (ks4b parts, the grid's last workgroups)
};

// Row mix: slice `sl` of a tile's slices -> its segment (ti.fp6, ti.a_step0) and its steps there.
__device__ __forceinline__ void row_mix_slice(const GemmArgs& p, int sl, TileInfo& ti, int& begin, int& end)
{
    ti.fp6 = sl >= p.slices4;
    if (!ti.fp6) {
        begin = slice_begin(p.rule[0], sl) * 4;
        end = slice_begin(p.rule[0], sl + 1) * 4;
        ti.a_step0 = 0;
    } else {
        begin = slice_begin(p.rule[1], sl - p.slices4) * 2;
        end = slice_begin(p.rule[1], sl - p.slices4 + 1) * 2;
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
template <typename Args>
__device__ __forceinline__ PlaneGeometry plane_geometry(const Args& p, const TileInfo& ti)
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

// A kernel argument as a value the optimiser cannot look through: it otherwise turns a selection among three arguments
// into a selection among their addresses and one dependent scalar load (0.2-0.4 us in front of the first weight load).
__device__ __forceinline__ int held(int v)
{
    asm volatile("" : "+s"(v));
    return v;
}
__device__ __forceinline__ uint32_t held(uint32_t v)
{
    asm volatile("" : "+s"(v));
    return v;
}

// The m > 16 kernel's workgroup: blockIdx.x walks the FP6 tiles' (tile, k part) pairs first (ks6 parts each), then the
// INT4 tiles' (ks4 parts each); blockIdx.y the row tiles.
template <bool CLASSES = true>
__device__ __forceinline__ TileInfo locate_tile(const GemmArgs& p)
{
    TileInfo t;
    // (two classes of INT4 tiles: in launch order, so that the workgroups of the second class are the last to start)
    const int logical = CLASSES && p.groups4b > 0 ? (int)blockIdx.x : xcd_contiguous_id(blockIdx.x, gridDim.x);
    const int wgs6 = p.tiles6 * p.ks6;
    t.fp6 = logical < wgs6;
    int local = t.fp6 ? logical : logical - wgs6;
    const int first4 = p.tiles - p.tiles6 - p.groups4b;      // INT4 tiles of the first class
    // (uniform, like everything here; said so explicitly because the compiler otherwise keeps what hangs on it in vector
    // registers, and the loops' scalar-base loads need their addresses in scalar ones)
    t.later = CLASSES && p.groups4b > 0 && __builtin_amdgcn_readfirstlane((int)(!t.fp6 && local >= first4 * p.ks4)) != 0;
    if (t.later) local -= first4 * p.ks4;
    // (the entries are read at fixed offsets and selected by value: an index would become a dependent scalar load)
    FastDiv kdiv;
    int ks;
    kdiv = FastDiv{t.fp6 ? p.div[1].d : p.div[0].d, t.fp6 ? p.div[1].magic : p.div[0].magic};
    ks = t.fp6 ? p.ks6 : p.ks4;
    if constexpr (CLASSES) {
        const uint32_t db = held(p.div_b.d), mb = held(p.div_b.magic);
        const int kb = held(p.ks4b);
        kdiv = FastDiv{t.later ? db : kdiv.d, t.later ? mb : kdiv.magic};
        ks = t.later ? kb : ks;
    }
    const int q = __builtin_amdgcn_readfirstlane(fast_div(kdiv, local));
    t.part = local - q * ks;
    t.tcol = q + (t.later ? first4 : 0);
    t.tile = t.fp6 ? t.tcol : p.tiles6 + t.tcol;
    t.mtile = blockIdx.y;
    t.region_n = t.fp6 ? p.qc : p.n4;
    t.col0 = (t.fp6 ? p.n4 : 0) + t.tcol * kTileN;
    t.a_step0 = 0;
    return t;
}

// k range of one wave in steps of 32 (two k-blocks).  Units of two steps (four with group scales) keep
// every wave's step count even and group-aligned.
template <bool G128, int WK = kWaves>
__device__ __forceinline__ void wave_k_range(const GemmArgs& p, bool fp6, bool later, int part, int wave, int& begin, int& end)
{
    constexpr int unit_steps = G128 ? 4 : 2;
    // (the entries are read at fixed offsets and selected by value: an index would become a dependent scalar load)
    WaveRule rule;
    if (later) {                                           // (uniform; false at compile time where there is one class)
        rule = WaveRule{held(p.wrule_b.lo), held(p.wrule_b.ly), held(p.wrule_b.eo), held(p.wrule_b.ey)};
    } else {
        rule = WaveRule{fp6 ? p.wrule[1].lo : p.wrule[0].lo, fp6 ? p.wrule[1].ly : p.wrule[0].ly,
                        fp6 ? p.wrule[1].eo : p.wrule[0].eo, fp6 ? p.wrule[1].ey : p.wrule[0].ey};
    }
    begin = wave_rule_begin(rule, WK, part, wave) * unit_steps;
    end = wave_rule_begin(rule, WK, part, wave + 1) * unit_steps;
}

// ------------------------------------------------------------------------------------------------ loads, waits, dequantisers

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
// (the same with the destination already an LDS-space pointer)
__device__ __forceinline__ void dma16(const void* gsrc, FP6M_AS3 unsigned char* lds_dst)
{
    __builtin_amdgcn_global_load_lds((const FP6M_AS1 void*)gsrc, (FP6M_AS3 void*)lds_dst, 16, 0, 0);
}
__device__ __forceinline__ void dma16_stream(const void* gsrc, FP6M_AS3 unsigned char* lds_dst)
{
    __builtin_amdgcn_global_load_lds((const FP6M_AS1 void*)gsrc, (FP6M_AS3 void*)lds_dst, 16, 0, 2);
}
__device__ __forceinline__ void dma4(const void* gsrc, FP6M_AS3 unsigned char* lds_dst)
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

// 8-byte accesses of the partial tiles in scalar-base form: address = sbase + voff + OFF, so a tile's rows and parts
// cost no vector address arithmetic (the compiler's own code for them was ten instructions and a branch per access,
// and a last-arriving workgroup spent a microsecond issuing them).  AGENT: the access goes through to memory (visible
// to every XCD); otherwise it stops at this XCD's L2 and only bypasses the CU's own cache.  The loads are invisible to
// the compiler's wait insertion: callers wait (vmcnt) and pass the results through settle64 before using them.
template <int OFF, bool AGENT>
__device__ __forceinline__ void st8_sbase(const void* sbase, uint32_t voff, unsigned long long v)
{
    static_assert(OFF >= 0 && OFF < 4096, "13-bit signed immediate");
    if constexpr (AGENT)
        asm volatile("global_store_dwordx2 %0, %1, %2 offset:%3 sc1" : : "v"(voff), "v"(v), "s"(sbase), "n"(OFF) : "memory");
    else
        asm volatile("global_store_dwordx2 %0, %1, %2 offset:%3 sc0" : : "v"(voff), "v"(v), "s"(sbase), "n"(OFF) : "memory");
}
template <int OFF, bool AGENT>
__device__ __forceinline__ unsigned long long ld8_sbase(const void* sbase, uint32_t voff)
{
    static_assert(OFF >= 0 && OFF < 4096, "13-bit signed immediate");
    unsigned long long v;
    if constexpr (AGENT)
        asm volatile("global_load_dwordx2 %0, %1, %2 offset:%3 sc1" : "=v"(v) : "v"(voff), "s"(sbase), "n"(OFF) : "memory");
    else
        asm volatile("global_load_dwordx2 %0, %1, %2 offset:%3 sc0" : "=v"(v) : "v"(voff), "s"(sbase), "n"(OFF) : "memory");
    return v;
}
__device__ __forceinline__ void settle64(unsigned long long& v) { asm volatile("" : "+v"(v)); }
// The same for byte offset `row_bytes` (a multiple of 2 KiB below 8 KiB, constant once the caller's loop is unrolled)
// from lane offsets `lo` and `hi` = lo + 4096.
template <bool AGENT>
__device__ __forceinline__ void st8_row(const void* sbase, uint32_t lo, uint32_t hi, int row_bytes, unsigned long long v)
{
    switch (row_bytes) {
    case 0: st8_sbase<0, AGENT>(sbase, lo, v); break;
    case 2048: st8_sbase<2048, AGENT>(sbase, lo, v); break;
    case 4096: st8_sbase<0, AGENT>(sbase, hi, v); break;
    default: st8_sbase<2048, AGENT>(sbase, hi, v); break;
    }
}
template <bool AGENT>
__device__ __forceinline__ unsigned long long ld8_row(const void* sbase, uint32_t lo, uint32_t hi, int row_bytes)
{
    switch (row_bytes) {
    case 0: return ld8_sbase<0, AGENT>(sbase, lo);
    case 2048: return ld8_sbase<2048, AGENT>(sbase, lo);
    case 4096: return ld8_sbase<0, AGENT>(sbase, hi);
    default: return ld8_sbase<2048, AGENT>(sbase, hi);
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

}  // namespace fp6m
