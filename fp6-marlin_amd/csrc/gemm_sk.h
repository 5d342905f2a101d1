// gemm_sk_kernel: the decode kernel (m <= 4) of fp6m_gemm.hip for weights mixed along n.
#pragma once
#include "gemm_m16.h"

namespace fp6m {

// ------------------------------------------------------------------------------------------------ m <= 4: one wave per workgroup, equal shares
//
// The wave-level loop is gemm_m16.h's stream_tile (private LDS ring, direct-to-LDS loads, no barrier).  What
// differs is how work reaches the waves and how the parts of a column tile meet.
//
// Partition.  The reference's striped scheduler (fp6_marlin_cuda_kernel.cu:343-408) gives every CTA the same
// number of (k tile, n tile) units and lets a CTA run over the end of one column slice into the next; the property
// is that every SM streams the same number of bytes whatever the tile count.  Same property here at the
// granularity of a wave: a workgroup is ONE wave, and the (tile, k unit) pairs of a region, tile-major, are cut
// into one contiguous share per wave, equal to within one unit.  A wave walks its share segment by segment (a
// segment = its part of one tile).  The host picks the number of waves; shares shorter than a tile are chosen to
// divide it, so that only long shares ever cross a tile boundary.  INT4 and FP6 tiles are separate regions with
// their own unit length and share.  Nothing in the kernel synchronises waves: no barrier, no LDS shared
// between them.
//
// Reduction.  A segment that covers its tile's whole k range is scaled and stored.  Otherwise the tile is shared,
// and its parts meet in one 64-bit cell per output element in device memory: every wave adds, with ONE returning
// agent-scope atomic per element,
//         2^56  +  2^47  +  round(value * 2^29)            (count | biased fixed-point value, |value| < 2^17)
// to the cell.  The value returned tells the wave how many parts had arrived before it and what they summed to:
// the one that finds count == parts - 1 holds the complete sum (old sum + its own part), converts it, stores C and
// writes the cell back to zero.  Publish, count and gather are a single round trip to memory instead of three
// dependent ones, nobody spins, and because integer addition is associative the result does not depend on the
// order of arrival: results are bit-identical from run to run.  Values are in output units (after the scales), so
// the fixed-point grid of 2^-29 is at most 1/32 ulp of any normal fp16 result, and the range of +-2^17 exceeds
// fp16's; a part that is not finite or is out of range saturates, which makes the element infinite.  The cells
// live in the scratch region that belongs to the call's workspace, are zero when no call is in flight, and are left
// zero.
constexpr int kCellFracBits = 29;
constexpr unsigned long long kCellBias = 1ull << 47;        // makes every part's contribution positive
constexpr unsigned long long kCellOne = 1ull << 56;         // the arrival count sits above the sum
constexpr unsigned long long kCellSumMask = kCellOne - 1;
constexpr int kMaxParts = 255;                              // 255 * (2^47 + 2^46) < 2^56
constexpr size_t kCellBytes = size_t(8) << 20;              // cells of one workspace: n * m * 8 bytes at most

// Kernel arguments, laid out as three 64-byte blocks that the kernel fetches itself with three scalar loads
// behind one wait (left to the compiler, the loads of the fields come in several dependent batches, each a
// round trip to a cold line before the wave's first weight load).
struct SkArgs {
    // block 0
    const uint16_t* A;
    const uint32_t* b_int4;   // INT4 words
    const uint32_t* b_fp6_2;  // FP6 2-bit plane
    const uint32_t* b_fp6_4;  // FP6 4-bit plane
    const uint16_t* s_int4;   // per-column (permuted order) or [k/128][n4] group scales
    const uint16_t* s_fp6;    // per-column (permuted order)
    uint16_t* C;
    unsigned long long* cells;
    // block 1
    int m, n, k;
    int n4, qc;               // columns in the INT4 / FP6 region
    int tiles6;               // FP6 tiles come first in the tile list
    int waves, waves6;        // all waves; the FP6 region's come first
    int units4, units6;       // k units per tile (INT4: 128 rows with group scales, else 64; FP6: 64 rows)
    int q4, r4, q6, r6;       // shares: wave j of a region owns q units from j * q + min(j, r) on, one more if j < r
    int native, fused;
    // block 2: n / d as (n * magic) >> 40 for d = units4, units6, q4, q4 + 1, q6, q6 + 1 (exact for n < 2^24, d < 2^16)
    unsigned long long magic_u4, magic_u6, magic_q4, magic_q4p, magic_q6, magic_q6p;
    const int32_t* c_cols;    // optional epilogue work (fp6m_mul_fused), as in GemmArgs
    const uint16_t* bias;
    // block 3 (two more scalar loads)
    const uint16_t* residual;
    unsigned long long* timeline;   // performance debugging builds only
    static constexpr int k4 = 0;    // (the row mix does not come here)
};
static_assert(sizeof(SkArgs) == 208 && offsetof(SkArgs, m) == 64 && offsetof(SkArgs, magic_u4) == 128 &&
              offsetof(SkArgs, residual) == 192, "three 64-byte blocks and a tail");

__device__ __forceinline__ SkArgs load_sk_args()
{
    typedef uint32_t u16v __attribute__((ext_vector_type(16)));
    typedef uint32_t u4v __attribute__((ext_vector_type(4)));
    u16v b0, b1, b2;
    u4v b3;
    const uint64_t ka = (uint64_t)__builtin_amdgcn_kernarg_segment_ptr();
    asm volatile(
        "s_load_dwordx16 %0, %4, 0x0\n\ts_load_dwordx16 %1, %4, 0x40\n\ts_load_dwordx16 %2, %4, 0x80\n\t"
        "s_load_dwordx4 %3, %4, 0xc0\n\ts_waitcnt lgkmcnt(0)"
        : "=&s"(b0), "=&s"(b1), "=&s"(b2), "=&s"(b3) : "s"(ka));
    struct Words {
        uint32_t w[52];
    } raw;
#pragma unroll
    for (int i = 0; i < 16; i++) {
        raw.w[i] = b0[i];
        raw.w[16 + i] = b1[i];
        raw.w[32 + i] = b2[i];
    }
#pragma unroll
    for (int i = 0; i < 4; i++) raw.w[48 + i] = b3[i];
    return __builtin_bit_cast(SkArgs, raw);
}

__device__ __forceinline__ uint32_t mul_shift40(unsigned long long magic, uint32_t n)
{
    return (uint32_t)(((unsigned long long)n * magic) >> 40);
}

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

// Wave that owns unit x of a region whose shares are (q, r): the first r waves hold q + 1 units.
__device__ __forceinline__ int sk_owner(uint32_t x, int q, int r, unsigned long long magic_q, unsigned long long magic_qp)
{
    const uint32_t head = (uint32_t)r * (uint32_t)(q + 1);
    return x < head ? (int)mul_shift40(magic_qp, x) : r + (int)mul_shift40(magic_q, x - head);
}

// End of a segment.  `parts` = waves that share the tile (1: this segment is the whole tile); s0, s1 = the scales
// of the lane's two columns (1 where group scales were applied in the loop).
__device__ __forceinline__ void wave_finish_sk(const SkArgs& p, const TileInfo& ti, int parts, f4 (&acc)[1][8], float s0,
                                               float s1, unsigned char* ring)
{
    typedef float f2 __attribute__((ext_vector_type(2)));
    const int lane = threadIdx.x;
    const int c = lane & 15, q = lane >> 4;
    const int nrows = p.m;                                               // <= 4
    // MFMA fragments -> fp32 rows in the drained ring (lane c holds row c of the tile's 16), read back with lane L
    // owning columns 2L, 2L+1.  LDS operations of one wave execute in order: no barrier is needed.
    float* slab = reinterpret_cast<float*>(ring);
    if (c < nrows) {
        float* mine = slab + c * kRedStride + 64 * (q >> 1) + 4 * (q & 1);
#pragma unroll
        for (int t = 0; t < 8; t++) *reinterpret_cast<f4*>(mine + 16 * (t >> 1) + 8 * (t & 1)) = acc[0][t];
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    float v0[4], v1[4];
#pragma unroll
    for (int r = 0; r < 4; r++) {
        const f2 t = *reinterpret_cast<const f2*>(slab + (r < nrows ? r : 0) * kRedStride + 2 * lane);
        v0[r] = t[0] * s0;
        v1[r] = t[1] * s1;
    }
    FP6M_MARK(p, 3);

    uint16_t* c_out = p.C + ti.col0 + 2 * lane;
    const FusedCols fcols = fused_cols(p, ti.col0 + 2 * lane);
    if (parts == 1) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
            if (r >= nrows) continue;
            if (p.fused) {
                store_fused(p, fcols, (size_t)r, v0[r], v1[r]);
            } else {
                const h2 o = {(_Float16)v0[r], (_Float16)v1[r]};
                *reinterpret_cast<h2*>(c_out + (size_t)r * p.n) = o;
            }
        }
        return;
    }

    // Shared tile: one returning atomic per element (cells of a row: 64 of the even columns, then 64 of the odd).
    unsigned long long* cell = p.cells + (size_t)ti.tile * nrows * kTileN + lane;
    unsigned long long add[4][2], old[4][2];
#pragma unroll
    for (int r = 0; r < 4; r++) {
        add[r][0] = cell_contribution(v0[r]);
        add[r][1] = cell_contribution(v1[r]);
        if (r < nrows) {
            old[r][0] = __hip_atomic_fetch_add(cell + r * kTileN, add[r][0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            old[r][1] = __hip_atomic_fetch_add(cell + r * kTileN + 64, add[r][1], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    FP6M_MARK(p, 4);
#pragma unroll
    for (int r = 0; r < 4; r++) {
        if (r >= nrows) continue;
#pragma unroll
        for (int e = 0; e < 2; e++) {
            if ((int)(old[r][e] >> 56) != parts - 1) continue;           // somebody else arrives last at this element
            const float v = cell_total(old[r][e], add[r][e], parts);
            __hip_atomic_store(cell + r * kTileN + 64 * e, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (p.fused) {
                store_fused_one(p, fcols, (size_t)r, e, v);
            } else {
                c_out[(size_t)r * p.n + e] = __builtin_bit_cast(uint16_t, (_Float16)v);
            }
        }
    }
    FP6M_MARK(p, 6);
}

template <bool FP6, bool G128>
__device__ __forceinline__ void sk_wave(const SkArgs& p, int j, unsigned char* ring)
{
    constexpr int unit_steps = G128 && !FP6 ? 4 : 2;
    constexpr int DEPTH = FP6 ? 3 : 4;
    constexpr bool kColumnScale = FP6 || !G128;
    const int q = FP6 ? p.q6 : p.q4, r = FP6 ? p.r6 : p.r4;
    const int units = FP6 ? p.units6 : p.units4;
    uint32_t u = (uint32_t)j * (uint32_t)q + (uint32_t)(j < r ? j : r);
    const uint32_t u_end = u + (uint32_t)q + (j < r ? 1u : 0u);
    TileInfo ti;
    ti.fp6 = FP6;
    ti.mtile = 0;
    ti.part = 0;
    ti.a_step0 = 0;
    ti.region_n = FP6 ? p.qc : p.n4;
    ti.tcol = (int)mul_shift40(FP6 ? p.magic_u6 : p.magic_u4, u);
    while (u < u_end) {                                                  // (uniform) one segment per trip
        const int kb = (int)u - ti.tcol * units;
        const int left = (int)(u_end - u);
        const int len = units - kb < left ? units - kb : left;           // units of this tile in my share
        ti.tile = FP6 ? ti.tcol : p.tiles6 + ti.tcol;
        ti.col0 = (FP6 ? p.n4 : 0) + ti.tcol * kTileN;
        h2 sv = {(_Float16)1.0f, (_Float16)1.0f};
        if (kColumnScale) {                                              // fetched now, used after the loop
            const int nr = ti.tcol * kTileN + 2 * (int)threadIdx.x;      // even column inside the region
            sv = *reinterpret_cast<const h2*>((FP6 ? p.s_fp6 : p.s_int4) + (nr & ~31) + scale_slot(nr & 31));
        }
        f4 acc[1][8];
#pragma unroll
        for (int t = 0; t < 8; t++) acc[0][t] = f4{0.f, 0.f, 0.f, 0.f};
        stream_tile<FP6, G128, DEPTH, 4>(p, ti, ring, kb * unit_steps, (kb + len) * unit_steps, acc);
        FP6M_MARK(p, 2);
        int parts = 1;
        if (len < units) {
            const uint32_t t0 = (uint32_t)ti.tcol * (uint32_t)units;
            const unsigned long long mq = FP6 ? p.magic_q6 : p.magic_q4, mqp = FP6 ? p.magic_q6p : p.magic_q4p;
            parts = sk_owner(t0 + units - 1, q, r, mq, mqp) - sk_owner(t0, q, r, mq, mqp) + 1;
        }
        u += len;
        wave_finish_sk(p, ti, parts, acc, (float)sv[0], (float)sv[1], ring);
        ti.tcol++;
    }
}

constexpr int kSkWaveLds = wave_lds_bytes(4, 3, 4);

// second launch-bound argument = waves per SIMD the register budget must allow (HIP semantics)
template <bool G128>
__global__ __launch_bounds__(64, 3) void gemm_sk_kernel(const SkArgs in_kernarg_segment)
{
    __shared__ __attribute__((aligned(16))) unsigned char smem[kSkWaveLds];
    const SkArgs p = load_sk_args();
    FP6M_MARK(p, 0);
#ifdef FP6M_TIMELINE
    if (p.timeline) {                                                    // where the wave runs: HW_ID and XCC_ID registers
        const uint32_t hw = __builtin_amdgcn_s_getreg((4 << 0) | (0 << 6) | (31 << 11));
        const uint32_t xcc = __builtin_amdgcn_s_getreg((20 << 0) | (0 << 6) | (3 << 11));
        p.timeline[(size_t)blockIdx.x * 8 + 5] = ((unsigned long long)xcc << 32) | hw;
    }
#endif
    const int logical = xcd_contiguous_id(blockIdx.x, p.waves);
    if (logical < p.waves6)                                              // the FP6 region's waves come first
        sk_wave<true, G128>(p, logical, smem);
    else
        sk_wave<false, G128>(p, logical - p.waves6, smem);
    FP6M_MARK(p, 7);
}

}  // namespace fp6m
