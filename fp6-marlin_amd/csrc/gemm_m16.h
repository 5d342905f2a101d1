// gemm_m16_kernel: the m <= 16 (decode) kernel of fp6m_gemm.hip.
#pragma once
#include "gemm_common.h"

namespace fp6m {

// ------------------------------------------------------------------------------------------------ m <= 16: LDS-ring kernel
//
// Every wave keeps a private ring of DEPTH slots in LDS.  A slot is one k step (32 rows of k) of its
// tile's packed words (2 x 1 KiB 4-bit/INT4, + 2 x 512 B FP6 2-bit).  Slots are filled by direct-to-LDS
// global loads (no VGPR staging): lane L's data lands at slot + 16 L, so the *global* granule each lane
// fetches is permuted (inside aligned 64-byte quads, which keeps the loads coalesced) to obtain a layout
// that the permuted reads hit without bank conflicts.  The loads of step s + DEPTH - 1 are issued before
// step s is consumed; `s_waitcnt vmcnt` with a constant count is the only synchronisation in the loop.
// LDS reads are inline asm so that the compiler does not serialise them behind every outstanding
// direct-to-LDS load.
// The activations are fetched two steps at a time (a whole 128-byte line of every row per load) into a
// ring of their own behind the word slots: what limits a workgroup's rate is its requests in flight, and
// 64 bytes per row and step doubled the requests the activations cost (at m = 16 two fifths of all
// requests; one fetch per pair of steps took 6-10 % off those launches).

// Ring slots of A (one slot = a pair of steps): the pair being read, the pairs of the depth - 1 steps fetched
// ahead, and the one the next fetch fills.  A slot holds 128 bytes of each of its rows.
constexpr int pair_slots(int depth) { return (depth + 2) / 2; }
constexpr int pair_bytes(int arows) { return arows * 128; }
constexpr int a_ring_bytes(int depth, int arows) { return pair_slots(depth) * pair_bytes(arows); }
// Loads of n consecutive steps, the first with parity `first` within its pair: the words of each, and
// `a_ops` loads of A in front of every pair.
constexpr int newer_step_ops(int word_ops, int a_ops, int first, int n)
{
    int ops = word_ops * n;
    for (int t = 0; t < n; t++) ops += ((first + t) & 1) == 0 ? a_ops : 0;
    return ops;
}

struct StepRegs {
    u4 q0, q1;          // 4-bit plane / INT4 words of the two k-blocks
    u2 t0, t1;          // FP6 2-bit plane
    uint32_t a[4];      // activations in MFMA operand order
};

// AROWS = rows of A the ring holds (4 or 16).
template <bool FP6, bool G128, int DEPTH, int AROWS, typename Args>
__device__ __forceinline__ void stream_tile(const Args& p, const TileInfo& ti, unsigned char* ring,
                                            int step_begin, int step_end, f4 (&acc)[1][8])
{
    static_assert(DEPTH >= 3, "needs two steps of look-ahead");
    constexpr bool kGroup = G128 && !FP6;                 // group scales apply to INT4 tiles only
    constexpr int kPairSlots = pair_slots(DEPTH);         // step pairs of A alive at once
    constexpr int kPair = pair_bytes(AROWS);
    constexpr int kSlot = FP6 ? 3072 : 2048;              // a step's packed words
    constexpr int kWordOps = FP6 ? 3 : 2;                 // direct-to-LDS loads of the packed words per step
    constexpr int kAOps = AROWS == 16 ? 2 : 1;            // ... and of A per pair of steps
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
    // A: load o brings rows 8o .. 8o+7 (AROWS = 4: the lower half of the wave brings rows 0 .. 3), eight lanes
    // per row.  LDS position lane = 8 * row + chunk' holds the row's 16-byte chunk 4h + d (step parity h,
    // quarter d) at chunk' = 4h + (d ^ (row >> 1 & 3)).  Rows past m re-read row m-1, so the lanes that take
    // part never depend on m and neither does the count of loads in flight.
    const bool a_lane = AROWS == 16 || lane < 32;
    uint32_t vap[kAOps];
#pragma unroll
    for (int o = 0; o < kAOps; o++) {
        const int prow = (lane >> 3) & (AROWS - 1) & 7, pch = lane & 7;
        int row = ti.mtile * 16 + 8 * o + prow;
        row = row < p.m ? row : p.m - 1;
        vap[o] = (uint32_t)(row - ti.mtile * 16) * (uint32_t)p.k * 2 + 16 * ((pch & 4) | ((pch & 3) ^ ((prow >> 1) & 3)));
    }
    const unsigned char* base_a = reinterpret_cast<const unsigned char*>(p.A + (size_t)ti.mtile * 16 * p.k) +
                                  (size_t)(ti.a_step0 + step_begin) * 64;
    unsigned char* a_ring = ring + DEPTH * kSlot;
    const int last_pair = (step_end - step_begin) / 2 - 1;
    int pairs_issued = 0, pair_in = 0;
    const unsigned char* base_gs = reinterpret_cast<const unsigned char*>(p.s_int4 + (size_t)ti.tcol * kTileN);
    const uint32_t vgs = 4 * lane;
    constexpr int kScaleMask = DEPTH <= 5 ? 1 : 3;        // 256-byte slabs of group scales: 2 suffice up to depth 5
    unsigned char* gs_ring = a_ring + kPairSlots * kPair;

    int issued = step_begin;                              // next step to fetch (clamped at the last one)
    const int last = step_end - 1;
    // `even`: the step fetched is the first of its pair (counted from step_begin; a compile-time fact at every call)
    auto issue = [&](int slot, bool even) {
        unsigned char* dst = ring + slot * kSlot;
        if (even) {
            unsigned char* adst = a_ring + pair_in * kPair;
            if (a_lane) dma16(base_a + vap[0], adst);
            if (kAOps == 2) dma16(base_a + vap[kAOps - 1], adst + 1024);
            pair_in = pair_in + 1 == kPairSlots ? 0 : pair_in + 1;
            if (pairs_issued < last_pair) {               // (fetches past the end repeat the last pair)
                pairs_issued++;
                base_a += 128;
            }
        }
        dma16_stream(base4 + v4, dst);
        dma16_stream(base4 + row4 + v4, dst + 1024);
        if (FP6) dma16_stream(base2 + v2, dst + 2048);
        const bool scales = kGroup && (issued & 3) == 0;  // (never again once `issued` stops at the last, odd step)
        if (scales)
            dma4(base_gs + (size_t)(issued >> 2) * p.n4 * 2 + vgs, gs_ring + ((issued >> 2) & kScaleMask) * 256);
        if (issued < last) {                              // uniform: pointers move on the scalar unit
            issued++;
            base4 += 2 * row4;
            base2 += 2 * row2;
        }
        return scales;
    };
    // Loads that may stay in flight while the oldest fetched step must have landed: those of the DEPTH - 2 newer
    // steps, the first of which is the second of its pair (kWaitOdd) or the first (kWaitEven), plus the load of
    // group scales that closes the fetch of every fourth step, for as long as that step is among the newer ones
    // (left out of the count, it made two steps in four wait for a load issued only one step earlier).
    static_assert(!kGroup || DEPTH == 4, "the steps whose waits count a load of group scales are written out for depth 4");
    constexpr int kWaitOdd = newer_step_ops(kWordOps, kAOps, 1, DEPTH - 2);
    constexpr int kWaitEven = newer_step_ops(kWordOps, kAOps, 0, DEPTH - 2);

    // ---- read side (lane = MFMA identity)
    const int owner = p.native ? lane : 32 * sigma + 4 * l + i;   // whose granule of the k-block this lane needs
    const uint32_t ring_lds = lds_addr(ring);
    const uint32_t rd4 = ring_lds + (owner ^ ((owner >> 4) & 3)) * 16;
    const int gr2 = owner >> 1;
    const uint32_t rd2 = ring_lds + 2048 + (gr2 ^ (gr2 >> 4)) * 16 + (owner & 1) * 8;
    const int ar = c & (AROWS - 1);                       // rows beyond AROWS re-read a valid row; their sums are never stored
    uint32_t rda[4];
#pragma unroll
    for (int d = 0; d < 4; d++)
        rda[d] = lds_addr(a_ring) + (ar >> 3) * 1024 + (8 * (ar & 7) + (d ^ ((ar >> 1) & 3))) * 16 + 4 * i;
    const int q = i;                                      // result side: quarter of the column slots
    const uint32_t rdgs = lds_addr(gs_ring) + (64 * (q >> 1) + 4 * (q & 1)) * 2;

    // kReads LDS reads of one step, not waited for.
    auto fetch = [&](StepRegs& r, int slot, int pair_slot, bool odd) {
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
        const uint32_t ao = pair_slot * kPair;
        if (odd)                                // the second step of a pair: the other half of every row's line
            asm volatile("ds_read_b32 %0, %4 offset:64\n\tds_read_b32 %1, %5 offset:64\n\t"
                         "ds_read_b32 %2, %6 offset:64\n\tds_read_b32 %3, %7 offset:64"
                         : "=&v"(r.a[0]), "=&v"(r.a[1]), "=&v"(r.a[2]), "=&v"(r.a[3])
                         : "v"(rda[0] + ao), "v"(rda[1] + ao), "v"(rda[2] + ao), "v"(rda[3] + ao) : "memory");
        else
            asm volatile("ds_read_b32 %0, %4\n\tds_read_b32 %1, %5\n\tds_read_b32 %2, %6\n\tds_read_b32 %3, %7"
                         : "=&v"(r.a[0]), "=&v"(r.a[1]), "=&v"(r.a[2]), "=&v"(r.a[3])
                         : "v"(rda[0] + ao), "v"(rda[1] + ao), "v"(rda[2] + ao), "v"(rda[3] + ao) : "memory");
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
#pragma unroll
    for (int d = 0; d < DEPTH - 1; d++) {
        issue(slot_in, (d & 1) == 0);
        slot_in = slot_in + 1 == DEPTH ? 0 : slot_in + 1;
    }
    StepRegs regs[2];
    __builtin_amdgcn_s_waitcnt(vmcnt_only(kWaitOdd));         // step 0 has landed; step 1 is the oldest newer one
    FP6M_MARK(p, 1);
    fetch(regs[0], 0, 0, false);
    int slot_rd = 1;                                      // slot of the step whose LDS reads come next
    int pair_rd = 0;                                      // A ring slot of the pair that step belongs to
    bool scales_in_flight = false;
    f4 grp[8];
#pragma unroll 1
    for (int s = step_begin; s < step_end; s += kUnroll) {
#pragma unroll
        for (int u = 0; u < kUnroll; u++) {
            const bool scales = issue(slot_in, ((u + DEPTH - 1) & 1) == 0);
            slot_in = slot_in + 1 == DEPTH ? 0 : slot_in + 1;
            if (kGroup && u == 1) scales_in_flight = scales;              // the fetch of step s+4: a multiple of four
            const bool one_more = kGroup && (u == 1 || u == 2) && scales_in_flight;
            if (u & 1) {                                                  // step s+u+1 has landed
                if (one_more)
                    __builtin_amdgcn_s_waitcnt(vmcnt_only(kWaitOdd + 1));
                else
                    __builtin_amdgcn_s_waitcnt(vmcnt_only(kWaitOdd));
            } else {
                if (one_more)
                    __builtin_amdgcn_s_waitcnt(vmcnt_only(kWaitEven + 1));
                else
                    __builtin_amdgcn_s_waitcnt(vmcnt_only(kWaitEven));
            }
            if (u & 1) pair_rd = pair_rd + 1 == kPairSlots ? 0 : pair_rd + 1;   // step s+u+1 opens a pair
            fetch(regs[(u + 1) & 1], slot_rd, pair_rd, (u & 1) == 0);
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
    return max3(d4 * 2048 + a_ring_bytes(d4, arows) + scale_slab_bytes(d4), d6 * 3072 + a_ring_bytes(d6, arows),
                16 * kRedStride * 4);
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
// LOCAL: every workgroup that shares the tile runs on this XCD (xcd_place), so the partial tiles travel through its
// L2: stores acknowledged by the L2 and loads that bypass only the CU's own cache, instead of agent-scope accesses that
// go through to memory and back.  The counter stays an agent-scope atomic (atomics have no narrower scope); here it
// is a mask of the parts that have arrived rather than their number, so that a part arriving twice -- which would
// mean that two workgroups of one group of eight ran on the same XCD, against what the placement relies on -- is
// noticed: the tile is then stored as NaN instead of a sum with a part missing.
constexpr int kMaxLocalParts = 30;
constexpr unsigned kPoisoned = 1u << 31;
template <int WN, int WK, bool CELLS, bool LOCAL = false>
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
    const FusedCols fcols = fused_cols(p, tile_valid ? ti.col0 + 2 * lane : 0);
    auto store_row = [&](int m, float v0, float v1) {
        if (p.fused) {
            store_fused(p, fcols, (size_t)m, v0 * s0, v1 * s1);
            return;
        }
        h2 o = {(_Float16)(v0 * s0), (_Float16)(v1 * s1)};
        *reinterpret_cast<h2*>(c_out + (size_t)m * p.n) = o;
    };

    // Sum of the WK slices of my rows.
    // All LDS reads first (rows beyond m and waves without a tile read whatever the slab holds; it is never stored),
    // one wait, then the sums in slice order.
    f2 tv[RMAX][WK];
#pragma unroll
    for (int r = 0; r < RMAX; r++)
#pragma unroll
        for (int j = 0; j < WK; j++)
            tv[r][j] = *reinterpret_cast<const f2*>(reinterpret_cast<const float*>(smem + (j * WN + wn) * wave_lds) +
                                                    ((wk + r * WK) & 15) * kRedStride + 2 * lane);
    float v0[RMAX], v1[RMAX];
#pragma unroll
    for (int r = 0; r < RMAX; r++) {
        v0[r] = 0.f;
        v1[r] = 0.f;
        if (first_fp6 >= WK) {                                           // (uniform) the usual case: plain sums
#pragma unroll
            for (int j = 0; j < WK; j++) {
                v0[r] += tv[r][j][0];
                v1[r] += tv[r][j][1];
            }
        } else {
#pragma unroll
            for (int j = 0; j < WK; j++) {
                v0[r] += j >= first_fp6 ? tv[r][j][0] * x0 : tv[r][j][0];
                v1[r] += j >= first_fp6 ? tv[r][j][1] * x1 : tv[r][j][1];
            }
        }
    }
    if (ks == 1) {
#pragma unroll
        for (int r = 0; r < RMAX; r++)
            if (tile_valid && wk + r * WK < nrows) store_row(wk + r * WK, v0[r], v1[r]);
        return;
    }

    if constexpr (CELLS) {
        // The parts of the tile meet in its cells (see gemm_common.h): one returning atomic per element, values in output
        // units; whoever arrives last at an element stores it and writes its cell back to zero.  Nothing is published,
        // counted or gathered, and no barrier follows the sum through LDS.
        unsigned long long* cell = p.cells + (size_t)ti.tile * (16 * kTileN) + lane;   // [row][64 even | 64 odd columns]
        unsigned long long old[RMAX][2];
#pragma unroll
        for (int r = 0; r < RMAX; r++) {
            const int m = wk + r * WK;
            v0[r] *= s0;
            v1[r] *= s1;
            if (tile_valid && m < nrows) {
                old[r][0] = __hip_atomic_fetch_add(cell + m * kTileN, cell_contribution(v0[r]), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                old[r][1] = __hip_atomic_fetch_add(cell + m * kTileN + 64, cell_contribution(v1[r]), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
#pragma unroll
        for (int r = 0; r < RMAX; r++) {
            const int m = wk + r * WK;
            if (!(tile_valid && m < nrows)) continue;
#pragma unroll
            for (int e = 0; e < 2; e++) {
                if ((int)(old[r][e] >> 56) != ks - 1) continue;              // somebody else arrives last at this element
                const float v = cell_total(old[r][e], cell_contribution(e ? v1[r] : v0[r]), ks);
                __hip_atomic_store(cell + m * kTileN + 64 * e, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if (p.fused)
                    store_fused_one(p, fcols, (size_t)m, e, v);
                else
                    c_out[(size_t)m * p.n + e] = __builtin_bit_cast(uint16_t, (_Float16)v);
            }
        }
        FP6M_MARK(p, 6);
        return;
    }

    // Publish.  A slot holds [WN tiles][16 rows][128 columns] fp32: row m of a tile is 512 bytes, lane L's column
    // pair 8 bytes of it.  Rows wk + r * WK of this wave sit WK * 512 bytes apart: immediates below 4 KiB on one of two
    // lane offsets.
    constexpr int kSlotBytes = WN * 16 * kTileN * 4;
    const unsigned char* slot0 = reinterpret_cast<const unsigned char*>(p.scratch) + (size_t)slot_base * kSlotBytes +
                                 (size_t)wn * (16 * kTileN * 4);
    const unsigned char* my = uniform_ptr(slot0 + (size_t)ti.part * kSlotBytes);
    const uint32_t voff_lo = 8 * lane + 512 * wk, voff_hi = voff_lo + 4096;
    static_assert(WK == 4 || WK == 8, "row offsets of 2 or 4 KiB");
    if (tile_valid) {
#pragma unroll
        for (int r = 0; r < RMAX; r++)
            if (wk + r * WK < nrows) {                                   // (uniform)
                const f2 v = {v0[r], v1[r]};
                st8_row<!LOCAL>(my, voff_lo, voff_hi, r * WK * 512, __builtin_bit_cast(unsigned long long, v));
            }
    }
    // Every wave waits until its own partial-sum stores are acknowledged (agent scope: written through to memory and
    // so visible to every other CU; XCD-local: by this XCD's L2, which every reader of the tile shares), and only then
    // joins the barrier in front of the counter increment.  A workgroup-scope fence alone would not wait for them, and
    // neither does s_barrier.
    __builtin_amdgcn_s_waitcnt(vmcnt_only(0));
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");               // (keeps the compiler from moving accesses across)
    __syncthreads();
    FP6M_MARK(p, 4);
    if (threadIdx.x == 0) {
        if constexpr (LOCAL) {
            const unsigned mine = 1u << ti.part, all = (1u << ks) - 1;
            const unsigned seen = __hip_atomic_fetch_or(reinterpret_cast<unsigned*>(counter), mine, __ATOMIC_RELAXED,
                                                        __HIP_MEMORY_SCOPE_AGENT);
            if (seen & mine) {                                           // this part has been here before
                __hip_atomic_fetch_or(reinterpret_cast<unsigned*>(counter), kPoisoned, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                *flag = 2;
            } else {
                *flag = ((seen | mine) & all) == all ? ((seen & kPoisoned) ? 2 : 1) : 0;
            }
        } else {
            const int seen = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            *flag = seen == ks - 1;
        }
    }
    __syncthreads();
    FP6M_MARK(p, 5);
    const int finish = *flag;
    if (!finish) return;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
#pragma unroll
    for (int r = 0; r < RMAX; r++) {
        v0[r] = 0.f;
        v1[r] = 0.f;
    }
    // Gather: the loads of up to PCHUNK parts in flight together (rows past m are read too, they lie inside the slot,
    // and never stored), then the sums in part order.
    const unsigned char* part0 = uniform_ptr(slot0);
    for (int pp = 0; pp < ks; pp += PCHUNK) {
        unsigned long long t[PCHUNK][RMAX];
#pragma unroll
        for (int u = 0; u < PCHUNK; u++)
            if (tile_valid && pp + u < ks) {                             // (uniform)
                const unsigned char* src = part0 + (size_t)(pp + u) * kSlotBytes;
#pragma unroll
                for (int r = 0; r < RMAX; r++) t[u][r] = ld8_row<!LOCAL>(src, voff_lo, voff_hi, r * WK * 512);
            }
        __builtin_amdgcn_s_waitcnt(vmcnt_only(0));
#pragma unroll
        for (int u = 0; u < PCHUNK; u++)
            if (tile_valid && pp + u < ks) {
#pragma unroll
                for (int r = 0; r < RMAX; r++) {
                    settle64(t[u][r]);
                    const f2 v = __builtin_bit_cast(f2, t[u][r]);
                    v0[r] += v[0];
                    v1[r] += v[1];
                }
            }
    }
    if (LOCAL && finish == 2) {                                          // (see above: never on a device that fp6m_init has looked at)
        const float nan = __builtin_nanf("");
#pragma unroll
        for (int r = 0; r < RMAX; r++) v0[r] = v1[r] = nan;
    }
#pragma unroll
    for (int r = 0; r < RMAX; r++)
        if (tile_valid && wk + r * WK < nrows) store_row(wk + r * WK, v0[r], v1[r]);
    FP6M_MARK(p, 6);
    if (threadIdx.x == 0) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// CELLS: tiles shared by several workgroups are summed in the accumulate-and-count cells (up to four rows) instead of
// through published partial tiles; a compile-time choice, because the mere presence of the other path behind a
// run-time branch cost the partial-tile path 0.3-0.6 us (4096 x 4096 at 16 rows: 8.9 -> 9.4 us).
// EXTRAS = false: the build for calls without row mix, fused epilogue or gfx950 word order (their arguments are
// overwritten with constants; their presence cost the plain call 2-3 %).
// LOCAL: the workgroups of a tile are placed on one XCD and exchange their partial tiles through its L2.
template <bool G128, int AROWS, int WN, int WK, int D4, int D6, bool CELLS, bool EXTRAS = true, bool LOCAL = false>
// second launch-bound argument = waves per SIMD the register budget must allow (HIP semantics)
__global__ __launch_bounds__(64 * WN * WK, WK == 8 || AROWS == 16 ? 2 : 3) void gemm_m16_kernel(const GemmArgs args)
{
    static_assert(!LOCAL || (WN == 1 && !CELLS), "the cells are atomics, which have no XCD-local form");
    constexpr int NW = WN * WK;
    constexpr int kWaveLds = wave_lds_bytes(D4, D6, AROWS);
    __shared__ __attribute__((aligned(16))) unsigned char smem[NW * kWaveLds + 16];

    GemmArgs p = args;
    if constexpr (!EXTRAS) {
        p.k4 = 0;
        p.slices4 = 0;
        p.native = 0;
        p.fused = 0;
        p.c_cols = nullptr;
        p.bias = nullptr;
        p.residual = nullptr;
    }
    preload_args<false>(args);
    FP6M_MARK(p, 0);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // scalar: addresses stay on the SALU
    const int wn = wave % WN, wk = wave / WN;
    TileInfo ti;
    int group;
    bool later = false;                                                  // a tile of the second class of INT4 tiles
    if constexpr (LOCAL) {
        const XcdPlace pl = xcd_place(p, blockIdx.x, p.groups6, p.groups4);
        if (!pl.valid) return;                                           // (the grid is padded to a multiple of eight)
        ti.fp6 = pl.fp6;
        ti.part = pl.part;
        group = pl.group;
    } else {
        // (two classes of INT4 tiles: in launch order, so that the workgroups of the second class are the later ones)
        const int logical = p.groups4b > 0 ? (int)blockIdx.x : xcd_contiguous_id(blockIdx.x, gridDim.x);
        const int wgs6 = p.groups6 * p.ks6;                              // the FP6 region's workgroups come first
        ti.fp6 = logical < wgs6;
        int local = ti.fp6 ? logical : logical - wgs6;
        const int wgs4 = p.groups4 * p.ks4;
        later = !ti.fp6 && local >= wgs4;                                // (never with one class)
        if (later) local -= wgs4;
        const int groups = ti.fp6 ? p.groups6 : (later ? p.groups4b : p.groups4);
        // (the entries are read at fixed kernarg offsets and selected by value: an index computed here would turn
        // into a second, dependent scalar load, which measured 0.4 us before the first weight load)
        const FastDiv gdiv = {ti.fp6 ? p.div[1].d : (later ? p.div_b.d : p.div[0].d),
                              ti.fp6 ? p.div[1].magic : (later ? p.div_b.magic : p.div[0].magic)};
        ti.part = fast_div(gdiv, local);                                 // part-major: neighbours share k, adjoin in n
        group = local - ti.part * groups + (later ? p.groups4 : 0);
    }
    const int ks = ti.fp6 ? p.ks6 : (later ? p.ks4b : p.ks4);
    const WaveRule wrule = {ti.fp6 ? p.wrule[1].lo : (later ? p.wrule_b.lo : p.wrule[0].lo),
                            ti.fp6 ? p.wrule[1].ly : (later ? p.wrule_b.ly : p.wrule[0].ly),
                            ti.fp6 ? p.wrule[1].eo : (later ? p.wrule_b.eo : p.wrule[0].eo),
                            ti.fp6 ? p.wrule[1].ey : (later ? p.wrule_b.ey : p.wrule[0].ey)};
    ti.tcol = group * WN + wn;
    ti.region_n = ti.fp6 ? p.qc : p.n4;
    const bool tile_valid = ti.tcol * kTileN < ti.region_n;
    ti.tile = ti.fp6 ? ti.tcol : p.tiles6 + ti.tcol;
    ti.mtile = 0;
    ti.later = later;
    ti.col0 = (ti.fp6 ? p.n4 : 0) + ti.tcol * kTileN;

    constexpr int unit_steps = G128 ? 4 : 2;
    const int kp = ti.part * WK + wk;
    int step_begin = wave_rule_begin(wrule, WK, ti.part, wk) * unit_steps;
    int step_end = wave_rule_begin(wrule, WK, ti.part, wk + 1) * unit_steps;
    ti.a_step0 = 0;
    const bool region6 = ti.fp6;                                         // the workgroup's column region
    if (p.k4) row_mix_slice(p, kp, ti, step_begin, step_end);            // per wave: INT4 or FP6 rows of the tile

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
    const int slot_base = region6 ? group * p.ks6
                                  : (later ? p.groups6 * p.ks6 + p.groups4 * p.ks4 + (group - p.groups4) * p.ks4b
                                           : p.groups6 * p.ks6 + group * p.ks4);
    int* counter = p.counters + (region6 ? group : p.groups6 + group);
    wg_finish<WN, WK, CELLS, LOCAL>(p, ti, tile_valid, wn, wk, ks, slot_base, counter, acc, !p.k4 && (ti.fp6 || !G128), smem,
                                    kWaveLds, reinterpret_cast<int*>(smem + NW * kWaveLds),
                                    p.k4 ? p.slices4 - ti.part * WK : WK);
    FP6M_MARK(p, 7);
}

}  // namespace fp6m
