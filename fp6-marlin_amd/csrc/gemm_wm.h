// gemm_wm_kernel: a large-m kernel of fp6m_gemm.hip (four row tiles share a tile's dequantised fragments); the
// dispatcher prefers the 128-row tiles of gemm_mb.h, this one is reached through the tuning hook.
// Uses the MFMA, A-ring and epilogue pieces of gemm_mb.h.
#pragma once
#include "gemm_mb.h"

namespace fp6m {

// ------------------------------------------------------------------------------------------------ 128 < m: fragments shared by four row tiles
//
// The m > 16 kernel spends more issue slots on dequantisation than on MFMAs (a SIMD issues both from one
// pipe), and every row tile repeats that work.  Here a workgroup is eight waves = four row tiles (64 rows
// each) x two k slices of ONE tile: the four waves of a k slice fetch the tile's words once, each
// dequantises a quarter of a step's operand fragments (one 16-column group) into LDS, and all four multiply
// from there.  One workgroup barrier per step publishes the fragments and hands ring slots back to the
// fetches; A stays private to its wave.  LDS per k slice: a ring of five steps of words [+ 2-bit plane], a ring of
// three steps of A (four 4 KiB slabs each), two 8 KiB fragment buffers, two rows of group scales.

constexpr int kWmRows = 4;                                           // row tiles per workgroup
// WN adjacent tiles x (2 / WN) k slices: with WN = 2 the two tiles' waves also share the A slabs.
// LDS of a k slice: a ring of kWmWordDepth steps of packed words (3 KiB per tile and step), a ring of kWmADepth steps
// of A (a 4 KiB slab per row tile), two fragment buffers per tile, two rows of group scales per tile.  The words are
// small and come from memory, so they are fetched four steps ahead; A comes from the L2 and takes most of the LDS, so
// it is fetched two steps ahead.
constexpr int kWmWordDepth = 5, kWmADepth = 3;
template <int WN> constexpr int wm_a_off() { return kWmWordDepth * WN * 3072; }
template <int WN> constexpr int wm_frag_off() { return wm_a_off<WN>() + kWmADepth * kWmRows * 4096; }
template <int WN> constexpr int wm_scale_off() { return wm_frag_off<WN>() + WN * 2 * 8192; }
template <int WN> constexpr int wm_filler_off() { return wm_scale_off<WN>() + WN * 512; }   // 256 bytes nobody reads
template <int WN> constexpr int wm_slice_lds() { return wm_filler_off<WN>() + 256; }
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
    // VMW: before the first read of the next step's A, wait until at most VMW vector-memory loads (the ones issued
    // after that A) are outstanding.
    template <int phase, int VMW, typename Hook>
    static __device__ __forceinline__ void run(WmState& st, f4 (&acc)[4][8], Hook&& hook)
    {
        if constexpr (BLK < 4) {
            constexpr int nb = BLK + 2;
            uint32_t (&dst)[4] = st.abuf[(phase + nb) & 3];
            if constexpr (nb < 4) {
                lds_read_a4<nb * 1024>(dst, st.addr_cur);
            } else {
                if constexpr (nb == 4) __builtin_amdgcn_s_waitcnt(vmcnt_only(VMW));
                lds_read_a4<(nb - 4) * 1024>(dst, st.addr_next);
            }
            if constexpr (BLK > 0) __builtin_amdgcn_s_waitcnt(lgkmcnt_only(8));
            uint32_t (&src)[4] = st.abuf[(phase + BLK) & 3];
            asm volatile("" : "+v"(src[0]), "+v"(src[1]), "+v"(src[2]), "+v"(src[3]));
            const h8 av = __builtin_bit_cast(h8, u4{src[0], src[1], src[2], src[3]});
            step<0>(st, acc, av, hook);
            WmBlocks<BLK + 1>::template run<phase, VMW>(st, acc, hook);
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
    constexpr int MB = 4, WM = kWmRows;
    constexpr bool kGroup = G128 && !FP6;
    constexpr int kWSlot = WN * 3072;                                // a step's words of the WN tiles (3 KiB each, FP6 or not)
    constexpr int kASlot = WM * 4096;
    constexpr int kALoads = WN == 1 ? 4 : 2;                         // direct-to-LDS loads of A per wave and step
    constexpr int kGroupOps = kALoads + 1;                           // ... and one load of the words' side
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
    const uint32_t w_off = uniform32(wn * 3072);                      // this tile's words inside a word slot
    const uint32_t a_off = uniform32(wm_a_off<WN>() + wm * 4096);     // this row tile's slab (shared by the WN tiles)

    // Every wave issues, per step, its loads of A for the step two on and then exactly ONE load of the words' side
    // for the step four on (k-block 0 / k-block 1 / the 2-bit plane / the group scales; a wave whose share does not
    // exist for this tile or step loads 256 bytes into a corner of LDS that nobody reads), so that the counts in the waits below
    // are the same for every wave.
    int issued_a = step_begin, issued_w = step_begin;
    const int last = step_end - 1;
    auto issue_a = [&](int slot) {
        set_m0(slice_lds + a_off + slot * kASlot);
        if (WN == 1 || wn == 0) {                                     // with two tiles, each loads half of the slab
            dma16_m0<0, false>(base_a, va[0]);
            dma16_m0<1024, false>(base_a, va[1]);
        }
        if (WN == 1 || wn == 1) {
            dma16_m0<2048, false>(base_a, va[2]);
            dma16_m0<3072, false>(base_a, va[3]);
        }
        if (issued_a < last) {
            issued_a++;
            base_a += 64;
        }
    };
    auto issue_w = [&](int slot) {
        const uint32_t dst = slice_lds + slot * kWSlot + w_off;
        if (wm == 0) {
            set_m0(dst);
            dma16_m0<0, true>(base4, v4);
        } else if (wm == 1) {
            set_m0(dst);
            dma16_m0<1024, true>(base4, v4b);
        } else if (FP6 && wm == 2) {
            set_m0(dst + 2048);
            dma16_m0<0, true>(base2, v2);
        } else if (kGroup && wm == 3 && (issued_w & 3) == 0) {
            set_m0(gs_lds + ((issued_w >> 2) & 1) * 256);
            dma4_m0(base_gs + (size_t)(issued_w >> 2) * (size_t)uniform32(p.n4) * 2, vgs);
        } else {
            // (into LDS, not a register: a register nobody reads would be reused while the load is in flight)
            set_m0(slice_lds + wm_filler_off<WN>());
            dma4_m0(base4, vgs);
        }
        if (issued_w < last) {
            issued_w++;
            base4 += 2 * row4;
            base2 += 2 * row2;
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
        const uint32_t so = slot * kWSlot;
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
        const uint32_t so = slot * kASlot;
#pragma unroll
        for (int d = 0; d < 4; d++) addr[d] = rda[d] + so;
    };

    issue_a(0);
    issue_a(1);
#pragma unroll
    for (int d = 0; d < kWmWordDepth - 1; d++) issue_w(d);
    __builtin_amdgcn_s_waitcnt(vmcnt_only(0));                        // the steps fetched ahead: this wave's loads ...
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
    int a_in = 2, a_rd = 1, w_in = kWmWordDepth - 1, w_rd = 1;
#pragma unroll 1
    for (int s = step_begin; s < loop_end; s += kUnroll) {
#pragma unroll
        for (int u = 0; u < kUnroll; u++) {
            // The words' side of step s+u+1 has landed (this wave's share: the loads of the last two steps, issued
            // after it, may be outstanding) and the fragments of step s+u are written, for everybody; everybody has
            // left step s+u-1, whose A slot the loads of step s+u+2 overwrite and whose fragment buffer this step's
            // dequantisation refills (its word slot was read a step earlier still).
            __builtin_amdgcn_s_waitcnt(vmcnt_only(2 * kGroupOps) & lgkmcnt_only(0));
            __builtin_amdgcn_s_barrier();
            issue_a(a_in);
            issue_w(w_in);
            a_in = a_in + 1 == kWmADepth ? 0 : a_in + 1;
            w_in = w_in + 1 == kWmWordDepth ? 0 : w_in + 1;
            if (s >= step_end) continue;                              // (uniform) only keeping step with the others
#pragma unroll
            for (int d = 0; d < 4; d++) st.addr_cur[d] = st.addr_next[d];
            slot_addrs(st.addr_next, a_rd);
            fetch_raw(w_rd);
            const bool next_group = kGroup && u == kUnroll - 1;       // step s+u+1 starts a 128-row group
            if (next_group) fetch_scales((s + u + 1) >> 2);
            a_rd = a_rd + 1 == kWmADepth ? 0 : a_rd + 1;
            w_rd = w_rd + 1 == kWmWordDepth ? 0 : w_rd + 1;
            fetch_frags(u & 1);
            auto hook = [&](auto blk, auto t) {
                constexpr int mslot = decltype(blk)::value * 8 + decltype(t)::value;   // MFMA just issued
                if constexpr (mslot == 8) {
                    if (next_group) settle_scales();
                }
                if constexpr (mslot >= 8 && mslot < 24 && (mslot & 3) == 0) chunk((mslot - 8) >> 2);
                if constexpr (mslot == 31) publish((u + 1) & 1);
            };
            // the A of step s+u+1 was fetched a step ago: behind it in the queue are that step's load of the words'
            // side and this step's loads
            WmBlocks<>::template run<0, kGroupOps + 1>(st, acc, hook);
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

    preload_args(p);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wm = wave % WM, wn = WN == 2 ? wave / WM : 0, wk = WN == 2 ? 0 : wave / WM;
    const int logical = xcd_contiguous_id(blockIdx.x, gridDim.x);
    const int group = fast_div(p.div[0], logical);                   // WN adjacent tiles of one region
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

    // k slices: part-major, then wk; every wave of the workgroup runs the longest slice's step count.  Longer
    // slices come last (SliceRule), so begin + longest stays inside k for every slice that has work; a slice
    // without work keeps step with the others on steps [0, longest).
    constexpr int unit_steps = G128 ? 4 : 2;
    const int sl = ti.part * WK + wk;
    int step_begin = slice_begin(p.rule[0], sl) * unit_steps;
    int step_end = slice_begin(p.rule[0], sl + 1) * unit_steps;
    const int longest = (p.rule[0].q + (ti.part * WK + WK - 1 >= p.rule[0].first_long ? 1 : 0)) * unit_steps;
    if (step_begin == step_end) step_begin = step_end = 0;

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
    wg_finish_mb<MB, WK>(p, ti, wk, p.ksplit, (ti.mtile * p.tiles + ti.tile) * p.ksplit, acc, ti.fp6 || !G128,
                         smem + grp * WK * kWmRegion, kWmRegion, reinterpret_cast<int*>(smem + wm_lds<WN>() - 64) + grp, valid);
}

}  // namespace fp6m
