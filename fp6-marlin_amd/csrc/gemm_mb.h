// gemm_mb_kernel: the 16 < m kernel of fp6m_gemm.hip (private rings, MB 16-row blocks per wave, asm MFMAs).
#pragma once
#include "gemm_common.h"

namespace fp6m {

// ------------------------------------------------------------------------------------------------ 16 < m: ring kernel with MB row blocks
//
// Same lane routing and k-sliced workgroup as the m <= 16 kernel, but a wave multiplies MB blocks of 16 rows of A and
// every dequantised weight fragment feeds 2*MB MFMAs, so the packed words are read once per 16*MB rows.  MB = 2 or
// 4 (accumulators in ordinary registers, two waves per SIMD) or 8 (accumulators in the accumulation registers, one
// wave per SIMD; launches whose 128-row tiles fill the chip).  Two loops: stream_tile_mb keeps the words and one step of
// A (MB x 1 KiB) per slot of a ring; stream_tile_mbp (launches with more than 32 rows, and 32-row tiles in eight-wave
// workgroups) fetches A a pair of steps at a time and the words through registers.  Both dequantise through
// dequant_entry.  A workgroup is one tile x four or eight k slices; blockIdx.y walks the row tiles.  Group scales are
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
template <int I, int END, typename F>
__device__ __forceinline__ void static_for(F&& f)
{
    if constexpr (I < END) {
        f(Int<I>{});
        static_for<I + 1, END>(f);
    }
}

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

// Accumulators in the accumulation registers (eight 16-row blocks: 256 of them, next to the 256 ordinary registers
// a wave that has a SIMD to itself may use).  The register class is all the asm statements ask for.  With all 256
// taken the allocator still permutes some accumulators through ordinary registers at the loop's back edge (about a
// hundred copies per trip of 256 MFMAs); naming each accumulator's quad in the constraints ("+{a[0:3]}") made that
// worse: the copies in and out of the fixed registers around every statement no longer coalesced and spilled; the
// MFMA builtin in place of the asm statements moved ten times as many.
template <bool FIRST>
__device__ __forceinline__ void mfma_acc_a(f4& acc, const h8& w, const h8& a)
{
    if constexpr (FIRST)
        asm volatile("s_nop 1\n\tv_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc) : "v"(w), "v"(a));
    else
        asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc) : "v"(w), "v"(a));
}
// Passes every accumulator through an empty asm: no read of it can be scheduled above this point.
template <int MB, int I = 0>
__device__ __forceinline__ void pin_all_acc(f4 (&acc)[MB][8])
{
    if constexpr (I < MB * 8) {
        if constexpr (MB > 4)
            asm volatile("" : "+a"(acc[I / 8][I % 8]));
        else
            asm volatile("" : "+v"(acc[I / 8][I % 8]));
        pin_all_acc<MB, I + 1>(acc);
    }
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

// Dequantisation of one step's words, written as asm statements of two instructions each that the loops place one by
// one after consecutive MFMAs.  Why asm: a wave issues one instruction of any kind every four cycles, so with a SIMD
// to itself it has three instruction slots per MFMA, and the empty asm statements that used to tie compiler-generated
// code to its place each cost an s_nop (the hazard recogniser assumes that an asm statement may have written its
// outputs with a sub-dword destination and separates it from the next reader): 2.2 s_nop per MFMA.  A schedule entry
// works on a pair of chunks (the same (j, half) of the step's two k-blocks: words A and B) so that its two
// instructions are independent, and an entry's inputs come from the entry before the previous one.
//   INT4 entries: SHIFT (half 1 only)  ANDLO  ANDHI  SUB  FMA  [MUL0  MUL1 with group scales]
//   FP6 entries:  LO  HI (unless the shift is 0)  BFI  P8  ASHRA  ASHRB  ANDA  ANDB
// Entry E of a step: pair E / entries_per_pair (= 2j + half), kind E % entries_per_pair.  q4a / q4b: word j of the
// 4-bit plane (INT4 words) of the two k-blocks; q2a / q2b: word j / 2 of the 2-bit plane; gs: the group scale of
// columns (j, half) in both halves of a register.
template <bool FP6, bool GROUP> constexpr int dequant_entries_per_pair() { return FP6 ? 8 : (GROUP ? 7 : 5); }
struct DequantRegs {
    uint32_t tA, tB, uA, uB, x0A, x0B, x1A, x1B, r0A, r0B, r1A, r1B;
};
template <bool FP6, bool GROUP, int E>
__device__ __forceinline__ void dequant_entry(DequantRegs& d, uint32_t q4a, uint32_t q4b, uint32_t q2a, uint32_t q2b, h2 gs,
                                              uint32_t ex, uint32_t b72, h8 (&frag)[8])
{
    constexpr int kEPP = dequant_entries_per_pair<FP6, GROUP>();
    constexpr int pr = E / kEPP, kind = E % kEPP, j = pr >> 1, half = pr & 1;
    if constexpr (!FP6) {
        if constexpr (kind == 0) {
            if constexpr (half == 1)
                asm volatile("v_lshrrev_b32 %0, 8, %2\n\tv_lshrrev_b32 %1, 8, %3" : "=&v"(d.tA), "=&v"(d.tB) : "v"(q4a), "v"(q4b));
            else {
                d.tA = q4a;
                d.tB = q4b;
            }
        } else if constexpr (kind == 1) {
            asm volatile("v_and_or_b32 %0, %2, %4, %5\n\tv_and_or_b32 %1, %3, %4, %5"
                         : "=&v"(d.x0A), "=&v"(d.x0B) : "v"(d.tA), "v"(d.tB), "s"(0x000f000fu), "v"(ex));
        } else if constexpr (kind == 2) {
            asm volatile("v_and_or_b32 %0, %2, %4, %5\n\tv_and_or_b32 %1, %3, %4, %5"
                         : "=&v"(d.x1A), "=&v"(d.x1B) : "v"(d.tA), "v"(d.tB), "s"(0x00f000f0u), "v"(ex));
        } else if constexpr (kind == 3) {
            asm volatile("v_pk_add_f16 %0, %2, %4\n\tv_pk_add_f16 %1, %3, %4"
                         : "=&v"(d.r0A), "=&v"(d.r0B) : "v"(d.x0A), "v"(d.x0B), "s"(0xe408e408u));            // - 1032
        } else if constexpr (kind == 4) {
            asm volatile("v_pk_fma_f16 %0, %2, %4, %5\n\tv_pk_fma_f16 %1, %3, %4, %5"
                         : "=&v"(d.r1A), "=&v"(d.r1B) : "v"(d.x1A), "v"(d.x1B), "s"(0x2c002c00u), "v"(b72));   // / 16 - 72
        } else if constexpr (kind == 5) {
            asm volatile("v_pk_mul_f16 %0, %0, %2\n\tv_pk_mul_f16 %1, %1, %2" : "+v"(d.r0A), "+v"(d.r0B) : "v"(gs));
        } else {
            asm volatile("v_pk_mul_f16 %0, %0, %2\n\tv_pk_mul_f16 %1, %1, %2" : "+v"(d.r1A), "+v"(d.r1B) : "v"(gs));
        }
    } else {
        constexpr int sh = 4 * (j & 1) + 2 * half;        // the 2-bit plane's field of this (j, half) to the top of every byte
        if constexpr (kind == 0) {
            if constexpr (half == 0)
                asm volatile("v_lshrrev_b32 %0, 2, %2\n\tv_lshrrev_b32 %1, 2, %3" : "=&v"(d.tA), "=&v"(d.tB) : "v"(q4a), "v"(q4b));
            else
                asm volatile("v_lshlrev_b32 %0, 2, %2\n\tv_lshlrev_b32 %1, 2, %3" : "=&v"(d.tA), "=&v"(d.tB) : "v"(q4a), "v"(q4b));
        } else if constexpr (kind == 1) {
            if constexpr (sh != 0)
                asm volatile("v_lshlrev_b32 %0, %4, %2\n\tv_lshlrev_b32 %1, %4, %3"
                             : "=&v"(d.uA), "=&v"(d.uB) : "v"(q2a), "v"(q2b), "n"(sh));
            else {
                d.uA = q2a;
                d.uB = q2b;
            }
        } else if constexpr (kind == 2) {                 // s eeemm xx in every byte
            asm volatile("v_bfi_b32 %0, %4, %2, %0\n\tv_bfi_b32 %1, %4, %3, %1"
                         : "+v"(d.tA), "+v"(d.tB) : "v"(d.uA), "v"(d.uB), "s"(0xc0c0c0c0u));
        } else if constexpr (kind == 3) {
            asm volatile("v_lshlrev_b32 %0, 8, %2\n\tv_lshlrev_b32 %1, 8, %3" : "=&v"(d.x1A), "=&v"(d.x1B) : "v"(d.tA), "v"(d.tB));
        } else if constexpr (kind == 4) {
            asm volatile("v_pk_ashrrev_i16 %0, 2, %2 op_sel_hi:[0,1]\n\tv_pk_ashrrev_i16 %1, 2, %3 op_sel_hi:[0,1]"
                         : "=&v"(d.x0A), "=&v"(d.x0B) : "v"(d.tA), "v"(d.tB));
        } else if constexpr (kind == 5) {
            asm volatile("v_pk_ashrrev_i16 %0, 2, %0 op_sel_hi:[0,1]\n\tv_pk_ashrrev_i16 %1, 2, %1 op_sel_hi:[0,1]"
                         : "+v"(d.x1A), "+v"(d.x1B));
        } else if constexpr (kind == 6) {
            asm volatile("v_and_b32 %0, %4, %2\n\tv_and_b32 %1, %4, %3"
                         : "=&v"(d.r0A), "=&v"(d.r0B) : "v"(d.x0A), "v"(d.x0B), "s"(0x9f009f00u));
        } else {
            asm volatile("v_and_b32 %0, %4, %2\n\tv_and_b32 %1, %4, %3"
                         : "=&v"(d.r1A), "=&v"(d.r1B) : "v"(d.x1A), "v"(d.x1B), "s"(0x9f009f00u));
        }
    }
    if constexpr (kind == kEPP - 1) frag[2 * j + half] = join(as_h2(d.r0A), as_h2(d.r1A), as_h2(d.r0B), as_h2(d.r1B));
}

// A pair slot (two k steps of A): per 16-row block two loads of 8 rows x 128 bytes; the second lands 64 bytes
// further than it would back to back, so that rows 8 .. 15 use the other half of the banks and a read of one
// step's half-lines by all 16 rows is conflict-free.
constexpr int kPairHalf = 1024 + 64;                      // from a block's first load to its second
constexpr int kPairBlock = 2 * kPairHalf;                 // from block to block

// The eight MFMAs of one 16-row block, `hook(block, t)` after each.
template <int MB, int BLK, int T = 0, typename Hook>
__device__ __forceinline__ void mfma_blocks_row(f4 (&acc)[MB][8], const h8 (&frag)[8], const h8& av, Hook&& hook)
{
    if constexpr (T < 8) {
        if constexpr (MB > 4)
            mfma_acc_a<T == 0>(acc[BLK][T], frag[T], av);
        else
            mfma_acc<T == 0>(acc[BLK][T], frag[T], av);
        hook(Int<BLK>{}, Int<T>{});
        mfma_blocks_row<MB, BLK, T + 1>(acc, frag, av, hook);
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
// PAIRH < 0: a slot holds one step, blocks 1 KiB apart; addr_cur / addr_next are this step's and the next
// step's slot.  PAIRH = 0 / 1: a slot holds a pair of steps (blocks 2 KiB apart, the second step's half of
// every row 64 bytes on) and this is the pair's first / second step; addr_cur / addr_next are this pair's and
// the next pair's slot.
template <int MB, int kExtra, int BLK = 0>
struct MbBlocks {
    // VMW >= 0 (second step of a pair): the next pair may still be in flight when the step starts; before its first
    // read, wait until at most VMW vector-memory loads (the ones issued after it) are outstanding.
    template <int phase, int PAIRH = -1, int VMW = -1, typename Hook>
    static __device__ __forceinline__ void run(MbCtx& cx, const h8 (&frag)[8], f4 (&acc)[MB][8], Hook&& hook)
    {
        if constexpr (BLK < MB) {
            constexpr int nb = BLK + 2;
            uint32_t (&dst)[4] = cx.abuf[(phase + nb) & 3];
            if constexpr (PAIRH < 0) {
                if constexpr (nb < MB)
                    lds_read_a4<nb * 1024>(dst, cx.addr_cur);
                else
                    lds_read_a4<(nb - MB) * 1024>(dst, cx.addr_next);
            } else if constexpr (nb < MB) {
                lds_read_a4<nb * kPairBlock + PAIRH * 64>(dst, cx.addr_cur);
            } else if constexpr (PAIRH == 0) {
                lds_read_a4<(nb - MB) * kPairBlock + 64>(dst, cx.addr_cur);
            } else {
                if constexpr (nb == MB && VMW >= 0) __builtin_amdgcn_s_waitcnt(vmcnt_only(VMW));
                lds_read_a4<(nb - MB) * kPairBlock>(dst, cx.addr_next);
            }
            // block 0 needs A(0): A(1), the extra reads and A(2) may be outstanding; from block 1 on the
            // extra reads must be complete as well
            constexpr int allow = BLK == 0 ? (8 + kExtra < 15 ? 8 + kExtra : 15) : 8;
            __builtin_amdgcn_s_waitcnt(lgkmcnt_only(allow));
            uint32_t (&src)[4] = cx.abuf[(phase + BLK) & 3];
            asm volatile("" : "+v"(src[0]), "+v"(src[1]), "+v"(src[2]), "+v"(src[3]));
            const h8 av = __builtin_bit_cast(h8, u4{src[0], src[1], src[2], src[3]});
            mfma_blocks_row<MB, BLK>(acc, frag, av, hook);
            MbBlocks<MB, kExtra, BLK + 1>::template run<phase, PAIRH, VMW>(cx, frag, acc, hook);
        }
    }
};

template <bool FP6, bool G128, int DEPTH, int MB>
__device__ __forceinline__ void stream_tile_mb(const GemmArgs& p, const TileInfo& ti, unsigned char* ring,
                                               int step_begin, int step_end, f4 (&acc)[MB][8])
{
    static_assert(DEPTH >= 3, "needs two steps of look-ahead");
    static_assert(MB == 2 || MB == 4 || MB == 8, "the A register ring assumes that MB divides or is a multiple of four");
    constexpr bool kGroup = G128 && !FP6;
    static_assert(!FP6 || DEPTH == 3, "the 2-bit plane alternates between two register sets");
    constexpr int kAOff = 2048;
    constexpr int kSlot = kAOff + MB * 1024;
    constexpr int kOps = 2 + MB + (FP6 ? 2 : 0);          // vector-memory loads per step
    constexpr int kUnroll = kGroup ? 4 : 2;
    constexpr int kW = 2;                                 // LDS reads of one step's weight words
    static_assert(kOps * (DEPTH - 2) + 1 <= 63, "vmcnt is a 6-bit counter");
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
        const bool scales = kGroup && (issued & 3) == 0;  // (never again once `issued` stops at the last, odd step)
        if (scales) {
            set_m0(gs_lds + ((issued >> 2) & kScaleMask) * 256);
            dma4_m0(base_gs + (size_t)(issued >> 2) * (size_t)uniform32(p.n4) * 2, vgs);
        }
        if (issued < last) {
            issued++;
            base4 += 2 * row4;
            base2 += 2 * row2;
            base_a += 64;
        }
        return scales;
    };
    // The load of group scales closes the fetch of every fourth step and counts in the waits for as long as that
    // step is among the DEPTH - 2 newest: the fetch goes out in sub-step kScaleU of the unrolled loop.
    static_assert(!kGroup || DEPTH == 3 || DEPTH == 4, "sub-steps that count the load of group scales");
    constexpr int kScaleU = (5 - DEPTH) & 3;

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
    // Dequantisation: dequant_entry, one entry (or two) after each MFMA from the second block on.
    constexpr int kEPP = dequant_entries_per_pair<FP6, kGroup>();
    constexpr int kEntries = 8 * kEPP;
    DequantRegs dq = {};
    const uint32_t b72 = vgpr_const(0xd480d480u);         // -72
    auto entries = [&](auto first, auto last, int set, h8 (&frag)[8]) {
        constexpr int e0 = decltype(first)::value, e1 = decltype(last)::value;
        static_for<e0, e1>([&](auto e) {
            constexpr int E = decltype(e)::value, pr = E / kEPP, j = pr >> 1, half = pr & 1;
            dequant_entry<FP6, kGroup, E>(dq, w.q0[j], w.q1[j], FP6 ? tq[set][0][j >> 1] : 0u, FP6 ? tq[set][1][j >> 1] : 0u,
                                          kGroup ? gs_cur[2 * j + half] : h2{}, kc.ex, b72, frag);
        });
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
    entries(Int<0>{}, Int<kEntries>{}, 0, frag[0]);
    int slot_rd = 1;
    bool scales_in_flight = false;
#pragma unroll 1
    for (int s = step_begin; s < step_end; s += kUnroll) {
#pragma unroll
        for (int u = 0; u < kUnroll; u++) {
            const bool scales = issue(slot_in, u & 1);                // step s+u+2 (FP6: DEPTH is 3)
            slot_in = slot_in + 1 == DEPTH ? 0 : slot_in + 1;
#pragma unroll
            for (int d = 0; d < 4; d++) cx.addr_cur[d] = cx.addr_next[d];
            slot_addrs(cx.addr_next, slot_rd);
            if (kGroup && u == kScaleU) scales_in_flight = scales;
            if (kGroup && u >= kScaleU && u < kScaleU + DEPTH - 2 && scales_in_flight)
                __builtin_amdgcn_s_waitcnt(vmcnt_only(kOps * (DEPTH - 2) + 1));
            else
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
                constexpr int avail = 8 * MB - 8;                     // the entries go after the MFMAs of blocks >= 1
                if constexpr (mslot == 8) {
                    if (next_group) settle_scales();
                }
                if constexpr (mslot >= 8) {
                    constexpr int e0 = (mslot - 8) * kEntries / avail, e1 = (mslot - 7) * kEntries / avail;
                    entries(Int<e0>{}, Int<e1>{}, (u + 1) & 1, nxt);
                }
            };
            // (the LDS reads issued between A(1) and A(2): the words, and the group scales where a group starts)
            if ((u & 1) == 0) {                                        // buffer of block 0: (u * MB) mod 4
                if (next_group)
                    MbBlocks<MB, kW + 8>::template run<0>(cx, cur, acc, hook);
                else
                    MbBlocks<MB, kW>::template run<0>(cx, cur, acc, hook);
            } else {
                if (next_group)
                    MbBlocks<MB, kW + 8>::template run<(MB & 3)>(cx, cur, acc, hook);
                else
                    MbBlocks<MB, kW>::template run<(MB & 3)>(cx, cur, acc, hook);
            }
        }
    }
    __builtin_amdgcn_s_waitcnt(vmcnt_only(0) & lgkmcnt_only(0));
    // MFMA results -> VALU reads: the wait states, then every accumulator is passed through an (empty)
    // asm so that no read of it can be scheduled above them.
    asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 7");
    pin_all_acc<MB>(acc);
    if (FP6) {
#pragma unroll
        for (int mb = 0; mb < MB; mb++)
#pragma unroll
            for (int t = 0; t < 8; t++) acc[mb][t] *= 4096.0f;
    }
}

// The MB = 4 variant of stream_tile_mb: activations fetched a pair of k steps at a time, packed words through
// registers.
//
// What bounds a workgroup's rate is its requests in flight, and A dominated them: 64 half-lines per step and
// wave against 16 lines of words (fetching only half of the distinct lines measured 10-15 % faster at
// m = 64 .. 256).  Here one load brings 8 rows x 128 bytes -- whole lines, two steps of k -- into a ring of two
// pair slots (MB x 2 KiB each).  That is 4 KiB more LDS per wave than three one-step slots, which eight waves
// per CU only have if the words stay out of LDS: each lane loads its own two 16-byte granules of a step (the
// k-block row is contiguous, so the wave still reads whole lines) into one of two register sets, two steps
// ahead of the MFMAs and one ahead of the dequantisation, exactly the look-ahead the three-slot ring gave.
// A pair's first step issues the words two steps on, then the next pair of A; its second step only words.  Either
// step starts once the words of the following step have landed, which leaves that next pair and the newest words in
// flight; the second step waits for the pair in its middle, right before it reads the next step's first A block.
// A load of group scales goes out in front of the words of some first steps and is counted there.
constexpr int pair_load_imm(int q) { return ((q / 2) % 2) * kPairBlock + (q % 2) * kPairHalf; }
static_assert(pair_load_imm(3) < 4096, "immediate of a direct-to-LDS load");
template <int MB, int I = 0>
__device__ __forceinline__ void dma_a_pair(uint32_t slot_lds, const void* sbase_a, const uint32_t (&voff)[2 * MB])
{
    if constexpr (I < 2 * MB) {
        // four loads (two blocks) per value of M0: the immediate reaches 4 KiB
        if constexpr (I % 4 == 0) set_m0(slot_lds + (I / 2) * kPairBlock);
        dma16_m0<pair_load_imm(I), false>(sbase_a, voff[I]);
        dma_a_pair<MB, I + 1>(slot_lds, sbase_a, voff);
    }
}
constexpr int mbp_wave_lds(int mb) { return max3(2 * mb * kPairBlock + 512, 2 * 16 * kRedStride * 4, 0); }

template <bool FP6, bool G128, int MB>
__device__ __forceinline__ void stream_tile_mbp(const GemmArgs& p, const TileInfo& ti, unsigned char* ring,
                                                int step_begin, int step_end, f4 (&acc)[MB][8])
{
    static_assert(MB == 2 || MB == 4 || MB == 8, "the A register ring");
    constexpr int kOddPhase = MB == 2 ? 2 : 0;            // (two blocks per step walk the four register buffers in two steps)
    constexpr bool kGroup = G128 && !FP6;
    constexpr int kPair = MB * kPairBlock;                // one pair slot
    constexpr int kWOps = FP6 ? 4 : 2;                    // register loads per step
    constexpr int kAOps = 2 * MB;                         // direct-to-LDS loads per pair
    constexpr int kUnroll = kGroup ? 4 : 2;
    static_assert(kAOps + kWOps + 1 <= 63, "vmcnt is a 6-bit counter");
    const int lane = threadIdx.x & 63;
    const int i = lane >> 4, c = lane & 15, sigma = c >> 3, l = c & 7;

    DequantConsts kc;
    kc.lo = vgpr_const(0x000f000fu);
    kc.hi = vgpr_const(0x00f000f0u);
    kc.ex = vgpr_const(0x64006400u);
    kc.top2 = vgpr_const(0xc0c0c0c0u);
    kc.exp_man = vgpr_const(0x9f009f00u);

    // ---- fetch side
    const PlaneGeometry geo = plane_geometry(p, ti);
    const size_t row4 = geo.row4, row2 = geo.row2;
    const int owner = p.native ? lane : 32 * sigma + 4 * l + i;      // whose granule of the k-block this lane needs
    const uint32_t v4 = (uint32_t)owner * 16, v4b = v4 + (uint32_t)row4;
    const unsigned char* base4 = uniform_ptr(reinterpret_cast<const unsigned char*>(FP6 ? p.b_fp6_4 : p.b_int4) +
                                             geo.tile4 + (size_t)(2 * step_begin) * row4);
    const uint32_t v2 = (uint32_t)owner * 8, v2b = v2 + (uint32_t)row2;
    const unsigned char* base2 = uniform_ptr(reinterpret_cast<const unsigned char*>(p.b_fp6_2) +
                                             geo.tile2 + (size_t)(2 * step_begin) * row2);
    u4 wq[2][2];                                          // [register set][k-block]
    u2 tq[2][2];
    // A: load 2b + o brings rows 8o .. 8o+7 of block b, eight lanes per row; LDS position lane = 8 * row + chunk'
    // holds the row's 16-byte chunk 4h + d (step parity h, quarter d) at chunk' = 4h + (d ^ (row >> 1 & 3)).
    const int tile_row0 = ti.mtile * 16 * MB;
    const int prow = lane >> 3, pch = lane & 7;
    uint32_t va[2 * MB];
#pragma unroll
    for (int q = 0; q < 2 * MB; q++) {
        int row = tile_row0 + 8 * q + prow;
        row = row < p.m ? row : p.m - 1;
        va[q] = (uint32_t)(row - tile_row0) * (uint32_t)p.k * 2 + 16 * ((pch & 4) | ((pch & 3) ^ ((prow >> 1) & 3))) +
                4096 - pair_load_imm(q);
    }
    const unsigned char* base_a = uniform_ptr(reinterpret_cast<const unsigned char*>(p.A + (size_t)tile_row0 * p.k) +
                                              (size_t)(ti.a_step0 + step_begin) * 64 - 4096);
    const unsigned char* base_gs =
        uniform_ptr(reinterpret_cast<const unsigned char*>(p.s_int4 + (size_t)ti.tcol * kTileN));
    const uint32_t vgs = 4 * lane;
    const uint32_t ring_lds = uniform32(lds_addr(ring));
    const uint32_t gs_lds = ring_lds + 2 * kPair;

    int issued = step_begin;
    const int last = step_end - 1;
    int pairs_issued = 0, a_slot = 0;
    const int last_pair = (step_end - step_begin) / 2 - 1;
    auto issue_a = [&]() {
        dma_a_pair<MB>(ring_lds + a_slot * kPair, base_a, va);
        a_slot ^= 1;
        if (pairs_issued < last_pair) {                   // (fetches past the end repeat the last pair)
            pairs_issued++;
            base_a += 128;
        }
    };
    // returns whether a load of group scales went out in front of the words
    auto issue_w = [&](int set) {
        const bool scales = kGroup && (issued & 3) == 0;
        if (scales) {
            set_m0(gs_lds + ((issued >> 2) & 1) * 256);
            dma4_m0(base_gs + (size_t)(issued >> 2) * (size_t)uniform32(p.n4) * 2, vgs);
        }
        asm volatile("global_load_dwordx4 %0, %2, %4 nt\n\tglobal_load_dwordx4 %1, %3, %4 nt"
                     : "=&v"(wq[set][0]), "=&v"(wq[set][1]) : "v"(v4), "v"(v4b), "s"(base4) : "memory");
        if (FP6) {
            asm volatile("global_load_dwordx2 %0, %2, %4 nt\n\tglobal_load_dwordx2 %1, %3, %4 nt"
                         : "=&v"(tq[set][0]), "=&v"(tq[set][1]) : "v"(v2), "v"(v2b), "s"(base2) : "memory");
        }
        if (issued < last) {
            issued++;
            base4 += 2 * row4;
            base2 += 2 * row2;
        }
        return scales;
    };

    // ---- read side
    const uint32_t rdgs = gs_lds + (64 * sigma + l) * 2;    // weight side: column (j, half) at +32j +16half
    uint32_t gs_next[8];
    h2 gs_cur[8];
    MbCtx cx;
#pragma unroll
    for (int d = 0; d < 4; d++) {
        cx.addr_cur[d] = ring_lds + (c >> 3) * kPairHalf + (8 * (c & 7) + (d ^ ((c >> 1) & 3))) * 16 + 4 * i;
        cx.addr_next[d] = 0;
    }
    uint32_t to_next = kPair;                             // from this pair's slot to the other one (uniform)
    auto fetch_scales = [&](int group) {
        const uint32_t ga = rdgs + (group & 1) * 256;
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
    // Dequantisation: dequant_entry, one entry after each MFMA from the second block on.
    constexpr int kEPP = dequant_entries_per_pair<FP6, kGroup>();
    constexpr int kEntries = 8 * kEPP;
    DequantRegs dq = {};
    const uint32_t b72 = vgpr_const(0xd480d480u);         // -72 (one scalar operand per instruction: the other constants)
    auto entries = [&](auto first, auto last, int set, h8 (&frag)[8]) {
        constexpr int e0 = decltype(first)::value, e1 = decltype(last)::value;
        static_for<e0, e1>([&](auto e) {
            constexpr int E = decltype(e)::value, pr = E / kEPP, j = pr >> 1, half = pr & 1;
            dequant_entry<FP6, kGroup, E>(dq, wq[set][0][j], wq[set][1][j], FP6 ? tq[set][0][j >> 1] : 0u,
                                          FP6 ? tq[set][1][j >> 1] : 0u, kGroup ? gs_cur[2 * j + half] : h2{}, kc.ex, b72, frag);
        });
    };

    issue_a();                                            // pair 0
    issue_w(0);                                           // steps 0 and 1
    issue_w(1);                                           // (an odd step: never with group scales)
    h8 frag[2][8];
    __builtin_amdgcn_s_waitcnt(vmcnt_only(kWOps));        // all but the words of step 1
    lds_read_a4<0>(cx.abuf[0], cx.addr_cur);
    lds_read_a4<kPairBlock>(cx.abuf[1], cx.addr_cur);
    if (kGroup) fetch_scales(step_begin >> 2);
    __builtin_amdgcn_s_waitcnt(lgkmcnt_only(0));
    if (kGroup) settle_scales();
    entries(Int<0>{}, Int<kEntries>{}, 0, frag[0]);
#pragma unroll 1
    for (int s = step_begin; s < step_end; s += kUnroll) {
#pragma unroll
        for (int u = 0; u < kUnroll; u++) {
            const bool scales = issue_w(u & 1);                       // step s+u+2 (its set was drained a step ago)
            if ((u & 1) == 0) issue_a();                              // the pair after this one
            // the words of step s+u+1 have landed, and any group scales issued before them (its A did so half a
            // step earlier); group scales only ever go out in a pair's first step
            if ((u & 1) == 0 && scales)
                __builtin_amdgcn_s_waitcnt(vmcnt_only(kAOps + kWOps + 1));
            else
                __builtin_amdgcn_s_waitcnt(vmcnt_only(kAOps + kWOps));
            const bool next_group = kGroup && u == kUnroll - 1;       // step s+u+1 starts a 128-row group
            if (next_group) fetch_scales((s + u + 1) >> 2);
            h8 (&cur)[8] = frag[u & 1];
            h8 (&nxt)[8] = frag[(u + 1) & 1];
            auto hook = [&](auto blk, auto t) {
                constexpr int mslot = decltype(blk)::value * 8 + decltype(t)::value;   // MFMA just issued
                constexpr int avail = 8 * MB - 8;                     // the entries go after the MFMAs of blocks >= 1
                if constexpr (mslot == 8) {
                    if (next_group) settle_scales();
                }
                if constexpr (mslot >= 8) {
                    constexpr int e0 = (mslot - 8) * kEntries / avail, e1 = (mslot - 7) * kEntries / avail;
                    entries(Int<e0>{}, Int<e1>{}, (u + 1) & 1, nxt);
                }
            };
            if ((u & 1) == 0) {
                MbBlocks<MB, 0>::template run<0, 0>(cx, cur, acc, hook);
            } else {
#pragma unroll
                for (int d = 0; d < 4; d++) cx.addr_next[d] = cx.addr_cur[d] + to_next;
                if (next_group)                                        // (the reads of the group scales sit between A(1) and A(2))
                    MbBlocks<MB, 8>::template run<kOddPhase, 1, kWOps>(cx, cur, acc, hook);
                else
                    MbBlocks<MB, 0>::template run<kOddPhase, 1, kWOps>(cx, cur, acc, hook);
#pragma unroll
                for (int d = 0; d < 4; d++) cx.addr_cur[d] = cx.addr_next[d];   // on to the next pair's slot
                to_next = 0u - to_next;
            }
        }
    }
    __builtin_amdgcn_s_waitcnt(vmcnt_only(0) & lgkmcnt_only(0));
    // MFMA results -> VALU reads: the wait states, then every accumulator is passed through an (empty)
    // asm so that no read of it can be scheduled above them.
    asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 7");
    pin_all_acc<MB>(acc);
    // loads into the word registers may still have been in flight up to the wait above
#pragma unroll
    for (int set = 0; set < 2; set++) {
        asm volatile("" : "+v"(wq[set][0]), "+v"(wq[set][1]));
        if (FP6) asm volatile("" : "+v"(tq[set][0]), "+v"(tq[set][1]));
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
// `smem`, `flag` and `valid` belong to the WK waves that share a tile and a row tile (the whole workgroup); a
// workgroup without rows goes through the barriers without touching memory.
template <int MB, int WK = kWaves, int BPR = 1>
__device__ __forceinline__ void wg_finish_mb(const GemmArgs& p, const TileInfo& ti, int wk, int ks, int slot_base,
                                             f4 (&acc)[MB][8],
                                             bool per_column_scale, unsigned char* smem, int wave_lds, int* flag,
                                             bool valid = true, int first_fp6 = WK)
{
    // BPR: 16-row blocks per round of the reduction through LDS (a wave's region holds BPR * 16 rows of kRedStride
    // floats).  The rounds are bound by LDS bandwidth (every wave writes and reads its whole accumulator once) plus two
    // barriers each, so fewer rounds help; the gather below keeps the loads of up to 32 rows in flight per lane.
    static_assert(MB % BPR == 0, "whole rounds");
    constexpr int RMAX = 16 / WK;                                    // rows of a block one wave finishes
    // The gather keeps up to 32 8-byte loads per lane in flight.
    constexpr int kInFlight = 32;
    // (shared tiles) this workgroup's own sums stay in registers where there are few enough of them: if it turns out to
    // arrive last it takes them from there, in their place in the part order, instead of loading them back
    constexpr bool kKeep = MB * RMAX <= 32;
    constexpr int MBC = MB < kInFlight / RMAX ? MB : kInFlight / RMAX;                                 // blocks per gather round
    constexpr int PCH = kInFlight / (MBC * RMAX) > 0 ? kInFlight / (MBC * RMAX) : 1;                   // parts per gather round
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
    const FusedCols fcols = fused_cols(p, ti.col0 + 2 * lane);
    auto store_row = [&](int row, float v0, float v1) {
        if (p.fused) {
            store_fused(p, fcols, (size_t)(row0 + row), v0 * s0, v1 * s1);
            return;
        }
        h2 o = {(_Float16)(v0 * s0), (_Float16)(v1 * s1)};
        *reinterpret_cast<h2*>(c_out + (size_t)row * p.n) = o;
    };
    constexpr size_t kSlotU64 = (size_t)MB * 16 * kTileN / 2;
    unsigned long long* slot0 = reinterpret_cast<unsigned long long*>(p.scratch) + (size_t)slot_base * kSlotU64 + lane;
    unsigned long long* my = slot0 + (size_t)ti.part * kSlotU64;

    float keep0[kKeep ? MB : 1][RMAX], keep1[kKeep ? MB : 1][RMAX];
#pragma unroll
    for (int mb0 = 0; mb0 < MB; mb0 += BPR) {
        __syncthreads();
        if (mb0 == 0) FP6M_MARK(p, 1);                               // every wave of the group has left its loop
        float* mine = reinterpret_cast<float*>(smem + wk * wave_lds) + c * kRedStride + 64 * (q >> 1) + 4 * (q & 1);
#pragma unroll
        for (int b = 0; b < BPR; b++)
#pragma unroll
            for (int t = 0; t < 8; t++)
                *reinterpret_cast<f4*>(mine + b * 16 * kRedStride + 16 * (t >> 1) + 8 * (t & 1)) = acc[mb0 + b][t];
        __syncthreads();
        // all LDS reads of the round first (rows beyond m are read too: the slab is there), one wait, then the sums
        f2 tv[BPR][RMAX][WK];
#pragma unroll
        for (int b = 0; b < BPR; b++)
#pragma unroll
            for (int r = 0; r < RMAX; r++)
#pragma unroll
                for (int j = 0; j < WK; j++)
                    tv[b][r][j] = *reinterpret_cast<const f2*>(reinterpret_cast<const float*>(smem + j * wave_lds) +
                                                               (b * 16 + wk + r * WK) * kRedStride + 2 * lane);
#pragma unroll
        for (int b = 0; b < BPR; b++)
#pragma unroll
            for (int r = 0; r < RMAX; r++) {
                const int row = 16 * (mb0 + b) + wk + r * WK;
                float v0 = 0.f, v1 = 0.f;
                if (first_fp6 >= WK) {                               // (uniform) the usual case: plain sums
#pragma unroll
                    for (int j = 0; j < WK; j++) {
                        v0 += tv[b][r][j][0];
                        v1 += tv[b][r][j][1];
                    }
                } else {
#pragma unroll
                    for (int j = 0; j < WK; j++) {
                        v0 += j >= first_fp6 ? tv[b][r][j][0] * x0 : tv[b][r][j][0];
                        v1 += j >= first_fp6 ? tv[b][r][j][1] * x1 : tv[b][r][j][1];
                    }
                }
                if constexpr (kKeep) {
                    keep0[mb0 + b][r] = v0;
                    keep1[mb0 + b][r] = v1;
                }
                if (row < nrows) {
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
    // Every wave waits until its own partial-sum stores are acknowledged (agent-scope write-through stores: visible to
    // every other CU from then on) before it joins the barrier in front of the counter increment; neither a
    // workgroup-scope fence nor s_barrier waits for outstanding stores.
    __builtin_amdgcn_s_waitcnt(vmcnt_only(0));
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");           // (keeps the compiler from moving accesses across)
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
    // The last arrival sums all parts in part order: MBC blocks at a time, PCH parts' loads in flight together.
#pragma unroll
    for (int mb0 = 0; mb0 < MB; mb0 += MBC) {
        float v0[MBC][RMAX], v1[MBC][RMAX];
#pragma unroll
        for (int b = 0; b < MBC; b++)
#pragma unroll
            for (int r = 0; r < RMAX; r++) {
                v0[b][r] = 0.f;
                v1[b][r] = 0.f;
            }
        for (int pp = 0; pp < ks; pp += PCH) {
            unsigned long long t[PCH][MBC][RMAX];
#pragma unroll
            for (int u = 0; u < PCH; u++)
#pragma unroll
                for (int b = 0; b < MBC; b++)
#pragma unroll
                    for (int r = 0; r < RMAX; r++) {
                        const int row = 16 * (mb0 + b) + wk + r * WK;
                        t[u][b][r] = 0;
                        if (row < nrows && pp + u < ks && !(kKeep && pp + u == ti.part))
                            t[u][b][r] = __hip_atomic_load(slot0 + (size_t)(pp + u) * kSlotU64 + (size_t)row * (kTileN / 2),
                                                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
#pragma unroll
            for (int u = 0; u < PCH; u++)
#pragma unroll
                for (int b = 0; b < MBC; b++)
#pragma unroll
                    for (int r = 0; r < RMAX; r++) {
                        const f2 v = __builtin_bit_cast(f2, t[u][b][r]);
                        const bool own = kKeep && pp + u == ti.part;   // (uniform) the bits that were stored, from registers
                        v0[b][r] += own ? keep0[kKeep ? mb0 + b : 0][r] : v[0];
                        v1[b][r] += own ? keep1[kKeep ? mb0 + b : 0][r] : v[1];
                    }
        }
#pragma unroll
        for (int b = 0; b < MBC; b++)
#pragma unroll
            for (int r = 0; r < RMAX; r++) {
                const int row = 16 * (mb0 + b) + wk + r * WK;
                if (row < nrows) store_row(row, v0[b][r], v1[b][r]);
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
// PAIR: A is fetched by pairs of steps and the words through registers (stream_tile_mbp).
// EXTRAS = false: a build of the same kernel without the row mix, the fused epilogue and the gfx950 word order, for
// calls that use none of them (plain fp6m_mul on reference-order words).  Their run-time branches cost the plain path
// 2-6 % (4096 x 4096 at 64 rows 15.8 -> 14.8 us, 8192 x 8192 at 512 rows 68.4 -> 67.3): the arguments are overwritten
// with constants and the compiler removes what hangs on them.
// CLASSES: the build (of the one for plain calls) that knows two classes of INT4 tiles: the first in ks4 parts each, the
// other groups4b tiles in ks4b parts on the last workgroups of the grid (see the dispatcher).
template <bool G128, int MB, int D4, int D6, int WK, bool PAIR, bool EXTRAS = true, bool CLASSES = false>
__global__ __launch_bounds__(64 * WK, (WK == 4 && MB <= 4) ? 2 : 1) void gemm_mb_kernel(const GemmArgs args)
{
    GemmArgs p = args;
    static_assert(!CLASSES || !EXTRAS, "two classes of INT4 tiles: plain calls only");
    if constexpr (!EXTRAS) {
        p.k4 = 0;
        p.slices4 = 0;
        p.native = 0;
        p.fused = 0;
        p.c_cols = nullptr;
        p.bias = nullptr;
        p.residual = nullptr;
    }
    // FP6 tiles take the paired loop too: with the dequantisation as asm statements it fits 256 VGPRs with the 2-bit
    // plane's registers on top, and in a grid that is resident all at once the few FP6 workgroups set the length of
    // the launch (8192 x 8192 with 256 FP6 columns: m = 128 31.8 -> 27.1 us, m = 256 47.0 -> 40.3).
    constexpr bool kPaired = PAIR;
    constexpr int kWaveLds = kPaired ? max3(mbp_wave_lds(MB), mb_wave_lds(MB, 0, D6), 0) : mb_wave_lds(MB, D4, D6);
    static_assert(WK * kWaveLds + 16 <= 160 * 1024, "LDS of one CU");
    __shared__ __attribute__((aligned(16))) unsigned char smem[WK * kWaveLds + 16];

    preload_args<true, CLASSES>(args);
    FP6M_MARK(p, 0);
    // (The build with two classes of INT4 tiles takes tile and k range from the argument block itself: selecting among
    // fields of the copy, which the builds for plain calls modify, makes the compiler keep the copy in private memory.)
    TileInfo ti;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    int step_begin, step_end;
    if constexpr (!CLASSES) {
        ti = locate_tile<false>(p);
        wave_k_range<G128, WK>(p, ti.fp6, false, ti.part, wave, step_begin, step_end);
    } else {
        ti = locate_tile<true>(args);
        wave_k_range<G128, WK>(args, ti.fp6, ti.later, ti.part, wave, step_begin, step_end);
        step_begin = __builtin_amdgcn_readfirstlane(step_begin);         // (uniform: see locate_tile)
        step_end = __builtin_amdgcn_readfirstlane(step_end);
    }
    // partial-sum slots, row tile by row tile: the FP6 tiles' (tile, part), then the INT4 tiles'
    const int groups4b = CLASSES ? held(args.groups4b) : 0, ks4b = CLASSES ? held(args.ks4b) : 1;
    int ks = ti.fp6 ? p.ks6 : (ti.later ? ks4b : p.ks4);
    const int wgs6 = p.tiles6 * p.ks6;
    const int first4 = p.tiles - p.tiles6 - groups4b;                    // INT4 tiles of the first class (all, as a rule)
    int slot_base = ti.mtile * (wgs6 + first4 * p.ks4 + groups4b * ks4b) +
                    (ti.fp6 ? ti.tcol * p.ks6
                            : (ti.later ? wgs6 + first4 * p.ks4 + (ti.tcol - first4) * ks4b : wgs6 + ti.tcol * p.ks4));
    if constexpr (CLASSES) {                                             // (uniform: into scalar registers before the loops)
        ks = __builtin_amdgcn_readfirstlane(ks);
        slot_base = __builtin_amdgcn_readfirstlane(slot_base);
    }
    if (p.k4) row_mix_slice(p, ti.part * WK + wave, ti, step_begin, step_end);   // (no FP6 column tiles in a row mix)

    f4 acc[MB][8];
#pragma unroll
    for (int mb = 0; mb < MB; mb++)
#pragma unroll
        for (int t = 0; t < 8; t++) acc[mb][t] = f4{0.f, 0.f, 0.f, 0.f};
    unsigned char* ring = smem + wave * kWaveLds;
    if (step_begin < step_end) {
        if constexpr (kPaired) {
            if (ti.fp6) {
                stream_tile_mbp<true, G128, MB>(p, ti, ring, step_begin, step_end, acc);
            } else
                stream_tile_mbp<false, G128, MB>(p, ti, ring, step_begin, step_end, acc);
        } else {
            if (ti.fp6)
                stream_tile_mb<true, G128, D6, MB>(p, ti, ring, step_begin, step_end, acc);
            else
                stream_tile_mb<false, G128, D4, MB>(p, ti, ring, step_begin, step_end, acc);
        }
    }
    FP6M_MARK(p, 2);
    // the drained rings hold two blocks per wave; four in the eight-block kernel, which has the registers for a round
    // of that size (half the barriers: 139 -> 135 us at m = 1024 on 8192 x 8192)
    constexpr int BPR = (MB > 4 && kWaveLds >= 4 * 16 * kRedStride * 4) ? 4 : (kWaveLds >= 2 * 16 * kRedStride * 4 ? 2 : 1);
    wg_finish_mb<MB, WK, BPR>(p, ti, wave, ks, slot_base, acc, !p.k4 && (ti.fp6 || !G128), smem, kWaveLds,
                         reinterpret_cast<int*>(smem + WK * kWaveLds), true, p.k4 ? p.slices4 - ti.part * WK : WK);
    FP6M_MARK(p, 7);
}

}  // namespace fp6m
