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
// is that every SM streams the same number of bytes whatever the tile count.  Here the property is reached
// dynamically, at the granularity of a wave: a workgroup is ONE wave, every tile's k range is cut into chunks of
// a few k units, and the chunks of a region, tile-major, form one list.  Wave j starts on chunk j; whenever a wave's
// fetches reach the end of a chunk it moves on to the chunk it drew from a counter in `workspace` one chunk
// earlier (one agent-scope atomic by one lane, its latency hidden behind a whole chunk).  Equal static shares left a
// third of the run to a thinning tail of waves (those that share a SIMD with an older wave, or got their first
// data late, finish up to twice as late as the first); with chunks every wave works until the list is empty.  The
// counter is zero before and after the launch: each wave draws exactly one number past the end of the list, and the
// wave that draws the last of them writes the zero back.  INT4 and FP6 tiles are separate regions with their own
// unit length, chunk size, waves and counter.  Nothing in the kernel synchronises waves: no barrier, no LDS shared
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
// Kernel arguments, laid out as four 64-byte blocks that the kernel fetches itself with four
// scalar loads behind one wait (left to the compiler, the loads of the fields come in several dependent batches, each a
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
    int q4, cpt4, q6, cpt6;   // chunk: q units (the last of a tile may be shorter); chunks per tile
    int flags;                // bit 0: planes in the gfx950 order, bit 1: fused epilogue work
    int groups;               // counters (= sub-lists of chunks) of the INT4 region | of the FP6 region << 16
    // block 2
    unsigned long long magic_cpt4, magic_cpt6;   // n / cpt as (n * magic) >> 40 (exact for n < 2^24, cpt < 2^16)
    int total4, total6;       // chunks of each region (0: the region's waves own one chunk each and draw nothing)
    int* counters;            // the INT4 region's, then the FP6 region's; zero on entry, zero on exit
    const int32_t* c_cols;    // optional epilogue work (fp6m_mul_fused), as in GemmArgs
    const uint16_t* bias;
    const uint16_t* residual;
    unsigned long long* timeline;   // performance debugging builds only
    // block 3: the activation gather of fp6m_mul_fused, done by the kernel itself (GR > 0)
    const int32_t* a_cols;    // column kk of the GEMM's A is column a_cols[kk] (clamped) of the caller's matrix
    int lda;                  // the caller's row length
    // ... and the INT4 region's tiles in up to three sub-lists with a chunk length each (see sk_generation_order):
    // tiles [0, tiles4a) in chunks of q4 units, [tiles4a, tiles4a + tiles4b) of q4b, the rest of q4c.
    int gen_waves;            // waves of the whole chip that find a SIMD of their own (4 x CUs); 0: the plain order
    int q4b, cpt4b, q4c, cpt4c;
    int tiles4a, tiles4b;     // (all tiles in the first sub-list: tiles4a = the region's tiles)
    uint32_t magic32_cpt4b, magic32_cpt4c;   // n / cpt as the high half of n * magic (exact for n, cpt < 2^16: a wave per chunk)
    int pad[4];
    static constexpr int k4 = 0;    // (the row mix does not come here)
};
// What the fused-epilogue helpers of gemm_common.h read.
struct SkEpilogue {
    int fused, n;
    const int32_t* c_cols;
    const uint16_t* bias;
    const uint16_t* residual;
    uint16_t* C;
};
static_assert(sizeof(SkArgs) == 256 && offsetof(SkArgs, m) == 64 && offsetof(SkArgs, magic_cpt4) == 128 &&
                  offsetof(SkArgs, a_cols) == 192,
              "four 64-byte blocks");

__device__ __forceinline__ SkArgs load_sk_args()
{
    typedef uint32_t u16v __attribute__((ext_vector_type(16)));
    u16v b0, b1, b2, b3;
    const uint64_t ka = (uint64_t)__builtin_amdgcn_kernarg_segment_ptr();
    asm volatile(
        "s_load_dwordx16 %0, %4, 0x0\n\ts_load_dwordx16 %1, %4, 0x40\n\ts_load_dwordx16 %2, %4, 0x80\n\t"
        "s_load_dwordx16 %3, %4, 0xc0\n\ts_waitcnt lgkmcnt(0)"
        : "=&s"(b0), "=&s"(b1), "=&s"(b2), "=&s"(b3) : "s"(ka));
    struct Words {
        uint32_t w[64];
    } raw;
#pragma unroll
    for (int i = 0; i < 16; i++) {
        raw.w[i] = b0[i];
        raw.w[16 + i] = b1[i];
        raw.w[32 + i] = b2[i];
        raw.w[48 + i] = b3[i];
    }
    return __builtin_bit_cast(SkArgs, raw);
}

__device__ __forceinline__ uint32_t mul_shift40(unsigned long long magic, uint32_t n)
{
    return (uint32_t)(((unsigned long long)n * magic) >> 40);
}

// A shared tile's elements this wave has added to and not yet looked at: the atomics' results come back while the
// wave is already streaming its next segment.
struct PendingCells {
    unsigned long long* cell;      // this lane's cell of row 0 (even column; the odd one 64 cells on)
    unsigned long long old[4][2];
    float v[4][2];
    int parts;                     // 0: nothing pending
    int col0;                      // the tile's first column in C
};

// All chunks of a wave in one software pipeline.  This is stream_tile (gemm_m16.h) for at most four rows of A with
// two changes.  The fetch side walks from chunk to chunk by itself (past a chunk's last step its position moves to the
// first step of the next chunk), so when the multiply side finishes a chunk the words of the next one are already in
// the ring or on their way: a wave pays the latency of a first load once, not once per chunk.  And because the ring
// is never drained in between, a chunk's accumulators are turned into rows in a small slab of their own behind the
// ring.  A chunk has at least as many steps as the fetch side runs ahead (DEPTH - 1), so the fetch side is never
// more than one chunk ahead of the multiply side.
//
// GR > 0: the activation gather (fp6m_mul_fused's a_cols) happens here instead of in a pass of its own.  A step pair
// covers 64 columns of A, one per lane: the lane loads the pair's entry of the map (a dword, coalesced), then, with
// the map entry as the address, its element of each of the GR rows (ushort loads), and writes them into the pair's
// slot of the A ring where the direct-to-LDS load would have put them (ds_write_b16).  All three are scheduled by
// the loop's own waits: the element loads and the next map load close the load group of the pair's first step, so
// the wait that lets a step's words be read also covers them, the write to LDS follows that wait and precedes the
// LDS reads of the pair (LDS operations of a wave execute in order), and the next element loads follow the write,
// so one register per row suffices.  The map entry is fetched one pair earlier than the elements; the two dependent
// loads hit the L2 and together take less time than the first weights take to come from memory.  Only with one
// chunk per wave (the host sees to it).
// DRAW = false: every wave has exactly one chunk (the host's plan whenever the chunks fit the waves); the code
// that draws further chunks is left out, which frees a fifth of the registers.
template <bool FP6, bool G128, int GR, bool DRAW>
__device__ __forceinline__ void sk_wave(const SkArgs& p, int j, FP6M_AS3 unsigned char* ring)
{
    constexpr int DEPTH = FP6 ? 3 : 4;
    constexpr int AROWS = 4;
    constexpr bool kGroup = G128 && !FP6;                 // group scales apply to INT4 tiles only
    constexpr bool kColumnScale = FP6 || !G128;
    constexpr int unit_steps = kGroup ? 4 : 2;
    constexpr int kPairSlots = pair_slots(DEPTH);         // step pairs of A alive at once
    constexpr int kPair = pair_bytes(AROWS);
    constexpr int kSlot = FP6 ? 3072 : 2048;              // a step's packed words
    constexpr int kWordOps = FP6 ? 3 : 2;                 // direct-to-LDS loads of the packed words per step
    constexpr int kAOps = GR > 0 ? 0 : 1;                 // ... and of A in front of a pair of steps
    constexpr int kGatherOps = GR > 0 ? GR + 1 : 0;       // loads that close the group of a pair's first step (GR > 0)
    constexpr int kReads = FP6 ? 8 : 6;                   // LDS reads per step
    constexpr int kUnroll = kGroup ? 4 : 2;               // steps per loop trip (segments are multiples of it)
    typedef float f2 __attribute__((ext_vector_type(2)));
    const int lane = threadIdx.x;
    const int i = lane >> 4, c = lane & 15, sigma = c >> 3, l = c & 7;
    const int nrows = p.m;                                // <= 4

    DequantConsts kc;
    kc.lo = vgpr_const(0x000f000fu);
    kc.hi = vgpr_const(0x00f000f0u);
    kc.ex = vgpr_const(0x64006400u);
    kc.top2 = vgpr_const(0xc0c0c0c0u);
    kc.exp_man = vgpr_const(0x9f009f00u);

    // ---- chunks.  INT4 region without drawn chunks: the sub-list that chunk j lies in sets the chunk length (a wave has
    // one chunk, so one sub-list); `tile0` = tiles of the sub-lists before it, `j` becomes the index inside it.
    // (The later sub-lists' tile is found with a 32-bit multiply-high: selecting among three 64-bit constants made the
    // compiler keep them in an array in scratch memory, which cost every launch a microsecond.)
    int q = FP6 ? p.q6 : p.q4, cpt = FP6 ? p.cpt6 : p.cpt4, tile0 = 0;
    const int units = FP6 ? p.units6 : p.units4;
    const unsigned long long magic_cpt = FP6 ? p.magic_cpt6 : p.magic_cpt4;
    int first_tile = -1;                                   // tile, inside its sub-list, of the wave's own chunk
    if constexpr (!FP6 && !DRAW) {
        const int chunks_a = p.tiles4a * p.cpt4, chunks_b = p.tiles4b * p.cpt4b;
        if (j >= chunks_a + chunks_b) {                    // (uniform)
            j -= chunks_a + chunks_b;
            tile0 = p.tiles4a + p.tiles4b;
            q = p.q4c;
            cpt = p.cpt4c;
            first_tile = cpt <= 1 ? j : (int)__umulhi((uint32_t)j, p.magic32_cpt4c);
        } else if (j >= chunks_a) {
            j -= chunks_a;
            tile0 = p.tiles4a;
            q = p.q4b;
            cpt = p.cpt4b;
            first_tile = cpt <= 1 ? j : (int)__umulhi((uint32_t)j, p.magic32_cpt4b);
        }
    }
    if (first_tile < 0) first_tile = (int)mul_shift40(magic_cpt, (uint32_t)j);
    static_assert(GR == 0 || !DRAW, "the gather follows one chunk");
    const int total = !DRAW ? 0 : (FP6 ? p.total6 : p.total4);    // 0: one chunk per wave, nothing to draw
    const int region_waves = FP6 ? p.waves6 : p.waves - p.waves6;
    const int region_n = FP6 ? p.qc : p.n4;
    // chunk id -> tile of the region, first unit, units
    auto chunk_tile = [&](int ch) { return DRAW ? (int)mul_shift40(magic_cpt, (uint32_t)ch) : first_tile; };   // (no draw: ch == j)
    auto chunk_len = [&](int kb) { return units - kb < q ? units - kb : q; };
    // A single counter would see every wave's first draw at the same moment (thousands of atomics on one address:
    // tens of microseconds).  The list is therefore dealt into `groups` sub-lists (chunk c belongs to sub-list
    // c mod groups) with a counter each, and wave j draws from sub-list j mod groups: consecutive waves sit on the
    // same XCD, so every sub-list's waves are spread over the whole chip.
    const int groups = FP6 ? p.groups >> 16 : p.groups & 0xffff;
    const int group = j % groups;
    const int group_waves = (region_waves - group + groups - 1) / groups;   // waves j' = group mod groups
    const int group_total = (total - group + groups - 1) / groups;          // chunks of the sub-list
    int* counter = p.counters + (FP6 ? (p.groups & 0xffff) : 0) + group;
    // The next chunk of this wave: drawn by lane 0 with an atomic the compiler does not see (it would wait for every
    // load in flight before handing the result out); the result is used a whole chunk later, when waits for newer
    // loads have long covered it: a chunk issues at least seven loads, the waits let at most six stay in flight.
    uint32_t drawn = 0;                                   // (lane 0) value of the counter before this wave's draw
    auto draw = [&]() {
        if (lane == 0)
            asm volatile("global_atomic_add %0, %1, %2, off sc0 sc1" : "=&v"(drawn) : "v"(counter), "v"(1u) : "memory");
    };
    bool more_chunks = total != 0;                        // false once a draw has come back past the end of the list
    if (more_chunks) draw();

    // ---- fetch side (lane = position in the slot).  Uniform 64-bit bases advance on the scalar unit; each lane
    // only contributes a constant 32-bit offset.
    const uint32_t v4 = (lane ^ ((lane >> 4) & 3)) * 16;
    const size_t kblocks = (size_t)p.k / 16;
    const bool native = (p.flags & 1) != 0;
    const SkEpilogue ep = {(p.flags >> 1) & 1, p.n, p.c_cols, p.bias, p.residual, p.C};
    const size_t row4 = native ? 1024 : (size_t)region_n * 8, row2 = row4 / 2;
    const size_t tile_stride4 = native ? kblocks * 1024 : 1024, tile_stride2 = tile_stride4 / 2;
    const unsigned char* plane4 = reinterpret_cast<const unsigned char*>(FP6 ? p.b_fp6_4 : p.b_int4);
    const unsigned char* plane2 = reinterpret_cast<const unsigned char*>(p.b_fp6_2);
    // Fetch position: chunk, tile, step inside the tile, steps of the chunk not yet fetched; as 32-bit byte offsets
    // from the planes' bases (the host sends planes of 4 GiB and more to the other kernel).
    int f_chunk = j;
    int i_tcol = chunk_tile(j);
    int i_step = (j - i_tcol * cpt) * q * unit_steps;
    int i_left = chunk_len((j - i_tcol * cpt) * q) * unit_steps;
    i_tcol += tile0;
    const uint32_t step4 = 2 * (uint32_t)row4, step2 = 2 * (uint32_t)row2;
    uint32_t off4 = (uint32_t)i_tcol * (uint32_t)tile_stride4 + (uint32_t)i_step * step4;
    uint32_t off2 = (uint32_t)i_tcol * (uint32_t)tile_stride2 + (uint32_t)i_step * step2;
    const int lg = lane & 31;
    const uint32_t v2 = (uint32_t)((lane >> 5) * row2) + (lg ^ (lg >> 4)) * 16;
    // A: the lower half of the wave brings rows 0 .. 3, eight lanes per row (see stream_tile); rows past m re-read
    // row m-1, so the lanes that take part never depend on m.
    const bool a_lane = lane < 32;
    uint32_t vap;
    {
        const int prow = (lane >> 3) & 3, pch = lane & 7;
        const int row = prow < nrows ? prow : nrows - 1;
        vap = (uint32_t)row * (uint32_t)p.k * 2 + 16 * ((pch & 4) | ((pch & 3) ^ ((prow >> 1) & 3)));
    }
    const unsigned char* a0 = reinterpret_cast<const unsigned char*>(p.A);
    uint32_t offa = (uint32_t)i_step * 64;
    FP6M_AS3 unsigned char* a_ring = ring + DEPTH * kSlot;
    int pair_in = 0;
    const unsigned char* gs0 = reinterpret_cast<const unsigned char*>(p.s_int4);
    const uint32_t gs_row = (uint32_t)p.n4 * 2;          // bytes from one group's scales to the next
    const uint32_t vgs = 4 * lane;
    FP6M_AS3 unsigned char* gs_ring = a_ring + kPairSlots * kPair;
    int gs_in = 0;                                        // group-scale slab the next fetch fills (two alternate)

    // `even`: the step fetched is the first of its pair (a compile-time fact at every call).  Returns whether a
    // load of group scales went out.  With the current chunk used up, the position first moves to the wave's next
    // chunk (and the chunk after that is drawn); with no chunk left, the last step is fetched again.
    auto issue = [&](int slot, bool even) {
        if (i_left == 0 && more_chunks) {                 // (uniform)
            asm volatile("" : "+v"(drawn));
            const int drawn_index = group_waves + (int)__builtin_amdgcn_readfirstlane(drawn);   // position in the sub-list
            const int next = group + groups * drawn_index;
            if (drawn_index < group_total) {
                f_chunk = next;
                i_tcol = chunk_tile(next);                // (drawn chunks: one sub-list, tile0 = 0)
                const int kb = (next - i_tcol * cpt) * q;
                i_step = kb * unit_steps;
                i_left = chunk_len(kb) * unit_steps;
                off4 = (uint32_t)i_tcol * (uint32_t)tile_stride4 + (uint32_t)i_step * step4;
                off2 = (uint32_t)i_tcol * (uint32_t)tile_stride2 + (uint32_t)i_step * step2;
                offa = (uint32_t)i_step * 64;
                draw();
            } else {
                more_chunks = false;
                // every wave draws exactly one number past the end; whoever draws the last of them leaves the
                // counter at zero for the next launch
                if (lane == 0 && drawn_index == group_total + group_waves - 1)
                    __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
        FP6M_AS3 unsigned char* dst = ring + slot * kSlot;
        if (GR == 0 && even) {
            if (a_lane) dma16(a0 + offa + vap, a_ring + pair_in * kPair);
            pair_in = pair_in + 1 == kPairSlots ? 0 : pair_in + 1;
            offa += i_left > 2 ? 128u : 0u;               // (a chunk's last pair stays, for the repeats at the very end)
        }
        dma16_stream(plane4 + off4 + v4, dst);
        dma16_stream(plane4 + off4 + (uint32_t)row4 + v4, dst + 1024);
        if (FP6) dma16_stream(plane2 + off2 + v2, dst + 2048);
        const bool scales = kGroup && (i_step & 3) == 0 && i_left > 0;   // (not for the repeats)
        if (scales) {
            dma4(gs0 + (uint32_t)i_tcol * (kTileN * 2) + (uint32_t)(i_step >> 2) * gs_row + vgs, gs_ring + gs_in * 256);
            gs_in ^= 1;
        }
        // on to the chunk's next step; after its last step the position stays (i_left == 0)
        const bool more = i_left > 1;
        i_left -= i_left > 0 ? 1 : 0;
        i_step += more ? 1 : 0;
        off4 += more ? step4 : 0u;
        off2 += more ? step2 : 0u;
        return scales;
    };
    static_assert(!kGroup || DEPTH == 4, "the steps whose waits count a load of group scales are written out for depth 4");
    // Loads that may be outstanding when the step after the current one must have landed: those of the DEPTH - 2
    // newest steps, the first of them odd / even in its pair.  With the gather, the newest step's closing loads
    // have not been issued yet at that point (they follow the wait), those of the one before have.
    constexpr int kWaitOdd = newer_step_ops(kWordOps, kAOps, 1, DEPTH - 2);
    constexpr int kWaitEven = newer_step_ops(kWordOps, kAOps, 0, DEPTH - 2) + (DEPTH - 2 >= 2 ? kGatherOps : 0);
    static_assert(GR == 0 || DEPTH == 3 || DEPTH == 4, "where the gather's loads sit among the counted ones");

    // ---- gather (GR > 0): lane = column of the pair
    uint32_t midx = 0, gval[GR > 0 ? GR : 1] = {};
    const unsigned char* maps = reinterpret_cast<const unsigned char*>(p.a_cols);
    const unsigned char* arow[GR > 0 ? GR : 1];
    uint32_t wofs[GR > 0 ? GR : 1];
#pragma unroll
    for (int r = 0; r < (GR > 0 ? GR : 1); r++) {
        const int row = r < nrows ? r : nrows - 1;
        arow[r] = a0 + (size_t)row * (size_t)p.lda * 2;
        // position of column `lane` of the pair in row r of a slot: see the swizzle of the fetch side above
        wofs[r] = (uint32_t)(uintptr_t)a_ring +
                  (8 * r + 4 * (lane >> 5) + (((lane >> 3) & 3) ^ ((r >> 1) & 3))) * 16 + 2 * (lane & 7);
    }
    // byte offsets into the map of the pair whose entry is loaded next / of the chunk's last pair (a wave has one
    // chunk; past its end the last pair is loaded again, like the words)
    uint32_t m_off = (uint32_t)i_step * 128, m_last = m_off + (uint32_t)(i_left / 2 - 1) * 256;
    const int lda_max = p.lda - 1;
    auto load_map = [&](uint32_t& dst) {
        asm volatile("global_load_dword %0, %1, %2" : "=&v"(dst) : "v"(m_off + 4 * (uint32_t)lane), "s"(maps) : "memory");
        m_off += m_off < m_last ? 256u : 0u;
    };
    auto load_vals = [&](uint32_t& idx) {
        asm volatile("" : "+v"(idx));
        int col = (int)idx;
        col = col < 0 ? 0 : (col > lda_max ? lda_max : col);
        const uint32_t vo = 2 * (uint32_t)col;
#pragma unroll
        for (int r = 0; r < GR; r++)
            asm volatile("global_load_ushort %0, %1, %2" : "=&v"(gval[r]) : "v"(vo), "s"(arow[r]) : "memory");
    };
    auto write_vals = [&](int pair_slot) {
#pragma unroll
        for (int r = 0; r < GR; r++)
            asm volatile("ds_write_b16 %0, %1" : : "v"(wofs[r] + pair_slot * kPair), "v"(gval[r]) : "memory");
    };

    // ---- read side (lane = MFMA identity)
    const int owner = native ? lane : 32 * sigma + 4 * l + i;     // whose granule of the k-block this lane needs
    const uint32_t ring_lds = (uint32_t)(uintptr_t)ring;
    const uint32_t rd4 = ring_lds + (owner ^ ((owner >> 4) & 3)) * 16;
    const int gr2 = owner >> 1;
    const uint32_t rd2 = ring_lds + 2048 + (gr2 ^ (gr2 >> 4)) * 16 + (owner & 1) * 8;
    const int ar = c & (AROWS - 1);                       // rows beyond AROWS re-read a valid row; their sums are never stored
    uint32_t rda[4];
#pragma unroll
    for (int d = 0; d < 4; d++)
        rda[d] = (uint32_t)(uintptr_t)a_ring + (8 * ar + (d ^ ((ar >> 1) & 3))) * 16 + 4 * i;
    const uint32_t rdgs = (uint32_t)(uintptr_t)gs_ring + (64 * (i >> 1) + 4 * (i & 1)) * 2;
    int gs_rd = 0;
    // behind the ring: 4 rows of kRedStride floats (an LDS-space pointer: no generic-address arithmetic)
    FP6M_AS3 float* slab = (FP6M_AS3 float*)(ring + wave_lds_bytes(4, 3, 4));

    auto fetch = [&](StepRegs& rg, int slot, int pair_slot, bool odd) {
        const uint32_t so = slot * kSlot;
        if (FP6) {
            asm volatile(
                "ds_read_b128 %0, %4\n\tds_read_b128 %1, %4 offset:1024\n\t"
                "ds_read_b64 %2, %5\n\tds_read_b64 %3, %5 offset:512"
                : "=&v"(rg.q0), "=&v"(rg.q1), "=&v"(rg.t0), "=&v"(rg.t1) : "v"(rd4 + so), "v"(rd2 + so) : "memory");
        } else {
            asm volatile("ds_read_b128 %0, %2\n\tds_read_b128 %1, %2 offset:1024"
                         : "=&v"(rg.q0), "=&v"(rg.q1) : "v"(rd4 + so) : "memory");
        }
        const uint32_t ao = pair_slot * kPair;
        if (odd)                                // the second step of a pair: the other half of every row's line
            asm volatile("ds_read_b32 %0, %4 offset:64\n\tds_read_b32 %1, %5 offset:64\n\t"
                         "ds_read_b32 %2, %6 offset:64\n\tds_read_b32 %3, %7 offset:64"
                         : "=&v"(rg.a[0]), "=&v"(rg.a[1]), "=&v"(rg.a[2]), "=&v"(rg.a[3])
                         : "v"(rda[0] + ao), "v"(rda[1] + ao), "v"(rda[2] + ao), "v"(rda[3] + ao) : "memory");
        else
            asm volatile("ds_read_b32 %0, %4\n\tds_read_b32 %1, %5\n\tds_read_b32 %2, %6\n\tds_read_b32 %3, %7"
                         : "=&v"(rg.a[0]), "=&v"(rg.a[1]), "=&v"(rg.a[2]), "=&v"(rg.a[3])
                         : "v"(rda[0] + ao), "v"(rda[1] + ao), "v"(rda[2] + ao), "v"(rda[3] + ao) : "memory");
    };
    auto settle = [&](StepRegs& rg) {
        asm volatile("" : "+v"(rg.q0), "+v"(rg.q1), "+v"(rg.a[0]), "+v"(rg.a[1]), "+v"(rg.a[2]), "+v"(rg.a[3]));
        if (FP6) asm volatile("" : "+v"(rg.t0), "+v"(rg.t1));
    };
    auto compute = [&](const StepRegs& rg, f4 (&dst)[8], bool fresh) {
        const h8 av = __builtin_bit_cast(h8, u4{rg.a[0], rg.a[1], rg.a[2], rg.a[3]});
        const f4 zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int jj = 0; jj < 4; jj++) {
            h2 r0[4], r1[4];
            if (FP6) {
                dequant_fp6_fast(rg.t0[jj >> 1] << (4 * (jj & 1)), rg.q0[jj], kc, r0);
                dequant_fp6_fast(rg.t1[jj >> 1] << (4 * (jj & 1)), rg.q1[jj], kc, r1);
            } else {
                dequant_int4_fast(rg.q0[jj], kc, r0);
                dequant_int4_fast(rg.q1[jj], kc, r1);
            }
            const h8 w_lo = join(r0[0], r0[1], r1[0], r1[1]);  // columns 16j + l
            const h8 w_hi = join(r0[2], r0[3], r1[2], r1[3]);  // columns 16j + 8 + l
            dst[2 * jj + 0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(w_lo, av, fresh ? zero : dst[2 * jj + 0], 0, 0, 0);
            dst[2 * jj + 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(w_hi, av, fresh ? zero : dst[2 * jj + 1], 0, 0, 0);
        }
    };

    // ---- what has been added to shared tiles and not yet looked at
    PendingCells pend;
    pend.parts = 0;
    auto settle_pending = [&]() {
        if (pend.parts == 0) return;                                     // (uniform)
        const FusedCols fcols = fused_cols(ep, pend.col0 + 2 * lane);
        uint16_t* c_out = p.C + pend.col0 + 2 * lane;
#pragma unroll
        for (int rr = 0; rr < 4; rr++) {
            if (rr >= nrows) continue;
#pragma unroll
            for (int e = 0; e < 2; e++) {
                if ((int)(pend.old[rr][e] >> 56) != pend.parts - 1) continue;   // somebody else arrives last at this element
                const float v = cell_total(pend.old[rr][e], cell_contribution(pend.v[rr][e]), pend.parts);
                __hip_atomic_store(pend.cell + rr * kTileN + 64 * e, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if (ep.fused)
                    store_fused_one(ep, fcols, (size_t)rr, e, v);
                else
                    c_out[(size_t)rr * p.n + e] = __builtin_bit_cast(uint16_t, (_Float16)v);
            }
        }
        pend.parts = 0;
    };

    // Pipeline: while step s is being computed, the LDS reads of step s+1 are in flight and the
    // direct-to-LDS loads of steps s+2 .. s+DEPTH-1 are outstanding.
    int slot_in = 0;
    uint32_t midx0 = 0;
    if constexpr (GR > 0) {
        load_map(midx0);
        load_map(midx);
    }
#pragma unroll
    for (int d = 0; d < DEPTH - 1; d++) {
        issue(slot_in, (d & 1) == 0);
        slot_in = slot_in + 1 == DEPTH ? 0 : slot_in + 1;
    }
    constexpr int kPrologueOps = (DEPTH - 1) * kWordOps + (kGroup ? 1 : 0);   // (a chunk's first step starts a group)
    StepRegs regs[2];
    if constexpr (GR > 0) {
        // The map entries of the first two pairs were the oldest loads (see below): wait for them only, fetch the
        // first pair's elements, and wait for those, which also completes the words of the steps fetched ahead.
        __builtin_amdgcn_s_waitcnt(vmcnt_only(kPrologueOps));
        load_vals(midx0);
        __builtin_amdgcn_s_waitcnt(vmcnt_only(0));
        write_vals(0);
        if (DEPTH - 1 > 2) {                                   // the second pair's first step is among those fetched ahead
            load_vals(midx);
            load_map(midx);
        }
    } else {
        __builtin_amdgcn_s_waitcnt(vmcnt_only(kWaitOdd));     // step 0 has landed; step 1 is the oldest newer one
    }
    FP6M_MARK(p, 1);
    fetch(regs[0], 0, 0, false);
    int slot_rd = 1;                                      // slot of the step whose LDS reads come next
    int pair_rd = 0;                                      // A ring slot of the pair that step belongs to
    bool scales_in_flight = false;
    f4 grp[8];
    f4 acc[8];
#pragma unroll
    for (int t = 0; t < 8; t++) acc[t] = f4{0.f, 0.f, 0.f, 0.f};

    int c_chunk = j;                                      // the chunk the multiply side is on
    while (true) {                                                       // (uniform) one chunk per trip
        int tcol = chunk_tile(c_chunk);
        const int kb = (c_chunk - tcol * cpt) * q;
        const int len = chunk_len(kb);
        tcol += tile0;
        const int tile = FP6 ? tcol : p.tiles6 + tcol;
        const int col0 = (FP6 ? p.n4 : 0) + tcol * kTileN;
        h2 sv = {(_Float16)1.0f, (_Float16)1.0f};
        if (kColumnScale) {                                              // fetched now, used after the segment
            const int nr = tcol * kTileN + 2 * lane;                     // even column inside the region
            sv = *reinterpret_cast<const h2*>((FP6 ? p.s_fp6 : p.s_int4) + (nr & ~31) + scale_slot(nr & 31));
        }
        const int seg_steps = len * unit_steps;
#pragma unroll 1
        for (int s = 0; s < seg_steps; s += kUnroll) {
#pragma unroll
            for (int uu = 0; uu < kUnroll; uu++) {
                const bool scales = issue(slot_in, ((uu + DEPTH - 1) & 1) == 0);
                slot_in = slot_in + 1 == DEPTH ? 0 : slot_in + 1;
                if (kGroup && uu == 1) scales_in_flight = scales;         // the fetch of the step four on: a multiple of four
                const bool one_more = kGroup && (uu == 1 || uu == 2) && scales_in_flight;
                if (uu & 1) {                                             // the next step has landed
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
                if (uu & 1) pair_rd = pair_rd + 1 == kPairSlots ? 0 : pair_rd + 1;   // the next step opens a pair
                if constexpr (GR > 0) {
                    if (uu & 1) write_vals(pair_rd);                       // its elements have landed with its words
                    if (((uu + DEPTH - 1) & 1) == 0) {                     // the step just fetched opens a pair: close its group
                        load_vals(midx);
                        load_map(midx);
                    }
                }
                fetch(regs[(uu + 1) & 1], slot_rd, pair_rd, (uu & 1) == 0);
                slot_rd = slot_rd + 1 == DEPTH ? 0 : slot_rd + 1;
                __builtin_amdgcn_s_waitcnt(lgkmcnt_only(kReads));         // reads of this step (older) are done
                settle(regs[uu & 1]);
                if (kGroup)
                    compute(regs[uu & 1], grp, uu == 0);
                else
                    compute(regs[uu & 1], acc, false);
            }
            if (kGroup) {
                // end of a 128-row group: fold it into the running sum with its scales (fp32)
                const uint32_t ga = rdgs + gs_rd * 256;
                gs_rd ^= 1;
                u2 sc[8];
                asm volatile(
                    "ds_read_b64 %0, %8\n\tds_read_b64 %1, %8 offset:16\n\tds_read_b64 %2, %8 offset:32\n\t"
                    "ds_read_b64 %3, %8 offset:48\n\tds_read_b64 %4, %8 offset:64\n\tds_read_b64 %5, %8 offset:80\n\t"
                    "ds_read_b64 %6, %8 offset:96\n\tds_read_b64 %7, %8 offset:112\n\ts_waitcnt lgkmcnt(0)"
                    : "=&v"(sc[0]), "=&v"(sc[1]), "=&v"(sc[2]), "=&v"(sc[3]), "=&v"(sc[4]), "=&v"(sc[5]), "=&v"(sc[6]),
                      "=&v"(sc[7])
                    : "v"(ga) : "memory");
                settle(regs[0]);                              // lgkmcnt(0) also completed the look-ahead reads
#pragma unroll
                for (int t = 0; t < 8; t++) {
                    const h2 lo = as_h2(sc[t][0]), hi = as_h2(sc[t][1]);
                    acc[t][0] += (float)lo[0] * grp[t][0];
                    acc[t][1] += (float)lo[1] * grp[t][1];
                    acc[t][2] += (float)hi[0] * grp[t][2];
                    acc[t][3] += (float)hi[1] * grp[t][3];
                }
            }
        }
        FP6M_MARK(p, 2);

        // ---- end of the chunk: the look-ahead reads of the next step stay in flight, the ring is not touched
        __builtin_amdgcn_s_waitcnt(lgkmcnt_only(0));
        settle(regs[0]);
        const int parts = cpt;                                           // chunks (= waves) that share the tile
        settle_pending();                                                // the previous chunk's atomics are long back
        // MFMA fragments -> fp32 rows in the slab (lane c holds row c of the tile's 16), read back with lane L owning
        // columns 2L, 2L+1.  LDS operations of one wave execute in order: no barrier is needed.
        const float rescale = FP6 ? 4096.0f : 1.0f;                      // the deferred e3m2 exponent re-bias
        if (c < nrows) {
            FP6M_AS3 float* mine = slab + c * kRedStride + 64 * (i >> 1) + 4 * (i & 1);
#pragma unroll
            for (int t = 0; t < 8; t++) *(FP6M_AS3 f4*)(mine + 16 * (t >> 1) + 8 * (t & 1)) = acc[t];
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        const float s0 = (float)sv[0] * rescale, s1 = (float)sv[1] * rescale;
        float v0[4], v1[4];
#pragma unroll
        for (int rr = 0; rr < 4; rr++) {
            const f2 t = *(const FP6M_AS3 f2*)(slab + (rr < nrows ? rr : 0) * kRedStride + 2 * lane);
            v0[rr] = t[0] * s0;
            v1[rr] = t[1] * s1;
        }
#pragma unroll
        for (int t = 0; t < 8; t++) acc[t] = f4{0.f, 0.f, 0.f, 0.f};
        FP6M_MARK(p, 3);
        if (parts == 1) {
            const FusedCols fcols = fused_cols(ep, col0 + 2 * lane);
            uint16_t* c_out = p.C + col0 + 2 * lane;
#pragma unroll
            for (int rr = 0; rr < 4; rr++) {
                if (rr >= nrows) continue;
                if (ep.fused) {
                    store_fused(ep, fcols, (size_t)rr, v0[rr], v1[rr]);
                } else {
                    const h2 o = {(_Float16)v0[rr], (_Float16)v1[rr]};
                    *reinterpret_cast<h2*>(c_out + (size_t)rr * p.n) = o;
                }
            }
        } else {
            // Shared tile: one returning atomic per element (cells of a row: 64 of the even columns, then 64 of the odd)
            pend.cell = p.cells + (size_t)tile * nrows * kTileN + lane;
            pend.parts = parts;
            pend.col0 = col0;
#pragma unroll
            for (int rr = 0; rr < 4; rr++) {
                pend.v[rr][0] = v0[rr];
                pend.v[rr][1] = v1[rr];
                if (rr < nrows) {
                    pend.old[rr][0] = __hip_atomic_fetch_add(pend.cell + rr * kTileN, cell_contribution(v0[rr]), __ATOMIC_RELAXED,
                                                             __HIP_MEMORY_SCOPE_AGENT);
                    pend.old[rr][1] = __hip_atomic_fetch_add(pend.cell + rr * kTileN + 64, cell_contribution(v1[rr]),
                                                             __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            }
            FP6M_MARK(p, 4);
        }
        if (f_chunk == c_chunk) break;                                   // the fetch side found no further chunk
        c_chunk = f_chunk;                                               // (it is never more than one chunk ahead)
    }
    // Redundant tail prefetches and look-ahead reads may still be in flight.
    __builtin_amdgcn_s_waitcnt(vmcnt_only(0) & lgkmcnt_only(0));
    settle(regs[0]);
    settle(regs[1]);
    if constexpr (GR > 0) {
        asm volatile("" : "+v"(midx));
#pragma unroll
        for (int r = 0; r < GR; r++) asm volatile("" : "+v"(gval[r]));
    }
    settle_pending();
    FP6M_MARK(p, 6);
}

constexpr int kSkWaveLds = wave_lds_bytes(4, 3, 4) + 4 * kRedStride * 4;   // ring, then the four-row slab

// Position of workgroup (= wave) b in the chunk list.  The chip gives the first gen_waves waves of a launch a SIMD each
// (workgroup b is the (b / 8)-th on its XCD, and an XCD's first gen_waves / 8 land on different SIMDs); the next
// gen_waves share a SIMD with one of those, and so on.  A SIMD serves its older wave first: with equal chunks the
// second generation finishes a third later than the first and the third later still, and the launch ends on a thinning
// tail (8192 x 57344 at one row: loops end at 27.7 us in the first generation, at 37 us in the second).  The host
// therefore gives later generations shorter chunks, and this order puts them where they belong: generation-major, and
// inside a generation every XCD a contiguous range, as xcd_contiguous_id does for the whole list (gen_waves = 0).
__device__ __forceinline__ int sk_generation_order(int b, int total, int gen_waves)
{
    if (gen_waves == 0 || total <= gen_waves) return xcd_contiguous_id(b, total);
    const int per = gen_waves >> 3;                        // waves of one generation on one XCD
    const int x = b & 7, i = b >> 3;
    const int g = (i >= per) + (i >= 2 * per) + (i >= 3 * per);   // (the host plans at most four generations)
    const int rest = total - g * gen_waves;                // waves of this and later generations
    if (rest >= gen_waves) return g * gen_waves + x * per + (i - g * per);
    return g * gen_waves + xcd_contiguous_id(((i - g * per) << 3) | x, rest);   // the last, partly filled generation
}

// second launch-bound argument = waves per SIMD the register budget must allow (HIP semantics)
// EXTRAS = false: the build for one row, without a fused epilogue, on reference-order words (the arguments that select
// anything else are overwritten with constants: the presence of the epilogue's branches cost the plain call 1-3 %, the
// code for two to four rows another 1-5 %, 8192 x 8192 10.7 -> 10.2 us).
template <bool G128, int GR, bool DRAW, bool EXTRAS = true>
__global__ __launch_bounds__(64, 3) void gemm_sk_kernel(const SkArgs in_kernarg_segment)
{
    __shared__ __attribute__((aligned(16))) unsigned char smem[kSkWaveLds];
    SkArgs p = load_sk_args();
    if constexpr (!EXTRAS) {
        p.m = 1;
        p.flags = 0;
        p.c_cols = nullptr;
        p.bias = nullptr;
        p.residual = nullptr;
    }
    FP6M_MARK(p, 0);
#ifdef FP6M_TIMELINE
    if (p.timeline) {                                                    // where the wave runs: HW_ID and XCC_ID registers
        const uint32_t hw = __builtin_amdgcn_s_getreg((4 << 0) | (0 << 6) | (31 << 11));
        const uint32_t xcc = __builtin_amdgcn_s_getreg((20 << 0) | (0 << 6) | (3 << 11));
        p.timeline[(size_t)blockIdx.x * 8 + 5] = ((unsigned long long)xcc << 32) | hw;
    }
#endif
    const int logical = sk_generation_order(blockIdx.x, p.waves, p.gen_waves);
    if (logical < p.waves6)                                              // the FP6 region's waves come first
        sk_wave<true, G128, GR, DRAW>(p, logical, (FP6M_AS3 unsigned char*)smem);
    else
        sk_wave<false, G128, GR, DRAW>(p, logical - p.waves6, (FP6M_AS3 unsigned char*)smem);
    FP6M_MARK(p, 7);
}

}  // namespace fp6m
