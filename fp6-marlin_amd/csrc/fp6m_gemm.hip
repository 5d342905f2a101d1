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
//  * A workgroup is four (or eight) such waves splitting k; they are summed through LDS.  `ksplit` workgroups may
//    share a tile; each writes its fp32 partial tile to a per-device scratch, and the workgroup that
//    arrives last (one atomic counter per tile in `workspace`) sums the partials in a fixed order,
//    applies the scales and writes fp16 C.  Nobody spins, so there is nothing to deadlock on, and the
//    counters are zero again when the launch drains.
//  * INT4 and FP6 tiles are entries of one tile list handled by the same launch; FP6 tiles, whose steps cost
//    more, may have their k range cut into twice as many parts.
//  * Activations are fetched a whole 128-byte line of every row at a time (two k steps): a wave's rate is set by
//    its memory requests in flight, not by their bytes.
//  * The dispatcher picks the kernel by m, and for m <= 16 the waves per workgroup and the k split per shape
//    (a rule plus a small cost model fitted to per-workgroup timelines on MI355X).
//
// gemm_common.h  argument block, tile bookkeeping, load / wait / dequantisation helpers
// gemm_sk.h      gemm_sk_kernel (one row: the decode kernel)
// gemm_m16.h     gemm_m16_kernel (m <= 16)
// gemm_mb.h      gemm_mb_kernel (16 < m)
// this file      activation gather, per-device scratch, dispatch and the extern "C" entry points
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>

#include "fp6m.h"
#include "gemm_common.h"
#include "gemm_m16.h"
#include "gemm_sk.h"
#include "gemm_mb.h"

namespace fp6m {

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

// Overrides of the dispatcher's choices, for tests and tuning runs (fp6m_tuning_set).  The product path reads no
// environment variables; FP6M_VERBOSE alone is looked up once, when the library is loaded.
constexpr int kUnset = INT32_MIN;
const int g_env_verbose = getenv("FP6M_VERBOSE") ? 1 : 0;
struct Tuning {
    int mb = kUnset, ksplit = kUnset, wk16 = kUnset, wk = kUnset, pair = kUnset, wgs = kUnset, share = kUnset, share6 = kUnset, sk = kUnset, cap = kUnset, gather = kUnset, cells = kUnset, xcd = kUnset, gen = kUnset, gen2 = kUnset, gen3 = kUnset, young = kUnset, cls = kUnset, cus = kUnset, cap2 = kUnset;
    int verbose = g_env_verbose;
};
Tuning g_tuning;

// Device memory the GEMM needs beyond its operands: fp32 partial tiles of column tiles whose k range is shared by
// several workgroups, the accumulate-and-count cells, and the buffer that gathered activations pass through.  The
// reference keeps its partial sums in C under the locks in the caller's `workspace`, so its rule is one call at a
// time per workspace, and two calls with two workspaces may overlap.  Here the rule is the same because the scratch
// belongs to the workspace: every workspace address that is in use on a device owns a region.  A device has
// kMaxRegions of them.  The first kStaticSlots are slots of a file-scope device array, so an ordinary call allocates
// nothing and never waits for the device; the others get their memory from hipMalloc (synchronous) when a fifth,
// sixth .. workspace turns up, and keep it: memory that a captured graph may hold the address of is never freed
// behind the caller's back.  When every region is taken, the one whose workspace has gone unused longest is handed
// to the newcomer after a hipDeviceSynchronize (callers that make a new workspace per call, as the reference's own
// test.py:168 and bench.py:44 do, never run out); a call that is being captured cannot wait and is refused instead.
struct Region {
    const void* workspace = nullptr;   // null: nobody's
    float* partials = nullptr;      // kScratchBytes of partial tiles (m > 16, row mix), then kCellBytes of cells (m <= 16)
    uint16_t* gathered = nullptr;   // kGatherBytes, allocated by the first gathering call that gets this region
    unsigned long long last_use = 0;
    int pins = 0;                   // host threads between looking the region up and having launched with it
};
constexpr size_t kGatherBytes = size_t(64) << 20;
constexpr int kMaxDevices = 64;
constexpr int kMaxRegions = 16;     // per device
constexpr int kStaticSlots = 4;     // of them in the code object's own memory
constexpr size_t kRegionBytes = kScratchBytes + kCellBytes;
static __device__ __align__(256) unsigned char g_slot_scratch[kStaticSlots * kRegionBytes];   // (zero when loaded, like a fresh region)
// Partial-tile scratch of fp6m_mul_static, the entry point for callers that must not allocate: part of the loaded
// code object, so every GPU the library runs on holds its own copy until the process ends.  In host code the
// array's name is only a handle; its device address is looked up once per device (device_state) and kept there.
constexpr size_t kStaticTileBytes = size_t(12) << 20;                  // partial tiles, then kCellBytes of cells
constexpr size_t kStaticScratchBytes = kStaticTileBytes + kCellBytes;
static __device__ __align__(256) unsigned char g_static_scratch[kStaticScratchBytes];

struct DeviceState {
    int cus = 0;
    int xcd_placement = -1;            // 1: workgroup b of a grid runs on XCD b % 8 (verified by verify_placement), 0: not so, -1: not looked at yet
    float* static_scratch = nullptr;   // device address of this GPU's copy of g_static_scratch
    unsigned char* slot_scratch = nullptr;   // ... and of g_slot_scratch
    unsigned char* pool = nullptr;           // kStaticSlots regions from one hipMalloc (see workspace_region)
    unsigned long long tick = 0;
    void* pack_temp = nullptr;      // kPackTempBytes for the on-GPU packer's flag and column maxima
    Region regions[kMaxRegions];
};
DeviceState g_devices[kMaxDevices];
std::mutex g_scratch_mutex;

int hip_fail(hipError_t e)
{
    g_last_hip_error = (int)e;
    return FP6M_ERR_HIP;
}

// Runs `fn` with `dev` as the calling thread's current device and puts the previous one back.
template <typename F>
hipError_t on_device(int dev, F&& fn)
{
    int prev = 0;
    hipError_t e = hipGetDevice(&prev);
    if (e != hipSuccess) return e;
    if (prev != dev && (e = hipSetDevice(dev)) != hipSuccess) return e;
    e = fn();
    if (prev != dev) (void)hipSetDevice(prev);
    return e;
}

// Compute units of the device and the address of its copy of the static scratch (both looked up once, with the
// device current; no allocation).  Callers hold g_scratch_mutex.
int device_state(int dev, DeviceState** out)
{
    if (dev < 0 || dev >= kMaxDevices) return FP6M_ERR_ARG;
    DeviceState& d = g_devices[dev];
    if (!d.cus) {
        int cus = 0;
        void *sym = nullptr, *slots = nullptr;
        const hipError_t e = on_device(dev, [&] {
            hipError_t e2 = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
            if (e2 == hipSuccess) e2 = hipGetSymbolAddress(&sym, HIP_SYMBOL(g_static_scratch));
            if (e2 == hipSuccess) e2 = hipGetSymbolAddress(&slots, HIP_SYMBOL(g_slot_scratch));
            return e2;
        });
        if (e != hipSuccess) return hip_fail(e);
        if (!sym || !slots) return hip_fail(hipErrorInvalidSymbol);
        d.static_scratch = static_cast<float*>(sym);
        d.slot_scratch = static_cast<unsigned char*>(slots);
        d.cus = cus > 0 ? cus : 256;
    }
    *out = &d;
    return FP6M_OK;
}

// Every workgroup notes the XCD it runs on in the mask of its group of eight consecutive workgroups.
constexpr int kProbeGroups = 512;
__global__ __launch_bounds__(64) void placement_probe_kernel(unsigned* masks)
{
    if (threadIdx.x != 0) return;
    const unsigned linear = blockIdx.y * gridDim.x + blockIdx.x;
    if ((linear >> 3) < kProbeGroups) atomicOr(masks + (linear >> 3), 1u << (xcc_id() & 31));
}

// The XCD-local reduction (gemm_m16.h, wg_finish<LOCAL>) identifies a workgroup by the XCD it finds itself on and its
// index / 8, which covers the work exactly once if eight consecutive workgroups of a dispatch always run on eight
// different XCDs.  That is how these GPUs deal out workgroups (the XCD of the first one varies with the queue), but it
// is a property of the machine and of its partition mode, so it is looked at once per device before the dispatcher
// relies on it: a few grids of a probe kernel on the given stream.  This waits for the device (once), so it is
// skipped while `stream` is being captured; until it has run, launches use the agent-scope protocol.  Callers hold
// g_scratch_mutex.
void verify_placement(int dev, DeviceState& d, hipStream_t stream)
{
    if (d.xcd_placement >= 0 || !d.static_scratch) return;
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &cap) != hipSuccess || cap != hipStreamCaptureStatusNone) {
        (void)hipGetLastError();
        return;
    }
    bool ok = true;
    const hipError_t e = on_device(dev, [&] {
        unsigned* masks = reinterpret_cast<unsigned*>(d.static_scratch);   // (partial-tile part of the scratch: no contents to keep)
        static unsigned host[kProbeGroups];
        const dim3 grids[] = {dim3(8), dim3(264), dim3(8 * kProbeGroups), dim3(40, 5), dim3(272, 2)};
        hipError_t e2 = hipDeviceSynchronize();                       // nothing in flight may be using the scratch
        for (const dim3& g : grids) {
            const unsigned groups = g.x * g.y / 8;
            if (e2 == hipSuccess) e2 = hipMemsetAsync(masks, 0, sizeof(host), stream);
            if (e2 != hipSuccess) break;
            hipLaunchKernelGGL(placement_probe_kernel, g, dim3(64), 0, stream, masks);
            e2 = hipGetLastError();
            if (e2 == hipSuccess) e2 = hipStreamSynchronize(stream);
            if (e2 == hipSuccess) e2 = hipMemcpy(host, masks, sizeof(host), hipMemcpyDeviceToHost);
            for (unsigned i = 0; i < groups && e2 == hipSuccess; i++) ok = ok && host[i] == 0xffu;
        }
        return e2;
    });
    if (e != hipSuccess) {
        (void)hipGetLastError();
        ok = false;
    }
    d.xcd_placement = ok ? 1 : 0;
}

// What a call needs to know about its device and its workspace's region, by value: the table may change under
// another thread as soon as the lock is dropped (the region itself is pinned until the call has launched).
struct Scratch {
    int dev = -1, region = -1;
    int cus = 0;
    float* static_scratch = nullptr;
    float* partials = nullptr;
    uint16_t* gathered = nullptr;
    int xcd_placement = 0;
    ~Scratch()
    {
        if (region < 0) return;
        std::lock_guard<std::mutex> lock(g_scratch_mutex);
        g_devices[dev].regions[region].pins--;
    }
};

bool capturing(hipStream_t stream)
{
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &cap) != hipSuccess) {
        (void)hipGetLastError();
        return true;                                                  // (cannot tell: do nothing that a capture forbids)
    }
    return cap != hipStreamCaptureStatusNone;
}

// The region of `workspace` on `dev`, pinned until `out` goes out of scope.  A workspace that has none takes, in this
// order: a region nobody owns that has memory (the built-in slots always do), one without memory (hipMalloc +
// hipMemset, synchronous: the reduction protocols leave what they use zeroed and rely on finding it so), or the
// unpinned region that has gone unused longest, after waiting for the device.  The last two are refused
// (FP6M_ERR_SCRATCH) while `stream` is being captured.
int workspace_region(int dev, const void* workspace, bool want_region, bool want_gather, hipStream_t stream, Scratch* out)
{
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    DeviceState* d = nullptr;
    if (int rc = device_state(dev, &d)) return rc;
    verify_placement(dev, *d, stream);
    out->cus = d->cus;
    out->static_scratch = d->static_scratch;
    out->xcd_placement = d->xcd_placement;
    if (!want_region) return FP6M_OK;
    Region* r = nullptr;
    for (Region& c : d->regions)
        if (c.workspace == workspace) r = &c;
    if (!r) {
        const bool may_wait = !capturing(stream);
        Region *builtin = nullptr, *idle = nullptr, *bare = nullptr, *oldest = nullptr;
        for (int i = 0; i < kMaxRegions; i++) {
            Region& c = d->regions[i];
            if (!c.workspace && i < kStaticSlots && !builtin) builtin = &c;
            if (!c.workspace && i >= kStaticSlots && c.partials && !idle) idle = &c;
            if (!c.workspace && i >= kStaticSlots && !c.partials && !bare) bare = &c;
            if (c.workspace && !c.pins && (!oldest || c.last_use < oldest->last_use)) oldest = &c;
        }
        auto allocate = [&](size_t bytes, void** mem) {
            const hipError_t e = on_device(dev, [&] {
                hipError_t e2 = hipMalloc(mem, bytes);
                if (e2 == hipSuccess) e2 = hipMemset(*mem, 0, bytes);
                return e2;
            });
            if (e != hipSuccess && *mem) (void)hipFree(*mem);
            return e;
        };
        if (builtin) {
            // The first kStaticSlots regions: their memory is the device's pool, one hipMalloc made the first time a
            // call may wait for it (so not by a call that is being captured), and until then the slots of the code
            // object's own array.  Atomics on the latter are slower (the cells of a 4096 x 4096 decode GEMM: 5.7 -> 6.6 us
            // per launch), so the pool is preferred as soon as it exists.
            const int i = (int)(builtin - d->regions);
            if (!d->pool && may_wait) {
                void* mem = nullptr;
                const hipError_t e = allocate(kStaticSlots * kRegionBytes, &mem);
                if (e != hipSuccess) return hip_fail(e);
                d->pool = static_cast<unsigned char*>(mem);
            }
            builtin->partials = reinterpret_cast<float*>((d->pool ? d->pool : d->slot_scratch) + (size_t)i * kRegionBytes);
            r = builtin;
        } else if (idle) {
            r = idle;
        } else if (!may_wait) {
            return FP6M_ERR_SCRATCH;
        } else if (bare) {
            void* mem = nullptr;
            const hipError_t e = allocate(kRegionBytes, &mem);
            if (e != hipSuccess) return hip_fail(e);
            bare->partials = static_cast<float*>(mem);
            r = bare;
        } else if (oldest) {
            const hipError_t e = on_device(dev, [&] { return hipDeviceSynchronize(); });   // nothing in flight uses it now
            if (e != hipSuccess) return hip_fail(e);
            r = oldest;
        } else {
            return FP6M_ERR_SCRATCH;                                  // (every region pinned by a call in progress)
        }
        r->workspace = workspace;
    }
    if (want_gather && !r->gathered) {
        if (capturing(stream)) return FP6M_ERR_SCRATCH;
        void* mem = nullptr;
        const hipError_t e = on_device(dev, [&] { return hipMalloc(&mem, kGatherBytes); });
        if (e != hipSuccess) return hip_fail(e);
        r->gathered = static_cast<uint16_t*>(mem);
    }
    r->last_use = ++d->tick;
    r->pins++;
    out->dev = dev;
    out->region = (int)(r - d->regions);
    out->partials = r->partials;
    out->gathered = r->gathered;
    return FP6M_OK;
}

// Scratch of the on-GPU packer (fp6m_pack.hip): one buffer per device (a pack call waits for its kernels).
int pack_temp(int dev, void** ptr)
{
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    DeviceState* d = nullptr;
    if (int rc = device_state(dev, &d)) return rc;
    if (!d->pack_temp) {
        void* mem = nullptr;
        const hipError_t e = on_device(dev, [&] { return hipMalloc(&mem, kPackTempBytes); });
        if (e != hipSuccess) return hip_fail(e);
        d->pack_temp = mem;
    }
    *ptr = d->pack_temp;
    return FP6M_OK;
}

inline SliceRule make_rule(int units, int nslices)
{
    SliceRule r;
    r.q = units / nslices;
    r.first_long = nslices - units % nslices;
    return r;
}

// k slices of the `ks` parts x `wk` waves of a tile (WaveRule, gemm_common.h).  With eight waves per workgroup and at
// least two units for every wave, the second wave of every SIMD (waves 4-7) gets `young_pct` per cent of what the
// first gets; otherwise all waves get the same.  What does not divide goes to the older waves first.
inline WaveRule make_wave_rule(long long units, long long ks, int wk, int young_pct)
{
    WaveRule r;
    if (ks < 1) ks = 1;
    const long long per_part = units / ks;
    long long lo = per_part / wk, ly = lo;
    if (wk == 8 && per_part >= 16 && young_pct > 0 && young_pct < 100) {
        lo = (per_part * 100 + 2 * (100 + young_pct)) / (4 * (100 + young_pct));     // per_part / (4 (1 + share)), rounded
        if (4 * lo > per_part) lo = per_part / 4;
        ly = (per_part - 4 * lo) / 4;
        if (ly > lo) ly = lo;
    }
    const long long rem = units - ks * (4 * lo + (wk - 4) * ly);
    r.lo = (int)lo;
    r.ly = (int)ly;
    r.eo = (int)(rem < 4 * ks ? rem : 4 * ks);
    r.ey = (int)(rem - r.eo);
    return r;
}

inline FastDiv make_div(long long d, long long max_n)
{
    FastDiv f;
    f.d = (uint32_t)d;
    f.magic = d > 1 && d < 65536 && max_n < 65536 ? (uint32_t)((0x100000000ULL + (unsigned long long)d - 1) / (unsigned long long)d) : 0;
    return f;
}

// m <= 16 configurations: rows of A per ring slot, WN x WK waves, ring depths of INT4 / FP6 tiles.
//   0: rows <= 4,  one tile x four k slices per workgroup, four ring slots (three for FP6 tiles)
//   1: rows <= 16, same shape, 1 KiB of A per slot
// Workgroups of several adjacent tiles (WN > 1) were measured and were never faster on MI355X; the
// kernel keeps the template parameter, only WN = 1 is instantiated.
// Whether a call needs the kernel build with the row mix, the fused epilogue and the gfx950 word order in it.
inline bool needs_extras(const GemmArgs& a) { return a.k4 != 0 || a.fused != 0 || a.native != 0; }

template <bool G128, int AROWS, int WN, int WK, int D4, int D6, bool EXTRAS>
void launch_m16_one(const GemmArgs& a, dim3 grid, hipStream_t stream)
{
    void (*kernel)(const GemmArgs) = gemm_m16_kernel<G128, AROWS, WN, WK, D4, D6, false, EXTRAS>;
    if constexpr (AROWS == 4) {                                       // (the cells serve up to four rows)
        if (a.cells) kernel = gemm_m16_kernel<G128, AROWS, WN, WK, D4, D6, true, EXTRAS>;
    } else {                                                          // (beyond, partial tiles: through one XCD's L2 where placed so)
        if (a.xcd_local) kernel = gemm_m16_kernel<G128, AROWS, WN, WK, D4, D6, false, EXTRAS, true>;
    }
    hipLaunchKernelGGL(kernel, grid, dim3(64 * WN * WK), 0, stream, a);
}

template <int AROWS, int WN, int WK, int D4, int D6>
void launch_m16(const GemmArgs& a, bool g128, dim3 grid, hipStream_t stream)
{
    if (needs_extras(a)) {
        if (g128)
            launch_m16_one<true, AROWS, WN, WK, D4, D6, true>(a, grid, stream);
        else
            launch_m16_one<false, AROWS, WN, WK, D4, D6, true>(a, grid, stream);
    } else {
        if (g128)
            launch_m16_one<true, AROWS, WN, WK, D4, D6, false>(a, grid, stream);
        else
            launch_m16_one<false, AROWS, WN, WK, D4, D6, false>(a, grid, stream);
    }
}

// n / d as (n * magic) >> 40: exact for n < 2^24 and d < 2^16.
inline unsigned long long magic40(long long d) { return ((1ULL << 40) + (unsigned long long)d - 1) / (unsigned long long)d; }

struct M16Config {
    int id, wn, wk;
};

inline M16Config m16_config(int m)
{
    return m <= 4 ? M16Config{0, 1, 4} : M16Config{1, 1, 4};
}

inline void launch_m16_any(const M16Config& cfg, const GemmArgs& a, bool g128, dim3 grid, hipStream_t stream)
{
    if (cfg.wk == 8) {
        if (cfg.id == 0)
            launch_m16<4, 1, 8, 4, 3>(a, g128, grid, stream);
        else
            launch_m16<16, 1, 8, 4, 3>(a, g128, grid, stream);
        return;
    }
    if (cfg.id == 0)
        launch_m16<4, 1, 4, 4, 3>(a, g128, grid, stream);
    else
        launch_m16<16, 1, 4, 4, 3>(a, g128, grid, stream);
}

template <bool G128, int MB, int D4, int D6, int WK, bool PAIR, bool LEAN>
void launch_mb_one(const GemmArgs& a, dim3 grid, hipStream_t stream)
{
    void (*kernel)(const GemmArgs) = gemm_mb_kernel<G128, MB, D4, D6, WK, PAIR, true>;
    // (One of them does not: without the extras the allocator of the four-wave 64-row kernel with per-column scales
    // ends up one register short of its 256 and spills.)
    if constexpr (LEAN && !(MB == 4 && WK == 4 && !G128)) {
        if (!needs_extras(a)) kernel = gemm_mb_kernel<G128, MB, D4, D6, WK, PAIR, false>;
    }
    // (two classes of INT4 tiles: a build of its own of the configurations the dispatcher plans them for)
    // (64-row tiles with per-column scales are two registers short of a build of this kind: the dispatcher knows)
    if constexpr (LEAN && PAIR && MB <= 4 && WK == 8 && !(MB == 4 && !G128)) {
        if (a.groups4b > 0) kernel = gemm_mb_kernel<G128, MB, D4, D6, WK, PAIR, false, true>;
    }
    hipLaunchKernelGGL(kernel, grid, dim3(64 * WK), 0, stream, a);
}

// LEAN: the kernels the dispatcher picks by itself also exist without the extras (those only the tuning hook reaches do not).
template <int MB, int D4, int D6, bool PAIR, bool LEAN = true>
void launch_mb(const GemmArgs& a, bool g128, int wk, dim3 grid, hipStream_t stream)
{
    if (wk == 8) {
        if (g128)
            launch_mb_one<true, MB, D4, D6, 8, PAIR, LEAN>(a, grid, stream);
        else
            launch_mb_one<false, MB, D4, D6, 8, PAIR, LEAN>(a, grid, stream);
    } else {
        if (g128)
            launch_mb_one<true, MB, D4, D6, 4, PAIR, LEAN>(a, grid, stream);
        else
            launch_mb_one<false, MB, D4, D6, 4, PAIR, LEAN>(a, grid, stream);
    }
}

}  // namespace fp6m

extern "C" {

int fp6m_last_hip_error(void) { return fp6m::g_last_hip_error; }

int fp6m_tuning_set(const char* knob, int value)
{
    using fp6m::g_tuning;
    if (!knob) {                                                      // NULL: back to the dispatcher's own choices
        g_tuning = fp6m::Tuning{};                                    // (`verbose` back to what FP6M_VERBOSE said at load time)
        return FP6M_OK;
    }
    const struct { const char* name; int* field; } knobs[] = {
        {"mb", &g_tuning.mb}, {"ksplit", &g_tuning.ksplit},
        {"wk16", &g_tuning.wk16}, {"wk", &g_tuning.wk}, {"pair", &g_tuning.pair}, {"wgs", &g_tuning.wgs}, {"share", &g_tuning.share}, {"share6", &g_tuning.share6}, {"cap", &g_tuning.cap}, {"sk", &g_tuning.sk}, {"gather", &g_tuning.gather}, {"cells", &g_tuning.cells}, {"xcd", &g_tuning.xcd}, {"gen", &g_tuning.gen}, {"gen2", &g_tuning.gen2}, {"gen3", &g_tuning.gen3}, {"young", &g_tuning.young}, {"cls", &g_tuning.cls}, {"cus", &g_tuning.cus}, {"cap2", &g_tuning.cap2},
        {"verbose", &g_tuning.verbose}};
    for (const auto& k : knobs)
        if (!strcmp(knob, k.name)) {
            *k.field = value;
            return FP6M_OK;
        }
    return FP6M_ERR_ARG;
}

int fp6m_init(int dev)
{
    fp6m::Scratch sc;
    return fp6m::workspace_region(dev, nullptr, false, false, nullptr, &sc);
}

int fp6m_init_workspace(int dev, const void* workspace, int with_gather)
{
    if (!workspace) return FP6M_ERR_ARG;
    fp6m::Scratch sc;
    return fp6m::workspace_region(dev, workspace, true, with_gather != 0, nullptr, &sc);
}

int fp6m_release_workspace(int dev, const void* workspace)
{
    using namespace fp6m;
    if (dev < 0 || dev >= kMaxDevices) return FP6M_ERR_ARG;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    DeviceState& d = g_devices[dev];
    bool waited = false;
    for (Region& r : d.regions) {                                     // workspace = NULL: every region of the device
        if (!r.workspace || (workspace && r.workspace != workspace)) continue;
        if (r.pins) return FP6M_ERR_ARG;                              // a call with this workspace is being made right now
        if (!waited) {                                                // nothing in flight may still use the region
            const hipError_t e = on_device(dev, [&] { return hipDeviceSynchronize(); });
            if (e != hipSuccess) return hip_fail(e);
            waited = true;
        }
        r.workspace = nullptr;                                        // (its memory stays with the region for the next owner)
    }
    return FP6M_OK;                                                   // no region: nothing to release
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
// `fixed_scratch` (fp6m_mul_static): partial tiles go to the device's static scratch instead of the workspace's
// region, nothing is allocated, and a launch whose split needs more than the array holds is refused rather than
// given a smaller split.

int mul_common(const void* A, const void* B, void* C, const void* s, int prob_m, int prob_n, int prob_k,
               void* workspace, int dev, void* stream, int thread_k, int thread_n, int sms, int max_par,
               int quant_cols, int group_size, const Fusion& fu, bool fixed_scratch = false)
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

    hipStream_t st = static_cast<hipStream_t>(stream);
    Scratch sc;
    size_t scratch_bytes = kScratchBytes;
    if (fixed_scratch) {
        if (fu.a_cols) return FP6M_ERR_ARG;                           // the gathered activations need a region's buffer
        scratch_bytes = kStaticTileBytes;
    }
    if (int rc = workspace_region(dev, workspace, !fixed_scratch, fu.a_cols != nullptr, st, &sc)) return rc;
    const int cus = g_tuning.cus != kUnset && g_tuning.cus > 0 ? g_tuning.cus : sc.cus;   // (the knob: small test problems on a pretended small chip)
    const int xcd_placement = sc.xcd_placement;
    float* const scratch = fixed_scratch ? sc.static_scratch : sc.partials;

    GemmArgs a;
    a.b_int4 = static_cast<const uint32_t*>(B);
    a.b_fp6_2 = a.b_int4 + (size_t)prob_k * n4 / 8;
    a.b_fp6_4 = a.b_fp6_2 + (size_t)prob_k * qc / 16;
    a.s_int4 = static_cast<const uint16_t*>(s);
    a.s_fp6 = a.s_int4 + (g128 ? (size_t)(prob_k / 128) * n4 : (size_t)n4);
    a.scratch = scratch;
    a.counters = static_cast<int*>(workspace);
    a.cells = nullptr;
    a.n = prob_n;
    a.k = prob_k;
    a.n4 = n4;
    a.qc = qc;
    a.tiles6 = qc / kTileN;
    a.tiles = prob_n / kTileN;
    a.k4 = 0;
    a.slices4 = 0;
    a.xcd_local = 0;
    a.xm4_lo = a.xm4_hi = a.xm6_lo = a.xm6_hi = 0;
    a.wrule[0] = a.wrule[1] = a.wrule_b = WaveRule{0, 0, 0, 0};
    a.groups4b = 0;
    a.ks4b = 1;
    a.div_b = FastDiv{1, 0};
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
    // workgroups per CU) beyond; 128 rows for large launches whose grid allows it (below).
    int mb = prob_m <= 16 ? 1 : (prob_m <= 32 ? 2 : 4);
    const Tuning tune = g_tuning;              // tuning/testing overrides (all unset in production)
    // share of a SIMD that the second of two waves of a workgroup gets, in per cent of the first one's (make_wave_rule).
    // Measured (alternating, us, equal slices -> 72 %): 8192 x 8192 at 8 / 16 / 128 / 256 rows 12.65 -> 12.03 / 13.2 -> 12.65 /
    // 27.95 -> 27.4 / 42.3 -> 41.2, 8192 x 10240 at 16 rows 14.3 -> 13.7; 60 % and 85 % within 1 % of it.
    const int young_pct = tune.young != kUnset ? tune.young : 72;
    if (tune.mb != kUnset && prob_m > 16 && (tune.mb == 2 || tune.mb == 4 || tune.mb == 8)) mb = tune.mb;
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
    // 128-row tiles (eight blocks per wave, accumulators in the accumulation registers, one wave per SIMD): every
    // dequantised fragment feeds 16 MFMAs instead of 8.  One workgroup per CU is resident, so the launch takes whole
    // rounds of 128 rows per CU; 64-row tiles (two workgroups per CU, or one of eight waves) take 1.13-1.32 x as long for
    // the same rows (eight shapes, m = 320 .. 2048) but come in finer grain, and below one
    // workgroup per CU they spread their k slices over the idle CUs.  Hence: 128-row tiles when the 64-row tiles
    // would not fit one per CU and  rounds of 128-row workgroups <= 1.25 x max(1, the same work in rounds).
    // (8192 x 8192: m = 384 74 -> 62 us, m = 512 88 -> 69, m = 768 136 -> 121, m = 1024 177 -> 137; 4096 x 4096 at
    // m = 640 40 -> 36, at m = 512 the rule keeps 64-row tiles: 28 vs 36; 8192 x 5120 at m = 512 69 -> 60, at m = 2048
    // 233 -> 188, at m = 896 it keeps them: 109 vs 117.)
    if (!row_mix && tune.mb == kUnset && mb == 4 && prob_m > 64) {
        const long long rows8 = prob_m < 128LL * max_par ? prob_m : 128LL * max_par;
        const long long tiles_n = prob_n / kTileN;
        const long long wgs8 = tiles_n * ((rows8 + 127) / 128), wgs4 = tiles_n * ((rows8 + 63) / 64);
        const long long rounds8 = (wgs8 + cus - 1) / cus;
        // rounds8 <= 1.25 * max(1, wgs4 / (2 cus))   <=>   4 * rounds8 * 2 cus <= 5 * max(2 cus, wgs4)
        if (wgs4 > cus && 8 * rounds8 * cus <= 5 * (wgs4 > 2LL * cus ? wgs4 : 2LL * cus)) mb = 8;
        // One more case: 64-row workgroups that occupy more than half of the CUs, so that they cannot be split, on a
        // long k.  128-row tiles with a k split that fills at least as many CUs (and three quarters of them) then win
        // although their partial tiles are twice the size (13824 x 5120 at 256 rows: 160 of 256 CUs, 58 -> 49 us;
        // 11008 x 5120 48.1 -> 42.5; on k = 8192 the trade is even, below it loses: 5120 x 5120 27.0 vs 30.4).
        const long long ks8 = wgs8 > 0 ? cus / wgs8 : 0;
        if (mb == 4 && wgs4 <= cus && 2 * wgs4 > cus && prob_k >= 10240 && ks8 >= 2 && 4 * wgs8 * ks8 >= 3 * cus &&
            wgs8 * ks8 >= wgs4 && ks8 <= prob_k / (16LL * 128) &&
            (size_t)(tiles_n + qc / kTileN) * ((rows8 + 127) / 128) * ks8 * (8 * 16 * kTileN * sizeof(float)) <= scratch_bytes)
            mb = 8;
    }
    const int rows_per_tile = 16 * mb;
    const int mtiles_total = (prob_m + rows_per_tile - 1) / rows_per_tile;
    const int units = g128 ? prob_k / 128 : prob_k / 64;

    if (fu.a_cols) {
        const long long launch_rows = prob_m < (long long)rows_per_tile * max_par ? prob_m : (long long)rows_per_tile * max_par;
        if ((size_t)launch_rows * prob_k * sizeof(uint16_t) > kGatherBytes) return FP6M_ERR_ARG;
    }
    for (int mt0 = 0; mt0 < mtiles_total; mt0 += max_par) {
        const int mtiles = mtiles_total - mt0 < max_par ? mtiles_total - mt0 : max_par;
        const int rows0 = mt0 * rows_per_tile;
        a.C = static_cast<uint16_t*>(C) + (size_t)rows0 * prob_n;
        a.residual = fu.residual ? fu.residual + (size_t)rows0 * prob_n : nullptr;
        a.m = prob_m - rows0 < mtiles * rows_per_tile ? prob_m - rows0 : mtiles * rows_per_tile;
        a.A = static_cast<const uint16_t*>(A) + (size_t)rows0 * (fu.a_cols ? fu.lda : prob_k);
        // fp6m_mul_fused's activation gather as a pass of its own: the launch's rows of A, gathered into the region's
        // buffer (stream order keeps the launches apart), become the GEMM's A.  Every kernel but the decode kernel
        // (which gathers by itself) starts with it.
        auto gather_pass = [&]() {
            if (!fu.a_cols) return;
            dim3 ggrid((unsigned)((prob_k / 2 + 255) / 256), (unsigned)a.m);
            hipLaunchKernelGGL(gather_a_kernel, ggrid, dim3(256), 0, st, a.A, fu.lda, fu.a_cols, sc.gathered, prob_k);
            a.A = sc.gathered;
        };

        const size_t tile_bytes = (size_t)mb * 16 * kTileN * sizeof(float);
        const long long traffic_cap = (long long)prob_k / (64LL * a.m) > 0 ? (long long)prob_k / (64LL * a.m) : 1;
        const long long env_ks = tune.ksplit != kUnset ? tune.ksplit : 0;
        if (mb == 1 && !row_mix && (tune.sk != kUnset ? tune.sk != 0 && a.m <= 4 : a.m == 1) && prob_k / 64 < 65536 && (long long)a.tiles * (prob_k / 64) < (1 << 24) &&
                   (long long)prob_k * prob_n / 2 < (1LL << 32) && (long long)(prob_n / 128) * max_par >= 2 &&
                   (g128 || n4 == 0 || units >= 2)) {
            // (k = 64 with per-column scales stays with the workgroup kernel: an INT4 chunk of that single unit is two
            // steps, shorter than the three the fetch side runs ahead, which the drawn-chunk variant cannot follow)
            // One row (decode), weight mixed along n: one wave per workgroup, equal shares of every region's (tile,
            // k unit) list (gemm_sk.h).  The kernel takes up to four rows, but every wave adds its part of a shared
            // tile with one atomic per element, and from two rows on that traffic costs more than the barriers and
            // the partial-tile round trips of the workgroup kernel below (measured: 4096 x 4096 6.5 us at one row,
            // 8.2 at two, 12.8 at four, against 8.2 - 8.3 there).
            SkArgs sk;
            sk.b_int4 = a.b_int4;
            sk.b_fp6_2 = a.b_fp6_2;
            sk.b_fp6_4 = a.b_fp6_4;
            sk.s_int4 = a.s_int4;
            sk.s_fp6 = a.s_fp6;
            sk.C = a.C;
            sk.cells = reinterpret_cast<unsigned long long*>(reinterpret_cast<unsigned char*>(a.scratch) + scratch_bytes);
            sk.m = a.m;
            sk.n = a.n;
            sk.k = a.k;
            sk.n4 = a.n4;
            sk.qc = a.qc;
            sk.tiles6 = a.tiles6;
            sk.flags = (a.native ? 1 : 0) | (a.fused ? 2 : 0);
            sk.c_cols = a.c_cols;
            sk.bias = a.bias;
            sk.residual = a.residual;
            sk.timeline = nullptr;
#ifdef FP6M_TIMELINE
            sk.timeline = a.timeline;
#endif
            const long long tiles4 = a.tiles - a.tiles6;
            const long long u4 = units, u6 = prob_k / 64;              // FP6 tiles have no group scales: 64-row units
            // Chunks and waves (measured on MI355X over 17 shapes).  Shorter chunks are faster as long as every chunk
            // has a wave of its own resident at once (twelve waves per CU fit by registers; eleven are used) and a
            // tile is not cut into more than 32 chunks (more made the adds to one cell queue up; the few FP6 tiles, whose
            // steps take twice as long, may have up to 64 as k grows (24 + a chunk per 512 of k), so that their waves do not finish last: 43 took
            // 11008 x 4096 from 9.9 to 8.8 us and 56 took 28672 x 8192 from 25.2 to 24.7, while 64 chunks of one or two
            // units cost 4096 x 4096 and 8192 x 8192 half a microsecond: short chunks all finish at the same time).  Chunks beyond the
            // waves are drawn from the counters and processed correctly, but every draw and every further chunk's
            // adds are returning atomics that the wave's loads queue behind, so that is the overflow path for
            // problems too large for one chunk per wave, not the plan.  Hence: the shortest chunk that keeps the
            // chunks below eleven per CU and a tile's at 32, moved to a divisor of the tile within 1.5 x if there is
            // one (the largest from six units on, where fewer chunks per tile weighed more).  An FP6 unit (64 rows,
            // 6 KiB) counts like an INT4 unit (8 KiB with group scales, 4 KiB without): fewer bytes, more work per
            // byte.  Further bounds: a chunk has at least as many steps as the fetch side runs ahead (three; an INT4
            // unit without group scales has two); `sms` caps the chunks of a tile (1: whole tiles only), a forced
            // split cuts every tile into that many; and without room for the cells of every tile nothing is shared.
            long long waves_wanted = 11LL * cus;
            if (tune.cap != kUnset && tune.cap > 0) waves_wanted = tune.cap;
            if (tune.wgs != kUnset && tune.wgs > 0) waves_wanted = tune.wgs;
            const long long work4 = tiles4 * u4, work6 = (long long)a.tiles6 * u6;
            long long want4 = (work4 + work6 + waves_wanted - 1) / waves_wanted;
            long long want6 = 1;
            if (tune.wgs != kUnset) want4 = 1;                         // (tests: few waves, many chunks each)
            const bool cells_fit = (size_t)prob_n * a.m * sizeof(unsigned long long) <= kCellBytes;
            auto chunk_units = [&](long long units_r, long long want, long long min_units, long long max_chunks, bool fp6_region) {
                const long long floor_q = (units_r + max_chunks - 1) / max_chunks;
                long long q = want > floor_q ? want : floor_q;
                if (q < units_r) {                                     // a divisor of the tile nearby
                    long long best = 0;
                    for (long long d = q; d < units_r && 2 * d <= 3 * q; d++)
                        if (units_r % d == 0) {
                            best = d;
                            if (q < 6) break;
                        }
                    if (best) q = best;
                }
                if (tune.share != kUnset && tune.share > 0) q = tune.share;
                if (fp6_region && tune.share6 != kUnset && tune.share6 > 0) q = tune.share6;
                if (env_ks >= 1) q = (units_r + env_ks - 1) / env_ks;
                if (sms > 1 && q * sms < units_r) q = (units_r + sms - 1) / sms;
                if (q < min_units) q = min_units;
                if (q * kMaxParts < units_r) q = (units_r + kMaxParts - 1) / kMaxParts;
                while (q < units_r && units_r % q != 0 && units_r % q < min_units) q++;   // (a tile's last chunk too)
                if (sms == 1 || !cells_fit || q > units_r) q = units_r;
                return q;
            };
            const long long max_chunks6 = 24 + u6 / 8 < 64 ? 24 + u6 / 8 : 64;
            long long q4, q6, cpt4, cpt6, chunks4, chunks6;
            for (;; want4++) {                                         // (a last, shorter chunk per tile may push the count over)
                want6 = g128 ? want4 : (want4 + 1) / 2;
                // (40 chunks per tile where so few tiles would otherwise leave SIMDs without a wave: 14336 x 2048, 14
                // INT4 tiles, 28 chunks of 512 rows 8.85 us, 38 of 384 rows 8.2)
                q4 = chunk_units(u4, want4, g128 ? 1 : 2, tiles4 * 40 <= 3LL * cus ? 40 : 32, false);
                q6 = chunk_units(u6, want6, 1, max_chunks6, true);
                cpt4 = (u4 + q4 - 1) / q4;
                cpt6 = (u6 + q6 - 1) / q6;
                chunks4 = tiles4 * cpt4;
                chunks6 = (long long)a.tiles6 * cpt6;
                // An FP6 chunk of half an INT4 chunk's rows takes as long as that one; where the bound on a tile's chunks
                // leaves the FP6 chunks longer, their waves end last (8192 x 3072: 256-row chunks in both regions 7.6 us,
                // 128-row FP6 chunks 7.0; 14336 x 4096 10.6 -> 9.5; 5120 x 5120 7.25 -> 6.85).  Up to 64 chunks per
                // tile then, unless the extra waves start another generation of waves (8192 x 8192: 2048 waves
                // 10.6 us, 2112 11.5).
                if (a.tiles6 && tiles4 && max_chunks6 < 64 && tune.share6 == kUnset) {
                    const long long q6p = chunk_units(u6, want6, 2, 64, true), cpt6p = (u6 + q6p - 1) / q6p;   // (four steps at least)
                    const long long gen = 4LL * cus, with = chunks4 + a.tiles6 * cpt6p;
                    if (q6p < q6 && (with + gen - 1) / gen == (chunks4 + chunks6 + gen - 1) / gen) {
                        q6 = q6p;
                        cpt6 = cpt6p;
                        chunks6 = (long long)a.tiles6 * cpt6;
                    }
                }
                if (chunks4 + chunks6 <= waves_wanted || want4 >= u4 || tune.wgs != kUnset || tune.share != kUnset ||
                    env_ks >= 1 || sms > 0)
                    break;
            }
            // Chunks of 128 rows (four steps, one more than the fetch side runs ahead) are mostly fill and drain: where they
            // would come in more than one generation of waves, 256 rows do better as long as those still give two thirds
            // of the SIMDs a wave (4096 x 6144: 1472 waves of 128 rows 7.1-7.5 us, 736 of 256 rows 6.7; 3072 x 8192
            // 7.1 -> 6.5; 2048 x 12288 6.8 -> 6.4).
            if (tiles4 > 0 && q4 * (g128 ? 128 : 64) == 128 && 2 * q4 <= u4 && chunks4 + chunks6 > 4LL * cus && cells_fit &&
                tune.wgs == kUnset && tune.share == kUnset && env_ks < 1 && sms <= 0 && !(tune.gen != kUnset && tune.gen == 0)) {
                const long long q2 = 2 * q4, cpt2 = (u4 + q2 - 1) / q2;
                if (3 * (tiles4 * cpt2 + chunks6) >= 2 * 4LL * cus && (u4 % q2 == 0 || u4 % q2 >= (g128 ? 1 : 2))) {
                    q4 = q2;
                    cpt4 = cpt2;
                    chunks4 = tiles4 * cpt4;
                }
            }
            // Few tiles and little work (at most a quarter as many INT4 tiles as CUs, 3.5 units per SIMD) in somewhat more
            // chunks than one generation of waves: the waves beyond the first generation start when those end and are
            // the launch's tail.  One generation of longer chunks instead, the FP6 chunks at half the INT4 chunks' rows
            // (best of ten forced lengths against the plan above: 8192 x 5632 1472 waves 9.6 us, 1010 waves 8.4;
            // 8192 x 7680 10.7 vs 9.6; 8192 x 6144 9.8 vs 9.25; with more work per SIMD generations of different
            // lengths win, 14336 x 8192 14.2 vs 15.0, and with more tiles too, 4096 x 12288 by up to 6 %).
            if (tiles4 > 0 && 4 * tiles4 <= cus && 2 * work4 <= 7 * 4LL * cus && chunks4 + chunks6 > 4LL * cus && cells_fit &&
                tune.wgs == kUnset && tune.share == kUnset && tune.share6 == kUnset && env_ks < 1 && sms <= 0 &&
                !(tune.gen != kUnset && tune.gen == 0)) {
                const long long min4 = g128 ? 1 : 2;
                for (long long q = q4; q <= u4; q++) {
                    if (q < u4 && u4 % q != 0 && u4 % q < min4) continue;
                    long long p6 = q * (g128 ? 128 : 64) / 128;                       // FP6 units (64 rows) in half the rows
                    if (p6 < q6) p6 = q6;
                    if (p6 > u6) p6 = u6;
                    while (p6 < u6 && u6 % p6 != 0 && u6 % p6 < 2) p6++;
                    const long long c4 = tiles4 * ((u4 + q - 1) / q), c6 = a.tiles6 ? a.tiles6 * ((u6 + p6 - 1) / p6) : 0;
                    if (c4 + c6 > 4LL * cus) continue;
                    q4 = q;
                    cpt4 = (u4 + q4 - 1) / q4;
                    chunks4 = c4;
                    if (a.tiles6) {
                        q6 = p6;
                        cpt6 = (u6 + q6 - 1) / q6;
                        chunks6 = c6;
                    }
                    break;
                }
            }
            // Waves: one per chunk, up to the number aimed at, which is dealt to the regions by their chunks.
            long long w6 = chunks6, w4 = chunks4;
            if (w4 + w6 > waves_wanted) {
                w6 = a.tiles6 ? (waves_wanted * chunks6 + (chunks4 + chunks6) / 2) / (chunks4 + chunks6) : 0;
                if (a.tiles6 && w6 < 1) w6 = 1;
                w4 = tiles4 ? waves_wanted - w6 : 0;
                if (tiles4 && w4 < 1) w4 = 1;
                if (w4 > chunks4) w4 = chunks4;
                if (w6 > chunks6) w6 = chunks6;
            }
            // Chunk lengths by generation.  The first 4 x CUs waves of a launch get a SIMD each, the next 4 x CUs share one
            // with an older wave, which the SIMD serves first: with equal chunks the generations finish one after the
            // other (per-wave timelines, loop ends in us: 8192 x 57344 27.7 / 37.0, 8192 x 8192 5.5 / 7.1,
            // 4096 x 22016 6.4 / 8.0 / 10.0) and the launch ends on a thinning tail.  So when the plan above needs more
            // than one generation, the INT4 tiles are dealt to the generations in order, each with its own chunk length:
            // a later generation's chunks shorter by about its waves' share of the SIMD (e), so that all end together.
            // Of the first generation's chunk counts per tile, the one with the smallest (chunk length / e) over the
            // generations that the tiles then reach is taken (kernel: sk_generation_order and the sub-lists of SkArgs).
            long long gen_cpt[3] = {cpt4, cpt4, cpt4}, gen_q[3] = {q4, q4, q4}, gen_tiles[3] = {tiles4, 0, 0};
            const long long gen_size = 4LL * cus;
            sk.gen_waves = 0;
            const bool plain_plan = tune.wgs == kUnset && tune.share == kUnset && tune.share6 == kUnset && env_ks < 1 && sms <= 0 &&
                                    cells_fit && w4 == chunks4 && w6 == chunks6;
            if (plain_plan && tiles4 > 0 && chunks4 + chunks6 > gen_size && chunks6 < gen_size && waves_wanted >= 2 * gen_size &&
                !(tune.gen != kUnset && tune.gen == 0)) {
                const double e[3] = {1.0, (tune.gen2 != kUnset ? tune.gen2 : 66) / 100.0, (tune.gen3 != kUnset ? tune.gen3 : 30) / 100.0};
                const long long cap[3] = {gen_size - chunks6, gen_size,
                                          waves_wanted - 2 * gen_size < gen_size ? waves_wanted - 2 * gen_size : gen_size};
                const long long min_units = g128 ? 1 : 2;
                // (chunks per tile: 32 for the first generation as in the plan above, 48 for the later ones, whose chunks
                // must come out a third shorter also on the few tiles of a long k: 17664 x 6656 15.6 -> 13.8 us,
                // 28672 x 5120 18.05 -> 16.5, 21760 x 8192 19.5 -> 19.0; 13824 x 5120 11.0 -> 11.4; 64 measured like 48)
                const long long later_cap = tune.cap2 != kUnset && tune.cap2 > 0 ? tune.cap2 : 48;
                auto fit = [&](long long len, int g) {                 // a length whose last chunk of a tile is not too short
                    const long long most = g == 0 ? 32 : later_cap;
                    if (len < min_units) len = min_units;
                    if (len * most < u4) len = (u4 + most - 1) / most;
                    while (len < u4 && u4 % len != 0 && u4 % len < min_units) len++;
                    return len > u4 ? u4 : len;
                };
                const long long last_gen = (chunks4 + chunks6 - 1) / gen_size;
                double best = (double)q4 / e[last_gen < 2 ? last_gen : 2];          // the plan above, under the same model
                for (long long cpt_a = 1; cpt_a <= 32 && cpt_a <= u4 / min_units; cpt_a++) {
                    long long len[3], cpt[3], t[3], left = tiles4;
                    double cost = 0;
                    for (int g = 0; g < 3; g++) {
                        len[g] = fit(g == 0 ? (u4 + cpt_a - 1) / cpt_a : (long long)((double)len[0] * e[g] + 0.5), g);
                        if (g > 0 && len[g] > len[g - 1]) len[g] = len[g - 1];
                        cpt[g] = (u4 + len[g] - 1) / len[g];
                        t[g] = cap[g] / cpt[g] < left ? cap[g] / cpt[g] : left;
                        left -= t[g];
                        if (t[g] > 0 && (double)len[g] / e[g] > cost) cost = (double)len[g] / e[g];
                    }
                    if (left > 0 || cost >= best) continue;
                    best = cost;
                    for (int g = 0; g < 3; g++) {
                        gen_cpt[g] = cpt[g];
                        gen_q[g] = len[g];
                        gen_tiles[g] = t[g];
                    }
                    sk.gen_waves = (int)gen_size;
                }
                if (sk.gen_waves) {
                    q4 = gen_q[0];
                    cpt4 = gen_cpt[0];
                    chunks4 = gen_tiles[0] * gen_cpt[0] + gen_tiles[1] * gen_cpt[1] + gen_tiles[2] * gen_cpt[2];
                    w4 = chunks4;
                }
            }
            sk.waves = (int)(w4 + w6);
            sk.waves6 = (int)w6;
            sk.units4 = (int)u4;
            sk.units6 = (int)u6;
            sk.q4 = (int)q4;
            sk.cpt4 = (int)cpt4;
            sk.q6 = (int)q6;
            sk.cpt6 = (int)cpt6;
            sk.magic_cpt4 = magic40(cpt4);
            sk.magic_cpt6 = magic40(cpt6);
            sk.tiles4a = (int)gen_tiles[0];
            sk.tiles4b = (int)gen_tiles[1];
            sk.q4b = (int)gen_q[1];
            sk.cpt4b = (int)gen_cpt[1];
            sk.q4c = (int)gen_q[2];
            sk.cpt4c = (int)gen_cpt[2];
            auto magic32 = [](long long d) { return d >= 2 ? (uint32_t)((0x100000000ULL + (unsigned long long)d - 1) / (unsigned long long)d) : 0u; };
            sk.magic32_cpt4b = magic32(gen_cpt[1]);
            sk.magic32_cpt4c = magic32(gen_cpt[2]);
            sk.pad[0] = sk.pad[1] = sk.pad[2] = sk.pad[3] = 0;
            sk.total4 = chunks4 > w4 ? (int)chunks4 : 0;               // 0: one chunk per wave, no counter traffic
            sk.total6 = chunks6 > w6 ? (int)chunks6 : 0;
            // The activation gather: by the kernel itself for one row and one chunk per wave (two dependent loads per
            // step pair and lane, hidden behind the weights' own latency), else by the pass.  From two rows on the
            // kernel's extra loads (one per row, lane and pair) cost what the pass costs.
            const bool gather_inside = fu.a_cols && a.m == 1 && !sk.total4 && !sk.total6 && (tune.gather == kUnset || tune.gather != 0);
            if (!gather_inside) gather_pass();
            sk.A = a.A;
            sk.a_cols = gather_inside ? fu.a_cols : nullptr;
            sk.lda = gather_inside ? fu.lda : 0;
            sk.counters = a.counters;
            // Counters: atomics on one address complete one after the other, about 0.3 us apart, and a wave's loads
            // queue behind its own draw, so no more than four waves share a counter (with 64 counters for 2560 waves
            // the first data arrived up to 15 us late).  They come out of the workspace the caller must provide
            // (prob_n / 128 * max_par elements): a quarter of it at most for the FP6 region.
            const long long ws_elems = (long long)(prob_n / 128) * max_par;
            long long groups6 = a.tiles6 ? (w6 + 3) / 4 : 0;
            if (groups6 > ws_elems / 4) groups6 = ws_elems / 4 > 0 ? ws_elems / 4 : 1;
            long long groups4 = tiles4 ? (w4 + 3) / 4 : 0;
            if (groups4 > ws_elems - groups6) groups4 = ws_elems - groups6;
            if (groups4 > 65535) groups4 = 65535;
            sk.groups = (int)(groups4 | (groups6 << 16));
            if (tune.verbose)
                fprintf(stderr, "fp6m_mul m=%d n=%d k=%d: one-wave workgroups %lld (FP6) + %lld (INT4), chunks %lld of %lld units + "
                        "%lld of %lld units%s", a.m, prob_n, prob_k, w6, w4, chunks6, q6, chunks4, q4, sk.gen_waves ? "" : "\n");
            if (tune.verbose && sk.gen_waves)
                fprintf(stderr, " (by generation: %lld tiles x %lld chunks of %lld, %lld x %lld of %lld, %lld x %lld of %lld)\n",
                        gen_tiles[0], gen_cpt[0], gen_q[0], gen_tiles[1], gen_cpt[1], gen_q[1], gen_tiles[2], gen_cpt[2], gen_q[2]);
            dim3 grid((unsigned)sk.waves, 1);
            // variants: group scales or not; one chunk per wave with or without the gather, or chunks drawn from counters
            void (*kernel)(const SkArgs) = nullptr;
            const bool draw = sk.total4 || sk.total6;
            const bool lean = sk.flags == 0 && sk.m == 1;             // (one row, no fused epilogue, reference-order words)
            if (gather_inside)
                kernel = g128 ? gemm_sk_kernel<true, 1, false> : gemm_sk_kernel<false, 1, false>;
            else if (draw && lean)
                kernel = g128 ? gemm_sk_kernel<true, 0, true, false> : gemm_sk_kernel<false, 0, true, false>;
            else if (draw)
                kernel = g128 ? gemm_sk_kernel<true, 0, true> : gemm_sk_kernel<false, 0, true>;
            else if (lean)
                kernel = g128 ? gemm_sk_kernel<true, 0, false, false> : gemm_sk_kernel<false, 0, false, false>;
            else
                kernel = g128 ? gemm_sk_kernel<true, 0, false> : gemm_sk_kernel<false, 0, false>;
            hipLaunchKernelGGL(kernel, grid, dim3(64), 0, st, sk);
        } else if (mb == 1) {
            gather_pass();
            // m <= 16 (the row mix, and 5 to 16 rows of the column mix).  Each region (FP6, INT4) has its own number of k parts (workgroups) per tile group;
            // FP6 steps cost about twice an INT4 step, so the FP6 region is split twice as finely.  The
            // split is bounded so that every wave keeps at least one k unit, partial-sum traffic stays
            // well below the weight stream and the partial tiles fit the scratch.
            M16Config cfg = m16_config(a.m);
            a.groups6 = (a.tiles6 + cfg.wn - 1) / cfg.wn;
            a.groups4 = (a.tiles - a.tiles6 + cfg.wn - 1) / cfg.wn;
            const long long groups = a.groups6 + a.groups4;
            const int unit_steps = g128 ? 4 : 2;
            // Bounds of the split for a workgroup of wk waves: at least one k unit and four k steps per wave, and the
            // partial-sum traffic well below the weight stream.
            auto ks_units = [&](int wk) { return units / wk > 0 ? (long long)(units / wk) : 1LL; };
            auto ks_limit = [&](int wk) {
                long long c = prob_k / 32 / (4 * wk) > 0 ? prob_k / 32 / (4 * wk) : 1;
                if (c > ks_units(wk)) c = ks_units(wk);
                // (a grid that leaves CUs idle even so may split twice as far: 2048 x 2048 .. 6144 at 16 rows 7.6-7.8 -> 6.9-7.3 us)
                const long long cap = groups * 2 * traffic_cap <= cus ? 2 * traffic_cap : traffic_cap;
                if (c > cap) c = cap;
                return c;
            };
            // FP6 tiles are split twice as finely as INT4 tiles (their steps move 1.5x the bytes); with FP6 tiles only
            // there is nothing to keep step with and the split is the one asked for
            auto ks6_of = [&](long long c, int wk) {
                if (a.groups4 == 0) return c < ks_units(wk) ? c : ks_units(wk);
                return 2 * c <= ks_units(wk) ? 2 * c : (c > ks_units(wk) ? c : ks_units(wk));
            };
            // Measured on MI355X: with four waves per workgroup the kernel is fastest with about one and a half
            // workgroups per CU (more concurrent k fronts cost DRAM efficiency, fewer leave CUs idle).
            const long long target_wgs = (long long)cus * 3 / 2;
            long long ks = (target_wgs + groups / 2) / groups;
            double cls_gain = 0.0;
            long long cls_na = 0, cls_cb = 0;                           // two classes of INT4 tiles (below): tiles of the first, parts of the second
            if (ks > ks_limit(cfg.wk)) ks = ks_limit(cfg.wk);
            if (ks < 1) ks = 1;
            // Second opinion from a small cost model (per-workgroup timelines on MI355X): a wave takes about 0.40 us per
            // k step when its four-wave workgroup has the CU to itself, 0.56 us when the CU hosts eight waves (two such
            // workgroups, or one of eight waves), 0.72 us when every CU does, 1.1 us beyond; the kernel lasts as long as
            // the longest slice on the busiest CU, plus 2.5 us and 0.15 us per partner when tiles are split across
            // workgroups, plus the partial sums' traffic.  Grids of exactly one or two workgroups per CU with equal slices, and eight-wave workgroups
            // that need no split at all, beat the rule by 4-15 % where the shape allows them; the rule's choice is kept
            // unless the model sees 8 % or more.
            {
                auto model_us = [&](int wk, long long c) -> double {
                    const long long c6 = a.groups6 ? ks6_of(c, wk) : 0;
                    const double load = (double)(a.groups4 * c + a.groups6 * c6) / cus;
                    double t;
                    if (wk == 4) {
                        if (load > (cfg.id == 1 ? 2.0 : 3.0)) return 1e9;   // what a CU's LDS holds at once (16 rows of A: two)
                        t = load <= 1.0 ? 0.40 : (load <= 1.9 ? 0.56 : (load <= 2.0 ? 0.72 : 1.10));
                    } else {
                        // eight waves per workgroup paid off only with one workgroup on (nearly) every CU: measured
                        // slower both when CUs hosted two of them and when a quarter or more of the CUs stayed idle
                        // (without a k split of the INT4 tiles there is no tail to lose, so fewer busy CUs still pay)
                        if (load > 1.0 || load < (c == 1 ? 0.5 : 0.65)) return 1e9;
                        // (and their waves keep five k steps: 2048 x 11264 with per-column scales, 2 parts of four steps
                        // per wave 8.8 us, four waves x 2 parts 8.0; 4096 x 8192 at 8 rows 4 parts 10.0, 3 parts 9.5)
                        if (c > 1 && prob_k < 160 * 8 * c) return 1e9;
                        t = 0.56;
                    }
                    auto longest = [&](long long slices) { return (double)((units + slices - 1) / slices) * unit_steps; };
                    auto tail = [](long long partners) { return partners > 1 ? 2.5 + 0.15 * partners : 0.0; };
                    const double int4_us = a.groups4 ? longest(c * wk) * t + tail(c) : 0.0;
                    const double fp6_us = a.groups6 ? 1.5 * longest(c6 * wk) * t + tail(c6) : 0.0;   // an FP6 step moves 1.5x the bytes
                    // every workgroup of a split tile writes its m x 128 partial sums and the last arrival reads them
                    // back, at about 2 TB/s all told (5120 x 13824 at 16 rows: 440 workgroups 15.4 us, 220 13.6)
                    const double partial_us = (c > 1 ? a.groups4 * c : 0) * a.m * 0.0005 + (c6 > 1 ? a.groups6 * c6 : 0) * a.m * 0.0005;
                    return (int4_us > fp6_us ? int4_us : fp6_us) + partial_us;
                };
                int best_wk = cfg.wk;
                long long best = ks;
                for (int wk = 4; wk <= 8; wk += 4)
                    for (long long c = 1; c <= ks_limit(wk); c++)
                        if (model_us(wk, c) < model_us(best_wk, best)) {
                            best_wk = wk;
                            best = c;
                        }
                if (model_us(best_wk, best) < 0.92 * model_us(cfg.wk, ks)) {
                    cfg.wk = best_wk;
                    ks = best;
                }
                // Few tiles on a long k (eight or more parts per tile): eight-wave workgroups cover the same slices
                // with half the partners, or halve the slices, and beyond eight partners the last arrival's gather costs
                // more than shorter slices gain (0.16-0.27 us per partner).  8192 x 2048 at 8 rows, us by parts: four waves
                // 8: 10.1, 12: 9.9, 16: 10.9; eight waves 6: 9.45, 8: 9.43, 12: 10.0; at 16 rows four waves x 8 parts 10.8,
                // eight x 8 9.8; 14336 x 2048 at 16 rows 12.1 (14 parts) -> 11.2; 8192 x 3072 10.8 -> 10.0.
                bool few_tiles = false;
                if (!row_mix && ks >= 8 && tune.wk16 == kUnset && env_ks < 1 && sms <= 0) {
                    const long long fill = cus * 3 / 4 / groups;                       // (8192 x 4096: 6 parts 10.0, 8 parts 10.5)
                    long long c = fill < 8 ? fill : 8;
                    if (c > ks_limit(8)) c = ks_limit(8);
                    // (eight parts of four waves against fewer of eight: even at 16 rows, 13 % slower at 2 and 4 rows,
                    // where partners meet in cells: 4096 x 2560 6.7 vs 7.6 us)
                    if (c >= 4 && (ks > 8 || c == 8 || a.m > 4)) {
                        cfg.wk = 8;
                        ks = c;
                        few_tiles = true;
                    }
                }
                // Eight-wave workgroups that fit one per CU and leave at most a third of the CUs idle: the finest such split
                // that leaves every wave five k steps (3072 x 9216 at 16 rows: eight waves x 3 parts, four steps per wave,
                // 9.7 us; four waves x 3 parts 8.9).  (Forced tables of 4- and 8-wave workgroups x 1 .. 16 parts: 11008 x 5120 at 8 rows
                // four waves at best 13.2 us (5 parts), eight waves 11.9 (5 parts: 210 workgroups), and 16.5 from 7
                // parts on, where they no longer fit; 11008 x 8192 at 5 rows 15.6 -> 13.9; 8192 x 5120 at 16 rows
                // 11.3 -> 10.8, 5120 x 6144 11.5 -> 10.1.)
                // On a short k (below 6144) four-wave workgroups that fill nine CUs in ten do better still: their waves
                // keep twice the steps (5120 x 15360 at 16 rows, 2 parts: four waves 12.4 us, eight 13.0; 4096 x 15360
                // 11.3 vs 12.2; 2048 x 15360 with per-column scales 9.4 -> 8.3; with fewer CUs busy the eight-wave
                // ones win, 5120 x 11264 at 6 rows 11.2 vs 12.4, and from k = 6656 on they do anyway).
                if (!row_mix && !few_tiles && ks >= 2 && tune.wk16 == kUnset && env_ks < 1 && sms <= 0) {
                    auto fit = [&](int wk, long long& c) {
                        auto wgs_fit = [&](long long cc) { return a.groups4 * cc + a.groups6 * (a.groups6 ? ks6_of(cc, wk) : 0); };
                        c = ks_limit(wk);
                        // (five k steps per wave at least; a CU per XCD stays free: a grid of exactly as many workgroups as
                        // CUs ran 5-11 % slower than the next coarser split, 2048 x 8192 at 4 rows 8.3 vs 7.4 us)
                        while (c >= 2 && (wgs_fit(c) > cus - cus / 32 || prob_k < 160 * wk * c)) c--;
                        return c >= 2 ? wgs_fit(c) : 0LL;
                    };
                    long long c4 = 0, c8 = 0;
                    const long long w4 = prob_k < 6144 ? fit(4, c4) : 0, w8 = fit(8, c8);
                    if (10 * w4 >= 9 * cus) {
                        cfg.wk = 4;
                        ks = c4;
                    } else if (100 * w8 >= 68 * cus) {
                        cfg.wk = 8;
                        ks = c8;
                    } else if (prob_k < 4096 && cfg.wk == 4 && 100 * w4 >= 68 * cus) {
                        // (a short k with some CUs hosting two workgroups and some one: 2048 x 11264 at 6 rows, per-column
                        // scales, 4 parts = 360 workgroups 9.0 us, 2 parts = 180 7.7)
                        const long long now = a.groups4 * ks + a.groups6 * (a.groups6 ? ks6_of(ks, 4) : 0);
                        if (now > cus && now < 2LL * cus) ks = c4;           // (2048 x 13312, 424 workgroups: 9.4 us; 212: 7.85)
                    }
                }
                // A grid of exactly (or all but) as many workgroups as CUs is slower than the next coarser split (2048 x 8192
                // at 4 rows: 4 parts = 256 workgroups 8.3 us, 3 parts 7.4; 4096 x 4096: 8 parts 8.3, 6 parts 7.4): one CU
                // per XCD stays free.
                if (!row_mix && tune.wk16 == kUnset && env_ks < 1 && sms <= 0) {
                    auto wgs_of = [&](long long cc) { return a.groups4 * cc + a.groups6 * (a.groups6 ? ks6_of(cc, cfg.wk) : 0); };
                    while (ks >= 2 && wgs_of(ks) <= cus && wgs_of(ks) > cus - cus / 32) ks--;
                }
                // Two classes of INT4 tiles.  A few more tiles than CUs leave the grid above lopsided whatever the split
                // (6656 x 35328: 274 INT4 tiles, so 22 CUs run two workgroups and end at 29 us where the others end at
                // 19: while two four-wave workgroups share a CU the first runs at 0.73 and the second at 0.52 of the
                // rate one has alone, so the doubled-up CUs take 1.76 x as long).  So: as many whole tiles as fill every
                // CU once make the first cus workgroups of the grid (with the FP6 region's); the tiles left over are cut
                // into cb parts and dealt, as the later workgroups of the grid, over the CUs a second time: 1 + 1 / cb
                // rounds and a second start instead of 1.76.  Taken where  k / 128 * (0.76 - 1 / cb) >= 7.5:  forced both
                // ways over 56 shapes (k = 2048 .. 14336, 312 .. 424 tiles, 8 and 16 rows) that is where it won (k = 2048
                // in four parts -7 .. -12 %, k >= 4096 in two or more -5 .. -19 %) and the rest was within -1 .. +4 %.
                // With the first class split as well (fewer tiles than CUs) every forced plan lost 5-30 %: not tried.
                if (!row_mix && cfg.wn == 1 && sms <= 0 && env_ks < 1 && tune.wk16 == kUnset && a.groups4 > 0 &&
                    !(tune.cls != kUnset && tune.cls == 0)) {
                    const long long c6 = a.groups6 ? ks6_of(1, 4) : 0;
                    const long long first = cus - a.groups6 * c6;                      // workgroups the first round has left
                    const long long na = a.groups4 < first ? a.groups4 : first, nb = a.groups4 - na;
                    if (first >= 1 && nb > 0 && nb <= cus) {                           // (else: one class does it / a third round)
                        // (the few tiles of the second class may be cut finer than a split of all tiles may: their partial
                        // tiles are a small part of the traffic)
                        long long cb = cus / nb;
                        const long long cb_limit = prob_k / 32 / 16 < ks_units(4) ? prob_k / 32 / 16 : ks_units(4);
                        if (cb > cb_limit) cb = cb_limit;
                        if (cb < 1) cb = 1;
                        cls_gain = prob_k / 128.0 * (0.76 - 1.0 / (double)cb);
                        if (tune.cls == 1 || (cb >= 2 && cls_gain >= 7.5)) {
                            cls_na = na;
                            cls_cb = cb;
                        }
                    }
                }
            }
            if (tune.wk16 != kUnset) cfg.wk = tune.wk16 == 8 ? 8 : 4;
            const long long ks_k = ks_units(cfg.wk);
            if (ks > ks_k) ks = ks_k;
            if (sms > 0 && ks > sms) ks = sms;
            if (env_ks >= 1) ks = env_ks;
            if (ks < 1) ks = 1;
            const size_t slot_bytes = (size_t)cfg.wn * 16 * kTileN * sizeof(float);
            if (fixed_scratch && ks > 1 && (size_t)(a.groups4 + 2 * a.groups6) * ks * slot_bytes > scratch_bytes) return FP6M_ERR_SCRATCH;
            while (ks > 1 && (size_t)(a.groups4 + 2 * a.groups6) * ks * slot_bytes > scratch_bytes) ks--;
            a.ks4 = (int)ks;
            a.ks6 = (int)ks6_of(ks, cfg.wk);
            if (sms > 0 && a.ks6 > sms) a.ks6 = sms;
            if (cls_na > 0) {
                const long long c6 = a.groups6 ? ks6_of(1, 4) : 0, nb = a.groups4 - cls_na;
                const size_t slots = (size_t)(a.groups6 * c6 + cls_na + nb * cls_cb);
                if (slots * slot_bytes <= scratch_bytes && cls_cb <= kMaxParts && c6 <= kMaxParts) {
                    cfg.wk = 4;
                    a.ks4 = 1;
                    a.ks6 = (int)c6;
                    a.groups4b = (int)nb;
                    a.ks4b = (int)cls_cb;
                    a.groups4 = (int)cls_na;
                }
            }
            a.ksplit = a.ks4;
            // Up to four rows, shared tiles meet in cells (one returning atomic per element and workgroup) instead of
            // being published, counted and gathered: one round trip after the loop instead of three (4096 x 4096 at two
            // rows 8.1 -> 7.0 us, 11008 x 4096 11.1 -> 10.1, 8192 x 8192 12.2 -> 11.6; even at four rows; the atomics of
            // eight and sixteen rows cost more than the round trips: 4096 x 4096 at sixteen rows 9.3 -> 10.3 us).
            const bool want_cells = a.m <= 4 && !(tune.cells != kUnset && tune.cells == 0);
            if (want_cells && (size_t)prob_n * 16 * sizeof(unsigned long long) <= kCellBytes && a.ks4 <= kMaxParts &&
                a.ks6 <= kMaxParts)
                a.cells = reinterpret_cast<unsigned long long*>(reinterpret_cast<unsigned char*>(a.scratch) + scratch_bytes);
            if (row_mix) {
                a.ks6 = 0;                                            // no FP6 column region: groups6 is 0
                a.slices4 = deal_slices(a.ks4 * cfg.wk);
                a.rule[0] = make_rule(k4 / 128, a.slices4);
                a.rule[1] = make_rule(fu.quant_rows / 64, a.ks4 * cfg.wk - a.slices4);
            } else {
                a.rule[0] = make_rule(units, a.ks4 * cfg.wk);
                a.rule[1] = make_rule(units, (a.ks6 > 0 ? a.ks6 : 1) * cfg.wk);
                a.wrule[0] = make_wave_rule(units, a.ks4, cfg.wk, young_pct);
                a.wrule[1] = make_wave_rule(units, a.ks6 > 0 ? a.ks6 : 1, cfg.wk, young_pct);
                a.wrule_b = make_wave_rule(units, a.ks4b, cfg.wk, young_pct);
            }
            long long wgs = (long long)a.groups6 * a.ks6 + (long long)a.groups4 * a.ks4 + (long long)a.groups4b * a.ks4b;
            a.div[0] = make_div(a.groups4, wgs);
            a.div[1] = make_div(a.groups6, wgs);
            a.div_b = make_div(a.groups4b > 0 ? a.groups4b : 1, wgs);
            // Tiles shared by several workgroups, more than four rows: the workgroups of a tile may be placed on one XCD
            // (xcd_place in gemm_common.h) and exchange their partial tiles through its L2 instead of through memory:
            // the publishing stores are acknowledged 0.2-0.3 us earlier and the gather is 0.1-0.2 us shorter.  The grid
            // is eight times the largest number of workgroups any XCD gets, so a few workgroups have nothing to do,
            // and the tiles are dealt to the XCDs whole, which leaves the XCDs with an FP6 tile more to do than the others.
            // Measured (alternating, us): four-wave workgroups gain 2-4 % (4096 x 4096 at 16 rows 8.54 -> 8.35, at 5
            // rows 8.42 -> 8.11, 11008 x 4096 11.65 -> 11.41, 28672 x 8192 28.25 -> 27.45); eight-wave workgroups,
            // one per CU, gain nothing where the XCDs' shares stay below their 32 CUs (8192 x 8192 13.1 both) and
            // lose a whole round where they do not (8192 x 10240 14.1 -> 19.4), so those keep the agent-scope exchange.
            a.xcd_local = 0;
            bool want_local = cfg.wk == 4 && a.ks4 > 1;
            if (tune.xcd != kUnset) want_local = tune.xcd != 0;
            if (a.groups4b > 0) want_local = false;
            if (want_local && cfg.id == 1 && cfg.wn == 1 && !a.cells && xcd_placement == 1 && (a.ks4 > 1 || a.ks6 > 1) &&
                a.ks4 <= kMaxLocalParts && a.ks6 <= kMaxLocalParts) {
                long long most = 0;
                for (int x = 0; x < 8; x++) {
                    const long long c6 = (a.groups6 + 7 - x) >> 3, g0 = (x - a.groups6) & 7, c4 = (a.groups4 + 7 - g0) >> 3;
                    const long long w = c6 * a.ks6 + c4 * a.ks4;
                    most = w > most ? w : most;
                }
                // (no XCD may get more workgroups than its CUs hold at once: two of four waves each; and a grid that fits
                // one workgroup per CU must still do so on every XCD: 3072 x 4608 at 6 rows in 6 parts, 228 workgroups,
                // up to 42 on an XCD: 9.1 us against 7.8 in 4 parts)
                if (most < 8192 && (tune.xcd != kUnset || (8 * most <= 2LL * cus && (wgs > cus || 8 * most <= cus)))) {
                    a.xcd_local = 1;
                    wgs = 8 * most;
                    auto magic32 = [](int d) { return d >= 2 ? (uint32_t)((0x100000000ULL + d - 1) / (unsigned long long)d) : 0u; };
                    a.xm4_lo = magic32(a.groups4 >> 3);
                    a.xm4_hi = magic32((a.groups4 >> 3) + 1);
                    a.xm6_lo = magic32(a.groups6 >> 3);
                    a.xm6_hi = magic32((a.groups6 >> 3) + 1);
                }
            }
            dim3 grid((unsigned)wgs, 1);
            if (tune.verbose)
                fprintf(stderr, "fp6m_mul m=%d n=%d k=%d: cfg %d (%dx%d waves) groups %d+%d ks4=%d ks6=%d (+ %d tiles in %d parts) gain %.1f grid=%u%s\n", a.m, prob_n,
                        prob_k, cfg.id, cfg.wn, cfg.wk, a.groups6, a.groups4, a.ks4, a.ks6, a.groups4b, a.ks4b, cls_gain, grid.x, a.xcd_local ? " (tiles placed per XCD)" : "");
            launch_m16_any(cfg, a, g128, grid, st);
        } else {
            gather_pass();
            // m > 16: a task is one workgroup (one tile x four k slices) on one row tile and k part.
            // Split k only as far as needed to give every CU a workgroup; partial tiles are 16*MB rows
            // of fp32, so the split is also capped by their traffic relative to the weight stream.
            const long long base = (long long)a.tiles * mtiles;
            long long ks = cus / base;
            // (two k units per wave at least, one on a short k up to four parts; a grid that leaves half of the CUs idle even
            // so may split twice as far as the partial tiles' traffic would otherwise allow: 2048 x 2560 .. 7680 at 32 and
            // 64 rows 10.4 -> 9.2-9.8 us and 13.8 -> 12.7-13.0; eight parts instead of four on k = 4096 cost 6-12 %)
            long long ks_k = units / (kWaves * 2);
            if (ks_k < 4) ks_k = units / kWaves < 4 ? units / kWaves : 4;
            if (ks_k < 1) ks_k = 1;
            long long cap = (long long)prob_k / (16LL * rows_per_tile) > 0 ? (long long)prob_k / (16LL * rows_per_tile) : 1;
            if (base * 2 * cap <= cus) cap *= 2;
            if (ks > ks_k) ks = ks_k;
            if (ks > cap) ks = cap;
            if (sms > 0 && ks > sms) ks = sms;
            if (env_ks >= 1) ks = env_ks;
            if (ks < 1) ks = 1;
            if (fixed_scratch && ks > 1 && (size_t)(a.tiles + a.tiles6) * mtiles * ks * tile_bytes > scratch_bytes) return FP6M_ERR_SCRATCH;
            while (ks > 1 && (size_t)(a.tiles + a.tiles6) * mtiles * ks * tile_bytes > scratch_bytes) ks--;   // (FP6 tiles: 2 ks)
            a.ksplit = (int)ks;
            // A grid of at most one workgroup per CU would leave every SIMD a single wave: give the workgroup eight
            // k slices instead of four (same partial-sum traffic, two waves per SIMD) when k is long enough.
            // (Two waves on a SIMD take turns at its one VALU/MFMA port: eight half-length slices last as long as four
            // whole ones, so eight (which hide latency better: 13824 x 5120 at 256 rows 60.6 vs 67.8 us) only pay while
            // their longest slice, in whole k units, is no more than 0.58 of the longest of four: 5120 x 13824 at 64
            // rows, 40 units over 16 slices of up to 3: 24.1 us, over 8 slices of 5: 21.7.)
            // From forced tables (4 or 8 slices x 1 .. 8 parts, 32 / 64 / 128 rows): a split is no finer than its longest
            // slice needs (8192 x 6144 at 32 rows: 64 units in 5 parts = 20 slices of up to 4, 16.7 us; in 4 parts = 16
            // slices of 4, 16.0; as eight-wave workgroups 14.3); one unit per wave is enough for eight (8192 x 2048 at
            // 32 rows 12.8 -> 12.0); 0.58 rather than 0.55 (14336 x 8192 at 32 rows, 4 against 7 units, 23.0 -> 20.5);
            // and beyond eight parts the partners' partial tiles cost more than shorter slices gain (14336 x 2048 at
            // 32 rows: 14 parts of four slices 16.7 us, 8 parts of eight 14.8; at 64 rows 24.0 -> 21.0).
            auto longest = [&](long long slices) { return (units + slices - 1) / slices; };
            const bool free_split = env_ks < 1 && sms <= 0 && !row_mix && mb != 8;
            if (free_split)
                while (ks > 1 && longest(4 * (ks - 1)) == longest(4 * ks)) ks--;
            // (32-row tiles are not issue-bound: two waves per SIMD pay up to two thirds, 11008 x 2560 at 32 rows 14.9 -> 13.2)
            const bool eight_pays = mb == 2 ? 3 * longest(8 * ks) <= 2 * longest(4 * ks) : 50 * longest(8 * ks) <= 29 * longest(4 * ks);
            int wk = base * ks <= cus && units / 8 >= ks && eight_pays ? 8 : kWaves;
            if (free_split && tune.wk == kUnset && ks > 8 && base * 8 <= cus && units / 8 >= 8) {
                wk = 8;
                ks = 8;
            }
            if (tune.wk != kUnset) wk = tune.wk == 8 ? 8 : kWaves;
            if (mb == 8) wk = kWaves;                                  // (512 registers per wave: one wave per SIMD)
            a.ksplit = (int)ks;
            // An FP6 step costs more issue slots than an INT4 one, and in a grid that is resident all at once the few
            // FP6 tiles' workgroups set the length of the launch (8192 x 8192 at m = 128: 33 us against 29 us with INT4
            // only).  Their k range is cut twice as finely where every slice still gets two units and the grid still
            // fits the CUs in one go (5120 x 13824 at m = 128: 40 -> 31 us; a grid whose last workgroups must wait for
            // a free CU loses far more than that).  A forced split applies to both kinds.
            a.ks4 = (int)ks;
            a.ks6 = (int)ks;
            // (a grid that fits one workgroup per CU must still do so afterwards: a CU with two runs both at little
            // more than half speed, 11008 x 4096 at 256 rows 34 -> 52 us with 272 workgroups)
            const long long resident = (long long)cus * (wk == 8 || mb == 8 || base * ks <= cus ? 1 : 2);
            // (Not for 128-row tiles, whose FP6 workgroups are only a few per cent behind: there the second partner's
            // partial tiles cost more than the shorter loop gains, 8192 x 8192 at m = 384 61.8 vs 58.4 us.)
            // Re-measured with every tile on the paired loop (ten shapes x 32 .. 256 rows, alternating): still 5-13 % on
            // wide weights up to two row tiles (4096 x 11008 at 128 rows 25.3 -> 22.2 us, 8192 x 28672 at 32 rows
            // 38.2 -> 34.5), but 3-8 % slower from three row tiles on (5120 x 5120 at 256 rows 27.4 -> 29.7): up to two.
            if (env_ks < 1 && !row_mix && a.tiles6 > 0 && units >= 4 * ks * wk && mb != 8 && mtiles <= 2 &&
                (base + (long long)a.tiles6 * mtiles) * ks <= resident)
                a.ks6 = 2 * (int)ks;
            // One row tile and somewhat more tiles than CUs: workgroups of four waves, two to a CU, run both at little more
            // than half speed, so the CUs that get two set the launch's length at 1.76 x that of a grid that fits
            // (8192 x 36864 at 32 rows: 288 tiles 60.9 us, 256 tiles 34.6).  Two classes of INT4 tiles instead (as in the
            // m <= 16 kernel): as many whole tiles as there are CUs, one workgroup per CU with two waves per SIMD, and the
            // tiles left over in cb >= 2 parts on workgroups that start as those end: 1 + 1 / cb rounds instead of 1.76.
            a.groups4b = 0;
            a.ks4b = 1;
            const long long tiles4 = a.tiles - a.tiles6;
            if (!row_mix && !needs_extras(a) && tune.pair == kUnset && mb <= 4 && !(mb == 4 && !g128) && mtiles == 1 && mtiles_total == 1 && sms <= 0 && env_ks < 1 && tune.wk == kUnset && ks == 1 && base > cus &&
                tiles4 > 0 && !(tune.cls != kUnset && tune.cls == 0)) {
                const int wk_c = 8;
                const long long c6 = a.tiles6 && units >= 4 * wk_c ? 2 : 1;
                const long long first = cus - a.tiles6 * c6;
                const long long na = tiles4 < first ? tiles4 : first, nb = tiles4 - na;
                if (first >= 1 && nb > 0 && nb <= cus) {
                    long long cb = cus / nb;
                    const long long cb_k = prob_k / 1024 > 0 ? prob_k / 1024 : 1;               // 128 rows of k per wave at least
                    if (cb > cb_k) cb = cb_k;
                    if (cb > cap) cb = cap;
                    // (partial-tile slots are numbered over all tiles, the whole ones of the first class included)
                    while (cb > 1 && (size_t)(a.tiles6 * c6 + na + nb * cb) * tile_bytes > scratch_bytes) cb--;
                    // Taken by the m <= 16 kernel's measure (rounds saved x 128-row units of k), with a bar that follows the
                    // rows of 32-row tiles: a ragged tile gains less (the one-class grid's four-wave workgroups get
                    // faster with fewer rows, the eight-wave ones of this plan hardly); 64-row tiles need twice the
                    // bar.  Fitted to runs against the one-class grid over 236 shapes (17 .. 64 rows x k = 2048 .. 8192 x
                    // 264 .. 360 tiles, both scale modes): what these bars take gained 0-33 %, what they leave out
                    // was within -4 .. +8 % when forced.
                    const double gain = prob_k / 128.0 * (0.76 - 1.0 / (double)cb);
                    const double bar = mb == 4 ? 16.0 : 7.5 + 0.37 * (32 - a.m);
                    if ((cb >= 2 && gain >= bar) || (tune.cls == 1 && cb >= 1)) {
                        wk = wk_c;
                        a.ks4 = 1;
                        a.ks6 = (int)c6;
                        a.groups4b = (int)nb;
                        a.ks4b = (int)cb;
                    }
                }
            }
            if (row_mix) {
                a.slices4 = deal_slices(a.ksplit * wk);
                a.rule[0] = make_rule(k4 / 128, a.slices4);
                a.rule[1] = make_rule(fu.quant_rows / 64, a.ksplit * wk - a.slices4);
            } else {
                a.rule[0] = make_rule(units, a.ks4 * wk);
                a.rule[1] = make_rule(units, a.ks6 * wk);
                a.wrule[0] = make_wave_rule(units, a.ks4, wk, young_pct);
                a.wrule[1] = make_wave_rule(units, a.ks6, wk, young_pct);
                a.wrule_b = make_wave_rule(units, a.ks4b, wk, young_pct);
            }
            const long long wgs = (long long)a.tiles6 * a.ks6 + (tiles4 - a.groups4b) * a.ks4 + (long long)a.groups4b * a.ks4b;
            a.div[0] = make_div(a.ks4, wgs);
            a.div[1] = make_div(a.ks6, wgs);
            a.div_b = make_div(a.ks4b, wgs);
            dim3 grid((unsigned)wgs, (unsigned)mtiles);
            if (tune.verbose)
                fprintf(stderr, "fp6m_mul m=%d n=%d k=%d: MB=%d row tiles %d ks4=%d ks6=%d (+ %d tiles in %d parts) k slices %d grid=%ux%u\n",
                        a.m, prob_n, prob_k, mb, mtiles, a.ks4, a.ks6, a.groups4b, a.ks4b, wk, grid.x, grid.y);
            // Every launch of 64-row tiles takes the paired loop (33 rows: -5 % .. +5 % over five shapes, 40 rows 0-9 % faster,
            // 64 rows 9-16 %, from 65 rows on 12-20 %; before the FP6 tiles had it too, whose workgroups set a resident
            // grid's length, it paid from 65 rows on only).  The ring loop stays for the tuning hook and for 32-row tiles in
            // four-wave workgroups (below).
            bool pair = true;
            if (tune.pair != kUnset) pair = mb >= 4 && tune.pair != 0;
            if (mb == 8) {
                // (always the paired loop: the ring loop's 30 KiB per wave would fit, but it was slower at every size)
                if (g128)
                    launch_mb_one<true, 8, 3, 3, 4, true, true>(a, grid, st);
                else
                    launch_mb_one<false, 8, 3, 3, 4, true, true>(a, grid, st);
            } else if (mb == 2) {
                // 32-row tiles: the paired loop where two waves share a SIMD (4096 x 11008 at 32 rows 15.4 -> 14.0 us,
                // per-column scales 14.9 -> 12.8; 8192 x 8192 16.6 -> 15.8), the ring loop, with its longer look-ahead,
                // where a wave has the SIMD to itself (5120 x 13824 with group scales: 16.7 vs 17.4 paired)
                bool pair2 = wk == 8;
                if (tune.pair != kUnset) pair2 = wk == 8 && tune.pair != 0;
                if (pair2) {
                    if (g128)
                        launch_mb_one<true, 2, 4, 3, 8, true, true>(a, grid, st);
                    else
                        launch_mb_one<false, 2, 4, 3, 8, true, true>(a, grid, st);
                } else {
                    launch_mb<2, 4, 3, false>(a, g128, wk, grid, st);
                }
            }
            else if (pair) launch_mb<4, 3, 3, true>(a, g128, wk, grid, st);
            else launch_mb<4, 3, 3, false, false>(a, g128, wk, grid, st);
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

int fp6m_mul_static(const void* A, const void* B, void* C, const void* s, int prob_m, int prob_n, int prob_k,
                    void* workspace, int dev, void* stream, int thread_k, int thread_n, int sms, int max_par,
                    int quant_cols, int group_size)
{
    return fp6m::mul_common(A, B, C, s, prob_m, prob_n, prob_k, workspace, dev, stream, thread_k, thread_n, sms, max_par,
                            quant_cols, group_size, fp6m::Fusion{}, true);
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
