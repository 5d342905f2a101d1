// Host side of the C ABI: FP6 (e3m2) quantise / 2+4-bit prepack / dequantise, symmetric INT4
// quantise / Marlin pack, scale permutation, and the inverse of both packers.  Closed-form,
// table-driven and threaded; results do not depend on the thread count.
//
// Reference behaviour being reproduced bit for bit (paths relative to liuchuan22/FP6-Marlin):
//   fp6m_fp6_quantize    fp6_marlin/weight_quant.cpp:27-124
//   fp6m_fp6_prepack     fp6_marlin/weight_prepacking.cpp:26-177
//   fp6m_fp6_dequant     fp6_marlin/weight_prepacking.cpp:180-217
//   fp6m_int4_quantize   test.py:85-101
//   fp6m_int4_pack       test.py:60-79, 106-113
//   fp6m_permute_scales  test.py:80-83, 102-105
//   fp6m_unpack_to_fp16  inverse of the two packers (kernel decode rules fp6_marlin_cuda_kernel.cu:195-286)
#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <thread>
#include <vector>

#include "fp6m.h"
#include "fp6m_layout.h"

namespace {

using fp6m::fp6_byte_of;
using fp6m::k_off;
using fp6m::scale_slot;

// ---------------------------------------------------------------------------------------- threads

unsigned worker_count()
{
    if (const char* e = std::getenv("FP6M_NUM_THREADS")) {
        int v = std::atoi(e);
        if (v > 0) return (unsigned)v;
    }
    unsigned hw = std::thread::hardware_concurrency();
    return std::max(1u, std::min(hw ? hw : 1u, 16u));
}

// Runs body(begin, end) over [0, n) split into contiguous chunks, one per worker.
template <class F>
void parallel_chunks(size_t n, size_t min_chunk, F&& body)
{
    size_t workers = std::min<size_t>(worker_count(), std::max<size_t>(1, n / std::max<size_t>(1, min_chunk)));
    if (workers <= 1) {
        body(size_t(0), n);
        return;
    }
    std::vector<std::thread> pool;
    pool.reserve(workers);
    for (size_t w = 0; w < workers; w++) {
        size_t b = n * w / workers, e = n * (w + 1) / workers;
        pool.emplace_back([=, &body] { body(b, e); });
    }
    for (auto& t : pool) t.join();
}

// ---------------------------------------------------------------------------------------- binary16

inline float half_to_float(uint16_t h)
{
    const uint32_t e = (h >> 10) & 31u, m = h & 0x3ffu;
    float f;
    if (e == 0) {
        f = (float)m * 5.9604644775390625e-8f;  // m * 2^-24; no binary32 sub-normal is ever formed
    } else {
        uint32_t b = e == 31 ? (0x7f800000u | (m << 13)) : (((e + 112u) << 23) | (m << 13));
        std::memcpy(&f, &b, 4);
    }
    return (h & 0x8000u) ? -f : f;
}

inline uint16_t float_to_half(float f)
{
    uint32_t x;
    std::memcpy(&x, &f, 4);
    const uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    x &= 0x7fffffffu;
    if (x > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);
    if (x >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);  // >= 65520 rounds to inf
    if (x < 0x38800000u) {
        // below 2^-14: adding 0.5 aligns the value so the low mantissa bits of the sum are the
        // sub-normal binary16 mantissa, rounded to nearest even by the FPU.
        float a;
        std::memcpy(&a, &x, 4);
        a += 0.5f;
        uint32_t y;
        std::memcpy(&y, &a, 4);
        return (uint16_t)(sign | (y - 0x3f000000u));
    }
    uint32_t odd = (x >> 13) & 1u;
    x += 0xc8000000u + 0x0fffu + odd;  // re-bias exponent by -112 and round to nearest even
    return (uint16_t)(sign | (x >> 13));
}

inline uint16_t half_mul(uint16_t a, uint16_t b)
{
    return float_to_half(half_to_float(a) * half_to_float(b));  // the binary32 product is exact
}

// ---------------------------------------------------------------------------------------- FP6 tables

constexpr uint8_t kBadCode = 0xff;

struct Fp6Tables {
    uint8_t code_of_half[65536];  // binary16 pattern -> e3m2 code, or kBadCode when out of range
    uint16_t half_of_code[64];    // e3m2 code -> binary16 pattern of its exact value
    Fp6Tables()
    {
        double grid[32];
        for (int c = 0; c < 32; c++) {
            int e = c >> 2, m = c & 3;
            grid[c] = e == 0 ? m * 0.0625 : std::ldexp(1.0 + m / 4.0, e - 3);
        }
        for (int c = 0; c < 64; c++)
            half_of_code[c] = (uint16_t)(float_to_half((float)grid[c & 31]) | ((c & 32) ? 0x8000u : 0u));
        for (uint32_t h = 0; h < 65536; h++) {
            double mag = std::fabs((double)half_to_float((uint16_t)h));
            if (!(mag == mag) || (mag != 0.0 && mag < 0.0625) || mag > 28.0) {
                code_of_half[h] = kBadCode;
                continue;
            }
            int idx = 0;
            while (idx + 1 < 32 && grid[idx + 1] <= mag) idx++;  // round toward zero onto the grid
            code_of_half[h] = (uint8_t)(idx | ((h >> 15) << 5));
        }
    }
};

const Fp6Tables& tables()
{
    static const Fp6Tables t;
    return t;
}

// rows x cols*6/8 bytes (four codes per three bytes, MSB first) -> one byte per code
void expand_codes(const uint8_t* packed, uint8_t* codes, size_t rows, size_t cols)
{
    parallel_chunks(rows, 8, [=](size_t r0, size_t r1) {
        for (size_t r = r0; r < r1; r++) {
            const uint8_t* p = packed + r * (cols * 6 / 8);
            uint8_t* c = codes + r * cols;
            for (size_t q = 0; q < cols / 4; q++, p += 3, c += 4) {
                uint32_t v = ((uint32_t)p[0] << 16) | ((uint32_t)p[1] << 8) | p[2];
                c[0] = (v >> 18) & 63;
                c[1] = (v >> 12) & 63;
                c[2] = (v >> 6) & 63;
                c[3] = v & 63;
            }
        }
    });
}

// Nibble of element x inside a packed INT4 word.
inline int int4_nibble_of(int x) { return (x & 1) * 4 + (x >> 1); }

}  // namespace

extern "C" {

const char* fp6m_strerror(int code)
{
    switch (code) {
        case FP6M_OK: return "ok";
        case FP6M_ERR_PROB_SHAPE: return "problem shape not compatible with the tile shape";
        case FP6M_ERR_KERN_SHAPE: return "no kernel implementation for this thread_k/thread_n";
        case FP6M_ERR_RANGE: return "Input value out of range for FP6.";
        case FP6M_ERR_SHAPE: return "matrix dimensions not supported by this routine";
        case FP6M_ERR_ARG: return "invalid argument";
        case FP6M_ERR_HIP: return "HIP runtime error";
        case FP6M_ERR_NO_GPU_CODE: return "library built without gfx950 kernels";
        case FP6M_ERR_SCRATCH: return "no scratch for this call: its partial sums do not fit fp6m_mul_static's array (fp6m_mul has room for them), or a workspace beyond the built-in regions was first used while its stream was capturing (call fp6m_init_workspace before the capture)";
        default: return "unknown fp6m error";
    }
}

int fp6m_abi_version(void) { return 1; }

size_t fp6m_workspace_elems(int prob_n, int max_par)
{
    if (prob_n <= 0 || max_par <= 0) return 0;
    return (size_t)(prob_n / 128) * (size_t)max_par;
}

int fp6m_fp6_quantize(const uint16_t* w, uint8_t* out, size_t rows, size_t cols)
{
    if (!w || !out) return FP6M_ERR_ARG;
    if ((cols * 6) % 8 != 0) return FP6M_ERR_SHAPE;
    const Fp6Tables& T = tables();
    std::atomic<int> bad{0};
    parallel_chunks(rows, 8, [&, w, out, cols](size_t r0, size_t r1) {
        for (size_t r = r0; r < r1; r++) {
            const uint16_t* src = w + r * cols;
            uint8_t* dst = out + r * (cols * 6 / 8);
            for (size_t q = 0; q < cols / 4; q++, src += 4, dst += 3) {
                uint8_t c0 = T.code_of_half[src[0]], c1 = T.code_of_half[src[1]];
                uint8_t c2 = T.code_of_half[src[2]], c3 = T.code_of_half[src[3]];
                if ((c0 | c1 | c2 | c3) & 0x80) {
                    bad.store(1, std::memory_order_relaxed);
                    return;
                }
                uint32_t v = ((uint32_t)c0 << 18) | ((uint32_t)c1 << 12) | ((uint32_t)c2 << 6) | c3;
                dst[0] = (uint8_t)(v >> 16);
                dst[1] = (uint8_t)(v >> 8);
                dst[2] = (uint8_t)v;
            }
        }
    });
    return bad.load() ? FP6M_ERR_RANGE : FP6M_OK;
}

int fp6m_fp6_prepack(int32_t* packed, const int32_t* fp6, size_t oc, size_t ic)
{
    if (!packed || !fp6) return FP6M_ERR_ARG;
    if (oc == 0 || ic == 0 || oc % 64 || ic % 64) return FP6M_ERR_SHAPE;
    std::vector<uint8_t> codes(oc * ic);
    expand_codes(reinterpret_cast<const uint8_t*>(fp6), codes.data(), oc, ic);
    const uint8_t* cd = codes.data();
    uint32_t* plane2 = reinterpret_cast<uint32_t*>(packed);
    uint32_t* plane4 = plane2 + oc * ic * 2 / 32;
    const size_t groups = oc / 64;
    parallel_chunks(ic / 16, 1, [=](size_t kb0, size_t kb1) {
        for (size_t kb = kb0; kb < kb1; kb++)
            for (size_t g = 0; g < groups; g++)
                for (int t = 0; t < 32; t++) {
                    const int l = t >> 2, i = t & 3;
                    const size_t owner = (kb * groups + g) * 32 + t;
                    uint32_t w2[2] = {0, 0};
                    for (int j = 0; j < 4; j++) {
                        uint32_t w4 = 0;
                        for (int x = 0; x < 8; x++) {
                            size_t n = 64 * g + 16 * j + l + 8 * (x >> 2);
                            size_t k = 16 * kb + k_off(i, x & 3);
                            uint32_t c = cd[n * ic + k];
                            int b = fp6_byte_of(x), hi = x >> 2;
                            w4 |= (c & 15u) << (28 - 4 * (2 * b + hi));
                            w2[j >> 1] |= (c >> 4) << (30 - 2 * (4 * b + 2 * (j & 1) + hi));
                        }
                        plane4[owner * 4 + j] = w4;
                    }
                    plane2[owner * 2 + 0] = w2[0];
                    plane2[owner * 2 + 1] = w2[1];
                }
    });
    return FP6M_OK;
}

int fp6m_fp6_dequant(uint16_t* out, const uint8_t* fp6, size_t rows, size_t cols, const uint16_t* scale)
{
    if (!out || !fp6 || !scale) return FP6M_ERR_ARG;
    if (rows % 64 || cols % 64) return FP6M_ERR_SHAPE;
    const Fp6Tables& T = tables();
    parallel_chunks(rows, 8, [=, &T](size_t r0, size_t r1) {
        for (size_t r = r0; r < r1; r++) {
            const uint8_t* p = fp6 + r * (cols * 6 / 8);
            uint16_t* o = out + r * cols;
            const uint16_t s = scale[r];
            for (size_t q = 0; q < cols / 4; q++, p += 3, o += 4) {
                uint32_t v = ((uint32_t)p[0] << 16) | ((uint32_t)p[1] << 8) | p[2];
                o[0] = half_mul(T.half_of_code[(v >> 18) & 63], s);
                o[1] = half_mul(T.half_of_code[(v >> 12) & 63], s);
                o[2] = half_mul(T.half_of_code[(v >> 6) & 63], s);
                o[3] = half_mul(T.half_of_code[v & 63], s);
            }
        }
    });
    return FP6M_OK;
}

int fp6m_int4_quantize(const uint16_t* w, size_t k, size_t n, int group_size, uint8_t* codes,
                       uint16_t* scales, uint16_t* w_ref)
{
    if (!w) return FP6M_ERR_ARG;
    if (k == 0 || n == 0) return FP6M_OK;
    const size_t g = group_size == -1 ? k : (size_t)group_size;
    if (group_size == 0 || group_size < -1 || k % g) return FP6M_ERR_SHAPE;
    const float two_over_15 = (float)(2.0 / 15.0);  // the harness multiplies in binary32
    const size_t ngroups = k / g;
    parallel_chunks(n, 16, [=](size_t c0, size_t c1) {
        for (size_t gi = 0; gi < ngroups; gi++)
            for (size_t c = c0; c < c1; c++) {
                uint16_t amax = 0;
                for (size_t r = gi * g; r < (gi + 1) * g; r++) amax = std::max<uint16_t>(amax, w[r * n + c] & 0x7fffu);
                const uint16_t sh = float_to_half(half_to_float(amax) * two_over_15);
                const float sf = half_to_float(sh);
                if (scales) scales[gi * n + c] = sh;
                for (size_t r = gi * g; r < (gi + 1) * g; r++) {
                    int q = 8;
                    uint16_t ref = 0;
                    if (sf != 0.0f) {
                        // round(w / s) + 8, clamp; then the fake-quantised value and its own re-quantisation
                        float t = half_to_float(float_to_half(half_to_float(w[r * n + c]) / sf));
                        q = std::min(15, std::max(0, (int)std::nearbyintf(std::min(64.0f, std::max(-64.0f, t))) + 8));
                        ref = float_to_half((float)(q - 8) * sf);
                        float t2 = half_to_float(float_to_half(half_to_float(ref) / sf));
                        q = std::min(15, std::max(0, (int)std::nearbyintf(std::min(64.0f, std::max(-64.0f, t2))) + 8));
                    }
                    if (codes) codes[r * n + c] = (uint8_t)q;
                    if (w_ref) w_ref[r * n + c] = ref;
                }
            }
    });
    return FP6M_OK;
}

int fp6m_int4_pack(const uint8_t* codes, int32_t* packed, size_t k, size_t n)
{
    if (!codes || !packed) return FP6M_ERR_ARG;
    if (k % 16 || n % 64) return FP6M_ERR_SHAPE;
    uint32_t* out = reinterpret_cast<uint32_t*>(packed);
    const size_t groups = n / 64;
    parallel_chunks(k / 16, 1, [=](size_t kb0, size_t kb1) {
        for (size_t kb = kb0; kb < kb1; kb++)
            for (size_t g = 0; g < groups; g++)
                for (int t = 0; t < 32; t++) {
                    const int l = t >> 2, i = t & 3;
                    for (int j = 0; j < 4; j++) {
                        uint32_t word = 0;
                        for (int x = 0; x < 8; x++) {
                            size_t kk = 16 * kb + k_off(i, x & 3);
                            size_t nn = 64 * g + 16 * j + l + 8 * (x >> 2);
                            word |= (uint32_t)(codes[kk * n + nn] & 15u) << (4 * int4_nibble_of(x));
                        }
                        out[((kb * groups + g) * 32 + t) * 4 + j] = word;
                    }
                }
    });
    return FP6M_OK;
}

int fp6m_permute_scales(const uint16_t* in, uint16_t* out, size_t n)
{
    if (!in || !out) return FP6M_ERR_ARG;
    if (n % 32) return FP6M_ERR_SHAPE;
    for (size_t c = 0; c < n; c++) out[(c & ~size_t(31)) + scale_slot((int)(c & 31))] = in[c];
    return FP6M_OK;
}

namespace {

// One plane (rows x cols weights, `words` 32-bit words per lane and k-block) between the reference's granule order
// [k-block][64-column group][owner 4 l + i] and the gfx950 one [tile][k-block][lane 16 i + 8 sigma + l].
void repack_plane(const uint32_t* in, uint32_t* out, size_t rows, size_t cols, int words, bool to_gfx950)
{
    const size_t kblocks = rows / 16, tiles = cols / 128;
    parallel_chunks(kblocks, 1, [=](size_t kb0, size_t kb1) {
        for (size_t kb = kb0; kb < kb1; kb++)
            for (size_t t = 0; t < tiles; t++)
                for (int lane = 0; lane < 64; lane++) {
                    const int i = lane >> 4, sigma = (lane >> 3) & 1, l = lane & 7;
                    const size_t ref = ((kb * (cols / 64) + 2 * t + sigma) * 32 + 4 * l + i) * words;
                    const size_t nat = ((t * kblocks + kb) * 64 + lane) * words;
                    for (int w = 0; w < words; w++) {
                        if (to_gfx950) out[nat + w] = in[ref + w];
                        else out[ref + w] = in[nat + w];
                    }
                }
    });
}

}  // namespace

int fp6m_repack_gfx950(const int32_t* in, int32_t* out, size_t k, size_t n, int quant_cols, int quant_rows, int to_gfx950)
{
    if (!in || !out || in == out) return FP6M_ERR_ARG;
    const uint32_t* src = reinterpret_cast<const uint32_t*>(in);
    uint32_t* dst = reinterpret_cast<uint32_t*>(out);
    size_t rows4, cols4, rows6, cols6;                                // the INT4 block and the FP6 block
    if (quant_rows > 0) {
        if ((size_t)quant_rows >= k) return FP6M_ERR_ARG;
        rows4 = k - (size_t)quant_rows, cols4 = n, rows6 = (size_t)quant_rows, cols6 = n;
    } else {
        const size_t qc = quant_cols <= 0 ? 0 : (size_t)quant_cols;
        if (qc > n) return FP6M_ERR_ARG;
        rows4 = k, cols4 = n - qc, rows6 = k, cols6 = qc;
    }
    if (rows4 % 16 || rows6 % 16 || cols4 % 128 || cols6 % 128) return FP6M_ERR_SHAPE;
    const size_t words4 = rows4 * cols4 / 8, words2 = rows6 * cols6 / 16;
    if (cols4) repack_plane(src, dst, rows4, cols4, 4, to_gfx950 != 0);
    if (cols6) {
        repack_plane(src + words4, dst + words4, rows6, cols6, 2, to_gfx950 != 0);
        repack_plane(src + words4 + words2, dst + words4 + words2, rows6, cols6, 4, to_gfx950 != 0);
    }
    return FP6M_OK;
}

int fp6m_unpack_to_fp16(const int32_t* B, const uint16_t* s, uint16_t* w_ref, size_t k, size_t n,
                        int quant_cols, int group_size)
{
    if (!B || !s || !w_ref) return FP6M_ERR_ARG;
    size_t qc = quant_cols <= 0 ? 0 : (size_t)quant_cols;
    if (qc > n) return FP6M_ERR_ARG;
    const size_t n4 = n - qc;
    if (k % 16 || n4 % 64 || qc % 64) return FP6M_ERR_SHAPE;
    if (group_size != -1 && (group_size <= 0 || k % (size_t)group_size)) return FP6M_ERR_ARG;
    const Fp6Tables& T = tables();
    const uint32_t* b4 = reinterpret_cast<const uint32_t*>(B);
    const uint32_t* p2 = b4 + k * n4 / 8;
    const uint32_t* p4 = p2 + k * qc / 16;
    const uint16_t* s6 = s + (group_size == -1 ? n4 : (k / (size_t)group_size) * n4);
    const size_t g4 = n4 / 64, g6 = qc / 64;
    parallel_chunks(k / 16, 1, [=, &T](size_t kb0, size_t kb1) {
        for (size_t kb = kb0; kb < kb1; kb++) {
            for (size_t g = 0; g < g4; g++)
                for (int t = 0; t < 32; t++)
                    for (int j = 0; j < 4; j++) {
                        uint32_t word = b4[((kb * g4 + g) * 32 + t) * 4 + j];
                        for (int x = 0; x < 8; x++) {
                            size_t kk = 16 * kb + k_off(t & 3, x & 3);
                            size_t nn = 64 * g + 16 * j + (t >> 2) + 8 * (x >> 2);
                            int q = (int)((word >> (4 * int4_nibble_of(x))) & 15u) - 8;
                            uint16_t sc = group_size == -1 ? s[(nn & ~size_t(31)) + scale_slot((int)(nn & 31))]
                                                           : s[(kk / (size_t)group_size) * n4 + nn];
                            w_ref[kk * n + nn] = float_to_half((float)q * half_to_float(sc));
                        }
                    }
            for (size_t g = 0; g < g6; g++)
                for (int t = 0; t < 32; t++) {
                    const size_t owner = (kb * g6 + g) * 32 + t;
                    for (int j = 0; j < 4; j++) {
                        uint32_t w4 = p4[owner * 4 + j], w2 = p2[owner * 2 + (j >> 1)];
                        for (int x = 0; x < 8; x++) {
                            int b = fp6_byte_of(x), hi = x >> 2;
                            uint32_t lo4 = (w4 >> (28 - 4 * (2 * b + hi))) & 15u;
                            uint32_t hi2 = (w2 >> (30 - 2 * (4 * b + 2 * (j & 1) + hi))) & 3u;
                            size_t kk = 16 * kb + k_off(t & 3, x & 3);
                            size_t nn = 64 * g + 16 * j + (t >> 2) + 8 * (x >> 2);
                            uint16_t sc = s6[(nn & ~size_t(31)) + scale_slot((int)(nn & 31))];
                            w_ref[kk * n + n4 + nn] = half_mul(T.half_of_code[(hi2 << 4) | lo4], sc);
                        }
                    }
                }
        }
    });
    return FP6M_OK;
}

}  // extern "C"
