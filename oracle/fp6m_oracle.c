/*
 * TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.
 *
 * Plain-C restatement of the CPU side of liuchuan22/FP6-Marlin, written to be
 * read next to the reference, step for step, so that the shipped (closed-form,
 * OpenMP, HIP) code paths can be checked bit-for-bit against an independent,
 * deliberately slow implementation.  Only tests/, __graft_entry__.smoke() and
 * the cpu_baseline leg of bench.py may load this library.  The product never
 * links or calls it.
 *
 * What each function follows (paths relative to the reference checkout):
 *   orc_half_to_float / orc_float_to_half   IEEE-754 binary16 <-> binary32,
 *                                           round-to-nearest-even (what the
 *                                           host `half` type of the reference
 *                                           does; no reference line)
 *   orc_fp6_cast4        fp6_marlin/weight_quant.cpp:27-96   (cast_fp16_fp6)
 *   orc_fp6_quantize     fp6_marlin/weight_quant.cpp:106-124
 *   orc_fp6_prepack      fp6_marlin/weight_prepacking.cpp:26-177
 *   orc_fp6_dequant      fp6_marlin/weight_prepacking.cpp:180-217
 *
 * How each one is pinned (the reference ships no golden vectors and its C++
 * cannot be compiled in this image: it includes <cuda_fp16.h>, whose only copy
 * here needs the absent <nv/target>):
 *   orc_fp6_cast4/quantize  exhaustive over all 65,536 binary16 patterns
 *                           against "largest e3m2 grid value not above |x|"
 *                           computed in floating point from the format's
 *                           closed form; byte packing against a bit-string
 *                           construction.
 *   orc_fp6_prepack         decoded with the reference *kernel's* own read and
 *                           bit rules (fp6_marlin_cuda_kernel.cu:195-237,
 *                           421-445, 548-600 and the PTX mma.m16n8k16 B
 *                           fragment map), every (n,k) code must come back;
 *                           plus bit-permutation invariants.
 *   orc_fp6_dequant         64-entry value table times scale in numpy float16.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_OK 0
#define ORC_ERR_RANGE 1 /* weight_quant.cpp:48-53 throws */
#define ORC_ERR_SHAPE 2 /* weight_quant.cpp:112, weight_prepacking.cpp:124-125,182-183 */

float orc_half_to_float(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 31u, m = h & 0x3ffu, bits;
    float f;
    if (e == 0) {
        f = (float)m * 5.9604644775390625e-8f; /* m * 2^-24, exact */
        memcpy(&bits, &f, 4);
        bits |= sign;
    } else if (e == 31) {
        bits = sign | 0x7f800000u | (m << 13);
    } else {
        bits = sign | ((e + 112u) << 23) | (m << 13);
    }
    memcpy(&f, &bits, 4);
    return f;
}

uint16_t orc_float_to_half(float f)
{
    uint32_t x;
    memcpy(&x, &f, 4);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    uint32_t ax = x & 0x7fffffffu;
    if (ax >= 0x7f800000u)
        return (uint16_t)(sign | 0x7c00u | (ax > 0x7f800000u ? 0x200u : 0u));
    int e = (int)(ax >> 23) - 127;
    uint32_t m = ax & 0x7fffffu;
    if (e > 15) return (uint16_t)(sign | 0x7c00u);
    if (e >= -14) {
        uint32_t h = ((uint32_t)(e + 15) << 10) | (m >> 13);
        uint32_t rest = m & 0x1fffu;
        if (rest > 0x1000u || (rest == 0x1000u && (h & 1u))) h++;
        return (uint16_t)(sign | h);
    }
    if (e < -25) return sign;
    uint32_t full = m | 0x800000u;
    int s = -(e + 1); /* 14..24 */
    uint32_t hm = full >> s, rest = full & ((1u << s) - 1u), half = 1u << (s - 1);
    if (rest > half || (rest == half && (hm & 1u))) hm++;
    return (uint16_t)(sign | hm);
}

/* binary16 multiply, one rounding: the binary32 product of two binary16 values is exact. */
static uint16_t orc_hmul(uint16_t a, uint16_t b)
{
    return orc_float_to_half(orc_half_to_float(a) * orc_half_to_float(b));
}

/* weight_quant.cpp:27-96.  Four binary16 values -> four e3m2 codes -> three bytes. */
int orc_fp6_cast4(const uint16_t in[4], uint8_t out[3])
{
    int code[4];
    for (int i = 0; i < 4; i++) {
        uint16_t src = in[i];
        float mag = fabsf(orc_half_to_float(src));
        /* :47-53  range test (NaN passes it in the reference and then yields
         * an out-of-range exponent field; the restatement reports it instead) */
        if (mag != mag) return ORC_ERR_RANGE;
        if ((mag != 0.0f && mag < 0.0625f) || mag > 28.0f) return ORC_ERR_RANGE;
        int bits = (int)src;
        int sgn = bits >> 15;                 /* :58 */
        int e16 = (bits & 0x7fff) >> 10;      /* :60 */
        int m16 = bits & 0x3ff;               /* :62 */
        int e6, m6;
        if (e16 == 0) {                       /* :67-70 binary16 sub-normal -> zero */
            e6 = 0;
            m6 = 0;
        } else {
            m6 = m16 >> 8;                    /* :72 drop 8 mantissa bits: truncation */
            e6 = e16 - 15 + 3;                /* :73 re-bias 15 -> 3 */
            int unb = e16 - 15;               /* :76 */
            int emin = -3 + 1;                /* :77 */
            if (unb < emin) {                 /* :78-86 e3m2 sub-normal */
                e6 = 0;
                m6 = (m6 | 4) >> (emin - unb);
            }
        }
        code[i] = (sgn << 5) | (e6 << 2) | m6; /* :89-90 */
    }
    out[0] = (uint8_t)((code[0] << 2) | (code[1] >> 4));          /* :93 */
    out[1] = (uint8_t)(((code[1] & 0x0f) << 4) | (code[2] >> 2)); /* :94 */
    out[2] = (uint8_t)(((code[2] & 0x03) << 6) | code[3]);        /* :95 */
    return ORC_OK;
}

/* weight_quant.cpp:106-124.  rows x cols binary16, flat row-major -> rows x cols*6/8 bytes. */
int orc_fp6_quantize(const uint16_t* w, uint8_t* out, size_t rows, size_t cols)
{
    if ((cols * 6) % 8 != 0) return ORC_ERR_SHAPE; /* :112 */
    size_t bpr = cols * 6 / 8;
    for (size_t r = 0; r < rows; r++)
        for (size_t c = 0; c < cols; c += 4) {
            int rc = orc_fp6_cast4(w + r * cols + c, out + r * bpr + (c / 4) * 3);
            if (rc) return rc;
        }
    return ORC_OK;
}

/* weight_prepacking.cpp:40-54: the 6-bit field that starts `bit` bits into
 * byte `p[0]`, returned left-aligned in a byte (cccccc00). */
static uint8_t orc_take6(const uint8_t* p, int bit)
{
    uint32_t w = (uint32_t)p[0] << 8;
    if (bit > 2) w |= p[1]; /* the field only spills into p[1] when bit > 2 */
    w = (w << bit) & 0xffffu;
    return (uint8_t)((w >> 8) & 0xfcu);
}

/* weight_prepacking.cpp:92-121: field i (counted from the MSB) of the result
 * is field order[i]-1 of the input. */
static uint32_t orc_interleave(uint32_t in, int width)
{
    static const int ord2[16] = {2, 6, 10, 14, 4, 8, 12, 16, 1, 5, 9, 13, 3, 7, 11, 15}; /* :103 */
    static const int ord4[8] = {2, 6, 4, 8, 1, 5, 3, 7};                                 /* :104 */
    const int* ord = width == 2 ? ord2 : ord4;
    uint32_t top = width == 2 ? 0xc0000000u : 0xf0000000u;
    uint32_t outw = 0;
    for (int i = 0; i < 32 / width; i++) {
        uint32_t frag = (in << (width * (ord[i] - 1))) & top; /* :116 */
        outw |= frag >> (i * width);                          /* :117 */
    }
    return outw;
}

static uint32_t orc_ld32(const uint8_t* p)
{
    return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24);
}
static void orc_st32(uint8_t* p, uint32_t v)
{
    p[0] = (uint8_t)v; p[1] = (uint8_t)(v >> 8); p[2] = (uint8_t)(v >> 16); p[3] = (uint8_t)(v >> 24);
}

/*
 * weight_prepacking.cpp:123-177.  `in6` is rows x (cols*6/8) bytes of row-packed
 * codes (rows = output channels n, cols = input channels k: the reference calls
 * them K and N in this routine, pybind.cpp:30 passes (OC, IC)).  `out` receives
 * rows*cols*2/8 bytes of "2-bit" words followed by rows*cols*4/8 bytes of
 * "4-bit" words (:129-130).
 */
int orc_fp6_prepack(uint8_t* out, const uint8_t* in6, size_t rows, size_t cols)
{
    if (rows % 64 || cols % 64 || rows == 0 || cols == 0) return ORC_ERR_SHAPE; /* :124-125 */
    size_t bpr = cols * 6 / 8;
    size_t len2 = rows * cols * 2 / 8 / 32, len4 = rows * cols * 4 / 8 / 32; /* :156-157 */
    uint8_t* s2 = (uint8_t*)malloc(32 * len2);
    uint8_t* s4 = (uint8_t*)malloc(32 * len4);
    if (!s2 || !s4) { free(s2); free(s4); return ORC_ERR_SHAPE; }
    size_t fill2 = 0, fill4 = 0; /* every lane stream grows in lock step */

    for (size_t kb = 0; kb < cols / 16; kb++)        /* :135 outer loop: 16 input channels */
        for (size_t nb = 0; nb < rows / 16; nb++) {  /* :136 inner loop: 16 output channels */
            const uint8_t* q1 = in6 + (nb * 16) * bpr + (kb * 16) * 6 / 8; /* :141 */
            const uint8_t* q3 = q1 + 8 * bpr;                               /* :142 */
            const uint8_t* q2 = q1 + 6;                                     /* :143  8 codes on */
            const uint8_t* q4 = q3 + 6;                                     /* :144 */
            for (int l = 0; l < 8; l++) {                                   /* :146-149 */
                const uint8_t* quad[4] = {q1 + l * bpr, q2 + l * bpr, q3 + l * bpr, q4 + l * bpr};
                for (int i = 0; i < 4; i++) { /* :56-90, one of the four lanes sharing row l */
                    uint8_t pad[8];
                    for (int j = 0; j < 8; j++) {
                        int off = (i * 2 + j % 2) * 6;             /* :66 */
                        pad[j] = orc_take6(quad[j / 2] + off / 8, off % 8); /* :69 */
                    }
                    uint8_t a2[2] = {0, 0}, a4[4] = {0, 0, 0, 0};
                    for (int j = 0; j < 8; j++) {                  /* :26-38 twice (:77-78) */
                        uint8_t hi2 = (uint8_t)(pad[j] & 0xc0u);          /* offset 0, width 2 */
                        uint8_t lo4 = (uint8_t)((pad[j] << 2) & 0xf0u);   /* offset 2, width 4 */
                        a2[(j * 2) / 8] |= (uint8_t)(hi2 >> ((j * 2) % 8));
                        a4[(j * 4) / 8] |= (uint8_t)(lo4 >> ((j * 4) % 8));
                    }
                    int lane = l * 4 + i;                          /* :148 */
                    memcpy(s2 + lane * len2 + fill2, a2, 2);       /* :83-84 */
                    memcpy(s4 + lane * len4 + fill4, a4, 4);       /* :85-88 */
                }
            }
            fill2 += 2;
            fill4 += 4;
        }

    uint8_t* w2 = out;
    uint8_t* w4 = out + rows * cols * 2 / 8;
    for (size_t i = 0; i < len2 / 8; i++)          /* :162-166 */
        for (int t = 0; t < 32; t++)
            for (int a = 0; a < 2; a++)
                for (int b = 0; b < 4; b++)
                    w2[i * 256 + t * 8 + a * 4 + (3 - b)] = s2[t * len2 + i * 8 + a * 4 + b];
    for (size_t i = 0; i < len4 / 16; i++)         /* :167-171 */
        for (int t = 0; t < 32; t++)
            for (int a = 0; a < 4; a++)
                for (int b = 0; b < 4; b++)
                    w4[i * 512 + t * 16 + a * 4 + (3 - b)] = s4[t * len4 + i * 16 + a * 4 + b];
    for (size_t i = 0; i < len2 * 32 / 4; i++)     /* :173-174 */
        orc_st32(w2 + 4 * i, orc_interleave(orc_ld32(w2 + 4 * i), 2));
    for (size_t i = 0; i < len4 * 32 / 4; i++)     /* :175-176 */
        orc_st32(w4 + 4 * i, orc_interleave(orc_ld32(w4 + 4 * i), 4));
    free(s2);
    free(s4);
    return ORC_OK;
}

/* weight_prepacking.cpp:180-217.  rows x cols*6/8 bytes + one binary16 scale per row -> binary16. */
int orc_fp6_dequant(uint16_t* out, const uint8_t* in6, size_t rows, size_t cols, const uint16_t* scale)
{
    if (rows % 64 || cols % 64) return ORC_ERR_SHAPE; /* :182-183 */
    size_t groups = rows * cols * 6 / 8 / 6;          /* :188, six bytes = eight codes */
    for (size_t g = 0; g < groups; g++) {
        const uint8_t* b = in6 + g * 6;
        for (int x = 0; x < 8; x++) {
            uint8_t c = orc_take6(b + (6 * x) / 8, (6 * x) % 8); /* :193-197 */
            uint32_t v = (uint32_t)c << 24;                      /* :205 */
            v = (v & 0x80000000u) | ((v & 0x7c000000u) >> 2);    /* :206 */
            uint16_t h = (uint16_t)(v >> 16);                    /* :207 */
            uint16_t s = scale[(8 * g) / cols];                  /* :212 row of this group */
            out[g * 8 + x] = orc_hmul(orc_hmul(h, 0x6c00u /* 4096.0 */), s); /* :212 */
        }
    }
    return ORC_OK;
}
