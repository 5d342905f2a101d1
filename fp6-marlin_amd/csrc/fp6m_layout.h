// Packed-weight layout shared by the host packers and the gfx950 kernels.
//
// Both weight formats are organised for a 32-lane "fragment owner" t = 4*l + i
// (l = 0..7, i = 0..3) inside a 16-row k-block and a 64-column group g.  For
// tile j = 0..3 of the group, owner t holds eight weights e0..e7:
//
//     e_x :  k = 16*kb + kOff(i, x % 4),   n = 64*g + 16*j + l + 8*(x / 4)
//     kOff(i, r) = 2*i + (r & 1) + 8*(r >> 1)          ->  {2i, 2i+1, 2i+8, 2i+9}
//
// (reference: test.py:60-79 for INT4, weight_prepacking.cpp:56-90,135-150 for FP6).
//
// INT4   : one 32-bit word per (kb, g, t, j) at word index ((kb*G + g)*32 + t)*4 + j, G = n/64;
//          element e_x sits in nibble (x % 2)*4 + x/2, stored value = q + 8.
// FP6    : the low four bits of the eight codes form a "4-bit" word with the same addressing as
//          INT4; fields, MSB first, are e1 e5 e3 e7 e0 e4 e2 e6.  The top two bits of the codes of
//          tiles 2a and 2a+1 share a "2-bit" word at index ((kb*G + g)*32 + t)*2 + a; byte b of
//          it (MSB first) holds, two bits each, [T0 e_x, T0 e_{x+4}, T1 e_x, T1 e_{x+4}] with
//          x = {1, 3, 0, 2}[b].  The 2-bit plane (k*n/16 words) precedes the 4-bit plane.
#pragma once
#include <stdint.h>

namespace fp6m {

#if defined(__HIPCC__)
#define FP6M_HD __host__ __device__ inline
#else
#define FP6M_HD inline
#endif

FP6M_HD int k_off(int i, int r) { return 2 * i + (r & 1) + 8 * (r >> 1); }

// Byte-group b (MSB first) that element x of a fragment lands in, FP6 planes: x%4 = 1,3,0,2 -> b = 0,1,2,3.
FP6M_HD int fp6_byte_of(int x) { return (0x1302 >> (4 * (x & 3))) & 3; }  // x%4: 0->2, 1->0, 2->3, 3->1

// Stored position, inside its group of 32 columns, of the per-column scale of column c (0..31):
// the inverse of the reference's scale permutation (test.py:80-83).
FP6M_HD int scale_slot(int c) { return 8 * ((c & 7) >> 1) + 4 * (c >> 4) + 2 * ((c >> 3) & 1) + (c & 1); }

}  // namespace fp6m
