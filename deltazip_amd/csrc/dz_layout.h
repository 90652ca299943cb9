// Native gfx950 layout of one 2:4-sparse, 2/4-bit delta: index arithmetic shared by the host
// repacker and the device kernels.
//
// Tiles.  "n-pair": 32 output rows = two 16-row fragments (s = 0, 1).  "k-block": 256 input
// columns = four 64-column steps (j = 0..3).  A fragment is 16 rows x 64 columns, the sparse
// operand of one v_smfmac_f32_16x16x64_f16.  Lane la = 16*ga + i of the wavefront owns row i
// and four aligned groups of 4 columns; group p (0..3) starts at column
//     dz_group_k0(ga, p) = 16*(ga & 1) + 32*(ga >> 1) + 8*(p >> 1) + 4*(p & 1)
// of the step.  Each group contributes its two kept columns in ascending order: element
// e = 2*p + w, w = 0, 1.  The matching dense operand holds, in lane 16*gb + token, values
// eb = 0..15 for columns 8*gb + (eb & 7) + 32*(eb >> 3) of the step, which is also the order in
// which two v_mfma_f32_16x16x32_f16 consume a dense row (columns 32*h + 8*g + e).
//
// Arrays (uint32 words, each lane's 4 words contiguous so a wavefront reads 1 KiB per load):
//   meta        [N/32][K/256][64 lanes][4]       word j: bits [16*s + 2*e, +2) = kept column (0..3)
//                                                of element e, fragment (2*np + s, 4*kb + j)
//   codes 2-bit [N/32][K/256][64 lanes][4]       word j; t = 4*s + m: bits [2t, +2) = element 2m,
//                                                bits [16 + 2t, +2) = element 2m + 1
//   codes 4-bit [N/32][K/256][2][64 lanes][4]    half hf = j >> 1, word 2*(j & 1) + s:
//                                                bits [4m, +4) = element 2m, bits [16 + 4m, +4) = 2m + 1
//   scales fp16 [G][N]                           as in the GPTQ layout
#pragma once
#include <stddef.h>
#include <stdint.h>

#define DZ_KBLOCK 256
#define DZ_NPAIR 32

#if defined(__HIPCC__)
#define DZ_HD __host__ __device__
#else
#define DZ_HD
#endif

DZ_HD static inline int dz_group_k0(int ga, int p) {
  return 16 * (ga & 1) + 32 * (ga >> 1) + 8 * (p >> 1) + 4 * (p & 1);
}
// word index (in uint32) of lane la, word w inside the arrays
DZ_HD static inline size_t dz_meta_word(int np, int kb, int la, int j, int nkb) {
  return (((size_t)np * nkb + kb) * 64 + la) * 4 + j;
}
DZ_HD static inline size_t dz_code2_word(int np, int kb, int la, int j, int nkb) {
  return (((size_t)np * nkb + kb) * 64 + la) * 4 + j;
}
DZ_HD static inline size_t dz_code4_word(int np, int kb, int la, int j, int s, int nkb) {
  return ((((size_t)np * nkb + kb) * 2 + (j >> 1)) * 64 + la) * 4 + 2 * (j & 1) + s;
}
// Base weight in tiles (optional; the fused kernel for up to 128 tokens reads either form).  Tile
// (np, kb) = 32 rows x 256 columns = 16 KiB, stored contiguously; inside it 16 fragments of 1 KiB,
// fragment (s, j, h) = the dense operand of one v_mfma_f32_16x16x32_f16: lane la = 16*g + i holds
// the 8 values W[32*np + 16*s + i][256*kb + 64*j + 16*g + 8*h + e], e = 0..7 (16 bytes per lane, a
// wavefront reads one fragment per load).  The matching activation order is the one the kernel
// uses for the row-major form, so both forms give the same sums in the same order.
DZ_HD static inline size_t dz_base_tile_offset(int np, int kb, int nkb) { return ((size_t)np * nkb + kb) * 16384; }
DZ_HD static inline int dz_base_frag_offset(int s, int j, int h) { return ((s * 4 + j) * 2 + h) * 1024; }
DZ_HD static inline int dz_meta_shift(int s, int e) { return 16 * s + 2 * e; }
DZ_HD static inline int dz_code2_shift(int s, int e) { return 2 * (4 * s + (e >> 1)) + 16 * (e & 1); }
DZ_HD static inline int dz_code4_shift(int e) { return 4 * (e >> 1) + 16 * (e & 1); }
