// Host-side converter: GPTQ-style packed delta -> native gfx950 layout.
//
// Input format as written by QuantLinear.pack in the reference
// (deltazip/nn_modules/qlinear_cuda.py:144-244): qweight[r, n] holds codes k = r*pf .. r*pf+pf-1
// from the low bits up; qzeros holds (zero - 1) packed along N; scales [G, N] fp16;
// g_idx[k] = k / group_size.  This function plays the part of the layout conversion the
// reference runs once per checkpoint (deltazip/utils/converter.py:13-101).
#include <cstring>
#include <vector>

#include "../../include/dz_amd.h"
#include "dz_layout.h"

extern "C" int dz_native_sizes(int K, int N, int bits, int group_size, size_t* codes_bytes,
                               size_t* meta_bytes, size_t* scales_bytes) {
  if (bits != 2 && bits != 4) return DZ_EBITS;
  if (K <= 0 || N <= 0 || K % DZ_KBLOCK || N % DZ_NPAIR) return DZ_ESHAPE;
  int gs = (group_size == -1 || group_size == K) ? K : group_size;
  if (gs <= 0 || K % gs || (gs != K && gs % 64)) return DZ_EGROUP;
  size_t kept = (size_t)K * N / 2;
  if (codes_bytes) *codes_bytes = kept * bits / 8;
  if (meta_bytes) *meta_bytes = kept * 2 / 8;
  if (scales_bytes) *scales_bytes = (size_t)(K / gs) * N * 2;
  return DZ_OK;
}

extern "C" int dz_repack_2of4(const int32_t* qweight, const int32_t* qzeros, const uint16_t* scales,
                              const int32_t* g_idx, int K, int N, int bits, int group_size,
                              void* out_codes, void* out_meta, void* out_scales) {
  if (!qweight || !qzeros || !scales || !out_codes || !out_meta || !out_scales) return DZ_EINVAL;
  size_t cb, mb, sb;
  int rc = dz_native_sizes(K, N, bits, group_size, &cb, &mb, &sb);
  if (rc) return rc;
  const int gs = (group_size == -1) ? K : group_size;
  const int G = K / gs;
  const int pf = 32 / bits;
  const uint32_t mask = (1u << bits) - 1u;
  const uint32_t zp = 1u << (bits - 1);
  const int nkb = K / DZ_KBLOCK;

  // zero-points: every (group, channel) must carry 2^(bits-1); stored value is zero - 1
  for (int g = 0; g < G; ++g)
    for (int n = 0; n < N; ++n) {
      uint32_t w = (uint32_t)qzeros[(size_t)g * (N / pf) + n / pf];
      uint32_t z = ((w >> (bits * (n % pf))) & mask) + 1u;
      if (z != zp) return DZ_EZERO;
    }
  if (g_idx)
    for (int k = 0; k < K; ++k)
      if (g_idx[k] != k / gs) return DZ_EGIDX;

  uint32_t* codes = (uint32_t*)out_codes;
  uint32_t* meta = (uint32_t*)out_meta;
  memset(codes, 0, cb);
  memset(meta, 0, mb);
  memcpy(out_scales, scales, sb);

  auto code_at = [&](int k, int n) -> uint32_t {
    uint32_t w = (uint32_t)qweight[(size_t)(k / pf) * N + n];
    return (w >> (bits * (k % pf))) & mask;
  };

  for (int np = 0; np < N / DZ_NPAIR; ++np)
    for (int kb = 0; kb < nkb; ++kb)
      for (int la = 0; la < 64; ++la) {
        const int ga = la >> 4, i = la & 15;
        for (int j = 0; j < 4; ++j)
          for (int s = 0; s < 2; ++s) {
            const int n = np * DZ_NPAIR + 16 * s + i;
            for (int p = 0; p < 4; ++p) {
              const int k0 = kb * DZ_KBLOCK + 64 * j + dz_group_k0(ga, p);
              uint32_t c[4];
              int kept[2], nk = 0, nnz = 0;
              for (int q = 0; q < 4; ++q) {
                c[q] = code_at(k0 + q, n);
                if (c[q] != zp) ++nnz;
              }
              if (nnz > 2) return DZ_ENOT24;
              // keep the non-zero-point columns, completed with the lowest free columns
              bool use[4] = {c[0] != zp, c[1] != zp, c[2] != zp, c[3] != zp};
              for (int q = 0; q < 4 && nnz < 2; ++q)
                if (!use[q]) { use[q] = true; ++nnz; }
              for (int q = 0; q < 4; ++q)
                if (use[q]) kept[nk++] = q;
              for (int w = 0; w < 2; ++w) {
                const int e = 2 * p + w;
                meta[dz_meta_word(np, kb, la, j, nkb)] |= (uint32_t)kept[w] << dz_meta_shift(s, e);
                if (bits == 2)
                  codes[dz_code2_word(np, kb, la, j, nkb)] |= c[kept[w]] << dz_code2_shift(s, e);
                else
                  codes[dz_code4_word(np, kb, la, j, s, nkb)] |= c[kept[w]] << dz_code4_shift(e);
              }
            }
          }
      }
  return DZ_OK;
}

// The inverse: native layout -> the reference's GPTQ-style tensors.  Pruned columns get the
// zero-point code (they dequantise to 0, as the reference's own packing of a pruned weight does:
// round(0 / scale) + zero), qzeros holds zero - 1 in every field, g_idx[k] = k / group_size.
extern "C" int dz_unrepack_2of4(const void* codes_in, const void* meta_in, const uint16_t* scales, int K, int N,
                                int bits, int group_size, int32_t* out_qweight, int32_t* out_qzeros,
                                uint16_t* out_scales, int32_t* out_g_idx) {
  if (!codes_in || !meta_in || !scales || !out_qweight || !out_qzeros || !out_scales) return DZ_EINVAL;
  size_t cb, mb, sb;
  int rc = dz_native_sizes(K, N, bits, group_size, &cb, &mb, &sb);
  if (rc) return rc;
  const int gs = (group_size == -1) ? K : group_size;
  const int G = K / gs;
  const int pf = 32 / bits;
  const uint32_t mask = (1u << bits) - 1u;
  const uint32_t zp = 1u << (bits - 1);
  const int nkb = K / DZ_KBLOCK;
  const uint32_t* codes = (const uint32_t*)codes_in;
  const uint32_t* meta = (const uint32_t*)meta_in;

  // every field = zero-point (qweight) and zero-point - 1 (qzeros)
  uint32_t wz = 0, wq = 0;
  for (int f = 0; f < pf; ++f) {
    wz |= zp << (bits * f);
    wq |= (zp - 1u) << (bits * f);
  }
  const size_t nq = (size_t)(K / pf) * N, nz = (size_t)G * (N / pf);
  for (size_t i = 0; i < nq; ++i) out_qweight[i] = (int32_t)wz;
  for (size_t i = 0; i < nz; ++i) out_qzeros[i] = (int32_t)wq;
  memcpy(out_scales, scales, sb);
  if (out_g_idx)
    for (int k = 0; k < K; ++k) out_g_idx[k] = k / gs;

  for (int np = 0; np < N / DZ_NPAIR; ++np)
    for (int kb = 0; kb < nkb; ++kb)
      for (int la = 0; la < 64; ++la) {
        const int ga = la >> 4, i = la & 15;
        for (int j = 0; j < 4; ++j) {
          const uint32_t mw = meta[dz_meta_word(np, kb, la, j, nkb)];
          for (int s = 0; s < 2; ++s) {
            const int n = np * DZ_NPAIR + 16 * s + i;
            for (int e = 0; e < 8; ++e) {
              const int pos = (int)((mw >> dz_meta_shift(s, e)) & 3u);
              const uint32_t c = bits == 2
                  ? (codes[dz_code2_word(np, kb, la, j, nkb)] >> dz_code2_shift(s, e)) & mask
                  : (codes[dz_code4_word(np, kb, la, j, s, nkb)] >> dz_code4_shift(e)) & mask;
              const int k = kb * DZ_KBLOCK + 64 * j + dz_group_k0(ga, e >> 1) + pos;
              uint32_t& w = (uint32_t&)out_qweight[(size_t)(k / pf) * N + n];
              const int sh = bits * (k % pf);
              w = (w & ~(mask << sh)) | (c << sh);
            }
          }
        }
      }
  return DZ_OK;
}
