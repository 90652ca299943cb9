// Dense fp16 GEMM on the gfx950 matrix cores for prefill-sized token counts:
//   y[t, :] (+)= x[t, :] @ w^T  (+ x[t, :] @ w2[g(t)]^T),   fp32 accumulation, fp16 in and out.
// The optional second weight differs per block of rows ("grouped"): the rows are tokens sorted by
// delta id, w is the base weight and w2[g] the dequantised delta of group g, and both products
// share the fp32 accumulators, so base and delta are never added in fp16.
//
// One workgroup (4 wavefronts, 2 x 2) computes a 256 (tokens) x 256 (output features) tile; each
// wavefront owns 128 x 128 of it as 4 x 4 v_mfma_f32_32x32x16_f16 tiles (256 accumulator
// registers).  K is walked in slabs of 64: both operand slabs (2 x 32 KiB) go from global memory
// straight into LDS (LDS-direct loads, 16 bytes per lane) into one of two buffers, so the next
// slab is on its way while the matrix cores work on the current one; one barrier per slab.
// Operand rows in LDS are 128 bytes; the 16-byte chunk index is XOR-ed with half the row number,
// which keeps the 32-row fragment reads off shared banks.  Workgroups are numbered so that the 32 that run
// together on one XCD form a 4 x 8 block of tiles and share operand slabs in that XCD's L2.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/dz_amd.h"
#include "dz_device.h"

typedef _Float16 h8_t __attribute__((ext_vector_type(8)));
typedef _Float16 h4_t __attribute__((ext_vector_type(4)));
typedef float f16_t __attribute__((ext_vector_type(16)));

namespace {

constexpr int BM = 256, BN = 256, BK = 64;
constexpr int SLAB = 256 * BK * 2;        // bytes of one operand slab in LDS
constexpr int GM = 4, GN = 8;             // tiles per XCD block

struct GemmParams {
  const _Float16* x;
  const _Float16* w;             // first weight [N, K], or nullptr (second product only)
  const _Float16* w2;            // stack of second weights or nullptr
  long long w2_stride;           // elements between consecutive second weights
  const dz_gemm_tile* tiles;     // row blocks, or nullptr: blocks of 256 rows, second weight 0
  const int* perm;               // row blocks count positions of this token order (rows of x and y), or nullptr
  _Float16* y;
  int T, K, N, accumulate, ldy, tiles_m, tiles_n;
  int select;                    // a block with a second weight is multiplied by that weight only
};

__global__ __launch_bounds__(256, 1) void dz_gemm_kernel(const GemmParams P) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];   // [2 buffers][w slab | x slab]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;

  // workgroup -> tile: XCD-local blocks of GM x GN tiles
  const int xcd = blockIdx.x & 7, q = blockIdx.x >> 3;
  const int sbn = (P.tiles_n + GN - 1) / GN;
  const int sb = (q / (GM * GN)) * 8 + xcd, r = q % (GM * GN);
  const int tm = (sb / sbn) * GM + r / GN, tn = (sb % sbn) * GN + r % GN;
  if (tm >= P.tiles_m || tn >= P.tiles_n) return;
  int row_lo = tm * BM, row_hi = min(P.T, row_lo + BM), widx = 0;   // no table: one group, second weight 0
  if (P.tiles) {
    row_lo = P.tiles[tm].row_lo;
    row_hi = P.tiles[tm].row_hi;
    widx = P.tiles[tm].group;
    if (row_hi <= row_lo) return;   // unused entry of the table
  }
  const int n0 = tn * BN;
  const _Float16* w2 = (P.w2 && widx >= 0) ? P.w2 + (size_t)widx * P.w2_stride : nullptr;
  const int nslab1 = P.K / BK, nslab = w2 ? 2 * nslab1 : nslab1;
  const int s_begin = (P.w && !(P.select && w2)) ? 0 : nslab1;   // no first weight (for this block): second product only
  if (s_begin >= nslab) return;           // neither: the tile is left as it is
  const unsigned Kb = (unsigned)P.K * 2u;
  // A block of few rows (a decode batch spread over several tables): token rows beyond the block
  // are neither requested nor multiplied -- a request covers 8 rows, a product 32 -- so that such a
  // block costs the stream of its weight slab and little else.  (What the skipped rows' LDS bytes
  // hold only reaches output columns that are never stored.)
  const int nrows = row_hi - row_lo;
  const int nb = min(4, max(0, (nrows - wm * 128 + 31) / 32));   // this wavefront's 32-token tiles in use

  f16_t acc[4][4];
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int b = 0; b < 4; ++b)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[a][b][e] = 0.f;

  // ---- slab loader: 64 requests of 1 KiB (8 rows x 128 bytes) per slab pair, 16 per wavefront.
  // Lane l fills LDS row l/8, physical chunk l%8 with global chunk (l%8) ^ ((row >> 1) & 7): a
  // 16-byte read is served 16 lanes (256 bytes, two rows' worth of banks) per cycle, and 16
  // consecutive rows then fall on 16 different bank groups.
  const int lr = lane >> 3;
  unsigned goff[16];   // global byte offset of this lane's row start + chunk, per request
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int rq = wave * 16 + i, sub = rq & 31, R = sub * 8 + lr;
    unsigned rowoff;
    if (rq < 32) rowoff = (unsigned)min(n0 + R, P.N - 1);           // weight rows (clamped: never stored)
    else {                                                          // token rows
      const int pos = min(row_lo + R, row_hi - 1);
      rowoff = (unsigned)(P.perm ? P.perm[pos] : pos);
    }
    const int lc = (lane & 7) ^ ((R >> 1) & 7);
    goff[i] = rowoff * Kb + (unsigned)lc * 16u;
  }
  // (buffer form of the LDS-direct load: scalar descriptor + 32-bit lane offset + scalar slab
  // offset, so no 64-bit per-lane address is ever built or kept)
  const __amdgpu_buffer_rsrc_t rw =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<_Float16*>(P.w ? P.w : w2), 0, 0x7fffffff, 0x00020000);
  const __amdgpu_buffer_rsrc_t rw2 =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<_Float16*>(w2 ? w2 : P.w), 0, 0x7fffffff, 0x00020000);
  const __amdgpu_buffer_rsrc_t rx =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<_Float16*>(P.x), 0, 0x7fffffff, 0x00020000);
  auto issue = [&](int s, int buf) {
    const bool second = s >= nslab1;
    const int soff = (second ? s - nslab1 : s) * (BK * 2);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int rq = wave * 16 + i, sub = rq & 31;
      unsigned char* dst = smem + buf * (2 * SLAB) + (rq < 32 ? 0 : SLAB) + sub * 1024;
      __attribute__((address_space(3))) void* d3 = (__attribute__((address_space(3))) void*)dst;
      if (rq >= 32) {
        if (sub * 8 < nrows) __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, d3, 16, (int)goff[i], soff, 0, 0);
      }
      else if (second) __builtin_amdgcn_raw_ptr_buffer_load_lds(rw2, d3, 16, (int)goff[i], soff, 0, 0);
      else __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, d3, 16, (int)goff[i], soff, 0, 0);
    }
  };

  // ---- fragment addresses: lane (i = lane % 32, g = lane / 32) reads row i of a 32-row tile,
  // chunk 2*kk + g of the slab row
  const int li = lane & 31, lg = lane >> 5;
  int foff[4];   // byte offset inside a slab row for the four k-steps, before adding the row
#pragma unroll
  for (int kk = 0; kk < 4; ++kk) foff[kk] = (((2 * kk + lg) ^ ((li >> 1) & 7)) << 4);
  const int wrow = (wn * 128 + li) * 128, xrow = (wm * 128 + li) * 128;

  issue(s_begin, s_begin & 1);
  for (int s = s_begin; s < nslab; ++s) {
    const int buf = s & 1;
    // the slab of this turn has been requested one turn ago: wait for this wavefront's share,
    // then meet the others (their shares are in, and nobody still reads the buffer filled next)
    __builtin_amdgcn_s_waitcnt(0x0070);   // vmcnt(0) lgkmcnt(0)
    __syncthreads();
    if (s + 1 < nslab) issue(s + 1, buf ^ 1);
    const unsigned char* wb = smem + buf * (2 * SLAB);
    const unsigned char* xb = wb + SLAB;
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      h8_t fw[4], fx[4];
#pragma unroll
      for (int a = 0; a < 4; ++a) fw[a] = *(const h8_t*)(wb + wrow + a * 32 * 128 + foff[kk]);
#pragma unroll
      for (int b = 0; b < 4; ++b)
        if (b < nb) fx[b] = *(const h8_t*)(xb + xrow + b * 32 * 128 + foff[kk]);
      // operand order (w, x): result rows = output features, columns = tokens, so each lane ends
      // up with 4 consecutive output features of one token = one 8-byte store
#pragma unroll
      for (int b = 0; b < 4; ++b)
        if (b < nb) {
#pragma unroll
          for (int a = 0; a < 4; ++a)
            acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fw[a], fx[b], acc[a][b], 0, 0, 0);
        }
    }
  }

#pragma unroll
  for (int b = 0; b < 4; ++b) {
    const int pos = row_lo + wm * 128 + b * 32 + li;
    if (pos >= row_hi) continue;
    const int tok = P.perm ? P.perm[pos] : pos;
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      // The accumulators live in the accumulation registers; pinning each block there until its
      // turn keeps the compiler from moving all 256 values to ordinary registers at once (which
      // would push the loop's own values out to scratch memory).
      f16_t blk = acc[a][b];
      asm volatile("" : "+a"(blk));
#pragma unroll
      for (int rq = 0; rq < 4; ++rq) {
        const int n = n0 + wn * 128 + a * 32 + 8 * rq + 4 * lg;
        if (n >= P.N) continue;
        _Float16* yp = P.y + (size_t)tok * P.ldy + n;
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = blk[rq * 4 + e];
        if (P.accumulate) {
          const h4_t o = *(const h4_t*)yp;
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] += (float)o[e];
        }
        const h4_t o = {(_Float16)v[0], (_Float16)v[1], (_Float16)v[2], (_Float16)v[3]};
        *(h4_t*)yp = o;
      }
    }
    __builtin_amdgcn_sched_barrier(0);   // one token block at a time: the rest stays in the accumulators
  }
}

int gemm_launch(GemmParams P, int ntiles_m, void* stream) {
  if (!P.x || (!P.w && !P.w2) || !P.y) return DZ_EINVAL;
  if (P.T < 1 || P.K < 1 || P.N < 1 || P.K % BK || P.N % 4 || P.ldy < P.N || P.ldy % 4 || ntiles_m < 1) return DZ_ESHAPE;
  if (((uintptr_t)P.x & 15) || ((uintptr_t)P.w & 15) || ((uintptr_t)P.w2 & 15) || ((uintptr_t)P.y & 7) ||
      (P.w2 && (P.w2_stride & 7)))
    return DZ_EALIGN;
  if ((unsigned long long)P.T * (unsigned)P.K * 2ull >= (1ull << 31) ||
      (unsigned long long)P.N * (unsigned)P.K * 2ull >= (1ull << 31))
    return DZ_ESHAPE;   // byte offsets inside one operand stay below 2^31 (buffer addressing)
  P.tiles_m = ntiles_m;
  P.tiles_n = (P.N + BN - 1) / BN;
  const int sbm = (P.tiles_m + GM - 1) / GM, sbn = (P.tiles_n + GN - 1) / GN;
  const int nsb = (sbm * sbn + 7) / 8 * 8;
  const unsigned grid = (unsigned)nsb * GM * GN;
  const size_t lds = 2 * 2 * SLAB;
  static std::atomic<unsigned long long> attr_done{0};
  if (!dz_lds_limit_once(attr_done, (const void*)dz_gemm_kernel, (int)lds)) return DZ_ELAUNCH;
  hipLaunchKernelGGL(dz_gemm_kernel, dim3(grid), dim3(256), lds, (hipStream_t)stream, P);
  return hipGetLastError() == hipSuccess ? DZ_OK : DZ_ELAUNCH;
}

GemmParams base_params(const uint16_t* x, const uint16_t* w, uint16_t* y, int T, int K, int N,
                       int accumulate, int ldy) {
  GemmParams P{};
  P.x = (const _Float16*)x; P.w = (const _Float16*)w; P.y = (_Float16*)y;
  P.T = T; P.K = K; P.N = N; P.accumulate = accumulate; P.ldy = ldy;
  return P;
}

}  // namespace

extern "C" int dz_gemm_f16(const uint16_t* x, const uint16_t* w, uint16_t* y, int T, int K, int N,
                           int accumulate, int ldy, void* stream) {
  if (!w) return DZ_EINVAL;
  return gemm_launch(base_params(x, w, y, T, K, N, accumulate, ldy), T < 1 ? 0 : (T + BM - 1) / BM, stream);
}

extern "C" int dz_gemm_f16_pair(const uint16_t* x, const uint16_t* w_a, const uint16_t* w_b, uint16_t* y,
                                int T, int K, int N, int accumulate, int ldy, void* stream) {
  if (!w_a || !w_b) return DZ_EINVAL;
  // one group that spans all rows: the implicit 256-row blocks, all with second weight 0
  GemmParams P = base_params(x, w_a, y, T, K, N, accumulate, ldy);
  P.w2 = (const _Float16*)w_b;
  return gemm_launch(P, T < 1 ? 0 : (T + BM - 1) / BM, stream);
}

extern "C" int dz_gemm_f16_grouped(const uint16_t* x, const uint16_t* w, const uint16_t* w2_stack,
                                   long long w2_stride, const dz_gemm_tile* tiles, int ntiles, uint16_t* y,
                                   int T, int K, int N, int accumulate, int ldy, void* stream) {
  if (!tiles || ntiles < 1) return DZ_EINVAL;
  GemmParams P = base_params(x, w, y, T, K, N, accumulate, ldy);
  P.w2 = (const _Float16*)w2_stack; P.w2_stride = w2_stride; P.tiles = tiles;
  return gemm_launch(P, ntiles, stream);
}

extern "C" int dz_gemm_f16_select(const uint16_t* x, const uint16_t* w_base, const uint16_t* w_stack,
                                  long long w_stride, const dz_gemm_tile* tiles, int ntiles, const int32_t* perm,
                                  uint16_t* y, int T, int K, int N, int accumulate, int ldy, void* stream) {
  if (!tiles || ntiles < 1 || !w_base || !w_stack) return DZ_EINVAL;
  GemmParams P = base_params(x, w_base, y, T, K, N, accumulate, ldy);
  P.w2 = (const _Float16*)w_stack; P.w2_stride = w_stride; P.tiles = tiles; P.perm = perm; P.select = 1;
  return gemm_launch(P, ntiles, stream);
}
