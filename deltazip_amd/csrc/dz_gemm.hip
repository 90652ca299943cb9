// Dense fp16 GEMM on the gfx950 matrix cores: y[T, N] (+)= x[T, K] @ w[N, K]^T, fp32 accumulate.
// Used for the base product at prefill-sized token counts.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/dz_amd.h"

typedef _Float16 h8_t __attribute__((ext_vector_type(8)));
typedef _Float16 h4_t __attribute__((ext_vector_type(4)));
typedef float f16_t __attribute__((ext_vector_type(16)));

namespace {

// Workgroup tile 128 (tokens) x 128 (outputs), 4 wavefronts in 2 x 2, each 64 x 64 as 2 x 2
// v_mfma_f32_32x32x16_f16 tiles.  Both operands are K-contiguous, so every lane's 8 halves of an
// operand are one 16-byte load.  Tiles are staged through LDS in 64-column slabs.
constexpr int TM = 128, TN = 128, TK = 64;
constexpr int LDS_STRIDE = TK + 8;  // halves; the pad keeps 16-byte row reads off shared banks

// With w2 != nullptr the contraction runs over both weights, y = x @ w^T + x @ w2^T, in the same
// fp32 accumulators (base weight and a dequantised delta, never summed in fp16).
__global__ __launch_bounds__(256) void dz_gemm_kernel(const _Float16* __restrict__ x,
                                                      const _Float16* __restrict__ w,
                                                      const _Float16* __restrict__ w2,
                                                      _Float16* __restrict__ y, int T, int K, int N,
                                                      int accumulate, int ldy) {
  __shared__ __attribute__((aligned(16))) _Float16 sa[TM * LDS_STRIDE];
  __shared__ __attribute__((aligned(16))) _Float16 sb[TN * LDS_STRIDE];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  // XCD-aware tile order: consecutive workgroups land on different XCDs, so give each XCD a
  // contiguous band of token tiles to keep its share of x and w hot in its own L2
  const int tiles_n = N / TN;
  const int tiles_m = (T + TM - 1) / TM;
  const int total = tiles_m * tiles_n;
  const int per_xcd = (total + 7) / 8;
  const int lin = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (lin >= total) return;
  const int tm = lin / tiles_n, tn = lin % tiles_n;
  const int m0 = tm * TM, n0 = tn * TN;

  f16_t acc[2][2];
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;

  const int li = lane & 31, lh = lane >> 5;
  const int npass = w2 ? 2 : 1;
  for (int pass = 0; pass < npass; ++pass) {
  const _Float16* wp = pass ? w2 : w;
  for (int k0 = 0; k0 < K; k0 += TK) {
    // stage: 128 rows x 64 halves per operand = 1024 chunks of 16 bytes, 4 per thread
#pragma unroll
    for (int it = 0; it < 4; ++it) {
      const int c = it * 256 + tid, row = c >> 3, ch = c & 7;
      h8_t va = {0, 0, 0, 0, 0, 0, 0, 0};
      if (m0 + row < T) va = *(const h8_t*)(x + (size_t)(m0 + row) * K + k0 + ch * 8);
      *(h8_t*)(sa + row * LDS_STRIDE + ch * 8) = va;
      const h8_t vb = *(const h8_t*)(wp + (size_t)(n0 + row) * K + k0 + ch * 8);
      *(h8_t*)(sb + row * LDS_STRIDE + ch * 8) = vb;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < TK; kk += 16) {
      h8_t fa[2], fb[2];
#pragma unroll
      for (int a = 0; a < 2; ++a)
        fa[a] = *(const h8_t*)(sa + (wm * 64 + a * 32 + li) * LDS_STRIDE + kk + 8 * lh);
#pragma unroll
      for (int b = 0; b < 2; ++b)
        fb[b] = *(const h8_t*)(sb + (wn * 64 + b * 32 + li) * LDS_STRIDE + kk + 8 * lh);
      // operand order (w, x): result rows = output features, columns = tokens, so each lane
      // ends up with 4 consecutive output features of one token = one 8-byte store
#pragma unroll
      for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b)
          acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[b], fa[a], acc[a][b], 0, 0, 0);
    }
    __syncthreads();
  }
  }
#pragma unroll
  for (int a = 0; a < 2; ++a) {
    const int tok = m0 + wm * 64 + a * 32 + li;
    if (tok >= T) continue;
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int rq = 0; rq < 4; ++rq) {
        const int n = n0 + wn * 64 + b * 32 + 8 * rq + 4 * lh;
        _Float16* yp = y + (size_t)tok * ldy + n;
        float v[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) v[r] = acc[a][b][rq * 4 + r];
        if (accumulate) {
          const h4_t o = *(const h4_t*)yp;
#pragma unroll
          for (int r = 0; r < 4; ++r) v[r] += (float)o[r];
        }
        h4_t o = {(_Float16)v[0], (_Float16)v[1], (_Float16)v[2], (_Float16)v[3]};
        *(h4_t*)yp = o;
      }
  }
}

}  // namespace

static int gemm_launch(const uint16_t* x, const uint16_t* w, const uint16_t* w2, uint16_t* y, int T,
                       int K, int N, int accumulate, int ldy, void* stream) {
  if (!x || !w || !y) return DZ_EINVAL;
  if (T < 1 || K < 1 || N < 1 || K % TK || N % TN || ldy < N || ldy % 4) return DZ_ESHAPE;
  if (((uintptr_t)x & 15) || ((uintptr_t)w & 15) || ((uintptr_t)w2 & 15) || ((uintptr_t)y & 7)) return DZ_EALIGN;
  const int total = ((T + TM - 1) / TM) * (N / TN);
  const int grid = (total + 7) / 8 * 8;
  hipLaunchKernelGGL(dz_gemm_kernel, dim3(grid), dim3(256), 0, (hipStream_t)stream,
                     (const _Float16*)x, (const _Float16*)w, (const _Float16*)w2, (_Float16*)y, T, K, N,
                     accumulate, ldy);
  return hipGetLastError() == hipSuccess ? DZ_OK : DZ_ELAUNCH;
}

extern "C" int dz_gemm_f16(const uint16_t* x, const uint16_t* w, uint16_t* y, int T, int K, int N,
                           int accumulate, int ldy, void* stream) {
  return gemm_launch(x, w, nullptr, y, T, K, N, accumulate, ldy, stream);
}

extern "C" int dz_gemm_f16_pair(const uint16_t* x, const uint16_t* w_a, const uint16_t* w_b, uint16_t* y,
                                int T, int K, int N, int accumulate, int ldy, void* stream) {
  if (!w_b) return DZ_EINVAL;
  return gemm_launch(x, w_a, w_b, y, T, K, N, accumulate, ldy, stream);
}
