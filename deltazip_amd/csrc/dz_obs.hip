// Hessian-aware compression of a delta: n:m pruning and quantisation, column by column, with the
// error of every column spread over the columns still to come (deltazip/core/sparsegpt.py:25-146).
//
//   dz_hessian_add   H <- H * s0 + (s1 x)^T (s1 x)                         (sparsegpt.py:27-40)
//   dz_obs_sweep     the sweep over blocks of 128 columns                   (sparsegpt.py:92-146)
//
// Rows of the weight are independent given the inverse Hessian, so one wavefront sweeps one row:
// its 128 block columns sit in two registers per lane, the column being processed is broadcast
// with v_readlane, the update of the columns to its right is one multiply and one subtract per
// lane.  Between blocks the accumulated errors are carried to the remaining columns by a tiled
// product.  Every sum runs in ascending index order with one rounding per operation (no fused
// multiply-add), so that the result is the same bit for bit as a plain fp32 restatement with
// that order; speed is secondary here (the sweep runs once per layer, offline).
#include "../../include/dz_amd.h"
#include "dz_device.h"

namespace {

constexpr int OBS_BLOCK = 128;

// ---- H <- H * s0 + sum_t (s1 x[t, a]) * (s1 x[t, b]), t ascending.  64 x 64 outputs per
// workgroup, 4 x 4 per thread, 32 tokens staged at a time.
template <typename XT>
__global__ __launch_bounds__(256) void dz_hessian_kernel(float* __restrict__ H, const XT* __restrict__ x, int T,
                                                         int K, float s0, float s1) {
#pragma clang fp contract(off)
  __shared__ float xa[32][64], xb[32][64];
  const int a0 = blockIdx.y * 64, b0 = blockIdx.x * 64;
  const int tid = threadIdx.x, tr = tid >> 4, tc = tid & 15;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
  for (int t0 = 0; t0 < T; t0 += 32) {
    __syncthreads();
    for (int e = tid; e < 32 * 64; e += 256) {
      const int tt = e >> 6, c = e & 63;
      const bool in = t0 + tt < T;
      xa[tt][c] = in ? s1 * (float)x[(size_t)(t0 + tt) * K + a0 + c] : 0.f;
      xb[tt][c] = in ? s1 * (float)x[(size_t)(t0 + tt) * K + b0 + c] : 0.f;
    }
    __syncthreads();
    const int nt = min(32, T - t0);
    for (int tt = 0; tt < nt; ++tt) {
      float va[4], vb[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        va[i] = xa[tt][tr * 4 + i];
        vb[i] = xb[tt][tc * 4 + i];
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float p = va[i] * vb[j];
          acc[i][j] = acc[i][j] + p;
        }
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float* h = H + (size_t)(a0 + tr * 4 + i) * K + b0 + tc * 4 + j;
      const float scaled = *h * s0;
      *h = scaled + acc[i][j];
    }
}

__device__ __forceinline__ float lane_value(float v, int l) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), l));
}

// ---- one block of 128 columns, one wavefront per row (sparsegpt.py:98-142)
template <bool QUANT>
__global__ __launch_bounds__(256) void dz_obs_block_kernel(float* __restrict__ W, const float* __restrict__ hinv,
                                                           const float* __restrict__ scale, int N, int K, int i1,
                                                           float maxq, float zero, int prunen, int prunem,
                                                           float* __restrict__ err, float* __restrict__ loss) {
#pragma clang fp contract(off)
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  if (row >= N) return;
  float* wr = W + (size_t)row * K + i1;
  float w0 = wr[lane], w1 = wr[64 + lane];
  float q0 = 0.f, q1 = 0.f, e0 = 0.f, e1 = 0.f, lsum = 0.f;
  const float sc = QUANT ? scale[row] : 1.f;
  unsigned pruned_bits = 0;   // bit c: column (start of the current group) + c is pruned
  for (int i = 0; i < OBS_BLOCK; ++i) {
    const float* hr = hinv + (size_t)(i1 + i) * K + i1;
    const float h0 = hr[lane], h1 = hr[64 + lane];
    const int li = i & 63;
    const bool hi = i >= 64;
    if (prunen != 0 && i % prunem == 0) {
      // w^2 / diag^2 of the group's columns (the same half of the block: prunem divides 64); the
      // prunen smallest are pruned, ties keep the lower column (sparsegpt.py:123-125)
      float t[8];
#pragma unroll
      for (int c = 0; c < 8; ++c) {
        t[c] = 0.f;
        if (c < prunem) {
          const float wv = lane_value(hi ? w1 : w0, li + c);
          const float dv = hinv[(size_t)(i1 + i + c) * K + i1 + i + c];
          t[c] = (wv * wv) / (dv * dv);
        }
      }
      pruned_bits = 0;
#pragma unroll
      for (int a = 0; a < 8; ++a) {
        int rank = 0;
#pragma unroll
        for (int b = 0; b < 8; ++b)
          if (a != b && b < prunem) rank += (b > a) ? (t[b] > t[a]) : (t[b] >= t[a]);
        if (a < prunem && rank >= prunem - prunen) pruned_bits |= 1u << a;
      }
    }
    const float w = lane_value(hi ? w1 : w0, li);
    const float d = lane_value(hi ? h1 : h0, li);
    const bool pruned = prunen != 0 && ((pruned_bits >> (i % prunem)) & 1u);
    float q = pruned ? 0.f : w;
    if (QUANT) {
      const float code = fminf(fmaxf(rintf(q / sc) + zero, 0.f), maxq);
      q = sc * (code - zero);
    }
    const float diff = w - q;
    lsum = lsum + (diff * diff) / (d * d);
    const float er = diff / d;
    const float p0 = er * h0, p1 = er * h1;
    if (!hi) {
      if (lane >= li) w0 = w0 - p0;
      w1 = w1 - p1;
      if (lane == li) {
        q0 = q;
        e0 = er;
      }
    } else {
      if (lane >= li) w1 = w1 - p1;
      if (lane == li) {
        q1 = q;
        e1 = er;
      }
    }
  }
  wr[lane] = q0;
  wr[64 + lane] = q1;
  err[(size_t)row * OBS_BLOCK + lane] = e0;
  err[(size_t)row * OBS_BLOCK + 64 + lane] = e1;
  if (lane == 0) loss[row] = loss[row] + lsum / 2.f;
}

// ---- W[:, i2:] -= Err @ hinv[i1:i2, i2:], the sum over the block's 128 columns in ascending
// order (sparsegpt.py:146).  64 rows x 64 columns per workgroup, 4 x 4 per thread.
__global__ __launch_bounds__(256) void dz_obs_propagate_kernel(float* __restrict__ W, const float* __restrict__ err,
                                                               const float* __restrict__ hinv, int N, int K, int i1,
                                                               int i2) {
#pragma clang fp contract(off)
  __shared__ float es[64][OBS_BLOCK], hs[OBS_BLOCK][64];
  const int r0 = blockIdx.y * 64, c0 = i2 + blockIdx.x * 64;
  const int tid = threadIdx.x, tr = tid >> 4, tc = tid & 15;
  for (int e = tid; e < 64 * OBS_BLOCK; e += 256) {
    const int r = e / OBS_BLOCK, k = e % OBS_BLOCK;
    es[r][k] = r0 + r < N ? err[(size_t)(r0 + r) * OBS_BLOCK + k] : 0.f;
  }
  for (int e = tid; e < OBS_BLOCK * 64; e += 256) {
    const int k = e >> 6, c = e & 63;
    hs[k][c] = hinv[(size_t)(i1 + k) * K + c0 + c];
  }
  __syncthreads();
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
  for (int k = 0; k < OBS_BLOCK; ++k) {
    float va[4], vb[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      va[i] = es[tr * 4 + i][k];
      vb[i] = hs[k][tc * 4 + i];
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float p = va[i] * vb[j];
        acc[i][j] = acc[i][j] + p;
      }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = r0 + tr * 4 + i;
    if (r >= N) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float* w = W + (size_t)r * K + c0 + tc * 4 + j;
      *w = *w - acc[i][j];
    }
  }
}

}  // namespace

extern "C" {

int dz_hessian_add(float* H, const void* x, int x_is_fp16, int T, int K, float scale_h, float scale_x,
                   void* stream) {
  if (!H || !x) return DZ_EINVAL;
  if (T < 1 || K < 64 || K % 64) return DZ_ESHAPE;
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid(K / 64, K / 64);
  if (x_is_fp16)
    hipLaunchKernelGGL(dz_hessian_kernel<_Float16>, grid, dim3(256), 0, st, H, (const _Float16*)x, T, K, scale_h,
                       scale_x);
  else
    hipLaunchKernelGGL(dz_hessian_kernel<float>, grid, dim3(256), 0, st, H, (const float*)x, T, K, scale_h,
                       scale_x);
  return hipGetLastError() == hipSuccess ? DZ_OK : DZ_ELAUNCH;
}

int dz_obs_sweep(float* W, const float* hinv_upper, const float* scale, int N, int K, int bits, int prunen,
                 int prunem, float* err_workspace, float* loss, void* stream) {
  if (!W || !hinv_upper || !err_workspace || !loss) return DZ_EINVAL;
  if (N < 1 || K < OBS_BLOCK || K % OBS_BLOCK) return DZ_ESHAPE;
  if (scale && bits != 2 && bits != 3 && bits != 4 && bits != 8) return DZ_EBITS;
  if (prunen < 0 || prunem < 0 || (prunen != 0 && (prunem > 8 || prunen >= prunem || 64 % prunem))) return DZ_ESHAPE;
  hipStream_t st = (hipStream_t)stream;
  const float maxq = (float)((1 << bits) - 1), zero = (float)(1 << (bits - 1));
  for (int i1 = 0; i1 < K; i1 += OBS_BLOCK) {
    const int i2 = i1 + OBS_BLOCK;
    if (scale)
      hipLaunchKernelGGL(dz_obs_block_kernel<true>, dim3((N + 3) / 4), dim3(256), 0, st, W, hinv_upper, scale, N, K,
                         i1, maxq, zero, prunen, prunem, err_workspace, loss);
    else
      hipLaunchKernelGGL(dz_obs_block_kernel<false>, dim3((N + 3) / 4), dim3(256), 0, st, W, hinv_upper, scale, N,
                         K, i1, maxq, zero, prunen, prunem, err_workspace, loss);
    if (i2 < K)
      hipLaunchKernelGGL(dz_obs_propagate_kernel, dim3((K - i2) / 64, (N + 63) / 64), dim3(256), 0, st, W,
                         err_workspace, hinv_upper, N, K, i1, i2);
  }
  return hipGetLastError() == hipSuccess ? DZ_OK : DZ_ELAUNCH;
}

}  // extern "C"
