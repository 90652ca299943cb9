// gfx950 kernels of the multi-delta linear layer and their C ABI.
//
//   dz_dequant_kernel / merge   native delta -> fp16 [N, K] (bit-exact with the reference's
//                               QuantLinear.unpack, deltazip/nn_modules/qlinear_cuda.py:246-329)
//   dz_segment_kernel           tokens grouped by delta id
// and the host entry points of the C ABI (the fused layer kernel itself is in dz_mdl32.hip).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/dz_amd.h"
#include "../../include/dz_amd_tuning.h"
#include <atomic>

#include "dz_device.h"

namespace {

// ---------------------------------------------------------------------------------------------
// dequant / merge: one wavefront per (n-pair, k-block) tile, transposed through LDS so that the
// fp16 rows leave as 512-byte runs.
// ---------------------------------------------------------------------------------------------
template <int BITS, bool MERGE>
__global__ __launch_bounds__(64) void dz_dequant_kernel(const uint32_t* __restrict__ codes,
                                                        const uint32_t* __restrict__ meta,
                                                        const _Float16* __restrict__ scales,
                                                        const _Float16* __restrict__ wbase,
                                                        _Float16* __restrict__ out, int K, int N,
                                                        int gs) {
  constexpr int LDT = DZ_KBLOCK + 8;  // padded row of the LDS tile, in halves
  __shared__ __attribute__((aligned(16))) _Float16 tile[DZ_NPAIR * LDT];
  const int nkb = K / DZ_KBLOCK;
  const int np = blockIdx.x / nkb, kb = blockIdx.x % nkb;
  const int la = threadIdx.x, ga = la >> 4, i = la & 15;
  const int zp = 1 << (BITS - 1);
  const u4_t m4 = *(const u4_t*)(meta + dz_meta_word(np, kb, la, 0, nkb));
  u4_t c4[2];
  if (BITS == 2) {
    c4[0] = *(const u4_t*)(codes + dz_code2_word(np, kb, la, 0, nkb));
    c4[1] = c4[0];
  } else {
    c4[0] = *(const u4_t*)(codes + dz_code4_word(np, kb, la, 0, 0, nkb));
    c4[1] = *(const u4_t*)(codes + dz_code4_word(np, kb, la, 2, 0, nkb));
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const uint32_t mw = m4[j];
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const int n = np * DZ_NPAIR + 16 * s + i;
      const int g = (kb * DZ_KBLOCK + 64 * j) / gs;
      const float sc = (float)scales[(size_t)g * N + n];
      uint32_t cw;
      if (BITS == 2) cw = c4[0][j];
      else cw = c4[j >> 1][2 * (j & 1) + s];
#pragma unroll
      for (int p = 0; p < 4; ++p) {
        h4_t v = {(_Float16)0.f, (_Float16)0.f, (_Float16)0.f, (_Float16)0.f};
#pragma unroll
        for (int w = 0; w < 2; ++w) {
          const int e = 2 * p + w;
          const int pos = (mw >> dz_meta_shift(s, e)) & 3;
          int q;
          if (BITS == 2) q = (cw >> dz_code2_shift(s, e)) & 3;
          else q = (cw >> dz_code4_shift(e)) & 15;
          // one exact fp32 product, one round-to-nearest-even to fp16
          const _Float16 val = (_Float16)(sc * (float)(q - zp));
          // a kept column whose code is the zero-point must not hide a value already placed
          // (positions are distinct, so plain selects suffice)
          v[0] = pos == 0 ? val : v[0];
          v[1] = pos == 1 ? val : v[1];
          v[2] = pos == 2 ? val : v[2];
          v[3] = pos == 3 ? val : v[3];
        }
        *(h4_t*)(tile + (16 * s + i) * LDT + 64 * j + dz_group_k0(ga, p)) = v;
      }
    }
  }
  __syncthreads();
  // 32 rows x 512 bytes: lane -> (row half, 16-byte chunk)
#pragma unroll
  for (int it = 0; it < 16; ++it) {
    const int row = it * 2 + (la >> 5), ch = la & 31;
    h8_t v = *(const h8_t*)(tile + row * LDT + ch * 8);
    const size_t o = (size_t)(np * DZ_NPAIR + row) * K + kb * DZ_KBLOCK + ch * 8;
    if (MERGE) {
      h8_t b = *(const h8_t*)(wbase + o);
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = (_Float16)((float)b[e] + (float)v[e]);
    }
    *(h8_t*)(out + o) = v;
  }
}

// ---------------------------------------------------------------------------------------------
// segment: stable counting sort of tokens by delta id.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(1024) void dz_segment_kernel(const long long* __restrict__ idx, int T,
                                                          int S, int* __restrict__ perm,
                                                          int* __restrict__ seg_off) {
  // hist[S+2] (exclusive offsets after the scan), running[S+1] (tokens of a key placed by earlier
  // chunks), cnt[16][S+1] (tokens of a key per wavefront of the current chunk)
  extern __shared__ int sm[];
  int* hist = sm;
  int* running = sm + (S + 2);
  int* cnt = running + (S + 1);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int nk = S + 1;
  for (int s = tid; s < S + 2; s += 1024) hist[s] = 0;
  for (int s = tid; s < nk; s += 1024) running[s] = 0;
  __syncthreads();
  for (int t = tid; t < T; t += 1024) {
    long long id = idx[t];
    int key = (id < 0 || id >= S) ? 0 : (int)id + 1;
    atomicAdd(&hist[key + 1], 1);
  }
  __syncthreads();
  if (tid == 0) {
    for (int s = 1; s < S + 2; ++s) hist[s] += hist[s - 1];
  }
  __syncthreads();
  for (int s = tid; s < S + 2; s += 1024) seg_off[s] = hist[s];
  // chunks of 1024 tokens in order; inside a chunk a token's place among equal keys is
  // (tokens of that key in earlier wavefronts) + (in lower lanes of its own wavefront)
  for (int base = 0; base < T; base += 1024) {
    for (int c = tid; c < 16 * nk; c += 1024) cnt[c] = 0;
    __syncthreads();
    const int t = base + tid;
    int key = -1;
    if (t < T) {
      long long id = idx[t];
      key = (id < 0 || id >= S) ? 0 : (int)id + 1;
    }
    int rank = 0;
    unsigned long long todo = __builtin_amdgcn_ballot_w64(key >= 0);
    while (todo) {
      const int k = __builtin_amdgcn_readlane(key, __builtin_ctzll(todo));
      const unsigned long long m = __builtin_amdgcn_ballot_w64(key == k);
      if (key == k) rank = __builtin_popcountll(m & ((1ull << lane) - 1ull));
      if (lane == 0) cnt[wave * nk + k] = __builtin_popcountll(m);
      todo &= ~m;
    }
    __syncthreads();
    if (t < T) {
      int before = 0;
      for (int w = 0; w < wave; ++w) before += cnt[w * nk + key];
      perm[hist[key] + running[key] + before + rank] = t;
    }
    __syncthreads();
    for (int k = tid; k < nk; k += 1024) {
      int tot = 0;
      for (int w = 0; w < 16; ++w) tot += cnt[w * nk + k];
      running[k] += tot;
    }
    __syncthreads();
  }
}

// ---------------------------------------------------------------------------------------------
// delta id -> slot index for every token and every sampled row (the manager's index tensors).
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void dz_map_ids_kernel(const long long* __restrict__ token_ids, int T,
                                                         const long long* __restrict__ prompt_ids, int P,
                                                         const long long* __restrict__ slot_ids, int S,
                                                         long long pad_slot, long long vocab,
                                                         long long extra_vocab,
                                                         long long* __restrict__ base_indices,
                                                         long long* __restrict__ sampler_indices,
                                                         long long* __restrict__ sampler_padded,
                                                         long long* __restrict__ emb_indices, int ld_emb,
                                                         int* __restrict__ n_missing) {
  extern __shared__ long long table[];
  for (int s = threadIdx.x; s < S; s += 256) table[s] = slot_ids[s];
  __syncthreads();
  const int i = blockIdx.x * 256 + threadIdx.x;
  auto find = [&](long long id, bool& missing) -> long long {
    missing = false;
    if (id <= 0) return -1;
    for (int s = 0; s < S; ++s)
      if (table[s] == id) return s;
    missing = true;
    return -1;
  };
  bool miss;
  if (i < T) {
    const long long id = token_ids[i];
    const long long slot = find(id, miss);
    if (miss && n_missing) atomicAdd(n_missing, 1);
    base_indices[i] = slot;
    if (emb_indices) {
      const long long e = id > 0 ? slot : 0;
      long long e0 = e * extra_vocab, e1 = e * (vocab + extra_vocab);
      emb_indices[i] = e0 == -1 ? pad_slot : e0;
      emb_indices[ld_emb + i] = e1 == -1 ? pad_slot : e1;
    }
  }
  if (i < P && sampler_indices) {
    const long long slot = find(prompt_ids[i], miss);
    if (miss && n_missing) atomicAdd(n_missing, 1);
    sampler_indices[i] = slot;
    if (sampler_padded) sampler_padded[i] = (long long)i + (slot == -1 ? pad_slot : slot) * (long long)P;
  }
}

// ---------------------------------------------------------------------------------------------
// embedding rows picked from the base table or from a delta's own table, per token.
// One workgroup per token; 16 bytes per lane and step.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void dz_embedding_select_kernel(const long long* __restrict__ tokens,
                                                                  const long long* __restrict__ idx,
                                                                  const _Float16* __restrict__ base,
                                                                  const _Float16* __restrict__ stack,
                                                                  long long stack_stride, int S, int V,
                                                                  int H, _Float16* __restrict__ out,
                                                                  int ldo) {
  const int t = blockIdx.x;
  const long long tok = tokens[t];
  const long long id = idx[t];
  const _Float16* table = (id >= 0 && id < S) ? stack + id * stack_stride : base;
  u4_t* dst = (u4_t*)(out + (size_t)t * ldo);
  const bool valid = tok >= 0 && tok < V && table != nullptr;
  const u4_t* src = (const u4_t*)(table + (valid ? (size_t)tok * H : 0));
  for (int c = threadIdx.x; c < H / 8; c += 256) {
    u4_t v = {0u, 0u, 0u, 0u};
    if (valid) v = src[c];
    dst[c] = v;
  }
}

// ---------------------------------------------------------------------------------------------
// compressor: fp32 delta [N, K] -> symmetric scales, 2:4 magnitude pruning, codes, native layout
// ---------------------------------------------------------------------------------------------
// One wavefront per (row, scale group): min / max of the group, then the symmetric parameters of
// deltazip/core/quant.py:69-83 (perchannel, sym): the range is widened to [-m, m] when the group
// has a negative value, an all-zero group gets [-1, 1], scale = (xmax - xmin) / maxq.
__global__ __launch_bounds__(64) void dz_scales_kernel(const float* __restrict__ delta, int K, int N, int gs,
                                                       int G, float maxq, float* __restrict__ scale32,
                                                       _Float16* __restrict__ scale16) {
  const int row = blockIdx.x / G, g = blockIdx.x % G, lane = threadIdx.x;
  const float* p = delta + (size_t)row * K + (size_t)g * gs;
  float mn = 0.f, mx = 0.f;
  for (int c = lane * 4; c < gs; c += 256) {
    const f4_t v = *(const f4_t*)(p + c);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      mn = fminf(mn, v[e]);
      mx = fmaxf(mx, v[e]);
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    mn = fminf(mn, __shfl_xor(mn, o));
    mx = fmaxf(mx, __shfl_xor(mx, o));
  }
  if (lane == 0) {
    float xmin = mn, xmax = fmaxf(fabsf(mn), mx);
    if (xmin < 0.f) xmin = -xmax;
    if (xmin == 0.f && xmax == 0.f) {
      xmin = -1.f;
      xmax = 1.f;
    }
    const float sc = (xmax - xmin) / maxq;
    scale32[(size_t)g * N + row] = sc;
    scale16[(size_t)g * N + row] = (_Float16)sc;
  }
}

// The same with the reference's grid search over the clipping range (deltazip/core/quant.py:85-101,
// mse=True, sym): for i = 0 .. int(maxshrink * grid) - 1 the range is shrunk by p = 1 - i / grid,
// the group is rounded to that grid and the candidate with the smallest sum of |q(x) - x|^norm
// wins (the first one on a tie: `err < best`).  One wavefront per (row, scale group); the group
// is re-read from cache for every candidate; sums: fp32 per lane in element order, then a
// butterfly over the lanes.
__global__ __launch_bounds__(64) void dz_scales_mse_kernel(const float* __restrict__ delta, int K, int N, int gs,
                                                           int G, float maxq, float norm, int grid, int ncand,
                                                           float* __restrict__ scale32,
                                                           _Float16* __restrict__ scale16) {
  const int row = blockIdx.x / G, g = blockIdx.x % G, lane = threadIdx.x;
  const float* p = delta + (size_t)row * K + (size_t)g * gs;
  float mn = 0.f, mx = 0.f;
  for (int c = lane * 4; c < gs; c += 256) {
    const f4_t v = *(const f4_t*)(p + c);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      mn = fminf(mn, v[e]);
      mx = fmaxf(mx, v[e]);
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    mn = fminf(mn, __shfl_xor(mn, o));
    mx = fmaxf(mx, __shfl_xor(mx, o));
  }
  float xmin = mn, xmax = fmaxf(fabsf(mn), mx);
  if (xmin < 0.f) xmin = -xmax;
  if (xmin == 0.f && xmax == 0.f) {
    xmin = -1.f;
    xmax = 1.f;
  }
  const float zero = (maxq + 1.f) * 0.5f;
  float best = INFINITY, best_scale = (xmax - xmin) / maxq;
  for (int i = 0; i < ncand; ++i) {
    const float pf = (float)(1.0 - (double)i / (double)grid);
    const float sc = __fsub_rn(__fmul_rn(pf, xmax), __fmul_rn(pf, xmin)) / maxq;   // every product rounded, as the reference's tensor ops
    float err = 0.f;
    for (int c = lane * 4; c < gs; c += 256) {
      const f4_t v = *(const f4_t*)(p + c);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float q = fminf(fmaxf(rintf(v[e] / sc) + zero, 0.f), maxq);
        err += powf(fabsf(__fsub_rn(__fmul_rn(sc, q - zero), v[e])), norm);
      }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) err += __shfl_xor(err, o);
    if (err < best) {
      best = err;
      best_scale = sc;
    }
  }
  if (lane == 0) {
    scale32[(size_t)g * N + row] = best_scale;
    scale16[(size_t)g * N + row] = (_Float16)best_scale;
  }
}

// One wavefront per (n-pair, k-block) tile; lane 16*ga + i produces its own four words of the
// native arrays from rows i and 16 + i, columns 64*j + 16*ga .. + 15 of the k-block.
//   pruning   in every aligned group of 4 columns the 2 values of largest magnitude stay (ties:
//             the lower column), the others become 0 -- deltazip/core/sparsegpt.py:123-135 with an
//             identity Hessian
//   codes     q = clamp(rint(x / scale) + zero, 0, maxq), fp32, zero = 2^(bits-1) -- quant.py:9-18
//   positions the columns whose code differs from the zero-point, completed with the lowest
//             remaining columns: what the repacker stores for the same codes
template <int BITS>
__global__ __launch_bounds__(64) void dz_compress_kernel(const float* __restrict__ delta,
                                                         const float* __restrict__ scale32, int K, int N,
                                                         int gs, uint32_t* __restrict__ codes,
                                                         uint32_t* __restrict__ meta) {
  const int nkb = K / DZ_KBLOCK;
  const int np = blockIdx.x / nkb, kb = blockIdx.x % nkb;
  const int la = threadIdx.x, ga = la >> 4, i = la & 15;
  constexpr int zp = 1 << (BITS - 1);
  constexpr float maxq = (float)((1 << BITS) - 1);
  uint32_t mword[4] = {0u, 0u, 0u, 0u};
  uint32_t cword[2][4] = {{0u, 0u, 0u, 0u}, {0u, 0u, 0u, 0u}};
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int col0 = kb * DZ_KBLOCK + 64 * j + 16 * ga;
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const int row = np * DZ_NPAIR + 16 * s + i;
      const float sc = scale32[(size_t)(col0 / gs) * N + row];
      const float* src = delta + (size_t)row * K + col0;
#pragma unroll
      for (int p = 0; p < 4; ++p) {
        const f4_t v = *(const f4_t*)(src + 4 * p);
        int c[4];
#pragma unroll
        for (int a = 0; a < 4; ++a) {
          int rank = 0;   // entries ahead of a: larger magnitude, or equal magnitude at a lower column
#pragma unroll
          for (int b = 0; b < 4; ++b)
            if (b != a) rank += (b > a) ? (fabsf(v[b]) > fabsf(v[a])) : (fabsf(v[b]) >= fabsf(v[a]));
          const float x = rank < 2 ? v[a] : 0.f;
          const float qf = fminf(fmaxf(rintf(x / sc) + (float)zp, 0.f), maxq);
          c[a] = (int)qf;
        }
        int pa = -1, pb = -1;
#pragma unroll
        for (int a = 0; a < 4; ++a)
          if (c[a] != zp) {
            if (pa < 0) pa = a;
            else if (pb < 0) pb = a;
          }
#pragma unroll
        for (int a = 0; a < 4; ++a)
          if (c[a] == zp) {
            if (pa < 0) pa = a;
            else if (pb < 0) pb = a;
          }
        const int lo = min(pa, pb), hi = max(pa, pb);
        const uint32_t clo = (uint32_t)(lo == 0 ? c[0] : lo == 1 ? c[1] : c[2]);
        const uint32_t chi = (uint32_t)(hi == 1 ? c[1] : hi == 2 ? c[2] : c[3]);
        mword[j] |= ((uint32_t)lo << dz_meta_shift(s, 2 * p)) | ((uint32_t)hi << dz_meta_shift(s, 2 * p + 1));
        if (BITS == 2) {
          cword[0][j] |= (clo << dz_code2_shift(s, 2 * p)) | (chi << dz_code2_shift(s, 2 * p + 1));
        } else {
          cword[j >> 1][2 * (j & 1) + s] |= (clo << dz_code4_shift(2 * p)) | (chi << dz_code4_shift(2 * p + 1));
        }
      }
    }
  }
  *(u4_t*)(meta + dz_meta_word(np, kb, la, 0, nkb)) = (u4_t){mword[0], mword[1], mword[2], mword[3]};
  if (BITS == 2) {
    *(u4_t*)(codes + dz_code2_word(np, kb, la, 0, nkb)) = (u4_t){cword[0][0], cword[0][1], cword[0][2], cword[0][3]};
  } else {
    *(u4_t*)(codes + dz_code4_word(np, kb, la, 0, 0, nkb)) = (u4_t){cword[0][0], cword[0][1], cword[0][2], cword[0][3]};
    *(u4_t*)(codes + dz_code4_word(np, kb, la, 2, 0, nkb)) = (u4_t){cword[1][0], cword[1][1], cword[1][2], cword[1][3]};
  }
}

// ---------------------------------------------------------------------------------------------
// 33..128 tokens: the order in which the fused kernel takes the tokens, 32 per chunk.  Tokens of
// one delta stay together, and the chunks are made to meet about the same number of distinct
// deltas (the kernel's time per chunk grows with that number; a plain cut of the id-sorted order
// puts one popular delta alone into a chunk and all the rare ones together into another).
// The segments -- one per delta present -- are ranked by size; counting from the largest, segment
// r goes to group r mod nchunk; the groups are laid out one after the other, each smallest
// segment first, and the chunks are the 32-token cuts of that layout.  Every group holds the same
// number of segments and group g is at least as long as group g + 1, so a cut falls into the tail
// of a group: what spills into the next chunk is part of a popular delta, not several rare ones.
// One workgroup, one thread per token, everything by counting over the (at most 128) tokens: no
// per-slot table, so any number of slots is fine.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(128) void dz_deal_kernel(const long long* __restrict__ idx, int T, int S,
                                                      int* __restrict__ perm_out) {
  __shared__ __attribute__((aligned(16))) int s_key[128], s_size[128], s_dkey[128];
  __shared__ int s_pos[128], s_wcount[2];
  const int tid = threadIdx.x;
  const int nchunk = (T + 31) / 32;
  int key = 0x7fffffff;   // threads beyond T hold no token; their entries never match or count
  if (tid < T) {
    const long long id = idx[tid];
    key = (id < 0 || id >= S) ? 0 : (int)id + 1;
  }
  s_key[tid] = key;
  __syncthreads();
  // Tables are read four entries per LDS read with several reads in flight (a loop that takes one
  // entry per turn waits out the LDS latency every time).
  typedef int i4_t __attribute__((ext_vector_type(4)));
  // my segment: its size, my place in it, its first token (the segment's "leader")
  int size = 0, rin = 0, leader = tid;
#pragma unroll 8
  for (int q = 0; q < 32; ++q) {
    const i4_t v = ((const i4_t*)s_key)[q];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int j = 4 * q + e;
      const bool same = v[e] == key;
      size += same;
      rin += same && j < tid;
      leader = (same && j < leader) ? j : leader;
    }
  }
  const bool is_leader = tid < T && leader == tid;
  // the segments, compacted (order of their first tokens): size | first token << 8; zero-padded
  const unsigned long long lm = __builtin_amdgcn_ballot_w64(is_leader);
  const int lane = tid & 63, wave = tid >> 6;
  if (lane == 0) s_wcount[wave] = __builtin_popcountll(lm);
  s_size[tid] = 0;
  s_dkey[tid] = 0x7fffffff;
  __syncthreads();
  const int nseg = s_wcount[0] + s_wcount[1];
  const int slot = (wave ? s_wcount[0] : 0) + __builtin_popcountll(lm & ((1ull << lane) - 1ull));
  if (is_leader) s_size[slot] = size | (tid << 8);
  __syncthreads();
  const int nq = (nseg + 3) >> 2;
  // leaders: rank of the segment by (size, first token)
  int rank = 0;
  for (int q = 0; q < nq; ++q) {
    const i4_t v = ((const i4_t*)s_size)[q];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int sj = v[e] & 0xff, fj = v[e] >> 8;
      rank += v[e] != 0 && (sj < size || (sj == size && fj < tid));
    }
  }
  const int dkey = is_leader ? ((((nseg - 1 - rank) % nchunk) << 16) | rank) : 0x7fffffff;
  if (is_leader) s_dkey[slot] = dkey;
  __syncthreads();
  int pos = 0;   // tokens of the segments laid out before mine
  for (int q = 0; q < nq; ++q) {
    const i4_t d = ((const i4_t*)s_dkey)[q];
    const i4_t z = ((const i4_t*)s_size)[q];
#pragma unroll
    for (int e = 0; e < 4; ++e) pos += (d[e] < dkey) ? (z[e] & 0xff) : 0;
  }
  s_pos[tid] = pos;
  __syncthreads();
  if (tid < T) perm_out[s_pos[leader] + rin] = tid;
}

// Base weight, row-major [N, K] -> tiles (dz_layout.h: dz_base_tile_offset / dz_base_frag_offset).
// One thread moves 16 bytes: output chunk c = ((tile * 16 + fragment) * 64 + lane).
__global__ __launch_bounds__(256) void dz_tile_base_kernel(const u4_t* __restrict__ w, u4_t* __restrict__ out,
                                                           int K, int N) {
  const long long c = (long long)blockIdx.x * 256 + threadIdx.x;
  if (c >= (long long)N * K / 8) return;
  const int lane = (int)(c & 63), frag = (int)((c >> 6) & 15);
  const long long tile = c >> 10;
  const int nkb = K / DZ_KBLOCK;
  const int np = (int)(tile / nkb), kb = (int)(tile % nkb);
  const int h = frag & 1, j = (frag >> 1) & 3, s = frag >> 3;
  const int i = lane & 15, g = lane >> 4;
  const long long row = (long long)np * DZ_NPAIR + 16 * s + i;
  const int col = kb * DZ_KBLOCK + 64 * j + 16 * g + 8 * h;
  out[c] = w[(row * K + col) / 8];
}

// ---------------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------------
// K-slice override of the tuning hook (include/dz_amd_tuning.h): per host thread, so that a test
// or a sweep that sets it changes no other caller's launches
thread_local int g_ksplit_override = 0;

inline int check_group(int K, int group_size, int* gs_out) {
  int gs = (group_size == -1 || group_size == K) ? K : group_size;
  if (gs <= 0 || K % gs || (gs != K && gs % 64)) return DZ_EGROUP;
  *gs_out = gs;
  return DZ_OK;
}

constexpr size_t WS_HEADER = 256;  // status word
constexpr int MAX_KSPLIT = 16;
constexpr size_t WS_PERM_BYTES = 4096 + (size_t)DZ_MAX_TOKENS_FUSED * 4;   // reserved + token order

// Workspace of dz_multi_delta_linear_static: device memory that belongs to the library's code
// object (zero bits when the object is loaded; every GPU holds its own copy at its own address).
// Host code must not use the array's name as an address: it asks the runtime for the device
// address once per device (static_scratch_ptr) and passes that on.
constexpr size_t STATIC_SCRATCH_BYTES =
    WS_HEADER + WS_PERM_BYTES + (size_t)MAX_KSPLIT * 32 * (size_t)DZ_STATIC_MAX_N * 4;
static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];

constexpr int MAX_DEVICES = 64;
std::atomic<void*> g_scratch_ptr[MAX_DEVICES];

// Device address of `scratch` on the current device, looked up on the first call per device.
void* static_scratch_ptr() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return nullptr;
  void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (p) return p;
  if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return nullptr;
  g_scratch_ptr[dev].store(p, std::memory_order_release);   // two racing threads store the same address
  return p;
}

}  // namespace

extern "C" {

#ifdef DZ_TIMING
void dz_set_timing_buffer(void* p) { hipMemcpyToSymbol(HIP_SYMBOL(g_dz_ts), &p, sizeof(p)); }
#endif

int dz_version(void) { return 100; }

const char* dz_strerror(int code) {
  switch (code) {
    case DZ_OK: return "ok";
    case DZ_EINVAL: return "invalid argument";
    case DZ_ESHAPE: return "unsupported shape (need K % 256 == 0, N % 32 == 0, ldy % 4 == 0, T >= 1)";
    case DZ_EBITS: return "bits must be 2 or 4";
    case DZ_EGROUP: return "group_size must be -1, K, or a multiple of 64 dividing K";
    case DZ_ENOT24: return "delta is not 2:4 sparse";
    case DZ_EZERO: return "zero-point is not 2^(bits-1) (only symmetric quantisation is supported)";
    case DZ_EGIDX: return "g_idx is not k / group_size";
    case DZ_EWORKSPACE: return "workspace missing or too small";
    case DZ_ELAUNCH: return "HIP launch failed";
    case DZ_EALIGN: return "pointer or leading dimension not aligned";
    case DZ_ESTATICMAX: return "N exceeds DZ_STATIC_MAX_N, the largest layer the library's built-in workspace serves";
    default: return "unknown error";
  }
}

void dz_set_ksplit(int nsplit) { g_ksplit_override = nsplit; }

int dz_dequant(const void* codes, const void* meta, const void* scales, int K, int N, int bits,
               int group_size, uint16_t* out, void* stream) {
  if (!codes || !meta || !scales || !out) return DZ_EINVAL;
  int rc = dz_native_sizes(K, N, bits, group_size, nullptr, nullptr, nullptr);
  if (rc) return rc;
  int gs;
  if ((rc = check_group(K, group_size, &gs))) return rc;
  const int grid = (N / DZ_NPAIR) * (K / DZ_KBLOCK);
  hipStream_t st = (hipStream_t)stream;
  if (bits == 2)
    hipLaunchKernelGGL((dz_dequant_kernel<2, false>), dim3(grid), dim3(64), 0, st, (const uint32_t*)codes,
                       (const uint32_t*)meta, (const _Float16*)scales, nullptr, (_Float16*)out, K, N, gs);
  else
    hipLaunchKernelGGL((dz_dequant_kernel<4, false>), dim3(grid), dim3(64), 0, st, (const uint32_t*)codes,
                       (const uint32_t*)meta, (const _Float16*)scales, nullptr, (_Float16*)out, K, N, gs);
  return hipGetLastError() == hipSuccess ? DZ_OK : DZ_ELAUNCH;
}

int dz_merge(const uint16_t* w_base, const void* codes, const void* meta, const void* scales, int K,
             int N, int bits, int group_size, uint16_t* out, void* stream) {
  if (!w_base || !codes || !meta || !scales || !out) return DZ_EINVAL;
  int rc = dz_native_sizes(K, N, bits, group_size, nullptr, nullptr, nullptr);
  if (rc) return rc;
  int gs;
  if ((rc = check_group(K, group_size, &gs))) return rc;
  const int grid = (N / DZ_NPAIR) * (K / DZ_KBLOCK);
  hipStream_t st = (hipStream_t)stream;
  if (bits == 2)
    hipLaunchKernelGGL((dz_dequant_kernel<2, true>), dim3(grid), dim3(64), 0, st, (const uint32_t*)codes,
                       (const uint32_t*)meta, (const _Float16*)scales, (const _Float16*)w_base,
                       (_Float16*)out, K, N, gs);
  else
    hipLaunchKernelGGL((dz_dequant_kernel<4, true>), dim3(grid), dim3(64), 0, st, (const uint32_t*)codes,
                       (const uint32_t*)meta, (const _Float16*)scales, (const _Float16*)w_base,
                       (_Float16*)out, K, N, gs);
  return hipGetLastError() == hipSuccess ? DZ_OK : DZ_ELAUNCH;
}

int dz_segment(const int64_t* indices, int T, int S, int32_t* perm, int32_t* seg_off, void* stream) {
  if (!indices || !perm || !seg_off) return DZ_EINVAL;
  if (T < 1 || S < 0 || S > DZ_MAX_SLOTS_SEGMENT) return DZ_ESHAPE;
  const size_t lds = (size_t)((S + 2) + (S + 1) + 16 * (S + 1)) * 4;   // < 64 KiB
  hipLaunchKernelGGL(dz_segment_kernel, dim3(1), dim3(1024), lds, (hipStream_t)stream,
                     (const long long*)indices, T, S, perm, seg_off);
  return hipGetLastError() == hipSuccess ? DZ_OK : DZ_ELAUNCH;
}

int dz_map_ids(const int64_t* token_ids, int T, const int64_t* prompt_ids, int P,
               const int64_t* slot_ids, int S, int max_deltas, int vocab_size, int extra_vocab_size,
               int64_t* base_indices, int64_t* sampler_indices, int64_t* sampler_indices_padded,
               int64_t* embeddings_indices, int ld_emb, int32_t* n_missing, void* stream) {
  if (!token_ids || !slot_ids || !base_indices) return DZ_EINVAL;
  if (P > 0 && (!prompt_ids || !sampler_indices)) return DZ_EINVAL;
  if (T < 1 || P < 0 || S < 1 || S > DZ_MAX_SLOTS_MAP || max_deltas < 1) return DZ_ESHAPE;
  if (embeddings_indices && ld_emb < T) return DZ_ESHAPE;
  const int n = T > P ? T : P;
  hipLaunchKernelGGL(dz_map_ids_kernel, dim3((n + 255) / 256), dim3(256), (size_t)S * 8,
                     (hipStream_t)stream, (const long long*)token_ids, T, (const long long*)prompt_ids,
                     P, (const long long*)slot_ids, S, (long long)max_deltas - 1, (long long)vocab_size,
                     (long long)extra_vocab_size, (long long*)base_indices, (long long*)sampler_indices,
                     (long long*)sampler_indices_padded, (long long*)embeddings_indices, ld_emb, n_missing);
  return hipGetLastError() == hipSuccess ? DZ_OK : DZ_ELAUNCH;
}

int dz_embedding_select(const int64_t* tokens, const int64_t* indices, const uint16_t* base_weight,
                        const uint16_t* weight_stack, long long stack_stride, int S, uint16_t* out, int T,
                        int V, int H, int ldo, void* stream) {
  if (!tokens || !indices || !out || (!base_weight && !weight_stack)) return DZ_EINVAL;
  if (T < 1 || V < 1 || H < 8 || H % 8 || ldo < H || ldo % 8 || S < 0 || (S > 0 && !weight_stack)) return DZ_ESHAPE;
  if (((uintptr_t)base_weight & 15) || ((uintptr_t)weight_stack & 15) || ((uintptr_t)out & 15) ||
      (stack_stride & 7))
    return DZ_EALIGN;
  hipLaunchKernelGGL(dz_embedding_select_kernel, dim3(T), dim3(256), 0, (hipStream_t)stream,
                     (const long long*)tokens, (const long long*)indices, (const _Float16*)base_weight,
                     (const _Float16*)weight_stack, stack_stride, S, V, H, (_Float16*)out, ldo);
  return hipGetLastError() == hipSuccess ? DZ_OK : DZ_ELAUNCH;
}

int dz_compress_2of4(const float* delta, int K, int N, int bits, int group_size, void* out_codes,
                     void* out_meta, uint16_t* out_scales, float* scale_workspace, void* stream) {
  if (!delta || !out_codes || !out_meta || !out_scales || !scale_workspace) return DZ_EINVAL;
  size_t cb, mb, sb;
  int rc = dz_native_sizes(K, N, bits, group_size, &cb, &mb, &sb);
  if (rc) return rc;
  int gs;
  if ((rc = check_group(K, group_size, &gs))) return rc;
  if ((uintptr_t)delta & 15) return DZ_EALIGN;
  const int G = K / gs;
  hipStream_t st = (hipStream_t)stream;
  hipLaunchKernelGGL(dz_scales_kernel, dim3((unsigned)N * G), dim3(64), 0, st, delta, K, N, gs, G,
                     (float)((1 << bits) - 1), scale_workspace, (_Float16*)out_scales);
  const unsigned tiles = (unsigned)(N / DZ_NPAIR) * (K / DZ_KBLOCK);
  if (bits == 2)
    hipLaunchKernelGGL(dz_compress_kernel<2>, dim3(tiles), dim3(64), 0, st, delta, scale_workspace, K, N, gs,
                       (uint32_t*)out_codes, (uint32_t*)out_meta);
  else
    hipLaunchKernelGGL(dz_compress_kernel<4>, dim3(tiles), dim3(64), 0, st, delta, scale_workspace, K, N, gs,
                       (uint32_t*)out_codes, (uint32_t*)out_meta);
  return hipGetLastError() == hipSuccess ? DZ_OK : DZ_ELAUNCH;
}

int dz_quant_scales(const float* delta, int K, int N, int bits, int group_size, float* scale32,
                    uint16_t* scale16, void* stream) {
  if (!delta || !scale32 || !scale16) return DZ_EINVAL;
  int rc = dz_native_sizes(K, N, bits, group_size, nullptr, nullptr, nullptr);
  if (rc) return rc;
  int gs;
  if ((rc = check_group(K, group_size, &gs))) return rc;
  if ((uintptr_t)delta & 15) return DZ_EALIGN;
  const int G = K / gs;
  hipLaunchKernelGGL(dz_scales_kernel, dim3((unsigned)N * G), dim3(64), 0, (hipStream_t)stream, delta, K, N, gs, G,
                     (float)((1 << bits) - 1), scale32, (_Float16*)scale16);
  return hipGetLastError() == hipSuccess ? DZ_OK : DZ_ELAUNCH;
}

int dz_quant_scales_mse(const float* delta, int K, int N, int bits, int group_size, float norm, int grid,
                        float maxshrink, float* scale32, uint16_t* scale16, void* stream) {
  if (!delta || !scale32 || !scale16) return DZ_EINVAL;
  if (!(norm > 0.f) || grid < 1 || !(maxshrink >= 0.f) || maxshrink > 1.f) return DZ_EINVAL;
  int rc = dz_native_sizes(K, N, bits, group_size, nullptr, nullptr, nullptr);
  if (rc) return rc;
  int gs;
  if ((rc = check_group(K, group_size, &gs))) return rc;
  if ((uintptr_t)delta & 15) return DZ_EALIGN;
  const int G = K / gs;
  const int ncand = (int)((double)maxshrink * (double)grid);   // int(maxshrink * grid), quant.py:87
  hipLaunchKernelGGL(dz_scales_mse_kernel, dim3((unsigned)N * G), dim3(64), 0, (hipStream_t)stream, delta, K, N, gs,
                     G, (float)((1 << bits) - 1), norm, grid, ncand, scale32, (_Float16*)scale16);
  return hipGetLastError() == hipSuccess ? DZ_OK : DZ_ELAUNCH;
}

int dz_pack_2of4(const float* w, const float* scale32, int K, int N, int bits, int group_size, void* out_codes,
                 void* out_meta, void* stream) {
  if (!w || !scale32 || !out_codes || !out_meta) return DZ_EINVAL;
  int rc = dz_native_sizes(K, N, bits, group_size, nullptr, nullptr, nullptr);
  if (rc) return rc;
  int gs;
  if ((rc = check_group(K, group_size, &gs))) return rc;
  if ((uintptr_t)w & 15) return DZ_EALIGN;
  const unsigned tiles = (unsigned)(N / DZ_NPAIR) * (K / DZ_KBLOCK);
  hipStream_t st = (hipStream_t)stream;
  if (bits == 2)
    hipLaunchKernelGGL(dz_compress_kernel<2>, dim3(tiles), dim3(64), 0, st, w, scale32, K, N, gs,
                       (uint32_t*)out_codes, (uint32_t*)out_meta);
  else
    hipLaunchKernelGGL(dz_compress_kernel<4>, dim3(tiles), dim3(64), 0, st, w, scale32, K, N, gs,
                       (uint32_t*)out_codes, (uint32_t*)out_meta);
  return hipGetLastError() == hipSuccess ? DZ_OK : DZ_ELAUNCH;
}

// workspace: [status 256 B][token order][per call: partial sums].  The partial-sum slots are
// their own "ready" marks (all zero bits = empty) and every launch leaves them empty again, so the
// workspace is zero-filled once by its owner and never again.
size_t dz_workspace_bytes(int T, int K, int N) {
  (void)K;
  if (T < 1 || N < 1) return 0;
  return WS_HEADER + WS_PERM_BYTES + (size_t)MAX_KSPLIT * 32 * (size_t)N * 4;
}

static int multi_delta_linear_batch(int ncalls, const uint16_t* const* x, const uint16_t* const* w_base,
                                    const void* const* codes_stacked, const void* const* meta_stacked,
                                    const void* const* scales_stacked, const int64_t* indices,
                                    uint16_t* const* y, const int* N, const int* ldy, int T, int K, int S,
                                    int bits, int group_size, int accumulate, const int32_t* order,
                                    void* workspace, size_t workspace_bytes, void* stream, int base_tiled) {
  if (ncalls < 1 || ncalls > DZ_MAX_BATCH_CALLS) return DZ_ESHAPE;
  if (!x || !w_base || !indices || !y || !N || !ldy) return DZ_EINVAL;
  if (S > 0 && (!codes_stacked || !meta_stacked || !scales_stacked)) return DZ_EINVAL;
  const void* const none[DZ_MAX_BATCH_CALLS] = {nullptr, nullptr, nullptr, nullptr};
  if (S == 0) codes_stacked = meta_stacked = scales_stacked = none;
  if (S < 0) return DZ_EINVAL;
  if (T < 1 || T > DZ_MAX_TOKENS_FUSED) return DZ_ESHAPE;
  int gs, rc;
  if ((rc = check_group(K, group_size, &gs))) return rc;
  long long n_total = 0;
  for (int j = 0; j < ncalls; ++j) {
    size_t cb, mb, sb;
    if ((rc = dz_native_sizes(K, N[j], bits, group_size, &cb, &mb, &sb))) return rc;
    if (!x[j] || !y[j]) return DZ_EINVAL;
    // S = 0: a plain dense product with the base weight (every id counts as "no delta")
    if (S == 0 ? !w_base[j] : (!codes_stacked[j] || !meta_stacked[j] || !scales_stacked[j])) return DZ_EINVAL;
    if (ldy[j] < N[j] || ldy[j] % 4) return DZ_ESHAPE;
    if (((uintptr_t)x[j] & 15) || ((uintptr_t)y[j] & 7) || (w_base[j] && ((uintptr_t)w_base[j] & 15))) return DZ_EALIGN;
    n_total += N[j];
  }
  if (!workspace || workspace_bytes < dz_workspace_bytes(T, K, (int)n_total)) return DZ_EWORKSPACE;

  hipStream_t st = (hipStream_t)stream;
  int* perm = (int*)((char*)workspace + WS_HEADER) + 1024;
  char* region = (char*)workspace + WS_HEADER + WS_PERM_BYTES;
  MdlParams P[DZ_MAX_BATCH_CALLS];
  for (int j = 0; j < ncalls; ++j) {
    size_t cb, mb, sb;
    dz_native_sizes(K, N[j], bits, group_size, &cb, &mb, &sb);
    MdlParams& Q = P[j];
    Q.x = (const _Float16*)x[j];
    Q.wb = (const _Float16*)w_base[j];
    // The kernel issues a fixed number of requests per round; those of absent deltas re-read 16
    // bytes of slot 0.  Without slots they re-read the base weight instead (offsets stay inside
    // it: a tile index times 1 or 2 KiB is below N*K/4 bytes, the weight has 2*N*K).
    Q.codes = (const u4_t*)(S == 0 ? (const void*)w_base[j] : codes_stacked[j]);
    Q.meta = (const u4_t*)(S == 0 ? (const void*)w_base[j] : meta_stacked[j]);
    Q.scales = (const _Float16*)(S == 0 ? (const void*)w_base[j] : scales_stacked[j]);
    Q.idx = (const long long*)indices;
    Q.y = (_Float16*)y[j];
    Q.status = (unsigned*)workspace;
    Q.partials = (float*)region;
    region += (size_t)MAX_KSPLIT * 32 * (size_t)N[j] * 4;
    Q.codes_slot_u4 = (long long)(cb / 16);
    Q.meta_slot_u4 = (long long)(mb / 16);
    Q.scales_slot = (long long)(sb / 2);
    Q.T = T; Q.K = K; Q.N = N[j]; Q.S = S; Q.gs = gs; Q.G = K / gs;
    Q.accumulate = accumulate; Q.ldy = ldy[j];
    Q.NP = N[j] / DZ_NPAIR; Q.NKB = K / DZ_KBLOCK;
    Q.nsplit = 1; Q.cb = Q.NKB; Q.NPG = 0;
    Q.base_tiled = (base_tiled && w_base[j]) ? 1 : 0;
    Q.perm = T <= 32 ? nullptr : (order ? order : perm);
    Q.tok0 = 0;
    Q.nchunk = 1;
  }
  // 0: 2-bit, one scale per row (applied to the sums); else scales applied to the operands, with
  // one request (a k-block spans at most two groups) or two (groups of 64) per delta and k-block
  const int pre = (bits == 2 && gs == K) ? 0 : (gs >= 128 ? 1 : 2);
  // 33..128 tokens: group the tokens by delta id on the device (no host round trip) and deal the
  // groups to the chunks of 32; one launch carries all chunks
  if (T > 32 && !order)
    hipLaunchKernelGGL(dz_deal_kernel, dim3(1), dim3(128), 0, st, (const long long*)indices, T, S, perm);
  return dz_launch_mdl32_batch(P, ncalls, bits, pre, st, g_ksplit_override);
}

int dz_multi_delta_linear_batch(int ncalls, const uint16_t* const* x, const uint16_t* const* w_base,
                                const void* const* codes_stacked, const void* const* meta_stacked,
                                const void* const* scales_stacked, const int64_t* indices,
                                uint16_t* const* y, const int* N, const int* ldy, int T, int K, int S,
                                int bits, int group_size, int accumulate, const int32_t* order,
                                void* workspace, size_t workspace_bytes, void* stream) {
  return multi_delta_linear_batch(ncalls, x, w_base, codes_stacked, meta_stacked, scales_stacked, indices, y, N, ldy,
                                  T, K, S, bits, group_size, accumulate, order, workspace, workspace_bytes, stream, 0);
}

int dz_multi_delta_linear_batch_tiled(int ncalls, const uint16_t* const* x, const uint16_t* const* w_base_tiled,
                                      const void* const* codes_stacked, const void* const* meta_stacked,
                                      const void* const* scales_stacked, const int64_t* indices,
                                      uint16_t* const* y, const int* N, const int* ldy, int T, int K, int S,
                                      int bits, int group_size, int accumulate, const int32_t* order,
                                      void* workspace, size_t workspace_bytes, void* stream) {
  return multi_delta_linear_batch(ncalls, x, w_base_tiled, codes_stacked, meta_stacked, scales_stacked, indices, y, N,
                                  ldy, T, K, S, bits, group_size, accumulate, order, workspace, workspace_bytes,
                                  stream, 1);
}

int dz_tile_base(const uint16_t* w, int K, int N, uint16_t* out, void* stream) {
  if (!w || !out) return DZ_EINVAL;
  if (K < DZ_KBLOCK || N < DZ_NPAIR || K % DZ_KBLOCK || N % DZ_NPAIR) return DZ_ESHAPE;
  if (((uintptr_t)w & 15) || ((uintptr_t)out & 15)) return DZ_EALIGN;
  const uintptr_t bytes = (uintptr_t)N * K * 2;
  if ((uintptr_t)w < (uintptr_t)out + bytes && (uintptr_t)out < (uintptr_t)w + bytes) return DZ_EINVAL;   // a permutation: not in place
  const long long chunks = (long long)N * K / 8;   // 16 bytes each
  hipLaunchKernelGGL(dz_tile_base_kernel, dim3((unsigned)((chunks + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                     (const u4_t*)w, (u4_t*)out, K, N);
  return hipGetLastError() == hipSuccess ? DZ_OK : DZ_ELAUNCH;
}

int dz_token_order(const int64_t* indices, int T, int S, int32_t* order, void* stream) {
  if (!indices || !order) return DZ_EINVAL;
  if (T < 1 || T > DZ_MAX_TOKENS_FUSED || S < 0) return DZ_ESHAPE;
  hipLaunchKernelGGL(dz_deal_kernel, dim3(1), dim3(128), 0, (hipStream_t)stream, (const long long*)indices, T, S, order);
  return hipGetLastError() == hipSuccess ? DZ_OK : DZ_ELAUNCH;
}

int dz_multi_delta_linear(const uint16_t* x, const uint16_t* w_base, const void* codes_stacked,
                          const void* meta_stacked, const void* scales_stacked,
                          const int64_t* indices, uint16_t* y, int T, int K, int N, int S, int bits,
                          int group_size, int accumulate, int ldy, void* workspace,
                          size_t workspace_bytes, void* stream) {
  if (!x || !indices || !y) return DZ_EINVAL;
  if (S > 0 && (!codes_stacked || !meta_stacked || !scales_stacked)) return DZ_EINVAL;
  if (S == 0 && !w_base) return DZ_EINVAL;
  return dz_multi_delta_linear_batch(1, &x, &w_base, &codes_stacked, &meta_stacked, &scales_stacked, indices, &y,
                                     &N, &ldy, T, K, S, bits, group_size, accumulate, nullptr, workspace,
                                     workspace_bytes, stream);
}

int dz_multi_delta_linear_static(const uint16_t* x, const uint16_t* w_base, const void* codes_stacked,
                                 const void* meta_stacked, const void* scales_stacked,
                                 const int64_t* indices, uint16_t* y, int T, int K, int N, int S, int bits,
                                 int group_size, int accumulate, int ldy, void* stream) {
  if (N > DZ_STATIC_MAX_N) return DZ_ESTATICMAX;
  void* ws = static_scratch_ptr();
  if (!ws) return DZ_ELAUNCH;
  return dz_multi_delta_linear(x, w_base, codes_stacked, meta_stacked, scales_stacked, indices, y, T, K, N, S,
                               bits, group_size, accumulate, ldy, ws, STATIC_SCRATCH_BYTES, stream);
}

}  // extern "C"
