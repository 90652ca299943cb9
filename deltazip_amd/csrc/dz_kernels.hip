// gfx950 kernels of the multi-delta linear layer and their C ABI.
//
//   dz_dequant_kernel / merge   native delta -> fp16 [N, K] (bit-exact with the reference's
//                               QuantLinear.unpack, deltazip/nn_modules/qlinear_cuda.py:246-329)
//   dz_segment_kernel           tokens grouped by delta id
//   dz_mdl_kernel               the fused decode kernel: base weights on the dense matrix-core
//                               instruction, every delta on the 2:4-sparse one, all deltas of a
//                               batch in one launch; each packed word is read from HBM once.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/dz_amd.h"
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
// fused decode kernel
// ---------------------------------------------------------------------------------------------
// PRE = true: the fp16 scale is multiplied into the sparse operand (one fp16 rounding per
// element, exactly the reference's dequantised value).  PRE = false (2-bit, per-channel scales
// only, where scale * {-2,-1,0,1} is exact in fp16): raw code sums are scaled once at the end.
template <int BITS, int TT, int WN, int WK, bool PRE>
__global__ __launch_bounds__(64 * WN * WK) void dz_mdl_kernel(const MdlParams P) {
  constexpr int NT = 64 * WN * WK;
  constexpr int TP = 16 * TT;  // padded token count
  constexpr int PD = 4;        // delta prefetch depth
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  _Float16* xs = (_Float16*)smem;                             // [WK][TP][XS]
  int* s_key = (int*)(smem + (size_t)WK * TP * XS * 2);       // [TP]
  int* s_skey = s_key + TP;
  int* s_perm = s_skey + TP;
  int* s_dl = s_perm + TP;
  int* s_lo = s_dl + TP;
  int* s_hi = s_lo + TP;
  int* s_misc = s_hi + TP;  // [0] = nd, [1] = last flag
  f4_t* red = (f4_t*)smem;  // aliases xs after the last round: [WN][WK][2][64]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wn = wave % WN, wk = wave / WN;
  const int jj = lane & 15, ga = lane >> 4;
  const uint32_t MAGIC = magic_vgpr();

  // workgroup -> (n-pair group, k-chunk); the chunks of one n-pair group sit on one XCD
  // (workgroups are dealt round-robin over the 8 XCDs) so their partial sums meet in one L2
  const int xcd = blockIdx.x & 7, q = blockIdx.x >> 3;
  const int npg = (q / P.nsplit) * 8 + xcd, kc = q % P.nsplit;
  if (npg >= P.NPG) return;
  const int np = npg * WN + wn;
  const bool np_ok = np < P.NP;
  const int n0 = np * DZ_NPAIR;
  const int kb_lo = kc * P.cb, kb_hi = min(P.NKB, kb_lo + P.cb);
  const int nrounds = (kb_hi - kb_lo + WK - 1) / WK;

  DZ_TS(0);
  // ---- base weights of the first round: issue before anything else
  u4_t a[2][4][2];
  auto load_base = [&](int kb) {
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int h = 0; h < 2; ++h)
          a[s][j][h] = __builtin_nontemporal_load(
              (const u4_t*)(P.wb + (size_t)(n0 + 16 * s + jj) * P.K + (size_t)kb * DZ_KBLOCK +
                            64 * j + 32 * h + 8 * ga));
  };
  {
    const int kb = kb_lo + wk;
    if (P.wb && np_ok && kb < kb_hi) load_base(kb);
  }

  // ---- group tokens by delta id (every workgroup redoes this tiny sort; T <= 128)
  for (int t = tid; t < TP; t += NT) {
    int key = 0x7fffffff;
    if (t < P.T) {
      long long id = P.idx[t];
      key = (id < 0 || id >= P.S) ? 0 : (int)id + 1;
      if ((id < -1 || id >= P.S) && blockIdx.x == 0) atomicOr(P.status, 1u);
    }
    s_key[t] = key;
  }
  __syncthreads();
  for (int t = tid; t < TP; t += NT) {
    if (t < P.T) {
      const int key = s_key[t];
      int r = 0;
      for (int u = 0; u < P.T; ++u) {
        const int ku = s_key[u];
        r += (ku < key) || (ku == key && u < t);
      }
      s_skey[r] = key;
      s_perm[r] = t;
    } else {
      s_skey[t] = 0x7fffffff;
      s_perm[t] = -1;
    }
  }
  __syncthreads();
  for (int r = tid; r < P.T; r += NT) {
    const int key = s_skey[r];
    const bool head = key != 0 && (r == 0 || s_skey[r - 1] != key);
    if (head) {
      int dd = 0;  // number of segment heads before r
      for (int u = 0; u < r; ++u) {
        const int ku = s_skey[u];
        dd += (ku != 0 && (u == 0 || s_skey[u - 1] != ku));
      }
      int e = r + 1;
      while (e < P.T && s_skey[e] == key) ++e;
      s_dl[dd] = key - 1;
      s_lo[dd] = r;
      s_hi[dd] = e;
    }
  }
  if (tid == 0) {
    int nd = 0;
    for (int u = 0; u < P.T; ++u) nd += (s_skey[u] != 0 && (u == 0 || s_skey[u - 1] != s_skey[u]));
    s_misc[0] = nd;
  }
  __syncthreads();
  const int nd = s_misc[0];
  DZ_TS(1);

  f4_t accb[2][TT], accd[2][TT];
#pragma unroll
  for (int s = 0; s < 2; ++s)
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) {
      accb[s][tt] = (f4_t){0.f, 0.f, 0.f, 0.f};
      accd[s][tt] = (f4_t){0.f, 0.f, 0.f, 0.f};
    }

  for (int r = 0; r < nrounds; ++r) {
    const int kb = kb_lo + r * WK + wk;
    const bool active = np_ok && kb < kb_hi;
    if (r > 0) {
      if (P.wb && active) load_base(kb);
      __syncthreads();  // everyone is done with the previous round's activations
    }
    // ---- delta prefetch ring
    Frag<BITS> ring[PD];
#pragma unroll
    for (int u = 0; u < PD; ++u)
      if (active && u < nd) ring[u] = load_frag<BITS>(P, s_dl[u], np, kb, lane);

    if (r == 0) DZ_TS(2);
    // ---- stage the activations of this round's k-blocks, rows in sorted token order
    for (int c = tid; c < WK * TP * 32; c += NT) {
      const int w2 = c / (TP * 32), rem = c % (TP * 32), row = rem >> 5, ch = rem & 31;
      const int kb2 = kb_lo + r * WK + w2;
      const int tok = s_perm[row];
      u4_t v = {0u, 0u, 0u, 0u};
      if (tok >= 0 && kb2 < kb_hi)
        v = *(const u4_t*)(P.x + (size_t)tok * P.K + (size_t)kb2 * DZ_KBLOCK + ch * 8);
      *(u4_t*)(xs + ((size_t)w2 * TP + row) * XS + ch * 8) = v;
    }
    __syncthreads();

    if (r == 0) DZ_TS(3);
    if (active) {
      const _Float16* xw = xs + (size_t)wk * TP * XS;
      auto ldsB = [&](int tt, int j, h8_t& lo, h8_t& hi) {
        const _Float16* p = xw + (tt * 16 + jj) * XS + 64 * j + 8 * ga;
        lo = *(const h8_t*)p;
        hi = *(const h8_t*)(p + 32);
      };
      // ---- base: dense matrix-core product over all token tiles
      if (P.wb) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int tt = 0; tt < TT; ++tt) {
            if (tt * 16 < P.T) {
              h8_t blo, bhi;
              ldsB(tt, j, blo, bhi);
#pragma unroll
              for (int s = 0; s < 2; ++s) {
                H8U a0, a1;
                a0.v = a[s][j][0];
                a1.v = a[s][j][1];
                accb[s][tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0.h, blo, accb[s][tt], 0, 0, 0);
                accb[s][tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a1.h, bhi, accb[s][tt], 0, 0, 0);
              }
            }
          }
      }
      if (r == 0) DZ_TS(4);
      // ---- deltas: sparse matrix-core product, one delta at a time
      for (int dd0 = 0; dd0 < nd; dd0 += PD) {
#pragma unroll
        for (int u = 0; u < PD; ++u) {
          const int dd = dd0 + u;
          if (dd < nd) {
            const Frag<BITS> cur = ring[u];
            if (dd + PD < nd) ring[u] = load_frag<BITS>(P, s_dl[dd + PD], np, kb, lane);
            const int d = s_dl[dd], lo = s_lo[dd], hi = s_hi[dd];
            h8_t A[4][2];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              if (BITS == 2) {
                unpack2(cur.code[0][j], MAGIC, A[j][0], A[j][1]);
              } else {
                A[j][0] = unpack4(cur.code[(BITS == 2) ? 0 : (j >> 1)][2 * (j & 1) + 0], MAGIC);
                A[j][1] = unpack4(cur.code[(BITS == 2) ? 0 : (j >> 1)][2 * (j & 1) + 1], MAGIC);
              }
            }
            if (PRE) {
              // lane's operand row is n0 + 16*s + jj; one scale per (row, K-group)
              const _Float16* sp = P.scales + (size_t)d * P.scales_slot + n0 + jj;
              _Float16 s0 = (_Float16)0.f, s1 = (_Float16)0.f;
              int gprev = -1;
#pragma unroll
              for (int j = 0; j < 4; ++j) {
                const int g = (kb * DZ_KBLOCK + 64 * j) / P.gs;
                if (g != gprev) {
                  s0 = sp[(size_t)g * P.N];
                  s1 = sp[(size_t)g * P.N + 16];
                  gprev = g;
                }
                A[j][0] *= s0;
                A[j][1] *= s1;
              }
            }
#pragma unroll
            for (int tt = 0; tt < TT; ++tt) {
              if (tt * 16 < hi && tt * 16 + 16 > lo) {
                const int pos = tt * 16 + jj;
                const float in = (pos >= lo && pos < hi) ? 1.0f : 0.0f;
                f4_t t0 = {0.f, 0.f, 0.f, 0.f}, t1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                  h8_t blo, bhi;
                  ldsB(tt, j, blo, bhi);
                  h16_t B = __builtin_shufflevector(blo, bhi, 0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11,
                                                    12, 13, 14, 15);
                  const int mw = (int)cur.meta[j];
                  t0 = __builtin_amdgcn_smfmac_f32_16x16x64_f16(A[j][0], B, t0, mw, 0, 0);
                  t1 = __builtin_amdgcn_smfmac_f32_16x16x64_f16(A[j][1], B, t1, mw, 0, 1);
                }
                accd[0][tt] += t0 * in;
                accd[1][tt] += t1 * in;
              }
            }
          }
        }
      }
    }
  }

  DZ_TS(5);
  if (!PRE) {
    // scale the raw code sums: column (token) tt*16 + jj belongs to exactly one delta
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) {
      const int key = s_skey[tt * 16 + jj];
      if (key > 0 && key != 0x7fffffff && np_ok) {
        const _Float16* sp = P.scales + (size_t)(key - 1) * P.scales_slot + n0 + 4 * ga;
#pragma unroll
        for (int s = 0; s < 2; ++s) {
          const h4_t v = *(const h4_t*)(sp + 16 * s);
          accd[s][tt] *= (f4_t){(float)v[0], (float)v[1], (float)v[2], (float)v[3]};
        }
      }
    }
  }

  // ---- reduce over the WK waves of each n-pair, then over the k-chunks of other workgroups
  auto final_store = [&](int s, int tt, f4_t v) {
    const int tok = s_perm[tt * 16 + jj];
    if (tok >= 0 && np_ok) {
      _Float16* yp = P.y + (size_t)tok * P.ldy + n0 + 16 * s + 4 * ga;
      if (P.accumulate) {
        h4_t o = *(const h4_t*)yp;
        v += (f4_t){(float)o[0], (float)o[1], (float)o[2], (float)o[3]};
      }
      h4_t r = {(_Float16)v[0], (_Float16)v[1], (_Float16)v[2], (_Float16)v[3]};
      *(h4_t*)yp = r;
    }
  };
  auto part_ptr = [&](int kc2, int s, int tt) -> f4_t* {
    return (f4_t*)P.partials + (((size_t)kc2 * P.NP + np) * (2 * TT) + (tt * 2 + s)) * 64 + lane;
  };

  __syncthreads();  // activations no longer needed: LDS becomes the reduction buffer
  DZ_TS(6);
#pragma unroll
  for (int tt = 0; tt < TT; ++tt) {
    if (tt * 16 < P.T) {
      f4_t v0 = accb[0][tt] + accd[0][tt], v1 = accb[1][tt] + accd[1][tt];
      if (WK > 1) {
        red[((wn * WK + wk) * 2 + 0) * 64 + lane] = v0;
        red[((wn * WK + wk) * 2 + 1) * 64 + lane] = v1;
        __syncthreads();
        if (wk < 2) {
          f4_t sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int w2 = 0; w2 < WK; ++w2) sum += red[((wn * WK + w2) * 2 + wk) * 64 + lane];
          if (P.nsplit == 1) final_store(wk, tt, sum);
          else if (np_ok) *part_ptr(kc, wk, tt) = sum;
        }
        __syncthreads();
      } else {
        if (P.nsplit == 1) {
          final_store(0, tt, v0);
          final_store(1, tt, v1);
        } else if (np_ok) {
          *part_ptr(kc, 0, tt) = v0;
          *part_ptr(kc, 1, tt) = v1;
        }
      }
    }
  }
  DZ_TS(7);
  if (P.nsplit > 1) {
    __syncthreads();
    DZ_TS(8);
    if (tid == 0) {
      __threadfence();  // one release for the whole workgroup's partial sums
      const unsigned old = atomicAdd(P.counters + npg, 1u);
      const int last = (old == (unsigned)(P.nsplit - 1));
      if (last) __threadfence();  // acquire the other chunks' sums
      s_misc[1] = last;
    }
    __syncthreads();
    if (s_misc[1]) {
      if ((WK == 1 || wk < 2) && np_ok) {
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) {
          if (tt * 16 < P.T) {
#pragma unroll
            for (int s = 0; s < 2; ++s) {
              if (WK == 1 || s == wk) {
                f4_t sum = {0.f, 0.f, 0.f, 0.f};
                for (int k2 = 0; k2 < P.nsplit; ++k2)
                  sum += __builtin_nontemporal_load(part_ptr(k2, s, tt));
                final_store(s, tt, sum);
              }
            }
          }
        }
      }
      if (tid == 0) P.counters[npg] = 0u;
    }
  }
  DZ_TS(9);
}

// ---------------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------------
int g_ksplit_override = 0;

inline int check_group(int K, int group_size, int* gs_out) {
  int gs = (group_size == -1 || group_size == K) ? K : group_size;
  if (gs <= 0 || K % gs || (gs != K && gs % 64)) return DZ_EGROUP;
  *gs_out = gs;
  return DZ_OK;
}

constexpr size_t WS_HEADER = 256;  // status word
inline size_t ws_counter_bytes(int N) { return (((size_t)(N / DZ_NPAIR + 8) * 4) + 255) / 256 * 256; }
constexpr int MAX_KSPLIT = 16;

template <int BITS, int TT, int WN, int WK>
int launch_mdl(const MdlParams& P0, bool pre, hipStream_t st) {
  MdlParams P = P0;
  P.NPG = (P.NP + WN - 1) / WN;
  // K split across workgroups: enough workgroups to fill 256 CUs about twice, few partials
  int nsplit = g_ksplit_override;
  if (nsplit <= 0) {
    nsplit = 1;
    while (nsplit < MAX_KSPLIT && (long long)P.NPG * nsplit < 256 && (P.NKB / (nsplit * 2)) >= WK)
      nsplit *= 2;
    // keep rounds per workgroup small when K is long
    while (nsplit < MAX_KSPLIT && (P.NKB + nsplit - 1) / nsplit > 2 * WK) ++nsplit;
  }
  if (nsplit > MAX_KSPLIT) nsplit = MAX_KSPLIT;
  if (nsplit > P.NKB) nsplit = P.NKB;
  P.cb = (P.NKB + nsplit - 1) / nsplit;
  P.cb = (P.cb + WK - 1) / WK * WK;  // whole rounds
  nsplit = (P.NKB + P.cb - 1) / P.cb;
  P.nsplit = nsplit;
  const int npg_pad = (P.NPG + 7) / 8 * 8;
  const int grid = npg_pad * nsplit;
  const size_t lds = (size_t)WK * 16 * TT * XS * 2 + (size_t)(6 * 16 * TT + 8) * 4;
  static bool attr_done[2] = {false, false};  // per template instantiation
  if (pre) {
    auto kern = dz_mdl_kernel<BITS, TT, WN, WK, true>;
    if (!attr_done[1]) {
      if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
        return DZ_ELAUNCH;
      attr_done[1] = true;
    }
    hipLaunchKernelGGL(kern, dim3(grid), dim3(64 * WN * WK), lds, st, P);
  } else {
    auto kern = dz_mdl_kernel<BITS, TT, WN, WK, false>;
    if (!attr_done[0]) {
      if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
        return DZ_ELAUNCH;
      attr_done[0] = true;
    }
    hipLaunchKernelGGL(kern, dim3(grid), dim3(64 * WN * WK), lds, st, P);
  }
  return hipGetLastError() == hipSuccess ? DZ_OK : DZ_ELAUNCH;
}

template <int BITS>
int launch_mdl_bits(const MdlParams& P, bool pre, hipStream_t st) {
  if (P.T <= 64) return launch_mdl<BITS, 4, 4, 2>(P, pre, st);
  return launch_mdl<BITS, 8, 4, 2>(P, pre, st);
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

size_t dz_workspace_bytes(int T, int K, int N) {
  (void)K;
  if (T < 1 || N < 1) return 0;
  const size_t tp = (size_t)(T <= DZ_MAX_TOKENS_FUSED ? (T + 15) / 16 * 16 : 16);
  return WS_HEADER + ws_counter_bytes(N) + (size_t)MAX_KSPLIT * tp * (size_t)N * 4;
}

int dz_multi_delta_linear(const uint16_t* x, const uint16_t* w_base, const void* codes_stacked,
                          const void* meta_stacked, const void* scales_stacked,
                          const int64_t* indices, uint16_t* y, int T, int K, int N, int S, int bits,
                          int group_size, int accumulate, int ldy, void* workspace,
                          size_t workspace_bytes, void* stream) {
  if (!x || !indices || !y) return DZ_EINVAL;
  if (S > 0 && (!codes_stacked || !meta_stacked || !scales_stacked)) return DZ_EINVAL;
  if (S < 1) return DZ_EINVAL;  // at least one slot: the kernels always address slot 0
  size_t cb, mb, sb;
  int rc = dz_native_sizes(K, N, bits, group_size, &cb, &mb, &sb);
  if (rc) return rc;
  int gs;
  if ((rc = check_group(K, group_size, &gs))) return rc;
  if (T < 1 || T > DZ_MAX_TOKENS_FUSED || ldy < N || ldy % 4) return DZ_ESHAPE;
  if (((uintptr_t)x & 15) || ((uintptr_t)y & 7) || (w_base && ((uintptr_t)w_base & 15))) return DZ_EALIGN;
  if (!workspace || workspace_bytes < dz_workspace_bytes(T, K, N)) return DZ_EWORKSPACE;

  MdlParams P;
  P.x = (const _Float16*)x;
  P.wb = (const _Float16*)w_base;
  P.codes = (const u4_t*)codes_stacked;
  P.meta = (const u4_t*)meta_stacked;
  P.scales = (const _Float16*)scales_stacked;
  P.idx = (const long long*)indices;
  P.y = (_Float16*)y;
  P.status = (unsigned*)workspace;
  P.counters = (unsigned*)((char*)workspace + WS_HEADER);
  P.partials = (float*)((char*)workspace + WS_HEADER + ws_counter_bytes(N));
  P.codes_slot_u4 = (long long)(cb / 16);
  P.meta_slot_u4 = (long long)(mb / 16);
  P.scales_slot = (long long)(sb / 2);
  P.T = T; P.K = K; P.N = N; P.S = S; P.gs = gs; P.G = K / gs;
  P.accumulate = accumulate; P.ldy = ldy;
  P.NP = N / DZ_NPAIR; P.NKB = K / DZ_KBLOCK;
  P.nsplit = 1; P.cb = P.NKB; P.NPG = 0;
  const bool pre = !(bits == 2 && gs == K);
  hipStream_t st = (hipStream_t)stream;
  if (T <= 32) return dz_launch_mdl32(P, bits, pre, st, g_ksplit_override);
  return bits == 2 ? launch_mdl_bits<2>(P, pre, st) : launch_mdl_bits<4>(P, pre, st);
}

}  // extern "C"
