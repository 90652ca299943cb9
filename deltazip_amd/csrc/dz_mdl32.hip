// Fused multi-delta linear kernel for decode-sized batches (T <= 32 tokens).
//
// One workgroup = 4 wavefronts = one n-pair (32 output rows) x a chunk of k-blocks; each
// wavefront owns whole k-blocks (256 input columns) of that n-pair and is self-sufficient until
// the final reduction:
//   * at entry it issues, back to back, the loads of its activations slice (straight into LDS,
//     global_load_lds_dwordx4), of the token ids and of its 32 x 256 base-weight tile (16 x
//     128-bit loads per lane), so HBM traffic starts at once;
//   * the token ids arrive through scalar loads (a path that does not queue behind the vector
//     loads); the distinct deltas of the batch are enumerated with ballots (no sort, no barrier):
//     output columns stay in token order and each delta gets a per-column mask.  Batches that
//     arrive sorted by id (as the reference's scheduler delivers them) touch fewer column tiles;
//   * the packed words of the first deltas are then requested together;
//   * base tile x activations runs on v_mfma_f32_16x16x32_f16, each delta on the 2:4-sparse
//     v_smfmac_f32_16x16x64_f16 with the unpacked codes as the sparse operand and the stored
//     positions as its index operand; the dense operand (activations) is read from the
//     wavefront's own LDS slice;
//   * partial sums of the 4 wavefronts meet in LDS; when K is split over several workgroups the
//     per-chunk sums go to a workspace and the last workgroup to arrive adds them in a fixed
//     order (deterministic) and writes y.
#include "../../include/dz_amd.h"
#include "dz_device.h"

namespace {

constexpr int WK32 = 4;

template <int BITS, int TT, bool PRE>
__global__ __launch_bounds__(64 * WK32, 2) void dz_mdl32_kernel(const MdlParams P) {
  constexpr int TP = 16 * TT;                  // padded token count (16 or 32)
  constexpr int PD = (BITS == 2) ? (TT == 1 ? 8 : 6) : 4;  // deltas in flight per wavefront
  constexpr int NX = TP / 2;                   // activation loads per wavefront (2 rows each)
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  __shared__ int s_last;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wavefront-uniform, in a scalar register
  const int jj = lane & 15, ga = lane >> 4;
  _Float16* xw = (_Float16*)smem + (size_t)wave * TP * DZ_KBLOCK;   // this wavefront's activations
  f4_t* red = (f4_t*)smem;                                   // reduction buffer, after the barrier

  // workgroup -> (n-pair, k-chunk); the chunks of one n-pair are dealt to one XCD so that their
  // partial sums can meet in that XCD's L2
  const int xcd = blockIdx.x & 7, q = blockIdx.x >> 3;
  const int np = (q / P.nsplit) * 8 + xcd, kc = q % P.nsplit;
  if (np >= P.NP) return;
  const int n0 = np * DZ_NPAIR;
  const int kb_lo = kc * P.cb, kb_hi = min(P.NKB, kb_lo + P.cb);
  const int nrounds = (kb_hi - kb_lo + WK32 - 1) / WK32;
  DZ_TS(0);
  // token ids first, through scalar loads (wavefront-uniform addresses): lane t keeps the key of
  // token t.  key: 0 = base only, id + 1 otherwise, INT_MAX for padding lanes.
  int key = 0x7fffffff;
  {
    long long ids[TP];
#pragma unroll
    for (int t = 0; t < TP; ++t) ids[t] = P.idx[min(t, P.T - 1)];
    bool bad = false;
#pragma unroll
    for (int t = 0; t < TP; ++t) {
      const long long v = ids[t];
      const int k = (v < 0 || v >= P.S) ? 0 : (int)v + 1;
      bad |= (v < -1 || v >= P.S);
      if (t < P.T) key = (lane == t) ? k : key;
    }
    if (bad && blockIdx.x == 0 && tid == 0) atomicOr(P.status, 1u);
  }
  // tokens that carry a delta; lanes >= T never match
  const unsigned long long mdelta = __builtin_amdgcn_ballot_w64(key != 0 && key != 0x7fffffff);
  DZ_TS(1);

  f4_t accb[2][TT], accd[2][TT];
#pragma unroll
  for (int s = 0; s < 2; ++s)
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) {
      accb[s][tt] = (f4_t){0.f, 0.f, 0.f, 0.f};
      accd[s][tt] = (f4_t){0.f, 0.f, 0.f, 0.f};
    }

  // LDS byte offsets of this lane's operand chunks: row = token tt*16 + jj, chunk index
  // 8*j + 4*h + ga with its low 4 bits swizzled by the row; index = (j & 1) * 2 + h
  int boff[TT][4];
#pragma unroll
  for (int tt = 0; tt < TT; ++tt)
#pragma unroll
    for (int c = 0; c < 4; ++c)
      boff[tt][c] = (tt * 16 + jj) * (DZ_KBLOCK * 2) + ((((c << 2) | ga) ^ jj) << 4);

  for (int r = 0; r < nrounds; ++r) {
    const int kb = kb_lo + r * WK32 + wave;
    const bool active = kb < kb_hi;  // wavefront-uniform
    // Per-round copy of the lane id that the optimiser cannot prove loop-invariant: otherwise it
    // precomputes every load offset of the round outside the loop and spills them.
    int lane_r = lane;
    asm volatile("" : "+v"(lane_r));
    const int jj_r = lane_r & 15, ga_r = lane_r >> 4;

    // ---- issue order: [later rounds: packed deltas], activations slice (L2 -> LDS directly), base
    // tile (HBM).  LDS row t = token t, 512 bytes, its 16-byte chunks XOR-swizzled with (t & 15)
    // so that the 16 rows one operand read gathers fall on different banks.  Rows >= T repeat row
    // T-1: they only feed output columns that are never stored.
    // Addresses are a wavefront-uniform base plus one 32-bit lane offset.
    u4_t a[2][4][2];
    const unsigned Kb = (unsigned)P.K * 2u;  // row pitch in bytes
    // ---- delta walk: pop the lowest token that still has an unvisited delta, take its id and
    // clear every token of that delta (all scalar work)
    unsigned long long m_use = mdelta, m_load = mdelta;
    auto pop = [&](unsigned long long& m, int& d, unsigned long long& dm) {
      const int l = __builtin_ctzll(m);
      const int kd = __builtin_amdgcn_readlane(key, l);
      dm = __builtin_amdgcn_ballot_w64(key == kd);
      m &= ~dm;
      d = kd - 1;
    };
    Frag<BITS> ring[PD];
    auto fill_ring = [&]() {
#pragma unroll
      for (int u = 0; u < PD; ++u)
        if (m_load) {
          int d;
          unsigned long long dm;
          pop(m_load, d, dm);
          ring[u] = load_frag<BITS>(P, d, np, kb, lane_r);
        }
    };
    // the packed words of the first deltas go out first
    if (active) fill_ring();
    __builtin_amdgcn_sched_barrier(0);
    if (active) {
      const char* xb = (const char*)(P.x + (size_t)kb * DZ_KBLOCK);
#pragma unroll
      for (int i = 0; i < NX; ++i) {
        const int t = min(2 * i + (lane_r >> 5), P.T - 1), c = lane_r & 31;
        const unsigned off = (unsigned)t * Kb + (unsigned)((c ^ (t & 15)) << 4);
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(xb + off),
                                         (__attribute__((address_space(3))) void*)(xw + 2 * i * DZ_KBLOCK),
                                         16, 0, 0);
      }
    }

    __builtin_amdgcn_sched_barrier(0);
    if (active && P.wb) {
      const char* wbb = (const char*)(P.wb + (size_t)n0 * P.K + (size_t)kb * DZ_KBLOCK);
      const unsigned loff = (unsigned)jj_r * Kb + (unsigned)ga_r * 16u;
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        const char* ws = wbb + (size_t)(16 * s) * Kb;
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int h = 0; h < 2; ++h)
            a[s][j][h] = __builtin_nontemporal_load((const u4_t*)(ws + loff + (128 * j + 64 * h)));
      }
    }
    __builtin_amdgcn_sched_barrier(0);

    // Loads return in order: once at most the 16 base loads are outstanding, the packed deltas and
    // this wavefront's LDS slice are complete.  (The compiler
    // does not order LDS reads after LDS-direct loads by itself.)
    if (P.wb) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);

    if (active) {
      if (r == 0) DZ_TS(2);

      // chunk index of step j, half h is 8*j + 4*h + ga; its low 4 bits are swizzled per row
      auto ldsB = [&](int tt, int j, h8_t& lo, h8_t& hi) {
        const char* p = (const char*)xw + (j >> 1) * 256;
        lo = *(const h8_t*)(p + boff[tt][(j & 1) * 2 + 0]);
        hi = *(const h8_t*)(p + boff[tt][(j & 1) * 2 + 1]);
      };
      // ---- base: dense matrix-core product over all token tiles
      if (P.wb) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int tt = 0; tt < TT; ++tt) {
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
      if (r == 0) DZ_TS(4);

      // ---- deltas: sparse matrix-core product, one delta at a time
      while (m_use) {
#pragma unroll
        for (int u = 0; u < PD; ++u) {
          if (m_use) {
            int d;
            unsigned long long dm;
            pop(m_use, d, dm);
            const Frag<BITS> cur = ring[u];
            if (m_load) {
              int d2;
              unsigned long long dm2;
              pop(m_load, d2, dm2);
              ring[u] = load_frag<BITS>(P, d2, np, kb, lane_r);
            }
            // lane's operand row is n0 + 16*s + jj; one scale per (row, K-group) when PRE
            const _Float16* sp = P.scales + (size_t)d * P.scales_slot + n0 + jj;
            _Float16 s0 = (_Float16)0.f, s1 = (_Float16)0.f;
            int gprev = -1;
            f4_t t0[TT], t1[TT];
            bool in[TT];
#pragma unroll
            for (int tt = 0; tt < TT; ++tt) {
              t0[tt] = (f4_t){0.f, 0.f, 0.f, 0.f};
              t1[tt] = (f4_t){0.f, 0.f, 0.f, 0.f};
              in[tt] = (dm >> (tt * 16 + jj)) & 1ull;
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              h8_t A0, A1;
              if (BITS == 2) {
                unpack2(cur.code[0][j], A0, A1);
              } else {
                A0 = unpack4(cur.code[(BITS == 2) ? 0 : (j >> 1)][2 * (j & 1) + 0]);
                A1 = unpack4(cur.code[(BITS == 2) ? 0 : (j >> 1)][2 * (j & 1) + 1]);
              }
              if (PRE) {
                const int g = (kb * DZ_KBLOCK + 64 * j) / P.gs;
                if (g != gprev) {
                  s0 = sp[(size_t)g * P.N];
                  s1 = sp[(size_t)g * P.N + 16];
                  gprev = g;
                }
                A0 *= s0;
                A1 *= s1;
              }
              const int mw = (int)cur.meta[j];
#pragma unroll
              for (int tt = 0; tt < TT; ++tt) {
                if ((dm >> (tt * 16)) & 0xffffull) {
                  h8_t blo, bhi;
                  ldsB(tt, j, blo, bhi);
                  h16_t B = __builtin_shufflevector(blo, bhi, 0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11,
                                                    12, 13, 14, 15);
                  t0[tt] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(A0, B, t0[tt], mw, 0, 0);
                  t1[tt] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(A1, B, t1[tt], mw, 0, 1);
                }
              }
            }
#pragma unroll
            for (int tt = 0; tt < TT; ++tt) {
              // select, not multiply: columns outside the segment may hold anything
              accd[0][tt] += in[tt] ? t0[tt] : (f4_t){0.f, 0.f, 0.f, 0.f};
              accd[1][tt] += in[tt] ? t1[tt] : (f4_t){0.f, 0.f, 0.f, 0.f};
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
      const int kcol = __builtin_amdgcn_ds_bpermute((tt * 16 + jj) << 2, key);
      if (kcol > 0 && kcol != 0x7fffffff) {
        const _Float16* sp = P.scales + (size_t)(kcol - 1) * P.scales_slot + n0 + 4 * ga;
#pragma unroll
        for (int s = 0; s < 2; ++s) {
          const h4_t v = *(const h4_t*)(sp + 16 * s);
          accd[s][tt] *= (f4_t){(float)v[0], (float)v[1], (float)v[2], (float)v[3]};
        }
      }
    }
  }

  // ---- reduce over the 4 wavefronts (LDS), then over the k-chunks of other workgroups
  auto final_store = [&](int s, int tt, f4_t v) {
    if (tt * 16 + jj < P.T) {
      _Float16* yp = P.y + (size_t)(tt * 16 + jj) * P.ldy + n0 + 16 * s + 4 * ga;
      if (P.accumulate) {
        const h4_t o = *(const h4_t*)yp;
        v += (f4_t){(float)o[0], (float)o[1], (float)o[2], (float)o[3]};
      }
      const h4_t o = {(_Float16)v[0], (_Float16)v[1], (_Float16)v[2], (_Float16)v[3]};
      *(h4_t*)yp = o;
    }
  };
  // partial sums of one k-chunk: [chunk][n-pair][item][4 values][64 lanes] floats.  They are
  // written and read with agent-scope accesses (write-through / cache-bypassing), so that no
  // whole-cache write-back or invalidate is needed to pass them between XCDs.
  auto part_ptr = [&](int kc2, int item) -> float* {
    return P.partials + (((size_t)kc2 * P.NP + np) * (2 * TT) + item) * 256 + lane;
  };
  __syncthreads();  // every wavefront is done with its activations: LDS becomes the buffer
  DZ_TS(6);
  // item = tt*2 + s; red[wave][item][lane]
#pragma unroll
  for (int tt = 0; tt < TT; ++tt)
#pragma unroll
    for (int s = 0; s < 2; ++s)
      red[(wave * (2 * TT) + tt * 2 + s) * 64 + lane] = accb[s][tt] + accd[s][tt];
  __syncthreads();
  // wavefront w sums item w (TT = 1: items 0..1, TT = 2: items 0..3)
  f4_t sum = {0.f, 0.f, 0.f, 0.f};
  const bool has_item = wave < 2 * TT;
  if (has_item) {
#pragma unroll
    for (int w2 = 0; w2 < WK32; ++w2) sum += red[(w2 * (2 * TT) + wave) * 64 + lane];
  }
  const int my_tt = wave >> 1, my_s = wave & 1;
  auto store_item = [&](f4_t v) {
#pragma unroll
    for (int tt = 0; tt < TT; ++tt)
      if (tt == my_tt) final_store(my_s, tt, v);
  };
  DZ_TS(7);
  if (P.nsplit == 1) {
    if (has_item) store_item(sum);
    return;
  }
  if (has_item) {
    float* pp = part_ptr(kc, wave);
#pragma unroll
    for (int e = 0; e < 4; ++e)
      __hip_atomic_store(pp + 64 * e, sum[e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the sums have left this CU
  }
  __syncthreads();
  if (tid == 0) {
    const unsigned old = atomicAdd(P.counters + np, 1u);
    s_last = (old == (unsigned)(P.nsplit - 1));
  }
  __syncthreads();
  DZ_TS(8);
  if (s_last) {
    if (has_item) {
      f4_t tot = {0.f, 0.f, 0.f, 0.f};
      for (int k2 = 0; k2 < P.nsplit; ++k2) {
        const float* pp = part_ptr(k2, wave);
#pragma unroll
        for (int e = 0; e < 4; ++e)
          tot[e] += __hip_atomic_load(pp + 64 * e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      store_item(tot);
    }
    if (tid == 0) P.counters[np] = 0u;
  }
  DZ_TS(9);
}

template <int BITS, int TT>
int launch32(MdlParams P, bool pre, hipStream_t st, int ksplit_override) {
  // K split over workgroups: aim at two resident workgroups per CU (512) with few rounds each
  int nsplit = ksplit_override;
  if (nsplit <= 0) {
    nsplit = 1;
    const int max_split = (P.NKB + WK32 - 1) / WK32;  // at least one round of 4 k-blocks each
    while (nsplit < max_split && (long long)P.NP * nsplit < 512) ++nsplit;
  }
  if (nsplit > 16) nsplit = 16;
  if (nsplit > P.NKB) nsplit = P.NKB;
  P.cb = (P.NKB + nsplit - 1) / nsplit;
  P.cb = (P.cb + WK32 - 1) / WK32 * WK32;  // whole rounds
  P.nsplit = (P.NKB + P.cb - 1) / P.cb;
  const int grid = (P.NP + 7) / 8 * 8 * P.nsplit;
  const size_t lds = (size_t)WK32 * 16 * TT * DZ_KBLOCK * 2;
  static bool attr_done[2] = {false, false};
  if (pre) {
    auto kern = dz_mdl32_kernel<BITS, TT, true>;
    if (!attr_done[1]) {
      if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
        return DZ_ELAUNCH;
      attr_done[1] = true;
    }
    hipLaunchKernelGGL(kern, dim3(grid), dim3(64 * WK32), lds, st, P);
  } else {
    auto kern = dz_mdl32_kernel<BITS, TT, false>;
    if (!attr_done[0]) {
      if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
        return DZ_ELAUNCH;
      attr_done[0] = true;
    }
    hipLaunchKernelGGL(kern, dim3(grid), dim3(64 * WK32), lds, st, P);
  }
  return hipGetLastError() == hipSuccess ? DZ_OK : DZ_ELAUNCH;
}

}  // namespace

// Launch of the T <= 32 kernel; called by dz_multi_delta_linear.
int dz_launch_mdl32(const MdlParams& P, int bits, bool pre, hipStream_t st, int ksplit_override) {
  if (bits == 2) return P.T <= 16 ? launch32<2, 1>(P, pre, st, ksplit_override) : launch32<2, 2>(P, pre, st, ksplit_override);
  return P.T <= 16 ? launch32<4, 1>(P, pre, st, ksplit_override) : launch32<4, 2>(P, pre, st, ksplit_override);
}

#ifdef DZ_TIMING
extern "C" void dz_set_timing_buffer32(void* p) { (void)hipMemcpyToSymbol(HIP_SYMBOL(g_dz_ts), &p, sizeof(p)); }
#endif
