// Fused multi-delta linear kernel for decode-sized batches: up to 128 tokens per launch, in chunks
// of 32 (several chunks: the tokens are taken in an order that spreads the deltas over the chunks).
//
// One workgroup = 4 wavefronts = one n-pair (32 output rows) x a slice of k-blocks x one chunk; each
// wavefront owns whole k-blocks (256 input columns) of that n-pair and is self-sufficient until
// the final reduction:
//   * the token ids are fetched first; the distinct deltas of the batch are enumerated
//     with ballots (no sort, no barrier): output columns stay in token order and each delta gets a
//     per-column mask.  Batches that arrive sorted by id (as the reference's scheduler delivers
//     them) touch fewer column tiles;
//   * the activations slice goes first (straight into LDS; it does not depend on the ids), then
//     the packed words of up to 8 deltas (two batches of 4); the base tile -- row-major or in
//     16 KiB tiles, streamed or, with several chunks, left in L2 for the next chunk's workgroup --
//     is requested once the first batch has been multiplied, so that a wavefront is not held at
//     its request queue while data it could work on has arrived.  The number of requests is
//     fixed, so the wait in front of each use is exact;
//   * one read of the dense operand (activations, from the wavefront's own LDS slice) feeds every
//     delta of the current batch (2:4-sparse v_smfmac_f32_16x16x64_f16, unpacked codes as the
//     sparse operand, stored positions as its index operand); the base tile follows on
//     v_mfma_f32_16x16x32_f16;
//   * partial sums of the 4 wavefronts meet in LDS; when K is split over several workgroups the
//     per-slice sums go to a workspace whose slots are their own "ready" marks (all zero bits =
//     empty): the workgroups of all but the last slice store and leave, the workgroup of the last
//     slice adds the slices in a fixed order (deterministic), writes y and empties the slots.
#include "../../include/dz_amd.h"
#include "dz_device.h"

namespace {

constexpr int WK32 = 4;
constexpr int DZ_SPIN_LIMIT = 1 << 16;   // polls of the partial sums (a poll is about a microsecond)

// The work of one workgroup: n-pair `np`, K-slice `kc`, token chunk `ch` of the layer call P.
template <int BITS, int TT, int PRE, int BASE, bool EARLY, bool IDL>
__device__ __forceinline__ void mdl32_body(const MdlParams& P, const int np, const int kc, const int ch,
                                           unsigned char* smem) {
  // BASE: 0 no base weight; 1 row-major [N, K]; 2 in tiles (dz_layout.h); 3, 4 and 5: 1, 2 and 0
  // for launches with several chunks of tokens (33 .. 128 tokens), where rows of x / idx / y go
  // through the token order P.perm and the base tile is requested as cacheable data.  A
  // compile-time choice: a wavefront-uniform branch around requests costs 3 % of the 7B step (the
  // compiler's wait-count pass sees two paths with different requests outstanding and makes
  // every later wait stricter).
  constexpr bool HAS_BASE = BASE >= 1 && BASE <= 4;
  constexpr bool TILED = BASE == 2 || BASE == 4;
  constexpr bool MULTI = BASE >= 3;          // P.nchunk > 1 and P.perm != nullptr
  constexpr bool SHARED_TILE = MULTI;
  constexpr int TP = 16 * TT;              // padded token count (16 or 32)
  constexpr int G = (BITS == 2) ? (PRE == 2 ? 3 : 4) : (TT == 2 ? 2 : 3);   // deltas per batch (two batches are in flight); 3 where 4 would not fit the registers
  constexpr int NX = TP / 2;               // activation loads per wavefront (2 rows each)
  // Requests per unit, from which the hand-written wait counts below are built (the request loops
  // run over the same constants): a delta batch = G x (positions, codes, PRE scale words); one row
  // fragment of the base tile = 4 steps x 2 halves.
  constexpr int BATCH_LOADS = G * (Frag<BITS>::NLOADS + PRE);
  constexpr int BASE_FRAG_LOADS = 4 * 2;
  constexpr int EARLY_LOADS = EARLY ? BASE_FRAG_LOADS : 0;   // EARLY: fragment 0 goes out with the activations
  static_assert(NX + 2 * BATCH_LOADS + 2 * BASE_FRAG_LOADS <= 63, "more requests in flight than vmcnt can count");
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wavefront-uniform, in a scalar register
  const int jj = lane & 15, ga = lane >> 4;
  const uint32_t MAGIC = magic_vgpr();
  _Float16* xw = (_Float16*)smem + (size_t)wave * TP * DZ_KBLOCK;   // this wavefront's activations
  f4_t* red = (f4_t*)smem;                                          // reduction buffer, after the barrier

  const int tok0 = P.tok0 + 32 * ch;
  const int Tc = min(32, P.T - 32 * ch);   // tokens of this chunk
  const int n0 = np * DZ_NPAIR;
  const int kb_lo = kc * P.cb, kb_hi = min(P.NKB, kb_lo + P.cb);
  const int nrounds = (kb_hi - kb_lo + WK32 - 1) / WK32;
  const unsigned Kb = (unsigned)P.K * 2u;  // row pitch of x and w_base in bytes
  DZ_TS(0);

  f4_t accb[2][TT], accd[2][TT];
#pragma unroll
  for (int s = 0; s < 2; ++s)
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) {
      accb[s][tt] = (f4_t){0.f, 0.f, 0.f, 0.f};
      accd[s][tt] = (f4_t){0.f, 0.f, 0.f, 0.f};
    }

  // LDS byte offsets of this lane's operand chunks: row = token tt*16 + jj (512 bytes per row),
  // chunk index 8*j + 4*h + ga with its low 4 bits XOR-swizzled by the row so that the 16 rows of
  // one operand read fall on different banks; index = (j & 1) * 2 + h, (j >> 1) adds 256 bytes
  int boff[TT][4];
#pragma unroll
  for (int tt = 0; tt < TT; ++tt)
#pragma unroll
    for (int c = 0; c < 4; ++c)
      boff[tt][c] = (tt * 16 + jj) * (DZ_KBLOCK * 2) + ((((c << 2) | ga) ^ jj) << 4);

  u4_t a[2][4][2];  // base tile: [row fragment][step][half]
  int prow = 0;     // row of x / y / idx that holds this launch's token `lane`

  // Activations slice of k-block kb -> LDS, rows in token order; rows >= T repeat row T-1 (they
  // only feed output columns that are never stored).  Addresses are a wavefront-uniform base plus
  // one 32-bit lane offset.
  auto issue_x = [&](int kb, int lane_r) {
    const char* xb = (const char*)(P.x + (size_t)kb * DZ_KBLOCK);
    const int c = lane_r & 31;
    if constexpr (MULTI) {
#pragma unroll
      for (int i = 0; i < NX; ++i) {
        const int t = min(2 * i + (lane_r >> 5), Tc - 1);
        const int row = __builtin_amdgcn_ds_bpermute(t << 2, prow);
        const unsigned off = (unsigned)row * Kb + (unsigned)((c ^ (t & 15)) << 4);
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(xb + off),
                                         (__attribute__((address_space(3))) void*)(xw + 2 * i * DZ_KBLOCK),
                                         16, 0, 0);
      }
    } else {
#pragma unroll
      for (int i = 0; i < NX; ++i) {
        const int t = min(2 * i + (lane_r >> 5), Tc - 1);
        const unsigned off = (unsigned)(tok0 + t) * Kb + (unsigned)((c ^ (t & 15)) << 4);
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(xb + off),
                                         (__attribute__((address_space(3))) void*)(xw + 2 * i * DZ_KBLOCK),
                                         16, 0, 0);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  // The 32 x 256 base tile: 16 loads of 16 bytes per lane.  One load covers 8 rows x 128 bytes
  // (a request for 16 rows x 64 bytes moves 15 % fewer bytes per second on this memory system):
  // lane (ga, jj) fetches row 16*s + 8*half + jj % 8, 16-byte chunk 2*ga + jj / 8 of the step's 128
  // bytes.  The matrix instruction wants row jj in lane jj, so before use the upper eight lanes of
  // each group of 16 trade places between the two halves (`base_operands`).
  auto issue_base = [&](int kb, int lane_r, const int s_lo, const int s_hi) {   // row fragments s_lo .. s_hi - 1
    static_assert(sizeof(a[0]) / sizeof(u4_t) == BASE_FRAG_LOADS, "one request per 16-byte register group of a row fragment");
    if constexpr (TILED) {
      // the tile is 16 requests of 1 KiB, each already in the order the matrix instruction takes
      const char* tb = (const char*)P.wb + dz_base_tile_offset(np, kb, P.NKB) + ((size_t)lane_r << 4);
#pragma unroll
      for (int s = s_lo; s < s_hi; ++s)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            const u4_t* q = (const u4_t*)(tb + dz_base_frag_offset(s, j, h));
            if constexpr (SHARED_TILE) a[s][j][h] = *q;
            else a[s][j][h] = __builtin_nontemporal_load(q);
          }
      return;
    }
    const char* wbb = (const char*)(P.wb + (size_t)n0 * P.K + (size_t)kb * DZ_KBLOCK);
    const unsigned loff = (unsigned)(lane_r & 7) * Kb + (unsigned)(lane_r >> 4) * 32u + (unsigned)((lane_r >> 3) & 1) * 16u;
    // One chunk of tokens: the tile is read once in the whole launch and is requested as streaming
    // data.  Several chunks: the workgroups of the other chunks of this (n-pair, K-slice) read it
    // too, a moment later, on the same XCD; an ordinary request leaves it in that L2 for them
    // (measured on 64 tokens / 4-bit deltas: 24 % more bytes from memory than the layer holds
    // when every chunk streams the tile for itself).
#pragma unroll
    for (int s = s_lo; s < s_hi; ++s)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const u4_t* q = (const u4_t*)(wbb + (size_t)(16 * s + 8 * h) * Kb + loff + 128 * j);
          if constexpr (SHARED_TILE) a[s][j][h] = *q;
          else a[s][j][h] = __builtin_nontemporal_load(q);
        }
  };
  // u: row jj, chunk 2*ga of step j (lanes jj < 8 have it in the first half's register, lanes
  // jj >= 8 take it from lane jj - 8 of the second half's); v: row jj, chunk 2*ga + 1.
  auto base_operands = [&](const u4_t& ra, const u4_t& rb, h8_t& u, h8_t& v) {
    H8U uu, vv;
    if constexpr (TILED) {
      uu.v = ra; vv.v = rb;
      u = uu.h; v = vv.h;
      return;
    }
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      // row_ror:8 inside each group of 16 lanes; bank mask 0xC = lanes 8..15, 0x3 = lanes 0..7
      uu.u[d] = (uint32_t)__builtin_amdgcn_update_dpp((int)ra[d], (int)rb[d], 0x128, 0xF, 0xC, false);
      vv.u[d] = (uint32_t)__builtin_amdgcn_update_dpp((int)rb[d], (int)ra[d], 0x128, 0xF, 0x3, false);
    }
    u = uu.h;
    v = vv.h;
  };

  // token ids: lane t keeps the key of token t (0 = base only, id + 1 otherwise, INT_MAX for
  // padding lanes); mdelta marks the tokens that carry a delta.  Both are set in the first pass
  // of the loop over k-blocks.
  int key = 0x7fffffff;
  unsigned long long mdelta = 0;
  // Nothing from HBM can be requested before the token ids are in (which deltas to fetch depends
  // on them), and a request queued behind this kernel's own flood of weight loads takes several
  // microseconds: the ids go out with the round's activations (L2 hits) and are awaited with them.
  // They are requested outside the compiler's bookkeeping -- it would wait for every LDS-direct
  // load in flight, being unable to tell them apart -- which needs care: the compiler takes the
  // destination register of an asm statement for valid the moment the statement ends and is free
  // to spill or copy it while the load is still in flight.  So either the ids go to LDS and no
  // register is involved until they are read back (IDL: launches of one call), or the load and its
  // wait sit in one statement (the batched launches, where the first way measured 1 % slower).
  long long id = -1;
  if constexpr (IDL) {
    // Order: ids -> LDS, activations, then (EARLY) half the base tile; "at most NX (+ 8) requests
    // outstanding" then means the ids have arrived.  EARLY, launches of a single turn: every
    // workgroup starts on an idle memory system and would leave it idle until its ids are in, so
    // the first row fragment of the base tile, which does not depend on the ids, is requested right
    // away.  (In launches of several turns the later workgroups start while others stream, and
    // extra requests in front of the first batch of deltas cost as much as they gain there.)
    // LDS layout of the ids: 64 low words, 64 high words, behind the activation slices.
    const unsigned id_lds = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char*)smem +
                            (unsigned)(WK32 * TP * DZ_KBLOCK * 2 + wave * 512);
    if (lane < Tc) {
      prow = MULTI ? P.perm[tok0 + lane] : tok0 + lane;
      const char* ip = (const char*)(P.idx + prow);
      asm volatile(
          "s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %2, off\n\t"
          "s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %3, off"
          :
          : "s"(id_lds), "s"(id_lds + 256u), "v"(ip), "v"(ip + 4)
          : "memory", "m0");
    }
    __builtin_amdgcn_sched_barrier(0);
    {
      // round 0's activations (a wavefront without a k-block fetches a slice it will not use)
      int lane_0 = lane;
      asm volatile("" : "+v"(lane_0));
      issue_x(min(kb_lo + wave, P.NKB - 1), lane_0);
      if (EARLY) issue_base(min(kb_lo + wave, P.NKB - 1), lane_0, 0, 1);
      // nothing of the compiler's between the two waits: a scalar load scheduled in there would
      // be waited for by the lgkmcnt(0) below instead of behind the ids' latency
      __builtin_amdgcn_sched_barrier(0);
      asm volatile("s_waitcnt vmcnt(%0)" : : "n"(NX + EARLY_LOADS) : "memory");
    }
    {
      unsigned lo, hi;   // read and wait in one statement
      asm volatile("ds_read_b32 %0, %2\n\tds_read_b32 %1, %2 offset:256\n\ts_waitcnt lgkmcnt(0)"
                   : "=&v"(lo), "=&v"(hi)
                   : "v"(id_lds + 4u * (unsigned)lane)
                   : "memory");
      if (lane < Tc) id = (long long)(((unsigned long long)hi << 32) | lo);
    }
  } else {
    // Activations first, then the ids and the wait for everything so far in one statement: the
    // ids return behind the activations, which are L2 hits and long in by then.
    const char* ip = nullptr;
    if (lane < Tc) {
      prow = MULTI ? P.perm[tok0 + lane] : tok0 + lane;
      ip = (const char*)(P.idx + prow);
    }
    {
      int lane_0 = lane;
      asm volatile("" : "+v"(lane_0));
      issue_x(min(kb_lo + wave, P.NKB - 1), lane_0);
    }
    __builtin_amdgcn_sched_barrier(0);
    if (lane < Tc)
      asm volatile("global_load_dwordx2 %0, %1, off\n\ts_waitcnt vmcnt(0)" : "+v"(id) : "v"(ip) : "memory");
  }
  __builtin_amdgcn_sched_barrier(0);

  for (int r = 0; r < nrounds; ++r) {
    const int kb = kb_lo + r * WK32 + wave;
    const bool active = kb < kb_hi;  // wavefront-uniform
    // Per-round copy of the lane id that the optimiser cannot prove loop-invariant: otherwise it
    // precomputes every load offset of the round outside the loop and spills them.
    int lane_r = lane;
    asm volatile("" : "+v"(lane_r));

    // the activations do not depend on the ids: they go first, the ids are awaited behind them
    if (r > 0 && active) {
      issue_x(kb, lane_r);
      if (EARLY) issue_base(kb, lane_r, 0, 1);
    }
    if (r == 0) {
      if (lane < Tc) {
        key = (id < 0 || id >= P.S) ? 0 : (int)id + 1;
        if ((id < -1 || (P.S > 0 && id >= P.S)) && np == 0 && kc == 0 && wave == 0) atomicOr(P.status, 1u);   // without slots the ids mean nothing
      }
      // tokens that carry a delta; lanes >= T never match
      mdelta = __builtin_amdgcn_ballot_w64(key != 0 && key != 0x7fffffff);
      DZ_TS(1);
    }
    if (!active) continue;

    // ---- delta walk (scalar state only).  The distinct deltas of the batch are visited in order
    // of their first token, G at a time; `pop` takes the next one and returns the output columns
    // (tokens) that belong to it.  The loader runs two batches ahead of the consumer.
    Frag<BITS> ring[2][G];
    // PRE: scales of the batch, one fp16 per lane and register: lane l holds row n0 + l%32 of the
    // k-block's scale group l/32 (register 0) and, when a k-block spans four groups (PRE == 2:
    // groups of 64), l/32 + 2 (register 1); a step's scale reaches the lane that multiplies with it
    // through a cross-lane move, not through memory
    unsigned rsc[2][G][2];
    unsigned long long ld_m = mdelta, use_m = mdelta;
    auto pop = [&](unsigned long long& m, int& kd, unsigned long long& cols) {
      const int l = __builtin_ctzll(m);
      kd = __builtin_amdgcn_readlane(key, l);
      cols = __builtin_amdgcn_ballot_w64(key == kd);
      m &= ~cols;
    };
    // Always G requests, so that the number of loads in flight is known at compile time and the
    // waits in front of each use can be exact: a slot without a delta re-reads 16 bytes.
    auto load_batch = [&](Frag<BITS> (&slot)[G], unsigned (&rs)[G][2]) {
#pragma unroll
      for (int g = 0; g < G; ++g) {
        int kd = 1;
        unsigned long long cols;
        const bool real = ld_m != 0;
        if (real) pop(ld_m, kd, cols);
        slot[g] = load_frag<BITS>(P, kd - 1, np, kb, real ? lane_r : 0);
        if (PRE) {
          const int ls = real ? lane_r : 0;
          const int gb0 = (kb * DZ_KBLOCK) / P.gs + (ls >> 5);
          const _Float16* sb = P.scales + (size_t)(kd - 1) * P.scales_slot + n0 + (ls & 31);
#pragma unroll
          for (int i = 0; i < PRE; ++i)   // PRE requests: scale groups gb0 (and gb0 + 2 for groups of 64)
            rs[g][i] = *(const unsigned short*)(sb + (size_t)min(gb0 + 2 * i, P.G - 1) * P.N);
        }
      }
    };

    // ---- issue order: activations (L2 -> LDS, above), packed deltas of two batches, base tile
    load_batch(ring[0], rsc[0]);
    load_batch(ring[1], rsc[1]);
    __builtin_amdgcn_sched_barrier(0);
    if (r == 0) DZ_TS(2);
    // Loads return in order and the activations were requested first: once only the loads issued
    // after them can be outstanding, this wavefront's LDS slice is complete.  (The compiler does
    // not order LDS reads after LDS-direct loads by itself.)
    {
      constexpr int later = 2 * BATCH_LOADS + EARLY_LOADS;   // both batches: words and, with PRE, scales; the early fragment of the base tile
      // s_waitcnt immediate on gfx9: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[5:4] << 14
      // lgkmcnt(0) as well: the compiler books an LDS-direct load on both counters and, while it
      // believes one outstanding, turns every later vmcnt wait into vmcnt(0)
      __builtin_amdgcn_s_waitcnt((later & 15) | (7 << 4) | (0 << 8) | ((later >> 4) << 14));
      asm volatile("" ::: "memory");
    }
    __builtin_amdgcn_sched_barrier(0);
    if (r == 0) DZ_TS(3);

    auto ldsB = [&](int tt, int j, h8_t& lo, h8_t& hi) {
      const char* p = (const char*)xw + (j >> 1) * 256;
      lo = *(const h8_t*)(p + boff[tt][(j & 1) * 2 + 0]);
      hi = *(const h8_t*)(p + boff[tt][(j & 1) * 2 + 1]);
    };
    // one batch: for every column tile that holds tokens of these deltas, one pass over the four
    // steps in which each operand read feeds all deltas of the batch
    auto consume = [&](Frag<BITS> (&slot)[G], unsigned (&rs)[G][2]) {
      int kd[G];
      unsigned long long cols[G];
      unsigned long long any = 0;
#pragma unroll
      for (int g = 0; g < G; ++g) {
        kd[g] = 1;
        cols[g] = 0;
        if (use_m) pop(use_m, kd[g], cols[g]);
        any |= cols[g];
      }
#pragma unroll
      for (int tt = 0; tt < TT; ++tt) {
        if (((any >> (16 * tt)) & 0xffffull) == 0) continue;
        f4_t t0[G], t1[G];
#pragma unroll
        for (int g = 0; g < G; ++g) {
          t0[g] = (f4_t){0.f, 0.f, 0.f, 0.f};
          t1[g] = (f4_t){0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          h8_t blo, bhi;
          ldsB(tt, j, blo, bhi);
          const h16_t B = __builtin_shufflevector(blo, bhi, 0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12,
                                                  13, 14, 15);
#pragma unroll
          for (int g = 0; g < G; ++g) {
            if ((cols[g] >> (16 * tt)) & 0xffffull) {
              h8_t A0, A1;
              if (BITS == 2) {
                unpack2(slot[g].code[0][j], MAGIC, A0, A1);
              } else {
                A0 = unpack4(slot[g].code[(BITS == 2) ? 0 : (j >> 1)][2 * (j & 1) + 0], MAGIC);
                A1 = unpack4(slot[g].code[(BITS == 2) ? 0 : (j >> 1)][2 * (j & 1) + 1], MAGIC);
              }
              if (PRE) {
                // the lane's operand rows are n0 + jj and n0 + 16 + jj; one scale per (row, K-group)
                const int gk = (kb * DZ_KBLOCK + 64 * j) / P.gs - (kb * DZ_KBLOCK) / P.gs;   // 0..3
                int v = (int)rs[g][0];
                if (PRE == 2) {
                  const unsigned pick = 0u - (unsigned)((gk >> 1) & 1);   // all ones: groups 2, 3
                  v = (int)((rs[g][1] & pick) | (rs[g][0] & ~pick));
                }
                const int src = (jj + ((gk & 1) << 5)) << 2;
                const unsigned short s0 = (unsigned short)__builtin_amdgcn_ds_bpermute(src, v);
                const unsigned short s1 = (unsigned short)__builtin_amdgcn_ds_bpermute(src + 64, v);
                A0 *= __builtin_bit_cast(_Float16, s0);
                A1 *= __builtin_bit_cast(_Float16, s1);
              }
              const int mw = (int)slot[g].meta[j];
              t0[g] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(A0, B, t0[g], mw, 0, 0);
              t1[g] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(A1, B, t1[g], mw, 0, 1);
            }
          }
          // keep the steps in program order: hoisting the next steps' operand reads and unpacking
          // above this point costs more registers than the latency it hides
          __builtin_amdgcn_sched_barrier(0);
        }
        // keep only the columns of each delta.  A 0/1 multiplier is enough: a column is computed
        // from that token's activations alone, so a non-finite value can only come from, and stay
        // in, the column of the token that supplied it.
#pragma unroll
        for (int g = 0; g < G; ++g) {
          const float in = (float)((unsigned)(cols[g] >> (16 * tt + jj)) & 1u);
          accd[0][tt] += t0[g] * in;
          accd[1][tt] += t1[g] * in;
        }
      }
    };

    // first two batches in straight-line code; their data arrives before the base tile does
    consume(ring[0], rsc[0]);
    if (ld_m) load_batch(ring[0], rsc[0]);
    __builtin_amdgcn_sched_barrier(0);
    if (HAS_BASE) issue_base(kb, lane_r, EARLY ? 1 : 0, 2);
    __builtin_amdgcn_sched_barrier(0);
    consume(ring[1], rsc[1]);
    if (ld_m) load_batch(ring[1], rsc[1]);
    // ---- base: dense matrix-core product over all token tiles
    if (HAS_BASE) {
#pragma unroll
      for (int tt = 0; tt < TT; ++tt)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          // activations of chunks 2*ga and 2*ga + 1 of step j (the base operands' columns)
          const char* px = (const char*)xw + (tt * 16 + jj) * (DZ_KBLOCK * 2) + (j >> 1) * 256;
          const int c0 = (j & 1) * 8 + 2 * ga;
          const h8_t blo = *(const h8_t*)(px + ((c0 ^ jj) << 4));
          const h8_t bhi = *(const h8_t*)(px + (((c0 + 1) ^ jj) << 4));
#pragma unroll
          for (int s = 0; s < 2; ++s) {
            h8_t u, v;
            base_operands(a[s][j][0], a[s][j][1], u, v);
            accb[s][tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(u, blo, accb[s][tt], 0, 0, 0);
            accb[s][tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(v, bhi, accb[s][tt], 0, 0, 0);
          }
        }
    }
    // more than 2*G deltas: keep going, two batches per turn
    while (use_m) {
      consume(ring[0], rsc[0]);
      if (ld_m) load_batch(ring[0], rsc[0]);
      if (use_m) {
        consume(ring[1], rsc[1]);
        if (ld_m) load_batch(ring[1], rsc[1]);
      }
    }
    // Every load of this round has been consumed by now; saying so keeps the waits of the next
    // round exact (the compiler would otherwise assume refill loads may still be pending).
    __builtin_amdgcn_s_waitcnt(0 | (7 << 4) | (15 << 8));
    if (r == 0) DZ_TS(4);
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
  int yrow[TT];   // output row of column tt*16 + jj
#pragma unroll
  for (int tt = 0; tt < TT; ++tt) yrow[tt] = __builtin_amdgcn_ds_bpermute((tt * 16 + jj) << 2, prow);
  auto final_store = [&](int s, int tt, f4_t v) {
    if (tt * 16 + jj < Tc) {
      _Float16* yp = P.y + (size_t)yrow[tt] * P.ldy + n0 + 16 * s + 4 * ga;
      if (P.accumulate) {
        const h4_t o = *(const h4_t*)yp;
        v += (f4_t){(float)o[0], (float)o[1], (float)o[2], (float)o[3]};
      }
      const h4_t o = {(_Float16)v[0], (_Float16)v[1], (_Float16)v[2], (_Float16)v[3]};
      *(h4_t*)yp = o;
    }
  };
  // partial sums of one K-slice: [chunk][slice][n-pair][item][4 values][64 lanes] floats.  They
  // are written and read with agent-scope accesses (write-through / cache-bypassing), so that no
  // whole-cache write-back or invalidate is needed to pass them between XCDs.
  auto part_ptr = [&](int kc2, int item) -> float* {
    return P.partials + (((size_t)(ch * P.nsplit + kc2) * P.NP + np) * (2 * TT) + item) * 256 + lane;
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
  // The partial sums carry their own "ready" mark: a slot of the workspace is all zero bits while
  // empty, and a sum of +0.0 is written as -0.0.  The workgroups of the K-slices 0 .. nsplit - 2
  // store theirs and leave at once.  The workgroup of the last K-slice (dispatched after them) reads
  // the slots until every value is in, adds them in slice order, its own last, writes y and empties
  // the slots again.  The wait is bounded: if a slot stays empty the launch reports it in the
  // status word instead of spinning for ever.
  if (kc != P.nsplit - 1) {
    if (has_item) {
      unsigned* pp = (unsigned*)part_ptr(kc, wave);
      const u4_t sb = __builtin_bit_cast(u4_t, sum);
      __hip_atomic_store(pp, sb[0] ? sb[0] : 0x80000000u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(pp + 64, sb[1] ? sb[1] : 0x80000000u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(pp + 128, sb[2] ? sb[2] : 0x80000000u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(pp + 192, sb[3] ? sb[3] : 0x80000000u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    DZ_TS(8);
    return;
  }
  if (has_item) {
    f4_t tot = {0.f, 0.f, 0.f, 0.f};
    const int nother = P.nsplit - 1;
    for (int k0 = 0; k0 < nother; k0 += 4) {
      unsigned v[4][4];
      int spins = 0;
      for (;;) {
        unsigned all = 0xffffffffu;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const unsigned* pp = (const unsigned*)part_ptr(min(k0 + u, nother - 1), wave);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            v[u][e] = __hip_atomic_load(pp + 64 * e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            all = v[u][e] ? all : 0u;
          }
        }
        if (__builtin_amdgcn_ballot_w64(all == 0u) == 0ull) break;
        if (++spins > DZ_SPIN_LIMIT) {
          if (lane == 0) atomicOr(P.status, 2u);
          break;
        }
        __builtin_amdgcn_s_sleep(1);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u)
        if (k0 + u < nother) {
#pragma unroll
          for (int e = 0; e < 4; ++e) tot[e] += __builtin_bit_cast(float, v[u][e]);
          unsigned* pp = (unsigned*)part_ptr(k0 + u, wave);
#pragma unroll
          for (int e = 0; e < 4; ++e) __hip_atomic_store(pp + 64 * e, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    tot += sum;
    store_item(tot);
  }
  DZ_TS(9);
}

// workgroup -> (n-pair, k-chunk, token chunk); the chunks of one n-pair are dealt to one XCD so
// that their partial sums can meet in that XCD's L2.  A launch may carry up to 4 chunks of 32 tokens
// (33..128 tokens, grouped by delta id): the workgroups of the chunks of one (n-pair, k-chunk)
// follow each other on the same XCD, so the base tile they all read comes from HBM once.
template <int BITS, int TT, int PRE, int BASE, bool EARLY>
__global__ __launch_bounds__(64 * WK32, 2) void dz_mdl32_kernel(const MdlParams P) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int xcd = blockIdx.x & 7, q = blockIdx.x >> 3;
  const int per = P.nsplit * P.nchunk, rem = q % per;
  const int np = (q / per) * 8 + xcd, kc = rem / P.nchunk, ch = rem % P.nchunk;
  if (np >= P.NP) return;
  mdl32_body<BITS, TT, PRE, BASE, EARLY, true>(P, np, kc, ch, smem);
}

// Several layer calls that share tokens, K and the slot table (the projections a fused layer
// would hold in one weight: q/k/v, gate/up) in one launch: the n-pairs of the calls are numbered
// through, a workgroup picks its call by its n-pair.  One call's tail (reduction, stores) then
// overlaps the next one's loads instead of leaving the memory system idle between launches.
template <int BITS, int TT, int PRE, int BASE>
__global__ __launch_bounds__(64 * WK32, 2) void dz_mdl32_batch_kernel(const MdlBatch B) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int xcd = blockIdx.x & 7, q = blockIdx.x >> 3;
  const int per = B.p[0].nsplit * B.p[0].nchunk, rem = q % per;
  const int npg = (q / per) * 8 + xcd, kc = rem / B.p[0].nchunk, ch = rem % B.p[0].nchunk;
  if (npg >= B.np_end[DZ_MAX_BATCH - 1]) return;
  // wavefront-uniform choice among the calls (np_end of unused entries repeats the total)
  const int j = (npg >= B.np_end[0]) + (npg >= B.np_end[1]) + (npg >= B.np_end[2]);
  const int first = j == 0 ? 0 : B.np_end[j - 1];
  mdl32_body<BITS, TT, PRE, BASE, false, false>(B.p[j], npg - first, kc, ch, smem);
}

// K split over workgroups: aim at two resident workgroups per CU (512) with few rounds each.  The
// split depends on the shapes only, not on the form of the base weight: both forms give the same
// bits.  (q + k + v of 4096 rows each as 384 unsplit workgroups of four rounds instead of 768 of two:
// the same time over tiles, slower over rows.)
static int choose_split(const MdlParams& P, int np_total, int ksplit_override) {
  int nsplit = ksplit_override;
  if (nsplit <= 0) {
    nsplit = 1;
    const int max_split = (P.NKB + WK32 - 1) / WK32;  // at least one round of 4 k-blocks each
    while (nsplit < max_split && (long long)np_total * nsplit * P.nchunk < 512) ++nsplit;
  }
  if (nsplit > 16 / P.nchunk) nsplit = 16 / P.nchunk;   // the workspace holds 16 sets of partial sums
  if (nsplit > P.NKB) nsplit = P.NKB;
  return nsplit;
}

}  // namespace

// Launch geometry of the fused kernel for a batch of calls (P[j].NP, NKB and nchunk set): K is
// split as far as the launch needs to fill the GPU -- a batch counts the n-pairs of all its calls
// (gate + up together fill it without a split, and then exchange no partial sums at all).
// K-slices need not be whole rounds of WK32 k-blocks: a wavefront without a k-block in a slice's
// last round idles; the slices are of equal length up to one k-block.
void dz_mdl32_geometry(const MdlParams* P, int nprob, int ksplit_override, int* nsplit_out, int* cb_out, int* grid_out) {
  int np_all = 0;
  for (int j = 0; j < nprob; ++j) np_all += P[j].NP;
  const int nsplit0 = choose_split(P[0], np_all, ksplit_override);
  const int cb = (P[0].NKB + nsplit0 - 1) / nsplit0;
  const int nsplit = (P[0].NKB + cb - 1) / cb;
  *nsplit_out = nsplit;
  *cb_out = cb;
  *grid_out = (np_all + 7) / 8 * 8 * nsplit * P[0].nchunk;
}

namespace {

template <int BITS, int TT>
int launch32(MdlBatch B, int nprob, int pre, hipStream_t st, int ksplit_override) {
  int nsplit, cb, grid;
  dz_mdl32_geometry(B.p, nprob, ksplit_override, &nsplit, &cb, &grid);
  int np_total = 0;
  bool has_base = B.p[0].wb != nullptr;
  for (int j = 0; j < DZ_MAX_BATCH; ++j) {
    if (j < nprob) {
      B.p[j].cb = cb;
      B.p[j].nsplit = nsplit;
      np_total += B.p[j].NP;
      if ((B.p[j].wb != nullptr) != has_base) return DZ_EINVAL;   // all with a base weight or none
      if (B.p[j].base_tiled != B.p[0].base_tiled) return DZ_EINVAL; // ... and all in the same layout
    }
    B.np_end[j] = np_total;
  }
  const size_t lds = (size_t)WK32 * 16 * TT * DZ_KBLOCK * 2 + WK32 * 512;   // activation slices + the token ids
  // single launches of at most one turn (two workgroups per CU) take the variant that requests half
  // the base tile before the ids are in (not over tiles with several chunks of tokens: no gain there)
  const bool tiled = has_base && B.p[0].base_tiled != 0;
  const bool early = nprob == 1 && has_base && grid <= 2 * dz_cu_count();
  static std::atomic<unsigned long long> attr_done[78];   // one per kernel: 3 x 13 variants, single and batched
  auto go = [&](auto kern, auto bkern, int slot) -> int {
    const void* f = nprob == 1 ? (const void*)kern : (const void*)bkern;
    if (!dz_lds_limit_once(attr_done[2 * slot + (nprob > 1)], f, (int)lds)) return DZ_ELAUNCH;
    if (nprob == 1) hipLaunchKernelGGL(kern, dim3(grid), dim3(64 * WK32), lds, st, B.p[0]);
    else hipLaunchKernelGGL(bkern, dim3(grid), dim3(64 * WK32), lds, st, B);
    return DZ_OK;
  };
  // several chunks of tokens (33 .. 128 tokens, always two token tiles): variants of their own
  const bool multi = B.p[0].nchunk > 1;
  auto pick = [&](auto pre_c) -> int {
    constexpr int PRE_ = decltype(pre_c)::value;
    const int s0 = 13 * PRE_;
    if constexpr (TT == 2) {
      if (multi) {
        if (!has_base) return go(dz_mdl32_kernel<BITS, TT, PRE_, 5, false>, dz_mdl32_batch_kernel<BITS, TT, PRE_, 5>, s0);
        if (tiled) return go(dz_mdl32_kernel<BITS, TT, PRE_, 4, false>, dz_mdl32_batch_kernel<BITS, TT, PRE_, 4>, s0 + 1);
        return early ? go(dz_mdl32_kernel<BITS, TT, PRE_, 3, true>, dz_mdl32_batch_kernel<BITS, TT, PRE_, 3>, s0 + 2)
                     : go(dz_mdl32_kernel<BITS, TT, PRE_, 3, false>, dz_mdl32_batch_kernel<BITS, TT, PRE_, 3>, s0 + 3);
      }
    }
    if (multi) return DZ_ESHAPE;   // more than 32 tokens always run with two token tiles
    if (!has_base) return go(dz_mdl32_kernel<BITS, TT, PRE_, 0, false>, dz_mdl32_batch_kernel<BITS, TT, PRE_, 0>, s0 + 4);
    if (tiled)
      return early ? go(dz_mdl32_kernel<BITS, TT, PRE_, 2, true>, dz_mdl32_batch_kernel<BITS, TT, PRE_, 2>, s0 + 8)
                   : go(dz_mdl32_kernel<BITS, TT, PRE_, 2, false>, dz_mdl32_batch_kernel<BITS, TT, PRE_, 2>, s0 + 5);
    return early ? go(dz_mdl32_kernel<BITS, TT, PRE_, 1, true>, dz_mdl32_batch_kernel<BITS, TT, PRE_, 1>, s0 + 6)
                 : go(dz_mdl32_kernel<BITS, TT, PRE_, 1, false>, dz_mdl32_batch_kernel<BITS, TT, PRE_, 1>, s0 + 7);
  };
  int rc = pre == 2 ? pick(std::integral_constant<int, 2>{}) : pre == 1 ? pick(std::integral_constant<int, 1>{})
                                                                       : pick(std::integral_constant<int, 0>{});
  if (rc) return rc;
  return hipGetLastError() == hipSuccess ? DZ_OK : DZ_ELAUNCH;
}

}  // namespace

// Launch of the fused kernel for one layer call or a batch of calls that share T, K, bits, the
// scale grouping and the token order; called by dz_multi_delta_linear[_batch].
int dz_launch_mdl32_batch(const MdlParams* P0, int nprob, int bits, int pre, hipStream_t st, int ksplit_override) {
  if (nprob < 1 || nprob > DZ_MAX_BATCH) return DZ_ESHAPE;
  MdlBatch B;
  for (int j = 0; j < DZ_MAX_BATCH; ++j) {
    B.p[j] = P0[j < nprob ? j : 0];
    B.p[j].nchunk = (P0[0].T + 31) / 32;
  }
  const int nchunk = B.p[0].nchunk, T = P0[0].T;
  if (nchunk < 1 || nchunk > 4) return DZ_ESHAPE;
  // several chunks of tokens are read through the token order, a single chunk never is: the
  // kernel variants are compiled for exactly these two cases
  for (int j = 0; j < nprob; ++j)
    if ((B.p[j].perm != nullptr) != (nchunk > 1)) return DZ_EINVAL;
  if (bits == 2) return T <= 16 ? launch32<2, 1>(B, nprob, pre, st, ksplit_override) : launch32<2, 2>(B, nprob, pre, st, ksplit_override);
  return T <= 16 ? launch32<4, 1>(B, nprob, pre, st, ksplit_override) : launch32<4, 2>(B, nprob, pre, st, ksplit_override);
}

int dz_launch_mdl32(const MdlParams& P0, int bits, int pre, hipStream_t st, int ksplit_override) {
  return dz_launch_mdl32_batch(&P0, 1, bits, pre, st, ksplit_override);
}

#ifdef DZ_TIMING
extern "C" void dz_set_timing_buffer32(void* p) { (void)hipMemcpyToSymbol(HIP_SYMBOL(g_dz_ts), &p, sizeof(p)); }
#endif
