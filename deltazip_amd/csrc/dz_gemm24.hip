// Prefill-sized multi-delta linear layer on the gfx950 matrix cores, deltas taken in packed form:
//   y[t, :] (+)= x[t, :] @ w_base^T + x[t, :] @ dequant(delta[slot(t)])^T
// for tokens grouped by delta slot (a table of row blocks, each with one slot).
//
// One workgroup (8 wavefronts, two per SIMD) computes 256 output features x 256 tokens of one row
// block; each wavefront owns 64 features x 128 tokens as 4 x 8 tiles of 16 x 16 (128 fp32
// accumulators, in ordinary vector registers: the sparse instruction does not accumulate in the
// accumulation registers).  64 features are two n-pairs of the delta: their packed words are
// unpacked and scaled once per slab and used for all eight token tiles (with 128 features x 64
// tokens per wavefront the same four n-pairs were unpacked by four wavefronts each).  K is walked in slabs of 64 columns; weight slab and activation slab go
// from global memory straight into LDS (two buffers, the next slab is on its way while this one is
// multiplied).  The delta's packed codes and 2-bit positions (native layout: 16 bytes per lane per
// 32 x 256 tile, already in operand order) are staged in LDS one k-block ahead, read back by the
// lanes that use them, unpacked to fp16(scale * (q - zero)) -- the reference's rounding point,
// qlinear_cuda.py:306-308 -- and fed to the 2:4-sparse v_smfmac_f32_16x16x64_f16 together with
// their positions: half the matrix-core time of a dense product, and no dequantised copy of the
// delta ever exists in memory.
//   2-bit deltas  one walk: every slab is multiplied by the base weight (v_mfma_f32_16x16x32_f16)
//                 and by the delta's 64 columns from the same activation operands; a block without
//                 a delta, or a call without a base weight, skips the half it does not have.
//   4-bit deltas  two walks into the same accumulators (two staged k-blocks of 4-bit words do not
//                 fit beside the slab buffers): base pass, then a delta pass with the activations
//                 in a ring of four stages.
// Rows of x and y are addressed through an optional token order (the output of the segment sort),
// so the batch is neither gathered nor scattered.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/dz_amd.h"
#include "dz_device.h"

namespace {

constexpr int BM = 256, BN = 256, BK = 64;
constexpr int SLAB = 256 * BK * 2;        // bytes of one operand slab in LDS
constexpr int GM = 4, GN = 8;             // tiles per XCD block

struct Gemm24Params {
  const _Float16* x;
  const _Float16* w;             // base weight: [N, K], or in tiles (w_tiled), or nullptr
  const u4_t* codes;
  const u4_t* meta;
  const _Float16* scales;
  long long codes_slot_u4, meta_slot_u4, scales_slot;
  const dz_gemm_tile* tiles;     // row blocks (device memory)
  const int* perm;               // token order or nullptr
  _Float16* y;
  int T, K, N, S, G, gslabs, accumulate, ldy, tiles_m, tiles_n, NKB, NP, m_first, w_tiled;   // gslabs: slabs per scale group
};

template <int BITS>
__global__ __launch_bounds__(512, 2) void dz_gemm24_kernel(const Gemm24Params P) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];   // [2 buffers][w slab | x slab]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wn = wave & 3, wq = wave >> 2;       // feature quarter (64), token half (128)
  const int li = lane & 15, lg = lane >> 4;
  const uint32_t MAGIC = magic_vgpr();

  // workgroup -> tile: XCD-local blocks of GM x GN tiles
  const int xcd = blockIdx.x & 7, q = blockIdx.x >> 3;
  const int sbn = (P.tiles_n + GN - 1) / GN, sbm = (P.tiles_m + GM - 1) / GM;
  const int sb = (q / (GM * GN)) * 8 + xcd, r = q % (GM * GN);
  // consecutive blocks -- the ones the eight XCDs work on at the same time -- walk the smaller
  // operand: the larger one is then fetched from memory once, and the smaller one, fetched once per
  // block row or column, is found in the last-level cache
  const int sbi = P.m_first ? sb % sbm : sb / sbn, sbj = P.m_first ? sb / sbm : sb % sbn;
  const int tm = sbi * GM + r / GN, tn = sbj * GN + r % GN;
  if (tm >= P.tiles_m || tn >= P.tiles_n) return;
  const int row_lo = P.tiles[tm].row_lo, row_hi = P.tiles[tm].row_hi, slot = P.tiles[tm].group;
  if (row_hi <= row_lo) return;                  // unused entry of the table
  const int n0 = tn * BN;
  const bool has_delta = slot >= 0 && slot < P.S;
  const int nslab1 = P.K / BK;
  const int nb = P.w ? nslab1 : 0, nd = has_delta ? nslab1 : 0, total = nb + nd;
  const unsigned Kb = (unsigned)P.K * 2u;
  // a wavefront whose 128 token rows lie beyond the block only helps with the loads
  const bool has_rows = row_lo + wq * 128 < row_hi;

  f4_t acc[4][8];   // [feature tile][token tile]
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int b = 0; b < 8; ++b) acc[a][b] = (f4_t){0.f, 0.f, 0.f, 0.f};

  // ---- slab loader.  A slab is 32 requests of 1 KiB (8 rows x 128 bytes); every wavefront issues 4
  // of the weight slab and 4 of the activation slab.  Lane l fills LDS row l/8, physical chunk l%8
  // with global chunk (l%8) ^ ((row >> 1) & 7): a 16-byte read is served 16 lanes per cycle, and
  // 16 consecutive rows then fall on 16 different bank groups.
  const int lr = lane >> 3;
  unsigned goff_w[4], goff_x[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int R = (wave * 4 + i) * 8 + lr;
    const int lc = (lane & 7) ^ ((R >> 1) & 7);
    goff_w[i] = (unsigned)min(n0 + R, P.N - 1) * Kb + (unsigned)lc * 16u;     // clamped rows: never stored
    if (P.w_tiled) {
      // Base weight in tiles: request f = 4 * wave + i is the 1 KiB fragment (feature tile f / 2,
      // half f % 2) of the slab, contiguous in memory and already in lane order; it lands at the
      // same place of the slab buffer.  (n-pairs beyond N repeat the last one: never stored.)
      const int f = wave * 4 + i;
      const int np = min(n0 / DZ_NPAIR + (f >> 2), P.NP - 1);
      goff_w[i] = ((unsigned)np * (unsigned)P.NKB * 16u + (unsigned)(((f >> 1) & 1) * 8 + (f & 1))) * 1024u + (unsigned)lane * 16u;
    }
    const int pos = min(row_lo + R, row_hi - 1);
    const int row = P.perm ? P.perm[pos] : pos;
    goff_x[i] = (unsigned)row * Kb + (unsigned)lc * 16u;
  }
  const __amdgpu_buffer_rsrc_t rw =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<_Float16*>(P.w ? P.w : P.x), 0, 0x7fffffff, 0x00020000);
  const __amdgpu_buffer_rsrc_t rx =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<_Float16*>(P.x), 0, 0x7fffffff, 0x00020000);
  // base pass: slab s -> buffer s & 1, [weight slab | activation slab]
  auto issue = [&](int s, int buf, bool with_w = true) {
    const int soff = s * (BK * 2);
    const int soff_w = P.w_tiled ? (s >> 2) * 16384 + (s & 3) * 2048 : soff;   // tile of the k-block, fragments of step s % 4
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      unsigned char* dst = smem + buf * (2 * SLAB) + (wave * 4 + i) * 1024;
      if (with_w)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, (__attribute__((address_space(3))) void*)dst, 16,
                                                 (int)goff_w[i], soff_w, 0, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, (__attribute__((address_space(3))) void*)(dst + SLAB), 16,
                                               (int)goff_x[i], soff, 0, 0);
    }
  };
  // delta pass: activation slab sd -> stage sd & 3 of a ring of four (the same 128 KiB)
  auto issue_xd = [&](int sd) {
    const int soff = sd * (BK * 2);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      unsigned char* dst = smem + (sd & 3) * SLAB + (wave * 4 + i) * 1024;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, (__attribute__((address_space(3))) void*)dst, 16,
                                               (int)goff_x[i], soff, 0, 0);
    }
  };

  // ---- packed delta operands: the 8 n-pairs (256 rows) of the workgroup's tile, one k-block at a
  // time, staged in LDS behind the ring: wavefront w fetches n-pair w -- 1 KiB of positions and 1
  // or 2 KiB of codes, already in lane order -- and every wavefront later reads the four n-pairs
  // of its own feature half from there.
  constexpr int DT = (BITS == 2) ? 2048 : 3072;          // staged bytes per n-pair
  unsigned char* const dstage = smem + 4 * SLAB;
  const int slot_c = has_delta ? slot : 0;
  const __amdgpu_buffer_rsrc_t rmeta = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<u4_t*>(P.meta + (size_t)slot_c * P.meta_slot_u4), 0, 0x7fffffff, 0x00020000);
  const __amdgpu_buffer_rsrc_t rcode = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<u4_t*>(P.codes + (size_t)slot_c * P.codes_slot_u4), 0, 0x7fffffff, 0x00020000);
  const int np_w = min(n0 / DZ_NPAIR + wave, P.NP - 1);
  auto issue_delta = [&](int kb, int stage = 0) {
    unsigned char* dst = dstage + stage * (8 * DT) + wave * DT;
    const int tile = np_w * P.NKB + kb;
    const int lo = lane * 16;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rmeta, (__attribute__((address_space(3))) void*)dst, 16, lo,
                                             tile * 1024, 0, 0);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rcode, (__attribute__((address_space(3))) void*)(dst + 1024), 16, lo,
                                             tile * (BITS == 2 ? 1024 : 2048), 0, 0);
    if (BITS == 4)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rcode, (__attribute__((address_space(3))) void*)(dst + 2048), 16,
                                               lo, tile * 2048 + 1024, 0, 0);
  };
  // scales of scale group gi: lane l fetches the scale of row 32*p + l % 32 of n-pair p (one
  // 2-byte load per n-pair, nothing depends on it until the group starts); the two values a lane
  // multiplies with -- rows i and 16 + i -- reach it by a cross-lane move when the group starts
  auto load_scales = [&](int (&raw)[2], int gi) {
    const _Float16* sp = P.scales + (size_t)slot * P.scales_slot + (size_t)min(gi, P.G - 1) * P.N;
#pragma unroll
    for (int p = 0; p < 2; ++p)
      raw[p] = *(const unsigned short*)(sp + min(n0 + wn * 64 + 32 * p + (lane & 31), P.N - 1));
  };
  auto spread_scales = [&](h2_t (&sc)[2], const int (&raw)[2]) {
#pragma unroll
    for (int p = 0; p < 2; ++p) {
      const unsigned lo = (unsigned)__builtin_amdgcn_ds_bpermute(li << 2, raw[p]) & 0xffffu;
      const unsigned hi = (unsigned)__builtin_amdgcn_ds_bpermute((16 + li) << 2, raw[p]);
      H2U u;
      u.u = lo | (hi << 16);
      sc[p] = u.h;
    }
  };

  // ---- operand addresses: lane (i = lane % 16, g = lane / 16) reads row i of a 16-row tile, chunk
  // 4*h + g of the slab row (columns 32*h + 8*g ..): the dense operand order of two 16x16x32
  // products, and the order the sparse product expects of its dense operand
  int foff[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) foff[h] = (((4 * h + lg) ^ ((li >> 1) & 7)) << 4);
  const int wrow = (wn * 64 + li) * 128, xrow = (wq * 128 + li) * 128;
  // weight operand of half h, feature tile a: woff[h] + a * 2048 into the weight slab.  From
  // fragments the lane takes the same columns 32*h + 8*g .. as from the row-major slab: they sit
  // in fragment g % 2 at lane position 16 * (2*h + g/2) + i (a fragment holds columns
  // 16*g' + 8*h' + e at position 16*g' + i), so the sums are the same whichever form is read.
  int woff[2];
#pragma unroll
  for (int h = 0; h < 2; ++h)
    woff[h] = P.w_tiled ? wn * 8192 + (lg & 1) * 1024 + ((2 * h + (lg >> 1)) * 16 + li) * 16 : wrow + foff[h];

  // The delta pass starts with activation slabs 0 and 1 and the first k-block's packed operands
  // already requested: at the start when there is no base pass, else during the last base slab
  // (which sits in buffer 1 -- the slab count is a multiple of 4 -- so ring stages 0 and 1, the
  // bytes of buffer 0, are free by then).
  auto delta_prologue = [&]() {
    issue_xd(0);
    issue_xd(1);
    issue_delta(0);
  };
  // ---- 2-bit deltas: one walk over K for every kind of row block.  Every slab is multiplied by the
  // base weight (dense instruction; skipped without a base weight) and by the delta's 64 columns
  // (sparse instruction; skipped for a block without a delta) from the same activation operands,
  // read from LDS once; the delta's packed words are staged one k-block ahead, alternating between
  // two stages.  A second walk would fetch every activation slab again and spend a barrier per
  // slab on half as much matrix work.
  constexpr bool FUSE = BITS == 2;   // (two staged k-blocks of 4-bit operands do not fit beside the slab buffers)
  if constexpr (FUSE) {
    const bool do_w = nb > 0, do_d = nd > 0;   // workgroup-uniform
    h2_t sc[2];
    int scn[2];
    if (total > 0) issue(0, 0, do_w);
    if (do_d) {
      issue_delta(0, 0);
      load_scales(scn, 0);
    }
    int gi = 0, gleft = P.gslabs;   // current scale group, slabs left in it
    for (int s = 0; s < (total > 0 ? nslab1 : 0); ++s) {
      const int buf = s & 1, kb = s >> 2, j = s & 3;
      __builtin_amdgcn_s_waitcnt(0x0070);   // vmcnt(0) lgkmcnt(0): this wavefront's share of slab s (and of the staged k-block)
      __syncthreads();
      if (s + 1 < nslab1) issue(s + 1, buf ^ 1, do_w);
      if (do_d) {
        // the packed words of k-block kb sit in stage kb & 1 (each lane's words j of its two
        // n-pairs are read from there slab by slab); the other stage, last read during k-block
        // kb - 1, takes k-block kb + 1
        if (j == 1 && kb + 1 < P.NKB) issue_delta(kb + 1, (kb + 1) & 1);
        if (gleft == P.gslabs) spread_scales(sc, scn);
        if (gleft == 1 && s + 1 < nslab1) load_scales(scn, gi + 1);
        if (--gleft == 0) {
          gleft = P.gslabs;
          ++gi;
        }
      }
      if (!has_rows) continue;
      const unsigned char* wb = smem + buf * (2 * SLAB);
      const unsigned char* xb = wb + SLAB;
      // Reads from LDS run ahead of the matrix instructions that use them: the slab's packed delta
      // words, its weight operands and the first two token tiles are requested at once, the delta
      // operands are unpacked while those reads are in flight, and every pair of token tiles is
      // requested before the products of the pair before it are issued.  (With all reads of a
      // group of tiles followed by all of its products, the eight wavefronts -- in step after the
      // barrier -- first queue at the LDS together and then at the matrix cores together.)
      uint32_t mw[2] = {0u, 0u}, cw[2] = {0u, 0u};
      if (do_d) {
        const unsigned char* dsrc = dstage + (kb & 1) * (8 * DT) + (wn * 2) * DT + lane * 16 + j * 4;
#pragma unroll
        for (int p = 0; p < 2; ++p) {
          mw[p] = *(const uint32_t*)(dsrc + p * DT);
          cw[p] = *(const uint32_t*)(dsrc + p * DT + 1024);
        }
      }
      // (read without a base weight too -- stale bytes that nothing uses: under a branch the
      // compiler no longer counts these requests when it waits for the packed words before them)
      h8_t fw[2][4];
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int a = 0; a < 4; ++a) fw[h][a] = *(const h8_t*)(wb + woff[h] + a * 2048);
      auto read_pair = [&](h16_t (&B)[2], int tg) {
#pragma unroll
        for (int b = 0; b < 2; ++b) {
          const h8_t lo = *(const h8_t*)(xb + xrow + (2 * tg + b) * 16 * 128 + foff[0]);
          const h8_t hi = *(const h8_t*)(xb + xrow + (2 * tg + b) * 16 * 128 + foff[1]);
          B[b] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15);
        }
      };
      h16_t Bc[2], Bn[2];
      read_pair(Bc, 0);
      __builtin_amdgcn_sched_barrier(0);
      h8_t A0[2], A1[2];
      if (do_d) {
#pragma unroll
        for (int p = 0; p < 2; ++p) {
          unpack2(cw[p], MAGIC, A0[p], A1[p]);
          A0[p] *= sc[p][0];
          A1[p] *= sc[p][1];
        }
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int tg = 0; tg < 4; ++tg) {
        if (tg < 3) read_pair(Bn, tg + 1);
        __builtin_amdgcn_sched_barrier(0);
        if (do_w) {
#pragma unroll
          for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int b = 0; b < 2; ++b) {
              const h8_t fxb = h == 0 ? __builtin_shufflevector(Bc[b], Bc[b], 0, 1, 2, 3, 4, 5, 6, 7)
                                      : __builtin_shufflevector(Bc[b], Bc[b], 8, 9, 10, 11, 12, 13, 14, 15);
#pragma unroll
              for (int a = 0; a < 4; ++a)
                acc[a][2 * tg + b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fw[h][a], fxb, acc[a][2 * tg + b], 0, 0, 0);
            }
        }
        if (do_d) {
#pragma unroll
          for (int p = 0; p < 2; ++p)
#pragma unroll
            for (int b = 0; b < 2; ++b) {
              acc[2 * p][2 * tg + b] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(A0[p], Bc[b], acc[2 * p][2 * tg + b], (int)mw[p], 0, 0);
              acc[2 * p + 1][2 * tg + b] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(A1[p], Bc[b], acc[2 * p + 1][2 * tg + b], (int)mw[p], 0, 1);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        if (tg < 3) {
          Bc[0] = Bn[0];
          Bc[1] = Bn[1];
        }
      }
    }
  }
  if constexpr (!FUSE) {
  // ---- 4-bit deltas: base pass, then delta pass
  if (nb > 0) issue(0, 0);
  else if (nd > 0) delta_prologue();
  for (int s = 0; s < nb; ++s) {
    const int buf = s & 1;
    // the slab of this turn was requested one turn ago: wait for this wavefront's share, then meet
    // the others (their shares are in, and nobody still reads the buffer filled next)
    __builtin_amdgcn_s_waitcnt(0x0070);   // vmcnt(0) lgkmcnt(0)
    __syncthreads();
    if (s + 1 < nb) issue(s + 1, buf ^ 1);
    else if (nd > 0) delta_prologue();
    if (!has_rows) continue;
    const unsigned char* wb = smem + buf * (2 * SLAB);
    const unsigned char* xb = wb + SLAB;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      h8_t fw[4], fx[8];
#pragma unroll
      for (int a = 0; a < 4; ++a) fw[a] = *(const h8_t*)(wb + woff[h] + a * 2048);
#pragma unroll
      for (int b = 0; b < 8; ++b) fx[b] = *(const h8_t*)(xb + xrow + b * 16 * 128 + foff[h]);
#pragma unroll
      for (int b = 0; b < 8; ++b)
#pragma unroll
        for (int a = 0; a < 4; ++a)
          acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fw[a], fx[b], acc[a][b], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);   // one half-slab's operands at a time
    }
  }
  // ---- delta pass
  Frag<BITS> cur[2];
  h2_t sc[2];
  int scn[2];
  if (nd > 0) load_scales(scn, 0);
  int gi = 0, gleft = P.gslabs;   // current scale group, slabs left in it
  for (int sd = 0; sd < nd; ++sd) {
    const int kb = sd >> 2, j = sd & 3;
    // Slab sd was requested three turns ago (slabs 0 and 1: before the pass).  Loads complete in
    // order and at least the 8 requests of slabs sd + 1 and sd + 2 follow it, so "at most 8
    // outstanding" means slab sd -- and anything requested before slab sd + 1, the staged k-block
    // included -- has arrived.  s_waitcnt immediate: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8].
    if (sd == 0 || sd + 1 >= nd) __builtin_amdgcn_s_waitcnt(0x0070);
    else if (sd + 2 >= nd) __builtin_amdgcn_s_waitcnt(0x0074);
    else __builtin_amdgcn_s_waitcnt(0x0078);
    wg_barrier_nofence();   // __syncthreads() would wait for the whole ring
    if (sd == 0) {
      if (2 < nd) issue_xd(2);
      if (3 < nd) issue_xd(3);
    } else if (sd + 3 < nd) {
      issue_xd(sd + 3);
    }
    if (j == 0) {
      // this k-block's packed operands were staged during the previous k-block
      const unsigned char* dsrc = dstage + (wn * 2) * DT + lane * 16;
#pragma unroll
      for (int p = 0; p < 2; ++p) {
        cur[p].meta = *(const u4_t*)(dsrc + p * DT);
        cur[p].code[0] = *(const u4_t*)(dsrc + p * DT + 1024);
        if (BITS == 4) cur[p].code[BITS == 2 ? 0 : 1] = *(const u4_t*)(dsrc + p * DT + 2048);
      }
    } else if (j == 1 && kb + 1 < P.NKB) {
      // every wavefront has taken its copy (they all passed the barrier above): refill
      issue_delta(kb + 1);
    }
    // scales: a scale group spans whole slabs (group size is a multiple of 64); the next group's
    // scales are requested during the last slab of the current one
    if (gleft == P.gslabs) spread_scales(sc, scn);
    if (gleft == 1 && sd + 1 < nd) load_scales(scn, gi + 1);
    if (--gleft == 0) {
      gleft = P.gslabs;
      ++gi;
    }
    if (!has_rows) continue;
    const unsigned char* xb = smem + (sd & 3) * SLAB;
    h8_t A0[2], A1[2];
    uint32_t mwp[2];
#pragma unroll
    for (int p = 0; p < 2; ++p) {
      // word j of the lane's four words; a compile-time index after unrolling over the four cases
      uint32_t cw0 = 0, cw1 = 0, mw = 0;
#pragma unroll
      for (int jj = 0; jj < 4; ++jj) {
        if (jj == j) {
          mw = cur[p].meta[jj];
          if (BITS == 2) {
            cw0 = cur[p].code[0][jj];
          } else {
            cw0 = cur[p].code[BITS == 2 ? 0 : (jj >> 1)][2 * (jj & 1) + 0];
            cw1 = cur[p].code[BITS == 2 ? 0 : (jj >> 1)][2 * (jj & 1) + 1];
          }
        }
      }
      if (BITS == 2) {
        unpack2(cw0, MAGIC, A0[p], A1[p]);
      } else {
        A0[p] = unpack4(cw0, MAGIC);
        A1[p] = unpack4(cw1, MAGIC);
      }
      A0[p] *= sc[p][0];
      A1[p] *= sc[p][1];
      mwp[p] = mw;
    }
#pragma unroll
    for (int tg = 0; tg < 2; ++tg) {
      h16_t B[4];
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const h8_t lo = *(const h8_t*)(xb + xrow + (4 * tg + b) * 16 * 128 + foff[0]);
        const h8_t hi = *(const h8_t*)(xb + xrow + (4 * tg + b) * 16 * 128 + foff[1]);
        B[b] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15);
      }
#pragma unroll
      for (int p = 0; p < 2; ++p)
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          acc[2 * p][4 * tg + b] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(A0[p], B[b], acc[2 * p][4 * tg + b], (int)mwp[p], 0, 0);
          acc[2 * p + 1][4 * tg + b] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(A1[p], B[b], acc[2 * p + 1][4 * tg + b], (int)mwp[p], 0, 1);
        }
    }
  }

  }   // 4-bit passes

  // ---- store: lane (i, g) holds features 4*g .. 4*g + 3 of tile a for token i of tile b
#pragma unroll
  for (int b = 0; b < 8; ++b) {
    const int pos = row_lo + wq * 128 + b * 16 + li;
    if (pos >= row_hi) continue;
    const int row = P.perm ? P.perm[pos] : pos;
    _Float16* yrow = P.y + (size_t)row * P.ldy + n0 + wn * 64 + 4 * lg;
    h4_t old[4];
    if (P.accumulate) {
      // all four reads of the token's row in flight together
#pragma unroll
      for (int a = 0; a < 4; ++a)
        old[a] = (n0 + wn * 64 + a * 16 + 4 * lg < P.N) ? *(const h4_t*)(yrow + a * 16) : (h4_t){0, 0, 0, 0};
    }
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      if (n0 + wn * 64 + a * 16 + 4 * lg >= P.N) continue;
      f4_t v = acc[a][b];
      if (P.accumulate) v += (f4_t){(float)old[a][0], (float)old[a][1], (float)old[a][2], (float)old[a][3]};
      const h4_t o = {(_Float16)v[0], (_Float16)v[1], (_Float16)v[2], (_Float16)v[3]};
      *(h4_t*)(yrow + a * 16) = o;
    }
  }
}

// Row blocks from segment offsets: segment k (k = 0: tokens without a delta, k >= 1: slot k - 1)
// is cut into blocks of at most 256 rows; unused entries of the table are left empty.
__global__ __launch_bounds__(1024) void dz_build_tiles_kernel(const int* __restrict__ seg_off, int S,
                                                              dz_gemm_tile* __restrict__ tiles, int max_tiles) {
  extern __shared__ int first[];    // first[k]: index of segment k's first block; first[S + 1]: total
  const int tid = threadIdx.x, nseg = S + 1;
  for (int k = tid; k < nseg; k += 1024) first[k + 1] = (seg_off[k + 1] - seg_off[k] + BM - 1) / BM;
  if (tid == 0) first[0] = 0;
  __syncthreads();
  if (tid == 0)
    for (int k = 1; k <= nseg; ++k) first[k] += first[k - 1];
  __syncthreads();
  for (int k = tid; k < nseg; k += 1024) {
    const int lo = seg_off[k], hi = seg_off[k + 1];
    for (int t = first[k], r = lo; r < hi && t < max_tiles; ++t, r += BM)
      tiles[t] = dz_gemm_tile{r, min(r + BM, hi), k - 1, 0};
  }
  for (int t = first[nseg] + tid; t < max_tiles; t += 1024) tiles[t] = dz_gemm_tile{0, 0, -1, 0};
}

}  // namespace

extern "C" int dz_build_tiles(const int32_t* seg_off, int S, dz_gemm_tile* tiles, int max_tiles, void* stream) {
  if (!seg_off || !tiles) return DZ_EINVAL;
  if (S < 0 || S > DZ_MAX_SLOTS_SEGMENT || max_tiles < 1) return DZ_ESHAPE;
  hipLaunchKernelGGL(dz_build_tiles_kernel, dim3(1), dim3(1024), (size_t)(S + 2) * 4, (hipStream_t)stream,
                     seg_off, S, tiles, max_tiles);
  return hipGetLastError() == hipSuccess ? DZ_OK : DZ_ELAUNCH;
}

static int multi_delta_gemm(const uint16_t* x, const uint16_t* w_base, bool w_tiled, const void* codes_stacked,
                            const void* meta_stacked, const void* scales_stacked, int S, int bits,
                            int group_size, const dz_gemm_tile* tiles, int ntiles, const int32_t* perm,
                            uint16_t* y, int T, int K, int N, int accumulate, int ldy, void* stream) {
  if (!x || !y || !tiles || ntiles < 1 || S < 0) return DZ_EINVAL;
  if (S > 0 && (!codes_stacked || !meta_stacked || !scales_stacked)) return DZ_EINVAL;
  size_t cb, mb, sb;
  int rc = dz_native_sizes(K, N, bits, group_size, &cb, &mb, &sb);
  if (rc) return rc;
  const int gs = (group_size == -1 || group_size == K) ? K : group_size;
  if (T < 1 || ldy < N || ldy % 4) return DZ_ESHAPE;
  if (((uintptr_t)x & 15) || ((uintptr_t)w_base & 15) || ((uintptr_t)y & 7)) return DZ_EALIGN;
  if ((unsigned long long)T * (unsigned)K * 2ull >= (1ull << 31) ||
      (unsigned long long)N * (unsigned)K * 2ull >= (1ull << 31))
    return DZ_ESHAPE;   // byte offsets inside one operand stay below 2^31 (buffer addressing)
  Gemm24Params P{};
  P.x = (const _Float16*)x; P.w = (const _Float16*)w_base; P.y = (_Float16*)y;
  P.codes = (const u4_t*)codes_stacked; P.meta = (const u4_t*)meta_stacked;
  P.scales = (const _Float16*)scales_stacked;
  P.codes_slot_u4 = (long long)(cb / 16); P.meta_slot_u4 = (long long)(mb / 16); P.scales_slot = (long long)(sb / 2);
  P.tiles = tiles; P.perm = perm;
  P.T = T; P.K = K; P.N = N; P.S = S; P.gslabs = gs / BK; P.G = K / gs; P.accumulate = accumulate; P.ldy = ldy;
  P.NKB = K / DZ_KBLOCK; P.NP = N / DZ_NPAIR;
  P.tiles_m = ntiles;
  P.tiles_n = (N + BN - 1) / BN;
  const int sbm = (P.tiles_m + GM - 1) / GM, sbn = (P.tiles_n + GN - 1) / GN;
  P.m_first = N > T;   // the weight is the larger operand
  P.w_tiled = (w_tiled && w_base) ? 1 : 0;
  const int nsb = (sbm * sbn + 7) / 8 * 8;
  const unsigned grid = (unsigned)nsb * GM * GN;
  // two slab buffers (= four ring stages of the delta pass) + the staged packed operands: one
  // k-block of 8 n-pairs at 4 bits, two of them (the single walk over K alternates) at 2 bits
  const size_t lds = 4 * SLAB + (bits == 2 ? 2 * 8 * 2048 : 8 * 3072);
  static std::atomic<unsigned long long> attr_done[2];
  auto go = [&](auto kern, int which) -> int {
    if (!dz_lds_limit_once(attr_done[which], (const void*)kern, (int)lds)) return DZ_ELAUNCH;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(512), lds, (hipStream_t)stream, P);
    return DZ_OK;
  };
  rc = bits == 2 ? go(dz_gemm24_kernel<2>, 0) : go(dz_gemm24_kernel<4>, 1);
  if (rc) return rc;
  return hipGetLastError() == hipSuccess ? DZ_OK : DZ_ELAUNCH;
}

extern "C" int dz_multi_delta_gemm(const uint16_t* x, const uint16_t* w_base, const void* codes_stacked,
                                   const void* meta_stacked, const void* scales_stacked, int S, int bits,
                                   int group_size, const dz_gemm_tile* tiles, int ntiles, const int32_t* perm,
                                   uint16_t* y, int T, int K, int N, int accumulate, int ldy, void* stream) {
  return multi_delta_gemm(x, w_base, false, codes_stacked, meta_stacked, scales_stacked, S, bits, group_size, tiles,
                          ntiles, perm, y, T, K, N, accumulate, ldy, stream);
}

extern "C" int dz_multi_delta_gemm_tiled(const uint16_t* x, const uint16_t* w_base_tiled, const void* codes_stacked,
                                         const void* meta_stacked, const void* scales_stacked, int S, int bits,
                                         int group_size, const dz_gemm_tile* tiles, int ntiles, const int32_t* perm,
                                         uint16_t* y, int T, int K, int N, int accumulate, int ldy, void* stream) {
  if (!w_base_tiled) return DZ_EINVAL;
  return multi_delta_gemm(x, w_base_tiled, true, codes_stacked, meta_stacked, scales_stacked, S, bits, group_size,
                          tiles, ntiles, perm, y, T, K, N, accumulate, ldy, stream);
}
