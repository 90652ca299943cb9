// Device helpers shared by the kernels of the multi-delta linear layer: vector types, the
// 2/4-bit code unpackers, the launch parameter block and the delta fragment loader.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "dz_layout.h"

typedef _Float16 h2_t __attribute__((ext_vector_type(2)));
typedef _Float16 h4_t __attribute__((ext_vector_type(4)));
typedef _Float16 h8_t __attribute__((ext_vector_type(8)));
typedef _Float16 h16_t __attribute__((ext_vector_type(16)));
typedef float f4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u2_t __attribute__((ext_vector_type(2)));

// Phase timestamps for kernel tuning; compiled out unless DZ_TIMING is defined.
#ifdef DZ_TIMING
static __device__ unsigned long long* g_dz_ts;
#define DZ_TS(i) do { if (lane == 0) g_dz_ts[((size_t)blockIdx.x * 16 + wave) * 16 + (i)] = wall_clock64(); } while (0)
#else
#define DZ_TS(i) do { } while (0)
#endif

// ---------------------------------------------------------------------------------------------
// code unpacking: packed 2/4-bit codes -> fp16 (q - zero), two values per instruction.
// OR-ing a code into the mantissa of 1024.0 (0x6400) gives 1024 + q * 2^shift exactly; one packed
// fma maps that to q - zero.
// ---------------------------------------------------------------------------------------------
union H2U { uint32_t u; h2_t h; };
union H8U { uint32_t u[4]; h8_t h; u4_t v; };

__device__ __forceinline__ uint32_t pkfma(uint32_t v, float mul, float add) {
  H2U a, r;
  a.u = v;
  h2_t m = {(_Float16)mul, (_Float16)mul};
  h2_t c = {(_Float16)add, (_Float16)add};
  r.h = __builtin_elementwise_fma(a.h, m, c);
  return r.u;
}

// v_and_or_b32 takes one scalar operand at most: the masks live in scalar registers, the magic
// constant in a vector register (the asm keeps the compiler from turning it back into a literal).
__device__ __forceinline__ uint32_t magic_vgpr() {
  uint32_t m = 0x64006400u;
  asm volatile("" : "+v"(m));
  return m;
}

// 2-bit: one word holds both fragments (s = 0, 1) of a step.
__device__ __forceinline__ void unpack2(uint32_t w, uint32_t MAGIC, h8_t& a0, h8_t& a1) {
  const uint32_t w2 = w >> 10;
  H8U r0, r1;
  r0.u[0] = pkfma((w & 0x00030003u) | MAGIC, 1.0f, -1026.0f);
  r0.u[1] = pkfma((w & 0x000C000Cu) | MAGIC, 0.25f, -258.0f);
  r0.u[2] = pkfma((w & 0x00300030u) | MAGIC, 0.0625f, -66.0f);
  r0.u[3] = pkfma((w & 0x00C000C0u) | MAGIC, 0.015625f, -18.0f);
  r1.u[0] = pkfma((w & 0x03000300u) | MAGIC, 0.00390625f, -6.0f);
  r1.u[1] = pkfma((w2 & 0x00030003u) | MAGIC, 1.0f, -1026.0f);
  r1.u[2] = pkfma((w2 & 0x000C000Cu) | MAGIC, 0.25f, -258.0f);
  r1.u[3] = pkfma((w2 & 0x00300030u) | MAGIC, 0.0625f, -66.0f);
  a0 = r0.h;
  a1 = r1.h;
}

// 4-bit: one word holds one fragment.
__device__ __forceinline__ h8_t unpack4(uint32_t w, uint32_t MAGIC) {
  const uint32_t w2 = w >> 8;
  H8U r;
  r.u[0] = pkfma((w & 0x000F000Fu) | MAGIC, 1.0f, -1032.0f);
  r.u[1] = pkfma((w & 0x00F000F0u) | MAGIC, 0.0625f, -72.0f);
  r.u[2] = pkfma((w2 & 0x000F000Fu) | MAGIC, 1.0f, -1032.0f);
  r.u[3] = pkfma((w2 & 0x00F000F0u) | MAGIC, 0.0625f, -72.0f);
  return r.h;
}

// Workgroup barrier without the memory fences of __syncthreads().  Those fences make the compiler
// wait for every outstanding vector-memory request, which empties a ring of prefetched loads at
// each barrier.  Callers order their LDS traffic themselves: an explicit s_waitcnt for LDS-direct
// loads and LDS reads in front of the barrier.
__device__ __forceinline__ void wg_barrier_nofence() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

struct MdlParams {
  const _Float16* x;
  const _Float16* wb;
  const u4_t* codes;
  const u4_t* meta;
  const _Float16* scales;
  const long long* idx;
  _Float16* y;
  float* partials;
  unsigned* status;
  const int* perm;   // token order (rows of x / y / idx) or nullptr: rows tok0, tok0 + 1, ...
  int tok0;          // first position of this launch in that order; T counts from there
  int nchunk;        // chunks of 32 tokens in this launch (1..4)
  long long codes_slot_u4, meta_slot_u4, scales_slot;
  int T, K, N, S, G, gs;
  int accumulate, ldy, nsplit, cb;
  int NP, NKB, NPG;
  int base_tiled;    // wb holds the base weight in tiles (dz_layout.h) instead of row-major [N, K]
};

// Up to DZ_MAX_BATCH layer calls in one launch; np_end[j] = n-pairs of calls 0..j (entries beyond
// the last call repeat the total).
constexpr int DZ_MAX_BATCH = DZ_MAX_BATCH_CALLS;
struct MdlBatch {
  MdlParams p[DZ_MAX_BATCH];
  int np_end[DZ_MAX_BATCH];
};

constexpr int XS = DZ_KBLOCK + 8;  // LDS row stride of the staged activations, in halves

// Packed words of one delta for one (n-pair, k-block): 16 bytes of positions and NCODE x 16 bytes of
// codes per lane.  NLOADS is the number of requests load_frag makes; the kernels' hand-written
// wait counts are built from it, so the two cannot drift apart.
template <int BITS>
struct Frag {
  static constexpr int NCODE = BITS == 2 ? 1 : 2;
  static constexpr int NLOADS = 1 + NCODE;
  u4_t meta;
  u4_t code[NCODE];
};

template <int BITS>
__device__ __forceinline__ Frag<BITS> load_frag(const MdlParams& P, int d, int np, int kb,
                                                int lane) {
  // wavefront-uniform tile base + 16 bytes per lane
  Frag<BITS> f;
  const size_t tile = (size_t)np * P.NKB + kb;
  const unsigned lo = (unsigned)lane * 16u;
  const char* mb = (const char*)(P.meta + (size_t)d * P.meta_slot_u4 + tile * 64);
  f.meta = __builtin_nontemporal_load((const u4_t*)(mb + lo));
  // one request per 1 KiB of codes: exactly Frag<BITS>::NCODE of them
  const char* cb = (const char*)(P.codes + (size_t)d * P.codes_slot_u4 + tile * (64 * Frag<BITS>::NCODE));
#pragma unroll
  for (int c = 0; c < Frag<BITS>::NCODE; ++c) f.code[c] = __builtin_nontemporal_load((const u4_t*)(cb + lo + 1024 * c));
  return f;
}

// Raises a kernel's dynamic-LDS limit once per device (the attribute belongs to the device's copy
// of the kernel).  `done` holds one bit per device; two threads that meet here at the same time
// both set the attribute, which is harmless.
inline bool dz_lds_limit_once(std::atomic<unsigned long long>& done, const void* kernel, int bytes) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev > 63) return false;
  const unsigned long long bit = 1ull << dev;
  if (done.load(std::memory_order_acquire) & bit) return true;
  if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess) return false;
  done.fetch_or(bit, std::memory_order_release);
  return true;
}

// Compute units of the current device (looked up once per device).
inline int dz_cu_count() {
  static std::atomic<int> cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev > 63) return 256;
  int v = cached[dev].load(std::memory_order_relaxed);
  if (v == 0) {
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0) v = 256;
    cached[dev].store(v, std::memory_order_relaxed);
  }
  return v;
}

// Launch of the T <= 32 kernel (dz_mdl32.hip).
int dz_launch_mdl32(const MdlParams& P, int bits, int pre, hipStream_t st, int ksplit_override);
int dz_launch_mdl32_batch(const MdlParams* P, int nprob, int bits, int pre, hipStream_t st, int ksplit_override);
void dz_mdl32_geometry(const MdlParams* P, int nprob, int ksplit_override, int* nsplit, int* cb, int* grid);
