/* Tuning and test hooks of libdz_amd.so.  Not part of the layer's interface (include/dz_amd.h): a
 * serving engine has no reason to call anything declared here.  No counterpart in the reference. */
#ifndef DZ_AMD_TUNING_H
#define DZ_AMD_TUNING_H
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

/* Overrides the number of K-slices of the fused kernel for the later calls of the calling host
 * thread only (0 = automatic, the default); other threads' launches are untouched.  The results
 * do not depend on it beyond the order of the fp32 additions.  Used by the tests that drive every
 * split through the same shapes and by timing sweeps. */
void dz_set_ksplit(int nsplit);

/* Read-only yardstick for the fused kernel (up to 32 tokens): launches the fused kernel's grid for
 * these calls (same workgroup -> (n-pair, K-slice) mapping, same K split) and issues, per
 * wavefront and k-block, the same 16-byte streaming requests for the tiled base weight and for
 * the packed words of the deltas in slots 0 .. D-1 (D <= 8) -- with_x != 0: also the 32 x 256
 * activation slice into LDS -- and nothing else: no ids, no arithmetic on the matrix cores, no
 * reduction, no exchange of partial sums, no output.  Its duration is what the memory system
 * allows for that request pattern at that size.  sink: 4 bytes of device memory (never written
 * in practice; it keeps the loads alive).  Arrays as in dz_multi_delta_linear_batch_tiled. */
int dz_probe_read(int ncalls, const uint16_t* const* x, const uint16_t* const* w_base_tiled,
                  const void* const* codes_stacked, const void* const* meta_stacked, const int* N,
                  int T, int K, int bits, int D, int with_x, void* sink, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* DZ_AMD_TUNING_H */
