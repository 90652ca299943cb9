/* Tuning and test hooks of libdz_amd.so.  Not part of the layer's interface (include/dz_amd.h): a
 * serving engine has no reason to call anything declared here.  No counterpart in the reference. */
#ifndef DZ_AMD_TUNING_H
#define DZ_AMD_TUNING_H
#ifdef __cplusplus
extern "C" {
#endif

/* Overrides the number of K-slices of the fused kernel for the later calls of the calling host
 * thread only (0 = automatic, the default); other threads' launches are untouched.  The results
 * do not depend on it beyond the order of the fp32 additions.  Used by the tests that drive every
 * split through the same shapes and by timing sweeps. */
void dz_set_ksplit(int nsplit);

#ifdef __cplusplus
}
#endif
#endif /* DZ_AMD_TUNING_H */
