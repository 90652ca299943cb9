/*
 * dz_amd.h -- C ABI of the MI355X (gfx950) multi-delta linear layer.
 *
 *   y[t, :] = x[t, :] @ W_base^T  +  (ids[t] >= 0 ?  x[t, :] @ dequant(delta[ids[t]])^T : 0)
 *
 * Every delta is 2:4 sparse along the input dimension, quantised symmetrically to 2 or 4 bits
 * with fp16 scales (per output channel, or per (channel, K-group)).  All pointers are raw
 * device pointers unless a parameter is documented as host memory; the caller owns all
 * memory.  Functions return 0 on success or a negative DZ_E* code; dz_strerror() names it.
 * `stream` is a hipStream_t passed as void* (NULL = the default stream).  Launches are
 * asynchronous on that stream.  No function allocates device memory.
 *
 * Reference interfaces these entry points stand in for (paths relative to the
 * eth-easl/deltazip tree):
 *   serving/vllm/delta/deltazip_marlin.py:10-19    apply_delta -> sbmm_4bit_2_4_native
 *   serving/vllm/delta/deltazip.py:14-77           add_delta / add_delta_slice -> ibmm_sparse_marlin
 *   serving/vllm/delta/quant_linears/quant_linear_naive.py:35-96   QuantLinear.forward/from_tensors
 *   deltazip/nn_modules/qlinear_cuda.py:246-329    QuantLinear.unpack (dequantisation)
 *   deltazip/utils/converter.py:13-101             GPTQ layout -> kernel layout conversion
 *   serving/vllm/delta/models.py:69-145            convert_mapping (delta id -> slot index tensors)
 *   serving/vllm/delta/deltazip_marlin.py:21-86    per-delta embedding / output-projection tables
 *   deltazip/core/quant.py, core/sparsegpt.py:55-66,123-135   quantiser and 2:4 mask of the compressor
 */
#ifndef DZ_AMD_H
#define DZ_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DZ_OK            0
#define DZ_EINVAL       -1   /* bad argument (null pointer, negative size)                  */
#define DZ_ESHAPE       -2   /* shape not supported: K % 256, N % 32, ldy % 4, T range      */
#define DZ_EBITS        -3   /* bits not in {2, 4}                                         */
#define DZ_EGROUP       -4   /* group_size not -1/K or a multiple of 64 dividing K          */
#define DZ_ENOT24       -5   /* repack: a group of 4 holds more than 2 non-zero-point codes */
#define DZ_EZERO        -6   /* repack: zero-point differs from 2^(bits-1)                  */
#define DZ_EGIDX        -7   /* repack: g_idx is not k / group_size                         */
#define DZ_EWORKSPACE   -8   /* workspace missing or too small                             */
#define DZ_ELAUNCH      -9   /* the HIP runtime refused the launch                         */
#define DZ_EALIGN      -10   /* pointer not aligned as required                            */
#define DZ_ESTATICMAX  -11   /* dz_multi_delta_linear_static: N above DZ_STATIC_MAX_N       */

#define DZ_MAX_TOKENS_FUSED 128   /* largest T the fused decode kernel takes in one launch   */
#define DZ_MAX_BATCH_CALLS 4      /* layer calls dz_multi_delta_linear_batch takes at once    */
#define DZ_STATIC_MAX_N 16384      /* largest N dz_multi_delta_linear_static takes             */
#define DZ_MAX_SLOTS_SEGMENT 768   /* largest S dz_segment takes (its tables live in LDS)      */
#define DZ_MAX_SLOTS_MAP 4096      /* largest S dz_map_ids takes (the slot table lives in LDS) */

/* Library version (major*10000 + minor*100 + patch). */
int dz_version(void);

/* Static, human readable text for a return code. */
const char* dz_strerror(int code);

/* Byte sizes of one delta in the native layout (per slot strides of the stacked tensors).
 * Stands in for the shape arithmetic of BaseLayerWithDelta.create_delta_weights
 * (serving/vllm/delta/layers_marlin.py:311-333). */
int dz_native_sizes(int K, int N, int bits, int group_size,
                    size_t* codes_bytes, size_t* meta_bytes, size_t* scales_bytes);

/* HOST function, host pointers.  Converts one delta from the reference's GPTQ-style packing
 * (qweight [K*bits/32, N] int32, qzeros [G, N*bits/32] int32 holding zero-1, scales [G, N] fp16,
 * g_idx [K] int32; deltazip/nn_modules/qlinear_cuda.py:144-244) into the native layout
 * (codes, meta, scales) consumed by the kernels.  Takes the role of
 * deltazip/utils/converter.py:13-101 (the conversion the reference delegates to triteia). */
int dz_repack_2of4(const int32_t* qweight, const int32_t* qzeros, const uint16_t* scales,
                   const int32_t* g_idx, int K, int N, int bits, int group_size,
                   void* out_codes, void* out_meta, void* out_scales);

/* HOST function, host pointers.  The inverse of dz_repack_2of4: one delta in the native layout ->
 * the reference's GPTQ-style tensors as QuantLinear.pack writes them
 * (deltazip/nn_modules/qlinear_cuda.py:144-244): qweight [K*bits/32, N] int32 (pruned columns carry
 * the zero-point code, which dequantises to 0), qzeros [G, N*bits/32] int32 holding zero-1 =
 * 2^(bits-1)-1 in every field, scales [G, N] fp16, g_idx [K] int32 = k / group_size (may be NULL).
 * With it a delta compressed here can be saved in the format the reference's save_compressed
 * writes and its loaders read (deltazip/modeling/_base.py:597-648). */
int dz_unrepack_2of4(const void* codes, const void* meta, const uint16_t* scales, int K, int N,
                     int bits, int group_size, int32_t* out_qweight, int32_t* out_qzeros,
                     uint16_t* out_scales, int32_t* out_g_idx);

/* Dequantise one native delta to fp16, out[n * K + k] (row-major [N, K]).  Bit-exact with
 * QuantLinear.unpack (deltazip/nn_modules/qlinear_cuda.py:246-329): half(float(scale)*(q-zero)). */
int dz_dequant(const void* codes, const void* meta, const void* scales,
               int K, int N, int bits, int group_size, uint16_t* out, void* stream);

/* out[n*K+k] = w_base[n*K+k] + dequant(delta)[n, k], the addition done in fp32 and rounded once
 * to fp16 (the reference's merge, deltazip/utils/generate.py:9-20, at fp16 storage). */
int dz_merge(const uint16_t* w_base, const void* codes, const void* meta, const void* scales,
             int K, int N, int bits, int group_size, uint16_t* out, void* stream);

/* Group tokens by delta id: perm[T] lists token indices sorted by id (stable; id -1 first),
 * seg_off[S + 2] are the offsets of the segments for id = -1, 0, ..., S-1 in perm.
 * Ids outside [-1, S) are treated as -1; S <= DZ_MAX_SLOTS_SEGMENT.  (The reference's scheduler sorts the batch by delta
 * id, serving/vllm/core/scheduler.py:101-104; this makes the op independent of that.) */
int dz_segment(const int64_t* indices, int T, int S, int32_t* perm, int32_t* seg_off, void* stream);

/* Delta id -> slot index for a batch, on the device: the index tensors the reference's manager
 * builds in a Python loop over tokens (convert_mapping, serving/vllm/delta/models.py:69-145).
 * token_ids [T] and prompt_ids [P] hold delta ids (<= 0: base model); slot_ids [S] holds the id
 * resident in each slot (<= 0: free).  Writes
 *   base_indices[t]            = slot of token_ids[t], -1 for the base model
 *   sampler_indices[p]         = slot of prompt_ids[p], -1 for the base model
 *   sampler_indices_padded[p]  = p + (slot == -1 ? max_deltas - 1 : slot) * P
 *   embeddings_indices[0][t]   = e * extra_vocab_size, [1][t] = e * (vocab_size + extra_vocab_size),
 *                                e = slot for a delta and 0 for the base model, a result of -1
 *                                replaced by max_deltas - 1 (row stride ld_emb elements)
 * as the reference does.  sampler_indices_padded, embeddings_indices and n_missing may be NULL; P
 * may be 0.  An id > 0 that is in no slot maps to -1 and, when n_missing is given, adds one to
 * *n_missing (the caller zeroes it), where the reference's list.index raises.  S <= DZ_MAX_SLOTS_MAP. */
int dz_map_ids(const int64_t* token_ids, int T, const int64_t* prompt_ids, int P,
               const int64_t* slot_ids, int S, int max_deltas, int vocab_size, int extra_vocab_size,
               int64_t* base_indices, int64_t* sampler_indices, int64_t* sampler_indices_padded,
               int64_t* embeddings_indices, int ld_emb, int32_t* n_missing, void* stream);

/* Per-token embedding lookup with per-delta tables: out[t, :] = table(t)[tokens[t], :], where
 * table(t) is weight_stack + indices[t] * stack_stride (elements; a delta's own [V, H] fp16
 * table) for 0 <= indices[t] < S and base_weight [V, H] otherwise.  The fine-tuned table replaces
 * the base one, it is not added: apply_delta_embed, serving/vllm/delta/deltazip_marlin.py:56-86,
 * as called by VocabParallelEmbeddingWithDelta.forward, layers_marlin.py:143-160.  A token id
 * outside [0, V) gives a row of zeros.  H % 8 == 0, ldo % 8 == 0 (row stride of out, elements). */
int dz_embedding_select(const int64_t* tokens, const int64_t* indices, const uint16_t* base_weight,
                        const uint16_t* weight_stack, long long stack_stride, int S, uint16_t* out, int T,
                        int V, int H, int ldo, void* stream);

/* Compress one delta on the device: delta [N, K] fp32 row-major -> native codes / positions /
 * fp16 scales.  Symmetric scales per output row (group_size -1) or per (row, group) from the
 * un-pruned values (deltazip/core/quant.py:48-130 sym branch; sparsegpt.py:64-66), 2:4 pruning
 * by magnitude (sparsegpt.py:123-135 with an identity Hessian; ties keep the lower column), codes
 * q = clamp(rint(x / scale) + 2^(bits-1), 0, 2^bits - 1) with the fp32 scale (quant.py:9-18),
 * stored scale = fp16(scale) (qlinear_cuda.py:153-156).  The result equals, byte for byte, what
 * dz_repack_2of4 makes of the same delta compressed and packed the reference's way.  The
 * Hessian-weighted sweep of SparseGPT is dz_obs_sweep below.
 * scale_workspace: G * N floats of device memory (G = K / group_size, 1 for -1). */
int dz_compress_2of4(const float* delta, int K, int N, int bits, int group_size, void* out_codes,
                     void* out_meta, uint16_t* out_scales, float* scale_workspace, void* stream);

/* The two halves of dz_compress_2of4 on their own.  dz_quant_scales: the symmetric scales of
 * Quantizer.find_params (deltazip/core/quant.py:48-130, perchannel, sym) as fp32 [G, N] and fp16
 * [G, N].  dz_pack_2of4: codes and positions in the native layout from values that are already
 * 2:4 sparse and on the grid of the given fp32 scales (what dz_obs_sweep leaves in W); other
 * values are pruned by magnitude and rounded as in dz_compress_2of4. */
int dz_quant_scales(const float* delta, int K, int N, int bits, int group_size, float* scale32,
                    uint16_t* scale16, void* stream);
int dz_pack_2of4(const float* w, const float* scale32, int K, int N, int bits, int group_size, void* out_codes,
                 void* out_meta, void* stream);

/* dz_quant_scales with the search over the clipping range that Quantizer.find_params runs for
 * mse=True (deltazip/core/quant.py:85-101; sym, perchannel): for i = 0 .. int(maxshrink * grid) - 1
 * the symmetric range is shrunk by p = 1 - i / grid and the candidate whose rounding error
 * sum |q(x) - x|^norm over the row (or scale group) is smallest gives the scale; the first
 * candidate wins a tie.  The reference's defaults are norm = 2.4, grid = 100, maxshrink = 0.8. */
int dz_quant_scales_mse(const float* delta, int K, int N, int bits, int group_size, float norm, int grid,
                        float maxshrink, float* scale32, uint16_t* scale16, void* stream);

/* Layer Hessian of SparseGPT.add_batch (deltazip/core/sparsegpt.py:27-40):
 * H <- H * scale_h + (scale_x * x)^T (scale_x * x) for x [T, K] (fp16 if x_is_fp16, else fp32),
 * H [K, K] fp32; the caller passes scale_h = n / (n + b) and scale_x = sqrt(2 / (n + b)) for b new
 * samples after n.  The sum over tokens runs in ascending order, one rounding per operation.
 * K % 64 == 0. */
int dz_hessian_add(float* H, const void* x, int x_is_fp16, int T, int K, float scale_h, float scale_x,
                   void* stream);

/* The sweep of SparseGPT.fasterprune (deltazip/core/sparsegpt.py:92-146) over W [N, K] fp32 in
 * place, in blocks of 128 columns: in every aligned group of prunem columns the prunen columns
 * with the smallest w^2 / diag(hinv)^2 are set to 0 (ties keep the lower column; prunen = 0: no
 * pruning), every column is rounded to the grid scale[row] * (q - 2^(bits-1)), q in [0, 2^bits)
 * (scale = NULL: not rounded), and its error, divided by the diagonal, is subtracted from the
 * columns to its right along the row of hinv_upper -- the upper Cholesky factor of the inverse of
 * the dampened Hessian (sparsegpt.py:80-84), [K, K] fp32 row-major.  loss [N] += the row's
 * sum of (w - q)^2 / diag^2 / 2 per block.  err_workspace: N * 128 floats.  Sums run in
 * ascending column order with one rounding per operation, so the result equals a plain fp32
 * restatement with that order bit for bit.  K % 128 == 0, prunem <= 8 and a divisor of 64. */
int dz_obs_sweep(float* W, const float* hinv_upper, const float* scale, int N, int K, int bits, int prunen,
                 int prunem, float* err_workspace, float* loss, void* stream);

/* Bytes of device workspace dz_multi_delta_linear needs for these sizes.  The workspace must be
 * zero-filled once before first use; calls leave it zero-filled for the next call, whatever their
 * sizes (it carries the partial sums of a K dimension split over workgroups; an empty slot is all
 * zero bits).  Calls that share a workspace must be ordered on one stream.  Word 0 is a status
 * word: bit 0 = a delta id outside [-1, S) was met (treated as -1), bit 1 = a partial sum did not
 * arrive within the kernel's bounded wait (the output of that call is then invalid). */
size_t dz_workspace_bytes(int T, int K, int N);

/* The layer.  x [T, K] fp16 row-major; w_base [N, K] fp16 row-major or NULL (delta only);
 * codes/meta/scales: S slots of one native delta each, slot strides as dz_native_sizes reports;
 * indices [T] int64, -1 = base only, read on the device at execution time; y [T, ldy] fp16,
 * columns 0..N-1 written.  accumulate = 0: y = result; 1: y += result (fp32 add, one rounding).
 * Stands in for sbmm_4bit_2_4_native / ibmm_sparse_marlin at the call sites listed above.
 * S = 0 (no slots; the delta pointers may then be NULL, w_base must not be): the dense product
 * y (+)= x @ w_base^T alone, whatever the indices say.
 * Requires 1 <= T <= DZ_MAX_TOKENS_FUSED; above 32 tokens the tokens are grouped by id on the
 * device and handled 32 at a time, in one launch, the groups dealt so that every 32 meet about
 * the same number of deltas.  Larger batches are served by the host wrapper from dz_segment +
 * dz_build_tiles + dz_multi_delta_gemm. */
int dz_multi_delta_linear(const uint16_t* x, const uint16_t* w_base,
                          const void* codes_stacked, const void* meta_stacked,
                          const void* scales_stacked, const int64_t* indices, uint16_t* y,
                          int T, int K, int N, int S, int bits, int group_size,
                          int accumulate, int ldy, void* workspace, size_t workspace_bytes,
                          void* stream);

/* dz_multi_delta_linear for callers that cannot allocate device memory or hand over a workspace
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has
 * no counterpart in the reference.  Same arguments, results and error codes as
 * dz_multi_delta_linear without the workspace: the partial sums, the token order and the status
 * word live in a fixed array of device memory inside the library's code object (32 MiB + 5 KiB
 * per GPU the library runs on, held until the process ends), which serves N <= DZ_STATIC_MAX_N;
 * a larger N returns DZ_ESTATICMAX.  The call allocates nothing and frees nothing; its first
 * call on a device looks the array's address up (hipGetSymbolAddress), which is the only set-up.
 * All calls on one GPU share the array: calls that overlap in time on one GPU (two streams, two
 * host threads) race; order them on one stream.  The array is all zero bits at load and every
 * call leaves the partial-sum slots zero again, as with a caller's workspace.  The status word
 * inside the array cannot be read back through this interface: a caller that wants to see a bad
 * token id or a failed exchange of partial sums reported (and the slots emptied after one) uses
 * dz_multi_delta_linear with a workspace of its own. */
int dz_multi_delta_linear_static(const uint16_t* x, const uint16_t* w_base,
                                 const void* codes_stacked, const void* meta_stacked,
                                 const void* scales_stacked, const int64_t* indices, uint16_t* y,
                                 int T, int K, int N, int S, int bits, int group_size,
                                 int accumulate, int ldy, void* stream);

/* Up to DZ_MAX_BATCH_CALLS layer calls in one launch: calls that share the tokens (T, indices),
 * K, S, bits and group_size -- the projections the reference holds as one fused layer (q/k/v:
 * MergedQKVParallelLinearWithDelta, gate/up: MergedColumnParallelLinearWithDelta,
 * serving/vllm/delta/layers_marlin.py:281-487) when their weights are separate tensors.  Call j
 * computes y[j][T, ldy[j]] (+)= x[j] @ w_base[j]^T + x[j] @ dequant(delta_j[indices])^T with
 * N[j] output features, as dz_multi_delta_linear would (the launch splits K by the output rows of
 * all its calls together, so the fp32 partial sums over K may be added in another order than in a
 * separate call: equal up to that rounding, and identical from run to run); in one launch the
 * reduction and stores of one call overlap the loads of the next.  All calls have a base weight or none has.
 * order: NULL, or what dz_token_order wrote for these indices (then the grouping of the tokens is
 * not repeated: the reference, too, converts the mapping once per batch and every layer reuses
 * it, serving/vllm/delta/models.py:421-435).  workspace: dz_workspace_bytes(T, K, N[0] + ... +
 * N[ncalls-1]) bytes. */
int dz_multi_delta_linear_batch(int ncalls, const uint16_t* const* x, const uint16_t* const* w_base,
                                const void* const* codes_stacked, const void* const* meta_stacked,
                                const void* const* scales_stacked, const int64_t* indices,
                                uint16_t* const* y, const int* N, const int* ldy, int T, int K, int S,
                                int bits, int group_size, int accumulate, const int32_t* order,
                                void* workspace, size_t workspace_bytes, void* stream);

/* The base weight in tiles.  The fused kernel reads a base weight 8 rows x 128 bytes per request
 * from the row-major [N, K] form; from tiles -- 32 rows x 256 columns stored contiguously, in the
 * order the matrix instruction takes its operand -- every request is 1 KiB of consecutive bytes,
 * which the memory system streams faster.  A layer that keeps its base weight for the life of
 * the model converts it once (as the deltas are repacked once): out has N*K elements like w and
 * must not overlap it (the conversion is a permutation).  K % 256 == 0, N % 32 == 0.  No counterpart in the reference, whose base GEMM reads the
 * parameter as it is (serving/vllm/delta/deltazip_marlin.py:10-19). */
int dz_tile_base(const uint16_t* w, int K, int N, uint16_t* out, void* stream);

/* dz_multi_delta_linear_batch with every w_base_tiled[j] in the tiled form dz_tile_base writes
 * (ncalls = 1: the single layer call).  The same products summed in the same order as with the
 * row-major form: the results are the same, bit for bit. */
int dz_multi_delta_linear_batch_tiled(int ncalls, const uint16_t* const* x,
                                      const uint16_t* const* w_base_tiled,
                                      const void* const* codes_stacked, const void* const* meta_stacked,
                                      const void* const* scales_stacked, const int64_t* indices,
                                      uint16_t* const* y, const int* N, const int* ldy, int T, int K,
                                      int S, int bits, int group_size, int accumulate,
                                      const int32_t* order, void* workspace, size_t workspace_bytes,
                                      void* stream);

/* The order in which the fused kernel takes the tokens of a batch of up to DZ_MAX_TOKENS_FUSED
 * tokens, 32 per chunk: order[T], a permutation of 0..T-1 in which the tokens of one delta stay
 * together and every chunk of 32 meets about the same number of distinct deltas.  Depends on the
 * indices only, so one call serves every layer of a step (pass it as `order` above).  No
 * counterpart in the reference beyond the scheduler's sort by delta id
 * (serving/vllm/core/scheduler.py:101-104). */
int dz_token_order(const int64_t* indices, int T, int S, int32_t* order, void* stream);

/* Dense fp16 GEMM on the matrix cores: y[T, ldy] (+)= x[T, K] @ w[N, K]^T, fp32 accumulation.
 * Stands in for the base product of LinearMethodBase.apply_weights
 * (serving/vllm/model_executor/layers/linear.py:85-96) at prefill sizes. */
int dz_gemm_f16(const uint16_t* x, const uint16_t* w, uint16_t* y, int T, int K, int N,
                int accumulate, int ldy, void* stream);

/* As dz_gemm_f16 with two weights of the same shape: y (+)= x @ w_a^T + x @ w_b^T, both products in
 * the same fp32 accumulators.  Used at prefill sizes with w_a = base weight and w_b = one
 * dequantised delta, so that base and delta are never added in fp16 (the reference's CPU path adds
 * them in fp32: deltazip/utils/generate.py:9-20 as restated by the oracle). */
int dz_gemm_f16_pair(const uint16_t* x, const uint16_t* w_a, const uint16_t* w_b, uint16_t* y,
                     int T, int K, int N, int accumulate, int ldy, void* stream);

/* One block of consecutive rows (tokens) of a grouped GEMM: rows [row_lo, row_hi), at most 256 of
 * them, all using second weight `group` (-1: none). */
typedef struct dz_gemm_tile {
  int row_lo, row_hi, group, reserved;
} dz_gemm_tile;

/* Grouped form of dz_gemm_f16_pair for a batch sorted by delta id: y[t] (+)= x[t] @ w^T +
 * x[t] @ w2_stack[group(t)]^T, where `tiles` (device memory, ntiles entries) cuts the rows into
 * blocks that do not straddle groups and w2_stack + group * w2_stride (elements) is the [N, K]
 * second weight of a group.  w may be NULL (second product only).  Rows not covered by a tile
 * are not written.  This is the batched
 * form of the per-delta loop of the reference's dense fallbacks (for id in unique(indices):
 * F.linear(x[indices == id], W[id]); serving/vllm/delta/deltazip_marlin.py:44-53). */
int dz_gemm_f16_grouped(const uint16_t* x, const uint16_t* w, const uint16_t* w2_stack,
                        long long w2_stride, const dz_gemm_tile* tiles, int ntiles, uint16_t* y,
                        int T, int K, int N, int accumulate, int ldy, void* stream);

/* Per-row choice of one full weight: for every row block b of `tiles` and every position p in
 * [row_lo, row_hi), with t = perm ? perm[p] : p,
 *   y[t, 0..N) (+)= x[t] @ (group(b) >= 0 ? w_stack[group(b)] : w_base)^T
 * -- the output projection of the reference's LogitsProcessorWithDelta, whose
 * apply_delta_uncompressed loops over torch.unique(indices) on the host and multiplies each id's
 * rows by that delta's own table, the rows without a delta by the base table
 * (serving/vllm/delta/deltazip_marlin.py:21-53).  With perm = what dz_segment wrote and tiles =
 * what dz_build_tiles wrote, the whole call is three launches and nothing is gathered, scattered
 * or read back.  Rows outside every block are not written. */
int dz_gemm_f16_select(const uint16_t* x, const uint16_t* w_base, const uint16_t* w_stack,
                       long long w_stride, const dz_gemm_tile* tiles, int ntiles, const int32_t* perm,
                       uint16_t* y, int T, int K, int N, int accumulate, int ldy, void* stream);

/* Row blocks for dz_multi_delta_gemm from the segment offsets dz_segment wrote (device memory,
 * S + 2 entries): every segment is cut into blocks of at most 256 rows, group = slot (-1 for the
 * tokens without a delta); entries of `tiles` (device memory, max_tiles of them) beyond the blocks
 * in use are marked empty.  max_tiles >= (T + 255) / 256 + min(S + 1, T) always suffices, so the
 * host never needs to read the offsets back.  S <= DZ_MAX_SLOTS_SEGMENT. */
int dz_build_tiles(const int32_t* seg_off, int S, dz_gemm_tile* tiles, int max_tiles, void* stream);

/* The layer at prefill sizes, deltas in packed form: for every row block b of `tiles` and every
 * position p in [row_lo, row_hi), with t = perm ? perm[p] : p,
 *   y[t, 0..N) (+)= x[t] @ w_base^T + x[t] @ dequant(delta[group(b)])^T
 * (w_base may be NULL; group -1 or >= S: base only).  Base product on the dense matrix-core
 * instructions, delta product on the 2:4-sparse ones straight from the native layout; both in the
 * same fp32 accumulators, every delta value rounded to fp16 exactly as dz_dequant rounds it.
 * Stands in, like dz_multi_delta_linear, for sbmm_4bit_2_4_native at
 * serving/vllm/delta/deltazip_marlin.py:18, and for the exllama path's "reconstruct, then dense
 * GEMM" above 50 rows (q_gemm.cu:118-137) without the reconstruction.  Rows outside every block
 * are not written.  K % 256 == 0, N % 32 == 0, T * K and N * K below 2^31 elements. */
int dz_multi_delta_gemm(const uint16_t* x, const uint16_t* w_base, const void* codes_stacked,
                        const void* meta_stacked, const void* scales_stacked, int S, int bits,
                        int group_size, const dz_gemm_tile* tiles, int ntiles, const int32_t* perm,
                        uint16_t* y, int T, int K, int N, int accumulate, int ldy, void* stream);

/* dz_multi_delta_gemm with the base weight in the tiles dz_tile_base writes (the form the fused
 * kernel reads up to 128 tokens): a layer that keeps only the tiled copy serves every batch size
 * from it.  The same products are summed in the same order as from the row-major weight, so the
 * results are equal bit for bit.  w_base_tiled must not be NULL (delta only: dz_multi_delta_gemm
 * with w_base NULL).  Same reference call sites as dz_multi_delta_gemm. */
int dz_multi_delta_gemm_tiled(const uint16_t* x, const uint16_t* w_base_tiled, const void* codes_stacked,
                              const void* meta_stacked, const void* scales_stacked, int S, int bits,
                              int group_size, const dz_gemm_tile* tiles, int ntiles, const int32_t* perm,
                              uint16_t* y, int T, int K, int N, int accumulate, int ldy, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* DZ_AMD_H */
