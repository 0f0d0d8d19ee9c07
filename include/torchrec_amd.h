/*
 * torchrec_amd — C ABI of the MI355X (gfx950) quantized embedding inference
 * kernels.  Plain C: raw device pointers, sizes and a hipStream_t (passed as
 * void*).  The caller owns every buffer; calls are asynchronous on the given
 * stream and re-entrant; nothing here synchronizes unless stated.
 *
 * Every entry point returns TRA_OK (0) or a negative TRA_ERR_* code and never
 * throws.  tra_last_error() returns a thread-local message for the last
 * failure.
 *
 * What each entry point replaces in the reference (pytorch/torchrec) is cited
 * next to it; the operators themselves live in the un-vendored fbgemm_gpu
 * dependency, so the citations are the reference's call sites.
 */
#ifndef TORCHREC_AMD_H_
#define TORCHREC_AMD_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TRA_OK 0
#define TRA_ERR_INVALID_ARGUMENT (-1) /* bad dtype / shape / alignment / null */
#define TRA_ERR_UNSUPPORTED (-2)      /* valid but not implemented            */
#define TRA_ERR_HIP (-3)              /* a HIP runtime call failed            */
#define TRA_ERR_NO_DEVICE (-4)        /* no gfx950 device / wrong arch        */
#define TRA_ERR_TOO_LARGE (-5)        /* exceeds a documented limit           */

/* Weight / output element types: values of fbgemm_gpu SparseType.as_int(). */
#define TRA_FP32 0
#define TRA_FP16 1
#define TRA_INT8 2
#define TRA_INT4 3
#define TRA_INT2 4

/* Pooling modes: values of fbgemm_gpu PoolingMode. */
#define TRA_POOL_SUM 0
#define TRA_POOL_MEAN 1
#define TRA_POOL_NONE 2

/* One table of a table-batched embedding (TBE) group.  Rows are packed in one
 * uint8 buffer; table t starts at byte `offset`; row r starts at
 * offset + r * row_bytes.  INT8/INT4/INT2 rows are
 *   [fp16 scale][fp16 bias][payload dim*bits/8 bytes][pad]
 * FP16/FP32 rows are [payload][pad].  row_bytes is the distance between rows:
 * at least header + payload, and as much padding behind a row as the caller
 * likes (a 68-byte row stored every 128 bytes never straddles a 128-byte HBM
 * line).  row_bytes and offset must be multiples of 4.  (Reference: embedding_specs + row_alignment handed to
 * IntNBitTableBatchedEmbeddingBagsCodegen, torchrec/quant/embedding_modules.py:
 * 393-435.) */
typedef struct tra_table_spec {
  int64_t offset;
  int64_t rows;
  int32_t dim;
  int32_t dtype;
  int32_t row_bytes;
  int32_t reserved;
} tra_table_spec;

typedef struct tra_tbe* tra_tbe_t;

/* Library / device ------------------------------------------------------- */
int tra_version(void);
const char* tra_last_error(void);
/* Name of the current device's architecture ("gfx950..."); TRA_ERR_NO_DEVICE
 * if there is no usable GPU. */
int tra_device_arch(char* buf, int buf_len);

/* Tuning override for experiments and tests: name is one of "balanced" (1:
 * window kernel, 0: static kernel), "window" (bags per block), "unroll", "lds",
 * "xcd" (0: no remap of blocks to dies), "cost_floor", "fused_scan" (from-lengths
 * prologue inside the lookup kernel: 1 always, 0 never), "cb" (lane chunk bytes,
 * acts on plans created afterwards), "fork" (0: the launches of a call of five
 * or more launch classes all stay on the caller's stream instead of alternating
 * with the plan's second stream; k > 1, for plans created afterwards: from k
 * classes on instead of five); value < 0 restores the default.  The
 * same knobs are read from the environment (TRA_BALANCED, TRA_WINDOW, ...)
 * once, when the library is loaded; no lookup call reads the environment.
 * Process-wide; not meant to be changed while lookups are being issued.
 * No counterpart in the reference (fbgemm_gpu chooses its kernels internally,
 * behind the call at torchrec/quant/embedding_modules.py:547-557). */
int tra_set_tuning(const char* name, int32_t value);

/* TBE group plan ---------------------------------------------------------- */
/* Builds the immutable launch plan of one TBE group on the current device:
 * per-feature descriptors (feature f reads table feature_table_map[f] and
 * writes output columns D_offsets[f] .. D_offsets[f+1]) grouped by kernel
 * class.  feature_positions (may be NULL = identity) gives, for each feature,
 * the index of its bags in the offsets array passed to tra_tbe_forward: bag
 * (f, b) is offsets[feature_positions[f] * B + b].  This is how a caller looks
 * up from a KeyedJaggedTensor whose keys are ordered differently (or are a
 * superset) without permuting it first; the reference permutes
 * (torchrec/quant/embedding_modules.py:127-135, 535-537).  Allocates a few KB
 * of device memory, released by tra_tbe_destroy.  Replaces the constructor of
 * IntNBitTableBatchedEmbeddingBagsCodegen
 * (torchrec/quant/embedding_modules.py:427-435, 828-836). */
int tra_tbe_create(const tra_table_spec* tables, int32_t num_tables,
                   const int32_t* feature_table_map,
                   const int32_t* feature_positions, int32_t num_features,
                   tra_tbe_t* out);
int tra_tbe_destroy(tra_tbe_t tbe);

/* Pooled / sequence lookup.  Replaces
 * IntNBitTableBatchedEmbeddingBagsCodegen.forward(indices, offsets,
 * per_sample_weights) (torchrec/quant/embedding_modules.py:547-557 pooled,
 * :938-942 sequence).
 *   weights      device, the packed table buffer
 *   indices      device [L], int32 or int64 (idx_is_i64); -1 = pruned id, skipped
 *   offsets      device [K*B + 1] (K = number of input keys, F when
 *                feature_positions is identity), same integer type; bag (f,b)
 *                is offsets[p*B+b] .. offsets[p*B+b+1], p = feature_positions[f]
 *   per_sample_weights device [L] fp32 or NULL (ignored for TRA_POOL_NONE)
 *   out          device; pooled: [B, out_stride] elements, feature f at column
 *                D_offsets[f]; TRA_POOL_NONE: [L, dim] (all features share dim)
 *   out_dtype    TRA_FP32 or TRA_FP16
 *   num_indices  L, the number of elements of indices (required); it may
 *                exceed what the bags cover (a padded buffer): the excess is
 *                never read
 * Arithmetic per output column, ids in order: acc = fmaf(w*scale, q, acc +
 * w*bias) (fp16/fp32 rows: acc = fmaf(w, x, acc)); MEAN multiplies by 1.0f/len;
 * output rounded to nearest even.  Ids outside [0, rows) other than -1 are
 * counted (tra_tbe_error_count) and skipped, or pool row 0 where
 * tra_tbe_set_bounds_check_mode asked for that.  Every buffer sits at a multiple
 * of its element size (weights: 4 bytes), else TRA_ERR_INVALID_ARGUMENT.
 * Ordering: everything the call launches runs after what `stream` holds at the
 * call and before what is put on `stream` afterwards.  A plan of five or more
 * launch classes (weight type x lane chunk) runs every other launch on a second
 * stream of its own, forked from and joined to `stream` with events inside the
 * call; not while `stream` is being captured into a graph. */
int tra_tbe_forward(tra_tbe_t tbe, const void* weights, const void* indices,
                    const void* offsets, int32_t idx_is_i64,
                    const float* per_sample_weights, int32_t batch_size,
                    int64_t num_indices, int32_t pooling_mode,
                    int32_t out_dtype, void* out, int64_t out_stride,
                    void* stream);

/* The same lookup from the KJT's lengths instead of its offsets: what
 * QuantEmbeddingBagCollection.forward does when the KJT was built from
 * lengths, i.e. KeyedJaggedTensor.offsets() -> asynchronous_complete_cumsum
 * (torchrec/sparse/jagged_tensor.py:101-107, 79-80) followed by the TBE call
 * (torchrec/quant/embedding_modules.py:547-557), in one entry point.
 *   lengths      device [num_keys * batch_size], same integer type as indices
 *   num_keys     number of keys of the KJT (>= every feature position + 1)
 *   workspace    device scratch of tra_tbe_forward_lengths_workspace_bytes()
 *                bytes; contents unspecified afterwards
 * Large pooled calls derive each bag's start inside the lookup kernel (no
 * offsets array is produced); all others run tra_cumsum into the workspace
 * and then the ordinary lookup.  Results are those of tra_tbe_forward. */
int64_t tra_tbe_forward_lengths_workspace_bytes(int32_t num_keys, int32_t batch_size,
                                                int32_t idx_is_i64);
int tra_tbe_forward_lengths(tra_tbe_t tbe, const void* weights, const void* indices,
                            const void* lengths, int32_t idx_is_i64,
                            const float* per_sample_weights, int32_t batch_size,
                            int32_t num_keys, int64_t num_indices,
                            int32_t pooling_mode, int32_t out_dtype, void* out,
                            int64_t out_stride, void* workspace, void* stream);

/* tra_tbe_forward_lengths without a workspace argument and without any
 * allocation: the scratch (the offsets array and the scan's partial sums, the
 * same bytes tra_tbe_forward_lengths_workspace_bytes() asks for) lives in a
 * static device array of the library, tra_tbe_forward_lengths_static_max_bytes()
 * = 8 MiB per GPU, resolved when the first plan is created on that GPU.  No
 * counterpart in the reference; it is for callers that cannot allocate device
 * memory: code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc.  A call that needs more scratch returns TRA_ERR_TOO_LARGE.
 * Every call on a GPU shares that GPU's array: calls that overlap on one GPU
 * (several streams or host threads) race; nothing in it has to start at zero.
 * Results are those of tra_tbe_forward_lengths. */
int64_t tra_tbe_forward_lengths_static_max_bytes(void);
int tra_tbe_forward_lengths_static(tra_tbe_t tbe, const void* weights, const void* indices,
                                   const void* lengths, int32_t idx_is_i64,
                                   const float* per_sample_weights, int32_t batch_size,
                                   int32_t num_keys, int64_t num_indices,
                                   int32_t pooling_mode, int32_t out_dtype, void* out,
                                   int64_t out_stride, void* stream);

/* Pooled lookup with position weights: the id at position k of a bag of the
 * feature at key position p is weighted by
 *   position_weights[key_start[p] + min(k, key_len[p] - 1)],  or 1 if key_len[p] == 0,
 * inside the lookup kernel, in place of per_sample_weights.  Replaces the
 * three steps of the reference's feature-processed collection:
 * PositionWeightedModuleCollection.forward (fbgemm offsets_range + a gather per
 * key, torchrec/modules/feature_processor_.py:193-260), the weighted KJT it
 * builds (torchrec/modules/fp_embedding_modules.py:20-53) and the weighted TBE
 * call (torchrec/quant/embedding_modules.py:547-557).
 *   bags              device: offsets [num_keys*B + 1], or lengths [num_keys*B]
 *                     when bags_are_lengths (workspace as for
 *                     tra_tbe_forward_lengths, else NULL)
 *   position_weights  device fp32 [position_weights_len >= 1], all keys' vectors
 *   key_start/key_len HOST int32 [num_keys], checked against the table here
 * A launch class (one weight type and lane width) may hold at most 128
 * features (TRA_ERR_TOO_LARGE otherwise; the caller then materializes the
 * weights with tra_position_weights and calls tra_tbe_forward).  Other
 * arguments and the arithmetic as tra_tbe_forward; TRA_POOL_NONE is refused. */
int tra_tbe_forward_position_weighted(tra_tbe_t tbe, const void* weights, const void* indices,
                                      const void* bags, int32_t bags_are_lengths,
                                      int32_t idx_is_i64, const float* position_weights,
                                      int64_t position_weights_len, const int32_t* key_start,
                                      const int32_t* key_len, int32_t num_keys,
                                      int32_t batch_size, int64_t num_indices,
                                      int32_t pooling_mode, int32_t out_dtype, void* out,
                                      int64_t out_stride, void* workspace, void* stream);

/* Which kernels a tra_tbe_forward with these sizes launches, one entry per
 * launch in launch order, "; "-separated, e.g. "tbe_pooled_cu_kernel dtype=int4
 * lane_bytes=8 slices=26"; where the launches alternate between two streams
 * an entry also says which ("... on the plan's second stream").
 * lengths_num_keys > 0 asks about tra_tbe_forward_lengths with
 * that many keys instead (entries then end in " from_lengths" when the kernel
 * derives the offsets itself, else the scan kernels come first).  For
 * profiling: the names are the ones a kernel trace shows.
 * No counterpart in the reference: fbgemm_gpu picks its kernel inside the
 * TBE module's forward (called at torchrec/quant/embedding_modules.py:547-557)
 * and does not report it. */
int tra_tbe_launch_info(tra_tbe_t tbe, int32_t batch_size, int64_t num_indices,
                        int32_t pooling_mode, int32_t lengths_num_keys, char* buf,
                        int32_t buf_len);

/* What later forwards on this plan do with an id outside [0, rows) other than
 * -1, by fbgemm_gpu's BoundsCheckMode codes (the `bounds_check_mode` the
 * reference hands to the TBE constructor, default WARNING, at
 * torchrec/distributed/quant_embedding_kernel.py:281-283, 337-339):
 *   WARNING 1, IGNORE 2   the id pools row 0, as after bounds_check_indices,
 *                         which rewrites such an id to 0 in these modes
 *   FATAL 0, NONE 3, -1   the id is skipped (pools nothing); this is a new
 *                         plan's behaviour.  (The caller raises for FATAL from
 *                         tra_tbe_error_count; NONE means unchecked in fbgemm.)
 * Counted by tra_tbe_error_count in every mode.  Calls already launched keep
 * the mode they were launched with. */
int tra_tbe_set_bounds_check_mode(tra_tbe_t tbe, int32_t mode);

/* Number of out-of-range ids seen by forwards on this plan since the last
 * call (synchronizes the stream; resets the counter).  Stands in for the
 * report of fbgemm_gpu's bounds_check_indices. */
int tra_tbe_error_count(tra_tbe_t tbe, void* stream, int64_t* count);

/* Index math -------------------------------------------------------------- */
/* offsets[0] = 0, offsets[i+1] = sum(lengths[0..i]).  n <= 2^31-1 elements.
 * Replaces torch.ops.fbgemm.asynchronous_complete_cumsum
 * (torchrec/sparse/jagged_tensor.py:79-80).  workspace: device scratch of
 * tra_cumsum_workspace_bytes(n) bytes (may be NULL when that is 0). */
int64_t tra_cumsum_workspace_bytes(int64_t n);
int tra_cumsum(const void* lengths, int64_t n, int32_t is_i64, void* offsets,
               void* workspace, void* stream);

/* Per-feature totals: out[f] = sum(lengths[f*B .. (f+1)*B)) as int64.
 * Replaces torch.sum(lengths.view(F, B), 1) in KJT.length_per_key
 * (torchrec/sparse/jagged_tensor.py:1201-1212). */
int tra_length_per_key(const void* lengths, int32_t num_features,
                       int32_t batch_size, int32_t is_i64, int64_t* out,
                       void* stream);

/* Feature permutation of a KJT.  lengths is [T, B]; out_lengths[t', :] =
 * lengths[permute[t'], :]; values (and weights) segments follow in the new
 * order.  in_offsets / out_offsets are the complete cumsums ([T*B+1] /
 * [T'*B+1], same integer type as lengths) of lengths / out_lengths, computed by
 * the caller with tra_cumsum.  value_bytes is 4 or 8.  Replaces
 * torch.ops.fbgemm.permute_2D_sparse_data
 * (torchrec/sparse/jagged_tensor.py:2573-2583). */
int tra_permute_2d_lengths(const int32_t* permute, int32_t num_out_features,
                           int32_t num_features, int32_t batch_size,
                           const void* lengths, int32_t is_i64,
                           void* out_lengths, void* stream);
int tra_permute_2d_data(const int32_t* permute, int32_t num_out_features,
                        int32_t batch_size, const void* in_offsets,
                        const void* out_offsets, int32_t is_i64,
                        const void* values, int32_t value_bytes,
                        const float* weights, void* out_values,
                        float* out_weights, void* stream);

/* Block bucketization of ids (row-wise sharding index math).  Replaces
 * torch.ops.fbgemm.block_bucketize_sparse_features
 * (torchrec/distributed/embedding_sharding.py:153-198).
 * Step 1 writes new_lengths [W*F*B] (bucket-major); the caller cumsums them
 * into new_offsets [W*F*B+1]; step 2 scatters ids (id % block_size, or the id
 * itself if keep_orig_idx), weights, and optionally unbucketize_permute [L]
 * (output position of each input id, -1 if dropped).  Order inside one
 * (bucket, f, b) is the input order.  offsets is the complete cumsum of
 * lengths; cursor_workspace is device scratch of
 * tra_bucketize_workspace_bytes() bytes (0 up to 1024 buckets: NULL is then
 * accepted; W*F*B int64 beyond). */
int64_t tra_bucketize_workspace_bytes(int32_t num_features, int32_t batch_size,
                                      int32_t num_buckets);
int tra_bucketize_lengths(const void* offsets, const void* indices,
                          int32_t is_i64, const int64_t* block_sizes,
                          int32_t num_features, int32_t batch_size,
                          int32_t num_buckets, void* new_lengths, void* stream);
int tra_bucketize_scatter(const void* offsets, const void* indices,
                          int32_t is_i64, const float* weights,
                          const int64_t* block_sizes, int32_t num_features,
                          int32_t batch_size, int32_t num_buckets,
                          int32_t keep_orig_idx, const void* new_offsets,
                          int64_t* cursor_workspace, void* new_indices,
                          float* new_weights, int64_t* unbucketize_permute,
                          void* stream);

/* Row-wise quantization --------------------------------------------------- */
/* fp32 [rows, dim] -> packed TBE rows (header-first, row_bytes stride) written
 * straight into the table buffer at `out`; bits in {8, 4, 2}.  Same bytes as
 * torch.ops.fbgemm.FloatOrHalfToFusedNBitRowwiseQuantizedSBHalf followed by
 * the reference's trailer split (torchrec/quant/embedding_modules.py:261-276),
 * with scale/bias moved to the row header. */
int tra_quantize_rows(const float* in, int64_t rows, int32_t dim, int32_t bits,
                      uint8_t* out, int32_t row_bytes, void* stream);
/* Same input, fbgemm's own output format: [rows, dim*bits/8 + 4] with the
 * fp16 scale/bias at the END of each row. */
int tra_quantize_rows_sbhalf(const float* in, int64_t rows, int32_t dim,
                             int32_t bits, uint8_t* out, void* stream);

/* Positions inside bags ---------------------------------------------------- */
/* out[j] = j - offsets[bag(j)] for j < range_size; offsets has num_bags
 * entries (bag i ends where bag i+1 starts, the last at range_size), out the
 * same integer type.  Replaces torch.ops.fbgemm.offsets_range
 * (torchrec/modules/feature_processor_.py:82-84, 193-207). */
int tra_offsets_range(const void* offsets, int64_t num_bags, int32_t is_i64,
                      int64_t range_size, void* out, void* stream);
/* Per-id position weights of a KJT: for key k with key_len[k] > 0,
 * out[j] = table[key_start[k] + (j - start of j's bag)]; 1.0f for keys with
 * key_len[k] <= 0.  offsets: device [num_keys*batch_size + 1]; key_start,
 * key_len: device int32 [num_keys]; table: device fp32 (all keys' position
 * weights back to back).  One launch for what the reference does with
 * offsets_range + split by length_per_key (a host sync) + gather + cat
 * (torchrec/modules/feature_processor_.py:140-155, 193-220).  A position at
 * or beyond key_len[k] takes the last entry (the reference's gather raises). */
int tra_position_weights(const void* offsets, int32_t is_i64, int32_t num_keys,
                         int32_t batch_size, const int32_t* key_start,
                         const int32_t* key_len, const float* table, float* out,
                         void* stream);

/* Managed-collision id remap ------------------------------------------------ */
/* out[j] = mapping[i] if sorted_ids[i] == values[j], where i is the lower
 * bound of values[j] among the first table_size-1 entries of sorted_ids
 * (ascending int64; the last entry is the delimiter), else miss_id.  values
 * and out: device [n] int32 or int64; sorted_ids, mapping: device int64
 * [table_size].  Replaces _mch_remap (searchsorted + gather + masked writes,
 * torchrec/modules/mc_modules.py:959-989). */
int tra_mch_remap(const void* values, int64_t n, int32_t is_i64,
                  const int64_t* sorted_ids, const int64_t* mapping,
                  int64_t table_size, int64_t miss_id, void* out, void* stream);
/* The same remap for all keys of a KeyedJaggedTensor in one launch: key k's
 * ids are values[offsets[k*B] .. offsets[(k+1)*B]) (offsets: device
 * [num_keys*B + 1], same integer type as values) and are looked up in key k's
 * own table.  sorted_ids / mapping: HOST arrays of num_keys device pointers;
 * table_size / miss_id: HOST arrays.  Replaces the per-table loop of
 * ManagedCollisionCollection.forward (KJT split, one remap per table, cat;
 * torchrec/modules/mc_modules.py:383-430). */
int tra_mch_remap_keys(const void* values, int64_t n, const void* offsets, int32_t is_i64,
                       int32_t num_keys, int32_t batch_size, const int64_t* const* sorted_ids,
                       const int64_t* const* mapping, const int64_t* table_size,
                       const int64_t* miss_id, void* out, void* stream);

/* Measurement ------------------------------------------------------------- */
/* Column regroup of pooled outputs ------------------------------------------- */
/* Copies num_blocks column blocks between row-major matrices of `rows` rows:
 * block k is width[k] elements of every row, read at src[k] with row stride
 * src_stride[k] and written at dst[k] with row stride dst_stride[k] (strides in
 * elements; both pointers include the block's first column; elements of 2 or 4
 * bytes).  src, dst and the three arrays are HOST arrays.  One launch per 96
 * blocks.  Replaces the column gather behind KeyedTensor.regroup
 * (torch.ops.fbgemm.permute_pooled_embs / permute_multi_embedding or one
 * torch.cat, torchrec/sparse/jagged_tensor.py:146-172, 191-239, 3326-3344). */
int tra_regroup_columns(const void* const* src, const int64_t* src_stride, void* const* dst,
                        const int64_t* dst_stride, const int32_t* width, int32_t num_blocks,
                        int64_t rows, int32_t elem_bytes, void* stream);

/* Streaming device-to-device copy of `bytes` bytes (a multiple of 16, 16-byte
 * aligned pointers) by a kernel named tra_copy_kernel.  A copy of known size
 * under the same hardware counters calibrates FETCH_SIZE / WRITE_SIZE readings
 * of the lookup kernels.  No counterpart in the reference. */
int tra_copy_bytes(const void* src, void* dst, int64_t bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* TORCHREC_AMD_H_ */
