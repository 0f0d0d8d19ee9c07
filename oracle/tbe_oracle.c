/*
 * TEST INFRASTRUCTURE — CPU oracle for the quantized embedding inference path.
 *
 * Plain-C, scalar, single-threaded restatement of the arithmetic that
 * TorchRec's QuantEmbeddingBagCollection / QuantEmbeddingCollection forward
 * executes on CPU.  The reference (torchrec/quant/embedding_modules.py:547-557
 * pooled, :938-942 sequence, :261-265 row quantization;
 * torchrec/sparse/jagged_tensor.py:79-80 cumsum, :2573-2583 permute;
 * torchrec/distributed/embedding_sharding.py:153-198 bucketize) delegates all
 * of it to the un-vendored dependency fbgemm / fbgemm_gpu (requirements.txt:4,
 * unpinned).  The algorithms restated here are the published fbgemm ones
 * (torch/include/fbgemm/FbgemmEmbedding.h:28-45,90-175, QuantUtils.h:275-291).
 *
 * Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may
 * load this library.  The product never calls it.
 *
 * How each function is pinned (see tests/test_oracle.py):
 *   oracle_quantize_sbhalf    byte-identical to fbgemm's optimized and Ref
 *                             quantizers in libtorch_cpu (fbgemm_shim.cpp),
 *                             torch.ops.quantized.embedding_bag_{4,2}bit_prepack,
 *                             closed-form rows (constant row, exact ramps).
 *   oracle_tbe_forward        bit-identical to fbgemm's JIT kernels
 *                             GenerateEmbeddingSpMDM[NBit]WithStrides (all of
 *                             int8/int4/int2/fp16/fp32 rows x SUM/MEAN/weighted/
 *                             no_bag x fp32/fp16 out x int32/int64 ids), float64
 *                             brute force, invariants (empty bag -> 0, L=1).
 *   oracle_cumsum             numpy cumsum + golden vectors of
 *                             sparse/tests/test_keyed_jagged_tensor.py.
 *   oracle_permute_2d         golden vectors of
 *                             sparse/tests/test_keyed_jagged_tensor.py:415-626.
 *   oracle_bucketize          pure-Python block_bucketize_ref restated in the
 *                             test (distributed/tests/test_utils.py:299-466).
 *
 * Parity unpinned (nothing in the reference, fbgemm or the mathematics fixes
 * them; the oracle's choice is stated, not checked):
 *   - a -1 id in the sequence (no-bag) lookup writes a row of zeros; fbgemm's
 *     CPU no-bag kernels reject such an input instead.
 *   - an id outside [0, rows) other than -1 is skipped and reported through
 *     the return value; fbgemm_gpu's bounds-check modes are not restated.
 *
 * Build: gcc -O2 -ffp-contract=off -shared -fPIC (see oracle/Makefile).
 * -ffp-contract=off matters: the "acc + bias" add must not fuse with anything.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* SparseType codes (fbgemm_gpu SparseType.as_int()). */
enum { ST_FP32 = 0, ST_FP16 = 1, ST_INT8 = 2, ST_INT4 = 3, ST_INT2 = 4 };
/* PoolingMode codes. */
enum { PM_SUM = 0, PM_MEAN = 1, PM_NONE = 2 };

/* ---- fp16 <-> fp32, IEEE, round-to-nearest-even, denormals kept ---------- */
static float half_to_float(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1f;
  uint32_t man = h & 0x3ffu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else { /* subnormal: normalise */
      int e = -1;
      do {
        man <<= 1;
        e++;
      } while ((man & 0x400u) == 0);
      man &= 0x3ffu;
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7f800000u | (man << 13);
  } else {
    bits = sign | ((exp + 112) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

static uint16_t float_to_half_rn(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  uint32_t sign = (x >> 16) & 0x8000u;
  uint32_t abs = x & 0x7fffffffu;
  if (abs >= 0x7f800000u) { /* inf / nan */
    return (uint16_t)(sign | 0x7c00u | (abs > 0x7f800000u ? 0x200u : 0));
  }
  if (abs >= 0x477ff000u) { /* rounds to >= 65520 -> inf */
    return (uint16_t)(sign | 0x7c00u);
  }
  if (abs < 0x33000001u) { /* <= 2^-25 -> 0 (ties-to-even at exactly 2^-25) */
    return (uint16_t)sign;
  }
  int32_t e = (int32_t)(abs >> 23) - 127;
  uint32_t m = (abs & 0x7fffffu) | 0x800000u;
  uint32_t shift;
  uint32_t hexp;
  if (e < -14) { /* subnormal half */
    shift = (uint32_t)(13 + (-14 - e));
    hexp = 0;
  } else {
    shift = 13;
    hexp = (uint32_t)(e + 15);
  }
  uint32_t q = m >> shift;
  uint32_t rem = m & ((1u << shift) - 1);
  uint32_t half = 1u << (shift - 1);
  if (rem > half || (rem == half && (q & 1))) q++;
  /* q includes the implicit bit for normals; adding exp handles carry. */
  uint32_t out;
  if (hexp == 0) {
    out = q; /* may carry into exponent 1: correct */
  } else {
    out = ((hexp - 1) << 10) + q; /* q has bit 10 set */
  }
  return (uint16_t)(sign | out);
}

uint16_t oracle_float_to_half(float f) { return float_to_half_rn(f); }
float oracle_half_to_float(uint16_t h) { return half_to_float(h); }

/* ---- row-wise N-bit quantization, fp16 scale/bias TRAILER ---------------- */
/* Follows fbgemm FloatOrHalfToFusedNBitRowwiseQuantizedSBHalf (QuantUtils.h:
 * 275-291), called at torchrec/quant/embedding_modules.py:261-265.
 * out row = [payload: cols*bits/8 bytes][fp16 scale][fp16 bias].            */
int oracle_quantize_sbhalf(int bits, const float* in, int64_t rows, int cols,
                           uint8_t* out) {
  if (bits != 2 && bits != 4 && bits != 8) return -1;
  const int epb = 8 / bits;
  if (cols % epb != 0) return -2;
  const int payload = cols / epb;
  const int out_cols = payload + 4;
  const int qmax = (1 << bits) - 1;
  for (int64_t r = 0; r < rows; ++r) {
    const float* x = in + r * cols;
    uint8_t* o = out + r * out_cols;
    float mn = x[0], mx = x[0];
    for (int c = 1; c < cols; ++c) {
      if (x[c] < mn) mn = x[c];
      if (x[c] > mx) mx = x[c];
    }
    uint16_t bias_h = float_to_half_rn(mn);
    float bias = half_to_float(bias_h);
    float range = mx - bias;
    float scale = range == 0.0f ? 1.0f : range / (float)qmax;
    uint16_t scale_h = float_to_half_rn(scale);
    scale = half_to_float(scale_h);
    if (scale == 0.0f) scale = 1.0f;
    float inv = 1.0f / scale;
    if (isinf(inv)) {
      scale = 1.0f;
      inv = 1.0f;
    }
    scale_h = float_to_half_rn(scale);
    memset(o, 0, (size_t)payload);
    for (int c = 0; c < cols; ++c) {
      long q = lrintf((x[c] - bias) * inv);
      if (q < 0) q = 0;
      if (q > qmax) q = qmax;
      o[c / epb] |= (uint8_t)(q << ((c % epb) * bits));
    }
    memcpy(o + payload, &scale_h, 2);
    memcpy(o + payload + 2, &bias_h, 2);
  }
  return 0;
}

/* ---- the table-batched lookup ------------------------------------------- */
static inline int64_t load_idx(const void* p, int is64, int64_t i) {
  return is64 ? ((const int64_t*)p)[i] : (int64_t)((const int32_t*)p)[i];
}

static void store_out(void* out, int out_dtype, int64_t pos, float v) {
  if (out_dtype == ST_FP32) {
    ((float*)out)[pos] = v;
  } else {
    ((uint16_t*)out)[pos] = float_to_half_rn(v);
  }
}

/* Accumulate one table row into acc[0:D] with weight w (has_w selects the
 * weighted form).  Row layout (TBE, header first):
 *   int8/int4/int2: [fp16 scale][fp16 bias][payload]; fp16/fp32: [payload]. */
static void accumulate_row(float* acc, const uint8_t* row, int dtype, int D,
                           int has_w, float w) {
  if (dtype == ST_FP32) {
    const float* x = (const float*)row;
    for (int k = 0; k < D; ++k) acc[k] = fmaf(has_w ? w : 1.0f, x[k], acc[k]);
    return;
  }
  if (dtype == ST_FP16) {
    for (int k = 0; k < D; ++k) {
      uint16_t h;
      memcpy(&h, row + 2 * k, 2);
      acc[k] = fmaf(has_w ? w : 1.0f, half_to_float(h), acc[k]);
    }
    return;
  }
  uint16_t sh, bh;
  memcpy(&sh, row, 2);
  memcpy(&bh, row + 2, 2);
  float scale = half_to_float(sh);
  float bias = half_to_float(bh);
  if (has_w) {
    scale = w * scale; /* two separately rounded fp32 products */
    bias = w * bias;
  }
  const uint8_t* p = row + 4;
  const int bits = dtype == ST_INT8 ? 8 : (dtype == ST_INT4 ? 4 : 2);
  const int epb = 8 / bits;
  const int mask = (1 << bits) - 1;
  for (int k = 0; k < D; ++k) {
    int q = (p[k / epb] >> ((k % epb) * bits)) & mask;
    float t = acc[k] + bias; /* rounded add first ...            */
    acc[k] = fmaf(scale, (float)q, t); /* ... then one fused multiply-add */
  }
}

/*
 * One TBE group forward.  Bag (f, b) is offsets[f*B + b] .. offsets[f*B+b+1].
 * Pooled: out is [B, total_D] row-major, feature f at columns D_offsets[f].
 * PM_NONE: out is [L, D]; row j is the dequantized row of indices[j].
 * Index -1 is skipped (pruned id).  Returns 0, or -(1 + position) of the first
 * out-of-range index.
 */
int64_t oracle_tbe_forward(const uint8_t* weights, int32_t T,
                           const int64_t* table_offsets,
                           const int64_t* table_rows,
                           const int32_t* table_dims,
                           const int32_t* table_dtypes,
                           const int32_t* table_row_bytes, int32_t F,
                           const int32_t* feature_table_map,
                           const int32_t* D_offsets, int32_t B,
                           const void* indices, const void* offsets,
                           int32_t idx_is_i64,
                           const float* per_sample_weights,
                           int32_t pooling_mode, int32_t out_dtype, void* out) {
  (void)T;
  float acc[4096];
  const int64_t total_D = D_offsets[F];
  for (int32_t f = 0; f < F; ++f) {
    const int32_t t = feature_table_map[f];
    const int D = table_dims[t];
    if (D > 4096) return INT64_MIN;
    const uint8_t* base = weights + table_offsets[t];
    const int64_t stride = table_row_bytes[t];
    const int dtype = table_dtypes[t];
    for (int32_t b = 0; b < B; ++b) {
      const int64_t bag = (int64_t)f * B + b;
      const int64_t start = load_idx(offsets, idx_is_i64, bag);
      const int64_t end = load_idx(offsets, idx_is_i64, bag + 1);
      if (pooling_mode == PM_NONE) {
        for (int64_t j = start; j < end; ++j) {
          const int64_t id = load_idx(indices, idx_is_i64, j);
          for (int k = 0; k < D; ++k) acc[k] = 0.0f;
          if (id != -1) {
            if (id < 0 || id >= table_rows[t]) return -(1 + j);
            accumulate_row(acc, base + id * stride, dtype, D, 0, 1.0f);
          }
          for (int k = 0; k < D; ++k)
            store_out(out, out_dtype, j * (int64_t)D + k, acc[k]);
        }
        continue;
      }
      for (int k = 0; k < D; ++k) acc[k] = 0.0f;
      for (int64_t j = start; j < end; ++j) {
        const int64_t id = load_idx(indices, idx_is_i64, j);
        if (id == -1) continue;
        if (id < 0 || id >= table_rows[t]) return -(1 + j);
        const int has_w = per_sample_weights != 0;
        accumulate_row(acc, base + id * stride, dtype, D, has_w,
                       has_w ? per_sample_weights[j] : 1.0f);
      }
      if (pooling_mode == PM_MEAN && end > start) {
        const float inv = 1.0f / (float)(end - start);
        for (int k = 0; k < D; ++k) acc[k] *= inv;
      }
      for (int k = 0; k < D; ++k)
        store_out(out, out_dtype, (int64_t)b * total_D + D_offsets[f] + k,
                  acc[k]);
    }
  }
  return 0;
}

/* ---- index math ---------------------------------------------------------- */
/* lengths[n] -> offsets[n+1], offsets[0] = 0 (fbgemm
 * asynchronous_complete_cumsum, sparse/jagged_tensor.py:79-80).             */
void oracle_cumsum(const void* lengths, int64_t n, int is64, void* offsets) {
  int64_t run = 0;
  for (int64_t i = 0; i <= n; ++i) {
    if (is64)
      ((int64_t*)offsets)[i] = run;
    else
      ((int32_t*)offsets)[i] = (int32_t)run;
    if (i < n) run += load_idx(lengths, is64, i);
  }
}

/* permute_2D_sparse_data (sparse/jagged_tensor.py:2573-2583): lengths is
 * [T, B]; out_lengths[t', :] = lengths[permute[t'], :]; the value (and weight)
 * segments follow in the new feature order.  out_values must hold
 * sum(out_lengths) items of value_bytes each.  Returns that sum.            */
int64_t oracle_permute_2d(const int32_t* permute, int32_t Tp, int32_t T,
                          int32_t B, const void* lengths, int len_is64,
                          const void* values, int value_bytes,
                          const float* weights, void* out_lengths,
                          void* out_values, float* out_weights) {
  int64_t* in_off = (int64_t*)malloc(sizeof(int64_t) * (size_t)(T + 1));
  in_off[0] = 0;
  for (int32_t t = 0; t < T; ++t) {
    int64_t s = 0;
    for (int32_t b = 0; b < B; ++b) s += load_idx(lengths, len_is64, (int64_t)t * B + b);
    in_off[t + 1] = in_off[t] + s;
  }
  int64_t pos = 0;
  for (int32_t tp = 0; tp < Tp; ++tp) {
    const int32_t t = permute[tp];
    for (int32_t b = 0; b < B; ++b) {
      int64_t l = load_idx(lengths, len_is64, (int64_t)t * B + b);
      if (len_is64)
        ((int64_t*)out_lengths)[(int64_t)tp * B + b] = l;
      else
        ((int32_t*)out_lengths)[(int64_t)tp * B + b] = (int32_t)l;
    }
    const int64_t n = in_off[t + 1] - in_off[t];
    if (out_values)
      memcpy((uint8_t*)out_values + pos * value_bytes,
             (const uint8_t*)values + in_off[t] * value_bytes,
             (size_t)(n * value_bytes));
    if (weights && out_weights)
      memcpy(out_weights + pos, weights + in_off[t], (size_t)n * sizeof(float));
    pos += n;
  }
  free(in_off);
  return pos;
}

/* block_bucketize_sparse_features (distributed/embedding_sharding.py:153-198).
 * lengths is [F*B]; block_sizes is [F]; W buckets.  Bucket p = id / block_size
 * (ids with p >= W are dropped); new id = id % block_size (or the original id
 * if keep_orig_idx).  new_lengths is [W*F*B] bucket-major; within one
 * (bucket, f, b) the original order is kept.  unbucketize_permute[j] (optional)
 * is the output position of input j (or -1 if dropped).  Returns the number of
 * ids written.                                                              */
int64_t oracle_bucketize(const void* lengths, const void* indices, int is64,
                         const float* weights, const int64_t* block_sizes,
                         int32_t F, int32_t B, int32_t W, int keep_orig_idx,
                         void* new_lengths, void* new_indices,
                         float* new_weights, int64_t* unbucketize_permute,
                         int64_t* scratch /* [W*F*B + 1] */) {
  const int64_t n = (int64_t)F * B;
  for (int64_t i = 0; i < (int64_t)W * n; ++i) scratch[i] = 0;
  int64_t j = 0;
  for (int64_t i = 0; i < n; ++i) {
    const int64_t bs = block_sizes[i / B];
    const int64_t l = load_idx(lengths, is64, i);
    for (int64_t k = 0; k < l; ++k, ++j) {
      const int64_t id = load_idx(indices, is64, j);
      const int64_t p = id / bs;
      if (p < W) scratch[p * n + i]++;
    }
  }
  for (int64_t i = 0; i < (int64_t)W * n; ++i) {
    if (is64)
      ((int64_t*)new_lengths)[i] = scratch[i];
    else
      ((int32_t*)new_lengths)[i] = (int32_t)scratch[i];
  }
  /* exclusive scan in place -> write cursors */
  int64_t run = 0;
  for (int64_t i = 0; i < (int64_t)W * n; ++i) {
    int64_t c = scratch[i];
    scratch[i] = run;
    run += c;
  }
  j = 0;
  for (int64_t i = 0; i < n; ++i) {
    const int64_t bs = block_sizes[i / B];
    const int64_t l = load_idx(lengths, is64, i);
    for (int64_t k = 0; k < l; ++k, ++j) {
      const int64_t id = load_idx(indices, is64, j);
      const int64_t p = id / bs;
      if (p >= W) {
        if (unbucketize_permute) unbucketize_permute[j] = -1;
        continue;
      }
      const int64_t pos = scratch[p * n + i]++;
      const int64_t nid = keep_orig_idx ? id : id % bs;
      if (is64)
        ((int64_t*)new_indices)[pos] = nid;
      else
        ((int32_t*)new_indices)[pos] = (int32_t)nid;
      if (weights && new_weights) new_weights[pos] = weights[j];
      if (unbucketize_permute) unbucketize_permute[j] = pos;
    }
  }
  return run;
}
