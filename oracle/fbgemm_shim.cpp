// TEST INFRASTRUCTURE — C-ABI wrapper over the core fbgemm CPU library that
// ships inside PyTorch's libtorch_cpu.so (weak exported symbols, headers in
// torch/include/fbgemm/).  fbgemm is the library TorchRec's CPU quantized
// inference path bottoms out in: IntNBitTableBatchedEmbeddingBagsCodegen on
// HOST runs, per table, a JIT kernel from GenerateEmbeddingSpMDM[NBit]
// WithStrides with scale_bias_last=false (reference call site
// torchrec/quant/embedding_modules.py:547-557, :938-942), and
// quantize_state_dict calls FloatOrHalfToFusedNBitRowwiseQuantizedSBHalf
// (torchrec/quant/embedding_modules.py:261-265).
//
// This file holds no arithmetic of its own.  It is used (a) to pin the scalar
// restatement in tbe_oracle.c bit-for-bit and (b) as the timed CPU baseline.
// Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg load it.
//
// Same argument convention as oracle_tbe_forward in tbe_oracle.c.
#include <fbgemm/FbgemmEmbedding.h>
#include <fbgemm/QuantUtils.h>

#include <algorithm>
#include <cstdint>
#include <cstring>
#include <vector>

#ifdef _OPENMP
#include <omp.h>
#endif

namespace {
enum { ST_FP32 = 0, ST_FP16 = 1, ST_INT8 = 2, ST_INT4 = 3, ST_INT2 = 4 };
enum { PM_SUM = 0, PM_MEAN = 1, PM_NONE = 2 };

template <typename Idx, typename Out>
typename fbgemm::EmbeddingSpMDMKernelSignature<uint8_t, Idx, Idx, Out>::Type
make_u8_kernel(int dtype, int D, bool has_w, bool mean, int64_t out_stride,
               int64_t row_bytes, bool no_bag) {
  if (dtype == ST_INT8) {
    return fbgemm::GenerateEmbeddingSpMDMWithStrides<uint8_t, Idx, Idx, Out,
                                                     /*THREAD_LOCAL=*/true>(
        D, has_w, mean, /*prefetch=*/16, /*is_weight_positional=*/false,
        /*use_offsets=*/true, out_stride, row_bytes,
        /*scale_bias_last=*/false, no_bag);
  }
  const int bits = dtype == ST_INT4 ? 4 : 2;
  return fbgemm::GenerateEmbeddingSpMDMNBitWithStrides<Idx, Idx, Out,
                                                       /*THREAD_LOCAL=*/true>(
      bits, D, has_w, mean, 16, false, true, out_stride, row_bytes,
      /*scale_bias_last=*/false, /*is_bf16_out=*/false, no_bag);
}

template <typename Idx, typename Out>
int64_t run(const uint8_t* weights, const int64_t* table_offsets,
            const int64_t* table_rows, const int32_t* table_dims,
            const int32_t* table_dtypes, const int32_t* table_row_bytes,
            int32_t F, const int32_t* feature_table_map,
            const int32_t* D_offsets, int32_t B, const Idx* indices,
            const Idx* offsets, const float* psw, int32_t pooling_mode,
            Out* out, int nthreads) {
  const bool no_bag = pooling_mode == PM_NONE;
  const bool mean = pooling_mode == PM_MEAN;
  const bool has_w = psw != nullptr && !no_bag;
  const int64_t total_D = D_offsets[F];
  int64_t status = 0;
  for (int32_t f = 0; f < F; ++f) {
    const int32_t t = feature_table_map[f];
    const int D = table_dims[t];
    const int dtype = table_dtypes[t];
    const int64_t row_bytes = table_row_bytes[t];
    const int64_t out_stride = no_bag ? D : total_D;
    const uint8_t* base = weights + table_offsets[t];
    const Idx* offs = offsets + (int64_t)f * B;
    const int64_t first = offs[0];
    // Bags of this feature are split into contiguous chunks, one per thread.
    const int chunks = std::max(1, std::min<int>(nthreads, B));
#ifdef _OPENMP
#pragma omp parallel for num_threads(chunks) schedule(static)
#endif
    for (int c = 0; c < chunks; ++c) {
      const int32_t b0 = (int64_t)B * c / chunks;
      const int32_t b1 = (int64_t)B * (c + 1) / chunks;
      if (b1 == b0) continue;
      const int64_t i0 = offs[b0];
      const int64_t i1 = offs[b1];
      // fbgemm wants offsets relative to the indices pointer it is given.
      const int64_t index_size = i1 - i0;
      // Sequence mode: every id is its own output row.  The 8-bit / fp16 / fp32
      // generators have a no_bag flavour; the N-bit generator only offers it
      // for int4 -> int4 output, so there each id becomes a one-element bag
      // (same arithmetic: acc starts at 0).
      const bool nbit = dtype == ST_INT4 || dtype == ST_INT2;
      const bool kernel_no_bag = no_bag && !nbit;
      const int64_t output_size = no_bag ? index_size : b1 - b0;
      std::vector<Idx> rel(output_size + 1);
      if (no_bag) {
        for (int64_t j = 0; j <= index_size; ++j) rel[j] = (Idx)j;
      } else {
        for (int32_t b = b0; b <= b1; ++b) rel[b - b0] = offs[b] - (Idx)i0;
      }
      Out* o = no_bag ? out + i0 * D : out + (int64_t)b0 * total_D + D_offsets[f];
      bool ok = true;
      if (dtype == ST_FP16) {
        auto k = fbgemm::GenerateEmbeddingSpMDMWithStrides<
            fbgemm::float16, Idx, Idx, Out, true>(
            D, has_w, mean, 16, false, true, out_stride, row_bytes / 2,
            /*scale_bias_last=*/false, kernel_no_bag);
        ok = k(output_size, index_size, table_rows[t],
               reinterpret_cast<const fbgemm::float16*>(base), indices + i0,
               rel.data(), has_w ? psw + i0 : nullptr, o);
      } else if (dtype == ST_FP32) {
        auto k = fbgemm::GenerateEmbeddingSpMDMWithStrides<float, Idx, Idx, Out,
                                                           true>(
            D, has_w, mean, 16, false, true, out_stride, row_bytes / 4,
            /*scale_bias_last=*/false, kernel_no_bag);
        ok = k(output_size, index_size, table_rows[t],
               reinterpret_cast<const float*>(base), indices + i0, rel.data(),
               has_w ? psw + i0 : nullptr, o);
      } else {
        auto k = make_u8_kernel<Idx, Out>(dtype, D, has_w, mean, out_stride,
                                          row_bytes, kernel_no_bag);
        ok = k(output_size, index_size, table_rows[t], base, indices + i0,
               rel.data(), has_w ? psw + i0 : nullptr, o);
      }
      if (!ok) {
#ifdef _OPENMP
#pragma omp critical
#endif
        status = -(1 + first);
      }
    }
  }
  return status;
}
}  // namespace

extern "C" {

// 1 if this torch build exports the fbgemm embedding kernels.
int fbgemm_shim_available() { return 1; }

int fbgemm_shim_max_threads() {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

// fbgemm's row-wise N-bit quantizer (optimized path, or the Ref one).
int fbgemm_quantize_sbhalf(int bits, const float* in, int64_t rows, int cols,
                           uint8_t* out, int use_ref) {
  if (use_ref)
    fbgemm::FloatOrHalfToFusedNBitRowwiseQuantizedSBHalfRef<float>(
        bits, in, (size_t)rows, cols, out);
  else
    fbgemm::FloatOrHalfToFusedNBitRowwiseQuantizedSBHalf<float>(
        bits, in, (size_t)rows, cols, out);
  return 0;
}

int64_t fbgemm_tbe_forward(const uint8_t* weights, int32_t T,
                           const int64_t* table_offsets,
                           const int64_t* table_rows,
                           const int32_t* table_dims,
                           const int32_t* table_dtypes,
                           const int32_t* table_row_bytes, int32_t F,
                           const int32_t* feature_table_map,
                           const int32_t* D_offsets, int32_t B,
                           const void* indices, const void* offsets,
                           int32_t idx_is_i64, const float* psw,
                           int32_t pooling_mode, int32_t out_dtype, void* out,
                           int32_t nthreads) {
  (void)T;
#define GO(IDX, OUT)                                                          \
  return run<IDX, OUT>(weights, table_offsets, table_rows, table_dims,        \
                       table_dtypes, table_row_bytes, F, feature_table_map,   \
                       D_offsets, B, (const IDX*)indices, (const IDX*)offsets, \
                       psw, pooling_mode, (OUT*)out, nthreads)
  if (idx_is_i64) {
    if (out_dtype == ST_FP32) GO(int64_t, float);
    GO(int64_t, fbgemm::float16);
  }
  if (out_dtype == ST_FP32) GO(int32_t, float);
  GO(int32_t, fbgemm::float16);
#undef GO
}

}  // extern "C"
