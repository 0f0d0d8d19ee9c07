// Gather + dequantize + pool kernels for packed int-N / fp16 / fp32 embedding
// rows (gfx950, wave64).  Included by one .hip file per weight type so the
// instantiations compile in parallel.
//
// Work mapping.  A row's payload is cut into chunks of CB bytes (16, 8 or 4);
// a lane owns one chunk, i.e. a fixed, contiguous set of output columns, and
// keeps one fp32 accumulator per column in registers.  LPR = payload / CB
// lanes form a lane group that owns one bag and walks its ids in order, so the
// sum is evaluated in exactly the order and with exactly the operations of the
// CPU kernels (acc = fmaf(w*scale, q, acc + w*bias)): no cross-lane reduction
// and no reassociation.  A wave holds 64 / LPR lane groups; rows are loaded
// with one CB-byte vector load per lane, U rows per lane group in flight, with
// the next U rows requested before the current U are consumed.
#pragma once

#include <hip/hip_fp16.h>

#include <vector>

#include "tra_common.h"

namespace tra {

constexpr int kWavesPerBlock = 4;
constexpr int kBlockThreads = kWavesPerBlock * kWaveSize;
constexpr int kMaxSub = 8;

// Features of one launch that share LPR (i.e. share dim).
struct SubClass {
  int32_t first;           // index of the first feature in the class feature list
  int32_t count;           // features in this sub-class
  int32_t lpr;             // lanes per row
  int32_t tiles_per_feat;  // blocks per feature
  int32_t tile_start;      // first block of this sub-class in the grid
};

struct LookupArgs {
  const uint8_t* weights;
  const FeatureDesc* descs;  // all features of the plan (device)
  const int32_t* feats;      // feature ids of this launch (device)
  const void* indices;
  const void* offsets;
  const float* psw;
  void* out;
  int64_t out_stride;  // elements
  unsigned long long* err_count;
  int64_t num_indices;
  int32_t B;
  int32_t n_sub;
  int32_t mean;
  int32_t vec_store;  // 1: every lane's output slice is 16-byte aligned
  int32_t out_fp16;
  SubClass sub[kMaxSub];
};

// ---- element helpers ------------------------------------------------------
template <int DTYPE>
struct Traits;
template <>
struct Traits<TRA_INT8> {
  static constexpr int kBits = 8;
  static constexpr int kHeader = 4;
};
template <>
struct Traits<TRA_INT4> {
  static constexpr int kBits = 4;
  static constexpr int kHeader = 4;
};
template <>
struct Traits<TRA_INT2> {
  static constexpr int kBits = 2;
  static constexpr int kHeader = 4;
};
template <>
struct Traits<TRA_FP16> {
  static constexpr int kBits = 16;
  static constexpr int kHeader = 0;
};
template <>
struct Traits<TRA_FP32> {
  static constexpr int kBits = 32;
  static constexpr int kHeader = 0;
};

template <int CB>
struct Chunk {
  uint32_t v[CB / 4];
};

// CB bytes from a 4-byte aligned address in one vector load.
template <int CB>
__device__ __forceinline__ Chunk<CB> load_chunk(const uint8_t* p) {
  Chunk<CB> c;
  __builtin_memcpy(&c, __builtin_assume_aligned(p, 4), CB);
  return c;
}

// Byte K of x as float: a single v_cvt_f32_ubyteK.  Written as inline asm
// because the compiler otherwise extracts the byte first (v_bfe / SDWA and)
// and then converts, which costs a second VALU op per element.
template <int K>
__device__ __forceinline__ float byte_to_float(uint32_t x) {
  float f;
  if constexpr (K == 0)
    asm("v_cvt_f32_ubyte0 %0, %1" : "=v"(f) : "v"(x));
  else if constexpr (K == 1)
    asm("v_cvt_f32_ubyte1 %0, %1" : "=v"(f) : "v"(x));
  else if constexpr (K == 2)
    asm("v_cvt_f32_ubyte2 %0, %1" : "=v"(f) : "v"(x));
  else
    asm("v_cvt_f32_ubyte3 %0, %1" : "=v"(f) : "v"(x));
  return f;
}

__device__ __forceinline__ float half_bits_to_float(uint32_t h) {
  return (float)__builtin_bit_cast(_Float16, (uint16_t)h);
}

// acc = fmaf(s, q, acc + b): one rounded add, then one fused multiply-add.
__device__ __forceinline__ void fma_step(float& acc, float s, float q, float b) {
  float t = acc + b;
  acc = __builtin_fmaf(s, q, t);
}

// Accumulate the elements of one payload dword.  `acc` points at the
// accumulators of this dword's elements.  For the unweighted int4/int2 forms
// the sub-byte fields are converted in place (value q * 2^shift) and the scale
// is pre-divided by the same power of two: the product is the same real
// number, so the fused multiply-add rounds identically.  With per-sample
// weights the scale w*scale may be subnormal, where that division is inexact,
// so the fields are shifted down instead.
template <int DTYPE, bool WEIGHTED>
__device__ __forceinline__ void accumulate_dword(float* acc, uint32_t x, float s,
                                                 float b) {
  if constexpr (DTYPE == TRA_INT8) {
    fma_step(acc[0], s, byte_to_float<0>(x), b);
    fma_step(acc[1], s, byte_to_float<1>(x), b);
    fma_step(acc[2], s, byte_to_float<2>(x), b);
    fma_step(acc[3], s, byte_to_float<3>(x), b);
  } else if constexpr (DTYPE == TRA_INT4) {
    const uint32_t lo = x & 0x0f0f0f0fu;
    const uint32_t hi = WEIGHTED ? ((x >> 4) & 0x0f0f0f0fu) : (x & 0xf0f0f0f0u);
    const float sh = WEIGHTED ? s : s * 0.0625f;
    fma_step(acc[0], s, byte_to_float<0>(lo), b);
    fma_step(acc[1], sh, byte_to_float<0>(hi), b);
    fma_step(acc[2], s, byte_to_float<1>(lo), b);
    fma_step(acc[3], sh, byte_to_float<1>(hi), b);
    fma_step(acc[4], s, byte_to_float<2>(lo), b);
    fma_step(acc[5], sh, byte_to_float<2>(hi), b);
    fma_step(acc[6], s, byte_to_float<3>(lo), b);
    fma_step(acc[7], sh, byte_to_float<3>(hi), b);
  } else if constexpr (DTYPE == TRA_INT2) {
    float se = s;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const uint32_t m =
          WEIGHTED ? ((x >> (2 * e)) & 0x03030303u) : (x & (0x03030303u << (2 * e)));
      fma_step(acc[0 + e], se, byte_to_float<0>(m), b);
      fma_step(acc[4 + e], se, byte_to_float<1>(m), b);
      fma_step(acc[8 + e], se, byte_to_float<2>(m), b);
      fma_step(acc[12 + e], se, byte_to_float<3>(m), b);
      if constexpr (!WEIGHTED) se *= 0.25f;
    }
  } else if constexpr (DTYPE == TRA_FP16) {
    // s carries the per-sample weight (1.0f when unweighted).
    acc[0] = __builtin_fmaf(s, half_bits_to_float(x & 0xffffu), acc[0]);
    acc[1] = __builtin_fmaf(s, half_bits_to_float(x >> 16), acc[1]);
  } else {
    acc[0] = __builtin_fmaf(s, __builtin_bit_cast(float, x), acc[0]);
  }
}

template <typename T>
__device__ __forceinline__ int64_t load_index(const void* p, int64_t i) {
  return (int64_t) reinterpret_cast<const T*>(p)[i];
}

// One prefetched row chunk.
template <int CB>
struct RowBuf {
  Chunk<CB> d;
  uint32_t hdr;
  float w;
  int valid;  // 1: accumulate; 0: skip
};

template <int DTYPE, int CB, typename IdxT, bool WEIGHTED>
__device__ __forceinline__ void fetch_row(RowBuf<CB>& r, bool in_range, int64_t j,
                                          const LookupArgs& a, const uint8_t* table,
                                          int64_t rows, int64_t row_bytes,
                                          int chunk_off, bool count_errors) {
  r.valid = 0;
  r.hdr = 0;
  r.w = 1.0f;
  if (in_range) {
    const int64_t id = load_index<IdxT>(a.indices, j);
    if ((uint64_t)id < (uint64_t)rows) {
      const uint8_t* row = table + id * row_bytes;
      if constexpr (Traits<DTYPE>::kHeader != 0)
        r.hdr = *reinterpret_cast<const uint32_t*>(row);
      r.d = load_chunk<CB>(row + chunk_off);
      if constexpr (WEIGHTED) r.w = a.psw[j];
      r.valid = 1;
    } else if (id != -1 && count_errors) {
      atomicAdd(a.err_count, 1ull);
    }
  }
}

template <int DTYPE, int CB, bool WEIGHTED>
__device__ __forceinline__ void consume_row(float* acc, const RowBuf<CB>& r) {
  if (r.valid) {
    float s, b;
    if constexpr (Traits<DTYPE>::kHeader != 0) {
      s = half_bits_to_float(r.hdr & 0xffffu);
      b = half_bits_to_float(r.hdr >> 16);
      if constexpr (WEIGHTED) {
        s = r.w * s;
        b = r.w * b;
      }
    } else {
      s = r.w;
      b = 0.0f;
    }
    constexpr int EPD = 32 / Traits<DTYPE>::kBits;  // elements per dword
#pragma unroll
    for (int i = 0; i < CB / 4; ++i)
      accumulate_dword<DTYPE, WEIGHTED>(acc + i * EPD, r.d.v[i], s, b);
  }
}

// Store NE consecutive outputs starting at element `pos`.
template <int NE>
__device__ __forceinline__ void store_outputs(const LookupArgs& a, int64_t pos,
                                              const float* acc) {
  if (a.out_fp16) {
    __half* o = reinterpret_cast<__half*>(a.out) + pos;
    if constexpr (NE >= 8) {
      if (a.vec_store) {
#pragma unroll
        for (int i = 0; i < NE; i += 8) {
          uint4 v;
          uint32_t* pv = reinterpret_cast<uint32_t*>(&v);
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            const uint32_t lo = __half_as_ushort(__float2half_rn(acc[i + 2 * k]));
            const uint32_t hi = __half_as_ushort(__float2half_rn(acc[i + 2 * k + 1]));
            pv[k] = lo | (hi << 16);
          }
          *reinterpret_cast<uint4*>(o + i) = v;
        }
        return;
      }
    }
#pragma unroll
    for (int i = 0; i < NE; ++i) o[i] = __float2half_rn(acc[i]);
  } else {
    float* o = reinterpret_cast<float*>(a.out) + pos;
    if constexpr (NE >= 4) {
      if (a.vec_store) {
#pragma unroll
        for (int i = 0; i < NE; i += 4)
          *reinterpret_cast<float4*>(o + i) =
              make_float4(acc[i], acc[i + 1], acc[i + 2], acc[i + 3]);
        return;
      }
    }
#pragma unroll
    for (int i = 0; i < NE; ++i) o[i] = acc[i];
  }
}

__device__ __forceinline__ int wave_max(int v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const int o = __shfl_xor(v, off, 64);
    v = o > v ? o : v;
  }
  return v;
}

// Locate this block's (sub-class, feature, tile).  Uniform across the block.
__device__ __forceinline__ bool locate_tile(const LookupArgs& a, int& f, int& lpr,
                                            int& tile) {
  const int blk = blockIdx.x;
  int s = 0;
#pragma unroll
  for (int i = 1; i < kMaxSub; ++i)
    if (i < a.n_sub && blk >= a.sub[i].tile_start) s = i;
  const SubClass sc = a.sub[s];
  const int local = blk - sc.tile_start;
  const int fi = local / sc.tiles_per_feat;
  if (fi >= sc.count) return false;
  tile = local - fi * sc.tiles_per_feat;
  f = a.feats[sc.first + fi];
  lpr = sc.lpr;
  return true;
}

// ---- pooled lookup: one lane group per bag --------------------------------
template <int DTYPE, int CB, typename IdxT, bool WEIGHTED, int U>
__global__ __launch_bounds__(kBlockThreads) void tbe_pooled_kernel(const LookupArgs a) {
  constexpr int NE = CB * 8 / Traits<DTYPE>::kBits;  // columns per lane
  int f, lpr, tile;
  if (!locate_tile(a, f, lpr, tile)) return;
  const FeatureDesc d = a.descs[f];
  const int lane = threadIdx.x & (kWaveSize - 1);
  const int wave = threadIdx.x / kWaveSize;
  const int gpw = kWaveSize / lpr;  // lane groups (bags) per wave
  const int g = lane / lpr;
  const int c = lane - g * lpr;
  const int bag_in_feat = (tile * kWavesPerBlock + wave) * gpw + g;
  const bool active = g < gpw && bag_in_feat < a.B;

  int64_t start = 0, end = 0;
  if (active) {
    const int64_t bag = (int64_t)d.feature * a.B + bag_in_feat;
    start = load_index<IdxT>(a.offsets, bag);
    end = load_index<IdxT>(a.offsets, bag + 1);
  }
  const int len = (int)(end - start);
  const int max_len = wave_max(len);

  const uint8_t* table = a.weights + d.table_offset;
  const int chunk_off = Traits<DTYPE>::kHeader + d.payload_off + c * CB;
  const int64_t rows = d.rows;
  const int64_t row_bytes = d.row_bytes;
  const bool count_errors = c == 0 && d.payload_off == 0;

  float acc[NE];
#pragma unroll
  for (int i = 0; i < NE; ++i) acc[i] = 0.0f;

  RowBuf<CB> bufA[U], bufB[U];
#pragma unroll
  for (int u = 0; u < U; ++u)
    fetch_row<DTYPE, CB, IdxT, WEIGHTED>(bufA[u], u < len, start + u, a, table, rows,
                                          row_bytes, chunk_off, count_errors);
  for (int it = 0; it < max_len; it += 2 * U) {
#pragma unroll
    for (int u = 0; u < U; ++u)
      fetch_row<DTYPE, CB, IdxT, WEIGHTED>(bufB[u], it + U + u < len, start + it + U + u,
                                            a, table, rows, row_bytes, chunk_off, count_errors);
#pragma unroll
    for (int u = 0; u < U; ++u) consume_row<DTYPE, CB, WEIGHTED>(acc, bufA[u]);
    if (it + U >= max_len) break;
#pragma unroll
    for (int u = 0; u < U; ++u)
      fetch_row<DTYPE, CB, IdxT, WEIGHTED>(bufA[u], it + 2 * U + u < len,
                                            start + it + 2 * U + u, a, table, rows,
                                            row_bytes, chunk_off, count_errors);
#pragma unroll
    for (int u = 0; u < U; ++u) consume_row<DTYPE, CB, WEIGHTED>(acc, bufB[u]);
  }

  if (!active) return;
  if (a.mean && len > 0) {
    const float inv = 1.0f / (float)len;
#pragma unroll
    for (int i = 0; i < NE; ++i) acc[i] *= inv;
  }
  const int64_t pos = (int64_t)bag_in_feat * a.out_stride + d.out_col + (int64_t)c * NE;
  store_outputs<NE>(a, pos, acc);
}

// ---- sequence lookup: one lane group per id, no reduction -----------------
// Blocks of feature f stride over that feature's ids
// [offsets[f*B], offsets[(f+1)*B]); output row j is the dequantized row of
// indices[j] (zeros for a skipped id).
template <int DTYPE, int CB, typename IdxT>
__global__ __launch_bounds__(kBlockThreads) void tbe_nobag_kernel(const LookupArgs a) {
  constexpr int NE = CB * 8 / Traits<DTYPE>::kBits;
  int f, lpr, tile;
  if (!locate_tile(a, f, lpr, tile)) return;
  const FeatureDesc d = a.descs[f];
  const int lane = threadIdx.x & (kWaveSize - 1);
  const int wave = threadIdx.x / kWaveSize;
  const int gpw = kWaveSize / lpr;
  const int g = lane / lpr;
  const int c = lane - g * lpr;
  if (g >= gpw) return;
  const int64_t first = load_index<IdxT>(a.offsets, (int64_t)d.feature * a.B);
  const int64_t last = load_index<IdxT>(a.offsets, (int64_t)(d.feature + 1) * a.B);
  const int rows_per_block = gpw * kWavesPerBlock;
  // tiles_per_feat of the sub-class = number of blocks striding over one feature
  int s = 0;
#pragma unroll
  for (int i = 1; i < kMaxSub; ++i)
    if (i < a.n_sub && (int)blockIdx.x >= a.sub[i].tile_start) s = i;
  const int64_t stride = (int64_t)a.sub[s].tiles_per_feat * rows_per_block;

  const uint8_t* table = a.weights + d.table_offset;
  const int chunk_off = Traits<DTYPE>::kHeader + d.payload_off + c * CB;
  const bool count_errors = c == 0 && d.payload_off == 0;
  for (int64_t j = first + (int64_t)tile * rows_per_block + wave * gpw + g; j < last;
       j += stride) {
    RowBuf<CB> r;
    fetch_row<DTYPE, CB, IdxT, false>(r, true, j, a, table, d.rows, d.row_bytes, chunk_off, count_errors);
    float acc[NE];
#pragma unroll
    for (int i = 0; i < NE; ++i) acc[i] = 0.0f;
    consume_row<DTYPE, CB, false>(acc, r);
    store_outputs<NE>(a, j * (int64_t)d.dim + d.payload_off * 8 / Traits<DTYPE>::kBits + (int64_t)c * NE,
                      acc);
  }
}

// ---- host side of one launch ----------------------------------------------
struct LaunchClass {
  int dtype;
  int cb;
  std::vector<int32_t> feats;  // plan order: sorted by lpr
  std::vector<int32_t> lprs;   // lanes per row of each feature
  int32_t* feats_dev = nullptr;
};

template <int DTYPE>
int launch_lookup(const LaunchClass& cls, LookupArgs a, int cb, bool idx64, bool weighted,
                  bool nobag, int grid, hipStream_t stream);

template <int DTYPE, int CB>
int launch_lookup_cb(LookupArgs a, bool idx64, bool weighted, bool nobag, int grid,
                     hipStream_t stream) {
  constexpr int U = 4;
  dim3 g(grid), b(kBlockThreads);
  if (nobag) {
    if (idx64)
      hipLaunchKernelGGL((tbe_nobag_kernel<DTYPE, CB, int64_t>), g, b, 0, stream, a);
    else
      hipLaunchKernelGGL((tbe_nobag_kernel<DTYPE, CB, int32_t>), g, b, 0, stream, a);
  } else if (weighted) {
    if (idx64)
      hipLaunchKernelGGL((tbe_pooled_kernel<DTYPE, CB, int64_t, true, U>), g, b, 0, stream, a);
    else
      hipLaunchKernelGGL((tbe_pooled_kernel<DTYPE, CB, int32_t, true, U>), g, b, 0, stream, a);
  } else {
    if (idx64)
      hipLaunchKernelGGL((tbe_pooled_kernel<DTYPE, CB, int64_t, false, U>), g, b, 0, stream, a);
    else
      hipLaunchKernelGGL((tbe_pooled_kernel<DTYPE, CB, int32_t, false, U>), g, b, 0, stream, a);
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return hip_fail(e, "tbe lookup launch");
  return TRA_OK;
}

#define TRA_DEFINE_LAUNCH(DTYPE)                                                        \
  template <>                                                                           \
  int launch_lookup<DTYPE>(const LaunchClass&, LookupArgs a, int cb, bool idx64,        \
                           bool weighted, bool nobag, int grid, hipStream_t stream) {   \
    switch (cb) {                                                                       \
      case 16: return launch_lookup_cb<DTYPE, 16>(a, idx64, weighted, nobag, grid, stream); \
      case 8: return launch_lookup_cb<DTYPE, 8>(a, idx64, weighted, nobag, grid, stream);   \
      case 4: return launch_lookup_cb<DTYPE, 4>(a, idx64, weighted, nobag, grid, stream);   \
    }                                                                                   \
    set_error("bad chunk size %d", cb);                                                 \
    return TRA_ERR_INVALID_ARGUMENT;                                                    \
  }

}  // namespace tra
