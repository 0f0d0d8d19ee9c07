// Index math around the lookup (offsets, per-key totals, feature permutation,
// block bucketization) and the row-wise quantizer.  Integer results are
// bit-exact by construction; these are bandwidth-trivial next to the gather.
#include <hip/hip_fp16.h>

#include <algorithm>
#include <cstring>

#include "tra_common.h"

namespace tra {

constexpr int kScanThreads = 256;
constexpr int kScanItems = 16;
constexpr int kScanTile = kScanThreads * kScanItems;

template <typename T>
__device__ __forceinline__ int64_t ld(const void* p, int64_t i) {
  return (int64_t) reinterpret_cast<const T*>(p)[i];
}
template <typename T>
__device__ __forceinline__ void st(void* p, int64_t i, int64_t v) {
  reinterpret_cast<T*>(p)[i] = (T)v;
}

__device__ __forceinline__ int64_t wave_sum(int64_t v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

// Block-wide sum; result valid in every thread.  `smem` holds >= 4 int64.
__device__ __forceinline__ int64_t block_sum(int64_t v, int64_t* smem) {
  v = wave_sum(v);
  const int wave = threadIdx.x / kWaveSize;
  __syncthreads();
  if ((threadIdx.x & (kWaveSize - 1)) == 0) smem[wave] = v;
  __syncthreads();
  int64_t t = 0;
  for (int w = 0; w < (int)(blockDim.x / kWaveSize); ++w) t += smem[w];
  return t;
}

// ---- complete cumsum --------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(kScanThreads) void tile_sums_kernel(const void* in, int64_t n,
                                                                  int64_t* sums) {
  __shared__ int64_t smem[kScanThreads / kWaveSize];
  const int64_t base = (int64_t)blockIdx.x * kScanTile;
  int64_t x[kScanItems];
#pragma unroll
  for (int k = 0; k < kScanItems; ++k) {
    const int64_t i = base + k * kScanThreads + threadIdx.x;
    x[k] = i < n ? ld<T>(in, i) : 0;
  }
  int64_t v = 0;
#pragma unroll
  for (int k = 0; k < kScanItems; ++k) v += x[k];
  v = block_sum(v, smem);
  if (threadIdx.x == 0) sums[blockIdx.x] = v;
}

// One-launch variant for short inputs: every block first sums everything in
// front of its tile (redundant reads, a few hundred KB from L2 at most), then
// scans the tile.  Tiles are kSmallThreads * (16 / sizeof(T)) elements.
constexpr int kSmallThreads = 1024;
constexpr int kSmallMaxTiles = 64;

template <typename T, bool VEC>
__global__ __launch_bounds__(kSmallThreads) void scan_small_kernel(const T* __restrict__ in,
                                                                    int64_t n, T* __restrict__ out) {
  constexpr int V = 16 / (int)sizeof(T);
  struct __align__(16) Vec { T v[V]; };
  __shared__ int64_t smem[kSmallThreads / kWaveSize];
  __shared__ int64_t wave_tot[kSmallThreads / kWaveSize];
  const int t = threadIdx.x;
  int64_t pre = 0;
  if (VEC) {
    // The tiles in front of this block's: sixteen loads in flight per thread (the last block of
    // a 64-tile input reads 63 tiles; one load at a time would be 63 round trips).
    const Vec* vin = reinterpret_cast<const Vec*>(in);
    const int nk = (int)blockIdx.x;
    int k = 0;
    for (; k + 16 <= nk; k += 16) {
      Vec x[16];
#pragma unroll
      for (int j = 0; j < 16; ++j) x[j] = vin[(int64_t)(k + j) * kSmallThreads + t];
#pragma unroll
      for (int j = 0; j < 16; ++j)
#pragma unroll
        for (int i = 0; i < V; ++i) pre += (int64_t)x[j].v[i];
    }
    for (; k + 4 <= nk; k += 4) {
      Vec x[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) x[j] = vin[(int64_t)(k + j) * kSmallThreads + t];
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < V; ++i) pre += (int64_t)x[j].v[i];
    }
    for (; k < nk; ++k) {
      const Vec x = vin[(int64_t)k * kSmallThreads + t];
#pragma unroll
      for (int i = 0; i < V; ++i) pre += (int64_t)x.v[i];
    }
  } else {
#pragma unroll 4
    for (int k = 0; k < (int)blockIdx.x * V; ++k) pre += (int64_t)in[(int64_t)k * kSmallThreads + t];
  }
  pre = block_sum(pre, smem);
  const int64_t base = ((int64_t)blockIdx.x * kSmallThreads + t) * V;
  int64_t x[V];
  if (VEC && base + V <= n) {
    const Vec q = reinterpret_cast<const Vec*>(in)[base / V];
#pragma unroll
    for (int i = 0; i < V; ++i) x[i] = (int64_t)q.v[i];
  } else {
#pragma unroll
    for (int i = 0; i < V; ++i) x[i] = base + i < n ? (int64_t)in[base + i] : 0;
  }
  int64_t tsum = 0;
#pragma unroll
  for (int i = 0; i < V; ++i) tsum += x[i];
  const int lane = t & (kWaveSize - 1);
  const int wave = t / kWaveSize;
  int64_t inc = tsum;
#pragma unroll
  for (int off = 1; off < kWaveSize; off <<= 1) {
    const int64_t o = __shfl_up(inc, off, 64);
    if (lane >= off) inc += o;
  }
  if (lane == kWaveSize - 1) wave_tot[wave] = inc;
  __syncthreads();
  int64_t wprefix = 0;
  for (int w = 0; w < wave; ++w) wprefix += wave_tot[w];
  int64_t run = pre + wprefix + inc - tsum;
  if (blockIdx.x == 0 && t == 0) out[0] = 0;
#pragma unroll
  for (int i = 0; i < V; ++i) {
    run += x[i];
    if (base + i < n) out[base + i + 1] = (T)run;
  }
}

template <typename T>
__global__ __launch_bounds__(kScanThreads) void scan_tiles_kernel(const void* in, int64_t n,
                                                                   const int64_t* sums, void* out) {
  __shared__ int64_t smem[kScanThreads / kWaveSize];
  __shared__ int64_t wave_tot[kScanThreads / kWaveSize];
  // Sum of all earlier tiles.
  int64_t prefix = 0;
  if (sums) {
    for (int i = threadIdx.x; i < (int)blockIdx.x; i += kScanThreads) prefix += sums[i];
    prefix = block_sum(prefix, smem);
  }
  // Each thread owns kScanItems consecutive elements.
  const int64_t base = (int64_t)blockIdx.x * kScanTile + (int64_t)threadIdx.x * kScanItems;
  int64_t x[kScanItems];
  int64_t tsum = 0;
#pragma unroll
  for (int i = 0; i < kScanItems; ++i) {
    x[i] = base + i < n ? ld<T>(in, base + i) : 0;
    tsum += x[i];
  }
  // Exclusive scan of the per-thread sums: wave scan, then wave totals.
  const int lane = threadIdx.x & (kWaveSize - 1);
  const int wave = threadIdx.x / kWaveSize;
  int64_t inc = tsum;
#pragma unroll
  for (int off = 1; off < kWaveSize; off <<= 1) {
    const int64_t o = __shfl_up(inc, off, 64);
    if (lane >= off) inc += o;
  }
  if (lane == kWaveSize - 1) wave_tot[wave] = inc;
  __syncthreads();
  int64_t wprefix = 0;
  for (int w = 0; w < wave; ++w) wprefix += wave_tot[w];
  int64_t run = prefix + wprefix + inc - tsum;
  if (blockIdx.x == 0 && threadIdx.x == 0) st<T>(out, 0, 0);
#pragma unroll
  for (int i = 0; i < kScanItems; ++i) {
    run += x[i];
    if (base + i < n) st<T>(out, base + i + 1, run);
  }
}

// ---- per-key totals ---------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(kScanThreads) void length_per_key_kernel(const void* lengths,
                                                                       int32_t B, int64_t* out) {
  __shared__ int64_t smem[kScanThreads / kWaveSize];
  const int64_t base = (int64_t)blockIdx.x * B;
  int64_t v = 0;
  for (int i = threadIdx.x; i < B; i += kScanThreads) v += ld<T>(lengths, base + i);
  v = block_sum(v, smem);
  if (threadIdx.x == 0) out[blockIdx.x] = v;
}

// ---- feature permutation ----------------------------------------------------
template <typename T>
__global__ void permute_lengths_kernel(const int32_t* permute, int64_t total, int32_t B,
                                       const void* lengths, void* out) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const int64_t tp = i / B;
  const int64_t b = i - tp * B;
  st<T>(out, i, ld<T>(lengths, (int64_t)permute[tp] * B + b));
}

// All values of one feature are contiguous on both sides, so each output
// feature is one straight copy.  grid = (blocks per feature, T').
template <typename OffT, typename ValT>
__global__ void permute_data_kernel(const int32_t* permute, int32_t B, const void* in_off,
                                    const void* out_off, const ValT* values, const float* weights,
                                    ValT* out_values, float* out_weights) {
  const int tp = blockIdx.y;
  const int64_t src = ld<OffT>(in_off, (int64_t)permute[tp] * B);
  const int64_t dst = ld<OffT>(out_off, (int64_t)tp * B);
  const int64_t n = ld<OffT>(out_off, (int64_t)(tp + 1) * B) - dst;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x) {
    out_values[dst + i] = values[src + i];
    if (weights) out_weights[dst + i] = weights[src + i];
  }
}

// ---- block bucketization ----------------------------------------------------
// One thread per bag (f, b); a bag's ids are visited in order, so the order
// inside one (bucket, f, b) is the input order.
template <typename T>
__global__ void bucketize_lengths_kernel(const void* offsets, const void* indices,
                                         const int64_t* block_sizes, int32_t B, int64_t n,
                                         int32_t W, void* new_lengths) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  T* nl = reinterpret_cast<T*>(new_lengths);
  for (int p = 0; p < W; ++p) nl[(int64_t)p * n + i] = 0;
  const int64_t bs = block_sizes[i / B];
  const int64_t s = ld<T>(offsets, i), e = ld<T>(offsets, i + 1);
  for (int64_t j = s; j < e; ++j) {
    const int64_t id = ld<T>(indices, j);
    const uint64_t p = (uint64_t)id / (uint64_t)bs;
    if (p < (uint64_t)W) nl[(int64_t)p * n + i] += 1;
  }
}

template <typename T>
__global__ void bucketize_scatter_kernel(const void* offsets, const void* indices,
                                         const float* weights, const int64_t* block_sizes,
                                         int32_t B, int64_t n, int32_t W, int keep_orig,
                                         const void* new_offsets, int64_t* cursor,
                                         void* new_indices, float* new_weights,
                                         int64_t* unbucketize_permute) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  for (int p = 0; p < W; ++p) cursor[(int64_t)p * n + i] = ld<T>(new_offsets, (int64_t)p * n + i);
  const int64_t bs = block_sizes[i / B];
  const int64_t s = ld<T>(offsets, i), e = ld<T>(offsets, i + 1);
  for (int64_t j = s; j < e; ++j) {
    const int64_t id = ld<T>(indices, j);
    const uint64_t p = (uint64_t)id / (uint64_t)bs;
    if (p >= (uint64_t)W) {
      if (unbucketize_permute) unbucketize_permute[j] = -1;
      continue;
    }
    const int64_t pos = cursor[(int64_t)p * n + i]++;
    st<T>(new_indices, pos, keep_orig ? id : (int64_t)((uint64_t)id % (uint64_t)bs));
    if (weights) new_weights[pos] = weights[j];
    if (unbucketize_permute) unbucketize_permute[j] = pos;
  }
}

// ---- a wave walking the ids of its own run of bags ---------------------------
// The id-parallel kernels below (bucketization, positions in bags, position
// weights) share one mapping: a wave owns `bpw` consecutive bags (a power of
// two, at most 64), keeps their bounds in LDS and visits their ids in order,
// 64 at a time, so every load and store of ids is coalesced; the bag of an id
// is found by a branch-free search over the wave's bounds.  Waves never share
// LDS, so the only synchronization is program order inside the wave.
constexpr int kWalkThreads = 256;
constexpr int kWalkWaves = kWalkThreads / kWaveSize;
constexpr int kWalkMaxBuckets = 1024;  // wider bucketizations take the thread-per-bag kernels

__device__ __forceinline__ void wave_lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront", "local");
  __builtin_amdgcn_wave_barrier();
}

// Largest b in [0, cnt) with off[b] <= j; off[0] <= j holds.  top_step = bpw / 2.
__device__ __forceinline__ int find_bag(const int64_t* off, int cnt, int top_step, int64_t j) {
  int lo = 0;
  for (int step = top_step; step >= 1; step >>= 1) {
    const int c = lo + step;
    if (c < cnt && off[c] <= j) lo = c;
  }
  return lo;
}

// id / bs and id % bs; 32-bit arithmetic where both fit.
__device__ __forceinline__ void div_mod(uint64_t id, uint64_t bs, uint64_t& q, uint64_t& r) {
  if (((id | bs) >> 32) == 0) {
    const uint32_t a = (uint32_t)id, b = (uint32_t)bs;
    const uint32_t qq = a / b;
    q = qq;
    r = a - qq * b;
  } else {
    q = id / bs;
    r = id - q * bs;
  }
}

// Bags per wave for n bags.  The kernels are bound by the latency of a wave's
// chain (bounds, search, ids, stores), so many short waves beat few long ones:
// 64 bags, halved down to 8 while that leaves fewer than 16384 waves (measured
// on 131072 and 262144 bags: 1.5x faster than 4096 waves), further only while
// fewer than 4096 (a wave should still find about a wave's worth of ids), and
// never more than `cap`.
static int bags_per_wave(int64_t n, int cap) {
  int bpw = 64;
  while (bpw > 8 && (n + bpw - 1) / bpw < 16384) bpw >>= 1;
  while (bpw > 1 && (n + bpw - 1) / bpw < 4096) bpw >>= 1;
  while (bpw > cap) bpw >>= 1;
  return bpw;
}

template <typename T>
__global__ __launch_bounds__(kWalkThreads) void bucketize_lengths_wave_kernel(
    const T* __restrict__ offsets, const T* __restrict__ indices, const int64_t* __restrict__ block_sizes,
    int32_t B, int64_t n, int32_t W, int bpw, T* __restrict__ new_lengths) {
  extern __shared__ int64_t walk_smem[];
  const int lane = threadIdx.x & (kWaveSize - 1);
  const int wave = threadIdx.x / kWaveSize;
  const int per_wave = (bpw + 1) + bpw + (W * bpw + 1) / 2;  // int64 units
  int64_t* s_off = walk_smem + (size_t)wave * per_wave;
  int64_t* s_bs = s_off + bpw + 1;
  int32_t* s_cnt = reinterpret_cast<int32_t*>(s_bs + bpw);
  const int64_t i0 = ((int64_t)blockIdx.x * kWalkWaves + wave) * bpw;
  if (i0 >= n) return;
  const int cnt = (int)(n - i0 < bpw ? n - i0 : bpw);
  for (int k = lane; k <= cnt; k += kWaveSize) s_off[k] = (int64_t)offsets[i0 + k];
  for (int k = lane; k < cnt; k += kWaveSize) s_bs[k] = block_sizes[(i0 + k) / B];
  for (int k = lane; k < W * bpw; k += kWaveSize) s_cnt[k] = 0;
  wave_lds_sync();
  const int64_t first = s_off[0], last = s_off[cnt];
  for (int64_t j0 = first; j0 < last; j0 += kWaveSize) {
    const int64_t j = j0 + lane;
    if (j < last) {
      const int64_t id = (int64_t)indices[j];
      const int b = find_bag(s_off, cnt, bpw >> 1, j);
      uint64_t q, r;
      div_mod((uint64_t)id, (uint64_t)s_bs[b], q, r);
      if (q < (uint64_t)W) atomicAdd(&s_cnt[(int)q * bpw + b], 1);
    }
  }
  wave_lds_sync();
  for (int x = lane; x < W * cnt; x += kWaveSize) {
    const int p = x / cnt, k = x - p * cnt;
    new_lengths[(int64_t)p * n + i0 + k] = (T)s_cnt[p * bpw + k];
  }
}

template <typename T>
__global__ __launch_bounds__(kWalkThreads) void bucketize_scatter_wave_kernel(
    const T* __restrict__ offsets, const T* __restrict__ indices, const float* __restrict__ weights,
    const int64_t* __restrict__ block_sizes, int32_t B, int64_t n, int32_t W, int bpw, int keep_orig,
    const T* __restrict__ new_offsets, T* __restrict__ new_indices, float* __restrict__ new_weights,
    int64_t* __restrict__ unbucketize_permute) {
  extern __shared__ int64_t walk_smem[];
  const int lane = threadIdx.x & (kWaveSize - 1);
  const int wave = threadIdx.x / kWaveSize;
  const int per_wave = (bpw + 1) + bpw + W * bpw;
  int64_t* s_off = walk_smem + (size_t)wave * per_wave;
  int64_t* s_bs = s_off + bpw + 1;
  int64_t* s_cur = s_bs + bpw;  // next output position of (bucket p, bag b) at [p * bpw + b]
  const int64_t i0 = ((int64_t)blockIdx.x * kWalkWaves + wave) * bpw;
  if (i0 >= n) return;
  const int cnt = (int)(n - i0 < bpw ? n - i0 : bpw);
  for (int k = lane; k <= cnt; k += kWaveSize) s_off[k] = (int64_t)offsets[i0 + k];
  for (int k = lane; k < cnt; k += kWaveSize) s_bs[k] = block_sizes[(i0 + k) / B];
  for (int x = lane; x < W * cnt; x += kWaveSize) {
    const int p = x / cnt, k = x - p * cnt;
    s_cur[p * bpw + k] = (int64_t)new_offsets[(int64_t)p * n + i0 + k];
  }
  wave_lds_sync();
  const int64_t first = s_off[0], last = s_off[cnt];
  const uint64_t below_me = lane == 0 ? 0ull : (~0ull >> (kWaveSize - lane));
  for (int64_t j0 = first; j0 < last; j0 += kWaveSize) {
    const int64_t j = j0 + lane;
    const bool valid = j < last;
    const int64_t id = valid ? (int64_t)indices[j] : 0;
    const int b = find_bag(s_off, cnt, bpw >> 1, valid ? j : first);
    uint64_t q = 0, r = 0;
    div_mod((uint64_t)id, (uint64_t)s_bs[b], q, r);
    const bool in = valid && q < (uint64_t)W;
    const int p = in ? (int)q : -1;
    // The lanes of this chunk that hold ids of my bag: [lo_lane, hi_lane).
    const int64_t lo64 = s_off[b] - j0, hi64 = s_off[b + 1] - j0;
    const int lo_lane = lo64 < 0 ? 0 : (lo64 > kWaveSize - 1 ? kWaveSize - 1 : (int)lo64);
    const int hi_lane = hi64 > kWaveSize ? kWaveSize : (hi64 < 0 ? 0 : (int)hi64);
    const uint64_t my_bag = (hi_lane >= kWaveSize ? ~0ull : ((1ull << hi_lane) - 1)) & ~((1ull << lo_lane) - 1);
    // Rank of my id among the ids of the same bag and bucket in this chunk
    // (input order), one pass per bucket value present in the wave.
    int rank = 0, same_count = 0;
    uint64_t rem = __builtin_amdgcn_ballot_w64(in);
    while (rem != 0) {
      const int leader = __builtin_amdgcn_readfirstlane(__builtin_ctzll(rem));
      const int pl = __builtin_amdgcn_readlane(p, leader);
      const uint64_t m = __builtin_amdgcn_ballot_w64(in && p == pl);
      if (in && p == pl) {
        const uint64_t same = m & my_bag;
        rank = __builtin_popcountll(same & below_me);
        same_count = __builtin_popcountll(same);
      }
      rem &= ~m;
    }
    int64_t pos = -1;
    if (in) {
      pos = s_cur[p * bpw + b] + rank;
      new_indices[pos] = keep_orig ? (T)id : (T)r;
      if (weights) new_weights[pos] = weights[j];
    }
    if (valid && unbucketize_permute) unbucketize_permute[j] = pos;
    wave_lds_sync();  // every lane has read its cursor
    if (in && rank == same_count - 1) s_cur[p * bpw + b] = pos + 1;
    wave_lds_sync();
  }
}

// ---- row-wise N-bit quantization -------------------------------------------
// One wave per row.  Same operation order as fbgemm's
// FloatOrHalfToFusedNBitRowwiseQuantizedSBHalf: min/max, bias = fp16(min),
// scale = fp16((max - bias) / (2^bits - 1)), q = clamp(rint((x - bias) * (1/scale))).
// header_first: TBE row [scale][bias][payload]; otherwise fbgemm's trailer row.
template <int BITS>
__global__ __launch_bounds__(256) void quantize_rows_kernel(const float* in, int64_t rows,
                                                            int32_t dim, uint8_t* out,
                                                            int64_t row_bytes, int header_first) {
  const int lane = threadIdx.x & (kWaveSize - 1);
  const int64_t r = (int64_t)blockIdx.x * (blockDim.x / kWaveSize) + threadIdx.x / kWaveSize;
  if (r >= rows) return;
  const float* x = in + r * dim;
  float mn = x[0], mx = x[0];
  for (int c = lane; c < dim; c += kWaveSize) {
    const float v = x[c];
    mn = v < mn ? v : mn;
    mx = v > mx ? v : mx;
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float a = __shfl_xor(mn, off, 64), b = __shfl_xor(mx, off, 64);
    mn = a < mn ? a : mn;
    mx = b > mx ? b : mx;
  }
  constexpr int kQMax = (1 << BITS) - 1;
  constexpr int kEpb = 8 / BITS;
  const __half bias_h = __float2half_rn(mn);
  const float bias = __half2float(bias_h);
  const float range = mx - bias;
  float scale = range == 0.0f ? 1.0f : range / (float)kQMax;
  scale = __half2float(__float2half_rn(scale));
  if (scale == 0.0f) scale = 1.0f;
  float inv = 1.0f / scale;
  if (__builtin_isinf(inv)) {
    scale = 1.0f;
    inv = 1.0f;
  }
  const __half scale_h = __float2half_rn(scale);
  const int payload = dim / kEpb;
  uint8_t* o = out + r * row_bytes;
  uint8_t* pay = header_first ? o + 4 : o;
  uint8_t* hdr = header_first ? o : o + payload;
  for (int byte = lane; byte < payload; byte += kWaveSize) {
    uint32_t packed = 0;
#pragma unroll
    for (int e = 0; e < kEpb; ++e) {
      const float t = (x[byte * kEpb + e] - bias) * inv;
      float q = __builtin_rintf(t);
      q = q < 0.0f ? 0.0f : q;
      q = q > (float)kQMax ? (float)kQMax : q;
      packed |= (uint32_t)(int)q << (e * BITS);
    }
    pay[byte] = (uint8_t)packed;
  }
  if (lane == 0) {
    const uint16_t s = __half_as_ushort(scale_h), b = __half_as_ushort(bias_h);
    hdr[0] = (uint8_t)(s & 0xff);
    hdr[1] = (uint8_t)(s >> 8);
    hdr[2] = (uint8_t)(b & 0xff);
    hdr[3] = (uint8_t)(b >> 8);
  }
}

// The same quantizer for rows whose elements and output rows are 4-byte
// aligned (dim a multiple of 32 / BITS): a lane owns the 32 / BITS consecutive
// elements of one output dword, loads them 16 bytes at a time and stores the
// dword whole; `lpr` lanes (a power of two) share a row, 64 / lpr rows a wave.
// Per element the arithmetic is that of quantize_rows_kernel.
// DPL: output dwords a lane owns per step.  More than one means fewer lanes per
// row, fewer steps of the min / max exchange and fewer memory instructions per
// byte; 8-bit rows use two.
template <int BITS, int DPL = 1>
__global__ __launch_bounds__(256) void quantize_rows_vec_kernel(const float* __restrict__ in, int64_t rows,
                                                                int32_t dim, uint8_t* __restrict__ out,
                                                                int64_t row_bytes, int header_first,
                                                                int lpr) {
  constexpr int EPD = 32 / BITS;    // elements per output dword
  constexpr int EPL = DPL * EPD;    // elements per lane and step
  constexpr int kQMax = (1 << BITS) - 1;
  const int lane = threadIdx.x & (kWaveSize - 1);
  const int g = lane / lpr, c = lane - g * lpr;
  const int rows_per_wave = kWaveSize / lpr;
  const int64_t r_raw = ((int64_t)blockIdx.x * (blockDim.x / kWaveSize) + threadIdx.x / kWaveSize) * rows_per_wave + g;
  const bool active = r_raw < rows;
  const int64_t r = active ? r_raw : rows - 1;  // every lane takes part in the reductions
  const float* x = in + r * dim;
  const int chunks = dim / EPL;
  float mn = x[0], mx = mn;
  float keep[EPL];  // the lane's first chunk stays in registers for the second pass
#pragma unroll
  for (int e = 0; e < EPL; ++e) keep[e] = mn;
  for (int ch = c; ch < chunks; ch += lpr) {
    float v[EPL];
#pragma unroll
    for (int k = 0; k < EPL / 4; ++k) {
      const float4 q = *reinterpret_cast<const float4*>(x + ch * EPL + 4 * k);
      v[4 * k] = q.x; v[4 * k + 1] = q.y; v[4 * k + 2] = q.z; v[4 * k + 3] = q.w;
    }
#pragma unroll
    for (int e = 0; e < EPL; ++e) {
      mn = v[e] < mn ? v[e] : mn;
      mx = v[e] > mx ? v[e] : mx;
      if (ch == c) keep[e] = v[e];
    }
  }
  for (int off = lpr >> 1; off > 0; off >>= 1) {
    const float a = __shfl_xor(mn, off, 64), b = __shfl_xor(mx, off, 64);
    mn = a < mn ? a : mn;
    mx = b > mx ? b : mx;
  }
  const __half bias_h = __float2half_rn(mn);
  const float bias = __half2float(bias_h);
  const float range = mx - bias;
  float scale = range == 0.0f ? 1.0f : range / (float)kQMax;
  scale = __half2float(__float2half_rn(scale));
  if (scale == 0.0f) scale = 1.0f;
  float inv = 1.0f / scale;
  if (__builtin_isinf(inv)) {
    scale = 1.0f;
    inv = 1.0f;
  }
  const __half scale_h = __float2half_rn(scale);
  if (!active) return;
  uint8_t* o = out + r * row_bytes;
  uint32_t* pay = reinterpret_cast<uint32_t*>(header_first ? o + 4 : o);
  uint32_t* hdr = reinterpret_cast<uint32_t*>(header_first ? o : o + (int64_t)chunks * (4 * DPL));
  for (int ch = c; ch < chunks; ch += lpr) {
    float v[EPL];
    if (ch == c) {
#pragma unroll
      for (int e = 0; e < EPL; ++e) v[e] = keep[e];
    } else {
#pragma unroll
      for (int k = 0; k < EPL / 4; ++k) {
        const float4 q = *reinterpret_cast<const float4*>(x + ch * EPL + 4 * k);
        v[4 * k] = q.x; v[4 * k + 1] = q.y; v[4 * k + 2] = q.z; v[4 * k + 3] = q.w;
      }
    }
    uint32_t packed[DPL];
#pragma unroll
    for (int d = 0; d < DPL; ++d) packed[d] = 0;
#pragma unroll
    for (int e = 0; e < EPL; ++e) {
      const float t = (v[e] - bias) * inv;
      float q = __builtin_rintf(t);
      q = q < 0.0f ? 0.0f : q;
      q = q > (float)kQMax ? (float)kQMax : q;
      packed[e / EPD] |= (uint32_t)(int)q << ((e % EPD) * BITS);
    }
    // one store of DPL dwords (the payload is 4-byte aligned, not more)
    __builtin_memcpy(__builtin_assume_aligned(pay + ch * DPL, 4), packed, sizeof(packed));
  }
  if (c == 0) *hdr = (uint32_t)__half_as_ushort(scale_h) | ((uint32_t)__half_as_ushort(bias_h) << 16);
}

// ---- positions inside bags ---------------------------------------------------
// range[j] = j - start(bag of j), for j < range_size; `offsets` has n entries
// and the last bag ends at range_size.
template <typename T>
__global__ __launch_bounds__(kWalkThreads) void offsets_range_kernel(const T* __restrict__ offsets, int64_t n,
                                                                      int64_t range_size, int bpw,
                                                                      T* __restrict__ out) {
  extern __shared__ int64_t walk_smem[];
  const int lane = threadIdx.x & (kWaveSize - 1);
  const int wave = threadIdx.x / kWaveSize;
  int64_t* s_off = walk_smem + (size_t)wave * (bpw + 1);
  const int64_t i0 = ((int64_t)blockIdx.x * kWalkWaves + wave) * bpw;
  if (i0 >= n) return;
  const int cnt = (int)(n - i0 < bpw ? n - i0 : bpw);
  for (int k = lane; k <= cnt; k += kWaveSize) {
    int64_t v = i0 + k < n ? (int64_t)offsets[i0 + k] : range_size;
    v = v < 0 ? 0 : v;
    s_off[k] = v < range_size ? v : range_size;
  }
  wave_lds_sync();
  const int64_t first = s_off[0], last = s_off[cnt];
  for (int64_t j = first + lane; j < last; j += kWaveSize) {
    const int b = find_bag(s_off, cnt, bpw >> 1, j);
    out[j] = (T)(j - s_off[b]);
  }
}

// weight[j] = table[key_start[k] + (j - start of j's bag)] for an id of key k,
// 1.0 for keys without a table.  Positions at or beyond the key's table length
// take the last entry.
template <typename T>
__global__ __launch_bounds__(kWalkThreads) void position_weights_kernel(
    const T* __restrict__ offsets, int32_t B, int64_t n, const int32_t* __restrict__ key_start,
    const int32_t* __restrict__ key_len, const float* __restrict__ table, int bpw, float* __restrict__ out) {
  extern __shared__ int64_t walk_smem[];
  const int lane = threadIdx.x & (kWaveSize - 1);
  const int wave = threadIdx.x / kWaveSize;
  int64_t* s_off = walk_smem + (size_t)wave * (2 * bpw + 1);
  int32_t* s_start = reinterpret_cast<int32_t*>(s_off + bpw + 1);
  int32_t* s_len = s_start + bpw;
  const int64_t i0 = ((int64_t)blockIdx.x * kWalkWaves + wave) * bpw;
  if (i0 >= n) return;
  const int cnt = (int)(n - i0 < bpw ? n - i0 : bpw);
  for (int k = lane; k <= cnt; k += kWaveSize) s_off[k] = (int64_t)offsets[i0 + k];
  for (int k = lane; k < cnt; k += kWaveSize) {
    const int key = (int)((i0 + k) / B);
    s_start[k] = key_start[key];
    s_len[k] = key_len[key];
  }
  wave_lds_sync();
  const int64_t first = s_off[0], last = s_off[cnt];
  for (int64_t j = first + lane; j < last; j += kWaveSize) {
    const int b = find_bag(s_off, cnt, bpw >> 1, j);
    const int len = s_len[b];
    const int64_t pos = j - s_off[b];
    float w = 1.0f;
    if (len > 0) w = table[s_start[b] + (int)(pos < len ? pos : len - 1)];
    out[j] = w;
  }
}

// ---- id remapping through a sorted table --------------------------------------
// out[j] = mapping[i] when sorted_ids[i] == values[j] with i the first index in
// [0, size-1] whose entry is >= values[j] (searched over the first size-1
// entries; the last one is the table's delimiter), else miss_id.
template <typename T>
__global__ void mch_remap_kernel(const void* values, int64_t n, const int64_t* sorted_ids,
                                 const int64_t* mapping, int64_t size, int64_t miss_id, void* out) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t j = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; j < n; j += stride) {
    const int64_t v = ld<T>(values, j);
    int64_t lo = 0, hi = size - 1;  // lower bound in [0, size - 1)
    while (lo < hi) {
      const int64_t mid = lo + ((hi - lo) >> 1);
      if (sorted_ids[mid] < v) lo = mid + 1; else hi = mid;
    }
    st<T>(out, j, sorted_ids[lo] == v ? mapping[lo] : miss_id);
  }
}

// The same remap for every key of a KJT in one launch: blockIdx.y is the key,
// its ids are values[offsets[key*B] .. offsets[(key+1)*B]) and it has its own
// sorted table.  Tables travel in the launch arguments, kRemapKeys per launch.
constexpr int kRemapKeys = 64;
struct RemapTables {
  const int64_t* sorted_ids[kRemapKeys];
  const int64_t* mapping[kRemapKeys];
  int64_t size[kRemapKeys];
  int64_t miss_id[kRemapKeys];
  int32_t first_key;  // key of blockIdx.y == 0
};

template <typename T>
__global__ void mch_remap_keys_kernel(const void* values, int64_t n, const void* offsets, int32_t B,
                                      const RemapTables t, void* out) {
  const int k = blockIdx.y;
  const int64_t key = (int64_t)t.first_key + k;
  int64_t first = ld<T>(offsets, key * B), last = ld<T>(offsets, (key + 1) * B);
  first = first < 0 ? 0 : first;
  last = last > n ? n : last;
  const int64_t* sorted_ids = t.sorted_ids[k];
  const int64_t* mapping = t.mapping[k];
  const int64_t size = t.size[k], miss_id = t.miss_id[k];
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t j = first + (int64_t)blockIdx.x * blockDim.x + threadIdx.x; j < last; j += stride) {
    const int64_t v = ld<T>(values, j);
    int64_t lo = 0, hi = size - 1;
    while (lo < hi) {
      const int64_t mid = lo + ((hi - lo) >> 1);
      if (sorted_ids[mid] < v) lo = mid + 1; else hi = mid;
    }
    st<T>(out, j, sorted_ids[lo] == v ? mapping[lo] : miss_id);
  }
}

// Column blocks of row-major matrices copied into other matrices: block k is
// `width` elements of every row, from src[k] (row stride src_stride[k]) to
// dst[k] (row stride dst_stride[k]); both pointers already include the
// block's first column.  blockIdx.y is the block, blockIdx.x strides over its
// rows * width elements.  E = element size in bytes (2 or 4).
constexpr int kRegroupBlocks = 96;
struct RegroupBlocks {
  const void* src[kRegroupBlocks];
  void* dst[kRegroupBlocks];
  int64_t src_stride[kRegroupBlocks];
  int64_t dst_stride[kRegroupBlocks];
  int32_t width[kRegroupBlocks];
};

template <typename T>
__global__ __launch_bounds__(256) void regroup_kernel(const RegroupBlocks b, int64_t rows) {
  const int k = blockIdx.y;
  const T* __restrict__ src = reinterpret_cast<const T*>(b.src[k]);
  T* __restrict__ dst = reinterpret_cast<T*>(b.dst[k]);
  const int64_t ss = b.src_stride[k], ds = b.dst_stride[k];
  const int w = b.width[k];
  const int64_t n = rows * w;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    const int64_t r = i / w;
    const int c = (int)(i - r * w);
    dst[r * ds + c] = src[r * ss + c];
  }
}

// Plain streaming copy, 16 bytes per lane per step.
__global__ __launch_bounds__(256) void tra_copy_kernel(const uint4* __restrict__ src,
                                                        uint4* __restrict__ dst, int64_t n16) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride)
    dst[i] = src[i];
}

static int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return hip_fail(e, what);
  return TRA_OK;
}

static int quantize_impl(const float* in, int64_t rows, int32_t dim, int32_t bits, uint8_t* out,
                         int64_t row_bytes, int header_first, hipStream_t s) {
  if (bits != 8 && bits != 4 && bits != 2) {
    set_error("quantize: bits must be 8, 4 or 2 (got %d)", bits);
    return TRA_ERR_INVALID_ARGUMENT;
  }
  if (dim <= 0 || dim % (8 / bits) != 0 || rows < 0 || row_bytes < dim * bits / 8 + 4) {
    set_error("quantize: bad dim %d / row_bytes %lld for %d bits", dim, (long long)row_bytes, bits);
    return TRA_ERR_INVALID_ARGUMENT;
  }
  if (rows == 0) return TRA_OK;
  if (!in || !out) {
    set_error("quantize: null buffer");
    return TRA_ERR_INVALID_ARGUMENT;
  }
  int epl = 32 / bits;
  if (dim % epl == 0 && row_bytes % 4 == 0 && (uintptr_t)in % 16 == 0 && (uintptr_t)out % 4 == 0) {
    // 8-bit rows: two output dwords (8 elements, two 16-byte loads) per lane and step where the
    // dim allows.  Measured on 1 M rows x 128: 204 us with one dword per lane, 158 us with two,
    // 170 us with four; 4-bit rows are fastest with one (127 us against 133 us with two).
    const bool wide = bits == 8 && dim % 8 == 0;
    if (wide) epl = 8;
    const int chunks = dim / epl;
    int lpr = 1;
    while (lpr < chunks && lpr < kWaveSize) lpr <<= 1;
    const int64_t rows_per_block = 4 * (kWaveSize / lpr);
    const int64_t vblocks = (rows + rows_per_block - 1) / rows_per_block;
    if (vblocks > 0x7fffffff) {
      set_error("quantize: too many rows in one call");
      return TRA_ERR_TOO_LARGE;
    }
    dim3 vg((unsigned)vblocks), vb(256);
    if (wide)
      hipLaunchKernelGGL((quantize_rows_vec_kernel<8, 2>), vg, vb, 0, s, in, rows, dim, out, row_bytes, header_first, lpr);
    else if (bits == 8)
      hipLaunchKernelGGL(quantize_rows_vec_kernel<8>, vg, vb, 0, s, in, rows, dim, out, row_bytes, header_first, lpr);
    else if (bits == 4)
      hipLaunchKernelGGL(quantize_rows_vec_kernel<4>, vg, vb, 0, s, in, rows, dim, out, row_bytes, header_first, lpr);
    else
      hipLaunchKernelGGL(quantize_rows_vec_kernel<2>, vg, vb, 0, s, in, rows, dim, out, row_bytes, header_first, lpr);
    return check_launch("quantize_rows");
  }
  const int64_t blocks = (rows + 3) / 4;
  if (blocks > 0x7fffffff) {
    set_error("quantize: too many rows in one call");
    return TRA_ERR_TOO_LARGE;
  }
  dim3 g((unsigned)blocks), b(256);
  if (bits == 8)
    hipLaunchKernelGGL(quantize_rows_kernel<8>, g, b, 0, s, in, rows, dim, out, row_bytes, header_first);
  else if (bits == 4)
    hipLaunchKernelGGL(quantize_rows_kernel<4>, g, b, 0, s, in, rows, dim, out, row_bytes, header_first);
  else
    hipLaunchKernelGGL(quantize_rows_kernel<2>, g, b, 0, s, in, rows, dim, out, row_bytes, header_first);
  return check_launch("quantize_rows");
}

}  // namespace tra

using namespace tra;

extern "C" {

// The one-launch scan takes up to 131072 lengths: every block sums what lies in front of its tile
// itself, so the last block reads the whole input through one compute unit (512 KB of int32 in
// about 4 us).  At 262144 int32 lengths it measured 18 us against 16 us for the two-kernel scan.
constexpr int64_t kSmallScanMax = (int64_t)kSmallMaxTiles * kSmallThreads * 2;
int64_t tra_cumsum_workspace_bytes(int64_t n) {
  if (n <= kSmallScanMax) return 0;
  const int64_t tiles = (n + kScanTile - 1) / kScanTile;
  return tiles > 1 ? tiles * (int64_t)sizeof(int64_t) : 0;
}

int tra_cumsum(const void* lengths, int64_t n, int32_t is_i64, void* offsets, void* workspace,
               void* stream) {
  if (n < 0 || !offsets || (n > 0 && !lengths)) {
    set_error("tra_cumsum: bad argument");
    return TRA_ERR_INVALID_ARGUMENT;
  }
  if (n > 0x7fffffffLL) {
    set_error("tra_cumsum: n too large");
    return TRA_ERR_TOO_LARGE;
  }
  hipStream_t s = (hipStream_t)stream;
  if (n <= kSmallScanMax) {
    const int per_tile = kSmallThreads * (is_i64 ? 2 : 4);
    const unsigned g = (unsigned)std::max<int64_t>(1, (n + per_tile - 1) / per_tile);
    const bool vec = (uintptr_t)lengths % 16 == 0;
    if (is_i64) {
      if (vec)
        hipLaunchKernelGGL((scan_small_kernel<int64_t, true>), dim3(g), dim3(kSmallThreads), 0, s,
                           (const int64_t*)lengths, n, (int64_t*)offsets);
      else
        hipLaunchKernelGGL((scan_small_kernel<int64_t, false>), dim3(g), dim3(kSmallThreads), 0, s,
                           (const int64_t*)lengths, n, (int64_t*)offsets);
    } else {
      if (vec)
        hipLaunchKernelGGL((scan_small_kernel<int32_t, true>), dim3(g), dim3(kSmallThreads), 0, s,
                           (const int32_t*)lengths, n, (int32_t*)offsets);
      else
        hipLaunchKernelGGL((scan_small_kernel<int32_t, false>), dim3(g), dim3(kSmallThreads), 0, s,
                           (const int32_t*)lengths, n, (int32_t*)offsets);
    }
    return check_launch("tra_cumsum");
  }
  const int64_t tiles = n == 0 ? 1 : (n + kScanTile - 1) / kScanTile;
  int64_t* sums = nullptr;
  if (tiles > 1) {
    if (!workspace) {
      set_error("tra_cumsum: workspace of %lld bytes required",
                (long long)tra_cumsum_workspace_bytes(n));
      return TRA_ERR_INVALID_ARGUMENT;
    }
    sums = (int64_t*)workspace;
    if (is_i64)
      hipLaunchKernelGGL(tile_sums_kernel<int64_t>, dim3((unsigned)tiles), dim3(kScanThreads), 0, s,
                         lengths, n, sums);
    else
      hipLaunchKernelGGL(tile_sums_kernel<int32_t>, dim3((unsigned)tiles), dim3(kScanThreads), 0, s,
                         lengths, n, sums);
  }
  if (is_i64)
    hipLaunchKernelGGL(scan_tiles_kernel<int64_t>, dim3((unsigned)tiles), dim3(kScanThreads), 0, s,
                       lengths, n, sums, offsets);
  else
    hipLaunchKernelGGL(scan_tiles_kernel<int32_t>, dim3((unsigned)tiles), dim3(kScanThreads), 0, s,
                       lengths, n, sums, offsets);
  return check_launch("tra_cumsum");
}

int tra_length_per_key(const void* lengths, int32_t num_features, int32_t batch_size,
                       int32_t is_i64, int64_t* out, void* stream) {
  if (num_features < 0 || batch_size < 0 || (num_features > 0 && (!out || (!lengths && batch_size)))) {
    set_error("tra_length_per_key: bad argument");
    return TRA_ERR_INVALID_ARGUMENT;
  }
  if (num_features == 0) return TRA_OK;
  hipStream_t s = (hipStream_t)stream;
  if (is_i64)
    hipLaunchKernelGGL(length_per_key_kernel<int64_t>, dim3(num_features), dim3(kScanThreads), 0, s,
                       lengths, batch_size, out);
  else
    hipLaunchKernelGGL(length_per_key_kernel<int32_t>, dim3(num_features), dim3(kScanThreads), 0, s,
                       lengths, batch_size, out);
  return check_launch("tra_length_per_key");
}

int tra_permute_2d_lengths(const int32_t* permute, int32_t num_out_features, int32_t num_features,
                           int32_t batch_size, const void* lengths, int32_t is_i64,
                           void* out_lengths, void* stream) {
  (void)num_features;
  const int64_t total = (int64_t)num_out_features * batch_size;
  if (num_out_features < 0 || batch_size < 0) {
    set_error("tra_permute_2d_lengths: bad argument");
    return TRA_ERR_INVALID_ARGUMENT;
  }
  if (total == 0) return TRA_OK;
  if (!permute || !lengths || !out_lengths) {
    set_error("tra_permute_2d_lengths: null buffer");
    return TRA_ERR_INVALID_ARGUMENT;
  }
  hipStream_t s = (hipStream_t)stream;
  dim3 g((unsigned)((total + 255) / 256)), b(256);
  if (is_i64)
    hipLaunchKernelGGL(permute_lengths_kernel<int64_t>, g, b, 0, s, permute, total, batch_size,
                       lengths, out_lengths);
  else
    hipLaunchKernelGGL(permute_lengths_kernel<int32_t>, g, b, 0, s, permute, total, batch_size,
                       lengths, out_lengths);
  return check_launch("tra_permute_2d_lengths");
}

int tra_permute_2d_data(const int32_t* permute, int32_t num_out_features, int32_t batch_size,
                        const void* in_offsets, const void* out_offsets, int32_t is_i64,
                        const void* values, int32_t value_bytes, const float* weights,
                        void* out_values, float* out_weights, void* stream) {
  if (num_out_features < 0 || batch_size < 0 || (value_bytes != 4 && value_bytes != 8)) {
    set_error("tra_permute_2d_data: bad argument (value_bytes must be 4 or 8)");
    return TRA_ERR_INVALID_ARGUMENT;
  }
  if (num_out_features == 0 || batch_size == 0) return TRA_OK;
  if (!permute || !in_offsets || !out_offsets || (weights && !out_weights)) {
    set_error("tra_permute_2d_data: null buffer");
    return TRA_ERR_INVALID_ARGUMENT;
  }
  hipStream_t s = (hipStream_t)stream;
  dim3 g(64, (unsigned)num_out_features), b(256);
#define GO(OFF, VAL)                                                                          \
  hipLaunchKernelGGL((permute_data_kernel<OFF, VAL>), g, b, 0, s, permute, batch_size,        \
                     in_offsets, out_offsets, (const VAL*)values, weights, (VAL*)out_values,  \
                     out_weights)
  if (is_i64) {
    if (value_bytes == 8) GO(int64_t, int64_t); else GO(int64_t, int32_t);
  } else {
    if (value_bytes == 8) GO(int32_t, int64_t); else GO(int32_t, int32_t);
  }
#undef GO
  return check_launch("tra_permute_2d_data");
}

int tra_bucketize_lengths(const void* offsets, const void* indices, int32_t is_i64,
                          const int64_t* block_sizes, int32_t num_features, int32_t batch_size,
                          int32_t num_buckets, void* new_lengths, void* stream) {
  const int64_t n = (int64_t)num_features * batch_size;
  if (num_features < 0 || batch_size < 0 || num_buckets <= 0) {
    set_error("tra_bucketize_lengths: bad argument");
    return TRA_ERR_INVALID_ARGUMENT;
  }
  if (n == 0) return TRA_OK;
  if (!offsets || !block_sizes || !new_lengths) {
    set_error("tra_bucketize_lengths: null buffer");
    return TRA_ERR_INVALID_ARGUMENT;
  }
  hipStream_t s = (hipStream_t)stream;
  if (num_buckets <= kWalkMaxBuckets) {
    const int bpw = bags_per_wave(n, std::max(1, kWalkMaxBuckets / num_buckets));
    const int64_t waves = (n + bpw - 1) / bpw;
    dim3 g((unsigned)((waves + kWalkWaves - 1) / kWalkWaves)), b(kWalkThreads);
    const size_t lds = (size_t)kWalkWaves * ((bpw + 1) + bpw + ((size_t)num_buckets * bpw + 1) / 2) * sizeof(int64_t);
    if (is_i64)
      hipLaunchKernelGGL(bucketize_lengths_wave_kernel<int64_t>, g, b, lds, s, (const int64_t*)offsets,
                         (const int64_t*)indices, block_sizes, batch_size, n, num_buckets, bpw,
                         (int64_t*)new_lengths);
    else
      hipLaunchKernelGGL(bucketize_lengths_wave_kernel<int32_t>, g, b, lds, s, (const int32_t*)offsets,
                         (const int32_t*)indices, block_sizes, batch_size, n, num_buckets, bpw,
                         (int32_t*)new_lengths);
    return check_launch("tra_bucketize_lengths");
  }
  dim3 g((unsigned)((n + 127) / 128)), b(128);
  if (is_i64)
    hipLaunchKernelGGL(bucketize_lengths_kernel<int64_t>, g, b, 0, s, offsets, indices, block_sizes,
                       batch_size, n, num_buckets, new_lengths);
  else
    hipLaunchKernelGGL(bucketize_lengths_kernel<int32_t>, g, b, 0, s, offsets, indices, block_sizes,
                       batch_size, n, num_buckets, new_lengths);
  return check_launch("tra_bucketize_lengths");
}

int64_t tra_bucketize_workspace_bytes(int32_t num_features, int32_t batch_size, int32_t num_buckets) {
  if (num_features <= 0 || batch_size <= 0 || num_buckets <= kWalkMaxBuckets) return 0;
  return (int64_t)num_features * batch_size * num_buckets * (int64_t)sizeof(int64_t);
}

int tra_bucketize_scatter(const void* offsets, const void* indices, int32_t is_i64,
                          const float* weights, const int64_t* block_sizes, int32_t num_features,
                          int32_t batch_size, int32_t num_buckets, int32_t keep_orig_idx,
                          const void* new_offsets, int64_t* cursor_workspace, void* new_indices,
                          float* new_weights, int64_t* unbucketize_permute, void* stream) {
  const int64_t n = (int64_t)num_features * batch_size;
  if (num_features < 0 || batch_size < 0 || num_buckets <= 0) {
    set_error("tra_bucketize_scatter: bad argument");
    return TRA_ERR_INVALID_ARGUMENT;
  }
  if (n == 0) return TRA_OK;
  if (!offsets || !block_sizes || !new_offsets || (weights && !new_weights)) {
    set_error("tra_bucketize_scatter: null buffer");
    return TRA_ERR_INVALID_ARGUMENT;
  }
  hipStream_t s = (hipStream_t)stream;
  if (num_buckets <= kWalkMaxBuckets) {
    const int bpw = bags_per_wave(n, std::max(1, kWalkMaxBuckets / num_buckets));
    const int64_t waves = (n + bpw - 1) / bpw;
    dim3 g((unsigned)((waves + kWalkWaves - 1) / kWalkWaves)), b(kWalkThreads);
    const size_t lds = (size_t)kWalkWaves * ((bpw + 1) + bpw + (size_t)num_buckets * bpw) * sizeof(int64_t);
    if (is_i64)
      hipLaunchKernelGGL(bucketize_scatter_wave_kernel<int64_t>, g, b, lds, s, (const int64_t*)offsets,
                         (const int64_t*)indices, weights, block_sizes, batch_size, n, num_buckets, bpw,
                         keep_orig_idx, (const int64_t*)new_offsets, (int64_t*)new_indices, new_weights,
                         unbucketize_permute);
    else
      hipLaunchKernelGGL(bucketize_scatter_wave_kernel<int32_t>, g, b, lds, s, (const int32_t*)offsets,
                         (const int32_t*)indices, weights, block_sizes, batch_size, n, num_buckets, bpw,
                         keep_orig_idx, (const int32_t*)new_offsets, (int32_t*)new_indices, new_weights,
                         unbucketize_permute);
    return check_launch("tra_bucketize_scatter");
  }
  if (!cursor_workspace) {
    set_error("tra_bucketize_scatter: more than %d buckets need the cursor workspace", kWalkMaxBuckets);
    return TRA_ERR_INVALID_ARGUMENT;
  }
  dim3 g((unsigned)((n + 127) / 128)), b(128);
  if (is_i64)
    hipLaunchKernelGGL(bucketize_scatter_kernel<int64_t>, g, b, 0, s, offsets, indices, weights,
                       block_sizes, batch_size, n, num_buckets, keep_orig_idx, new_offsets,
                       cursor_workspace, new_indices, new_weights, unbucketize_permute);
  else
    hipLaunchKernelGGL(bucketize_scatter_kernel<int32_t>, g, b, 0, s, offsets, indices, weights,
                       block_sizes, batch_size, n, num_buckets, keep_orig_idx, new_offsets,
                       cursor_workspace, new_indices, new_weights, unbucketize_permute);
  return check_launch("tra_bucketize_scatter");
}

int tra_quantize_rows(const float* in, int64_t rows, int32_t dim, int32_t bits, uint8_t* out,
                      int32_t row_bytes, void* stream) {
  return quantize_impl(in, rows, dim, bits, out, row_bytes, 1, (hipStream_t)stream);
}

int tra_quantize_rows_sbhalf(const float* in, int64_t rows, int32_t dim, int32_t bits,
                             uint8_t* out, void* stream) {
  const int64_t rb = bits > 0 && bits <= 8 ? (int64_t)dim * bits / 8 + 4 : 0;
  return quantize_impl(in, rows, dim, bits, out, rb, 0, (hipStream_t)stream);
}

int tra_offsets_range(const void* offsets, int64_t num_bags, int32_t is_i64, int64_t range_size,
                      void* out, void* stream) {
  if (num_bags < 0 || range_size < 0) {
    set_error("tra_offsets_range: negative size");
    return TRA_ERR_INVALID_ARGUMENT;
  }
  if (num_bags == 0 || range_size == 0) return TRA_OK;
  if (!offsets || !out) {
    set_error("tra_offsets_range: null buffer");
    return TRA_ERR_INVALID_ARGUMENT;
  }
  const int bpw = bags_per_wave(num_bags, 64);
  const int64_t waves = (num_bags + bpw - 1) / bpw;
  dim3 g((unsigned)((waves + kWalkWaves - 1) / kWalkWaves)), b(kWalkThreads);
  const size_t lds = (size_t)kWalkWaves * (bpw + 1) * sizeof(int64_t);
  if (is_i64)
    hipLaunchKernelGGL(offsets_range_kernel<int64_t>, g, b, lds, (hipStream_t)stream, (const int64_t*)offsets,
                       num_bags, range_size, bpw, (int64_t*)out);
  else
    hipLaunchKernelGGL(offsets_range_kernel<int32_t>, g, b, lds, (hipStream_t)stream, (const int32_t*)offsets,
                       num_bags, range_size, bpw, (int32_t*)out);
  return check_launch("tra_offsets_range");
}

int tra_position_weights(const void* offsets, int32_t is_i64, int32_t num_keys, int32_t batch_size,
                         const int32_t* key_start, const int32_t* key_len, const float* table,
                         float* out, void* stream) {
  if (num_keys < 0 || batch_size < 0) {
    set_error("tra_position_weights: negative size");
    return TRA_ERR_INVALID_ARGUMENT;
  }
  const int64_t n = (int64_t)num_keys * batch_size;
  if (n == 0) return TRA_OK;
  if (!offsets || !key_start || !key_len || !out) {
    set_error("tra_position_weights: null buffer");
    return TRA_ERR_INVALID_ARGUMENT;
  }
  const int bpw = bags_per_wave(n, 64);
  const int64_t waves = (n + bpw - 1) / bpw;
  dim3 g((unsigned)((waves + kWalkWaves - 1) / kWalkWaves)), b(kWalkThreads);
  const size_t lds = (size_t)kWalkWaves * (2 * bpw + 1) * sizeof(int64_t);
  if (is_i64)
    hipLaunchKernelGGL(position_weights_kernel<int64_t>, g, b, lds, (hipStream_t)stream, (const int64_t*)offsets,
                       batch_size, n, key_start, key_len, table, bpw, out);
  else
    hipLaunchKernelGGL(position_weights_kernel<int32_t>, g, b, lds, (hipStream_t)stream, (const int32_t*)offsets,
                       batch_size, n, key_start, key_len, table, bpw, out);
  return check_launch("tra_position_weights");
}

int tra_mch_remap(const void* values, int64_t n, int32_t is_i64, const int64_t* sorted_ids,
                  const int64_t* mapping, int64_t table_size, int64_t miss_id, void* out,
                  void* stream) {
  if (n < 0 || table_size <= 0) {
    set_error("tra_mch_remap: bad size");
    return TRA_ERR_INVALID_ARGUMENT;
  }
  if (n == 0) return TRA_OK;
  if (!values || !sorted_ids || !mapping || !out) {
    set_error("tra_mch_remap: null buffer");
    return TRA_ERR_INVALID_ARGUMENT;
  }
  const unsigned grid = (unsigned)std::min<int64_t>((n + 255) / 256, 256 * 16);
  if (is_i64)
    hipLaunchKernelGGL(mch_remap_kernel<int64_t>, dim3(grid), dim3(256), 0, (hipStream_t)stream, values,
                       n, sorted_ids, mapping, table_size, miss_id, out);
  else
    hipLaunchKernelGGL(mch_remap_kernel<int32_t>, dim3(grid), dim3(256), 0, (hipStream_t)stream, values,
                       n, sorted_ids, mapping, table_size, miss_id, out);
  return check_launch("tra_mch_remap");
}

int tra_mch_remap_keys(const void* values, int64_t n, const void* offsets, int32_t is_i64,
                       int32_t num_keys, int32_t batch_size, const int64_t* const* sorted_ids,
                       const int64_t* const* mapping, const int64_t* table_size,
                       const int64_t* miss_id, void* out, void* stream) {
  if (n < 0 || num_keys < 0 || batch_size < 0) {
    set_error("tra_mch_remap_keys: negative size");
    return TRA_ERR_INVALID_ARGUMENT;
  }
  if (n == 0 || num_keys == 0) return TRA_OK;
  if (!values || !offsets || !out || !sorted_ids || !mapping || !table_size || !miss_id) {
    set_error("tra_mch_remap_keys: null argument");
    return TRA_ERR_INVALID_ARGUMENT;
  }
  for (int k = 0; k < num_keys; ++k)
    if (!sorted_ids[k] || !mapping[k] || table_size[k] < 1) {
      set_error("tra_mch_remap_keys: key %d has no table", k);
      return TRA_ERR_INVALID_ARGUMENT;
    }
  // blocks per key: enough for the average key, at most 1024
  const int64_t per_key = n / num_keys + 1;
  const unsigned gx = (unsigned)std::max<int64_t>(1, std::min<int64_t>((per_key + 255) / 256, 1024));
  for (int k0 = 0; k0 < num_keys; k0 += kRemapKeys) {
    const int nk = std::min(kRemapKeys, num_keys - k0);
    RemapTables t;
    std::memset(&t, 0, sizeof(t));
    for (int k = 0; k < nk; ++k) {
      t.sorted_ids[k] = sorted_ids[k0 + k];
      t.mapping[k] = mapping[k0 + k];
      t.size[k] = table_size[k0 + k];
      t.miss_id[k] = miss_id[k0 + k];
    }
    t.first_key = k0;
    if (is_i64)
      hipLaunchKernelGGL(mch_remap_keys_kernel<int64_t>, dim3(gx, nk), dim3(256), 0, (hipStream_t)stream,
                         values, n, offsets, batch_size, t, out);
    else
      hipLaunchKernelGGL(mch_remap_keys_kernel<int32_t>, dim3(gx, nk), dim3(256), 0, (hipStream_t)stream,
                         values, n, offsets, batch_size, t, out);
    const int rc = check_launch("tra_mch_remap_keys");
    if (rc != TRA_OK) return rc;
  }
  return TRA_OK;
}

int tra_regroup_columns(const void* const* src, const int64_t* src_stride, void* const* dst,
                        const int64_t* dst_stride, const int32_t* width, int32_t num_blocks,
                        int64_t rows, int32_t elem_bytes, void* stream) {
  if (num_blocks < 0 || rows < 0) {
    set_error("tra_regroup_columns: negative size");
    return TRA_ERR_INVALID_ARGUMENT;
  }
  if (elem_bytes != 2 && elem_bytes != 4) {
    set_error("tra_regroup_columns: element size %d (2 or 4 bytes are supported)", elem_bytes);
    return TRA_ERR_UNSUPPORTED;
  }
  if (num_blocks == 0 || rows == 0) return TRA_OK;
  if (!src || !dst || !src_stride || !dst_stride || !width) {
    set_error("tra_regroup_columns: null argument");
    return TRA_ERR_INVALID_ARGUMENT;
  }
  int64_t widest = 0;
  for (int k = 0; k < num_blocks; ++k) {
    if (!src[k] || !dst[k] || width[k] < 0 || src_stride[k] < width[k] || dst_stride[k] < width[k]) {
      set_error("tra_regroup_columns: block %d is null or wider than its row stride", k);
      return TRA_ERR_INVALID_ARGUMENT;
    }
    widest = std::max<int64_t>(widest, width[k]);
  }
  if (widest == 0) return TRA_OK;
  const unsigned gx = (unsigned)std::max<int64_t>(1, std::min<int64_t>((rows * widest + 255) / 256, 2048));
  for (int k0 = 0; k0 < num_blocks; k0 += kRegroupBlocks) {
    const int nk = std::min(kRegroupBlocks, num_blocks - k0);
    RegroupBlocks b;
    std::memset(&b, 0, sizeof(b));
    for (int k = 0; k < nk; ++k) {
      b.src[k] = src[k0 + k];
      b.dst[k] = dst[k0 + k];
      b.src_stride[k] = src_stride[k0 + k];
      b.dst_stride[k] = dst_stride[k0 + k];
      b.width[k] = width[k0 + k];
    }
    if (elem_bytes == 2)
      hipLaunchKernelGGL(regroup_kernel<uint16_t>, dim3(gx, nk), dim3(256), 0, (hipStream_t)stream, b, rows);
    else
      hipLaunchKernelGGL(regroup_kernel<uint32_t>, dim3(gx, nk), dim3(256), 0, (hipStream_t)stream, b, rows);
    const int rc = check_launch("tra_regroup_columns");
    if (rc != TRA_OK) return rc;
  }
  return TRA_OK;
}

int tra_copy_bytes(const void* src, void* dst, int64_t bytes, void* stream) {
  if (bytes < 0 || bytes % 16 != 0 || (uintptr_t)src % 16 != 0 || (uintptr_t)dst % 16 != 0) {
    set_error("tra_copy_bytes: size and pointers must be multiples of 16 bytes");
    return TRA_ERR_INVALID_ARGUMENT;
  }
  if (bytes == 0) return TRA_OK;
  if (!src || !dst) {
    set_error("tra_copy_bytes: null buffer");
    return TRA_ERR_INVALID_ARGUMENT;
  }
  const int64_t n16 = bytes / 16;
  const unsigned grid = (unsigned)std::min<int64_t>((n16 + 255) / 256, 256 * 32);
  hipLaunchKernelGGL(tra_copy_kernel, dim3(grid), dim3(256), 0, (hipStream_t)stream,
                     (const uint4*)src, (uint4*)dst, n16);
  return check_launch("tra_copy_bytes");
}

}  // extern "C"
