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

#include <type_traits>
#include <vector>

#include "tra_common.h"

namespace tra {

constexpr int kWavesPerBlock = 4;
constexpr int kBlockThreads = kWavesPerBlock * kWaveSize;
constexpr int kMaxSub = 8;
constexpr int kMaxPos = 128;

// Features of one launch that share LPR (i.e. share dim).
struct SubClass {
  int32_t first;           // index of the first feature in the class feature list
  int32_t count;           // features in this sub-class
  int32_t lpr;             // lanes per row
  int32_t tiles_per_feat;  // blocks per feature
  int32_t tile_start;      // first block of this sub-class in the grid
  int32_t window;          // window kernel: bags per block
  int32_t key0;            // key position of the first feature when the sub-class's features sit
                           // at consecutive key positions (feature fi at key0 + fi), else -1
};

struct LookupArgs {
  const uint8_t* weights;
  const FeatureDesc* descs;  // all features of the plan (device)
  const int32_t* feats;      // feature ids of this launch (device)
  const FeatureDesc* cdescs; // the same features' descriptors in launch order: cdescs[i] == descs[feats[i]]
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
  int32_t bad_to_row0;  // 1: an id outside its table (other than -1) reads row 0 instead of being skipped
  int32_t xcd_blocks;   // balanced pooled kernel: blocks per XCD (0: no XCD remap)
  int32_t xcd_count;    // balanced pooled kernel: XCDs the grid is dealt to
  int16_t feat_pos[kMaxPos];  // balanced pooled kernel: key position of the class's first features
  // Position weighting (posw != nullptr): the weight of the id at position k of
  // a bag of class feature ci is posw[pw_off[ci] + min(k, pw_len[ci] - 1)], or
  // 1 when pw_len[ci] is 0.  Takes the place of psw; classes of at most
  // kMaxPos features.
  const float* posw;
  int32_t pw_off[kMaxPos];
  int32_t pw_len[kMaxPos];
#ifdef TRA_INSTRUMENT
  unsigned long long* ts;  // [waves][8] wall-clock stamps
#endif
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
// Kernel-internal type codes for int-N rows too wide for one wave of lanes
// (more than 64 chunks of at most 8 bytes): such a row is cut into column
// slices, and only its first slice has the row header in front of it, so
// these variants load the header on its own (kHeaderWithChunk false).
constexpr int kSplitHeader = 16;
template <>
struct Traits<TRA_INT8 + kSplitHeader> : Traits<TRA_INT8> {};
template <>
struct Traits<TRA_INT4 + kSplitHeader> : Traits<TRA_INT4> {};
template <>
struct Traits<TRA_INT2 + kSplitHeader> : Traits<TRA_INT2> {};
// The weight type proper of a kernel type code.
constexpr int base_type(int dtype) { return dtype >= kSplitHeader ? dtype - kSplitHeader : dtype; }
// Does a lane load the dword in front of its chunk together with the chunk
// (for a row's first lane: the header)?  Rows with a header, 8- or 4-byte
// chunks, whole row in one slice.
template <int DTYPE, int CB>
constexpr bool header_with_chunk() { return Traits<DTYPE>::kHeader != 0 && CB <= 8 && DTYPE < kSplitHeader; }

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

typedef float float2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float half_bits_to_float(uint32_t h) {
  return (float)__builtin_bit_cast(_Float16, (uint16_t)h);
}

// acc = fmaf(s, q, acc + b): one rounded add, then one fused multiply-add.
__device__ __forceinline__ void fma_step(float& acc, float s, float q, float b) {
  float t = acc + b;
  acc = __builtin_fmaf(s, q, t);
}

// Sub-byte fields to floats on the matrix core.  Eight bytes 0x00 .. 0x0f per
// lane (two payload dwords' worth of masked fields) become eight floats with
// two v_mfma_f32_16x16x32_bf8_fp8: the lane's bytes are one column slice of the
// B operand (FP8 E4M3: a byte 0x0q is exactly q * 2^-9, subnormals and the
// first binade), the A operand holds 2^9 (BF8 0x60) where row m selects byte
// (m & 3) [+ 4] of lane group m >> 2, and C is zero; so output register r of a
// lane is 2^9 * (its own byte r [+ 4]) plus exact zeros: the integer q, with no
// rounding anywhere.  This takes the conversions (one v_cvt_pk_f32_fp8 per two
// elements otherwise) off the vector ALU, which the pooling loop saturates;
// the matrix core runs beside it.
typedef float float4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ long mfma_byte_selector(int lane, int half) {
  const int m = lane & 15, gp = lane >> 4;
  unsigned long long v = 0;
  if (gp == (m >> 2)) v = 0x60ull << (8 * ((m & 3) + 4 * half));
  return (long)v;
}

// Accumulate the elements of one payload dword.  `acc` points at the
// accumulators of this dword's elements.  int4 / int2 fields are converted on
// the matrix core (mfma_byte_selector above; sel0 / sel1 are the lane's two
// selector operands), int8 bytes by v_cvt_f32_ubyteN.
template <int DTYPE_CODE, bool WEIGHTED, bool MATRIX>
__device__ __forceinline__ void accumulate_dword(float* acc, uint32_t x, float s,
                                                 float b, long sel0, long sel1) {
  constexpr int DTYPE = base_type(DTYPE_CODE);
  if constexpr (DTYPE == TRA_INT4 && MATRIX) {
    // Low nibbles in the low dword, high nibbles in the high dword of the
    // matrix instruction's 8-byte operand; element 2k is byte k's low nibble.
    const uint32_t lo = x & 0x0f0f0f0fu;
    const uint32_t hi = (x >> 4) & 0x0f0f0f0fu;
    const long data = (long)(((unsigned long long)hi << 32) | lo);
    const float4_t z = {0.0f, 0.0f, 0.0f, 0.0f};
    const float4_t l = __builtin_amdgcn_mfma_f32_16x16x32_bf8_fp8(sel0, data, z, 0, 0, 0);
    const float4_t h = __builtin_amdgcn_mfma_f32_16x16x32_bf8_fp8(sel1, data, z, 0, 0, 0);
    fma_step(acc[0], s, l[0], b);
    fma_step(acc[1], s, h[0], b);
    fma_step(acc[2], s, l[1], b);
    fma_step(acc[3], s, h[1], b);
    fma_step(acc[4], s, l[2], b);
    fma_step(acc[5], s, h[2], b);
    fma_step(acc[6], s, l[3], b);
    fma_step(acc[7], s, h[3], b);
  } else if constexpr (DTYPE == TRA_INT8) {
    fma_step(acc[0], s, byte_to_float<0>(x), b);
    fma_step(acc[1], s, byte_to_float<1>(x), b);
    fma_step(acc[2], s, byte_to_float<2>(x), b);
    fma_step(acc[3], s, byte_to_float<3>(x), b);
  } else if constexpr (DTYPE == TRA_INT4 && !WEIGHTED) {
    // (16-byte lane chunks: 32 accumulators per lane leave no registers for the
    // matrix instruction's operands and results, so the vector ALU converts.)
    // A byte 0x0q read as an FP8 (E4M3) value is exactly q * 2^-9 for q = 0..15
    // (subnormals, then the first binade), and one instruction converts two
    // bytes.  The scale is multiplied by 2^9 instead (exact: s is at most
    // 65504 here), so every product is the same real number as s * q.
    const uint32_t lo = x & 0x0f0f0f0fu;
    const uint32_t hi = (x >> 4) & 0x0f0f0f0fu;
    const float s9 = s * 512.0f;
    const float2_t l01 = __builtin_amdgcn_cvt_pk_f32_fp8((int)lo, false);
    const float2_t l23 = __builtin_amdgcn_cvt_pk_f32_fp8((int)lo, true);
    const float2_t h01 = __builtin_amdgcn_cvt_pk_f32_fp8((int)hi, false);
    const float2_t h23 = __builtin_amdgcn_cvt_pk_f32_fp8((int)hi, true);
    fma_step(acc[0], s9, l01.x, b);
    fma_step(acc[1], s9, h01.x, b);
    fma_step(acc[2], s9, l01.y, b);
    fma_step(acc[3], s9, h01.y, b);
    fma_step(acc[4], s9, l23.x, b);
    fma_step(acc[5], s9, h23.x, b);
    fma_step(acc[6], s9, l23.y, b);
    fma_step(acc[7], s9, h23.y, b);
  } else if constexpr (DTYPE == TRA_INT4) {
    // With per-sample weights the scale w*scale may be subnormal, where a
    // multiplication by 2^9 is inexact, so the fields are shifted down instead.
    const uint32_t lo = x & 0x0f0f0f0fu;
    const uint32_t hi = (x >> 4) & 0x0f0f0f0fu;
    fma_step(acc[0], s, byte_to_float<0>(lo), b);
    fma_step(acc[1], s, byte_to_float<0>(hi), b);
    fma_step(acc[2], s, byte_to_float<1>(lo), b);
    fma_step(acc[3], s, byte_to_float<1>(hi), b);
    fma_step(acc[4], s, byte_to_float<2>(lo), b);
    fma_step(acc[5], s, byte_to_float<2>(hi), b);
    fma_step(acc[6], s, byte_to_float<3>(lo), b);
    fma_step(acc[7], s, byte_to_float<3>(hi), b);
  } else if constexpr (DTYPE == TRA_INT2 && MATRIX) {
    // The four 2-bit fields of every byte, two field positions per pair of
    // matrix instructions; element 4 * k + e is field e of byte k.
#pragma unroll
    for (int e = 0; e < 4; e += 2) {
      const uint32_t m0 = (x >> (2 * e)) & 0x03030303u;
      const uint32_t m1 = (x >> (2 * e + 2)) & 0x03030303u;
      const long data = (long)(((unsigned long long)m1 << 32) | m0);
      const float4_t z = {0.0f, 0.0f, 0.0f, 0.0f};
      const float4_t l = __builtin_amdgcn_mfma_f32_16x16x32_bf8_fp8(sel0, data, z, 0, 0, 0);
      const float4_t h = __builtin_amdgcn_mfma_f32_16x16x32_bf8_fp8(sel1, data, z, 0, 0, 0);
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        fma_step(acc[4 * k + e], s, l[k], b);
        fma_step(acc[4 * k + e + 1], s, h[k], b);
      }
    }
  } else if constexpr (DTYPE == TRA_INT2 && !WEIGHTED) {
    // Same FP8 reading as for int4, on the four 2-bit fields of every byte.
    const float s9 = s * 512.0f;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const uint32_t m = (x >> (2 * e)) & 0x03030303u;
      const float2_t m01 = __builtin_amdgcn_cvt_pk_f32_fp8((int)m, false);
      const float2_t m23 = __builtin_amdgcn_cvt_pk_f32_fp8((int)m, true);
      fma_step(acc[0 + e], s9, m01.x, b);
      fma_step(acc[4 + e], s9, m01.y, b);
      fma_step(acc[8 + e], s9, m23.x, b);
      fma_step(acc[12 + e], s9, m23.y, b);
    }
  } else if constexpr (DTYPE == TRA_INT2) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const uint32_t m = (x >> (2 * e)) & 0x03030303u;
      fma_step(acc[0 + e], s, byte_to_float<0>(m), b);
      fma_step(acc[4 + e], s, byte_to_float<1>(m), b);
      fma_step(acc[8 + e], s, byte_to_float<2>(m), b);
      fma_step(acc[12 + e], s, byte_to_float<3>(m), b);
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

// Everything a lane needs to walk rows of its feature's table.
struct RowWalk {
  const uint8_t* lane_base;  // table + this lane's chunk offset inside a row
  int64_t rows;
  uint32_t rows32;     // min(rows, 2^31): bound for int32 ids
  uint32_t row_bytes;
  int chunk_off;
  bool count_errors;
  // Where a lane loads the dword in front of its chunk together with the chunk
  // (header_with_chunk), the row's header arrives in the row's first lane.
  int hdr_lane;
  // Selector operands of the matrix instruction that converts int4 / int2
  // fields (mfma_byte_selector); they depend on the lane only.
  long sel0, sel1;
  // position weighting: this bag's weight vector (always readable), its last
  // index, whether the feature has one at all, and where the bag starts
  const float* pw;
  uint32_t pw_last;
  bool pw_on;
  int64_t bag_start;
  __device__ __forceinline__ void set_position_weights(const LookupArgs& a, int ci, int64_t start);
  __device__ __forceinline__ void set_rows(int64_t r, int32_t rb) {
    rows = r;
    rows32 = r < (int64_t(1) << 31) ? (uint32_t)r : 0x80000000u;
    row_bytes = (uint32_t)rb;
  }
};

__device__ __forceinline__ void RowWalk::set_position_weights(const LookupArgs& a, int ci,
                                                              int64_t start) {
  pw = a.posw;
  pw_last = 0;
  pw_on = false;
  bag_start = start;
  if (a.posw != nullptr) {
    const int n = ci < kMaxPos ? a.pw_len[ci] : 0;
    pw_on = n > 0;
    pw = a.posw + (n > 0 ? a.pw_off[ci] : 0);
    pw_last = (uint32_t)(n > 0 ? n - 1 : 0);
  }
}

// Id of position j, or -1 (= skip) when the position is outside the bag.  The
// load itself is unconditional (position clamped into the ids array) and the
// result is selected afterwards: a load under a lane predicate would be
// followed by a full wait at the re-convergence point and serialize the ids.
template <typename IdxT>
__device__ __forceinline__ IdxT fetch_id(const LookupArgs& a, bool in_range, IdxT j, IdxT last) {
  // Ids and positions stay in the width of the index type: with int32 ids the
  // whole address computation is 32-bit (plus one 64-bit add to the base).
  using UIdxT = typename std::make_unsigned<IdxT>::type;
  const IdxT jc = (UIdxT)j < (UIdxT)last ? j : last;  // also catches a wrapped position
  const IdxT id = reinterpret_cast<const IdxT*>(a.indices)[jc];
  return in_range ? id : (IdxT)-1;
}

// Values of the kernels' WEIGHTED parameter: how a row's weight is obtained.
constexpr int kUnweighted = 0;
constexpr int kPerSample = 1;   // psw[j]
constexpr int kByPosition = 2;  // position weight of the id's place in its bag

// Issue the loads of one row chunk (header dword, CB payload bytes, weight).
// Branch-free: an id outside [0, rows) (a pruned id -1, a lane past the end of
// its bag, or a bad id) is redirected to row 0 and flagged invalid; consume_row
// then multiplies it away exactly.  Returns 1 for a bad id (out of range and
// not -1).
// GIVEN_W: the caller already holds the row's weight (`given_w`), fetched a
// lane group at a time like the ids; no weight load is issued here.
template <int DTYPE, int CB, int WEIGHTED, typename IdxT, bool GIVEN_W = false>
__device__ __forceinline__ int fetch_row(RowBuf<CB>& r, IdxT id, IdxT j, IdxT last,
                                          const LookupArgs& a, const RowWalk& w, float given_w = 1.0f) {
  const uint8_t* lane_base = w.lane_base;  // table + this lane's chunk offset
  const int chunk_off = w.chunk_off;
  bool valid;
  const uint8_t* chunk;
  if constexpr (sizeof(IdxT) == 4) {
    // One unsigned compare covers negative ids; the row address is a single
    // 32 x 32 + 64 bit multiply-add.
    valid = (uint32_t)id < w.rows32;
    const uint32_t idc = valid ? (uint32_t)id : 0u;
    chunk = lane_base + (uint64_t)idc * (uint64_t)w.row_bytes;
  } else {
    valid = (uint64_t)id < (uint64_t)w.rows;
    const int64_t idc = valid ? (int64_t)id : 0;
    chunk = lane_base + idc * (int64_t)w.row_bytes;
  }
  if constexpr (header_with_chunk<DTYPE, CB>()) {
    // One load: the dword in front of the lane's chunk and the chunk.  For the
    // row's first lane that dword is the header; consume_row hands it round.
    const Chunk<CB + 4> t = load_chunk<CB + 4>(chunk - 4);
    r.hdr = t.v[0];
#pragma unroll
    for (int i = 0; i < CB / 4; ++i) r.d.v[i] = t.v[i + 1];
  } else {
    if constexpr (Traits<DTYPE>::kHeader != 0)
      r.hdr = *reinterpret_cast<const uint32_t*>(chunk - chunk_off);
    else
      r.hdr = 0;
    r.d = load_chunk<CB>(chunk);
  }
  if constexpr (WEIGHTED != 0 && GIVEN_W) {
    r.w = given_w;
  } else if constexpr (WEIGHTED) {
    using UIdxT = typename std::make_unsigned<IdxT>::type;
    if constexpr (WEIGHTED == kByPosition) {
      // The weight of this id's place in its bag, clamped into the feature's
      // weight vector (a slot past the end of its bag reads some valid weight
      // and is dropped later); 1 for a feature without position weights.
      const UIdxT k = (UIdxT)(j - (IdxT)w.bag_start);
      const uint32_t kc = k < (UIdxT)w.pw_last ? (uint32_t)k : w.pw_last;
      const float v = w.pw[kc];
      r.w = w.pw_on ? v : 1.0f;
    } else {
      const IdxT jc = (UIdxT)j < (UIdxT)last ? j : last;
      r.w = a.psw[jc];
    }
  } else {
    r.w = 1.0f;
  }
  r.valid = valid;
  return (!valid && id != (IdxT)-1) ? 1 : 0;
}

// Accumulate one fetched row chunk.  An invalid row contributes fmaf(+0, q,
// acc + (+0)), which leaves acc unchanged bit-for-bit: acc is never -0 (it
// starts at +0 and a round-to-nearest sum is -0 only if both addends are), and
// q is a finite integer.  For fp16 / fp32 rows the payload of an invalid row is
// zeroed as well, so a stored inf / nan in row 0 cannot leak in.
// WHOLE_WAVE: every lane of the wave is executing (the pooling loops: their
// trip counts are wave-uniform and skipped rows are masked, never branched
// around).  The matrix instruction reads its operands from all 64 lanes
// whatever the execution mask, so it is used only there.
template <int DTYPE, int CB, bool WEIGHTED, bool WHOLE_WAVE = true>
__device__ __forceinline__ void consume_row(float* acc, const RowBuf<CB>& r0, const RowWalk& w) {
  constexpr int EPD = 32 / Traits<DTYPE>::kBits;  // elements per dword
  RowBuf<CB> r = r0;
  if constexpr (header_with_chunk<DTYPE, CB>())
    r.hdr = (uint32_t)__shfl((int)r0.hdr, w.hdr_lane, kWaveSize);  // the header sits with the row's first lane
  float s, b;
  if constexpr (Traits<DTYPE>::kHeader != 0) {
    if constexpr (WEIGHTED) {
      // The weight of a skipped slot is whatever lies at the clamped
      // position, possibly inf / nan: select after the products.
      s = r.w * half_bits_to_float(r.hdr & 0xffffu);
      b = r.w * half_bits_to_float(r.hdr >> 16);
      s = r.valid ? s : 0.0f;
      b = r.valid ? b : 0.0f;
    } else {
      const uint32_t hdr = r.valid ? r.hdr : 0u;  // scale = bias = +0
      s = half_bits_to_float(hdr & 0xffffu);
      b = half_bits_to_float(hdr >> 16);
    }
    // int4 fields go through the matrix core where a lane holds at most 16
    // accumulators (8-byte chunks), int2 fields always.
    constexpr bool kMatrix =
        WHOLE_WAVE && (Traits<DTYPE>::kBits == 2 || (Traits<DTYPE>::kBits == 4 && CB <= 8));
    if constexpr (kMatrix)
      asm volatile("" : "+v"(s));  // the converted scale stays in a register: no fp16 operand in the fused multiply-adds
#pragma unroll
    for (int i = 0; i < CB / 4; ++i)
      accumulate_dword<DTYPE, WEIGHTED, kMatrix>(acc + i * EPD, r.d.v[i], s, b, w.sel0, w.sel1);
  } else {
    s = r.valid ? r.w : 0.0f;
#pragma unroll
    for (int i = 0; i < CB / 4; ++i)
      accumulate_dword<DTYPE, WEIGHTED, false>(acc + i * EPD, r.valid ? r.d.v[i] : 0u, s, 0.0f, 0, 0);
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
                                            int& tile, int* class_index = nullptr) {
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
  if (class_index) *class_index = sc.first + fi;
  lpr = sc.lpr;
  return true;
}

// Built with -DTRA_INSTRUMENT (never in the shipped library), every wave
// records wall-clock stamps at the phases of the window kernel into a.ts; a
// standalone harness that includes this header reads them back.
#ifdef TRA_INSTRUMENT
#define TRA_STAMP(k)                                                                      \
  do {                                                                                    \
    if ((threadIdx.x & 63) == 0)                                                          \
      a.ts[((size_t)blockIdx.x * (blockDim.x / 64) + threadIdx.x / 64) * 8 + (k)] = wall_clock64(); \
  } while (0)
#else
#define TRA_STAMP(k)
#endif

// ---- pooled lookup ----------------------------------------------------------

// Pool one bag per lane group: ids [start, start + len), in order, into acc.
// max_len is the longest bag among the wave's lane groups (wave-uniform trip
// count).  Software pipeline, per lane group: ids are requested two batches of
// U rows ahead, row chunks one batch ahead, so neither an id load nor a row
// load is waited for in the batch that issued it.
template <int DTYPE, int CB, typename IdxT, int WEIGHTED, int U, int NE>
__device__ __forceinline__ int pool_bag(float (&acc)[NE], const LookupArgs& a,
                                         const RowWalk& w, int64_t start64, int len,
                                         int max_len_any_lane) {
  // Wave-uniform by construction; telling the compiler keeps the loop control
  // on the scalar unit and the loads free of lane-mask bookkeeping.
  const int max_len = __builtin_amdgcn_readfirstlane(max_len_any_lane);
  const IdxT start = (IdxT)start64;
  const IdxT last = (IdxT)(a.num_indices - 1);
  IdxT idA[U], idB[U];
  RowBuf<CB> bufA[U], bufB[U];
  int bad = 0;
  // Row slots at or beyond max_len belong to no lane group: the (wave-uniform)
  // tests below skip their loads and their arithmetic altogether.
#pragma unroll
  for (int u = 0; u < U; ++u) idA[u] = fetch_id<IdxT>(a, u < len, start + u, last);
#pragma unroll
  for (int u = 0; u < U; ++u) idB[u] = fetch_id<IdxT>(a, U + u < len, start + U + u, last);
#pragma unroll
  for (int u = 0; u < U; ++u)
    bad += fetch_row<DTYPE, CB, WEIGHTED, IdxT>(bufA[u], idA[u], start + u, last, a, w);
  for (int it = 0; it < max_len; it += 2 * U) {
#pragma unroll
    for (int u = 0; u < U; ++u)
      idA[u] = fetch_id<IdxT>(a, it + 2 * U + u < len, start + it + 2 * U + u, last);
#pragma unroll
    for (int u = 0; u < U; ++u)
      bad += fetch_row<DTYPE, CB, WEIGHTED, IdxT>(bufB[u], idB[u], start + it + U + u, last, a, w);
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (it + u < max_len) consume_row<DTYPE, CB, (WEIGHTED != 0)>(acc, bufA[u], w);
    if (it + U >= max_len) break;
#pragma unroll
    for (int u = 0; u < U; ++u)
      idB[u] = fetch_id<IdxT>(a, it + 3 * U + u < len, start + it + 3 * U + u, last);
#pragma unroll
    for (int u = 0; u < U; ++u)
      bad += fetch_row<DTYPE, CB, WEIGHTED, IdxT>(bufA[u], idA[u], start + it + 2 * U + u, last, a, w);
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (it + U + u < max_len) consume_row<DTYPE, CB, (WEIGHTED != 0)>(acc, bufB[u], w);
  }
  // Bad ids are counted by the lane that owns column 0.
  if (bad != 0 && w.count_errors) atomicAdd(a.err_count, (unsigned long long)bad);
  return bad;
}

// The same pooling with the ids fetched a whole lane group at a time: lane c of
// the group loads id number j*lpr + c of the bag (block j), and each row's id
// is then passed to the group's lanes with a cross-lane read.  One id load per
// lpr rows instead of one per row.  Needs lpr >= 2*U (a power of two): the
// block after the current one, requested when the current one is entered, is
// then at least two batches ahead, like the ids of pool_bag.
// TWO_BATCHES: lpr == 2 * U, i.e. an id block feeds exactly the two batches of
// one loop iteration.  The block then changes at a fixed place in the loop and
// its load is unconditional, so the number of loads in flight is the same on
// every path and the compiler can wait for the oldest batch alone.  (Behind a
// conditional load it has to assume the worst and drains all loads, which
// undoes the double buffering once per iteration.)
template <int DTYPE, int CB, typename IdxT, int WEIGHTED, int U, int NE, bool TWO_BATCHES = false>
__device__ __forceinline__ int pool_bag_bulk(float (&acc)[NE], const LookupArgs& a,
                                              const RowWalk& w, int64_t start64, int len,
                                              int max_len_any_lane, int lpr, int c,
                                              int group_lane0) {
  const int max_len = __builtin_amdgcn_readfirstlane(max_len_any_lane);
  const int lpr_u = TWO_BATCHES ? 2 * U : __builtin_amdgcn_readfirstlane(lpr);
  const IdxT start = (IdxT)start64;
  const IdxT last = (IdxT)(a.num_indices - 1);
  auto load_block = [&](int j) -> IdxT {
    const int r = j * lpr_u + c;
    return fetch_id<IdxT>(a, r < len, start + (IdxT)r, last);
  };
  // Weights travel the same way: lane c of the group loads the weight of id
  // number j * lpr + c (per-sample weights: psw at that position; position
  // weights: the table entry of that place in the bag), one load per lpr rows.
  auto load_weights = [&](int j) -> float {
    if constexpr (WEIGHTED == kPerSample) {
      using UIdxT = typename std::make_unsigned<IdxT>::type;
      const IdxT p = start + (IdxT)(j * lpr_u + c);
      return a.psw[(UIdxT)p < (UIdxT)last ? p : last];
    } else if constexpr (WEIGHTED == kByPosition) {
      const uint32_t k = (uint32_t)(j * lpr_u + c);
      const float v = w.pw[k < w.pw_last ? k : w.pw_last];
      return w.pw_on ? v : 1.0f;
    } else {
      return 1.0f;
    }
  };
  IdxT cur = load_block(0);
  IdxT nxt = load_block(1);
  float wcur = load_weights(0);
  float wnxt = load_weights(1);
  int cur_j = 0;
  // Id of row r (wave-uniform), or -1 past the bag's end.  r lies in the
  // current block: a batch of U rows never straddles two blocks (U divides
  // lpr) and enter() is called before each batch.  Reading `cur` only matters:
  // a select between cur and nxt would wait for the load of nxt that enter()
  // has just issued.
  auto id_of = [&](int r) -> IdxT {
    const int src = group_lane0 + (r - cur_j * lpr_u);
    return (IdxT)__shfl(cur, src, kWaveSize);
  };
  auto weight_of = [&](int r) -> float {
    if constexpr (WEIGHTED == 0) return 1.0f;
    const int src = group_lane0 + (r - cur_j * lpr_u);
    return __shfl(wcur, src, kWaveSize);
  };
  // Entering the block of row rb: make it the current one and request the next.
  auto enter = [&](int rb) {
    const int j = rb / lpr_u;
    if (j > cur_j) {
      cur = nxt;
      nxt = load_block(j + 1);
      if constexpr (WEIGHTED != 0) {
        wcur = wnxt;
        wnxt = load_weights(j + 1);
      }
      cur_j = j;
    }
  };
  // The same step where it is known to happen (TWO_BATCHES: at every second batch).
  auto advance = [&]() {
    cur = nxt;
    ++cur_j;
    nxt = load_block(cur_j + 1);
    if constexpr (WEIGHTED != 0) {
      wcur = wnxt;
      wnxt = load_weights(cur_j + 1);
    }
  };
  RowBuf<CB> bufA[U], bufB[U];
  int bad = 0;
#pragma unroll
  for (int u = 0; u < U; ++u)
    bad += fetch_row<DTYPE, CB, WEIGHTED, IdxT, true>(bufA[u], id_of(u), start + u, last, a, w, weight_of(u));
  int it = 0;
  if constexpr (TWO_BATCHES) {
    // Whole iterations (2 * U rows, all inside the longest bag) run without the
    // per-row tests: every buffer is consumed on the way round, so the
    // compiler knows at the top of the loop that only the newest batch and
    // the id block are in flight and need not drain them before it reuses a
    // consumed buffer's registers.  The last, partial iteration follows below.
    for (; it + 2 * U <= max_len; it += 2 * U) {
#pragma unroll
      for (int u = 0; u < U; ++u)
        bad += fetch_row<DTYPE, CB, WEIGHTED, IdxT, true>(bufB[u], id_of(it + U + u), start + it + U + u, last, a, w, weight_of(it + U + u));
#pragma unroll
      for (int u = 0; u < U; ++u) consume_row<DTYPE, CB, (WEIGHTED != 0)>(acc, bufA[u], w);
      advance();
#pragma unroll
      for (int u = 0; u < U; ++u)
        bad += fetch_row<DTYPE, CB, WEIGHTED, IdxT, true>(bufA[u], id_of(it + 2 * U + u), start + it + 2 * U + u, last, a, w, weight_of(it + 2 * U + u));
#pragma unroll
      for (int u = 0; u < U; ++u) consume_row<DTYPE, CB, (WEIGHTED != 0)>(acc, bufB[u], w);
    }
  }
  for (; it < max_len; it += 2 * U) {
    if constexpr (!TWO_BATCHES) enter(it + U);
#pragma unroll
    for (int u = 0; u < U; ++u)
      bad += fetch_row<DTYPE, CB, WEIGHTED, IdxT, true>(bufB[u], id_of(it + U + u), start + it + U + u, last, a, w, weight_of(it + U + u));
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (it + u < max_len) consume_row<DTYPE, CB, (WEIGHTED != 0)>(acc, bufA[u], w);
    if (it + U >= max_len) break;
    if constexpr (TWO_BATCHES) advance(); else enter(it + 2 * U);
#pragma unroll
    for (int u = 0; u < U; ++u)
      bad += fetch_row<DTYPE, CB, WEIGHTED, IdxT, true>(bufA[u], id_of(it + 2 * U + u), start + it + 2 * U + u, last, a, w, weight_of(it + 2 * U + u));
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (it + U + u < max_len) consume_row<DTYPE, CB, (WEIGHTED != 0)>(acc, bufB[u], w);
  }
  if (bad != 0 && w.count_errors) atomicAdd(a.err_count, (unsigned long long)bad);
  return bad;
}

// The bags of a wave pooled once more, where the launch wants an id outside
// its table to pool row 0 (what fbgemm's bounds_check_indices makes of such an
// id in its WARNING and IGNORE modes: it rewrites it to 0) and one of the
// wave's bags held such an id.  The pooling loops above skip it; since the
// order of the additions is part of the result, the bag cannot be corrected
// afterwards and is pooled again from zero, one row at a time (rare by
// assumption: bad ids are an input error).  Bad ids are not counted again.
template <int DTYPE, int CB, typename IdxT, int WEIGHTED, int NE>
__device__ __forceinline__ void repool_bad_ids_as_row0(float (&acc)[NE], const LookupArgs& a,
                                                    const RowWalk& w, int64_t start64, int len,
                                                    int max_len_any_lane) {
  const int max_len = __builtin_amdgcn_readfirstlane(max_len_any_lane);
  const IdxT start = (IdxT)start64;
  const IdxT last = (IdxT)(a.num_indices - 1);
#pragma unroll
  for (int k = 0; k < NE; ++k) acc[k] = 0.0f;
  for (int r = 0; r < max_len; ++r) {
    const IdxT id = fetch_id<IdxT>(a, r < len, start + (IdxT)r, last);
    RowBuf<CB> buf;
    fetch_row<DTYPE, CB, WEIGHTED, IdxT>(buf, id, start + (IdxT)r, last, a, w);
    if (id != (IdxT)-1) buf.valid = 1;  // fetch_row has redirected an id outside the table to row 0
    consume_row<DTYPE, CB, (WEIGHTED != 0)>(acc, buf, w);
  }
}

// Finish one bag per lane group (MEAN scaling, rounding, store).  Lane c of the
// group's lpr lanes holds the NE outputs at columns row_pos + c * NE.  Every
// lane of the wave calls this; `active` says whether its group holds a bag.
// Where a lane's outputs are two 16-byte vectors, storing them as they lie
// would write every other 16 bytes of the group's row with each of the two
// store instructions, i.e. half lines.  The lanes exchange vectors first, so
// that store k writes the k-th half of the row in whole lines (lane c sends
// bytes [(k * lpr + c) * 16, + 16) of the row, which lane (k * lpr + c) / 2
// owns), and the stores carry the non-temporal hint: the output is written
// once and read by a later kernel, and whole lines leave the L2 as they come
// (-0.5 to -1 us on the 13.6 MB output of the C2 workload).
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

template <int NE>
__device__ __forceinline__ void finish_bag(float (&acc)[NE], const LookupArgs& a, int len,
                                           int64_t row_pos, int c, int lpr, int lane, bool active) {
  if (a.mean && len > 0) {
    const float inv = 1.0f / (float)len;
#pragma unroll
    for (int i = 0; i < NE; ++i) acc[i] *= inv;
  }
  if constexpr (NE == 16 || NE == 8) {
    const bool two_vectors = a.vec_store && lpr >= 2 && (lpr & (lpr - 1)) == 0 &&
                             (a.out_fp16 ? NE == 16 : NE == 8);  // wave-uniform
    if (two_vectors) {
      uint32_t v[2][4];
      if (a.out_fp16) {
        if constexpr (NE == 16) {
#pragma unroll
          for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int k = 0; k < 4; ++k) {
              const uint32_t lo = __half_as_ushort(__float2half_rn(acc[8 * h + 2 * k]));
              const uint32_t hi = __half_as_ushort(__float2half_rn(acc[8 * h + 2 * k + 1]));
              v[h][k] = lo | (hi << 16);
            }
        }
      } else {
        if constexpr (NE == 8) {
#pragma unroll
          for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int k = 0; k < 4; ++k) v[h][k] = __builtin_bit_cast(uint32_t, acc[4 * h + k]);
        }
      }
      unsigned char* row = reinterpret_cast<unsigned char*>(a.out) + row_pos * (a.out_fp16 ? 2 : 4);
#pragma unroll
      for (int k = 0; k < 2; ++k) {
        const int g = k * lpr + c;  // which 16 bytes of the row this lane stores
        const int src = (lane - c) + (g >> 1);
        u32x4_t x;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const uint32_t x0 = (uint32_t)__shfl((int)v[0][i], src, kWaveSize);
          const uint32_t x1 = (uint32_t)__shfl((int)v[1][i], src, kWaveSize);
          x[i] = (g & 1) ? x1 : x0;
        }
        if (active) __builtin_nontemporal_store(x, reinterpret_cast<u32x4_t*>(row + (int64_t)g * 16));
      }
      return;
    }
  }
  if (active) store_outputs<NE>(a, row_pos + (int64_t)c * NE, acc);
}

// Balanced mapping.  One 1024-thread block per compute unit owns a window of
// consecutive bags (of one sub-class, possibly spanning features).  It ranks
// them by length in LDS, longest first, and cuts the order into rounds of gpw
// bags; a round is pooled by one wave, one bag per lane group, so the lane
// groups that run in lock step hold bags of nearly equal length.  Rounds are
// dealt to the block's 16 waves in serpentine order over the four SIMDs (waves
// w, w+4, w+8, w+12 share SIMD w & 3), which evens out the work per SIMD.  A
// bag is still pooled whole and in id order by one lane group; there is no
// scratch memory, atomic or pre-pass.
#ifndef TRA_CU_THREADS  // (measurement builds override these two)
#define TRA_CU_THREADS 1024
#endif
#ifndef TRA_MAX_WINDOW
#define TRA_MAX_WINDOW 2048
#endif
constexpr int kCuThreads = TRA_CU_THREADS;
constexpr int kCuWaves = kCuThreads / kWaveSize;
static_assert(kCuWaves >= 2, "the window kernel splits its prologue between the first wave and the others");
constexpr int kMaxWindow = TRA_MAX_WINDOW;
constexpr int kBagBits = 20;  // window entry = (feature index in sub-class << 20) | sample

constexpr int kLenBins = 256;
constexpr int kMaxWinFeat = 32;  // feature descriptors a window keeps in LDS

// Sort key of a bag length: exact below 192, then steps of 64, then one bin.
// (A negative length, which only a malformed input holds, ranks as empty.)
__device__ __forceinline__ int length_bin(int len) {
  return len < 192 ? max(len, 0) : min(kLenBins - 1, 192 + ((len - 192) >> 6));
}

// Accumulator of the from-lengths prologue: as wide as the index type (with
// int32 offsets every partial sum fits 32 bits by definition).
template <typename IdxT>
struct SumOf { using type = int64_t; };
template <>
struct SumOf<int32_t> { using type = int32_t; };

// This thread's share of sum(lengths[0 .. p)).  The block reads the range 16
// bytes per lane per step, kPrefixBatch independent loads at a time (a lane's
// index past the end is clamped and its value dropped, so no load is
// predicated).
// start() adds up every batch but the last and leaves the last one in flight;
// finish() adds it, so the last round trip overlaps whatever the caller does
// between the two calls.
// Every block of the grid reads a prefix of the same array at the same moment;
// starting each block at a different 16 KB step to spread the L2 channels
// measured the same as all starting at the front, so they start at the front.
// `lengths` is 16-byte aligned.
constexpr int kPrefixBatch = 8;

template <typename IdxT>
struct PrefixSum {
  using S = typename SumOf<IdxT>::type;
  static constexpr int V = 16 / (int)sizeof(IdxT);
  struct __align__(16) Vec { IdxT v[V]; };

  const Vec* vin;
  int nvec, nk, last, k_last;
  S part;
  IdxT tail;
  Vec x[kPrefixBatch];

  // Step k of this thread covers vector k * kCuThreads + threadIdx.x; a step
  // past the end reads the last vector again (clamped) and adds nothing.
  __device__ __forceinline__ Vec fetch(int k) const {
    return vin[min(k * kCuThreads + (int)threadIdx.x, last)];
  }
  __device__ __forceinline__ void add(int k, const Vec& v) {
    S sum = 0;
#pragma unroll
    for (int i = 0; i < V; ++i) sum += (S)v.v[i];
    part += k * kCuThreads + (int)threadIdx.x < nvec ? sum : (S)0;
  }
  __device__ __forceinline__ void issue(int k0) {
#pragma unroll
    for (int k = 0; k < kPrefixBatch; ++k) x[k] = fetch(k0 + k);
  }
  __device__ __forceinline__ void consume(int k0) {
#pragma unroll
    for (int k = 0; k < kPrefixBatch; ++k) add(k0 + k, x[k]);
  }
  __device__ __forceinline__ void start(const IdxT* __restrict__ lengths, int64_t p) {
    vin = reinterpret_cast<const Vec*>(lengths);
    nvec = (int)(p / V);
    nk = (nvec + kCuThreads - 1) / kCuThreads;
    last = max(nvec - 1, 0);
    part = 0;
    // the elements after the last whole 16-byte step: one per lane, clamped like the rest
    const int64_t rest = p - (int64_t)nvec * V;
    const int64_t ti = (int64_t)nvec * V + min((int64_t)threadIdx.x, max(rest - 1, (int64_t)0));
    tail = lengths[max(min(ti, p - 1), (int64_t)0)];
    if ((int64_t)threadIdx.x >= rest) tail = 0;
    k_last = nk > 0 ? ((nk - 1) / kPrefixBatch) * kPrefixBatch : 0;
    // kPrefixBatch loads stay in flight: each step adds the oldest (loads
    // return in issue order) and puts the load of the step one batch ahead
    // in its place.  The last batch is left for finish().
    issue(0);
    for (int k0 = 0; k0 < k_last; k0 += kPrefixBatch) {
#pragma unroll
      for (int k = 0; k < kPrefixBatch; ++k) {
        add(k0 + k, x[k]);
        x[k] = fetch(k0 + kPrefixBatch + k);
      }
    }
  }
  __device__ __forceinline__ S finish() {
    consume(k_last);
    return part + (S)tail;
  }
};

// The same sum for waves that have nothing else in flight: the number of loads
// follows the length of the range (in steps of four per thread), and all of
// them are requested before the first is waited for.
template <typename IdxT>
struct PrefixSumAtOnce {
  using S = typename SumOf<IdxT>::type;
  static constexpr int V = 16 / (int)sizeof(IdxT);
  struct __align__(16) Vec { IdxT v[V]; };
  const Vec* vin;
  int tid, nt, nvec, last;

  template <int N>
  __device__ __forceinline__ S steps(int k0) const {
    Vec x[N];
#pragma unroll
    for (int k = 0; k < N; ++k) x[k] = vin[min((k0 + k) * nt + tid, last)];
    S part = 0;
#pragma unroll
    for (int k = 0; k < N; ++k) {
      S sum = 0;
#pragma unroll
      for (int i = 0; i < V; ++i) sum += (S)x[k].v[i];
      part += (k0 + k) * nt + tid < nvec ? sum : (S)0;
    }
    return part;
  }
  // This thread's share of sum(lengths[0 .. p)); thread tid_ of nt_.
  __device__ __forceinline__ S run(const IdxT* __restrict__ lengths, int64_t p, int tid_, int nt_) {
    tid = tid_;
    nt = nt_;
    vin = reinterpret_cast<const Vec*>(lengths);
    nvec = (int)(p / V);
    last = max(nvec - 1, 0);
    const int nk = (nvec + nt - 1) / nt;
    // the elements after the last whole 16-byte step: one per thread
    const int64_t rest = p - (int64_t)nvec * V;
    const int64_t ti = (int64_t)nvec * V + min((int64_t)tid, max(rest - 1, (int64_t)0));
    IdxT tail = lengths[max(min(ti, p - 1), (int64_t)0)];
    if ((int64_t)tid >= rest) tail = 0;
    S part = 0;
    int k0 = 0;
    for (; nk - k0 > 16; k0 += 16) part += steps<16>(k0);
    const int r = nk - k0;
    if (r > 12)
      part += steps<16>(k0);
    else if (r > 8)
      part += steps<12>(k0);
    else if (r > 4)
      part += steps<8>(k0);
    else if (r > 0)
      part += steps<4>(k0);
    return part + (S)tail;
  }
};

// Inclusive scan over the 64 lanes of a wave.  32-bit sums use the data-parallel
// lane moves of the VALU (shifts inside each row of 16 lanes, then lane 15 and
// lane 31 broadcast into the following rows): six adds, no trip through the LDS
// crossbar.  Lanes without a source receive 0.
__device__ __forceinline__ int32_t wave_scan_incl(int32_t v) {
  v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, true);   // row_shr:1
  v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, true);   // row_shr:2
  v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, true);   // row_shr:4
  v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, true);   // row_shr:8
  v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false);  // row_bcast:15 into rows 1 and 3
  v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false);  // row_bcast:31 into rows 2 and 3
  return v;
}
__device__ __forceinline__ int64_t wave_scan_incl(int64_t v) {
  const int ln = threadIdx.x & (kWaveSize - 1);
#pragma unroll
  for (int off = 1; off < kWaveSize; off <<= 1) {
    const int64_t o = __shfl_up(v, off, kWaveSize);
    if (ln >= off) v += o;
  }
  return v;
}
// Lane 63's value of v, in every lane.
__device__ __forceinline__ int32_t wave_last(int32_t v) { return __builtin_amdgcn_readlane(v, kWaveSize - 1); }
__device__ __forceinline__ int64_t wave_last(int64_t v) { return __shfl(v, kWaveSize - 1, kWaveSize); }

// Block barrier that orders LDS accesses only.  __syncthreads() also waits for
// every outstanding global load of the wave; the window kernel's prologue keeps
// loads in flight across its barriers (nothing there is handed from wave to
// wave through global memory).
// The same inside one wave: LDS writes of its lanes are visible to its other lanes.
__device__ __forceinline__ void wave_lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront", "local");
  __builtin_amdgcn_wave_barrier();
}
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// Position of feature `fi` of a sub-class among the input keys: from the launch
// arguments when the class is small enough, else from the descriptors.
__device__ __forceinline__ int feat_key_pos(const LookupArgs& a, const SubClass& sc, int fi) {
  if (sc.key0 >= 0) return sc.key0 + fi;  // no load: the bag bounds can be requested at once
  return sc.first + fi < kMaxPos ? (int)a.feat_pos[sc.first + fi]
                                 : a.descs[a.feats[sc.first + fi]].feature;
}

// Static mapping: lane group g of wave w of tile t owns bag (t*waves + w)*gpw + g.
// Used for small problems, where there are not enough bags to balance.
// FROM_LENGTHS: a.offsets points at the KJT's lengths; the block sums what
// lies in front of its first bag (every block reads that prefix again: this
// form is for calls with few bags, where a scan kernel of its own would cost
// more than the lookup) and scans its own bags, which are consecutive.
template <int DTYPE, int CB, typename IdxT, int WEIGHTED, int U, bool FROM_LENGTHS = false>
__global__ __launch_bounds__(kBlockThreads) void tbe_pooled_kernel(const LookupArgs a) {
  constexpr int NE = CB * 8 / Traits<DTYPE>::kBits;  // columns per lane
  TRA_STAMP(0);
  int f, lpr, tile, ci;
  if (!locate_tile(a, f, lpr, tile, &ci)) return;
  const FeatureDesc d = a.descs[f];
  const int lane = threadIdx.x & (kWaveSize - 1);
  const int wave = threadIdx.x / kWaveSize;
  const int gpw = kWaveSize / lpr;  // lane groups (bags) per wave
  const int g = lane / lpr;
  const int c = lane - g * lpr;
  const int bag_in_feat = (tile * kWavesPerBlock + wave) * gpw + g;
  const bool active = g < gpw && bag_in_feat < a.B;

  int64_t start = 0;
  int len = 0;
  if (FROM_LENGTHS) {
    using Sum = typename SumOf<IdxT>::type;
    constexpr int V = 16 / (int)sizeof(IdxT);
    struct __align__(16) Vec { IdxT v[V]; };
    __shared__ Sum s_front[kWavesPerBlock];
    __shared__ Sum s_wave_tot[kWavesPerBlock];
    const IdxT* lengths = reinterpret_cast<const IdxT*>(a.offsets);
    // this lane group's own length first: its load shares the latency of the prefix loads
    const int64_t bag = (int64_t)d.feature * a.B + min(bag_in_feat, a.B - 1);
    const Sum raw = active ? (Sum)lengths[bag] : (Sum)0;
    // sum(lengths[0 .. p)), p = position of the block's first bag (16-byte steps, then the rest)
    const int64_t p = (int64_t)d.feature * a.B + (int64_t)tile * kWavesPerBlock * gpw;
    const int nvec = (int)(p / V);
    Sum part = 0;
    for (int v0 = 0; v0 < nvec; v0 += 4 * kBlockThreads) {
      Vec x[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) x[k] = reinterpret_cast<const Vec*>(lengths)[min(v0 + k * kBlockThreads + (int)threadIdx.x, nvec - 1)];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        Sum sum = 0;
#pragma unroll
        for (int i = 0; i < V; ++i) sum += (Sum)x[k].v[i];
        part += v0 + k * kBlockThreads + (int)threadIdx.x < nvec ? sum : (Sum)0;
      }
    }
    {
      const int64_t ti = (int64_t)nvec * V + threadIdx.x;
      if (ti < p) part += (Sum)lengths[ti];
    }
    // bag starts inside the block: scan over the lane groups (the group's first
    // lane carries its length), then over the block's waves
    const Sum incl = wave_scan_incl(c == 0 && g < gpw ? raw : (Sum)0);
    const Sum front_w = wave_last(wave_scan_incl(part));
    if (lane == kWaveSize - 1) s_wave_tot[wave] = incl;
    if (lane == 0) s_front[wave] = front_w;
    __syncthreads();
    Sum before = 0, front = 0;
#pragma unroll
    for (int w = 0; w < kWavesPerBlock; ++w) {
      front += s_front[w];
      if (w < wave) before += s_wave_tot[w];
    }
    start = (int64_t)(front + before + incl - raw);
    len = raw > 0 ? (int)raw : 0;
  } else if (active) {
    const int64_t bag = (int64_t)d.feature * a.B + bag_in_feat;
    start = load_index<IdxT>(a.offsets, bag);
    len = (int)(load_index<IdxT>(a.offsets, bag + 1) - start);
  }
  const int max_len = wave_max(len);
  TRA_STAMP(1);

  RowWalk w;
  w.chunk_off = Traits<DTYPE>::kHeader + d.payload_off + c * CB;
  w.lane_base = a.weights + d.table_offset + w.chunk_off;
  w.set_rows(d.rows, d.row_bytes);
  w.count_errors = c == 0 && d.payload_off == 0;
  w.hdr_lane = lane - c;
  w.sel0 = mfma_byte_selector(lane, 0);
  w.sel1 = mfma_byte_selector(lane, 1);
  w.set_position_weights(a, ci, start);

  float acc[NE];
#pragma unroll
  for (int i = 0; i < NE; ++i) acc[i] = 0.0f;
  const int bad = pool_bag<DTYPE, CB, IdxT, WEIGHTED, U, NE>(acc, a, w, start, len, max_len);
  if (a.bad_to_row0 != 0 && __builtin_amdgcn_ballot_w64(bad != 0) != 0)
    repool_bad_ids_as_row0<DTYPE, CB, IdxT, WEIGHTED, NE>(acc, a, w, start, len, max_len);
  TRA_STAMP(2);
#ifdef TRA_INSTRUMENT
  if ((threadIdx.x & 63) == 0)
    a.ts[((size_t)blockIdx.x * (blockDim.x / 64) + threadIdx.x / 64) * 8 + 4] = max_len;
#endif
  finish_bag<NE>(acc, a, len, (int64_t)bag_in_feat * a.out_stride + d.out_col, c, lpr, lane, active);
  TRA_STAMP(3);
}

// FROM_LENGTHS: a.offsets points at the KJT's lengths instead of its offsets
// and the block derives its bags' start positions itself: one block-wide sum
// of everything in front of the window plus a scan of the window in LDS.
template <int DTYPE, int CB, typename IdxT, int WEIGHTED, int U, bool FROM_LENGTHS = false>
__global__ __launch_bounds__(kCuThreads) void tbe_pooled_cu_kernel(
    const void* p_offsets, const FeatureDesc* p_cdescs, int32_t p_B, int32_t p_xcd_blocks,
    int32_t p_xcd_count, int32_t p_n_sub, int32_t p_window0, int32_t p_count0, int32_t p_key0,
    const LookupArgs a) {
  constexpr int NE = CB * 8 / Traits<DTYPE>::kBits;
  extern __shared__ unsigned char tra_dyn_smem[];  // only its size matters (one block per CU)
  __shared__ int64_t s_start[kMaxWindow];
  __shared__ __align__(16) int s_len[kMaxWindow];
  __shared__ uint32_t s_ent[kMaxWindow];
  __shared__ uint16_t s_order[kMaxWindow];
  __shared__ uint16_t s_slot[kMaxWindow];
  __shared__ int s_hist[kLenBins];
  __shared__ FeatureDesc s_desc[kMaxWinFeat];

  TRA_STAMP(0);
  // Block -> (sub-class, window).  Consecutive windows go to the same XCD
  // (blocks are dealt round-robin to the 8 XCDs), so each L2 sees few tables.
  // The leading kernel parameters repeat what the first fetches need (the
  // hardware preloads them into SGPRs): the block's bag bounds can be
  // requested without waiting for the launch arguments to arrive from memory.
  int blk = blockIdx.x;
  if (p_xcd_blocks > 0) blk = (blk % p_xcd_count) * p_xcd_blocks + blk / p_xcd_count;
  SubClass sc;
  if (p_n_sub == 1) {
    sc.first = 0;
    sc.count = p_count0;
    sc.lpr = a.sub[0].lpr;
    sc.tiles_per_feat = 0;
    sc.tile_start = 0;
    sc.window = p_window0;
    sc.key0 = p_key0;
  } else {
    int s = 0;
#pragma unroll
    for (int i = 1; i < kMaxSub; ++i)
      if (i < a.n_sub && blk >= a.sub[i].tile_start) s = i;
    sc = a.sub[s];
  }
  const int nb_all = sc.count * p_B;
  const int q0 = (blk - sc.tile_start) * sc.window;
  if (q0 >= nb_all) return;
  const int nb = min(sc.window, nb_all - q0);

  const int fi_lo = q0 / p_B;
  using Sum = typename SumOf<IdxT>::type;

  // Bag q0 + i of the window: where it sits in the offsets (or lengths) array.
  auto bag_of = [&](int i, int& fi, int& b) -> int64_t {
    const int q = q0 + i;
    fi = q / p_B;
    b = q - fi * p_B;
    return (int64_t)feat_key_pos(a, sc, fi) * p_B + b;
  };
  // What a bag's start in LDS still lacks (from lengths, small windows: the sum
  // of everything in front of the window arrives last and is added on reading).
  Sum front_add = 0;
  __shared__ Sum s_red[kCuWaves];
  // A window of at most 4 x 64 bags is staged, scanned and ranked by the
  // block's first wave alone, four consecutive bags per lane, with no block
  // barrier on the way; from lengths, the other fifteen waves meanwhile sum
  // the lengths in front of the window.  One barrier joins the two.
  const bool solo = FROM_LENGTHS && nb <= 4 * kWaveSize && sc.key0 >= 0;
  if (solo) {
    const int wv = threadIdx.x / kWaveSize;
    const int ln = threadIdx.x & (kWaveSize - 1);
    if (wv == 0) {
      IdxT given[4];  // lengths as they stand in the KJT (lanes past the window repeat its last bag)
      int fis[4], bs[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const int64_t bag = bag_of(min(4 * ln + k, nb - 1), fis[k], bs[k]);
        given[k] = reinterpret_cast<const IdxT*>(p_offsets)[bag];
      }
      {
        const int nfeat = min((q0 + nb - 1) / p_B - fi_lo + 1, kMaxWinFeat);
        if (ln < nfeat) s_desc[ln] = p_cdescs[sc.first + fi_lo + ln];
      }
#pragma unroll
      for (int k = 0; k < kLenBins / kWaveSize; ++k) s_hist[ln + k * kWaveSize] = 0;
      wave_lds_sync();
      TRA_STAMP(6);
      int len[4], slot[4];
      Sum raw[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const int i = 4 * ln + k;
        raw[k] = 0;
        len[k] = 0;
        slot[k] = 0;
        if (i < nb) {
          // Kept as given: bag starts are the running sum of the lengths as
          // they are; a negative length only makes its own bag empty.
          raw[k] = (Sum)given[k];
          len[k] = (int)given[k];
          s_len[i] = len[k];
          s_ent[i] = ((uint32_t)fis[k] << kBagBits) | (uint32_t)bs[k];
          slot[k] = atomicAdd(&s_hist[length_bin(len[k])], 1);
        }
      }
      // Bag starts inside the window: exclusive scan in window order.
      const Sum tot = raw[0] + raw[1] + raw[2] + raw[3];
      Sum run = wave_scan_incl(tot) - tot;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        if (4 * ln + k < nb) s_start[4 * ln + k] = (int64_t)run;
        run += raw[k];
      }
      if (ln == 0) s_red[0] = 0;
      wave_lds_sync();
      TRA_STAMP(7);
      TRA_STAMP(1);
      {  // counting sort, longest first (as in the general route below)
        int h[kLenBins / kWaveSize];
        int sum = 0;
#pragma unroll
        for (int k = 0; k < kLenBins / kWaveSize; ++k) {
          h[k] = s_hist[kLenBins - 1 - (ln * (kLenBins / kWaveSize) + k)];
          sum += h[k];
        }
        const int incl = wave_scan_incl((int32_t)sum);
        int base = incl - sum;
#pragma unroll
        for (int k = 0; k < kLenBins / kWaveSize; ++k) {
          s_hist[kLenBins - 1 - (ln * (kLenBins / kWaveSize) + k)] = base;
          base += h[k];
        }
      }
      wave_lds_sync();
#pragma unroll
      for (int k = 0; k < 4; ++k)
        if (4 * ln + k < nb) s_order[s_hist[length_bin(len[k])] + slot[k]] = (uint16_t)(4 * ln + k);
    } else {
      PrefixSumAtOnce<IdxT> front_sum;
      const Sum mine = front_sum.run(reinterpret_cast<const IdxT*>(p_offsets),
                                     (int64_t)feat_key_pos(a, sc, fi_lo) * p_B + (q0 - fi_lo * p_B),
                                     (int)threadIdx.x - kWaveSize, kCuThreads - kWaveSize);
      const Sum front_w = wave_last(wave_scan_incl(mine));
      if (ln == 0) s_red[wv] = front_w;
    }
    lds_barrier();
#pragma unroll
    for (int w = 0; w < kCuWaves; ++w) front_add += s_red[w];
    TRA_STAMP(2);
  } else {
    // The first bag of every thread is requested before anything else: the
    // barrier below waits for outstanding loads, and this way the bag bounds
    // and the descriptors share one memory latency instead of queueing up.
    IdxT first_lo = 0, first_hi = 0;
    if ((int)threadIdx.x < nb) {
      int fi, b;
      const int64_t bag = bag_of(threadIdx.x, fi, b);
      first_lo = reinterpret_cast<const IdxT*>(p_offsets)[bag];
      if (!FROM_LENGTHS) first_hi = reinterpret_cast<const IdxT*>(p_offsets)[bag + 1];
    }
    // Descriptors of the features this window touches, kept in LDS so that a
    // round does not start with two dependent global loads.
    {
      const int nfeat = min((q0 + nb - 1) / p_B - fi_lo + 1, kMaxWinFeat);
      if ((int)threadIdx.x < nfeat) s_desc[threadIdx.x] = p_cdescs[sc.first + fi_lo + threadIdx.x];
    }
    // From lengths: the total of everything in front of the window.  Its loads
    // go out after the window's own (loads return in order: whatever is waited
    // for first has to be issued first) and stay in flight until the scan
    // below needs the sum.
    PrefixSum<IdxT> front_sum;
    if (FROM_LENGTHS)
      front_sum.start(reinterpret_cast<const IdxT*>(p_offsets),
                      (int64_t)feat_key_pos(a, sc, fi_lo) * p_B + (q0 - fi_lo * p_B));
    if (threadIdx.x < kLenBins) s_hist[threadIdx.x] = 0;
    lds_barrier();
    TRA_STAMP(6);
    for (int i = threadIdx.x; i < nb; i += kCuThreads) {
      int fi, b;
      const int64_t bag = bag_of(i, fi, b);
      const bool first = i == (int)threadIdx.x;
      int len;
      if (FROM_LENGTHS) {
        // Kept as given: bag starts are the running sum of the lengths as they
        // are (what a separate cumsum would produce); a negative length only
        // makes its own bag empty.
        len = (int)(first ? (int64_t)first_lo : load_index<IdxT>(p_offsets, bag));
      } else {
        const int64_t st = first ? (int64_t)first_lo : load_index<IdxT>(p_offsets, bag);
        const int64_t en = first ? (int64_t)first_hi : load_index<IdxT>(p_offsets, bag + 1);
        s_start[i] = st;
        len = max(0, (int)(en - st));
      }
      s_len[i] = len;
      s_ent[i] = ((uint32_t)fi << kBagBits) | (uint32_t)b;
      s_slot[i] = (uint16_t)atomicAdd(&s_hist[length_bin(len)], 1);
    }
    lds_barrier();
    TRA_STAMP(7);
    if (FROM_LENGTHS) {
      __shared__ Sum s_wave_tot[kCuWaves];
      const int t = threadIdx.x;
      const int wv = t / kWaveSize;
      const int ln = t & (kWaveSize - 1);
      // Exclusive scan of the window's lengths (window order): two bags per
      // thread, wave scan, then the 16 wave totals.  The same barrier carries
      // the block-wide total of everything in front of the window.
      // (Only the waves that hold bags scan; every instruction that all 16 waves
      // of the block execute costs 16 issue cycles per SIMD.)
      const bool holds_bags = 2 * wv * kWaveSize < nb;
      Sum x0 = 0, x1 = 0, inc = 0;
      if (holds_bags) {
        x0 = 2 * t < nb ? s_len[2 * t] : 0;
        x1 = 2 * t + 1 < nb ? s_len[2 * t + 1] : 0;
        inc = wave_scan_incl((Sum)(x0 + x1));
      }
      const Sum front_w = wave_last(wave_scan_incl(front_sum.finish()));
      if (ln == kWaveSize - 1) s_wave_tot[wv] = inc;
      if (ln == 0) s_red[wv] = front_w;
      lds_barrier();
      Sum before = 0, front = 0;
#pragma unroll
      for (int w = 0; w < kCuWaves; ++w) front += s_red[w];
      if (holds_bags) {
#pragma unroll
        for (int w = 0; w < kCuWaves; ++w)
          if (w < wv) before += s_wave_tot[w];
      }
      const Sum excl = before + inc - (x0 + x1);
      // The window covers bags of features fi_lo .. fi_hi of the sub-class.  A
      // feature's bags are contiguous in `lengths`; where the next feature's
      // key position follows directly, the run simply continues.
      const int fi_hi = (q0 + nb - 1) / p_B;
      bool one_run = true;
      if (sc.key0 < 0)
        for (int fi = fi_lo; fi < fi_hi; ++fi) one_run = one_run && feat_key_pos(a, sc, fi + 1) == feat_key_pos(a, sc, fi) + 1;
      if (one_run) {
        if (2 * t < nb) s_start[2 * t] = (int64_t)(front + excl);
        if (2 * t + 1 < nb) s_start[2 * t + 1] = (int64_t)(front + excl + x0);
        lds_barrier();
      } else {
        // General case: keep the bare scan, then add to each run what lies in
        // front of it (summed again for every run that does not continue the
        // previous one).
        if (2 * t < nb) s_start[2 * t] = (int64_t)excl;
        if (2 * t + 1 < nb) s_start[2 * t + 1] = (int64_t)(excl + x0);
        lds_barrier();
        int64_t adj = (int64_t)front;  // start = adj + scan value, for the current run
        int64_t next_pos = -1;
        for (int fi = fi_lo; fi <= fi_hi; ++fi) {
          const int first = max(0, fi * p_B - q0);        // first bag of this feature in the window
          const int last = min(nb, (fi + 1) * p_B - q0);  // one past its last bag
          const int64_t pos = (int64_t)feat_key_pos(a, sc, fi) * p_B + (q0 + first - fi * p_B);
          if (fi != fi_lo && pos != next_pos) {
            PrefixSum<IdxT> again;
            again.start(reinterpret_cast<const IdxT*>(p_offsets), pos);
            const Sum w_ = wave_last(wave_scan_incl(again.finish()));
            if (ln == 0) s_red[wv] = w_;
            lds_barrier();
            Sum total = 0;
#pragma unroll
            for (int w = 0; w < kCuWaves; ++w) total += s_red[w];
            adj = (int64_t)total - s_start[first];
          }
          next_pos = pos + (last - first);
          lds_barrier();  // s_red and s_start[first] have been read by everyone
          for (int i = first + t; i < last; i += kCuThreads) s_start[i] += adj;
          lds_barrier();
        }
      }
    }
    TRA_STAMP(1);
    // Counting sort, longest first: a permutation of 0..nb-1.  hist[] holds the
    // bin sizes and every bag already has its slot within its bin; one wave
    // turns the sizes into start positions (bins in descending order).
    if (threadIdx.x < kWaveSize) {
      const int l = threadIdx.x;
      int h[kLenBins / kWaveSize];
      int sum = 0;
#pragma unroll
      for (int k = 0; k < kLenBins / kWaveSize; ++k) {
        h[k] = s_hist[kLenBins - 1 - (l * (kLenBins / kWaveSize) + k)];
        sum += h[k];
      }
      const int incl = wave_scan_incl((int32_t)sum);
      int base = incl - sum;
#pragma unroll
      for (int k = 0; k < kLenBins / kWaveSize; ++k) {
        s_hist[kLenBins - 1 - (l * (kLenBins / kWaveSize) + k)] = base;
        base += h[k];
      }
    }
    lds_barrier();
    for (int i = threadIdx.x; i < nb; i += kCuThreads)
      s_order[s_hist[length_bin(s_len[i])] + s_slot[i]] = (uint16_t)i;
    lds_barrier();
    TRA_STAMP(2);
  }

  const int lane = threadIdx.x & (kWaveSize - 1);
  const int wave = threadIdx.x / kWaveSize;
  const int lpr = sc.lpr;
  const int gpw = kWaveSize / lpr;
  const int g = lane / lpr;
  const int c = lane - g * lpr;
  const int rounds = (nb + gpw - 1) / gpw;
  // Rounds are ordered longest first and dealt to the waves four at a time,
  // alternating direction over the four SIMDs.  (Dealing them in a strict
  // snake over all 16 waves, or evening out the rounds per wave, measured
  // slower, and handing rounds out from a counter as waves become free
  // measured the same: the waves that finish early leave the CU's memory
  // pipeline to the ones still running.)
  for (int pass = 0; pass * kCuWaves < rounds; ++pass) {
    const int slot = pass * (kCuWaves / 4) + (wave >> 2);
    const int r = slot * 4 + ((slot & 1) ? 3 - (wave & 3) : (wave & 3));
    if (r >= rounds) continue;
    const int pos = r * gpw + g;
    const bool active = g < gpw && pos < nb;
    const int i = s_order[active ? pos : r * gpw];
    const uint32_t ent = s_ent[i];
    const int fi = (int)(ent >> kBagBits);
    const int b = (int)(ent & ((1u << kBagBits) - 1));
    const FeatureDesc d = fi - fi_lo < kMaxWinFeat ? s_desc[fi - fi_lo] : a.cdescs[sc.first + fi];
    const int64_t start = s_start[i] + (int64_t)front_add;
    const int len = active ? max(s_len[i], 0) : 0;
    // The round's trip count.  Lengths below 192 have a sort bin each, so
    // the round's first bag is its longest; from 192 up a bin holds a range of
    // lengths in arrival order, and the longest of the round is found by
    // comparing what the lane groups actually hold.
    int max_len = s_len[s_order[r * gpw]];
    if (max_len >= 192) max_len = wave_max(len);

    RowWalk w;
    w.chunk_off = Traits<DTYPE>::kHeader + d.payload_off + c * CB;
    w.lane_base = a.weights + d.table_offset + w.chunk_off;
    w.set_rows(d.rows, d.row_bytes);
    w.count_errors = c == 0 && d.payload_off == 0;
    w.hdr_lane = lane - c;
    w.sel0 = mfma_byte_selector(lane, 0);
    w.sel1 = mfma_byte_selector(lane, 1);
  w.sel0 = mfma_byte_selector(lane, 0);
  w.sel1 = mfma_byte_selector(lane, 1);
    w.set_position_weights(a, sc.first + fi, start);

    float acc[NE];
#pragma unroll
    for (int k = 0; k < NE; ++k) acc[k] = 0.0f;
    int bad;
    if (U == 4 && lpr >= 2 * U && (lpr & (lpr - 1)) == 0)
      if (lpr == 2 * U)
        bad = pool_bag_bulk<DTYPE, CB, IdxT, WEIGHTED, U, NE, true>(acc, a, w, start, len, max_len, lpr, c, lane - c);
      else
        bad = pool_bag_bulk<DTYPE, CB, IdxT, WEIGHTED, U, NE>(acc, a, w, start, len, max_len, lpr, c, lane - c);
    else
      bad = pool_bag<DTYPE, CB, IdxT, WEIGHTED, U, NE>(acc, a, w, start, len, max_len);
    if (a.bad_to_row0 != 0 && __builtin_amdgcn_ballot_w64(bad != 0) != 0)
      repool_bad_ids_as_row0<DTYPE, CB, IdxT, WEIGHTED, NE>(acc, a, w, start, len, max_len);
    TRA_STAMP(3);
#ifdef TRA_INSTRUMENT
    if (lane == 0) a.ts[((size_t)blockIdx.x * (blockDim.x / 64) + wave) * 8 + 5] = (unsigned long long)max_len;
#endif
    finish_bag<NE>(acc, a, len, (int64_t)b * a.out_stride + d.out_col, c, lpr, lane, active);
    TRA_STAMP(4);
  }
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

  RowWalk w;
  w.chunk_off = Traits<DTYPE>::kHeader + d.payload_off + c * CB;
  w.lane_base = a.weights + d.table_offset + w.chunk_off;
  w.set_rows(d.rows, d.row_bytes);
  w.count_errors = c == 0 && d.payload_off == 0;
  w.hdr_lane = lane - c;
  w.sel0 = mfma_byte_selector(lane, 0);
  w.sel1 = mfma_byte_selector(lane, 1);
  for (int64_t j = first + (int64_t)tile * rows_per_block + wave * gpw + g; j < last;
       j += stride) {
    RowBuf<CB> r;
    const IdxT id = reinterpret_cast<const IdxT*>(a.indices)[j];
    const int bad = fetch_row<DTYPE, CB, false, IdxT>(r, id, (IdxT)j, (IdxT)(a.num_indices - 1), a, w);
    if (bad && w.count_errors) atomicAdd(a.err_count, 1ull);
    if (bad && a.bad_to_row0 != 0) r.valid = 1;  // the row fetched for it is row 0
    float acc[NE];
#pragma unroll
    for (int i = 0; i < NE; ++i) acc[i] = 0.0f;
    consume_row<DTYPE, CB, false, /*WHOLE_WAVE=*/false>(acc, r, w);  // lanes leave this loop one by one
    store_outputs<NE>(a, j * (int64_t)d.dim + d.payload_off * 8 / Traits<DTYPE>::kBits + (int64_t)c * NE,
                      acc);
  }
}

// ---- host side of one launch ----------------------------------------------
struct LaunchClass {
  int dtype;
  int cb;
  bool split = false;  // rows cut into several column slices, header loaded on its own (kSplitHeader)
  std::vector<int32_t> feats;  // plan order: sorted by lpr
  std::vector<int32_t> lprs;   // lanes per row of each feature
  int32_t* feats_dev = nullptr;
  // every slice's first output column is 16-byte aligned for fp16 / fp32 outputs
  bool cols_aligned_fp16 = true;
  bool cols_aligned_fp32 = true;
};

struct LaunchParams {
  int grid;
  int balanced;   // 1: one 1024-thread block per window of bags (tbe_pooled_cu_kernel)
  int lds_bytes;  // dynamic LDS of the balanced kernel (sized so one block fits per CU)
  int unroll;     // rows per pipeline batch: 2, 4 or 8
  bool idx64;
  bool weighted;
  bool nobag;
  bool from_lengths;  // window kernel reads lengths and derives offsets itself
};

template <int DTYPE>
int launch_lookup(const LookupArgs& a, int cb, const LaunchParams& p, hipStream_t stream);

template <int DTYPE, int CB, typename IdxT>
void launch_typed(const LookupArgs& a, const LaunchParams& p, hipStream_t stream) {
  dim3 g(p.grid);
  if (p.nobag) {
    hipLaunchKernelGGL((tbe_nobag_kernel<DTYPE, CB, IdxT>), g, dim3(kBlockThreads), 0, stream, a);
    return;
  }
// What the window kernel's first fetches need, repeated as its leading parameters.
#define TRA_CU_LEADING_ARGS                                                                   \
  a.offsets, a.cdescs, a.B, a.xcd_blocks, a.xcd_count, a.n_sub, a.sub[0].window, a.sub[0].count, \
      a.sub[0].key0
#define TRA_POOLED(W, U)                                                                       \
  do {                                                                                         \
    if (p.balanced && p.from_lengths)                                                          \
      hipLaunchKernelGGL((tbe_pooled_cu_kernel<DTYPE, CB, IdxT, W, 4, true>), g,               \
                         dim3(kCuThreads), p.lds_bytes, stream, TRA_CU_LEADING_ARGS, a);       \
    else if (p.balanced)                                                                       \
      hipLaunchKernelGGL((tbe_pooled_cu_kernel<DTYPE, CB, IdxT, W, U>), g, dim3(kCuThreads),   \
                         p.lds_bytes, stream, TRA_CU_LEADING_ARGS, a);                         \
    else if (p.from_lengths)                                                                   \
      hipLaunchKernelGGL((tbe_pooled_kernel<DTYPE, CB, IdxT, W, 4, true>), g,                  \
                         dim3(kBlockThreads), 0, stream, a);                                   \
    else                                                                                       \
      hipLaunchKernelGGL((tbe_pooled_kernel<DTYPE, CB, IdxT, W, U>), g, dim3(kBlockThreads), 0, \
                         stream, a);                                                           \
  } while (0)
  if constexpr (DTYPE >= kSplitHeader) {  // (one unroll depth for the rare split rows)
    if (a.posw != nullptr) TRA_POOLED(kByPosition, 4); else if (p.weighted) TRA_POOLED(kPerSample, 4); else TRA_POOLED(kUnweighted, 4);
  } else if (a.posw != nullptr) {
    TRA_POOLED(kByPosition, 4);  // (one unroll depth: the others are tuning variants)
  } else if (p.weighted) {
    if (p.unroll >= 8) TRA_POOLED(kPerSample, 8); else if (p.unroll >= 4) TRA_POOLED(kPerSample, 4); else TRA_POOLED(kPerSample, 2);
  } else {
    if (p.unroll >= 8) TRA_POOLED(kUnweighted, 8); else if (p.unroll >= 4) TRA_POOLED(kUnweighted, 4); else TRA_POOLED(kUnweighted, 2);
  }
#undef TRA_POOLED
#undef TRA_CU_LEADING_ARGS
}

template <int DTYPE, int CB>
int launch_lookup_cb(const LookupArgs& a, const LaunchParams& p, hipStream_t stream) {
  if (p.idx64)
    launch_typed<DTYPE, CB, int64_t>(a, p, stream);
  else
    launch_typed<DTYPE, CB, int32_t>(a, p, stream);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return hip_fail(e, "tbe lookup launch");
  return TRA_OK;
}

#define TRA_DEFINE_LAUNCH(DTYPE)                                                          \
  template <>                                                                             \
  int launch_lookup<DTYPE>(const LookupArgs& a, int cb, const LaunchParams& p,            \
                           hipStream_t stream) {                                          \
    switch (cb) {                                                                         \
      case 16:                                                                            \
        if constexpr (DTYPE < kSplitHeader) return launch_lookup_cb<DTYPE, 16>(a, p, stream); \
        break;                                                                            \
      case 8: return launch_lookup_cb<DTYPE, 8>(a, p, stream);                            \
      case 4: return launch_lookup_cb<DTYPE, 4>(a, p, stream);                            \
    }                                                                                     \
    set_error("bad chunk size %d", cb);                                                   \
    return TRA_ERR_INVALID_ARGUMENT;                                                      \
  }

}  // namespace tra
