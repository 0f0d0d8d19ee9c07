// Shared host/device declarations of the torchrec_amd kernel library (gfx950).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cstdarg>
#include <cstdio>

#include "../../include/torchrec_amd.h"

namespace tra {

constexpr int kWaveSize = 64;

// Device-side view of one feature of a TBE group (or of one column slice of a
// feature whose payload needs more than 64 lanes).
struct FeatureDesc {
  int64_t table_offset;  // byte offset of the feature's table in the weights buffer
  int64_t rows;          // rows of that table
  int32_t dim;           // embedding dim D of the table
  int32_t row_bytes;     // physical row stride
  int32_t out_col;       // first output column of this slice
  int32_t dtype;         // TRA_* weight type
  int32_t feature;       // feature index f: bag (f, b) is offsets[f*B + b]
  int32_t payload_off;   // byte offset of this slice inside the row payload
};

inline int bits_of(int dtype) {
  switch (dtype) {
    case TRA_FP32: return 32;
    case TRA_FP16: return 16;
    case TRA_INT8: return 8;
    case TRA_INT4: return 4;
    case TRA_INT2: return 2;
    default: return 0;
  }
}
inline int header_bytes(int dtype) {
  return (dtype == TRA_INT8 || dtype == TRA_INT4 || dtype == TRA_INT2) ? 4 : 0;
}

// Thread-local error text behind tra_last_error().
void set_error(const char* fmt, ...);
int hip_fail(hipError_t e, const char* what);

#define TRA_HIP(call)                                   \
  do {                                                  \
    hipError_t e__ = (call);                            \
    if (e__ != hipSuccess) return tra::hip_fail(e__, #call); \
  } while (0)

}  // namespace tra
