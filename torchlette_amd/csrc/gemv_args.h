// Kernel argument blocks of the VALU decode GEMV, shared by the kernels
// (gemv_kernel.h) and the host side (gemv.hip).
#pragma once
#include "device_utils.h"

namespace tlhip {

struct GemvArgs {
  const u32x4* packed;
  const void* scales;
  const void* x;
  void* y;
  int64_t n;
  int k;
  int m;
  int nchunks;           // 16-byte chunks per weight row
  int cpg_shift;         // grouped formats: log2(chunks sharing one scale)
  int groups_per_row;
  int lpr;               // lanes per row
  int lpr_shift;
  int kw;                // waves splitting K inside a workgroup (power of two)
  int kw_shift;
  int nsteps;            // batches per row block
  int nblocks;           // row blocks
  int rows_per_wave;
  int rows_per_wg;
  float alpha;
  float scale_mul;       // 1/127 for INT8_GROUPED, else 1
  int y_dtype;
  DevEpilogue epi;
  DevPrologue pro;
};

// Several problems of one shape class in one launch: workgroups
// [first[i], first[i+1]) work on problem i.
constexpr int kMaxGroup = 4;
struct GroupedGemvArgs {
  int count;
  int first[kMaxGroup + 1];
  GemvArgs p[kMaxGroup];
};

// Defined once per weight format (gemv_int4.hip, gemv_int8_grouped.hip, gemv_int8_row.hip).
#define TLHIP_DECLARE_GEMV_FORMAT(NAME)                                                                  \
  int launch_gemv_##NAME(int x_dtype, int mt, int r, int u, const GemvArgs& a, int threads, int grid,     \
                         size_t lds_bytes, hipStream_t stream);                                          \
  int launch_gemv_grouped_##NAME(int r, const GroupedGemvArgs& g, int threads, size_t lds_bytes,          \
                                 hipStream_t stream);
int launch_gemv_mf4_int4(int u, const GemvArgs& a, int threads, int grid, size_t lds_bytes, hipStream_t stream);
TLHIP_DECLARE_GEMV_FORMAT(int4)
TLHIP_DECLARE_GEMV_FORMAT(int8_grouped)
TLHIP_DECLARE_GEMV_FORMAT(int8_row)

}  // namespace tlhip
