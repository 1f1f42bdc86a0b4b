// Host-side parameter blocks and launcher declarations shared by the C ABI
// (lmk_api.hip) and the kernel translation units.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/lmk.h"

namespace lmk {

struct FwdParams {
  const void *q, *k, *v;
  void* o;
  float *L, *M;
  int B, H, Lq, Lk;
  int n_prefix;   // history blocks in front of the queries
  int n_qtiles;   // ceil(Lq / 128)
  int64_t qs_b, qs_h, qs_r, ks_b, ks_h, ks_r, vs_b, vs_h, vs_r, os_b, os_h, os_r;  // element strides
  float scale_log2;  // sm_scale * log2(e)
};

int launch_fwd(const FwdParams& p, int D, int BS, int dtype, hipStream_t stream);

}  // namespace lmk
