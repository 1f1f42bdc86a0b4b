// Rotated landmark keys and their norms (llama/llama_mem.py:357-366): the body shared by the kernel that does
// only this and by the one that runs it beside the forward over the local window.
#pragma once

#include "lmk_common.hpp"
#include "lmk_launch.hpp"

namespace lmk {

// One workgroup of NTHR threads rotates NTHR / (D / 8) landmark keys; `wg` is its index among the workgroups that
// do so (the kernel of lmk_retrieval.hip runs nothing else, the one of lmk_fwd32.hip runs them beside a forward).
template <class T, int D, int NTHR>
__device__ __forceinline__ void landmark_keys_body(const RetrParams& p, int wg) {
  constexpr int LPR = D / 8;
  constexpr int RPW = NTHR / LPR;
  const int tid = threadIdx.x, j = tid % LPR;
  const int64_t row = (int64_t)wg * RPW + tid / LPR;      // (bh, m)
  const int64_t total = (int64_t)p.B * p.H * p.num_mems;
  float nrm = 0.f;
  if (row < total) {
    const int bh = (int)(row / p.num_mems), m = (int)(row % p.num_mems);
    const int b = bh / p.H, hh = bh % p.H;
    int age = m - p.ring_start;                            // ring caches: slot ring_start holds the oldest block
    age += age < 0 ? p.num_mems : 0;
    const int slot = (age < p.num_mems - p.k) ? 0 : age - (p.num_mems - p.k) + 1;
    const int64_t pos = (int64_t)slot * p.block + (p.block - 1) + p.prefix_len;
    // the landmark is the last row of block m of the cache -- or row m of an array that holds the landmark keys alone
    const int64_t lm_row = p.lm_dense ? (int64_t)m : (int64_t)m * p.block + p.block - 1;
    const char* src = (const char*)p.kcache + 2 * (b * p.kcs_b + hh * p.kcs_h + lm_row * p.kcs_r);
    const u32x4_t x = *(const u32x4_t*)(src + 16 * j);
    const u32x4_t other = *(const u32x4_t*)(src + 16 * (j ^ (LPR / 2)));
    const u32x4_t c = *(const u32x4_t*)((const char*)p.cos + 2 * (pos * p.cs_r) + 16 * j);
    const u32x4_t s = *(const u32x4_t*)((const char*)p.sin + 2 * (pos * p.cs_r) + 16 * j);
    float r[8];
    rotate_chunk<T>(x, other, c, s, j >= LPR / 2, r);
    u32x4_t o = {pack2<T>(r[0], r[1]), pack2<T>(r[2], r[3]), pack2<T>(r[4], r[5]), pack2<T>(r[6], r[7])};
    *(u32x4_t*)((char*)p.lk_rot + 2 * (row * D) + 16 * j) = o;
#pragma unroll
    for (int i = 0; i < 8; ++i) nrm += r[i] * r[i];
  }
#pragma unroll
  for (int msk = LPR / 2; msk >= 1; msk >>= 1) nrm += __shfl_xor(nrm, msk, 64);
  if (row < total && j == 0) p.lk_norm[row] = sqrtf(nrm) * 1.000001f;
}

}  // namespace lmk
