// Rotated landmark keys and their norms (llama/llama_mem.py:357-366): the body shared by the kernel that does
// only this and by the one that runs it beside the forward over the local window.
#pragma once

#include "lmk_common.hpp"
#include "lmk_launch.hpp"

namespace lmk {

// One workgroup of NTHR threads rotates R * NTHR / (D / 8) landmark keys, R per thread with the loads of all R in
// flight together; `wg` is its index among the workgroups that do so (the kernel of lmk_retrieval.hip runs nothing
// else; the one of lmk_fwd32.hip runs them beside a forward, whose registers and LDS leave room for few workgroups
// per compute unit, hence R > 1 there).
template <class T, int D, int NTHR, int R = 1>
__device__ __forceinline__ void landmark_keys_body(const RetrParams& p, int wg) {
  constexpr int LPR = D / 8;
  constexpr int RPW = NTHR / LPR;
  const int tid = threadIdx.x, j = tid % LPR;
  const int64_t total = (int64_t)p.B * p.H * p.num_mems;
  int64_t row[R];
  u32x4_t x[R], other[R], c[R], s[R];
#pragma unroll
  for (int i = 0; i < R; ++i) {
    row[i] = ((int64_t)wg * R + i) * RPW + tid / LPR;      // (bh, m)
    const int64_t rr = row[i] < total ? row[i] : total - 1;   // past the end: a re-read that is never stored
    const int bh = (int)(rr / p.num_mems), m = (int)(rr % p.num_mems);
    const int b = bh / p.H, hh = bh % p.H;
    int age = m - p.ring_start;                            // ring caches: slot ring_start holds the oldest block
    age += age < 0 ? p.num_mems : 0;
    const int slot = (age < p.num_mems - p.k) ? 0 : age - (p.num_mems - p.k) + 1;
    const int64_t pos = (int64_t)slot * p.block + (p.block - 1) + p.prefix_len;
    // the landmark is the last row of block m of the cache -- or row m of an array that holds the landmark keys alone
    const int64_t lm_row = p.lm_dense ? (int64_t)m : (int64_t)m * p.block + p.block - 1;
    const char* src = (const char*)p.kcache + 2 * (b * p.kcs_b + hh * p.kcs_h + lm_row * p.kcs_r);
    x[i] = *(const u32x4_t*)(src + 16 * j);
    other[i] = *(const u32x4_t*)(src + 16 * (j ^ (LPR / 2)));
    c[i] = *(const u32x4_t*)((const char*)p.cos + 2 * (pos * p.cs_r) + 16 * j);
    s[i] = *(const u32x4_t*)((const char*)p.sin + 2 * (pos * p.cs_r) + 16 * j);
  }
#pragma unroll
  for (int i = 0; i < R; ++i) {
    float r[8];
    rotate_chunk<T>(x[i], other[i], c[i], s[i], j >= LPR / 2, r);
    const bool ok = row[i] < total;
    u32x4_t o = {pack2<T>(r[0], r[1]), pack2<T>(r[2], r[3]), pack2<T>(r[4], r[5]), pack2<T>(r[6], r[7])};
    if (ok) {
      const int64_t bh = row[i] / p.num_mems;
      const int m = (int)(row[i] % p.num_mems);
      *(u32x4_t*)((char*)p.lk_rot + bh * lk_tiles(p.num_mems) * lk_tile_bytes(D) + lk_key_offset(m, D) + 512 * j) = o;
    }
    float nrm = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) nrm += r[e] * r[e];
#pragma unroll
    for (int msk = LPR / 2; msk >= 1; msk >>= 1) nrm += __shfl_xor(nrm, msk, 64);
    if (ok && j == 0) p.lk_norm[row[i]] = sqrtf(nrm) * 1.000001f;
  }
}

}  // namespace lmk
