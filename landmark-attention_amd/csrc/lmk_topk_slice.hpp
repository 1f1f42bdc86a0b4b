// Pieces of the block selection shared by the kernels of lmk_retrieval.hip and by the launch of lmk_fwd32.hip that
// runs the decode-time selection beside the forward over the local window: the rounding contract of a score, the
// wave-wide reductions, the order the picked blocks are written in, and the selection by slices
// (llama/llama_mem.py:367-384 for a handful of query rows).
#pragma once

#include "lmk_common.hpp"
#include "lmk_launch.hpp"

namespace lmk {

// ---------------------------------------------------------------------------
// helpers of the selection: the rounding contract and a wave-wide arg-best
// ---------------------------------------------------------------------------
template <class T>
__device__ __forceinline__ float contract(float dot, float sqrt_hd) {
  return round_to<T>(__fdiv_rn(round_to<T>(dot), sqrt_hd));
}

// wave-wide arg-best under (value desc, index asc); every lane gets the winner.  Inside a row of 16
// lanes the exchange partners come from DPP (no LDS round trip); the four row results are then read
// as scalars.
template <int CTRL>
__device__ __forceinline__ void best_step_dpp(float& v, int& i) {
  const float ov = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
  const int oi = __builtin_amdgcn_update_dpp(0, i, CTRL, 0xf, 0xf, false);
  if (ov > v || (ov == v && oi < i)) {
    v = ov;
    i = oi;
  }
}
__device__ __forceinline__ void wave_best(float& v, int& i) {
  best_step_dpp<0xB1>(v, i);                                      // quad_perm [1,0,3,2]
  best_step_dpp<0x4E>(v, i);                                      // quad_perm [2,3,0,1]
  best_step_dpp<0x141>(v, i);                                     // row_half_mirror
  best_step_dpp<0x140>(v, i);                                     // row_mirror: every lane has its row's best
  float bv = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0));
  int bi = __builtin_amdgcn_readlane(i, 0);
#pragma unroll
  for (int r = 1; r < 4; ++r) {
    const float ov = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 16 * r));
    const int oi = __builtin_amdgcn_readlane(i, 16 * r);
    if (ov > bv || (ov == bv && oi < bi)) {
      bv = ov;
      bi = oi;
    }
  }
  v = bv;
  i = bi;
}

// wave-wide maximum / minimum, every lane gets it (a NaN never wins against a number)
template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}
__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, dpp_f<0xB1>(v));
  v = fmaxf(v, dpp_f<0x4E>(v));
  v = fmaxf(v, dpp_f<0x141>(v));
  v = fmaxf(v, dpp_f<0x140>(v));                                  // every lane has its row's maximum
  const float a = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0));
  const float b = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 16));
  const float c = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 32));
  const float d = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 48));
  return fmaxf(fmaxf(a, b), fmaxf(c, d));
}
__device__ __forceinline__ int wave_min(int v) {
  v = min(v, __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xf, 0xf, false));
  v = min(v, __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xf, 0xf, false));
  v = min(v, __builtin_amdgcn_update_dpp(0, v, 0x141, 0xf, 0xf, false));
  v = min(v, __builtin_amdgcn_update_dpp(0, v, 0x140, 0xf, 0xf, false));
  return min(min(__builtin_amdgcn_readlane(v, 0), __builtin_amdgcn_readlane(v, 16)),
             min(__builtin_amdgcn_readlane(v, 32), __builtin_amdgcn_readlane(v, 48)));
}
// wave-wide arg-best under (value desc, id asc) of one candidate per lane: the maximum first, the ids only where
// several lanes hold it (seldom)
__device__ __forceinline__ void wave_best_one(float v, int id, float& bv, int& bi) {
  bv = wave_max(v);
  const uint64_t eq = __ballot(v == bv);
  if (__popcll(eq) == 1) bi = __builtin_amdgcn_readlane(id, __builtin_ctzll(eq));   // wave-uniform
  else bi = wave_min(v == bv ? id : 0x7fffffff);                 // no lane at all (NaN everywhere): 0x7fffffff
}

// Lane j < k holds the j-th pick of a row; the k picks are written in ascending order as int64.
// Every value is first clamped into the cache (a row whose scores are all NaN picks nothing, and a
// pick left at its initial value must not become a block index), and equal values are ranked by
// lane, so that all k slots of the row are always written with indices the gather may follow.
__device__ __forceinline__ int rank_ascending(int& mine, int lane, int k, int num_mems, int ring_start) {
  mine = min(max(mine, 0), num_mems - 1);
  int age = mine - ring_start;                             // oldest block first: slot order unless the cache is a ring
  age += age < 0 ? num_mems : 0;
  int rank = 0;
  for (int j = 0; j < k; ++j) {
    const int o = __shfl(age, j, 64);
    rank += (o < age || (o == age && j < lane)) ? 1 : 0;
  }
  return rank;
}
__device__ __forceinline__ void write_ascending(int64_t* row_out, int mine, int lane, int k, int num_mems, int ring_start) {
  const int rank = rank_ascending(mine, lane, k, num_mems, ring_start);
  if (lane < k) row_out[rank] = (int64_t)mine;
}

// ---------------------------------------------------------------------------
// select without the bracket, for a handful of query rows (decoding).  The fused kernel gives a
// workgroup 32 rows and a row one wave: with one row per head fifteen of its sixteen waves idle and
// the row's steps run one behind the other on 32 CUs.  Here a row's cached blocks are split into
// slices of 256 over as many workgroups (one wave per SIMD, one block per thread): every score is
// evaluated as the contract defines it (one sequential dot product per lane), a workgroup leaves its
// slice's k best (score, index) in the workspace, and a row's slices are merged by a small kernel -- or
// by the gather step that follows, which needs the row's blocks first thing (merge_slices_row).
// ---------------------------------------------------------------------------

// LDS one workgroup of the slice step needs: the query row in fp32, then the four waves' lists of (score, index)
constexpr int kSliceLdsBytes = 4 * 128 + 2 * kSliceWaves * 64 * 4;

// `wg` = index among the workgroups of the slice step (row-major: query row, then slice); `lds` = kSliceLdsBytes of
// LDS, 16-byte aligned.  Runs as a kernel of its own (lmk_retrieval.hip) or beside the forward over the local
// window (lmk_fwd32.hip).
template <class T, int D>
__device__ __forceinline__ void topk_slice_body(const RetrParams& p, int n_slices, int wg, unsigned char* lds) {
  constexpr int NQ = D / 32;                                      // a key is worked on in quarters of 32 dims
  float* q_lds = (float*)lds;                                     // [D]
  float (*list_v)[64] = (float (*)[64])(lds + 4 * 128);           // [kSliceWaves][64]
  int (*list_i)[64] = (int (*)[64])(lds + 4 * 128 + kSliceWaves * 64 * 4);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int NM = p.num_mems;
  const int64_t row = wg / n_slices;                              // (batch, head, query)
  const int slice = wg % n_slices;
  const int bh = (int)(row / p.T), t = (int)(row % p.T);
  const int b = bh / p.H, hh = bh % p.H;
  const char* qr = (const char*)p.q + 2 * (b * p.qs_b + hh * p.qs_h + (int64_t)t * p.qs_r);
  const char* lk = (const char*)p.lk_rot + (int64_t)bh * lk_tiles(NM) * lk_tile_bytes(D);
  // The wave's 64 blocks (lane l scores block mw + l): in the tiled layout of the keys a load instruction
  // brings one 16-byte chunk of each of them, 512 contiguous bytes per half-wave.
  const int mw = slice * kSliceMems + 64 * wave;
  const char* kr = lk + lk_key_offset(min(mw + lane, (int)(32 * lk_tiles(NM)) - 1), D);   // past the last tile: a re-read whose score is dropped
  u32x4_t ld[NQ][4];
#pragma unroll
  for (int qt = 0; qt < NQ; ++qt)
#pragma unroll
    for (int i = 0; i < 4; ++i) ld[qt][i] = *(const u32x4_t*)(kr + 512 * (4 * qt + i));
  if (tid < D / 2) {
    const uint32_t u = *(const uint32_t*)(qr + 4 * tid);
    q_lds[2 * tid] = unpack_lo<T>(u);
    q_lds[2 * tid + 1] = unpack_hi<T>(u);
  }
  __syncthreads();

  float acc = 0.f;
#pragma unroll
  for (int qt = 0; qt < NQ; ++qt) {
    int q0 = 0;
    asm volatile("" : "+v"(q0) : : "memory");                       // q is read from LDS quarter by quarter ...
#pragma unroll
    for (int c = 0; c < 4; ++c) {                                   // the sequential dot product of the contract, d ascending
      const u32x4_t kk = ld[qt][c];
      const float4 qa = *(const float4*)&q_lds[q0 + 32 * qt + 8 * c];
      const float4 qb = *(const float4*)&q_lds[q0 + 32 * qt + 8 * c + 4];
      acc = __builtin_fmaf(qa.x, unpack_lo<T>(kk[0]), acc);
      acc = __builtin_fmaf(qa.y, unpack_hi<T>(kk[0]), acc);
      acc = __builtin_fmaf(qa.z, unpack_lo<T>(kk[1]), acc);
      acc = __builtin_fmaf(qa.w, unpack_hi<T>(kk[1]), acc);
      acc = __builtin_fmaf(qb.x, unpack_lo<T>(kk[2]), acc);
      acc = __builtin_fmaf(qb.y, unpack_hi<T>(kk[2]), acc);
      acc = __builtin_fmaf(qb.z, unpack_lo<T>(kk[3]), acc);
      acc = __builtin_fmaf(qb.w, unpack_hi<T>(kk[3]), acc);
    }
    asm volatile("" : "+v"(acc));                                   // ... and its 32 fmas are done before the next one is read:
                                                                    // left alone the compiler reads all of q first and spills
  }
  const int m = mw + lane;
  float cv = (m < NM) ? contract<T>(acc, p.sqrt_hd) : -INFINITY;
  int ci = (m < NM) ? m : 0x7fffffff;
  // lane j <- the j-th best of the wave's 64 scores
  float rv = -INFINITY;
  int rx = 0x7fffffff;
  for (int j = 0; j < p.k; ++j) {
    float bv;
    int bi;
    wave_best_one(cv, ci, bv, bi);
    if (bi == ci) cv = -INFINITY;
    if (lane == j) {
      rv = bv;
      rx = bi;
    }
  }
  list_v[wave][lane] = rv;
  list_i[wave][lane] = rx;
  __syncthreads();
  if (wave != 0) return;

  // lane j holds the j-th entry of every wave's list; k picks over the lists, pick j -> candidate j of the slice
  float x[kSliceWaves];
  int xi[kSliceWaves];
#pragma unroll
  for (int w = 0; w < kSliceWaves; ++w) {
    x[w] = list_v[w][lane];
    xi[w] = list_i[w][lane];
  }
  float out_v = -INFINITY;
  int out_i = 0x7fffffff;
  for (int j = 0; j < p.k; ++j) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
#pragma unroll
    for (int w = 0; w < kSliceWaves; ++w)
      if (x[w] > bv || (x[w] == bv && xi[w] < bi)) {
        bv = x[w];
        bi = xi[w];
      }
    const int own = bi;                                             // block indices are unique over the lists
    wave_best(bv, bi);
#pragma unroll
    for (int w = 0; w < kSliceWaves; ++w)
      if (own == bi && xi[w] == bi) x[w] = -INFINITY;
    if (lane == j) {
      out_v = bv;
      out_i = bi;
    }
  }
  if (lane < p.k) {
    const int64_t at = row * NM + (int64_t)slice * p.k + lane;      // n_slices * k <= num_mems: a row of the score planes holds them
    p.approx[at] = out_v;
    ((int*)p.exact)[at] = out_i;
  }
}

// The k best of a row's n_slices * k candidates under (score desc, index asc): lane j < k gets the j-th.  One wave.
__device__ __forceinline__ int merge_slices_row(const RetrParams& p, int n_slices, int64_t row, int lane) {
  const int n_cand = n_slices * p.k;
  if (n_cand <= 64) {                                               // the usual case: a candidate per lane (wave-uniform)
    float cv = -INFINITY;
    int ci = 0x7fffffff;
    if (lane < n_cand) {
      cv = p.approx[row * p.num_mems + lane];
      ci = ((const int*)p.exact)[row * p.num_mems + lane];
    }
    int mine = 0x7fffffff;
    for (int j = 0; j < p.k; ++j) {
      float bv;
      int bi;
      wave_best_one(cv, ci, bv, bi);
      if (bi == ci) cv = -INFINITY;
      if (lane == j) mine = bi;
    }
    return mine;
  }
  constexpr int NJ = kSliceMaxCand / 64;
  float x[NJ];
  int xi[NJ];
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    const int c = 64 * j + lane;
    x[j] = -INFINITY;
    xi[j] = 0x7fffffff;
    if (c < n_cand) {
      x[j] = p.approx[row * p.num_mems + c];
      xi[j] = ((const int*)p.exact)[row * p.num_mems + c];
    }
  }
  int mine = 0x7fffffff;
  for (int j = 0; j < p.k; ++j) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
#pragma unroll
    for (int w = 0; w < NJ; ++w)
      if (x[w] > bv || (x[w] == bv && xi[w] < bi)) {
        bv = x[w];
        bi = xi[w];
      }
    const int own = bi;
    wave_best(bv, bi);
#pragma unroll
    for (int w = 0; w < NJ; ++w)
      if (own == bi && xi[w] == bi) x[w] = -INFINITY;
    if (lane == j) mine = bi;
  }
  return mine;
}

}  // namespace lmk
