// Backward kernels of fused landmark attention for gfx950.
//
// Replace `_bwd_preprocess` and `_bwd_kernel` of the reference
// (llama/ltriton/flash_landmark_attention.py:125-149, :152-305).  The reference runs one
// program per (batch, head) and read-modify-writes dQ in global memory; here the work is
// split so that every accumulator stays in registers and no atomics are needed:
//
//   pre    delta = rowsum(O * dO),  mhat = M*log2(e) + log2(L)          (per query row)
//   dq     query-stationary, S^T layout (lane = query): recomputes the local softmax of
//          every earlier block, the gate, nD = rowsum(P * dP), forms dS and accumulates
//          dQ^T = K^T dS^T.  It also writes, per (query, earlier block), the three numbers
//          the third kernel needs:  a  with  gate*P = exp2(s*c - a),  nD,  and dS at the
//          block's landmark key.
//   dkdv   key-stationary, S layout (lane = key): purely elementwise between its four
//          products S = Q K^T, dP = dO V^T, dV^T += dO^T W, dK^T += Q^T dS
//          (lmk_bwd_dkdv32.hip, all block sizes).
// This file holds the pre kernel, the dQ kernel for blocks of 64 and 128 keys (block 32 has its own in
// lmk_bwd_dq32.hip) and the dispatch.
//
// All probabilities are used normalised (exp2(s*c - mhat) already divides by L), so dO is
// consumed as is; the reference's rescaled copy dO/L (:147) is not needed.
#include <cstdlib>
#include <type_traits>

#include "lmk_common.hpp"
#include "lmk_launch.hpp"

namespace lmk {

// ---------------------------------------------------------------------------
// pre: delta and mhat
// ---------------------------------------------------------------------------
template <class T, int D>
__global__ __launch_bounds__(256) void lmk_bwd_pre_kernel(BwdParams p) {
  constexpr int LPR = D / 8;          // lanes per row (16 bytes each)
  constexpr int RPW = 256 / LPR;      // rows per workgroup
  const int tid = threadIdx.x;
  const int64_t row = (int64_t)blockIdx.x * RPW + tid / LPR;
  const int64_t total = (int64_t)p.B * p.H * p.Lq;
  float sum = 0.f;
  if (row < total) {
    const int bh = (int)(row / p.Lq), qi = (int)(row % p.Lq);
    const int b = bh / p.H, hh = bh % p.H;
    const int d0 = 8 * (tid % LPR);
    const u32x4_t o4 = *(const u32x4_t*)((const char*)p.o + 2 * (b * p.os_b + hh * p.os_h + (int64_t)qi * p.os_r + d0));
    const u32x4_t g4 = *(const u32x4_t*)((const char*)p.dout + 2 * (b * p.dos_b + hh * p.dos_h + (int64_t)qi * p.dos_r + d0));
#pragma unroll
    for (int i = 0; i < 4; ++i)
      sum += unpack_lo<T>(o4[i]) * unpack_lo<T>(g4[i]) + unpack_hi<T>(o4[i]) * unpack_hi<T>(g4[i]);
  }
#pragma unroll
  for (int m = LPR / 2; m >= 1; m >>= 1) sum += __shfl_xor(sum, m, 64);
  if (row < total && (tid % LPR) == 0) {
    p.delta[row] = sum;
    p.mhat[row] = p.M[row] * kLog2e + fast_log2(p.L[row]);
  }
}

// ---------------------------------------------------------------------------
// dq (+ per-block statistics)
// ---------------------------------------------------------------------------
template <class T, int D, int BS>
struct DqCfg {
  static constexpr int NT = BS / 32;
  static constexpr int NB = (BS >= 64) ? 1 : 64 / BS;
  static constexpr int SK = NB * BS;
  static constexpr int CH = D / 8;
  static constexpr int TILE_BYTES = SK * 2 * D;
  static constexpr int NCH = SK * CH / 256;
  static constexpr int KS = D / 16;
  static constexpr int DC = D / 32;
  static constexpr int LDS_BYTES = 4 * TILE_BYTES;
};

template <class T, int D, int BS>
__global__ __launch_bounds__(256, 1) void lmk_bwd_dq_kernel(BwdParams p) {
  using C = DqCfg<T, D, BS>;
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int ql = lane & 31, h = lane >> 5;

  int bh, qtile;
  {
    const int bid = blockIdx.x, BH = p.B * p.H;
    if ((BH & 7) == 0) {
      const int xcd = bid & 7, j = bid >> 3, ngrp = BH >> 3;
      qtile = p.n_qtiles - 1 - j / ngrp;
      bh = (j % ngrp) * 8 + xcd;
    } else {
      qtile = p.n_qtiles - 1 - bid / BH;
      bh = bid % BH;
    }
  }
  const int b = bh / p.H, hh = bh % p.H;
  const char* qp = (const char*)p.q + 2 * (b * p.qs_b + hh * p.qs_h);
  const char* kp = (const char*)p.k + 2 * (b * p.ks_b + hh * p.ks_h);
  const char* vp = (const char*)p.v + 2 * (b * p.vs_b + hh * p.vs_h);
  const char* gp = (const char*)p.dout + 2 * (b * p.dos_b + hh * p.dos_h);
  char* dqp = (char*)p.dq + 2 * (b * p.dqs_b + hh * p.dqs_h);

  const int q0 = qtile * 128 + wave * 32;
  const int dt = p.n_prefix * C::NT + (q0 >> 5);
  const int cblk = dt / C::NT, tsub = dt % C::NT;
  const bool active = q0 < p.Lq;
  const int qrow = q0 + ql;
  const bool rowok = qrow < p.Lq;

  u32x4_t qf[C::KS], gf[C::KS];
#pragma unroll
  for (int ks = 0; ks < C::KS; ++ks) {
    u32x4_t z = {0, 0, 0, 0};
    qf[ks] = z;
    gf[ks] = z;
    if (rowok) {
      qf[ks] = *(const u32x4_t*)(qp + 2 * ((int64_t)qrow * p.qs_r + 16 * ks + 8 * h));
      gf[ks] = *(const u32x4_t*)(gp + 2 * ((int64_t)qrow * p.dos_r + 16 * ks + 8 * h));
    }
  }
  const float mhat = rowok ? p.mhat[(int64_t)bh * p.Lq + qrow] : 0.f;
  const float delta = rowok ? p.delta[(int64_t)bh * p.Lq + qrow] : 0.f;

  const int tiles_needed = min(p.Lk >> 5, p.n_prefix * C::NT + qtile * 4 + 4);
  const int n_stages = (tiles_needed * 32 + C::SK - 1) / C::SK;
  u32x4_t kreg[C::NCH], vreg[C::NCH];
  auto load_stage = [&](int s) {
#pragma unroll
    for (int i = 0; i < C::NCH; ++i) {
      const int id = tid + 256 * i, row = id / C::CH, ch = id % C::CH;
      const int key = s * C::SK + row;
      u32x4_t z = {0, 0, 0, 0};
      kreg[i] = z;
      vreg[i] = z;
      if (key < p.Lk) {
        kreg[i] = *(const u32x4_t*)(kp + 2 * ((int64_t)key * p.ks_r + 8 * ch));
        vreg[i] = *(const u32x4_t*)(vp + 2 * ((int64_t)key * p.vs_r + 8 * ch));
      }
    }
  };
  auto store_stage = [&](int buf) {
    unsigned char* kb = smem + buf * 2 * C::TILE_BYTES;
    unsigned char* vb = kb + C::TILE_BYTES;
#pragma unroll
    for (int i = 0; i < C::NCH; ++i) {
      const int id = tid + 256 * i, row = id / C::CH, ch = id % C::CH;
      *(u32x4_t*)(kb + tile_off<D>(row, ch)) = kreg[i];
      *(u32x4_t*)(vb + tile_off<D>(row, ch)) = vreg[i];
    }
  };

  f32x16_t acc[C::DC];
#pragma unroll
  for (int dc = 0; dc < C::DC; ++dc)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[dc][r] = 0.f;
  const float c2 = p.scale_log2;

  auto row_tile = [&](const unsigned char* buf, int rb, const u32x4_t* bf) {
    f32x16_t s;
#pragma unroll
    for (int r = 0; r < 16; ++r) s[r] = 0.f;
#pragma unroll
    for (int ks = 0; ks < C::KS; ++ks) s = mfma32<T>(load_row_frag<D>(buf, rb, ks, lane), bf[ks], s);
    return s;
  };
  auto dq_tile = [&](const unsigned char* kb, int rb, const float* ds) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      u32x4_t wf = {pack2<T>(ds[8 * j + 0], ds[8 * j + 1]), pack2<T>(ds[8 * j + 2], ds[8 * j + 3]),
                    pack2<T>(ds[8 * j + 4], ds[8 * j + 5]), pack2<T>(ds[8 * j + 6], ds[8 * j + 7])};
#pragma unroll
      for (int dc = 0; dc < C::DC; ++dc) acc[dc] = mfma32<T>(load_tr_frag<D>(kb, rb, j, dc, lane), wf, acc[dc]);
    }
  };

  load_stage(0);
  store_stage(0);
  __syncthreads();

  for (int s = 0; s < n_stages; ++s) {
    const int buf = s & 1;
    if (s + 1 < n_stages) load_stage(s + 1);
    const unsigned char* kb = smem + buf * 2 * C::TILE_BYTES;
    const unsigned char* vb = kb + C::TILE_BYTES;

    if (active) {
#pragma unroll
      for (int jb = 0; jb < C::NB; ++jb) {
        const int blk = s * C::NB + jb;
        const int rb0 = jb * BS;
        if (blk < cblk) {
          f32x16_t sc[C::NT], dp[C::NT];
#pragma unroll
          for (int u = 0; u < C::NT; ++u) sc[u] = row_tile(kb, rb0 + 32 * u, qf);
#pragma unroll
          for (int u = 0; u < C::NT; ++u) dp[u] = row_tile(vb, rb0 + 32 * u, gf);
          const float s_last = sc[C::NT - 1][15];
          float mx = (h == 0) ? s_last : -INFINITY;
#pragma unroll
          for (int u = 0; u < C::NT; ++u)
#pragma unroll
            for (int r = 0; r < 16; ++r)
              if (!(u == C::NT - 1 && r == 15)) mx = fmaxf(mx, sc[u][r]);
          mx = pair_max(mx);
          const float t_lm = pair_hi(s_last) * c2;
          const float mloc = mx * c2;
          float den = 0.f, spd = 0.f;
#pragma unroll
          for (int u = 0; u < C::NT; ++u)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              float e = fast_exp2(__builtin_fmaf(sc[u][r], c2, -mloc));
              if (u == C::NT - 1 && r == 15) e = (h == 0) ? e : 0.f;
              sc[u][r] = e;
              den += e;
              spd = __builtin_fmaf(e, dp[u][r], spd);
            }
          den = pair_sum(den);
          spd = pair_sum(spd);
          const float invden = fast_rcp(den);
          const float nD = spd * invden;
          const float glog = t_lm - mhat;               // log2 of the normalised gate
          const float g = fast_exp2(glog);
          const float f = g * invden;
          if (h == 0 && rowok) {
            const int64_t si = ((int64_t)bh * p.n_blocks + blk) * p.Lq + qrow;
            p.stat_a[si] = mloc + fast_log2(den) - glog;
            p.stat_n[si] = nD;
            p.stat_l[si] = g * (nD - delta);              // dS at the block's landmark key
          }
#pragma unroll
          for (int u = 0; u < C::NT; ++u) {
            float ds[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) ds[r] = sc[u][r] * f * (dp[u][r] - nD);
            if (u == C::NT - 1 && h == 1) ds[15] = g * (nD - delta);
            dq_tile(kb, rb0 + 32 * u, ds);
          }
        } else if (blk == cblk) {
          const int lim = ql - ((tsub == C::NT - 1 && ql == 31) ? 1 : 0);
#pragma unroll
          for (int u = 0; u < C::NT; ++u) {
            if (u <= tsub) {
              f32x16_t sc = row_tile(kb, rb0 + 32 * u, qf);
              f32x16_t dp = row_tile(vb, rb0 + 32 * u, gf);
              float ds[16];
#pragma unroll
              for (int r = 0; r < 16; ++r) {
                const int key = 8 * (r >> 2) + 4 * h + (r & 3);
                const float pr = (u < tsub || key <= lim) ? fast_exp2(__builtin_fmaf(sc[r], c2, -mhat)) : 0.f;
                ds[r] = pr * (dp[r] - delta);
              }
              dq_tile(kb, rb0 + 32 * u, ds);
            }
          }
        }
      }
    }
    if (s + 1 < n_stages) store_stage(buf ^ 1);
    __syncthreads();
  }

  if (active && rowok) {
    const float sc = p.scale;
#pragma unroll
    for (int dc = 0; dc < C::DC; ++dc)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        u32x2_t o2 = {pack2<T>(acc[dc][4 * g + 0] * sc, acc[dc][4 * g + 1] * sc),
                      pack2<T>(acc[dc][4 * g + 2] * sc, acc[dc][4 * g + 3] * sc)};
        *(u32x2_t*)(dqp + 2 * ((int64_t)qrow * p.dqs_r + 32 * dc + 8 * g + 4 * h)) = o2;
      }
  }
}

// ---------------------------------------------------------------------------
// launchers
// ---------------------------------------------------------------------------
template <class T, int D, int BS>
static int launch_bwd_t(const BwdParams& p, int phases, hipStream_t stream) {
  int rc;
  // block 32: the dQ kernel computes delta and mhat itself, so the separate pass only runs when asked for alone
  if ((phases & 1) && !(BS == 32 && (phases & 2))) {
    constexpr int RPW = 256 / (D / 8);
    const int64_t rows = (int64_t)p.B * p.H * p.Lq;
    hipLaunchKernelGGL((lmk_bwd_pre_kernel<T, D>), dim3((unsigned)((rows + RPW - 1) / RPW)), dim3(256), 0, stream, p);
    if ((rc = (int)hipGetLastError())) return rc;
  }
  if (phases & 2) {
    if constexpr (BS == 32) {
      if ((rc = launch_bwd_dq32(p, D, std::is_same<T, bf16_t>::value ? LMK_DTYPE_BF16 : LMK_DTYPE_F16, stream))) return rc;
    } else {
      using C = DqCfg<T, D, BS>;
      auto kern = lmk_bwd_dq_kernel<T, D, BS>;
      static std::atomic<uint64_t> lds_ok{0};
      if ((rc = allow_dynamic_lds(kern, C::LDS_BYTES, lds_ok))) return rc;
      hipLaunchKernelGGL(kern, dim3(p.n_qtiles * p.B * p.H), dim3(256), C::LDS_BYTES, stream, p);
      if ((rc = (int)hipGetLastError())) return rc;
    }
  }
  if (phases & 4) {
    return launch_bwd_dkdv32(p, D, BS, std::is_same<T, bf16_t>::value ? LMK_DTYPE_BF16 : LMK_DTYPE_F16, stream);
  }
  return 0;
}

template <class T>
static int launch_bwd_d(const BwdParams& p, int D, int BS, int phases, hipStream_t stream) {
  if (D == 128) {
    if (BS == 32) return launch_bwd_t<T, 128, 32>(p, phases, stream);
    if (BS == 64) return launch_bwd_t<T, 128, 64>(p, phases, stream);
    if (BS == 128) return launch_bwd_t<T, 128, 128>(p, phases, stream);
  } else if (D == 64) {
    if (BS == 32) return launch_bwd_t<T, 64, 32>(p, phases, stream);
    if (BS == 64) return launch_bwd_t<T, 64, 64>(p, phases, stream);
    if (BS == 128) return launch_bwd_t<T, 64, 128>(p, phases, stream);
  }
  return LMK_ERR_UNSUPPORTED;
}

int launch_bwd(const BwdParams& p, int D, int BS, int dtype, int phases, hipStream_t stream) {
  if (dtype == LMK_DTYPE_BF16) return launch_bwd_d<bf16_t>(p, D, BS, phases, stream);
  if (dtype == LMK_DTYPE_F16) return launch_bwd_d<f16_t>(p, D, BS, phases, stream);
  return LMK_ERR_UNSUPPORTED;
}

}  // namespace lmk
