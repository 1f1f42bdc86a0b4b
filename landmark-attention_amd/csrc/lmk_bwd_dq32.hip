// dQ kernel of the backward pass (plus the per-block terms for the dK/dV kernel), landmark
// block = 32 keys.
//
// Query-stationary, S^T layout (lane = query): a workgroup is 8 waves = 256 query rows, two waves
// per SIMD; wave w owns landmark block c0 + w and keeps Q and dO fragments (B operands) and its
// dQ^T accumulator in registers.  K/V blocks stream through a ring of six LDS slots filled by
// direct global->LDS loads (tile k+4 is requested while tile k is computed; vmcnt is counted by
// hand, two requests per wave and tile).  Per block a wave does three things:
//     X  S^T = K Q^T and dP^T = V dO^T                       16 MFMA, row fragments from LDS
//     Y  local softmax, gate, nD, dS (and the terms a, nD, dS_landmark)      vector ALU only
//     Z  dQ^T += K^T dS^T                                     8 MFMA, transposed fragments
// The two waves of a SIMD would run X, Y, Z in lock-step behind the per-block barrier and fight
// for the same pipe, so the upper four waves run half a period late: between two barriers the
// lower waves do X(k) Y(k) Z(k) while the upper waves do Z(k-1) X(k) Y(k); one group's vector
// phase then overlaps the other group's matrix phase.  A slot stays valid for two periods.
// The per-block terms are collected in LDS and flushed to global memory every 8 blocks, so that
// stores do not sit between the hand-counted loads.
#include <type_traits>

#include "lmk_common.hpp"
#include "lmk_launch.hpp"

namespace lmk {

template <class T, int D>
struct Dq32Cfg {
  static constexpr int NW = 8;
  static constexpr int NTHR = 64 * NW;
  static constexpr int QT = 32 * NW;
  static constexpr int CH = D / 8;
  static constexpr int KS = D / 16;
  static constexpr int DC = D / 32;
  static constexpr int ROWB = 2 * D;
  static constexpr int BLK_BYTES = 32 * ROWB;              // one block of K (or of V)
  static constexpr int BUF_BYTES = 2 * BLK_BYTES;          // K then V
  static constexpr int NBUF = 4;                           // ring slots: 2 in use, 2 in flight
  static constexpr int DIST = 2;
  static constexpr int RPD = 1024 / ROWB;                  // block rows covered by one 1 KB request
  static constexpr int NREQ = 2 * (32 / RPD);              // requests per block (K and V)
  static constexpr int PER_TILE = NREQ / NW;               // requests per wave and block
  static constexpr int FL = 8;                             // blocks between flushes of the per-block terms
  static constexpr int STAT_WAVE = 3 * FL * 32 * 4;        // a, nD, dS_landmark for FL blocks x 32 queries
  static constexpr int GO_OFF = NBUF * BUF_BYTES;          // per wave: its 32 rows of dO (B operand of dP^T)
  static constexpr int STAT_OFF = GO_OFF + NW * BLK_BYTES;
  static constexpr int LDS_BYTES = STAT_OFF + NW * STAT_WAVE;
  static constexpr bool SKEW = false;
};

__device__ __forceinline__ void dq_dma16(const void* base_uniform, uint32_t voff, uint32_t lds_off) {
  // one 1 KB request of a wave: lane i's 16 bytes land at lds_off + 16*i (lds_off travels in M0)
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               :: "v"(voff), "s"(base_uniform), "s"(__builtin_amdgcn_readfirstlane(lds_off)) : "memory");
}
template <int N>
__device__ __forceinline__ void dq_wait_vmcnt() {          // s_waitcnt vmcnt(N) only (gfx9 encoding)
  __builtin_amdgcn_s_waitcnt(0x0f70 | (N & 15) | ((N >> 4) << 14));
}

template <class T, int D>
__global__ __launch_bounds__(512, 2) void lmk_bwd_dq32_kernel(BwdParams p) {
  using C = Dq32Cfg<T, D>;
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ql = lane & 31, h = lane >> 5;

  const int n_qt = (p.Lq + C::QT - 1) / C::QT;
  int bh, qtile;
  {
    const int bid = blockIdx.x, BH = p.B * p.H;
    if ((BH & 7) == 0) {
      const int xcd = bid & 7, j = bid >> 3, ngrp = BH >> 3;
      qtile = n_qt - 1 - j / ngrp;
      bh = (j % ngrp) * 8 + xcd;
    } else {
      qtile = n_qt - 1 - bid / BH;
      bh = bid % BH;
    }
  }
  const int b_ = bh / p.H, hh = bh % p.H;
  const char* qp = (const char*)p.q + 2 * (b_ * p.qs_b + hh * p.qs_h);
  const char* kp = (const char*)p.k + 2 * (b_ * p.ks_b + hh * p.ks_h);
  const char* vp = (const char*)p.v + 2 * (b_ * p.vs_b + hh * p.vs_h);
  const char* gp = (const char*)p.dout + 2 * (b_ * p.dos_b + hh * p.dos_h);
  char* dqp = (char*)p.dq + 2 * (b_ * p.dqs_b + hh * p.dqs_h);

  const int c0 = p.n_prefix + qtile * C::NW;
  const int cblk = c0 + wave;
  const int q0 = qtile * C::QT + wave * 32;
  const int qrow = q0 + ql;
  const bool rowok = qrow < p.Lq;                          // Lq is a multiple of 32 here: all or none of a wave
  const int nkb = p.Lk >> 5;
  const int nblk = min(nkb, c0 + C::NW);
  const float c2 = p.scale_log2;

  u32x4_t qf[C::KS];
#pragma unroll
  for (int ks = 0; ks < C::KS; ++ks) {
    u32x4_t z = {0, 0, 0, 0};
    qf[ks] = z;
    if (rowok) qf[ks] = *(const u32x4_t*)(qp + 2 * ((int64_t)qrow * p.qs_r + 16 * ks + 8 * h));
  }
  const float mhat = rowok ? p.mhat[(int64_t)bh * p.Lq + qrow] : 0.f;
  const float delta = rowok ? p.delta[(int64_t)bh * p.Lq + qrow] : 0.f;

  int koff[C::KS];
#pragma unroll
  for (int ks = 0; ks < C::KS; ++ks) koff[ks] = tile_off<D>(ql, 2 * ks + h);
  int voff[C::DC][2];
  {
    const int i = lane & 15, g2 = (lane >> 4) & 1;
#pragma unroll
    for (int dc = 0; dc < C::DC; ++dc) {
      const int col = 32 * dc + 16 * g2 + 4 * (i & 3);
#pragma unroll
      for (int hf = 0; hf < 2; ++hf)
        voff[dc][hf] = tile_off<D>(4 * h + (i >> 2) + 8 * hf, col >> 3) + ((col >> 2) & 1) * 8;
    }
  }

  // ---- requests: wave w issues request n = w*PER_TILE + d of each block (K first, then V)
  uint32_t r_vo[C::PER_TILE];
  int r_lds[C::PER_TILE];
  bool r_isv[C::PER_TILE];
#pragma unroll
  for (int d = 0; d < C::PER_TILE; ++d) {
    const int n = wave * C::PER_TILE + d;
    const int per = 32 / C::RPD;                           // requests per tensor
    const int part = n % per;
    r_isv[d] = n >= per;
    const int row = C::RPD * part + lane / C::CH, chp = lane % C::CH;
    const int f = (((row & 3) << 2) | ((row >> 2) & 3)) & (C::CH - 1);
    const int64_t rs = r_isv[d] ? p.vs_r : p.ks_r;
    r_vo[d] = (uint32_t)(2 * (row * rs + 8 * (chp ^ f)));
    r_lds[d] = (r_isv[d] ? C::BLK_BYTES : 0) + part * 1024;
  }
  auto request = [&](int slot_bytes, int blk) {
    const int bb = min(blk, nkb - 1);                      // past the end: re-read the last block (never used)
#pragma unroll
    for (int d = 0; d < C::PER_TILE; ++d) {
      const char* base = r_isv[d] ? vp + 2 * ((int64_t)bb * 32 * p.vs_r) : kp + 2 * ((int64_t)bb * 32 * p.ks_r);
      dq_dma16(base, r_vo[d], slot_bytes + r_lds[d]);
    }
  };

  f32x16_t acc[C::DC];
#pragma unroll
  for (int dc = 0; dc < C::DC; ++dc)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[dc][r] = 0.f;

  unsigned char* stat_lds = smem + C::STAT_OFF + wave * C::STAT_WAVE;   // [plane 3][FL][32] floats
  auto flush = [&](int blast) {                            // write blocks 8*(blast/8) .. blast of this wave's terms
    const int b0 = blast & ~(C::FL - 1), bi = lane >> 3, part = lane & 7;
    if (b0 + bi <= blast) {
      const int64_t dst = ((int64_t)bh * p.n_blocks + b0 + bi) * p.Lq + q0 + 4 * part;
      *(float4*)(p.stat_a + dst) = *(const float4*)(stat_lds + ((0 * C::FL + bi) * 32 + 4 * part) * 4);
      *(float4*)(p.stat_n + dst) = *(const float4*)(stat_lds + ((1 * C::FL + bi) * 32 + 4 * part) * 4);
      *(float4*)(p.stat_l + dst) = *(const float4*)(stat_lds + ((2 * C::FL + bi) * 32 + 4 * part) * 4);
    }
  };

  // ---- the three stages
  f32x16_t sc, dp;
  u32x4_t dsf[2];                                           // packed dS^T of the block: keys 0..15, 16..31
  auto stage_x = [&](int slot) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      sc[r] = 0.f;
      dp[r] = 0.f;
    }
#pragma unroll
    for (int ks = 0; ks < C::KS; ++ks) {
      sc = mfma32<T>(*(const u32x4_t*)(smem + slot + koff[ks]), qf[ks], sc);
      dp = mfma32<T>(*(const u32x4_t*)(smem + slot + C::BLK_BYTES + koff[ks]),
                     *(const u32x4_t*)(smem + C::GO_OFF + wave * C::BLK_BYTES + koff[ks]), dp);
    }
  };
  auto pack_ds = [&](const float* ds) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      u32x4_t f = {pack2<T>(ds[8 * j + 0], ds[8 * j + 1]), pack2<T>(ds[8 * j + 2], ds[8 * j + 3]),
                   pack2<T>(ds[8 * j + 4], ds[8 * j + 5]), pack2<T>(ds[8 * j + 6], ds[8 * j + 7])};
      dsf[j] = f;
    }
  };
  auto stage_y = [&](int blk) {
    float ds[16];
    if (blk < cblk) {
      // earlier block: key of register r is 8*(r/4) + 4h + r%4; the landmark is (r = 15, h = 1)
      const float s_last = sc[15];
      float mx = (h == 0) ? s_last : -INFINITY;
#pragma unroll
      for (int r = 0; r < 15; ++r) mx = fmaxf(mx, sc[r]);
      mx = pair_max(mx);
      const float t_lm = pair_hi(s_last) * c2;
      const float mloc = mx * c2;
      float den = 0.f, spd = 0.f;
      float e[16];
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        float x = fast_exp2(__builtin_fmaf(sc[r], c2, -mloc));
        if (r == 15) x = (h == 0) ? x : 0.f;
        e[r] = x;
        den += x;
        spd = __builtin_fmaf(x, dp[r], spd);
      }
      den = pair_sum(den);
      spd = pair_sum(spd);
      const float invden = fast_rcp(den);
      const float nD = spd * invden;
      const float glog = t_lm - mhat;                      // log2 of the normalised gate
      const float g = fast_exp2(glog);
      const float f = g * invden;
      const float dslm = g * (nD - delta);
      if (h == 0) {
        const int bi = blk & (C::FL - 1);
        *(float*)(stat_lds + ((0 * C::FL + bi) * 32 + ql) * 4) = mloc + fast_log2(den) - glog;
        *(float*)(stat_lds + ((1 * C::FL + bi) * 32 + ql) * 4) = nD;
        *(float*)(stat_lds + ((2 * C::FL + bi) * 32 + ql) * 4) = dslm;
      }
#pragma unroll
      for (int r = 0; r < 16; ++r) ds[r] = e[r] * f * (dp[r] - nD);
      if (h == 1) ds[15] = dslm;
      if ((blk & (C::FL - 1)) == C::FL - 1 || blk == cblk - 1) flush(blk);
    } else {
      const int lim = ql - ((ql == 31) ? 1 : 0);           // the landmark query looks one to the left
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int key = 8 * (r >> 2) + 4 * h + (r & 3);
        const float pr = (key <= lim) ? fast_exp2(__builtin_fmaf(sc[r], c2, -mhat)) : 0.f;
        ds[r] = pr * (dp[r] - delta);
      }
    }
    pack_ds(ds);
  };
  auto stage_z = [&](int slot) {
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int dc = 0; dc < C::DC; ++dc) {
        const u32x2_t a0 = lds_read_tr(smem + slot + 16 * j * C::ROWB + voff[dc][0]);
        const u32x2_t a1 = lds_read_tr(smem + slot + 16 * j * C::ROWB + voff[dc][1]);
        const u32x4_t a = {a0[0], a0[1], a1[0], a1[1]};
        acc[dc] = mfma32<T>(a, dsf[j], acc[dc]);
      }
  };

  // ---- prologue: this wave's dO rows -> LDS; blocks 0 .. DIST-1 requested; block 0 must have landed
  {
    const int qb = min(q0, p.Lq - 32);                     // inactive waves re-read valid rows (never used)
    const char* gt = gp + 2 * ((int64_t)qb * p.dos_r);
#pragma unroll
    for (int n = 0; n < 32 / C::RPD; ++n) {
      const int row = C::RPD * n + lane / C::CH, chp = lane % C::CH;
      const int f = (((row & 3) << 2) | ((row >> 2) & 3)) & (C::CH - 1);
      dq_dma16(gt, (uint32_t)(2 * (row * p.dos_r + 8 * (chp ^ f))), C::GO_OFF + wave * C::BLK_BYTES + n * 1024);
    }
  }
#pragma unroll
  for (int t = 0; t < C::DIST; ++t) request(t * C::BUF_BYTES, t);
  dq_wait_vmcnt<(C::DIST - 1) * C::PER_TILE>();
  __syncthreads();

  const bool late = C::SKEW && wave >= C::NW / 2;          // upper waves run half a period behind
  const int periods = nblk + 1;
  auto period = [&](auto Rc, int k) {
    constexpr int R = decltype(Rc)::value;
    constexpr int CUR = R * C::BUF_BYTES, PRV = ((R + C::NBUF - 1) % C::NBUF) * C::BUF_BYTES;
    request(((R + C::DIST) % C::NBUF) * C::BUF_BYTES, k + C::DIST);   // into the slot block k-2 has left
    if (!late) {
      if (k < nblk && k <= cblk && rowok) {
        stage_x(CUR);
        stage_y(k);
        stage_z(CUR);
      }
    } else {
      if (k >= 1 && k - 1 <= cblk && rowok) stage_z(PRV);
      if (k < nblk && k <= cblk && rowok) {
        stage_x(CUR);
        stage_y(k);
      }
    }
    dq_wait_vmcnt<(C::DIST - 1) * C::PER_TILE>();          // block k+1 has landed (k+2 may be in flight)
    __syncthreads();
  };
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  using I2 = std::integral_constant<int, 2>;
  using I3 = std::integral_constant<int, 3>;
  for (int k = 0; k < periods; k += 4) {
    period(I0{}, k);
    if (k + 1 < periods) period(I1{}, k + 1);
    if (k + 2 < periods) period(I2{}, k + 2);
    if (k + 3 < periods) period(I3{}, k + 3);
  }
  dq_wait_vmcnt<0>();                                      // nothing may still be writing LDS when the wave ends

  if (rowok) {
    const float scl = p.scale;
#pragma unroll
    for (int dc = 0; dc < C::DC; ++dc)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        u32x2_t o2 = {pack2<T>(acc[dc][4 * g + 0] * scl, acc[dc][4 * g + 1] * scl),
                      pack2<T>(acc[dc][4 * g + 2] * scl, acc[dc][4 * g + 3] * scl)};
        *(u32x2_t*)(dqp + 2 * ((int64_t)qrow * p.dqs_r + 32 * dc + 8 * g + 4 * h)) = o2;
      }
  }
}

template <class T, int D>
static int launch_dq32_t(const BwdParams& p, hipStream_t stream) {
  using C = Dq32Cfg<T, D>;
  auto kern = lmk_bwd_dq32_kernel<T, D>;
  static bool attr_done = false;
  if (!attr_done) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, C::LDS_BYTES);
    if (e != hipSuccess) return (int)e;
    attr_done = true;
  }
  const int n_qt = (p.Lq + C::QT - 1) / C::QT;
  hipLaunchKernelGGL(kern, dim3(n_qt * p.B * p.H), dim3(C::NTHR), C::LDS_BYTES, stream, p);
  return (int)hipGetLastError();
}

int launch_bwd_dq32(const BwdParams& p, int D, int dtype, hipStream_t stream) {
  if (dtype == LMK_DTYPE_BF16) {
    if (D == 128) return launch_dq32_t<bf16_t, 128>(p, stream);
    if (D == 64) return launch_dq32_t<bf16_t, 64>(p, stream);
  } else if (dtype == LMK_DTYPE_F16) {
    if (D == 128) return launch_dq32_t<f16_t, 128>(p, stream);
    if (D == 64) return launch_dq32_t<f16_t, 64>(p, stream);
  }
  return LMK_ERR_UNSUPPORTED;
}

}  // namespace lmk
