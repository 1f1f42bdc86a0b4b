// Forward kernel of fused landmark attention, landmark block = 32 keys (one MFMA tile).
//
// Same mathematics and layout as lmk_fwd.hip (S^T = K Q^T in the accumulator layout, lane =
// query), organised around memory latency and pipe overlap:
//   * a workgroup is 8 waves = 256 query rows sharing one K/V stream (wave w owns landmark block
//     c0 + w), so a head's K/V is read from L2 once per 256 queries;
//   * K/V blocks (32 keys) move global -> registers -> LDS through a ring of four LDS buffers and
//     four register sets: the load of block b+6 is issued while block b is computed, which covers
//     the L2/HBM latency that a one-block lookahead leaves exposed;
//   * the S^T product of block b+1 is issued before the softmax of block b, so the matrix pipe
//     works while the VALU does the exponentials; all LDS addresses are lane constants plus
//     immediates (the ring is unrolled by four);
//   * the running maximum is lazy: the reference value Mref only moves when a landmark score
//     exceeds it by 2^8, so the accumulator is rescaled a handful of times per query instead of
//     once per block; the true maximum is tracked on the side for the saved statistics.
// Blocks below c0 are "earlier" for all eight waves (straight-line main loop); blocks c0 .. c0+7
// are handled per wave (earlier / own / not visible).
#include <type_traits>

#include "lmk_common.hpp"
#include "lmk_launch.hpp"

namespace lmk {

template <class T, int D>
struct Fwd32Cfg {
  static constexpr int NW = 8;                             // waves per workgroup
  static constexpr int NTHR = 64 * NW;
  static constexpr int QT = 32 * NW;                       // query rows per workgroup
  static constexpr int CH = D / 8;
  static constexpr int KS = D / 16;
  static constexpr int DC = D / 32;
  static constexpr int ROWB = 2 * D;
  static constexpr int BLK_BYTES = 32 * ROWB;              // one block of K (or of V)
  static constexpr int BUF_BYTES = 2 * BLK_BYTES;          // K then V
  static constexpr int NBUF = 4;
  static constexpr int CPB = 32 * CH;                      // 16-byte chunks per block and tensor
  static constexpr int LDS_BYTES = NBUF * BUF_BYTES;
  static constexpr float LAZY = 8.0f;                      // log2 headroom before Mref moves
};

template <class T, int D>
__global__ __launch_bounds__(512, 2) void lmk_fwd32_kernel(FwdParams p) {
  using C = Fwd32Cfg<T, D>;
  extern __shared__ __align__(16) unsigned char smem[];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int ql = lane & 31, h = lane >> 5;

  const int n_qt = (p.Lq + C::QT - 1) / C::QT;
  int bh, qtile;
  {
    const int bid = blockIdx.x, BH = p.B * p.H;
    if ((BH & 7) == 0) {                                   // all workgroups of a head on one XCD, longest first
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
  char* op = (char*)p.o + 2 * (b_ * p.os_b + hh * p.os_h);

  const int c0 = p.n_prefix + qtile * C::NW;               // landmark block of wave 0's queries
  const int cblk = c0 + wave;
  const int q0 = qtile * C::QT + wave * 32;
  const int qrow = q0 + ql;
  const int nkb = (p.Lk + 31) >> 5;                        // key blocks that exist
  const int nblk = min(nkb, c0 + C::NW);                   // blocks this workgroup walks
  const float c2 = p.scale_log2;

  u32x4_t qf[C::KS];
#pragma unroll
  for (int ks = 0; ks < C::KS; ++ks) {
    u32x4_t z = {0, 0, 0, 0};
    qf[ks] = z;
    if (qrow < p.Lq) qf[ks] = *(const u32x4_t*)(qp + 2 * ((int64_t)qrow * p.qs_r + 16 * ks + 8 * h));
  }

  // lane-constant LDS offsets inside a 32-row tile (tile_off only looks at row & 15)
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

  // ---- block loader: thread tid moves chunk tid of K and of V (threads >= CPB idle when D = 64)
  const bool ld_on = tid < C::CPB;
  const int ld_row = tid / C::CH, ld_ch = tid % C::CH;
  const int ld_lds = tile_off<D>(ld_row, ld_ch);
  u32x4_t kreg[C::NBUF], vreg[C::NBUF];
  auto gload = [&](auto Sc, int blk) {
    constexpr int S = decltype(Sc)::value;
    const int key = blk * 32 + ld_row;
    u32x4_t z = {0, 0, 0, 0};
    kreg[S] = z;
    vreg[S] = z;
    if (ld_on && blk < nblk && key < p.Lk) {
      kreg[S] = *(const u32x4_t*)(kp + 2 * ((int64_t)key * p.ks_r + 8 * ld_ch));
      vreg[S] = *(const u32x4_t*)(vp + 2 * ((int64_t)key * p.vs_r + 8 * ld_ch));
    }
  };
  auto lstore = [&](auto Sc) {                              // register set S -> LDS buffer S
    constexpr int S = decltype(Sc)::value;
    if (ld_on) {
      *(u32x4_t*)(smem + S * C::BUF_BYTES + ld_lds) = kreg[S];
      *(u32x4_t*)(smem + S * C::BUF_BYTES + C::BLK_BYTES + ld_lds) = vreg[S];
    }
  };

  auto qk_tile = [&](int tileoff) {
    f32x16_t s;
#pragma unroll
    for (int r = 0; r < 16; ++r) s[r] = 0.f;
#pragma unroll
    for (int ks = 0; ks < C::KS; ++ks) s = mfma32<T>(*(const u32x4_t*)(smem + tileoff + koff[ks]), qf[ks], s);
    return s;
  };

  float Mref = -INFINITY, Mtrue = -INFINITY, lsum = 0.f;   // log2 domain
  f32x16_t acc[C::DC];
#pragma unroll
  for (int dc = 0; dc < C::DC; ++dc)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[dc][r] = 0.f;

  auto pv_tile = [&](int vtileoff, const float* w) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      u32x4_t wf = {pack2<T>(w[8 * j + 0], w[8 * j + 1]), pack2<T>(w[8 * j + 2], w[8 * j + 3]),
                    pack2<T>(w[8 * j + 4], w[8 * j + 5]), pack2<T>(w[8 * j + 6], w[8 * j + 7])};
#pragma unroll
      for (int dc = 0; dc < C::DC; ++dc) {
        const u32x2_t a0 = lds_read_tr(smem + vtileoff + 16 * j * C::ROWB + voff[dc][0]);
        const u32x2_t a1 = lds_read_tr(smem + vtileoff + 16 * j * C::ROWB + voff[dc][1]);
        const u32x4_t a = {a0[0], a0[1], a1[0], a1[1]};
        acc[dc] = mfma32<T>(a, wf, acc[dc]);
      }
    }
  };
  // move the reference maximum when a new score x (log2 domain) outgrows it; rare
  auto lazy_max = [&](float x) {
    Mtrue = fmaxf(Mtrue, x);
    if (__any(x > Mref + C::LAZY)) {
      const float Mnew = (x > Mref + C::LAZY) ? x : Mref;
      const float alpha = fast_exp2(Mref - Mnew);          // 1 for lanes that keep their reference
      Mref = Mnew;
      lsum *= alpha;
#pragma unroll
      for (int dc = 0; dc < C::DC; ++dc)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[dc][r] *= alpha;
    }
  };
  // earlier block: weights gate * P_local from raw scores s; t_lm = its landmark score (log2 domain)
  auto earlier_weights = [&](const f32x16_t& s, float t_lm, float* w) {
    float m0 = (h == 0) ? s[15] : -INFINITY;
#pragma unroll
    for (int r = 0; r < 15; ++r) m0 = fmaxf(m0, s[r]);
    const float mloc = pair_max(m0) * c2;
    float den = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      float e = fast_exp2(__builtin_fmaf(s[r], c2, -mloc));
      if (r == 15) e = (h == 0) ? e : 0.f;
      w[r] = e;
      den += e;
    }
    den = pair_sum(den);
    const float gate = fast_exp2(t_lm - Mref);
    lsum += gate;
    const float f = gate * fast_rcp(den);
#pragma unroll
    for (int r = 0; r < 16; ++r) w[r] *= f;
  };

  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  using I2 = std::integral_constant<int, 2>;
  using I3 = std::integral_constant<int, 3>;

  // ---- prologue: blocks 0, 1 in LDS; blocks 2..5 in flight in register sets 2, 3, 0, 1
  gload(I0{}, 0);
  gload(I1{}, 1);
  gload(I2{}, 2);
  gload(I3{}, 3);
  lstore(I0{});
  lstore(I1{});
  gload(I0{}, 4);
  gload(I1{}, 5);
  __syncthreads();

  // ---- main loop: blocks 0 .. c0-1 are earlier blocks for all waves
  f32x16_t s_cur;
  if (c0 > 0) s_cur = qk_tile(0);
  auto iter = [&](auto Rc, int b) {
    constexpr int R = decltype(Rc)::value;
    constexpr int CUR = R * C::BUF_BYTES, NXT = ((R + 1) % 4) * C::BUF_BYTES;
    using FIL = std::integral_constant<int, (R + 2) % 4>;
    lstore(FIL{});                                         // block b+2 (loaded four iterations ago)
    gload(FIL{}, b + 6);
    const float t_lm = pair_hi(s_cur[15]) * c2;
    lazy_max(t_lm);
    const f32x16_t s_next = qk_tile(NXT);                  // block b+1
    float w[16];
    earlier_weights(s_cur, t_lm, w);
    pv_tile(CUR + C::BLK_BYTES, w);
    s_cur = s_next;
    __syncthreads();
  };
  for (int b = 0; b < c0; b += 4) {
    iter(I0{}, b);
    if (b + 1 < c0) iter(I1{}, b + 1);
    if (b + 2 < c0) iter(I2{}, b + 2);
    if (b + 3 < c0) iter(I3{}, b + 3);
  }

  // ---- per-wave blocks c0 .. nblk-1 (ring positions continue; register set = block % 4)
  auto tail = [&](auto Rc, int blk) {
    constexpr int R = decltype(Rc)::value;
    constexpr int CUR = R * C::BUF_BYTES;
    using FIL = std::integral_constant<int, (R + 2) % 4>;
    lstore(FIL{});
    gload(FIL{}, blk + 6);
    if (blk <= cblk) {
      const f32x16_t s = qk_tile(CUR);
      float w[16];
      if (blk < cblk) {
        const float t_lm = pair_hi(s[15]) * c2;
        lazy_max(t_lm);
        earlier_weights(s, t_lm, w);
      } else {
        const int lim = ql - ((ql == 31) ? 1 : 0);         // the landmark query looks one to the left
        float x[16], mt = -INFINITY;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int key = 8 * (r >> 2) + 4 * h + (r & 3);
          x[r] = (key <= lim) ? s[r] * c2 : -INFINITY;
          mt = fmaxf(mt, x[r]);
        }
        lazy_max(pair_max(mt));
        float sum = 0.f;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          w[r] = fast_exp2(x[r] - Mref);
          sum += w[r];
        }
        lsum += pair_sum(sum);
      }
      pv_tile(CUR + C::BLK_BYTES, w);
    }
    __syncthreads();
  };
  for (int blk = c0; blk < nblk; ++blk) {
    switch (blk & 3) {
      case 0: tail(I0{}, blk); break;
      case 1: tail(I1{}, blk); break;
      case 2: tail(I2{}, blk); break;
      default: tail(I3{}, blk); break;
    }
  }

  if (qrow < p.Lq) {
    const float inv = 1.0f / lsum;
#pragma unroll
    for (int dc = 0; dc < C::DC; ++dc)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        u32x2_t o2 = {pack2<T>(acc[dc][4 * g + 0] * inv, acc[dc][4 * g + 1] * inv),
                      pack2<T>(acc[dc][4 * g + 2] * inv, acc[dc][4 * g + 3] * inv)};
        *(u32x2_t*)(op + 2 * ((int64_t)qrow * p.os_r + 32 * dc + 8 * g + 4 * h)) = o2;
      }
    if (h == 0) {                                          // statistics relative to the true maximum
      p.L[(int64_t)bh * p.Lq + qrow] = lsum * fast_exp2(Mref - Mtrue);
      p.M[(int64_t)bh * p.Lq + qrow] = Mtrue * kLn2;
    }
  }
}

template <class T, int D>
static int launch_fwd32_t(const FwdParams& p, hipStream_t stream) {
  using C = Fwd32Cfg<T, D>;
  auto kern = lmk_fwd32_kernel<T, D>;
  static std::atomic<uint64_t> lds_ok{0};
  if (int rc = allow_dynamic_lds(kern, C::LDS_BYTES, lds_ok)) return rc;
  const int n_qt = (p.Lq + C::QT - 1) / C::QT;
  hipLaunchKernelGGL(kern, dim3(n_qt * p.B * p.H), dim3(C::NTHR), C::LDS_BYTES, stream, p);
  return (int)hipGetLastError();
}

int launch_fwd32(const FwdParams& p, int D, int dtype, hipStream_t stream) {
  if (dtype == LMK_DTYPE_BF16) {
    if (D == 128) return launch_fwd32_t<bf16_t, 128>(p, stream);
    if (D == 64) return launch_fwd32_t<bf16_t, 64>(p, stream);
  } else if (dtype == LMK_DTYPE_F16) {
    if (D == 128) return launch_fwd32_t<f16_t, 128>(p, stream);
    if (D == 64) return launch_fwd32_t<f16_t, 64>(p, stream);
  }
  return LMK_ERR_UNSUPPORTED;
}

}  // namespace lmk
