// Forward kernel of fused landmark attention for gfx950.
//
// Replaces `_fwd_kernel` of the reference (llama/ltriton/flash_landmark_attention.py:6-122).
// One workgroup = 4 waves = 128 consecutive query rows; every wave owns 32 queries and
// keeps S^T = K Q^T tiles in the MFMA C layout (lane = query, registers = keys), so the
// landmark grouped softmax never leaves a lane pair:
//   earlier block b:  local softmax over its BS-1 normal keys, gate = online softmax over
//                     the landmark scores, acc = acc*alpha + (gate * P_local) V
//   own block:        plain causal online softmax joined to the same running (M, l)
// K and V stream through LDS in stages of SK = max(BS, 64) keys, double buffered;
// V is kept row-major and transposed on the way out of LDS by ds_read_b64_tr_b16.
#include <cstdlib>

#include "lmk_common.hpp"
#include "lmk_launch.hpp"

namespace lmk {

template <class T, int D, int BS>
struct FwdCfg {
  static constexpr int NT = BS / 32;                    // 32-key tiles per landmark block
  static constexpr int NB = (BS >= 64) ? 1 : 64 / BS;   // landmark blocks per LDS stage
  static constexpr int SK = NB * BS;                    // keys per stage
  static constexpr int ROWB = 2 * D;
  static constexpr int CH = D / 8;                      // 16-byte chunks per row
  static constexpr int TILE_BYTES = SK * ROWB;          // one stage of K (or of V)
  static constexpr int NCH = SK * CH / 256;             // chunks per thread per tensor per stage
  static constexpr int KS = D / 16;                     // MFMA k-steps over the head dim
  static constexpr int DC = D / 32;                     // 32-wide output chunks of the head dim
  static constexpr int LDS_BYTES = 4 * TILE_BYTES;      // 2 buffers x (K, V)
};

template <class T, int D, int BS>
__global__ __launch_bounds__(256, (BS >= 128 ? 1 : 2)) void lmk_fwd_kernel(FwdParams p) {
  using C = FwdCfg<T, D, BS>;
  extern __shared__ __align__(16) unsigned char smem[];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int ql = lane & 31, h = lane >> 5;

  // ---- workgroup -> (batch*head, 128-row query tile); heavy tiles first, one head per XCD slot
  int bh, qtile;
  {
    const int bid = blockIdx.x;
    const int BH = p.B * p.H;
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
  char* op = (char*)p.o + 2 * (b * p.os_b + hh * p.os_h);

  const int q0 = qtile * 128 + wave * 32;               // first query row of this wave
  const int dt = p.n_prefix * C::NT + (q0 >> 5);        // its diagonal 32-key tile (absolute)
  const int cblk = dt / C::NT, tsub = dt % C::NT;       // its landmark block and sub-tile
  const bool active = q0 < p.Lq;
  const int qrow = q0 + ql;

  // ---- Q fragments (B operand): query qrow, head dims 16*ks + 8h .. +7
  u32x4_t qf[C::KS];
#pragma unroll
  for (int ks = 0; ks < C::KS; ++ks) {
    u32x4_t z = {0, 0, 0, 0};
    qf[ks] = z;
    if (qrow < p.Lq) qf[ks] = *(const u32x4_t*)(qp + 2 * ((int64_t)qrow * p.qs_r + 16 * ks + 8 * h));
  }

  // ---- stage loader: thread handles chunks id = tid + 256*i -> (row = id / CH, chunk = id % CH)
  const int tiles_needed = min((p.Lk + 31) >> 5, p.n_prefix * C::NT + qtile * 4 + 4);
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

  // ---- running state (log2 domain): M = max of the global bucket, l = its sum
  float Mrun = -INFINITY, lrun = 0.f;
  f32x16_t acc[C::DC];
#pragma unroll
  for (int dc = 0; dc < C::DC; ++dc)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[dc][r] = 0.f;

  const float c2 = p.scale_log2;

  auto qk_tile = [&](const unsigned char* kb, int rb) {
    f32x16_t s;
#pragma unroll
    for (int r = 0; r < 16; ++r) s[r] = 0.f;
#pragma unroll
    for (int ks = 0; ks < C::KS; ++ks) s = mfma32<T>(load_row_frag<D>(kb, rb, ks, lane), qf[ks], s);
    return s;
  };
  auto pv_tile = [&](const unsigned char* vb, int rb, const float* w) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      u32x4_t wf = {pack2<T>(w[8 * j + 0], w[8 * j + 1]), pack2<T>(w[8 * j + 2], w[8 * j + 3]),
                    pack2<T>(w[8 * j + 4], w[8 * j + 5]), pack2<T>(w[8 * j + 6], w[8 * j + 7])};
#pragma unroll
      for (int dc = 0; dc < C::DC; ++dc) acc[dc] = mfma32<T>(load_tr_frag<D>(vb, rb, j, dc, lane), wf, acc[dc]);
    }
  };
  auto rescale = [&](float alpha) {
    if (__any(alpha != 1.0f)) {
#pragma unroll
      for (int dc = 0; dc < C::DC; ++dc)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[dc][r] *= alpha;
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
        const int blk = s * C::NB + jb;                 // absolute landmark block
        const int rb0 = jb * BS;                        // its first LDS row
        if (blk < cblk) {
          // ---------------- earlier block: local softmax gated by its landmark
          f32x16_t sc[C::NT];
#pragma unroll
          for (int u = 0; u < C::NT; ++u) sc[u] = qk_tile(kb, rb0 + 32 * u);
          // key of register r in tile u: 32u + 8*(r/4) + 4h + r%4; the landmark is (NT-1, r=15, h=1)
          const float s_last = sc[C::NT - 1][15];
          float mx = (h == 0) ? s_last : -INFINITY;
#pragma unroll
          for (int u = 0; u < C::NT; ++u)
#pragma unroll
            for (int r = 0; r < 16; ++r)
              if (!(u == C::NT - 1 && r == 15)) mx = fmaxf(mx, sc[u][r]);
          mx = pair_max(mx);
          const float t_lm = pair_hi(s_last) * c2;      // landmark score, log2 domain
          const float mloc = mx * c2;
          float den = 0.f;
#pragma unroll
          for (int u = 0; u < C::NT; ++u)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              float e = fast_exp2(__builtin_fmaf(sc[u][r], c2, -mloc));
              if (u == C::NT - 1 && r == 15) e = (h == 0) ? e : 0.f;
              sc[u][r] = e;
              den += e;
            }
          den = pair_sum(den);
          const float Mnew = fmaxf(Mrun, t_lm);
          const float alpha = fast_exp2(Mrun - Mnew);
          const float gate = fast_exp2(t_lm - Mnew);
          lrun = lrun * alpha + gate;
          Mrun = Mnew;
          rescale(alpha);
          const float f = gate * fast_rcp(den);
#pragma unroll
          for (int u = 0; u < C::NT; ++u) {
            float w[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) w[r] = sc[u][r] * f;
            pv_tile(vb, rb0 + 32 * u, w);
          }
        } else if (blk == cblk) {
          // ---------------- own block: causal tiles 0..tsub join the global bucket
          const int lim = ql - ((tsub == C::NT - 1 && ql == 31) ? 1 : 0);  // landmark query looks one left
#pragma unroll
          for (int u = 0; u < C::NT; ++u) {
            if (u <= tsub) {
              f32x16_t sc = qk_tile(kb, rb0 + 32 * u);
              float x[16];
              float mt = -INFINITY;
#pragma unroll
              for (int r = 0; r < 16; ++r) {
                const int key = 8 * (r >> 2) + 4 * h + (r & 3);
                x[r] = (u < tsub || key <= lim) ? sc[r] * c2 : -INFINITY;
                mt = fmaxf(mt, x[r]);
              }
              mt = pair_max(mt);
              const float Mnew = fmaxf(Mrun, mt);
              const float alpha = fast_exp2(Mrun - Mnew);
              float sum = 0.f;
#pragma unroll
              for (int r = 0; r < 16; ++r) {
                x[r] = fast_exp2(x[r] - Mnew);
                sum += x[r];
              }
              sum = pair_sum(sum);
              lrun = lrun * alpha + sum;
              Mrun = Mnew;
              rescale(alpha);
              pv_tile(vb, rb0 + 32 * u, x);
            }
          }
        }
      }
    }
    if (s + 1 < n_stages) store_stage(buf ^ 1);
    __syncthreads();
  }

  // ---- epilogue: out = acc / l, statistics in natural-log units like the reference
  if (active && qrow < p.Lq) {
    const float inv = 1.0f / lrun;
#pragma unroll
    for (int dc = 0; dc < C::DC; ++dc)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        u32x2_t o2 = {pack2<T>(acc[dc][4 * g + 0] * inv, acc[dc][4 * g + 1] * inv),
                      pack2<T>(acc[dc][4 * g + 2] * inv, acc[dc][4 * g + 3] * inv)};
        *(u32x2_t*)(op + 2 * ((int64_t)qrow * p.os_r + 32 * dc + 8 * g + 4 * h)) = o2;
      }
    if (h == 0) {
      p.L[(int64_t)bh * p.Lq + qrow] = lrun;
      p.M[(int64_t)bh * p.Lq + qrow] = Mrun * kLn2;
    }
  }
}

template <class T, int D, int BS>
static int launch_fwd_t(const FwdParams& p, hipStream_t stream) {
  using C = FwdCfg<T, D, BS>;
  auto kern = lmk_fwd_kernel<T, D, BS>;
  static std::atomic<uint64_t> lds_ok{0};
  if (int rc = allow_dynamic_lds(kern, C::LDS_BYTES, lds_ok)) return rc;
  const int grid = p.n_qtiles * p.B * p.H;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(256), C::LDS_BYTES, stream, p);
  return (int)hipGetLastError();
}

template <class T>
static int launch_fwd_d(const FwdParams& p, int D, int BS, hipStream_t stream) {
  if (D == 128) {                                          // block 32 has its own kernel (lmk_fwd32.hip)
    if (BS == 64) return launch_fwd_t<T, 128, 64>(p, stream);
    if (BS == 128) return launch_fwd_t<T, 128, 128>(p, stream);
  } else if (D == 64) {
    if (BS == 64) return launch_fwd_t<T, 64, 64>(p, stream);
    if (BS == 128) return launch_fwd_t<T, 64, 128>(p, stream);
  }
  return LMK_ERR_UNSUPPORTED;
}

int launch_fwd(const FwdParams& p, int D, int BS, int dtype, hipStream_t stream) {
  if (BS == 32) return launch_fwd32(p, D, dtype, stream);
  if (dtype == LMK_DTYPE_BF16) return launch_fwd_d<bf16_t>(p, D, BS, stream);
  if (dtype == LMK_DTYPE_F16) return launch_fwd_d<f16_t>(p, D, BS, stream);
  return LMK_ERR_UNSUPPORTED;
}

}  // namespace lmk
