// dK/dV kernel of the backward pass, landmark block = 32 keys.
//
// Key-stationary: a workgroup is 4 waves, one per SIMD, each owning one 32-key tile whose K and V
// fragments stay in registers as B operands.  Query tiles (32 rows of Q and of dO) and the terms
// the elementwise step needs (per row: mhat, delta; per (row, block): a, nD, dS at the landmark,
// left behind by the dQ kernel) stream through a ring of five LDS slots filled by direct
// global->LDS loads (global_load_lds_dwordx4): tile j+4 is requested while tile j is computed, no
// registers are tied up by data in flight, and vmcnt is counted by hand (five requests per wave
// and tile).  The LDS swizzle is applied on the source side: lane i of a request lands at
// +16*i, so it fetches the chunk that belongs there.
// With one wave per SIMD the schedule is the instruction stream (see `body`):
//     S, dP of tile j+1 (16 MFMA)  ||  elementwise W, dS of tile j (VALU)
//     dV^T += dO^T W, dK^T += Q^T dS of tile j (16 MFMA)
// Layout: S = Q K^T in the accumulator layout, lane = key, register r = query row
// 8*(r/4) + 4*(l/32) + r%4 of the tile.  Everything between the products is elementwise:
//     earlier block (query tile past the key tile):  W = exp2(s*c - a),  dS = W (dP - nD);
//         at the block's landmark key W = 0 and dS is the value stored by the dQ kernel
//     own block / not yet visible:  W = [key <= lim] exp2(s*c - mhat),  dS = W (dP - delta)
#include <type_traits>

#include "lmk_common.hpp"
#include "lmk_launch.hpp"

namespace lmk {

template <class T, int D>
struct Dkv32Cfg {
  static constexpr int NW = 4;
  static constexpr int NTHR = 64 * NW;
  static constexpr int CH = D / 8;
  static constexpr int KS = D / 16;
  static constexpr int DC = D / 32;
  static constexpr int ROWB = 2 * D;
  static constexpr int TILE_BYTES = 32 * ROWB;             // one query tile of Q (or of dO)
  static constexpr int STAT_BYTES = 1024 * NW;             // per wave: a, nD, dslm, mhat, delta (128 B each) + pad
  static constexpr int BUF_BYTES = 2 * TILE_BYTES + STAT_BYTES;   // Q, dO, terms
  static constexpr int NBUF = 5;                           // ring slots: 2 in use, 3 in flight
  static constexpr int RPD = 1024 / ROWB;                  // tile rows covered by one 1 KB request
  static constexpr int NDMA = 32 / RPD / NW;               // requests per wave, tile and tensor
  static constexpr int PER_TILE = 2 * NDMA + 1;            // requests per wave and ring slot
  static constexpr int CONST_OFF = NBUF * BUF_BYTES;       // 32 x 1e30f, then 32 x 0.0f
  static constexpr int LDS_BYTES = CONST_OFF + 256;
};

// One 1 KB direct global->LDS request of a wave: lane i's 16 bytes land at lds_off + 16*i.
// lds_off must be wave-uniform (it travels in M0).
__device__ __forceinline__ void dma16_s(const void* base_uniform, uint32_t voff, uint32_t lds_off) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               :: "v"(voff), "s"(base_uniform), "s"(__builtin_amdgcn_readfirstlane(lds_off)) : "memory");
}
__device__ __forceinline__ void dma16_v(const void* ptr, uint32_t lds_off) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
               :: "v"(ptr), "s"(__builtin_amdgcn_readfirstlane(lds_off)) : "memory");
}
template <int N>
__device__ __forceinline__ void wait_vmcnt() {             // s_waitcnt vmcnt(N) only (gfx9 encoding)
  __builtin_amdgcn_s_waitcnt(0x0f70 | (N & 15) | ((N >> 4) << 14));
}

template <class T, int D>
__global__ __launch_bounds__(256, 1) void lmk_bwd_dkdv32_kernel(BwdParams p) {
  using C = Dkv32Cfg<T, D>;
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int ql = lane & 31, h = lane >> 5;

  int bh, kvt;                                             // (batch*head, 128-key tile); most work first
  {
    const int bid = blockIdx.x, BH = p.B * p.H;
    if ((BH & 7) == 0) {
      const int xcd = bid & 7, j = bid >> 3, ngrp = BH >> 3;
      kvt = j / ngrp;
      bh = (j % ngrp) * 8 + xcd;
    } else {
      kvt = bid / BH;
      bh = bid % BH;
    }
  }
  const int b_ = bh / p.H, hh = bh % p.H;
  const char* qp = (const char*)p.q + 2 * (b_ * p.qs_b + hh * p.qs_h);
  const char* kp = (const char*)p.k + 2 * (b_ * p.ks_b + hh * p.ks_h);
  const char* vp = (const char*)p.v + 2 * (b_ * p.vs_b + hh * p.vs_h);
  const char* gp = (const char*)p.dout + 2 * (b_ * p.dos_b + hh * p.dos_h);
  char* dkp = (char*)p.dk + 2 * (b_ * p.dks_b + hh * p.dks_h);
  char* dvp = (char*)p.dv + 2 * (b_ * p.dvs_b + hh * p.dvs_h);

  const int nkt = p.Lk >> 5;                               // key tiles (= landmark blocks)
  const int kt = kvt * 4 + wave;
  const bool active = kt < nkt;
  const int krow = kt * 32 + ql;
  const bool lm_lane = (ql == 31);                         // this lane's key is its block's landmark
  const int PT = p.n_prefix;                               // history blocks in front of the queries
  const int nq = p.Lq >> 5;
  const float c2 = p.scale_log2;

  u32x4_t kf[C::KS], vf[C::KS];
#pragma unroll
  for (int ks = 0; ks < C::KS; ++ks) {
    u32x4_t z = {0, 0, 0, 0};
    kf[ks] = z;
    vf[ks] = z;
    if (active) {
      kf[ks] = *(const u32x4_t*)(kp + 2 * ((int64_t)krow * p.ks_r + 16 * ks + 8 * h));
      vf[ks] = *(const u32x4_t*)(vp + 2 * ((int64_t)krow * p.vs_r + 16 * ks + 8 * h));
    }
  }

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

  // ---- loaders: per ring slot every wave issues NDMA requests for Q, NDMA for dO and one for its terms
  const int j_first = max(0, kvt * 4 - PT);                // first query tile any wave here can see
  uint32_t q_vo[C::NDMA], g_vo[C::NDMA];                   // per-lane source offsets inside a tile (bytes)
#pragma unroll
  for (int d = 0; d < C::NDMA; ++d) {
    const int n = wave * C::NDMA + d;                      // request n covers tile rows RPD*n ..
    const int row = C::RPD * n + lane / C::CH, chp = lane % C::CH;
    const int f = (((row & 3) << 2) | ((row >> 2) & 3)) & (C::CH - 1);
    q_vo[d] = (uint32_t)(2 * (row * p.qs_r + 8 * (chp ^ f)));   // the chunk that belongs at LDS position chp
    g_vo[d] = (uint32_t)(2 * (row * p.dos_r + 8 * (chp ^ f)));
  }
  const float* st_src;                                     // this lane's 16 bytes of terms for query tile 0
  {
    const int arr = min(lane / 8, 4), part = lane % 8;     // 0: a, 1: nD, 2: dS at landmark, 3: mhat, 4..: delta
    const int bk = min(kt, p.n_blocks - 1);
    const int64_t plane_row = ((int64_t)bh * p.n_blocks + bk) * p.Lq, head_row = (int64_t)bh * p.Lq;
    st_src = (arr == 0) ? p.stat_a + plane_row : (arr == 1) ? p.stat_n + plane_row : (arr == 2) ? p.stat_l + plane_row
             : (arr == 3) ? p.mhat + head_row : p.delta + head_row;
    st_src += 4 * part;
  }
  auto request = [&](int slot_bytes, int j) {              // everything of query tile j -> ring slot at slot_bytes
    const int jj = min(j, nq - 1);                         // past the end: re-read the last tile (never used)
    const char* qt = qp + 2 * ((int64_t)jj * 32 * p.qs_r);
    const char* gt = gp + 2 * ((int64_t)jj * 32 * p.dos_r);
#pragma unroll
    for (int d = 0; d < C::NDMA; ++d) {
      dma16_s(qt, q_vo[d], slot_bytes + (wave * C::NDMA + d) * 1024);
      dma16_s(gt, g_vo[d], slot_bytes + C::TILE_BYTES + (wave * C::NDMA + d) * 1024);
    }
    dma16_v(st_src + 32 * jj, slot_bytes + 2 * C::TILE_BYTES + wave * 1024);
  };

  f32x16_t dkacc[C::DC], dvacc[C::DC];
#pragma unroll
  for (int dc = 0; dc < C::DC; ++dc)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      dkacc[dc][r] = 0.f;
      dvacc[dc][r] = 0.f;
    }

  auto row_tile = [&](int tileoff, const u32x4_t* bf) {    // (32 rows of the LDS tile) x (this wave's 32 keys)
    f32x16_t s;
#pragma unroll
    for (int r = 0; r < 16; ++r) s[r] = 0.f;
#pragma unroll
    for (int ks = 0; ks < C::KS; ++ks) s = mfma32<T>(*(const u32x4_t*)(smem + tileoff + koff[ks]), bf[ks], s);
    return s;
  };

  // ---- prologue: tiles j_first .. +3 requested; the first two must have landed
  request(0 * C::BUF_BYTES, j_first);
  request(1 * C::BUF_BYTES, j_first + 1);
  request(2 * C::BUF_BYTES, j_first + 2);
  request(3 * C::BUF_BYTES, j_first + 3);
  if (tid < 64) ((float*)(smem + C::CONST_OFF))[tid] = (tid < 32) ? 1e30f : 0.f;
  wait_vmcnt<2 * C::PER_TILE>();
  __syncthreads();

  f32x16_t s_cur = row_tile(0, kf), dp_cur = row_tile(C::TILE_BYTES, vf);

  // One iteration = one query tile j against this wave's key tile.  The wave issues in order, so
  // the instruction stream itself is the schedule: every MFMA is followed by a few independent
  // instructions that run while the matrix pipe is busy (a 32x32x16 MFMA occupies it for ~33
  // cycles, a VALU instruction of a lone wave issues every ~5.5); sched_barrier(0) pins the order.
  //   phase A   16 MFMA: S and dP of tile j+1        + elementwise registers 0..11 of tile j
  //   phase B1   8 MFMA: dV, dK from rows 0..15      + elementwise registers 12..15
  //   phase B2   8 MFMA: dV, dK from rows 16..31
  // MASKED = false: the query tile lies in a later block than the keys (the common case): every key
  //   is visible, W = exp2(s*c - a), dS = W (dP - nD); the landmark lane reads 1e30 for `a` (W = 0)
  //   and the stored dS as addend.
  // MASKED = true: own block or not yet visible: W = [key <= lim] exp2(s*c - mhat), dS = W (dP - delta).
  auto body = [&](auto Rc, auto Mc, int j) {
    constexpr int R = decltype(Rc)::value;
    constexpr bool MASKED = decltype(Mc)::value;
    constexpr int CUR = R * C::BUF_BYTES, NXT = ((R + 1) % C::NBUF) * C::BUF_BYTES;
    const int CST = CUR + 2 * C::TILE_BYTES + wave * 1024;  // this wave's terms: a, nD, dslm, mhat, delta

    const int dtq = PT + j;                                // the tile's own landmark block
    const int krel = 32 * (kt - dtq) + ql;                 // key position relative to the query tile's first row
    // x: exponent offset, y: subtrahend of dP, z: addend of dS  (byte offsets of 32-float arrays)
    const int xoff = (MASKED ? CST + 384 : (lm_lane ? C::CONST_OFF : CST)) + 16 * h;
    const int yoff = (MASKED ? CST + 512 : CST + 128) + 16 * h;
    const int zoff = (lm_lane ? CST + 256 : C::CONST_OFF + 128) + 16 * h;
    float4 x4[4], y4[4], z4[4];                            // fetched one register group ahead of their use
    auto load_xyz = [&](int g) {
      x4[g] = *(const float4*)(smem + xoff + 32 * g);
      y4[g] = *(const float4*)(smem + yoff + 32 * g);
      if (!MASKED) z4[g] = *(const float4*)(smem + zoff + 32 * g);
    };
    load_xyz(0);
    float w[16], ds[16];
    u32x4_t wf[2], df[2];                                  // packed B operands: rows 0..15 and 16..31
    auto elementwise = [&](int r) {                        // register r <-> query row 8*(r/4) + 4h + r%4
      const int g = r >> 2, e = r & 3;
      if (e == 0 && g < 3) load_xyz(g + 1);
      const float xa = (e == 0) ? x4[g].x : (e == 1) ? x4[g].y : (e == 2) ? x4[g].z : x4[g].w;
      const float ya = (e == 0) ? y4[g].x : (e == 1) ? y4[g].y : (e == 2) ? y4[g].z : y4[g].w;
      float ex = fast_exp2(__builtin_fmaf(s_cur[r], c2, -xa));
      if (MASKED) {
        // key visible to this query row?  the landmark row of a block looks one position to the left
        const int qloc = 8 * g + 4 * h + e;
        ex = (krel <= qloc - ((qloc == 31) ? 1 : 0)) ? ex : 0.f;
        ds[r] = ex * (dp_cur[r] - ya);
      } else {
        const float za = (e == 0) ? z4[g].x : (e == 1) ? z4[g].y : (e == 2) ? z4[g].z : z4[g].w;
        ds[r] = __builtin_fmaf(ex, dp_cur[r] - ya, za);
      }
      w[r] = ex;
      if (r & 1) {                                         // pack pairs as soon as they exist
        wf[r >> 3][(r >> 1) & 3] = pack2<T>(w[r - 1], w[r]);
        df[r >> 3][(r >> 1) & 3] = pack2<T>(ds[r - 1], ds[r]);
      }
    };

    // ---- phase A
    f32x16_t s_next, dp_next;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      s_next[r] = 0.f;
      dp_next[r] = 0.f;
    }
    constexpr int NA = 2 * C::KS;                          // MFMAs in phase A (16 for D = 128, 8 for D = 64)
    auto frag = [&](int i) {
      return *(const u32x4_t*)(smem + NXT + (i < C::KS ? 0 : C::TILE_BYTES) + koff[i < C::KS ? i : i - C::KS]);
    };
    constexpr int PF = 4;                                  // LDS reads in flight ahead of their MFMA
    u32x4_t fr[NA + PF];
#pragma unroll
    for (int i = 0; i < PF; ++i) fr[i] = frag(i);
    __builtin_amdgcn_sched_barrier(0);
    constexpr int EA = 12;                                 // elementwise registers done under phase A
#pragma unroll
    for (int i = 0; i < NA; ++i) {
      if (i + PF < NA) fr[i + PF] = frag(i + PF);
      if (i < C::KS) s_next = mfma32<T>(fr[i], kf[i], s_next);
      else dp_next = mfma32<T>(fr[i], vf[i - C::KS], dp_next);
#pragma unroll
      for (int r = (i * EA) / NA; r < ((i + 1) * EA) / NA; ++r) elementwise(r);
      __builtin_amdgcn_sched_barrier(0);
    }

    // ---- phase B: dV^T += dO^T W, dK^T += Q^T dS
    constexpr int NB = 4 * C::DC;                          // MFMAs in phase B (16 for D = 128, 8 for D = 64)
    auto trindex = [&](int n) {                            // n-th MFMA -> j2 (row half), t (0: dO, 1: Q), dc
      const int j2 = n / (2 * C::DC), t = (n / C::DC) & 1, dc = n % C::DC;
      return (j2 << 3) | (t << 2) | dc;
    };
    auto trfrag = [&](int m) {
      const int dc = m & 3, t = (m >> 2) & 1, j2 = m >> 3;
      const int base = CUR + (t == 0 ? C::TILE_BYTES : 0) + 16 * j2 * C::ROWB;
      const u32x2_t a0 = lds_read_tr(smem + base + voff[dc][0]), a1 = lds_read_tr(smem + base + voff[dc][1]);
      const u32x4_t a = {a0[0], a0[1], a1[0], a1[1]};
      return a;
    };
    u32x4_t tf[NB + PF];
#pragma unroll
    for (int n = 0; n < PF; ++n) tf[n] = trfrag(trindex(n));
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int n = 0; n < NB; ++n) {
      if (n + PF < NB) tf[n + PF] = trfrag(trindex(n + PF));
      const int m = trindex(n);
      const int dc = m & 3, t = (m >> 2) & 1, j2 = m >> 3;
      if (t == 0) dvacc[dc] = mfma32<T>(tf[n], wf[j2], dvacc[dc]);
      else dkacc[dc] = mfma32<T>(tf[n], df[j2], dkacc[dc]);
      if (n < NB / 2) {                                    // remaining elementwise registers under the first half
#pragma unroll
        for (int r = EA + (n * (16 - EA)) / (NB / 2); r < EA + ((n + 1) * (16 - EA)) / (NB / 2); ++r) elementwise(r);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    s_cur = s_next;
    dp_cur = dp_next;
  };
  auto iter = [&](auto Rc, int j) {
    constexpr int R = decltype(Rc)::value;
    request(((R + 4) % C::NBUF) * C::BUF_BYTES, j + 4);    // into the slot tile j-1 has left
    if (PT + j > kt) body(Rc, std::false_type{}, j);       // wave-uniform choice
    else body(Rc, std::true_type{}, j);
    wait_vmcnt<2 * C::PER_TILE>();                         // tile j+2 has landed (tiles j+3, j+4 may be in flight)
    __syncthreads();
  };

  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  using I2 = std::integral_constant<int, 2>;
  using I3 = std::integral_constant<int, 3>;
  using I4 = std::integral_constant<int, 4>;
  int j = j_first;
  for (; j + 4 < nq; j += 5) {
    iter(I0{}, j);
    iter(I1{}, j + 1);
    iter(I2{}, j + 2);
    iter(I3{}, j + 3);
    iter(I4{}, j + 4);
  }
  if (j < nq) iter(I0{}, j);
  if (j + 1 < nq) iter(I1{}, j + 1);
  if (j + 2 < nq) iter(I2{}, j + 2);
  if (j + 3 < nq) iter(I3{}, j + 3);
  wait_vmcnt<0>();                                         // nothing may still be writing LDS when the wave ends

  if (active) {
    const float scl = p.scale;
#pragma unroll
    for (int dc = 0; dc < C::DC; ++dc)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        u32x2_t k2 = {pack2<T>(dkacc[dc][4 * g + 0] * scl, dkacc[dc][4 * g + 1] * scl),
                      pack2<T>(dkacc[dc][4 * g + 2] * scl, dkacc[dc][4 * g + 3] * scl)};
        u32x2_t v2 = {pack2<T>(dvacc[dc][4 * g + 0], dvacc[dc][4 * g + 1]),
                      pack2<T>(dvacc[dc][4 * g + 2], dvacc[dc][4 * g + 3])};
        *(u32x2_t*)(dkp + 2 * ((int64_t)krow * p.dks_r + 32 * dc + 8 * g + 4 * h)) = k2;
        *(u32x2_t*)(dvp + 2 * ((int64_t)krow * p.dvs_r + 32 * dc + 8 * g + 4 * h)) = v2;
      }
  }
}

template <class T, int D>
static int launch_dkdv32_t(const BwdParams& p, hipStream_t stream) {
  using C = Dkv32Cfg<T, D>;
  auto kern = lmk_bwd_dkdv32_kernel<T, D>;
  static bool attr_done = false;
  if (!attr_done) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, C::LDS_BYTES);
    if (e != hipSuccess) return (int)e;
    attr_done = true;
  }
  hipLaunchKernelGGL(kern, dim3(p.n_kvtiles * p.B * p.H), dim3(C::NTHR), C::LDS_BYTES, stream, p);
  return (int)hipGetLastError();
}

int launch_bwd_dkdv32(const BwdParams& p, int D, int dtype, hipStream_t stream) {
  if (dtype == LMK_DTYPE_BF16) {
    if (D == 128) return launch_dkdv32_t<bf16_t, 128>(p, stream);
    if (D == 64) return launch_dkdv32_t<bf16_t, 64>(p, stream);
  } else if (dtype == LMK_DTYPE_F16) {
    if (D == 128) return launch_dkdv32_t<f16_t, 128>(p, stream);
    if (D == 64) return launch_dkdv32_t<f16_t, 64>(p, stream);
  }
  return LMK_ERR_UNSUPPORTED;
}

}  // namespace lmk
