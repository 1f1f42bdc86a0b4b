// Backward kernels of fused landmark attention for gfx950.
//
// Replace `_bwd_preprocess` and `_bwd_kernel` of the reference
// (llama/ltriton/flash_landmark_attention.py:125-149, :152-305).  The reference runs one
// program per (batch, head) and read-modify-writes dQ in global memory; here the work is
// split so that every accumulator stays in registers and no atomics are needed:
//
//   pre    delta = rowsum(O * dO),  mhat = M*log2(e) + log2(L)          (per query row; the dQ kernels do
//          this in their prologue, the separate kernel exists for timing the phases one by one)
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
__global__ __launch_bounds__(256) void lmk_bwd_pre_kernel(BwdParams p, int block_slots) {
  constexpr int LPR = D / 8;          // lanes per row (16 bytes each)
  constexpr int RPW = 256 / LPR;      // rows per workgroup
  const int tid = threadIdx.x;
  const int64_t row = (int64_t)blockIdx.x * RPW + tid / LPR;
  const int64_t total = (int64_t)p.B * p.H * p.Lq;
  float sum = 0.f;
  int64_t li = row;                                         // index of the row in L and M; -1: a slot without a token
  if (row < total) {
    const int bh = (int)(row / p.Lq);
    int qi = (int)(row % p.Lq);
    if (p.Lq_real > 0) {                                    // token layout: the workspace rows are slots
      const int* seg_q = p.seg != nullptr ? p.seg + p.n_prefix : nullptr;   // the queries' first block
      qi = block_slots == 64 ? slot_to_token_row<64>(qi, p.n_real, p.n_full_q, seg_q)
                             : slot_to_token_row<128>(qi, p.n_real, p.n_full_q, seg_q);
      li = qi < 0 ? -1 : (int64_t)bh * p.Lq_real + qi;
    }
    if (qi >= 0) {
      const int b = bh / p.H, hh = bh % p.H;
      const int d0 = 8 * (tid % LPR);
      const u32x4_t o4 = *(const u32x4_t*)((const char*)p.o + 2 * (b * p.os_b + hh * p.os_h + (int64_t)qi * p.os_r + d0));
      const u32x4_t g4 = *(const u32x4_t*)((const char*)p.dout + 2 * (b * p.dos_b + hh * p.dos_h + (int64_t)qi * p.dos_r + d0));
#pragma unroll
      for (int i = 0; i < 4; ++i)
        sum += unpack_lo<T>(o4[i]) * unpack_lo<T>(g4[i]) + unpack_hi<T>(o4[i]) * unpack_hi<T>(g4[i]);
    }
  }
#pragma unroll
  for (int m = LPR / 2; m >= 1; m >>= 1) sum += __shfl_xor(sum, m, 64);
  if (row < total && (tid % LPR) == 0) {
    p.delta[row] = sum;
    p.mhat[row] = li < 0 ? 1e30f : p.M[li] * kLog2e + fast_log2(p.L[li]);
  }
}

// ---------------------------------------------------------------------------
// dq (+ per-block statistics), landmark blocks of 64 and 128 keys
// ---------------------------------------------------------------------------
// A workgroup is 8 waves = 256 query rows, two waves per SIMD; a wave keeps the fragments of its 32
// rows of Q and dO and its dQ^T accumulator in registers.  One stage is one landmark block: its K and
// V rows come into one of two LDS buffers by direct global->LDS loads (no staging registers: the kernel
// has to stay inside 256 registers for two waves to share a SIMD), requested one stage ahead, each wave
// fetching its share; one barrier per stage.  The block's local softmax needs all its scores before any
// weight is final, so the S^T tiles of the whole block stay in registers; with four tiles per block the
// dP^T tiles do not fit beside them and are computed twice (once for nD, once for dS).
template <class T, int D, int BS>
struct DqCfg {
  static constexpr int NT = BS / 32;                       // MFMA tiles per landmark block
  static constexpr int NW = 8;
  static constexpr int CH = D / 8;
  static constexpr int KS = D / 16;
  static constexpr int DC = D / 32;
  static constexpr int ROWB = 2 * D;
  static constexpr int TILE_BYTES = BS * ROWB;             // K (or V) of one block
  static constexpr int STAGE_BYTES = 2 * TILE_BYTES;       // K, then V
  static constexpr int LDS_BYTES = 2 * STAGE_BYTES;
  static constexpr int RPD = 1024 / ROWB;                  // rows covered by one 1 KB request
  static constexpr int NREQ = 2 * BS / RPD;                // requests per stage
  static constexpr int PER_WAVE = NREQ / NW;
  static constexpr bool KEEP_DP = NT <= 2;                 // dP^T tiles kept beside the S^T tiles
  static_assert(NREQ % NW == 0, "every wave issues the same number of requests");
};

// One 1 KB direct global->LDS request of a wave: lane i's 16 bytes land at lds_off + 16*i.
// lds_off must be wave-uniform (it travels in M0).
__device__ __forceinline__ void dq_dma16(const void* base_uniform, uint32_t voff, uint32_t lds_off) {
  const uint64_t b = (uint64_t)base_uniform;
  const uint64_t base = ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(b >> 32)) << 32) |
                        (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)b);
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               :: "v"(voff), "s"(base), "s"(__builtin_amdgcn_readfirstlane(lds_off)) : "memory");
}

// VIRT: tensors in token layout (p.Lq_real > 0); a template parameter because the slot arithmetic costs the
// slot-layout instantiations registers they do not have.
// SEG (with VIRT): blocks of unequal length, looked up in p.seg -- a template parameter for the same reason.
// PLAIN (without VIRT): every block has BS tokens in its BS slots -- no padding slots to mask; the masks' scalar
// registers and the branch are what it saves the common case.
template <class T, int D, int BS, bool VIRT, bool SEG = false, bool PLAIN = false>
__global__ __launch_bounds__(512, 2) void lmk_bwd_dq_kernel(BwdParams p) {
  static_assert(VIRT || !SEG, "the table describes tensors in token layout");
  static_assert(!PLAIN || !VIRT, "plain: the tensors' rows are the kernel's rows");
  using C = DqCfg<T, D, BS>;
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ql = lane & 31, h = lane >> 5;

  const int nq256 = (p.Lq + 255) >> 8;
  int bh, qt;                                              // (batch*head, 256-row query tile); most work first
  {
    const int bid = blockIdx.x, BH = p.B * p.H;
    if ((BH & 7) == 0) {
      const int xcd = bid & 7, j = bid >> 3, ngrp = BH >> 3;
      qt = nq256 - 1 - j / ngrp;
      bh = (j % ngrp) * 8 + xcd;
    } else {
      qt = nq256 - 1 - bid / BH;
      bh = bid % BH;
    }
  }
  const int b = bh / p.H, hh = bh % p.H;
  const char* qp = (const char*)p.q + 2 * (b * p.qs_b + hh * p.qs_h);
  const char* kp = (const char*)p.k + 2 * (b * p.ks_b + hh * p.ks_h);
  const char* vp = (const char*)p.v + 2 * (b * p.vs_b + hh * p.vs_h);
  const char* gp = (const char*)p.dout + 2 * (b * p.dos_b + hh * p.dos_h);
  char* dqp = (char*)p.dq + 2 * (b * p.dqs_b + hh * p.dqs_h);

  const int q0 = qt * 256 + wave * 32;
  const int dt = p.n_prefix * C::NT + (q0 >> 5);
  const int cblk = dt / C::NT, tsub = dt % C::NT;          // the wave's own block and its tile inside it
  const bool active = q0 < p.Lq;                           // Lq is a multiple of the block: whole tiles only
  const int qrow = q0 + ql;
  // token layout: the tensors' rows are tokens, the kernel's rows (and the workspace's) are slots.  A slot without
  // a token is a query row of zeros with mhat = 1e30: its gate, its weights and every term it leaves for the dK/dV
  // kernel come out as exact zeros (a = 1e30), whatever that kernel reads for its Q and dO rows.
  constexpr bool virt = VIRT;
  const int nfull_k = p.n_full_k;
  const int* seg_k = SEG ? p.seg : nullptr;
  const int* seg_q = SEG ? p.seg + p.n_prefix : nullptr;   // the queries' first block
  const int qtok = !active ? -1 : (virt ? slot_to_token_row<BS>(qrow, p.n_real, p.n_full_q, seg_q) : qrow);

  u32x4_t qf[C::KS], gf[C::KS];
#pragma unroll
  for (int ks = 0; ks < C::KS; ++ks) {
    u32x4_t z = {0, 0, 0, 0};
    qf[ks] = z;
    gf[ks] = z;
    if (qtok >= 0) {
      qf[ks] = *(const u32x4_t*)(qp + 2 * ((int64_t)qtok * p.qs_r + 16 * ks + 8 * h));
      gf[ks] = *(const u32x4_t*)(gp + 2 * ((int64_t)qtok * p.dos_r + 16 * ks + 8 * h));
    }
  }
  // row terms (the reference's _bwd_preprocess, flash_landmark_attention.py:125-149): delta = rowsum(O * dO)
  // from the dO fragments already in registers, mhat = M*log2(e) + log2(L); left in the workspace for the
  // dK/dV kernel as well
  float mhat = 0.f, delta = 0.f;
  if (active) {
    float sum = 0.f;
    mhat = 1e30f;
    if (qtok >= 0) {
      const char* orow = (const char*)p.o + 2 * (b * p.os_b + hh * p.os_h + (int64_t)qtok * p.os_r);
#pragma unroll
      for (int ks = 0; ks < C::KS; ++ks) {
        const u32x4_t o4 = *(const u32x4_t*)(orow + 2 * (16 * ks + 8 * h));
#pragma unroll
        for (int i = 0; i < 4; ++i)
          sum += unpack_lo<T>(o4[i]) * unpack_lo<T>(gf[ks][i]) + unpack_hi<T>(o4[i]) * unpack_hi<T>(gf[ks][i]);
      }
      const int64_t li = (int64_t)bh * (virt ? p.Lq_real : p.Lq) + qtok;   // L, M follow the tensors' layout
      mhat = p.M[li] * kLog2e + fast_log2(p.L[li]);
    }
    delta = pair_sum(sum);
    const int64_t ri = (int64_t)bh * p.Lq + qrow;
    if (h == 0) {
      p.delta[ri] = delta;
      p.mhat[ri] = mhat;
    }
  }

  // stages = blocks up to the own block of the workgroup's last query tile
  const int last_q0 = min(qt * 256 + 224, p.Lq - 32);
  const int n_stages = min(p.n_blocks, (p.n_prefix * C::NT + (last_q0 >> 5)) / C::NT + 1);

  // this wave's requests of a stage: request r covers rows RPD*(r % (BS/RPD)) .. of K (r < BS/RPD) or V.
  // The LDS swizzle is applied on the source side: lane i lands at +16*i, i.e. row i/CH, chunk position
  // i%CH, so it fetches the chunk tile_off() stores there.
  uint32_t src[C::PER_WAVE];                               // per-lane byte offset inside the (batch, head) slice of K or V
  const int n_k = BS / C::RPD;                             // requests that fetch K rows; the rest fetch V rows
#pragma unroll
  for (int i = 0; i < C::PER_WAVE; ++i) {
    const int r = wave * C::PER_WAVE + i;
    const bool is_v = r >= n_k;
    const int row = C::RPD * (r % n_k) + lane / C::CH, cp = lane % C::CH;
    const int f = (((row & 3) << 2) | ((row >> 2) & 3)) & (C::CH - 1);
    src[i] = (uint32_t)(2 * ((int64_t)row * (is_v ? p.vs_r : p.ks_r) + 8 * (cp ^ f)));
  }
  const uint32_t step_k = (uint32_t)(2 * (int64_t)BS * p.ks_r), step_v = (uint32_t)(2 * (int64_t)BS * p.vs_r);
  int blk_req = 0;                                         // block the next request fetches
  auto request = [&](int buf) __attribute__((always_inline)) {   // next block in key order -> buffer buf
#pragma unroll
    for (int i = 0; i < C::PER_WAVE; ++i) {
      const int r = wave * C::PER_WAVE + i;
      const bool is_v = r >= n_k;                          // wave-uniform
      const int dst = buf * C::STAGE_BYTES + (is_v ? C::TILE_BYTES : 0) + C::RPD * (r % n_k) * C::ROWB;
      if (virt) {                                          // the slot's token row, worked out per request
        const int row = C::RPD * (r % n_k) + lane / C::CH, cp = lane % C::CH;
        const int f = (((row & 3) << 2) | ((row >> 2) & 3)) & (C::CH - 1);
        const int tok = slot_to_token_row_clamped<BS>(blk_req * BS + row, p.n_real, nfull_k, seg_k);
        dq_dma16(is_v ? vp : kp, (uint32_t)(2 * ((int64_t)tok * (is_v ? p.vs_r : p.ks_r) + 8 * (cp ^ f))), dst);
      } else {
        dq_dma16(is_v ? vp : kp, src[i], dst);
        src[i] += is_v ? step_v : step_k;
      }
    }
    ++blk_req;
  };

  f32x16_t acc[C::DC];
#pragma unroll
  for (int dc = 0; dc < C::DC; ++dc)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[dc][r] = 0.f;
  const float c2 = p.scale_log2;
  // A block narrower than BS tokens is stored with its n_norm normal keys in front, its landmark in the
  // last slot and padding in between: slots n_norm .. BS-2 hold no key and no query may see them.
  // With blocks of unequal length n_norm is the stage's block's (uniform over the workgroup).
  const int n_norm_all = p.n_real - 1;
  const bool padded = !PLAIN && (n_norm_all < BS - 1 || seg_k != nullptr);   // uniform over the launch

  // LDS byte offsets of this lane's operand fragments inside a 32-row tile: the swizzle repeats every 16
  // rows, so a tile at row 32u is the same offsets plus 32u rows -- an immediate of the LDS instruction
  int koff[C::KS];
#pragma unroll
  for (int ks = 0; ks < C::KS; ++ks) {
    koff[ks] = tile_off<D>(ql, 2 * ks + h);
    // the compiler must not know the value's range: it would turn "offset + constant" into an OR computed by a
    // vector instruction per read; as a plain sum the constant stays the read's immediate offset
    asm volatile("" : "+v"(koff[ks]));
  }
  int voff[C::DC][2];
  {
    const int i = lane & 15, g2 = (lane >> 4) & 1;
#pragma unroll
    for (int dc = 0; dc < C::DC; ++dc) {
      const int col = 32 * dc + 16 * g2 + 4 * (i & 3);
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) {
        voff[dc][hf] = tile_off<D>(4 * h + (i >> 2) + 8 * hf, col >> 3) + ((col >> 2) & 1) * 8;
        asm volatile("" : "+v"(voff[dc][hf]));             // as for koff
      }
    }
  }
  // The wave issues in order, so in the earlier blocks' code the instruction stream is the schedule: every LDS
  // operand is asked for two MFMAs ahead of its use and the order is pinned.
  // (32 rows each of NTL consecutive LDS tiles) x (this wave's 32 queries)
  auto row_tiles = [&](int tile_bytes, const u32x4_t* bf, f32x16_t* out, auto ntl_c) __attribute__((always_inline)) {
    constexpr int NX = decltype(ntl_c)::value * C::KS, PFX = 2;
    u32x4_t fk[NX];
#pragma unroll
    for (int n = 0; n < PFX; ++n) fk[n] = lds_ld128(tile_bytes + 32 * (n / C::KS) * C::ROWB + koff[n % C::KS]);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int n = 0; n < NX; ++n) {
      if (n + PFX < NX) fk[n + PFX] = lds_ld128(tile_bytes + 32 * ((n + PFX) / C::KS) * C::ROWB + koff[(n + PFX) % C::KS]);
      const int u = n / C::KS, ks = n % C::KS;
      if (ks == 0) {
#pragma unroll
        for (int r = 0; r < 16; ++r) out[u][r] = 0.f;
      }
      out[u] = mfma32<T>(fk[n], bf[ks], out[u]);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // dQ^T += (K tiles)^T dS^T for NTL consecutive tiles, dS = e f (dP - nD) in slices of 16 keys: a slice is formed
  // and packed under the MFMAs of the one before.  u0: first tile's index in the block (the landmark is the last
  // tile's last key); dP of tile u0 + i is d[d_stride * i].
  auto dq_tiles = [&](int tile_bytes, int u0, const f32x16_t* e, const f32x16_t* d, int d_stride, float f, float nD,
                      float dslm, auto ntl_c) __attribute__((always_inline)) {
    constexpr int NTL = decltype(ntl_c)::value, NZ = NTL * 2 * C::DC, PFZ = 2;
    auto zload = [&](int n) __attribute__((always_inline)) {
      const int sl = n / C::DC, dc = n % C::DC;
      const int base = tile_bytes + 16 * sl * C::ROWB;
      const u32x2_t a0 = lds_ld_tr(base + voff[dc][0]), a1 = lds_ld_tr(base + voff[dc][1]);
      const u32x4_t a = {a0[0], a0[1], a1[0], a1[1]};
      return a;
    };
    auto slice = [&](int sl) __attribute__((always_inline)) {
      const int i = sl >> 1, j = sl & 1;
      float ds[8];
#pragma unroll
      for (int r = 0; r < 8; ++r) ds[r] = e[i][8 * j + r] * f * (d[d_stride * i][8 * j + r] - nD);
      if (j == 1 && u0 + i == C::NT - 1 && h == 1) ds[7] = dslm;
      const u32x4_t wf = {pack2<T>(ds[0], ds[1]), pack2<T>(ds[2], ds[3]), pack2<T>(ds[4], ds[5]), pack2<T>(ds[6], ds[7])};
      return wf;
    };
    u32x4_t zf[NZ], wf[2];
#pragma unroll
    for (int n = 0; n < PFZ; ++n) zf[n] = zload(n);
    wf[0] = slice(0);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int n = 0; n < NZ; ++n) {
      if (n + PFZ < NZ) zf[n + PFZ] = zload(n + PFZ);
      const int sl = n / C::DC, dc = n % C::DC;
      acc[dc] = mfma32<T>(zf[n], wf[sl & 1], acc[dc]);
      if (dc == 0 && sl + 1 < 2 * NTL) wf[(sl + 1) & 1] = slice(sl + 1);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  auto row_tile = [&](int tile_bytes, const u32x4_t* bf) __attribute__((always_inline)) {   // one tile, the compiler's order
    f32x16_t s;
#pragma unroll
    for (int r = 0; r < 16; ++r) s[r] = 0.f;
#pragma unroll
    for (int ks = 0; ks < C::KS; ++ks) s = mfma32<T>(lds_ld128(tile_bytes + koff[ks]), bf[ks], s);
    return s;
  };
  auto dq_tile = [&](int tile_bytes, const float* ds) __attribute__((always_inline)) {   // dQ^T += (K tile)^T dS^T
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      u32x4_t wf = {pack2<T>(ds[8 * j + 0], ds[8 * j + 1]), pack2<T>(ds[8 * j + 2], ds[8 * j + 3]),
                    pack2<T>(ds[8 * j + 4], ds[8 * j + 5]), pack2<T>(ds[8 * j + 6], ds[8 * j + 7])};
#pragma unroll
      for (int dc = 0; dc < C::DC; ++dc) {
        const int base = tile_bytes + 16 * j * C::ROWB;
        const u32x2_t a0 = lds_ld_tr(base + voff[dc][0]), a1 = lds_ld_tr(base + voff[dc][1]);
        const u32x4_t a = {a0[0], a0[1], a1[0], a1[1]};
        acc[dc] = mfma32<T>(a, wf, acc[dc]);
      }
    }
  };

  const uint32_t stat_row = 4u * (uint32_t)qrow;
  // ---------------- earlier block s at LDS byte addresses kb (K rows) / vb (V rows)
  auto earlier_block = [&](const int kb, const int vb, const int s) __attribute__((always_inline)) {
    int n_norm = n_norm_all;
    if constexpr (SEG) n_norm = block_normal_keys<BS>(s, p.n_real, nfull_k, seg_k);
    float gscale = 1.f;                                    // group dropout: this block's factor for this query row
    if constexpr (VIRT)
      if (p.group_scale != nullptr && qtok >= 0) gscale = p.group_scale[(int64_t)bh * p.gs_bh + (int64_t)s * p.gs_blk + qtok];
    f32x16_t sc[C::NT], dp[C::KEEP_DP ? C::NT : 1];
    row_tiles(kb, qf, sc, std::integral_constant<int, C::NT>{});
    if (padded) {                                          // padding slots leave the local softmax
#pragma unroll
      for (int u = 0; u < C::NT; ++u)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int kl = 32 * u + 8 * (r >> 2) + 4 * h + (r & 3);
          if (kl >= n_norm && kl < BS - 1) sc[u][r] = -INFINITY;
        }
    }
    const float s_last = sc[C::NT - 1][15];
    float mx = (h == 0) ? s_last : -INFINITY;
    float t_lm = 0.f, mloc = 0.f, den = 0.f, spd = 0.f;
    if constexpr (C::KEEP_DP) {
      // dP^T does not depend on S^T: at head dim 64 its MFMAs carry the local softmax of the scores, a slice behind
      // each -- first the maximum (one slice per tile), then the exponentials and their sum.  (At head dim 128 the
      // same placement measured 7 % slower than the softmax behind the MFMAs, in the compiler's order.)
      constexpr bool UNDER = D == 64;
      constexpr int NX = C::NT * C::KS, PFX = 2, NEXP = NX - C::NT, PER = (16 * C::NT + NEXP - 1) / NEXP;
      auto ywork = [&](int n) __attribute__((always_inline)) {
        if (n < C::NT) {
#pragma unroll
          for (int r = 0; r < 16; ++r)
            if (!(n == C::NT - 1 && r == 15)) mx = fmaxf(mx, sc[n][r]);
          if (n == C::NT - 1) {
            mx = pair_max(mx);
            t_lm = pair_hi(s_last) * c2;
            mloc = mx * c2;
          }
        } else {
#pragma unroll
          for (int i = (n - C::NT) * PER; i < (n - C::NT + 1) * PER && i < 16 * C::NT; ++i) {
            const int u = i >> 4, r = i & 15;
            float e = fast_exp2(__builtin_fmaf(sc[u][r], c2, -mloc));
            if (u == C::NT - 1 && r == 15) e = (h == 0) ? e : 0.f;
            sc[u][r] = e;
            den += e;
          }
        }
      };
      u32x4_t fk[NX];
#pragma unroll
      for (int n = 0; n < PFX; ++n) fk[n] = lds_ld128(vb + 32 * (n / C::KS) * C::ROWB + koff[n % C::KS]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int n = 0; n < NX; ++n) {
        if (n + PFX < NX) fk[n + PFX] = lds_ld128(vb + 32 * ((n + PFX) / C::KS) * C::ROWB + koff[(n + PFX) % C::KS]);
        const int u = n / C::KS, ks = n % C::KS;
        if (ks == 0) {
#pragma unroll
          for (int r = 0; r < 16; ++r) dp[u][r] = 0.f;
        }
        dp[u] = mfma32<T>(fk[n], gf[ks], dp[u]);
        if constexpr (UNDER) ywork(n);
        __builtin_amdgcn_sched_barrier(0);
      }
      if constexpr (!UNDER) {
#pragma unroll
        for (int n = 0; n < NX; ++n) ywork(n);
      }
#pragma unroll
      for (int u = 0; u < C::NT; ++u)
#pragma unroll
        for (int r = 0; r < 16; ++r) spd = __builtin_fmaf(sc[u][r], dp[u][r], spd);
    } else {
#pragma unroll
      for (int u = 0; u < C::NT; ++u)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          if (!(u == C::NT - 1 && r == 15)) mx = fmaxf(mx, sc[u][r]);
      mx = pair_max(mx);
      t_lm = pair_hi(s_last) * c2;
      mloc = mx * c2;
#pragma unroll
      for (int u = 0; u < C::NT; ++u) {
        row_tiles(vb + 32 * u * C::ROWB, gf, dp, std::integral_constant<int, 1>{});
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          float e = fast_exp2(__builtin_fmaf(sc[u][r], c2, -mloc));
          if (u == C::NT - 1 && r == 15) e = (h == 0) ? e : 0.f;
          sc[u][r] = e;
          den += e;
          spd = __builtin_fmaf(e, dp[0][r], spd);
        }
      }
    }
    den = pair_sum(den);
    spd = pair_sum(spd);
    const float invden = fast_rcp(den);
    const float nD = spd * invden;
    const float glog = t_lm - mhat;                        // log2 of the normalised gate
    const float g = fast_exp2(glog);
    // out_i = .. + gscale * g * (P V): the weights carry the factor, the landmark's dS sees it through nD
    const float f = g * invden * gscale;
    const float dslm = g * (gscale * nD - delta);          // dS at the block's landmark key
    if (h == 0) {                                          // a scalar base per (head, block) plus the row's 32-bit offset
      const int64_t sb = 4 * ((int64_t)bh * p.n_blocks + s) * p.Lq;
      *(float*)((char*)p.stat_a + sb + stat_row) = gscale > 0.f ? mloc + fast_log2(den) - glog - fast_log2(gscale) : 1e30f;
      *(float*)((char*)p.stat_n + sb + stat_row) = nD;
      *(float*)((char*)p.stat_l + sb + stat_row) = dslm;
    }
    if constexpr (C::KEEP_DP) {
      dq_tiles(kb, 0, sc, dp, 1, f, nD, dslm, std::integral_constant<int, C::NT>{});
    } else {
#pragma unroll
      for (int u = 0; u < C::NT; ++u) {
        row_tiles(vb + 32 * u * C::ROWB, gf, dp, std::integral_constant<int, 1>{});
        dq_tiles(kb + 32 * u * C::ROWB, u, sc + u, dp, 0, f, nD, dslm, std::integral_constant<int, 1>{});
      }
    }
  };

  // Stages in front of the workgroup's first query block are earlier blocks for every wave: they run two at a
  // time without a branch, the LDS addresses of both buffers as immediates of the instructions.
  const int first_cblk = (p.n_prefix * C::NT + qt * 8) / C::NT;   // wave 0's own block: the least of the workgroup's
  const int s_uniform = min(first_cblk, n_stages - 1);
  auto uniform_stage = [&](auto buf_c, int s) __attribute__((always_inline)) {
    constexpr int buf = decltype(buf_c)::value;
    __builtin_amdgcn_s_waitcnt(0x0f70);                    // vmcnt(0): this wave's share of stage s has landed
    __syncthreads();                                       // ... and everyone's; stage s-1 has been consumed
    request(buf ^ 1);
    if (active) earlier_block(buf * C::STAGE_BYTES, buf * C::STAGE_BYTES + C::TILE_BYTES, s);
  };

  request(0);
  int s = 0;
  for (; s + 2 <= s_uniform; s += 2) {
    uniform_stage(std::integral_constant<int, 0>{}, s);
    uniform_stage(std::integral_constant<int, 1>{}, s + 1);
  }
  for (; s < n_stages; ++s) {
    const int buf = s & 1;
    __builtin_amdgcn_s_waitcnt(0x0f70);
    __syncthreads();
    if (s + 1 < n_stages) request(buf ^ 1);
    const int kb = buf * C::STAGE_BYTES, vb = kb + C::TILE_BYTES;   // LDS byte addresses (the dynamic array starts at 0)
    if (!active) continue;
    if (s < cblk) {
      earlier_block(kb, vb, s);
    } else if (s == cblk) {
      int n_norm = n_norm_all;
      if constexpr (SEG) n_norm = block_normal_keys<BS>(s, p.n_real, nfull_k, seg_k);
      const int lim = ql - ((tsub == C::NT - 1 && ql == 31) ? 1 : 0);
#pragma unroll
      for (int u = 0; u < C::NT; ++u) {
        if (u <= tsub) {
          f32x16_t sc = row_tile(kb + 32 * u * C::ROWB, qf);
          f32x16_t d = row_tile(vb + 32 * u * C::ROWB, gf);
          float ds[16];
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int key = 8 * (r >> 2) + 4 * h + (r & 3);
            const int kl = 32 * u + key;
            const bool pad = padded && kl >= n_norm && kl < BS - 1;   // only the landmark query could reach one
            const float pr = ((u < tsub || key <= lim) && !pad) ? fast_exp2(__builtin_fmaf(sc[r], c2, -mhat)) : 0.f;
            ds[r] = pr * (d[r] - delta);
          }
          dq_tile(kb + 32 * u * C::ROWB, ds);
        }
      }
    }
  }

  // dQ leaves as row segments through the wave's share of the stage buffer the last stage did not use: every wave
  // is past the barrier in front of the last stage, so nobody reads that buffer and no request targets it
  if (active) {
    static_assert(C::STAGE_BYTES / C::NW >= 2048, "32 rows x 32 columns of 16 bits per wave");
    const int free_buf = (n_stages & 1) * C::STAGE_BYTES;  // the last stage sits in buffer (n_stages - 1) & 1
    store_tile_rows<T, C::DC>(acc, p.scale, free_buf + wave * (C::STAGE_BYTES / C::NW),
                              [&](int r) __attribute__((always_inline)) -> char* {
      const int tok = virt ? slot_to_token_row<BS>(q0 + r, p.n_real, p.n_full_q, seg_q) : q0 + r;
      return tok < 0 ? nullptr : dqp + 2 * ((int64_t)tok * p.dqs_r);
    });
  }
}

// ---------------------------------------------------------------------------
// launchers
// ---------------------------------------------------------------------------
template <class T, int D, int BS>
static int launch_bwd_t(const BwdParams& p, int phases, hipStream_t stream) {
  int rc;
  // the dQ kernels compute delta and mhat themselves, so the separate pass only runs when asked for alone
  if ((phases & 1) && !(phases & 2)) {
    constexpr int RPW = 256 / (D / 8);
    const int64_t rows = (int64_t)p.B * p.H * p.Lq;
    hipLaunchKernelGGL((lmk_bwd_pre_kernel<T, D>), dim3((unsigned)((rows + RPW - 1) / RPW)), dim3(256), 0, stream, p, BS);
    if ((rc = (int)hipGetLastError())) return rc;
  }
  if (phases & 2) {
    if constexpr (BS == 32) {
      if ((rc = launch_bwd_dq32(p, D, std::is_same<T, bf16_t>::value ? LMK_DTYPE_BF16 : LMK_DTYPE_F16, stream))) return rc;
    } else {
      using C = DqCfg<T, D, BS>;
      const dim3 grid(((p.Lq + 255) / 256) * p.B * p.H);
      if (p.Lq_real > 0 && p.seg != nullptr) {
        auto kern = lmk_bwd_dq_kernel<T, D, BS, true, true>;
        static std::atomic<uint64_t> lds_ok{0};
        if ((rc = allow_dynamic_lds(kern, C::LDS_BYTES, lds_ok))) return rc;
        hipLaunchKernelGGL(kern, grid, dim3(64 * C::NW), C::LDS_BYTES, stream, p);
      } else if (p.Lq_real > 0) {
        auto kern = lmk_bwd_dq_kernel<T, D, BS, true>;
        static std::atomic<uint64_t> lds_ok{0};
        if ((rc = allow_dynamic_lds(kern, C::LDS_BYTES, lds_ok))) return rc;
        hipLaunchKernelGGL(kern, grid, dim3(64 * C::NW), C::LDS_BYTES, stream, p);
      } else if (p.n_real == BS) {
        auto kern = lmk_bwd_dq_kernel<T, D, BS, false, false, true>;
        static std::atomic<uint64_t> lds_ok{0};
        if ((rc = allow_dynamic_lds(kern, C::LDS_BYTES, lds_ok))) return rc;
        hipLaunchKernelGGL(kern, grid, dim3(64 * C::NW), C::LDS_BYTES, stream, p);
      } else {
        auto kern = lmk_bwd_dq_kernel<T, D, BS, false>;
        static std::atomic<uint64_t> lds_ok{0};
        if ((rc = allow_dynamic_lds(kern, C::LDS_BYTES, lds_ok))) return rc;
        hipLaunchKernelGGL(kern, grid, dim3(64 * C::NW), C::LDS_BYTES, stream, p);
      }
      if ((rc = (int)hipGetLastError())) return rc;
    }
  }
  if (phases & 4) {
    if (p.ds_tiles != nullptr) {
      if (BS != 32) return LMK_ERR_UNSUPPORTED;
      return launch_bwd_dkdv32_handover(p, D, std::is_same<T, bf16_t>::value ? LMK_DTYPE_BF16 : LMK_DTYPE_F16, stream);
    }
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
