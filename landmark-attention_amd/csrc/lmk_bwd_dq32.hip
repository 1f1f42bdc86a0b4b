// dQ kernel of the backward pass (plus the per-block terms for the dK/dV kernel), landmark
// block = 32 keys.
//
// Query-stationary, S^T layout (lane = query): a workgroup is 8 waves = 256 query rows, two waves
// per SIMD; wave w owns landmark block c0 + w and keeps its Q fragments (B operands) and its dQ^T
// accumulator in registers; its 32 rows of dO sit in LDS (both in registers would pass the register
// budget).  K/V blocks stream through a ring of four LDS slots filled by direct global->LDS loads
// (block k+3 is requested while block k is computed; vmcnt is counted by hand, two requests per
// wave and block).  Per block a wave does three things:
//     X  S^T = K Q^T and dP^T = V dO^T                       16 MFMA, row fragments from LDS
//     Y  local softmax, gate, nD, dS (and the terms a, nD, dS_landmark)      vector ALU only
//     Z  dQ^T += K^T dS^T                                     8 MFMA, transposed fragments
// X of block k+1 is interleaved, MFMA by MFMA, with Y of block k (the wave issues in order, so the
// instruction stream is the schedule); Z of block k follows, its operands fetched two MFMAs ahead.
// The prologue also computes delta = rowsum(O * dO) and mhat = M log2(e) + log2(L) of the wave's
// rows (the reference's _bwd_preprocess, llama/ltriton/flash_landmark_attention.py:125-149).
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
  static constexpr int NBUF = 4;                           // ring slots: blocks k, k+1 in use, k+2, k+3 in flight
  static constexpr int RPD = 1024 / ROWB;                  // block rows covered by one 1 KB request
  static constexpr int NREQ = 2 * (32 / RPD);              // requests per block (K and V)
  static constexpr int PER_TILE = NREQ / NW;               // requests per wave and block
  static constexpr int FL = 8;                             // blocks between flushes of the per-block terms
  static constexpr int STAT_WAVE = 3 * FL * 32 * 4;        // a, nD, dS_landmark for FL blocks x 32 queries
  static constexpr int GO_OFF = NBUF * BUF_BYTES;          // per wave: its 32 rows of dO (B operand of dP^T)
  static constexpr int STAT_OFF = GO_OFF + NW * BLK_BYTES;
  static constexpr int LDS_BYTES = STAT_OFF + NW * STAT_WAVE;
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

// HO: the hand-over variant.  dS^T of every (query tile, key block) pair also goes to p.ds_tiles as a 2 KB tile
// [key step][query row][key of the step, in this kernel's register order], two 16-byte stores per lane and block, for the dK/dV
// kernel that then forms neither dP nor dS; of the per-block terms only `a` is still needed.
template <class T, int D, bool HO>
__global__ __launch_bounds__(512, 2) void lmk_bwd_dq32_kernel(BwdParams p) {
  using C = Dq32Cfg<T, D>;
  extern __shared__ __align__(16) unsigned char smem[];   // used through LDS byte addresses (it starts at 0)
  (void)smem;
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
  // hand-over: this wave's tiles are consecutive, one per key block (wave-uniform address)
  const char* ds_wave = nullptr;
  if (HO) {
    const int64_t j = qtile * C::NW + wave;
    ds_wave = (const char*)p.ds_tiles +
              (((int64_t)bh * handover_tiles_per_head(p.Lq >> 5, p.n_prefix) + j * (p.n_prefix + 1) + j * (j - 1) / 2) << 11);
  }
  auto store_ds = [&](int blk, const u32x4_t& d0, const u32x4_t& d1) __attribute__((always_inline)) {
    int l;
    asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(l));
    const uint32_t vo = (uint32_t)(((l & 31) << 5) | ((l >> 5) << 4));   // per key step 1 KB: row = query, 16 bytes per half-wave
    const char* tb = ds_wave + ((int64_t)blk << 11);
    asm volatile("global_store_dwordx4 %0, %1, %2" ::"v"(vo), "v"(d0), "s"(tb) : "memory");
    asm volatile("global_store_dwordx4 %0, %1, %2 offset:1024" ::"v"(vo), "v"(d1), "s"(tb) : "memory");
  };

  u32x4_t qf[C::KS];
#pragma unroll
  for (int ks = 0; ks < C::KS; ++ks) {
    u32x4_t z = {0, 0, 0, 0};
    qf[ks] = z;
    if (rowok) qf[ks] = *(const u32x4_t*)(qp + 2 * ((int64_t)qrow * p.qs_r + 16 * ks + 8 * h));
  }
  // delta = rowsum(O * dO) and mhat = M log2(e) + log2(L) of this lane's query row are computed here,
  // after the prologue (dO comes from LDS), and left in the workspace for the dK/dV kernel
  // (`_bwd_preprocess`, llama/ltriton/flash_landmark_attention.py:125-149)
  float mhat = 0.f, delta = 0.f;
  float row_M = 0.f, row_L = 1.f;                           // fetched here, with everything else the prologue waits for
  if (rowok) {
    row_M = p.M[(int64_t)bh * p.Lq + qrow];
    row_L = p.L[(int64_t)bh * p.Lq + qrow];
  }
  u32x4_t of[C::KS];                                        // this lane's part of its O row
  {
    const char* op = (const char*)p.o + 2 * (b_ * p.os_b + hh * p.os_h);
#pragma unroll
    for (int ks = 0; ks < C::KS; ++ks) {
      u32x4_t z = {0, 0, 0, 0};
      of[ks] = z;
      if (rowok) of[ks] = *(const u32x4_t*)(op + 2 * ((int64_t)qrow * p.os_r + 16 * ks + 8 * h));
    }
  }

  // row fragment ks of a tile sits at tile_off(ql, 2 ks + h) = tile_off(ql, h) ^ (32 ks): the swizzle
  // is an XOR on the 16-byte chunk index and 2 ks only touches bits the row term leaves zero
  const int koff0 = tile_off<D>(ql, h);
  auto koff = [&](int ks) __attribute__((always_inline)) { return koff0 ^ (ks << 5); };
  // transposed fragments: lane reads 8 bytes of row 4h + i/4 (+ 8 for the second half) at column
  // 32 dc + 16 g2 + 4 (i%4).  dc moves the chunk index by 4 dc (address bits 6, 7); row + 8 flips
  // bit 1 of the swizzle term (address bit 5) and adds 8 rows.  All of these are XORs on the
  // dc = 0, first-half offset because the bits involved are independent of the rest.
  int voff0;
  {
    const int i = lane & 15, g2 = (lane >> 4) & 1;
    const int col = 16 * g2 + 4 * (i & 3);
    voff0 = tile_off<D>(4 * h + (i >> 2), col >> 3) + ((col >> 2) & 1) * 8;
  }
  constexpr int VOFF_HI = (8 * C::ROWB) | 32;

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
  static_assert((32 / C::RPD) % C::PER_TILE == 0, "all of a wave's requests read one tensor");
  const bool rq_isv = wave * C::PER_TILE >= 32 / C::RPD;   // wave-uniform: this wave fetches V rows (else K rows)
  const char* rq_base = rq_isv ? vp : kp;
  const uint32_t rq_step = (uint32_t)(2 * 32 * (rq_isv ? p.vs_r : p.ks_r));   // bytes per block; a head's rows span < 4 GB (host check)
  auto request = [&](int slot_bytes, int blk) __attribute__((always_inline)) {
    const int bb = min(blk, nkb - 1);                      // past the end: re-read the last block (never used)
    const char* base = rq_base + (uint32_t)bb * rq_step;
#pragma unroll
    for (int d = 0; d < C::PER_TILE; ++d) dq_dma16(base, r_vo[d], slot_bytes + r_lds[d]);
  };

  f32x16_t acc[C::DC];
#pragma unroll
  for (int dc = 0; dc < C::DC; ++dc)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[dc][r] = 0.f;

  // per-wave staging of the per-block terms in LDS: [plane 3][FL][32] floats at STAT_OFF + wave * STAT_WAVE
  auto lane_now = []() __attribute__((always_inline)) {     // lane id without a long-lived register
    int l;
    asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(l));
    return l;
  };
  // flush: lane -> (block fl_bi of the group, queries 4 fl_part ..); wave-uniform base in SGPRs, one
  // 32-bit lane offset shared by the three planes.  Lane-only values are recomputed at each use:
  // held across the loop they cost registers the loop does not have.
  auto flush = [&](int blast) __attribute__((always_inline)) {   // blocks FL*(blast/FL) .. blast of this wave's terms
    const int ln = lane_now();
    const int fl_bi = ln >> 3, fl_part = ln & 7;
    const uint32_t fl_off = 4u * (uint32_t)(fl_bi * p.Lq + 4 * fl_part);
    const int fl_lds = C::STAT_OFF + wave * C::STAT_WAVE + (fl_bi * 32 + 4 * fl_part) * 4;
    const int b0 = __builtin_amdgcn_readfirstlane(blast & ~(C::FL - 1));
    const int64_t ub = ((int64_t)bh * p.n_blocks + b0) * p.Lq + q0;
    if (b0 + fl_bi <= blast) {
#pragma unroll
      for (int pl = 0; pl < (HO ? 1 : 3); ++pl) {
        const float* base = (pl == 0 ? p.stat_a : pl == 1 ? p.stat_n : p.stat_l) + ub;
        const u32x4_t val = lds_ld128(fl_lds + pl * C::FL * 128);
        asm volatile("global_store_dwordx4 %0, %1, %2" ::"v"(fl_off), "v"(val), "s"(base) : "memory");
      }
    }
  };

  // ---- the stages
  const int goff = C::GO_OFF + wave * C::BLK_BYTES;
  // row-fragment addresses of a tile at LDS address 0 (K, V: the slot is added as an immediate) and
  // of this wave's dO rows
  int kx[C::KS], gx[C::KS];
#pragma unroll
  for (int ks = 0; ks < C::KS; ++ks) {
    kx[ks] = koff0 ^ (ks << 5);
    gx[ks] = goff + kx[ks];
    // the compiler must not know the value's range: it would turn "offset + slot" into an OR computed by a
    // vector instruction per read; as a plain sum the slot stays the read's immediate offset
    asm volatile("" : "+v"(kx[ks]));
  }
  int zbc[2 * C::DC];                                       // the transposed-fragment offsets of a tile at LDS address 0;
#pragma unroll                                              // slot and key step are immediate offsets of the reads
  for (int dc = 0; dc < C::DC; ++dc) {
    zbc[2 * dc] = voff0 ^ (dc << 6);
    zbc[2 * dc + 1] = voff0 ^ ((dc << 6) | VOFF_HI);
    asm volatile("" : "+v"(zbc[2 * dc]), "+v"(zbc[2 * dc + 1]));   // as for kx
  }
  auto zero16 = [](f32x16_t& x) __attribute__((always_inline)) {
#pragma unroll
    for (int r = 0; r < 16; ++r) x[r] = 0.f;
  };
  u32x4_t dsf[2];                                           // packed dS^T of the block: keys 0..15, 16..31
  auto stage_x = [&](int slot_bytes, f32x16_t& s, f32x16_t& d) __attribute__((always_inline)) {
    zero16(s);
    zero16(d);
#pragma unroll
    for (int ks = 0; ks < C::KS; ++ks) {
      s = mfma32<T>(lds_ld128(kx[ks] + slot_bytes), qf[ks], s);
      d = mfma32<T>(lds_ld128(kx[ks] + slot_bytes + C::BLK_BYTES), lds_ld128(gx[ks]), d);
    }
  };
  auto ztr = [&](int slot_bytes, int n) __attribute__((always_inline)) {   // A operand of the n-th dQ^T MFMA: K^T, keys 16 j ..
    const int j = n / C::DC, dc = n % C::DC;
    const u32x2_t a0 = lds_ld_tr(zbc[2 * dc] + (slot_bytes + 16 * j * C::ROWB));
    const u32x2_t a1 = lds_ld_tr(zbc[2 * dc + 1] + (slot_bytes + 16 * j * C::ROWB));
    const u32x4_t a = {a0[0], a0[1], a1[0], a1[1]};
    return a;
  };
  auto stage_z = [&](int slot_bytes) __attribute__((always_inline)) {     // dQ^T += K^T dS^T
    // operands are fetched PFZ MFMAs ahead: a fetch that is awaited at once costs the LDS latency per MFMA
    constexpr int NZ = 2 * C::DC, PFZ = 2;
    u32x4_t zf[NZ];
#pragma unroll
    for (int n = 0; n < PFZ; ++n) zf[n] = ztr(slot_bytes, n);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int n = 0; n < NZ; ++n) {
      if (n + PFZ < NZ) zf[n + PFZ] = ztr(slot_bytes, n + PFZ);
      acc[n % C::DC] = mfma32<T>(zf[n], dsf[n / C::DC], acc[n % C::DC]);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // X of the next block interleaved with Y of an earlier block `blk`.  The wave issues in order, so
  // the instruction stream is the schedule: each MFMA is followed by a slice of Y that runs while
  // the matrix pipe is busy.  Key of register r is 8*(r/4) + 4h + r%4; the landmark is r = 15, h = 1.
  auto stage_xy = [&](int nslot, int blk, f32x16_t& s, f32x16_t& d, f32x16_t& sn, f32x16_t& dn)
                      __attribute__((always_inline)) {
    zero16(sn);
    zero16(dn);
    constexpr int NX = 2 * C::KS;
    u32x4_t fk[C::KS], fv[C::KS], fg[C::KS];
    auto frags = [&](int ks) __attribute__((always_inline)) {
      fk[ks] = lds_ld128(kx[ks] + nslot);
      fv[ks] = lds_ld128(kx[ks] + nslot + C::BLK_BYTES);
      fg[ks] = lds_ld128(gx[ks]);
    };
    frags(0);
    const float s_last = s[15];
    float mx = 0.f, mloc = 0.f, t_lm = 0.f, den = 0.f, spd = 0.f, nD = 0.f, f = 0.f, fn = 0.f, dslm = 0.f;
    float ds[16];
    auto ywork = [&](int u) __attribute__((always_inline)) {
      if (u == 0) {
        mx = fmaxf(fmaxf(s[0], s[1]), s[2]);
        mx = fmaxf(fmaxf(mx, s[3]), s[4]);
        mx = fmaxf(fmaxf(mx, s[5]), s[6]);
        mx = fmaxf(fmaxf(mx, s[7]), s[8]);
      } else if (u == 1) {
        mx = fmaxf(fmaxf(mx, s[9]), s[10]);
        mx = fmaxf(fmaxf(mx, s[11]), s[12]);
        mx = fmaxf(fmaxf(mx, s[13]), s[14]);
        mx = fmaxf(mx, (h == 0) ? s_last : -INFINITY);
        mx = pair_max(mx);
        t_lm = pair_hi(s_last) * c2;
        mloc = mx * c2;
      } else if (u < 10) {
#pragma unroll
        for (int r = 2 * (u - 2); r < 2 * (u - 2) + 2; ++r) {
          float x = fast_exp2(__builtin_fmaf(s[r], c2, -mloc));
          if (r == 15) x = (h == 0) ? x : 0.f;
          s[r] = x;
          den += x;
          spd = __builtin_fmaf(x, d[r], spd);
        }
      } else if (u == 10) {
        den = pair_sum(den);
        spd = pair_sum(spd);
      } else if (u == 11) {
        const float invden = fast_rcp(den);
        nD = spd * invden;
        const float glog = t_lm - mhat;                    // log2 of the normalised gate
        const float g = fast_exp2(glog);
        f = g * invden;
        fn = f * nD;
        dslm = g * (nD - delta);
        const int ln = lane_now();
        if (ln < 32) {                                     // h == 0: lane = query
          const int bi = blk & (C::FL - 1);
          const int sp = C::STAT_OFF + wave * C::STAT_WAVE + bi * 128 + ln * 4;
          lds_st32(sp + 0 * C::FL * 128, mloc + fast_log2(den) - glog);
          if (!HO) {
            lds_st32(sp + 1 * C::FL * 128, nD);
            lds_st32(sp + 2 * C::FL * 128, dslm);
          }
        }
      } else {
#pragma unroll
        for (int r = 4 * (u - 12); r < 4 * (u - 12) + 4; ++r) {
          ds[r] = s[r] * __builtin_fmaf(f, d[r], -fn);
          if (r == 15) ds[r] = (h == 1) ? dslm : ds[r];
          if (r & 1) dsf[r >> 3][(r >> 1) & 3] = pack2<T>(ds[r - 1], ds[r]);
        }
      }
    };
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int m = 0; m < NX; ++m) {
      const int ks = m >> 1;
      if ((m & 1) == 0 && ks + 1 < C::KS) frags(ks + 1);
      if ((m & 1) == 0) sn = mfma32<T>(fk[ks], qf[ks], sn);
      else dn = mfma32<T>(fv[ks], fg[ks], dn);
#pragma unroll
      for (int u = (m * 16) / NX; u < ((m + 1) * 16) / NX; ++u) ywork(u);
      __builtin_amdgcn_sched_barrier(0);
    }
    if (HO) store_ds(blk, dsf[0], dsf[1]);
    if ((blk & (C::FL - 1)) == C::FL - 1 || blk == cblk - 1) flush(blk);
  };
  auto stage_y_diag = [&](const f32x16_t& s, const f32x16_t& d) __attribute__((always_inline)) {   // the wave's own block
    float ds[16];
    const int lim = ql - ((ql == 31) ? 1 : 0);             // the landmark query looks one to the left
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int key = 8 * (r >> 2) + 4 * h + (r & 3);
      const float pr = (key <= lim) ? fast_exp2(__builtin_fmaf(s[r], c2, -mhat)) : 0.f;
      ds[r] = pr * (d[r] - delta);
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      u32x4_t fr = {pack2<T>(ds[8 * j + 0], ds[8 * j + 1]), pack2<T>(ds[8 * j + 2], ds[8 * j + 3]),
                    pack2<T>(ds[8 * j + 4], ds[8 * j + 5]), pack2<T>(ds[8 * j + 6], ds[8 * j + 7])};
      dsf[j] = fr;
    }
    if (HO) store_ds(cblk, dsf[0], dsf[1]);
  };

  // ---- prologue: this wave's dO rows -> LDS; blocks 0 .. 2 requested; blocks 0 and 1 must have landed
  {
    const int qb = min(q0, p.Lq - 32);                     // inactive waves re-read valid rows (never used)
    const char* gt = gp + 2 * ((int64_t)qb * p.dos_r);
#pragma unroll
    for (int n = 0; n < 32 / C::RPD; ++n) {
      const int row = C::RPD * n + lane / C::CH, chp = lane % C::CH;
      const int f = (((row & 3) << 2) | ((row >> 2) & 3)) & (C::CH - 1);
      dq_dma16(gt, (uint32_t)(2 * (row * p.dos_r + 8 * (chp ^ f))), goff + n * 1024);
    }
  }
#pragma unroll
  for (int t = 0; t < C::NBUF - 1; ++t) request(t * C::BUF_BYTES, t);
  dq_wait_vmcnt<C::PER_TILE>();
  __syncthreads();
  {
    float dsum = 0.f;
#pragma unroll
    for (int ks = 0; ks < C::KS; ++ks) {
      const u32x4_t g4 = lds_ld128(gx[ks]);
#pragma unroll
      for (int i = 0; i < 4; ++i)
        dsum += unpack_lo<T>(of[ks][i]) * unpack_lo<T>(g4[i]) + unpack_hi<T>(of[ks][i]) * unpack_hi<T>(g4[i]);
    }
    delta = pair_sum(dsum);
    if (rowok) {
      const int64_t r = (int64_t)bh * p.Lq + qrow;
      mhat = row_M * kLog2e + fast_log2(row_L);
      if (h == 0) {
        p.delta[r] = delta;
        p.mhat[r] = mhat;
      }
    }
    asm volatile("" : "+v"(mhat), "+v"(delta));             // their loads are waited for here, not in the loop
  }

  f32x16_t sA, dA, sB, dB;                                  // S^T, dP^T of the even / odd blocks
  zero16(sB);
  zero16(dB);
  stage_x(0, sA, dA);

  // ALL: block k lies in front of the whole workgroup and every wave has query rows, so no wave has
  // anything to decide
  auto period = [&](auto Rc, int k, auto all) __attribute__((always_inline)) {
    constexpr int R = decltype(Rc)::value;
    constexpr bool ALL = decltype(all)::value;
    constexpr int CUR = R * C::BUF_BYTES, NXT = ((R + 1) % C::NBUF) * C::BUF_BYTES;
    request(((R + 3) % C::NBUF) * C::BUF_BYTES, k + 3);    // into the slot block k-1 has left
    if (ALL || (rowok && k <= cblk)) {
      f32x16_t& s = (R & 1) ? sB : sA;
      f32x16_t& d = (R & 1) ? dB : dA;
      f32x16_t& sn = (R & 1) ? sA : sB;
      f32x16_t& dn = (R & 1) ? dA : dB;
      if (ALL || k < cblk) stage_xy(NXT, k, s, d, sn, dn);
      else stage_y_diag(s, d);
      stage_z(CUR);
      // block k+2 has landed (k+3 may be in flight).  Behind its requests this wave has issued at least the two
      // tile stores of the previous period (in the first period: the two row-term stores of the prologue), the
      // requests of block k+3 and the two tile stores of this period; memory operations of a wave complete in order
      dq_wait_vmcnt<C::PER_TILE + (HO ? 4 : 0)>();
    } else {
      dq_wait_vmcnt<C::PER_TILE>();
    }
    __syncthreads();
  };
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  using I2 = std::integral_constant<int, 2>;
  using I3 = std::integral_constant<int, 3>;
  // The blocks in front of the workgroup's first query block, in whole turns of the ring, run as straight-line
  // code without per-wave tests and their branches when every wave of the workgroup has query rows; the
  // workgroup's own eight blocks and what is left of the turn take the general path.
  const bool wg_full = (qtile + 1) * C::QT <= p.Lq;
  const int n_all = wg_full ? (min(nblk, c0) & ~3) : 0;
  int k = 0;
  for (; k < n_all; k += 4) {
    period(I0{}, k, std::true_type{});
    period(I1{}, k + 1, std::true_type{});
    period(I2{}, k + 2, std::true_type{});
    period(I3{}, k + 3, std::true_type{});
  }
  for (; k < nblk; k += 4) {
    period(I0{}, k, std::false_type{});
    if (k + 1 < nblk) period(I1{}, k + 1, std::false_type{});
    if (k + 2 < nblk) period(I2{}, k + 2, std::false_type{});
    if (k + 3 < nblk) period(I3{}, k + 3, std::false_type{});
  }
  dq_wait_vmcnt<0>();                                      // nothing may still be writing LDS when the wave ends

  // dQ leaves as row segments through the LDS that held the wave's dO rows, which it no longer needs
  if (q0 < p.Lq)                                           // (all or none of a wave's rows exist)
    store_tile_rows<T, C::DC>(acc, p.scale, C::GO_OFF + wave * C::BLK_BYTES, [&](int r) __attribute__((always_inline)) -> char* {
      return dqp + 2 * ((int64_t)(q0 + r) * p.dqs_r);
    });
}

template <class T, int D, bool HO>
static int launch_dq32_h(const BwdParams& p, hipStream_t stream) {
  using C = Dq32Cfg<T, D>;
  auto kern = lmk_bwd_dq32_kernel<T, D, HO>;
  static std::atomic<uint64_t> lds_ok{0};
  if (int rc = allow_dynamic_lds(kern, C::LDS_BYTES, lds_ok)) return rc;
  const int n_qt = (p.Lq + C::QT - 1) / C::QT;
  hipLaunchKernelGGL(kern, dim3(n_qt * p.B * p.H), dim3(C::NTHR), C::LDS_BYTES, stream, p);
  return (int)hipGetLastError();
}

template <class T, int D>
static int launch_dq32_t(const BwdParams& p, hipStream_t stream) {
  return p.ds_tiles != nullptr ? launch_dq32_h<T, D, true>(p, stream) : launch_dq32_h<T, D, false>(p, stream);
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
