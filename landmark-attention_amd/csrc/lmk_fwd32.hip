// Forward kernel of fused landmark attention, landmark block = 32 keys (one MFMA tile).
//
// Same mathematics and layout as lmk_fwd.hip (S^T = K Q^T in the accumulator layout, lane =
// query).  A workgroup is 8 waves = 256 query rows sharing one K/V stream, two waves per SIMD;
// wave w owns landmark block c0 + w and keeps its Q fragments (B operands) and its O^T accumulator
// in registers.  K/V blocks stream through a ring of four LDS slots filled by direct global->LDS
// loads (block k+3 is requested while block k is computed; vmcnt is counted by hand).
//
// The softmax over the global bucket (the landmarks of the earlier blocks and the keys of the own
// block) needs a reference maximum.  Only landmark scores enter it from the earlier blocks, so it
// is known before the main loop at 1/32 of the cost of the scores: a first pass multiplies the
// queries with the landmark keys alone (32 landmarks per MFMA tile) and keeps the row maximum R.
// With R fixed the main loop has no running maximum, no rescaling of the accumulator and no
// branch; per block a wave does
//     X  S^T = K Q^T of the next block                        8 MFMA, row fragments from LDS
//     Y  local softmax of the block, gate exp2(s_lm - R)       vector ALU only, interleaved with X
//     Z  O^T += V^T P^T                                        8 MFMA, transposed fragments
// and the own block at the end joins the bucket with one rescale by 2^(R - max(R, own maximum)).
// (The reference kernel carries a running maximum and rescales per block,
// llama/ltriton/flash_landmark_attention.py:64-76; the result is the same sum.)
#include <type_traits>
#include <utility>

#include "lmk_common.hpp"
#include "lmk_landmark_keys.hpp"
#include "lmk_launch.hpp"
#include "lmk_topk_slice.hpp"

namespace lmk {

template <class T, int D, int NW_ = 8>
struct Fwd32Cfg {
  static constexpr int NW = NW_;                           // waves per workgroup: 8, or 4 for launches that would not fill the chip
  static constexpr int NTHR = 64 * NW;
  static constexpr int QT = 32 * NW;                       // query rows per workgroup
  static constexpr int CH = D / 8;
  static constexpr int KS = D / 16;
  static constexpr int DC = D / 32;
  static constexpr int ROWB = 2 * D;
  static constexpr int BLK_BYTES = 32 * ROWB;              // one block of K (or of V)
  static constexpr int BUF_BYTES = 2 * BLK_BYTES;          // K then V
  // ring slots: blocks k, k+1 in use, the others in flight.  (A ring twice as deep helps neither the short sequences
  // that get the small workgroups -- 12.3 -> 15.0 us for 256 rows per head, and whatever shares the launch loses
  // LDS -- nor, with one barrier per two blocks, the long ones: 83.1 -> 84.1 us at B2 H32 L2048.)
  static constexpr int NBUF = 4;
  static constexpr int AHEAD = NBUF - 1;                   // a period requests the block this far in front of its own
  static constexpr int RPD = 1024 / ROWB;                  // block rows covered by one 1 KB request
  static constexpr int NREQ = 2 * (32 / RPD);              // requests per block (K and V)
  static constexpr int PER_TILE = NREQ / NW;               // requests per wave and block
  static constexpr int WAIT_REQ = (AHEAD - 2) * PER_TILE;  // requests that may be in flight when block k+2 must have landed
  static constexpr int LM_OFF = NBUF * BUF_BYTES;          // two tiles of 32 landmark keys for the first pass
  static constexpr int LM_TILES = 2;
  static constexpr int LM_REQ = (32 / RPD + NW - 1) / NW;  // requests per wave and landmark tile
  static constexpr int OUT_SHARE = 2048;                   // per wave: its output tile leaves through here, 32 columns at a time
  static constexpr int LM_BYTES = LM_TILES * BLK_BYTES > NW * OUT_SHARE ? LM_TILES * BLK_BYTES : NW * OUT_SHARE;
  static constexpr int LDS_BYTES = LM_OFF + LM_BYTES;
};

__device__ __forceinline__ void fw_dma16(const void* base_uniform, uint32_t voff, uint32_t lds_off) {
  // one 1 KB request of a wave: lane i's 16 bytes land at lds_off + 16*i (lds_off travels in M0)
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               :: "v"(voff), "s"(base_uniform), "s"(__builtin_amdgcn_readfirstlane(lds_off)) : "memory");
}
template <int N>
__device__ __forceinline__ void fw_wait_vmcnt() {          // s_waitcnt vmcnt(N) only (gfx9 encoding)
  __builtin_amdgcn_s_waitcnt(0x0f70 | (N & 15) | ((N >> 4) << 14));
}

#define LMK_INL __attribute__((always_inline))

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>)
template <class F, int... R>
__device__ __forceinline__ void fw_static_for(F&& f, std::integer_sequence<int, R...>) {
  (f(std::integral_constant<int, R>{}), ...);
}

// The whole forward of one workgroup; `bid` is its index among the forward's workgroups (the kernel's dynamic LDS
// array is used through LDS byte addresses: it starts at 0).
template <class T, int D, int NW>
__device__ __forceinline__ void fwd32_body(const FwdParams& p, const int bid_) {
  using C = Fwd32Cfg<T, D, NW>;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ql = lane & 31, h = lane >> 5;

  const int n_qt = (p.Lq + C::QT - 1) / C::QT;
  int bh, qtile;
  {
    const int bid = bid_, BH = p.B * p.H;
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
  const bool rowok = qrow < p.Lq;
  const bool waveok = q0 < p.Lq;                           // wave-uniform: the wave has at least one query row
  const int nkb = (p.Lk + 31) >> 5;                        // key blocks that exist (the last one may be partial)
  const int nblk = min(nkb, c0 + C::NW);                   // blocks this workgroup walks
  const float c2 = p.scale_log2;

  u32x4_t qf[C::KS];
#pragma unroll
  for (int ks = 0; ks < C::KS; ++ks) {
    u32x4_t z = {0, 0, 0, 0};
    qf[ks] = z;
    if (rowok) qf[ks] = *(const u32x4_t*)(qp + 2 * ((int64_t)qrow * p.qs_r + 16 * ks + 8 * h));
  }
  if (p.rope_cos != nullptr && rowok) {                      // q without rotary: rotate the fragments at the row's position
    int64_t pos = p.rope_pos[(int64_t)b_ * p.rope_pos_stride_b + qrow];
    pos = pos < 0 ? 0 : (pos >= p.rope_n_pos ? p.rope_n_pos - 1 : pos);
    rotate_fragments<T, C::KS>(qf, (const char*)p.rope_cos + 2 * pos * p.rope_cs_r, (const char*)p.rope_sin + 2 * pos * p.rope_cs_r, h);
  }

  // row fragment ks of a tile sits at tile_off(ql, 2 ks + h) = tile_off(ql, h) ^ (32 ks): the swizzle
  // is an XOR on the 16-byte chunk index and 2 ks only touches bits the row term leaves zero
  const int koff0 = tile_off<D>(ql, h);
  int kx[C::KS];
#pragma unroll
  for (int ks = 0; ks < C::KS; ++ks) {
    kx[ks] = koff0 ^ (ks << 5);
    // the compiler must not know the value's range: it would turn "offset + slot" into an OR computed by a
    // vector instruction per read; as a plain sum the slot stays the read's immediate offset
    asm volatile("" : "+v"(kx[ks]));
  }
  // transposed fragments: lane reads 8 bytes of row 4h + i/4 (+ 8 for the second half) at column
  // 32 dc + 16 g2 + 4 (i%4); dc and the second half are XORs on the dc = 0, first-half offset
  int voff0;
  {
    const int i = lane & 15, g2 = (lane >> 4) & 1;
    const int col = 16 * g2 + 4 * (i & 3);
    voff0 = tile_off<D>(4 * h + (i >> 2), col >> 3) + ((col >> 2) & 1) * 8;
  }
  constexpr int VOFF_HI = (8 * C::ROWB) | 32;
  int zbc[2 * C::DC];                                       // the transposed-fragment offsets of a tile at LDS address 0;
#pragma unroll                                              // slot and key step are immediate offsets of the reads
  for (int dc = 0; dc < C::DC; ++dc) {
    zbc[2 * dc] = voff0 ^ (dc << 6);
    zbc[2 * dc + 1] = voff0 ^ ((dc << 6) | VOFF_HI);
    asm volatile("" : "+v"(zbc[2 * dc]), "+v"(zbc[2 * dc + 1]));   // as for kx
  }

  // ---- requests: wave w issues request n = w*PER_TILE + d of each block (K first, then V).  In a
  // partial last block the rows past Lk re-read the last row (they are masked, but must be readable).
  uint32_t r_vo[C::PER_TILE], r_vo_last[C::PER_TILE];
  int r_lds[C::PER_TILE];
  bool r_isv[C::PER_TILE];
  const int last_rows = p.Lk - 32 * (nkb - 1);             // rows of the last block, 1 .. 32
#pragma unroll
  for (int d = 0; d < C::PER_TILE; ++d) {
    const int n = wave * C::PER_TILE + d;
    constexpr int per = 32 / C::RPD;                       // requests per tensor
    const int part = n % per;
    r_isv[d] = n >= per;
    const int row = C::RPD * part + lane / C::CH, chp = lane % C::CH;
    const int f = (((row & 3) << 2) | ((row >> 2) & 3)) & (C::CH - 1);
    const int64_t rs = r_isv[d] ? p.vs_r : p.ks_r;
    r_vo[d] = (uint32_t)(2 * (row * rs + 8 * (chp ^ f)));
    r_vo_last[d] = (uint32_t)(2 * (min(row, last_rows - 1) * rs + 8 * (chp ^ f)));
    r_lds[d] = (r_isv[d] ? C::BLK_BYTES : 0) + part * 1024;
  }
  static_assert((32 / C::RPD) % C::PER_TILE == 0, "all of a wave's requests read one tensor");
  const bool rq_isv = wave * C::PER_TILE >= 32 / C::RPD;   // wave-uniform: this wave fetches V rows (else K rows)
  const char* rq_base = rq_isv ? vp : kp;
  const uint32_t rq_step = (uint32_t)(2 * 32 * (rq_isv ? p.vs_r : p.ks_r));   // bytes per block; a head's rows span < 4 GB (host check)
  auto request = [&](int slot_bytes, int blk) LMK_INL {
    const int bb = min(blk, nkb - 1);                      // past the end: re-read the last block (never used)
    const bool last = bb == nkb - 1;                       // wave-uniform
    const char* base = rq_base + (uint32_t)bb * rq_step;
#pragma unroll
    for (int d = 0; d < C::PER_TILE; ++d) fw_dma16(base, last ? r_vo_last[d] : r_vo[d], slot_bytes + r_lds[d]);
  };
  // first pass: tile lt holds the landmark keys (row 31) of blocks 32 lt .. 32 lt + 31, row j of the tile =
  // block 32 lt + j, same swizzle as a K block.  Every wave issues LM_REQ requests per tile (with more waves than
  // requests the upper waves repeat the lower ones', so that all waves count the same).  Only landmarks of
  // complete earlier blocks are ever used; rows past them re-read the last complete block's landmark.
  const int n_lm = min(c0 + C::NW - 1, p.Lk >> 5);          // landmarks any wave here can need: blocks 0 .. n_lm-1
  const int n_lt = (n_lm + 31) >> 5;
  auto request_lm = [&](int lt) LMK_INL {
    constexpr int per = 32 / C::RPD;
#pragma unroll
    for (int i = 0; i < C::LM_REQ; ++i) {
      const int part = (wave * C::LM_REQ + i) % per;
      const int row = C::RPD * part + lane / C::CH, chp = lane % C::CH;
      const int f = (((row & 3) << 2) | ((row >> 2) & 3)) & (C::CH - 1);
      const int blk = min(32 * lt + row, max(n_lm - 1, 0));
      const uint32_t vo = (uint32_t)(2 * (((int64_t)blk * 32 + 31) * p.ks_r + 8 * (chp ^ f)));
      fw_dma16(kp, vo, C::LM_OFF + (lt & 1) * C::BLK_BYTES + part * 1024);
    }
  };

  f32x16_t acc[C::DC];
#pragma unroll
  for (int dc = 0; dc < C::DC; ++dc)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[dc][r] = 0.f;
  auto zero16 = [](f32x16_t& x) LMK_INL {
#pragma unroll
    for (int r = 0; r < 16; ++r) x[r] = 0.f;
  };

  // ---- the stages
  u32x4_t pf[2];                                            // packed P^T of the block: keys 0..15, 16..31
  float Rref = -1e30f, lsum = 0.f;                          // log2 domain; -1e30 stands for "no earlier block"
  auto stage_x = [&](int tile_bytes, f32x16_t& s) LMK_INL {
    zero16(s);
#pragma unroll
    for (int ks = 0; ks < C::KS; ++ks) s = mfma32<T>(lds_ld128(kx[ks] + tile_bytes), qf[ks], s);
  };
  auto ztr = [&](int tile_bytes, int n) LMK_INL {           // A operand of the n-th O^T MFMA: V^T, keys 16 j ..
    const int j = n / C::DC, dc = n % C::DC;
    const u32x2_t a0 = lds_ld_tr(zbc[2 * dc] + (tile_bytes + 16 * j * C::ROWB));
    const u32x2_t a1 = lds_ld_tr(zbc[2 * dc + 1] + (tile_bytes + 16 * j * C::ROWB));
    const u32x4_t a = {a0[0], a0[1], a1[0], a1[1]};
    return a;
  };
  auto stage_z = [&](int vtile_bytes) LMK_INL {            // O^T += V^T P^T
    constexpr int NZ = 2 * C::DC, PFZ = 2;                  // operands fetched PFZ MFMAs ahead
    u32x4_t zf[NZ];
#pragma unroll
    for (int n = 0; n < PFZ; ++n) zf[n] = ztr(vtile_bytes, n);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int n = 0; n < NZ; ++n) {
      if (n + PFZ < NZ) zf[n + PFZ] = ztr(vtile_bytes, n + PFZ);
      acc[n % C::DC] = mfma32<T>(zf[n], pf[n / C::DC], acc[n % C::DC]);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // X of the next block interleaved with Y of an earlier block.  The wave issues in order, so the
  // instruction stream is the schedule: each MFMA is followed by a slice of Y that runs while the matrix
  // pipe is busy.  Key of register r is 8*(r/4) + 4h + r%4; the landmark is r = 15, h = 1.
  auto stage_xy = [&](int nslot, f32x16_t& s, f32x16_t& sn) LMK_INL {
    zero16(sn);
    u32x4_t fk[C::KS];
    constexpr int PFX = 2;
#pragma unroll
    for (int ks = 0; ks < PFX; ++ks) fk[ks] = lds_ld128(kx[ks] + nslot);
    const float s_last = s[15];
    float mx = 0.f, mloc = 0.f, t_lm = 0.f, den = 0.f, f = 0.f;
    auto ywork = [&](int u) LMK_INL {
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
          if (r == 15) x = (h == 0) ? x : 0.f;             // the landmark's value row never contributes
          s[r] = x;
          den += x;
        }
      } else if (u == 10) {
        den = pair_sum(den);
      } else if (u == 11) {
        const float g = fast_exp2(t_lm - Rref);             // the block's share of the global bucket
        lsum += g;
        f = g * fast_rcp(den);
      } else {
#pragma unroll
        for (int r = 4 * (u - 12); r < 4 * (u - 12) + 4; ++r) {
          s[r] *= f;
          if (r & 1) {
            uint32_t pk = pack2<T>(s[r - 1], s[r]);
            asm volatile("" : "+v"(pk));                    // pins this slice between its two MFMAs
            pf[r >> 3][(r >> 1) & 3] = pk;
          }
        }
      }
    };
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int m = 0; m < C::KS; ++m) {
      if (m + PFX < C::KS) fk[m + PFX] = lds_ld128(kx[m + PFX] + nslot);
      sn = mfma32<T>(fk[m], qf[m], sn);
#pragma unroll
      for (int u = (m * 16) / C::KS; u < ((m + 1) * 16) / C::KS; ++u) ywork(u);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // the wave's own block: its visible keys join the global bucket; reference moves from R to max(R, own maximum)
  float Mfin = 0.f;
  auto stage_y_diag = [&](const f32x16_t& s) LMK_INL {
    const int lim = ql - ((ql == 31) ? 1 : 0);             // the landmark query looks one to the left
    float x[16], mt = -1e30f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int key = 8 * (r >> 2) + 4 * h + (r & 3);
      x[r] = (key <= lim) ? s[r] * c2 : -INFINITY;
      mt = fmaxf(mt, x[r]);
    }
    Mfin = fmaxf(Rref, pair_max(mt));
    const float alpha = fast_exp2(Rref - Mfin);            // 0 when there was no earlier block
    lsum *= alpha;
#pragma unroll
    for (int dc = 0; dc < C::DC; ++dc)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[dc][r] *= alpha;
    float sum = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      x[r] = fast_exp2(x[r] - Mfin);
      sum += x[r];
    }
    lsum += pair_sum(sum);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      u32x4_t fr = {pack2<T>(x[8 * j + 0], x[8 * j + 1]), pack2<T>(x[8 * j + 2], x[8 * j + 3]),
                    pack2<T>(x[8 * j + 4], x[8 * j + 5]), pack2<T>(x[8 * j + 6], x[8 * j + 7])};
      pf[j] = fr;
    }
  };

  // ---- prologue: landmark tiles 0, 1 and blocks 0 .. NBUF-2 requested; the tiles and blocks 0, 1 must have landed
  if (n_lt > 0) request_lm(0);
  if (n_lt > 1) request_lm(1);
#pragma unroll
  for (int t = 0; t < C::AHEAD; ++t) request(t * C::BUF_BYTES, t);
  fw_wait_vmcnt<C::WAIT_REQ>();
  __syncthreads();

  // ---- first pass: R = max over the earlier blocks' landmark scores (log2 domain)
  {
    float mx = -1e30f;
    for (int lt = 0; lt < n_lt; ++lt) {
      if (lt >= C::LM_TILES) {                             // requested one iteration ago, one newer tile's requests behind it
        fw_wait_vmcnt<C::LM_REQ>();
        __syncthreads();
      }
      f32x16_t s;
      stage_x(C::LM_OFF + (lt & 1) * C::BLK_BYTES, s);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int b = 32 * lt + 8 * (r >> 2) + 4 * h + (r & 3);
        mx = fmaxf(mx, (b < cblk) ? s[r] : -1e30f);
      }
      if (n_lt > C::LM_TILES) {                            // long sequences: keep streaming tiles (wave-uniform)
        __syncthreads();                                   // everyone has read this slot
        request_lm(lt + C::LM_TILES);                      // past the last tile: a re-read that is never used
      }
    }
    mx = pair_max(mx);
    Rref = (cblk > 0) ? mx * c2 : -1e30f;
  }

  f32x16_t sA, sB;                                         // S^T of the even / odd blocks
  zero16(sB);
  stage_x(0, sA);

  // ALL: block k lies in front of the whole workgroup, so no wave has anything to decide
  auto period = [&](auto Rc, int k, auto all) LMK_INL {
    constexpr int R = decltype(Rc)::value;
    constexpr bool ALL = decltype(all)::value;
    constexpr int CUR = R * C::BUF_BYTES, NXT = ((R + 1) % C::NBUF) * C::BUF_BYTES;
    request(((R + C::AHEAD) % C::NBUF) * C::BUF_BYTES, k + C::AHEAD);   // into the slot block k-1 has left
    if (ALL || (waveok && k <= cblk)) {
      f32x16_t& s = (R & 1) ? sB : sA;
      f32x16_t& sn = (R & 1) ? sA : sB;
      if (ALL || k < cblk) stage_xy(NXT, s, sn);
      else stage_y_diag(s);
      stage_z(CUR + C::BLK_BYTES);
    }
    fw_wait_vmcnt<C::WAIT_REQ>();                          // block k+2 has landed (the later ones may be in flight)
    __syncthreads();
  };
  constexpr auto ring = std::make_integer_sequence<int, C::NBUF>{};
  // The blocks in front of the workgroup's first query block, in whole turns of the ring, run as straight-line
  // code without per-wave tests and their branches (a wave past the last query row computes on zero queries
  // and stores nothing); the workgroup's own blocks and what is left of the turn take the general path.
  const int n_all = min(nblk, c0) & ~(C::NBUF - 1);
  int k = 0;
  for (; k < n_all; k += C::NBUF)
    fw_static_for([&](auto Rc) LMK_INL { period(Rc, k + decltype(Rc)::value, std::true_type{}); }, ring);
  for (; k < nblk; k += C::NBUF)
    fw_static_for([&](auto Rc) LMK_INL {
      if (k + decltype(Rc)::value < nblk) period(Rc, k + decltype(Rc)::value, std::false_type{});   // uniform over the workgroup
    }, ring);
  fw_wait_vmcnt<0>();                                      // nothing may still be writing LDS when the wave ends

  // the output leaves as row segments through the wave's share of the landmark tiles' LDS, which nothing has
  // touched since the first pass
  if (waveok)
    store_tile_rows<T, C::DC>(acc, 1.0f / lsum, C::LM_OFF + wave * C::OUT_SHARE, [&](int r) LMK_INL -> char* {
      return q0 + r < p.Lq ? op + 2 * ((int64_t)(q0 + r) * p.os_r) : nullptr;
    });
  if (rowok) {
    if (h == 0) {                                          // statistics of the global bucket, relative to its maximum
      p.L[(int64_t)bh * p.Lq + qrow] = lsum;
      p.M[(int64_t)bh * p.Lq + qrow] = Mfin * kLn2;
    }
  }
}

#undef LMK_INL

template <class T, int D, int NW>
__global__ __launch_bounds__(64 * NW, 2) void lmk_fwd32_kernel(FwdParams p) {
  extern __shared__ __align__(16) unsigned char smem[];
  (void)smem;
  fwd32_body<T, D, NW>(p, (int)blockIdx.x);
}

// The forward over a retrieval step's local window and the rotation of the cache's landmark keys in one launch:
// neither needs the other, the forward alone fills a fraction of the chip (one workgroup per 256 query rows), and
// both stand in front of the selection and the gather.  Workgroups 0 .. n_fwd-1 run the forward, the rest rotate keys.
constexpr int kLkRowsPerThread = 4;   // landmark keys per thread of the workgroups that rotate them

template <class T, int D, int NW>
__global__ __launch_bounds__(64 * NW, 2) void lmk_fwd32_landmark_keys_kernel(FwdParams pf, RetrParams pr, int n_fwd) {
  extern __shared__ __align__(16) unsigned char smem[];
  (void)smem;
  if ((int)blockIdx.x < n_fwd) fwd32_body<T, D, NW>(pf, (int)blockIdx.x);
  else landmark_keys_body<T, D, 64 * NW, kLkRowsPerThread>(pr, (int)blockIdx.x - n_fwd);
}

// Workgroups of 8 waves (256 query rows) share one K/V stream among the most rows; when that many rows per
// workgroup would leave compute units without one, workgroups of 4 waves (128 rows, one wave per SIMD, two
// workgroups per compute unit) are used -- and for sequences up to 512 keys, where the blocks a workgroup's waves
// do not all see (its last 8, or 4) are half or all of its stream: 5-11 % faster there, the same from 1024 on.
static bool fwd32_small_workgroups(const FwdParams& p) {
  return p.Lk <= 512 || (int64_t)((p.Lq + 255) / 256) * p.B * p.H < cu_count();
}

template <class T, int D, int NW>
static int launch_fwd32_lk_w(const FwdParams& pf, const RetrParams& pr, hipStream_t stream) {
  using C = Fwd32Cfg<T, D, NW>;
  auto kern = lmk_fwd32_landmark_keys_kernel<T, D, NW>;
  static std::atomic<uint64_t> lds_ok{0};
  if (int rc = allow_dynamic_lds(kern, C::LDS_BYTES, lds_ok)) return rc;
  const int n_fwd = ((pf.Lq + C::QT - 1) / C::QT) * pf.B * pf.H;
  constexpr int RPW = kLkRowsPerThread * C::NTHR / (D / 8);
  const int64_t lkrows = (int64_t)pr.B * pr.H * pr.num_mems;
  const int n_lk = (int)((lkrows + RPW - 1) / RPW);
  hipLaunchKernelGGL(kern, dim3(n_fwd + n_lk), dim3(C::NTHR), C::LDS_BYTES, stream, pf, pr, n_fwd);
  return (int)hipGetLastError();
}

template <class T, int D>
static int launch_fwd32_lk_t(const FwdParams& pf, const RetrParams& pr, hipStream_t stream) {
  return fwd32_small_workgroups(pf) ? launch_fwd32_lk_w<T, D, 4>(pf, pr, stream) : launch_fwd32_lk_w<T, D, 8>(pf, pr, stream);
}

int launch_fwd32_landmark_keys(const FwdParams& pf, const RetrParams& pr, int D, int dtype, hipStream_t stream) {
  if (dtype == LMK_DTYPE_BF16) {
    if (D == 128) return launch_fwd32_lk_t<bf16_t, 128>(pf, pr, stream);
    if (D == 64) return launch_fwd32_lk_t<bf16_t, 64>(pf, pr, stream);
  } else if (dtype == LMK_DTYPE_F16) {
    if (D == 128) return launch_fwd32_lk_t<f16_t, 128>(pf, pr, stream);
    if (D == 64) return launch_fwd32_lk_t<f16_t, 64>(pf, pr, stream);
  }
  return LMK_ERR_UNSUPPORTED;
}

// The decode step: the forward over the local window (a row or a few per head) beside the slice step of the block
// selection, which needs nothing from it; both are workgroups of four waves.
template <class T, int D>
__global__ __launch_bounds__(256, 2) void lmk_fwd32_topk_slices_kernel(FwdParams pf, RetrParams pr, int n_fwd, int n_slices) {
  extern __shared__ __align__(16) unsigned char smem[];
  if ((int)blockIdx.x < n_fwd) fwd32_body<T, D, 4>(pf, (int)blockIdx.x);
  else topk_slice_body<T, D>(pr, n_slices, (int)blockIdx.x - n_fwd, smem);
}

template <class T, int D>
static int launch_fwd32_slices_t(const FwdParams& pf, const RetrParams& pr, hipStream_t stream) {
  using C = Fwd32Cfg<T, D, 4>;
  static_assert(C::NTHR == 64 * kSliceWaves && kSliceLdsBytes <= C::LDS_BYTES, "one workgroup shape for both");
  const int n_slices = topk_slices(pr);
  if (n_slices <= 0) return LMK_ERR_UNSUPPORTED;
  auto kern = lmk_fwd32_topk_slices_kernel<T, D>;
  static std::atomic<uint64_t> lds_ok{0};
  if (int rc = allow_dynamic_lds(kern, C::LDS_BYTES, lds_ok)) return rc;
  const int n_fwd = ((pf.Lq + C::QT - 1) / C::QT) * pf.B * pf.H;
  const int64_t n_sel = (int64_t)pr.B * pr.H * pr.T * n_slices;
  hipLaunchKernelGGL(kern, dim3((unsigned)(n_fwd + n_sel)), dim3(C::NTHR), C::LDS_BYTES, stream, pf, pr, n_fwd, n_slices);
  return (int)hipGetLastError();
}

int launch_fwd32_topk_slices(const FwdParams& pf, const RetrParams& pr, int D, int dtype, hipStream_t stream) {
  if (dtype == LMK_DTYPE_BF16) {
    if (D == 128) return launch_fwd32_slices_t<bf16_t, 128>(pf, pr, stream);
    if (D == 64) return launch_fwd32_slices_t<bf16_t, 64>(pf, pr, stream);
  } else if (dtype == LMK_DTYPE_F16) {
    if (D == 128) return launch_fwd32_slices_t<f16_t, 128>(pf, pr, stream);
    if (D == 64) return launch_fwd32_slices_t<f16_t, 64>(pf, pr, stream);
  }
  return LMK_ERR_UNSUPPORTED;
}

template <class T, int D, int NW>
static int launch_fwd32_w(const FwdParams& p, hipStream_t stream) {
  using C = Fwd32Cfg<T, D, NW>;
  auto kern = lmk_fwd32_kernel<T, D, NW>;
  static std::atomic<uint64_t> lds_ok{0};
  if (int rc = allow_dynamic_lds(kern, C::LDS_BYTES, lds_ok)) return rc;
  const int n_qt = (p.Lq + C::QT - 1) / C::QT;
  hipLaunchKernelGGL(kern, dim3(n_qt * p.B * p.H), dim3(C::NTHR), C::LDS_BYTES, stream, p);
  return (int)hipGetLastError();
}

template <class T, int D>
static int launch_fwd32_t(const FwdParams& p, hipStream_t stream) {
  return fwd32_small_workgroups(p) ? launch_fwd32_w<T, D, 4>(p, stream) : launch_fwd32_w<T, D, 8>(p, stream);
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
