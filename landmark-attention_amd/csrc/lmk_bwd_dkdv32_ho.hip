// dK/dV kernel of the backward pass, hand-over variant (landmark block = 32 keys = one MFMA tile).
//
// The dQ kernel (lmk_bwd_dq32.hip, HO) has already formed dS of every (query tile, key block) pair and left
// it in memory as a 2 KB 16-bit tile [query row][key, in that kernel's register order].  This kernel therefore
// forms neither dP nor dS: of the reference's five products per tile pair (S, dP, dQ | dV, dK,
// llama/ltriton/flash_landmark_attention.py:246-299) it runs S, dV and dK.
//
// Key-stationary.  A workgroup is 8 waves = 4 key tiles of 32 keys x 2 roles; the two waves of a key tile sit
// on the same SIMD (waves t and t+4):
//     wave V (t):    S = Q K^T,  W = exp2(S c - x)  (the attention weights),  dV^T += dO^T W
//     wave K (t+4):  dK^T += Q^T dS,  dS read from the wave's own ring of handed-over tiles
// Both work on the same query tile in the same iteration; one barrier per query tile keeps the shared ring
// of query tiles in step.  A dS tile arrives in LDS as it lies in memory (two halves of 16 columns, row =
// query, 32 bytes); a transposed LDS read turns it into the B operand (lane = key column, 8 queries).  Column c
// of a tile is key
// 16 (c / 16) + 8 ((c / 4) % 2) + 4 ((c / 8) % 2) + c % 4 of the block (the dQ kernel's register order), which
// only decides the row a lane's dK accumulator is stored to.
//
// Query tiles (32 rows of Q and of dO) and the per-(row, block) term `a` with the per-row term mhat stream
// through a ring of five LDS slots filled by direct global->LDS loads issued by the V waves, as in
// lmk_bwd_dkdv32.hip; every K wave streams its dS tiles through a private ring of 2 KB slots.
//     earlier block (query tile past the key tile):  x = a; at the block's landmark key W = 0 (x = 1e30)
//     own block / not yet visible:  W = [key <= lim] exp2(s*c - mhat); dS = 0 where the tile does not exist
//
// A workgroup serves up to four 128-key tiles of one (batch, head) in a row, in a zig-zag over the head's
// tiles, and neither ring stops between them.
#include <type_traits>

#include "lmk_common.hpp"
#include "lmk_launch.hpp"

namespace lmk {

template <class T, int D>
struct DkvHoCfg {
  static constexpr int NKT = 4;                            // key tiles per workgroup
  static constexpr int NW = 2 * NKT;
  static constexpr int NTHR = 64 * NW;
  static constexpr int CH = D / 8;
  static constexpr int KS = D / 16;
  static constexpr int DC = D / 32;
  static constexpr int ROWB = 2 * D;
  static constexpr int TILE_BYTES = 32 * ROWB;             // one query tile of Q (or of dO)
  static constexpr int STAT_BYTES = 1024 * NKT;            // per key tile one 1 KB request: a at +0, mhat at +384
  static constexpr int BUF_BYTES = 2 * TILE_BYTES + STAT_BYTES;   // Q, dO, terms
  static constexpr int NBUF = 5;                           // ring slots: tiles i, i+1 in use, i+2 .. i+NBUF-2 in flight
  static constexpr int RA = NBUF - 2;                      // tile i+RA is requested while tile i is computed
  static constexpr int RPD = 1024 / ROWB;                  // tile rows covered by one 1 KB request
  static constexpr int NDMA = 32 / RPD / NKT;              // requests per V wave and tile for one tensor
  static constexpr int PER_TILE_V = 2 * NDMA + 1;
  static constexpr int NDS = 6;                            // dS ring of a K wave: tile i in use, i+1 .. i+NDS-1 in flight
  static constexpr int DS_TILE = 2048 + 128;               // two 1 KB halves, the second 128 bytes further on (LDS banks)
  static constexpr int DS_OFF = NBUF * BUF_BYTES;          // [key tile][NDS][2 KB]
  static constexpr int CONST_OFF = DS_OFF + NKT * NDS * DS_TILE;   // 32 x 1e30f
  static constexpr int LDS_BYTES = CONST_OFF + 128;
};

__device__ __forceinline__ void ho_dma16_s(const void* base_uniform, uint32_t voff, uint32_t lds_off) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               :: "v"(voff), "s"(base_uniform), "s"(__builtin_amdgcn_readfirstlane(lds_off)) : "memory");
}
__device__ __forceinline__ void ho_dma16_v(const void* ptr, uint32_t lds_off) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
               :: "v"(ptr), "s"(__builtin_amdgcn_readfirstlane(lds_off)) : "memory");
}
template <int N>
__device__ __forceinline__ void ho_wait_vmcnt() {          // s_waitcnt vmcnt(N) only (gfx9 encoding)
  __builtin_amdgcn_s_waitcnt(0x0f70 | (N & 15) | ((N >> 4) << 14));
}

#define LMK_INL __attribute__((always_inline))

template <class T, int D>
__global__ __launch_bounds__(512, 2) void lmk_bwd_dkdv32_ho_kernel(BwdParams p) {
  using C = DkvHoCfg<T, D>;
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int tile = wave & (C::NKT - 1);                    // key tile inside the workgroup
  const bool role_k = wave >= C::NKT;                      // false: S, W, dV; true: dK
  const int ql = lane & 31, h = lane >> 5;
  // the key (inside its tile) this lane's accumulator column belongs to: the lane itself in the V role, the
  // handed-over tiles' column order in the K role
  const int kl = role_k ? ((ql & 0x13) | ((ql & 4) << 1) | ((ql & 8) >> 1)) : ql;

  const int BH = p.B * p.H;
  const int G = (int)gridDim.x / BH;                       // workgroups per head
  const int n_c = (p.n_kvtiles + G - 1) / G;               // items per workgroup (some may fall past the last tile)
  int bh, g_;
  {
    const int bid = blockIdx.x;
    if ((BH & 7) == 0) {                                   // all workgroups of a head on one XCD
      const int xcd = bid & 7, j = bid >> 3, ngrp = BH >> 3;
      g_ = j / ngrp;
      bh = (j % ngrp) * 8 + xcd;
    } else {
      g_ = bid / BH;
      bh = bid % BH;
    }
  }
  auto item_kvt = [&](int c) LMK_INL { return (c & 1) ? (c + 1) * G - 1 - g_ : c * G + g_; };
  auto next_item = [&](int c) LMK_INL {                    // first item index >= c with a tile that exists, or n_c
    while (c < n_c && item_kvt(c) >= p.n_kvtiles) ++c;
    return c;
  };
  int kvt = item_kvt(0);                                   // item 0 always exists (g_ < G <= n_kvtiles)
  const int b_ = bh / p.H, hh = bh % p.H;
  const char* qp = (const char*)p.q + 2 * (b_ * p.qs_b + hh * p.qs_h);
  const char* gp = (const char*)p.dout + 2 * (b_ * p.dos_b + hh * p.dos_h);

  const int nkt = p.Lk >> 5;                               // key tiles = landmark blocks
  const int PT = p.n_prefix;                               // history tiles in front of the queries
  const int nq = p.Lq >> 5;
  int kt, krow, j_first;
  bool active, lm_lane;
  auto set_item = [&](int c) LMK_INL {
    kvt = item_kvt(c);
    kt = kvt * C::NKT + tile;
    active = kt < nkt;
    krow = kt * 32 + kl;
    lm_lane = ql == 31;                                    // V role: this lane's key is the block's landmark
    j_first = max(0, kvt * C::NKT - PT);                   // first query tile any wave here can see
  };
  set_item(0);
  const float c2 = p.scale_log2;

  u32x4_t bf[C::KS];                                       // V role: K fragments of the key tile

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

  // ---- the shared ring (V waves): as in lmk_bwd_dkdv32.hip.  The V wave of pair t fetches rows
  // RPD*(t*NDMA + d) .. of a query tile's Q and dO and the terms of key tile t.
  static_assert(C::NDMA <= 2, "two source offsets per tensor");
  uint32_t q_vo0 = 0, q_vo1 = 0, g_vo0 = 0, g_vo1 = 0;
  if (!role_k) {
    const int chp = lane % C::CH;
    const int row0 = C::RPD * (tile * C::NDMA) + lane / C::CH, row1 = row0 + C::RPD;
    const int f0 = (((row0 & 3) << 2) | ((row0 >> 2) & 3)) & (C::CH - 1);
    const int f1 = (((row1 & 3) << 2) | ((row1 >> 2) & 3)) & (C::CH - 1);
    q_vo0 = (uint32_t)(2 * (row0 * p.qs_r + 8 * (chp ^ f0)));      // the chunk that belongs at LDS position chp
    g_vo0 = (uint32_t)(2 * (row0 * p.dos_r + 8 * (chp ^ f0)));
    if (C::NDMA > 1) {
      q_vo1 = (uint32_t)(2 * (row1 * p.qs_r + 8 * (chp ^ f1)));
      g_vo1 = (uint32_t)(2 * (row1 * p.dos_r + 8 * (chp ^ f1)));
    }
  }
  const uint32_t q_step = (uint32_t)(2 * 32 * p.qs_r), g_step = (uint32_t)(2 * 32 * p.dos_r);
  // this lane's 16 bytes of a query tile's terms: lanes 0-23 a (plane, one row of Lq per block; the upper two
  // thirds of them fetch it again), 24-31 mhat, 32-63 mhat again (one row per head)
  const float* st_lane;
  {
    const int part = lane % 8;
    const int64_t plane0 = (int64_t)bh * p.n_blocks * p.Lq, head_row = (int64_t)bh * p.Lq;
    st_lane = (lane < 24) ? p.stat_a + plane0 : p.mhat + head_row;
    st_lane += 4 * part;
  }
  auto item_first = [&](int c) LMK_INL { return max(0, item_kvt(c) * C::NKT - PT); };
  auto item_plane = [&](int c) LMK_INL {                   // element offset of this wave's key tile's block inside the plane
    return (int64_t)min(item_kvt(c) * C::NKT + tile, p.n_blocks - 1) * p.Lq;
  };
  int j_req = item_first(0), jf_nx = 0;
  int64_t pl_req = item_plane(0), pl_nx = 0;
  bool has_nx = false;
  auto announce_next = [&](int c) LMK_INL {                // the arithmetic side starts item c: tell the stream what follows it
    const int c2 = next_item(c + 1);
    has_nx = c2 < n_c;
    if (has_nx) {
      jf_nx = item_first(c2);
      pl_nx = item_plane(c2);
    }
  };
  announce_next(0);
  const int dst_off = tile * C::NDMA * 1024;               // this wave's rows inside a tile of a slot
  auto request_piece = [&](int slot_bytes, auto Pc) LMK_INL {
    constexpr int P = decltype(Pc)::value;
    if constexpr (P == 0) {                                // a new tile: behind an item's last one, move to the next item
      const bool past = j_req >= nq, take = past && has_nx;    // (or re-read the last tile, which nobody uses)
      j_req = take ? jf_nx : (past ? nq - 1 : j_req);
      pl_req = take ? pl_nx : pl_req;
      has_nx = take ? false : has_nx;
    }
    if constexpr (P < C::NDMA) {
      ho_dma16_s(qp, ((P == 0) ? q_vo0 : q_vo1) + (uint32_t)j_req * q_step, slot_bytes + dst_off + P * 1024);
    } else if constexpr (P == C::NDMA) {
      const int64_t off = 32 * (int64_t)j_req + ((lane < 24) ? pl_req : 0);
      ho_dma16_v(st_lane + off, slot_bytes + 2 * C::TILE_BYTES + tile * 1024);
    } else if constexpr (P <= 2 * C::NDMA) {
      constexpr int Gp = P - C::NDMA - 1;
      ho_dma16_s(gp, ((Gp == 0) ? g_vo0 : g_vo1) + (uint32_t)j_req * g_step, slot_bytes + C::TILE_BYTES + dst_off + Gp * 1024);
      if (P == 2 * C::NDMA) ++j_req;
    }
  };
  using P0 = std::integral_constant<int, 0>;
  using P1 = std::integral_constant<int, 1>;
  using P2 = std::integral_constant<int, 2>;
  using P3 = std::integral_constant<int, 3>;
  using P4 = std::integral_constant<int, 4>;
  static_assert(C::PER_TILE_V <= 5 && C::PER_TILE_V <= C::KS, "a tile's pieces are P0 .. P4, one per MFMA slot");
  auto request = [&](int slot_bytes) LMK_INL {             // the whole share at once (prologue); V role only
    request_piece(slot_bytes, P0{});
    request_piece(slot_bytes, P1{});
    request_piece(slot_bytes, P2{});
    request_piece(slot_bytes, P3{});
    request_piece(slot_bytes, P4{});
  };

  // ---- the private dS ring of a K wave.  Its stream runs over the same (item, query tile) sequence, three
  // tiles ahead of the arithmetic.  Tile (j, k) of a head exists for k <= PT + j; where this wave's key tile is
  // not visible to query tile j yet (or lies past the last key) a tile that exists is fetched and not used.
  const char* ds_head = (const char*)p.ds_tiles + ((int64_t)bh * handover_tiles_per_head(nq, PT) << 11);
  const int ds_base = C::DS_OFF + tile * C::NDS * C::DS_TILE;
  int c_rq = 0, j_rq = j_first, kt_rq = kt, ds_rq = 0;
  auto ds_request = [&]() LMK_INL {
    if (j_rq >= nq) {
      const int c2 = next_item(c_rq + 1);
      if (c2 < n_c) {
        c_rq = c2;
        j_rq = item_first(c2);
        kt_rq = item_kvt(c2) * C::NKT + tile;
      }
    }
    const int j = min(j_rq, nq - 1);                       // behind the last item: the last tile again, which nobody uses
    const int k = min(kt_rq, PT + j);
    const char* src = ds_head + ((int64_t)(j * (PT + 1) + j * (j - 1) / 2 + k) << 11);
    const uint32_t vo = (uint32_t)lane << 4;
    ho_dma16_s(src, vo, ds_base + ds_rq * C::DS_TILE);
    ho_dma16_s(src + 1024, vo, ds_base + ds_rq * C::DS_TILE + 1024 + 128);
    ++j_rq;
    ds_rq = (ds_rq + 1 == C::NDS) ? 0 : ds_rq + 1;
  };

  auto zero16 = [](f32x16_t& x) LMK_INL {
#pragma unroll
    for (int r = 0; r < 16; ++r) x[r] = 0.f;
  };
  auto row_tile = [&](int tile_bytes, f32x16_t& s) LMK_INL {   // (32 rows of the LDS tile) x (this wave's 32 keys)
    zero16(s);
#pragma unroll
    for (int ks = 0; ks < C::KS; ++ks) s = mfma32<T>(*(const u32x4_t*)(smem + tile_bytes + koff[ks]), bf[ks], s);
  };
  constexpr int NB = 2 * C::DC;
  auto trfrag = [&](int tile_bytes, int n) LMK_INL {       // A operand n of a transposed product: (tile)^T, rows 16 j2 ..
    const int j2 = n / C::DC, dc = n % C::DC;
    const int base = tile_bytes + 16 * j2 * C::ROWB;
    const u32x2_t a0 = lds_read_tr(smem + base + voff[dc][0]), a1 = lds_read_tr(smem + base + voff[dc][1]);
    const u32x4_t a = {a0[0], a0[1], a1[0], a1[1]};
    return a;
  };
  auto tr_product = [&](const u32x4_t* tf, const u32x4_t* pk, f32x16_t* acc) LMK_INL {
#pragma unroll
    for (int n = 0; n < NB; ++n) acc[n % C::DC] = mfma32<T>(tf[n], pk[n / C::DC], acc[n % C::DC]);
  };

  // ---- V role: one query tile i.  S of tile i+1 (slot nslot) is interleaved with W of tile i.
  auto body_v = [&](auto Mc, int i, int cslot, int nslot, int rslot, f32x16_t& s, f32x16_t& sn, f32x16_t* acc, auto sync) LMK_INL {
    constexpr bool MASKED = decltype(Mc)::value;
    const int CST = cslot + 2 * C::TILE_BYTES + tile * 1024;   // this key tile's terms: a at +0, mhat at +384
    const int krel = 32 * (kt - (PT + i)) + ql;            // key position relative to the query tile's first row
    const int xoff = (MASKED ? CST + 384 : (lm_lane ? C::CONST_OFF : CST)) + 16 * h;
    float4 x4[4];
    auto ldx = [&](int g) LMK_INL { x4[g] = *(const float4*)(smem + xoff + 32 * g); };
    auto grp = [](int m) LMK_INL { return ((m * 16) / C::KS) >> 2; };
    u32x4_t wf[2];
    float w[16];
    auto elementwise = [&](int r) LMK_INL {                // register r <-> query row 8*(r/4) + 4h + r%4
      const int g = r >> 2, e = r & 3;
      const float xa = (e == 0) ? x4[g].x : (e == 1) ? x4[g].y : (e == 2) ? x4[g].z : x4[g].w;
      float ex = fast_exp2(__builtin_fmaf(s[r], c2, -xa));
      if (MASKED) {
        // key visible to this query row?  the landmark row (the tile's last) looks one position to the left
        const int qloc = 8 * g + 4 * h + e;
        ex = (krel <= qloc - ((qloc == 31) ? 1 : 0)) ? ex : 0.f;
      }
      w[r] = ex;
      if (r & 1) {
        uint32_t pk = pack2<T>(w[r - 1], w[r]);
        asm volatile("" : "+v"(pk));                       // pins this slice between its two MFMAs
        wf[r >> 3][(r >> 1) & 3] = pk;
      }
    };
    zero16(sn);
    constexpr int PF = 2;
    u32x4_t fr[C::KS + PF], tf[NB];
#pragma unroll
    for (int m = 0; m < PF; ++m) fr[m] = *(const u32x4_t*)(smem + nslot + koff[m]);
    __builtin_amdgcn_sched_barrier(0);
    ldx(0);
    if (grp(1) != 0) ldx(grp(1));
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int m = 0; m < C::KS; ++m) {
      if (m + PF < C::KS) fr[m + PF] = *(const u32x4_t*)(smem + nslot + koff[m + PF]);
      if (m + 2 < C::KS && grp(m + 2) != grp(m + 1)) ldx(grp(m + 2));
#pragma unroll
      for (int n = (m * NB) / C::KS; n < ((m + 1) * NB) / C::KS; ++n) tf[n] = trfrag(cslot + C::TILE_BYTES, n);
      if (m == 0) request_piece(rslot, P0{});              // tile i+RA, into the slot tile i-2 has left
      if (m == 1) request_piece(rslot, P1{});
      if (m == 2) request_piece(rslot, P2{});
      if (m == 3) request_piece(rslot, P3{});
      if (m == 4) request_piece(rslot, P4{});
      sn = mfma32<T>(fr[m], bf[m], sn);
#pragma unroll
      for (int r = (m * 16) / C::KS; r < ((m + 1) * 16) / C::KS; ++r) elementwise(r);
      __builtin_amdgcn_sched_barrier(0);
    }
    sync();                                                // the iteration's barrier: what follows needs no LDS
    __builtin_amdgcn_sched_barrier(0);                     // keeps the MFMAs below behind the barrier
    tr_product(tf, wf, acc);                               // dV^T += dO^T W
  };

  // ---- K role: dK^T += Q^T dS of query tile i (slot cslot); its dS tile sits in ring slot dsl of this wave.
  int dsoff;                                               // this lane's address inside a dS tile for the transposed read
  {
    const int i = lane & 15, g2 = (lane >> 4) & 1;
    dsoff = (4 * h + (i >> 2)) * 32 + 8 * (i & 3) + g2 * (1024 + 128);
  }
  auto body_k = [&](int cslot, int dsl, bool vis, f32x16_t* acc) LMK_INL {
    const int db = ds_base + dsl * C::DS_TILE + dsoff;
    u32x4_t df[2], tf[NB];
    constexpr int PFK = 2;
#pragma unroll
    for (int j2 = 0; j2 < 2; ++j2) {
      const u32x2_t a0 = lds_ld_tr(db + 512 * j2), a1 = lds_ld_tr(db + 512 * j2 + 256);
      u32x4_t a = {a0[0], a0[1], a1[0], a1[1]};
      const u32x4_t z = {0, 0, 0, 0};
      df[j2] = vis ? a : z;
    }
#pragma unroll
    for (int n = 0; n < PFK; ++n) tf[n] = trfrag(cslot, n);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int n = 0; n < NB; ++n) {
      if (n + PFK < NB) tf[n + PFK] = trfrag(cslot, n + PFK);
      acc[n % C::DC] = mfma32<T>(tf[n], df[n / C::DC], acc[n % C::DC]);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  auto load_stationary = [&]() LMK_INL {                   // V role: K fragments of the item's key tile, lane = key
    const char* src = (const char*)p.k + 2 * (b_ * p.ks_b + hh * p.ks_h);
    int kr = krow, h8 = 8 * h;
    asm volatile("" : "+v"(kr), "+v"(h8));                 // the address is formed here, not ahead of the loops (and spilled)
    const char* row = src + 2 * ((int64_t)kr * p.ks_r + h8);
#pragma unroll
    for (int ks = 0; ks < C::KS; ++ks) {
      u32x4_t z = {0, 0, 0, 0};
      bf[ks] = z;
      if (active) bf[ks] = *(const u32x4_t*)(row + 32 * ks);
    }
  };
  // consume the operand at once: no wait for these loads can then end up inside the loop, where it would
  // drain the ring; the explicit wait covers everything this wave has in flight, which the compiler does not count
  auto await_stationary = [&]() LMK_INL {
    ho_wait_vmcnt<0>();
#pragma unroll
    for (int ks = 0; ks < C::KS; ++ks) asm volatile("" : "+v"(bf[ks]));
  };

  // ---- prologue
  if (!role_k) {
    load_stationary();
    request(0);
    request(C::BUF_BYTES);
  } else {
#pragma unroll
    for (int t = 0; t < C::NDS - 1; ++t) ds_request();
  }
  if (tid < 32) ((float*)(smem + C::CONST_OFF))[tid] = 1e30f;
  if (!role_k) {
    await_stationary();                                    // the first two tiles have landed
#pragma unroll
    for (int t = 2; t < C::RA; ++t) request(t * C::BUF_BYTES);
  }
  __syncthreads();

  // Per item: iterations i = j_first .. nq-1, one barrier each, in both roles.  The ring slot of tile i is a
  // wave-uniform counter that runs on from item to item: the slots behind an item's last tile already hold the
  // next item's first tiles.
  auto wrap = [](int x) LMK_INL { return x >= C::NBUF ? x - C::NBUF : x; };
  auto store_acc = [&](const f32x16_t* acc, char* dst, int64_t rs, float scl) LMK_INL {
    int kr = krow, h4 = 4 * h;
    asm volatile("" : "+v"(kr), "+v"(h4));
    char* row = dst + 2 * ((int64_t)kr * rs + h4);
#pragma unroll
    for (int dc = 0; dc < C::DC; ++dc)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        u32x2_t o2 = {pack2<T>(acc[dc][4 * g + 0] * scl, acc[dc][4 * g + 1] * scl),
                      pack2<T>(acc[dc][4 * g + 2] * scl, acc[dc][4 * g + 3] * scl)};
        *(u32x2_t*)(row + 2 * (32 * dc + 8 * g)) = o2;
      }
  };
  if (!role_k) {
    f32x16_t acc[C::DC];                                   // dV^T: rows = d, lane = key
    f32x16_t cur, nxt;                                      // S of tiles i and i+1
    int sc = 0;                                            // slot of the item's tile i
    for (int c = 0; c < n_c; c = next_item(c + 1)) {
      if (c > 0) {                                         // the ring already holds this item's first tiles
        set_item(c);
        announce_next(c);
        load_stationary();
        await_stationary();
      }
#pragma unroll
      for (int dc = 0; dc < C::DC; ++dc) zero16(acc[dc]);
      row_tile(sc * C::BUF_BYTES, cur);                     // S of the first tile
      auto step = [&](auto Mc, int i) LMK_INL {
        auto sync = [&]() LMK_INL {
          ho_wait_vmcnt<(C::RA - 2) * C::PER_TILE_V>();     // tile i+2 has landed (tiles i+3 .. i+RA may be in flight)
          __syncthreads();
        };
        body_v(Mc, i, sc * C::BUF_BYTES, wrap(sc + 1) * C::BUF_BYTES, wrap(sc + C::RA) * C::BUF_BYTES, cur, nxt, acc, sync);
        cur = nxt;
        sc = wrap(sc + 1);
      };
      // the own block and the tiles that cannot see these keys yet come first, then every later tile sees all keys
      int i = j_first;
      const int i_full = min(nq, max(j_first, kt + 1 - PT));
      for (; i < i_full; ++i) step(std::true_type{}, i);
      for (; i < nq; ++i) step(std::false_type{}, i);
      if (active) store_acc(acc, (char*)p.dv + 2 * (b_ * p.dvs_b + hh * p.dvs_h), p.dvs_r, 1.f);
    }
    ho_wait_vmcnt<0>();                                    // nothing may still be writing LDS when the wave ends
  } else {
    f32x16_t acc[C::DC];                                   // dK^T: rows = d, lane = column of the dS tiles
    int sc = 0, dsl = 0;                                   // slots of tile i in the shared ring and in the dS ring
    for (int c = 0; c < n_c; c = next_item(c + 1)) {
      if (c > 0) set_item(c);
#pragma unroll
      for (int dc = 0; dc < C::DC; ++dc) zero16(acc[dc]);
      for (int i = j_first; i < nq; ++i) {
        ds_request();                                      // three tiles ahead, into the slot tile i-1 has left
        ho_wait_vmcnt<2 * (C::NDS - 1)>();                 // tile i's dS has landed
        body_k(sc * C::BUF_BYTES, dsl, active && PT + i >= kt, acc);
        __syncthreads();
        sc = wrap(sc + 1);
        dsl = (dsl + 1 == C::NDS) ? 0 : dsl + 1;
      }
      if (active) store_acc(acc, (char*)p.dk + 2 * (b_ * p.dks_b + hh * p.dks_h), p.dks_r, p.scale);
    }
    ho_wait_vmcnt<0>();
  }
}

#undef LMK_INL

template <class T, int D>
static int launch_dkdv32_ho_t(const BwdParams& p, hipStream_t stream) {
  using C = DkvHoCfg<T, D>;
  auto kern = lmk_bwd_dkdv32_ho_kernel<T, D>;
  static std::atomic<uint64_t> lds_ok{0};
  if (int rc = allow_dynamic_lds(kern, C::LDS_BYTES, lds_ok)) return rc;
  // workgroups per head: enough for about one workgroup per CU, at most four 128-key tiles each
  const int64_t items = (int64_t)p.n_kvtiles * p.B * p.H;
  int per_wg = (int)(items / cu_count());
  per_wg = per_wg < 1 ? 1 : (per_wg > 4 ? 4 : per_wg);
  const int groups = (p.n_kvtiles + per_wg - 1) / per_wg;
  hipLaunchKernelGGL(kern, dim3(groups * p.B * p.H), dim3(C::NTHR), C::LDS_BYTES, stream, p);
  return (int)hipGetLastError();
}

int launch_bwd_dkdv32_handover(const BwdParams& p, int D, int dtype, hipStream_t stream) {
  if (p.ds_tiles == nullptr) return LMK_ERR_NULL;
  if (dtype == LMK_DTYPE_BF16) {
    if (D == 128) return launch_dkdv32_ho_t<bf16_t, 128>(p, stream);
    if (D == 64) return launch_dkdv32_ho_t<bf16_t, 64>(p, stream);
  } else if (dtype == LMK_DTYPE_F16) {
    if (D == 128) return launch_dkdv32_ho_t<f16_t, 128>(p, stream);
    if (D == 64) return launch_dkdv32_ho_t<f16_t, 64>(p, stream);
  }
  return LMK_ERR_UNSUPPORTED;
}

}  // namespace lmk
